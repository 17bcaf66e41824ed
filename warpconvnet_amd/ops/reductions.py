"""Reductions over CSR row segments (reference: warpconvnet/ops/reductions.py:13-72, which calls
torch_scatter.segment_csr).  min, max, mean, sum, var, std and random are built; the device kernel
accumulates in fp32 whatever the feature dtype."""
import enum
from typing import Literal, Optional

import torch
from torch import Tensor
from torch.autograd import Function

from .._lib import DTYPE_CODE, check, lib, ptr, require_device, stream_ptr
from ..utils.gather import take_rows


class REDUCTIONS(enum.Enum):
    MIN = "min"
    MAX = "max"
    MEAN = "mean"
    SUM = "sum"
    MUL = "mul"
    VAR = "var"
    STD = "std"
    RANDOM = "random"


REDUCTION_TYPES_STR = Literal["min", "max", "mean", "sum", "mul", "var", "std", "random"]

_MODE = {REDUCTIONS.SUM: 0, REDUCTIONS.MEAN: 1, REDUCTIONS.MAX: 2, REDUCTIONS.MIN: 3}


def _segment_of_rows(offsets: Tensor, indices: Optional[Tensor], num_in: int) -> Tensor:
    """Segment of every feature row (-1 for rows in none)."""
    counts = offsets.diff()
    seg = torch.repeat_interleave(torch.arange(len(counts), device=offsets.device), counts)
    if indices is None:
        return seg
    out = torch.full((num_in,), -1, dtype=torch.int64, device=offsets.device)
    out[indices] = seg
    return out


class _SegmentReduceFunction(Function):
    """out[u] = reduce of features[indices[e]] over e in [offsets[u], offsets[u + 1]).  The
    gradient assumes that no feature row lies in two segments (true for the grouping of points by
    voxel); `segment_of` (a tensor, or a function returning it, called in the backward pass only)
    may be passed when the caller has the segment of every row (unique's inverse)."""

    @staticmethod
    def forward(ctx, features: Tensor, offsets: Tensor, indices: Optional[Tensor], mode: int,
                segment_of: Optional[Tensor]):
        require_device(features, "features")
        if features.dtype not in DTYPE_CODE:
            raise TypeError(f"unsupported feature dtype {features.dtype}")
        x = features.contiguous()
        n_in, channels = x.shape
        offsets = offsets.to(device=x.device, dtype=torch.int64).contiguous()
        if indices is not None:
            indices = indices.to(device=x.device, dtype=torch.int64).contiguous()
        m = len(offsets) - 1
        out = torch.empty((m, channels), dtype=x.dtype, device=x.device)
        arg = torch.empty((m, channels), dtype=torch.int64, device=x.device) if mode >= 2 else None
        entries = n_in if indices is None else indices.shape[0]
        check(lib().wcn_segment_reduce(ptr(x), n_in, channels, DTYPE_CODE[x.dtype], ptr(offsets),
                                       ptr(indices), entries, m, mode, ptr(out), ptr(arg),
                                       stream_ptr(x.device)),
              "wcn_segment_reduce")
        ctx.saved = (offsets, indices, segment_of, arg)
        ctx.mode, ctx.n_in = mode, n_in
        return out

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        offsets, indices, segment_of, arg = ctx.saved
        gy = grad_out.contiguous()
        m, channels = gy.shape
        if callable(segment_of):
            segment_of = segment_of()
        if segment_of is None:
            segment_of = _segment_of_rows(offsets, indices, ctx.n_in)
        segment_of = segment_of.to(torch.int64).contiguous()
        grad_in = torch.empty((ctx.n_in, channels), dtype=gy.dtype, device=gy.device)
        check(lib().wcn_segment_reduce_bwd(ptr(gy), m, channels, DTYPE_CODE[gy.dtype], ptr(offsets),
                                           ptr(segment_of), ctx.n_in, ctx.mode, ptr(arg), ptr(grad_in),
                                           stream_ptr(gy.device)), "wcn_segment_reduce_bwd")
        return grad_in, None, None, None, None


def segment_reduction(features: Tensor, offsets: Tensor, reduction, indices: Optional[Tensor] = None,
                      segment_of: Optional[Tensor] = None, eps: float = 1e-6) -> Tensor:
    """`row_reduction(features[indices], offsets, reduction)` without the gathered copy."""
    if isinstance(reduction, str):
        reduction = REDUCTIONS(reduction)
    if reduction in _MODE:
        return _SegmentReduceFunction.apply(features, offsets, indices, _MODE[reduction], segment_of)
    if reduction in (REDUCTIONS.VAR, REDUCTIONS.STD):  # reductions.py:27-34
        mean = _SegmentReduceFunction.apply(features, offsets, indices, 1, segment_of)
        var = _SegmentReduceFunction.apply(features ** 2, offsets, indices, 1, segment_of) - mean ** 2
        return var if reduction == REDUCTIONS.VAR else torch.sqrt(var + eps)
    if reduction == REDUCTIONS.RANDOM:  # reductions.py:62-68
        offsets = offsets.to(features.device)
        num_per_row = offsets.diff()
        pick = (torch.rand(len(num_per_row), device=features.device) * num_per_row).floor().long()
        entry = pick + offsets[:-1]
        return take_rows(features, indices[entry] if indices is not None else entry)
    raise NotImplementedError(f"reduction {reduction.value!r} is not built")


def row_reduction(features: Tensor, neighbor_row_splits: Tensor, reduction, eps: float = 1e-6) -> Tensor:
    """(M, C) reduction of the consecutive row segments given by (M + 1) splits
    (reductions.py:36-72)."""
    assert len(features) == int(neighbor_row_splits[-1]), \
        f"Features length {len(features)} must match the last row split {int(neighbor_row_splits[-1])}"
    return segment_reduction(features, neighbor_row_splits, reduction, eps=eps)
