"""Functional sparse convolution (reference: warpconvnet/nn/functional/sparse_conv.py).

`spatially_sparse_conv` keeps the reference signature and bookkeeping (1x1 shortcut, tensor
stride arithmetic, kernel-map cache with the transposed in/out swap, bias, output Voxels) and
sends the three device stages to the HIP library: output coordinates (`stride_coords`), kernel
map (`generate_kernel_map`) and the feature contraction (`wcn_sparse_conv_fwd`, one launch
sequence for all kernel offsets, fp32 accumulation, one rounding).

There is a single contraction algorithm; the `fwd_algo` / `bwd_algo` / block-size arguments of
the reference are accepted for call compatibility and do not select anything.  The backward pass
of the autograd Function runs in the same library (`wcn_sparse_conv_dgrad`: the contraction over
the map with in and out exchanged; `wcn_sparse_conv_wgrad`: per-offset X^T dY over the pairs;
reference: sparse_conv.py:314-355).
"""
import ctypes
import enum
import math
import os
import warnings
from typing import List, Optional, Tuple, Union

import numpy as np
import torch
from torch import Tensor
from torch.autograd import Function

from ..._lib import DTYPE_CODE, check, lib, ptr, require_device, stream_ptr, workspace
from ...geometry.coords.integer import IntCoords
from ...geometry.coords.ops.expand import expand_coords
from ...geometry.coords.ops.serialization import POINT_ORDERING, encode
from ...geometry.coords.ops.stride import stride_coords
from ...geometry.coords.search.cache import IntSearchCache, IntSearchCacheKey
from ...geometry.coords.search.search_results import IntSearchResult
from ...geometry.coords.search.torch_discrete import generate_kernel_map
from ...geometry.types.voxels import Voxels
from ...utils.ntuple import ntuple
from ...utils.gather import take_rows


class STRIDED_CONV_MODE(enum.Enum):
    REDUCE_AND_STRIDE = "reduce_and_stride"  # the input is pooled by the stride, then convolved
    STRIDE_ONLY = "stride_only"


class SPARSE_CONV_FWD_ALGO_MODE(enum.Enum):
    EXPLICIT_GEMM = "explicit_gemm"
    IMPLICIT_GEMM = "implicit_gemm"
    CUTLASS_IMPLICIT_GEMM = "cutlass_implicit_gemm"
    AUTO = "auto"


class SPARSE_CONV_BWD_ALGO_MODE(enum.Enum):
    EXPLICIT_GEMM = "explicit_gemm"
    IMPLICIT_GEMM = "implicit_gemm"
    CUTLASS_IMPLICIT_GEMM = "cutlass_implicit_gemm"
    AUTO = "auto"


def in_coords_of(voxels: Voxels):
    """The cached (N, D+1) batch-indexed rows of a tensor (the same object on every access)."""
    return voxels.batched_coordinates.batch_indexed_coordinates


def _is_random_order(order) -> bool:
    name = getattr(order, "name", order)
    return str(name).lower() in ("random", "point_ordering.random")


# ------------------------------------------------------------------------------------------------
# Feature contraction
# ------------------------------------------------------------------------------------------------

def _host_offsets_of(km: IntSearchResult):
    """(K + 1) ctypes int64 array of the map's offsets, made once per map object."""
    kept = km._host_offsets
    if kept is None or len(kept) != len(km.offsets):
        kept = (ctypes.c_int64 * len(km.offsets))(*[int(v) for v in km.offsets.tolist()])
        km._host_offsets = kept
    return kept


def _device_offsets_of(km: IntSearchResult, device) -> Tensor:
    """(K + 1) int64 copy of the map's offsets in device memory: left by the map builder, or made
    here once per map object (one small copy)."""
    kept = km._device_offsets
    if kept is None or kept.device != device or kept.numel() != len(km.offsets):
        kept = km.offsets.to(torch.int64).to(device)
        km._device_offsets = kept
    return kept


@torch.no_grad()
def _prepared_weight(weight: Tensor, make_w, dtype: torch.dtype, c_in: int) -> Tensor:
    """The kernels' tiles of make_w() (the weight as the contraction would receive it: detached,
    contiguous, its input channels zero-padded to c_in), made by wcn_conv_prepare_weight and kept
    on the tensor object `weight` until its version counter, address, dtype or shape changes."""
    key = (weight._version, weight.data_ptr(), weight.dtype, dtype, tuple(weight.shape), c_in)
    kept = getattr(weight, "_wcn_prepared", None)
    if kept is not None and kept[0] == key:
        # made on another stream (another thread's, say): this stream waits for that kernel
        if kept[3] != stream_ptr(weight.device):
            torch.cuda.current_stream(weight.device).wait_event(kept[2])
        return kept[1]
    L = lib()
    w = make_w()
    K, c_in, c_out = w.shape
    nbytes = L.wcn_conv_prepared_weight_bytes(K, c_in, c_out, DTYPE_CODE[dtype])
    tiles = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    stream = stream_ptr(w.device)
    check(L.wcn_conv_prepare_weight(ptr(w), DTYPE_CODE[w.dtype], K, c_in, c_out, DTYPE_CODE[dtype],
                                    ptr(tiles), nbytes, stream), "wcn_conv_prepare_weight")
    made = torch.cuda.Event()
    made.record(torch.cuda.current_stream(w.device))
    try:
        weight._wcn_prepared = (key, tiles, made, stream)
    except AttributeError:
        pass
    return tiles


@torch.no_grad()
def _pairs_sorted(km: IntSearchResult, by: str, num_rows: int):
    """The map's pair lists re-ordered so that the `by` side ("out" or "in") ascends inside every
    offset, with the table of per-64-row group starts of that order: made by the library on first
    use and kept on the map object, so a cached map pays for it once (the reference caches the
    exchanged map of a transposed convolution the same way, sparse_conv.py:1916-1939).
    Returns (gathered-side list, ascending-side list, group-start tensor)."""
    kept = km._by_out if by == "out" else km._by_in
    if kept is not None and kept[3] == num_rows:
        return kept[:3]
    gathered, ascending = (km.in_maps, km.out_maps) if by == "out" else (km.out_maps, km.in_maps)
    K = len(km)
    device = gathered.device
    L = lib()
    host_offsets = _host_offsets_of(km)
    num_pairs = int(host_offsets[K])
    g_sorted = torch.empty(num_pairs, dtype=torch.int32, device=device)
    a_sorted = torch.empty(num_pairs, dtype=torch.int32, device=device)
    groups = torch.empty(K * ((num_rows + 63) // 64 + 1), dtype=torch.int32, device=device)
    ws = workspace(L.wcn_pairs_sort_workspace_bytes(num_rows, K, num_pairs), device)
    check(L.wcn_pairs_sort_by_out(ptr(gathered.contiguous()), ptr(ascending.contiguous()),
                                  host_offsets, K, num_rows, ptr(g_sorted), ptr(a_sorted),
                                  ptr(groups), ptr(ws), ws.numel(), stream_ptr(device)),
          "wcn_pairs_sort_by_out")
    # The re-ordering keeps one pair per (offset, ascending-side row).  Kernel maps of duplicate-free
    # coordinate sets have no more than that.  Lists with more (hand-made ones, or a map over
    # coordinates that repeat rows) lose pairs here that the reference's atomic scatter adds up
    # (sparse_conv.py:495-544): for the forward product they are refused instead of contracted
    # wrongly; for the input gradient one contribution per row is what the reference's explicit path
    # keeps as well (`grad_in[in_map] += ...` without accumulation, sparse_conv.py:350), so that
    # case only warns.  One read of K counts (a wait for the stream) per map object, skipped for
    # the maps the builder made over a coordinate table that reported no repeated key.
    vouched = getattr(km, "_keys_unique", False) and getattr(km, "_from_builder", False)
    if num_pairs > 0 and not vouched:
        kept_pairs = int(groups.view(K, (num_rows + 63) // 64 + 1)[:, -1].sum())
        if kept_pairs != num_pairs:
            what = (f"kernel map holds {num_pairs - kept_pairs} pairs that repeat an (offset, "
                    f"{'output' if by == 'out' else 'input'} row) of another pair; the device contraction "
                    "takes one pair per offset and row (coordinates with repeated rows? make them unique first)")
            if by == "out":
                raise ValueError(what)
            warnings.warn(what + "; the input gradient keeps the pair with the lowest row", RuntimeWarning,
                          stacklevel=3)
    kept = (g_sorted, a_sorted, groups, num_rows)
    if by == "out":
        km._by_out = kept
    else:
        km._by_in = kept
    return kept[:3]


@torch.no_grad()
def sparse_conv_forward(in_features: Tensor, weight: Tensor, kernel_map: IntSearchResult,
                        num_out_coords: int, bias: Optional[Tensor] = None,
                        compute_dtype: Optional[torch.dtype] = None,
                        residual: Optional[Tensor] = None, relu: bool = False,
                        keep_prepared_weight: bool = False) -> Tensor:
    """out = bias + sum_k scatter(X[in_k] @ W[k]) on the GPU (replaces the per-offset loops of
    sparse_conv.py:281-311 / :358-415 / :495-544 and the native GEMMs they call).

    A map whose out_maps does not ascend inside every offset (a hand-made one, the exchanged map
    of a transposed convolution) is re-ordered once; that step takes at most one pair per (offset,
    output row), which every kernel map of duplicate-free coordinates satisfies, and raises
    ValueError for lists that hold more (the reference would add all of them up).

    `residual` ((num_out_coords, c_out), added to the sums) and `relu` (clamp at zero) are done in
    the kernel's epilogue before the one rounding (wcn_sparse_conv_fwd_fused): what a residual
    block does with two more elementwise kernels after the convolution.  Not in the reference.

    `keep_prepared_weight` (not in the reference either): the kernels read the weight as zero-padded
    transposed tiles, which every call makes anew with one more kernel.  With this flag the tiles
    are kept on the tensor object `weight` and the call enqueues the contraction alone
    (wcn_sparse_conv_fwd_prepared; same results bit for bit).  They are made again when the
    tensor's version counter, address, dtype or shape changes; a change that the counter does not
    see (through `weight.data`, say) is the caller's to avoid, which is why it is a flag."""
    require_device(in_features, "in_features")
    if in_features.ndim != 2 or weight.ndim != 3 or weight.shape[1] != in_features.shape[1]:
        raise ValueError(f"shape mismatch: features {tuple(in_features.shape)}, "
                         f"weight {tuple(weight.shape)}")
    if len(kernel_map) != weight.shape[0]:
        raise ValueError(f"kernel map has {len(kernel_map)} offsets, weight has {weight.shape[0]}")
    x = in_features if compute_dtype is None else in_features.to(compute_dtype)
    if x.dtype not in DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {x.dtype}")
    x = x.contiguous()

    def as_rows(t):  # another tensor of the call, in the features' dtype and contiguous
        if t is None or (t.dtype == x.dtype and t.is_contiguous()):
            return t
        return t.detach().to(x.dtype).contiguous()

    b = as_rows(bias)
    # Feature rows that are not whole 16-byte vectors (the 3-channel input of a network's stem)
    # would take the library's slow general kernel: zero-pad the channels instead (the matching
    # weight rows are zero, the result is unchanged).
    vec = 16 // x.element_size()
    pad = 0
    if x.shape[1] % vec != 0 and x.shape[0] > 0:
        pad = vec - x.shape[1] % vec
        x = torch.nn.functional.pad(x, (0, pad))

    def make_w():
        w = weight.detach()
        if w.dtype != x.dtype and w.dtype != torch.float32:
            w = w.to(x.dtype)
        if pad:
            w = torch.nn.functional.pad(w, (0, 0, 0, pad))
        return w.contiguous()

    km = kernel_map
    K, c_in, c_out = weight.shape[0], weight.shape[1] + pad, weight.shape[2]
    device = x.device
    out = torch.empty((num_out_coords, c_out), dtype=x.dtype, device=device)
    L = lib()
    in_maps, out_maps = km.in_maps, km.out_maps
    if km._single_out and num_out_coords > 0 and x.shape[0] > 0 and x.dtype in (torch.float16, torch.bfloat16) \
            and int(km.offsets[-1]) == num_out_coords \
            and L.wcn_conv_single_supported(DTYPE_CODE[x.dtype], c_in, c_out, K):
        # one pair per output row: nothing is summed, the lists are taken in the order they have
        host_offsets = _host_offsets_of(km)
        r = None
        if residual is not None:
            if tuple(residual.shape) != (num_out_coords, c_out):
                raise ValueError(f"residual has shape {tuple(residual.shape)}, the output {(num_out_coords, c_out)}")
            require_device(residual, "residual")
            r = as_rows(residual)
        code = DTYPE_CODE[x.dtype]
        if keep_prepared_weight:
            tiles = _prepared_weight(weight, make_w, x.dtype, c_in)
            check(L.wcn_sparse_conv_fwd_single(ptr(x), x.shape[0], c_in, code, ptr(tiles), code, 1, K, c_out, ptr(b),
                                               ptr(in_maps), ptr(out_maps), host_offsets, ptr(r), 1 if relu else 0,
                                               ptr(out), num_out_coords, None, 0, stream_ptr(device)),
                  "wcn_sparse_conv_fwd_single")
        else:
            w = make_w()
            nbytes = L.wcn_conv_prepared_weight_bytes(K, c_in, c_out, code)
            ws = workspace(nbytes, device)
            check(L.wcn_sparse_conv_fwd_single(ptr(x), x.shape[0], c_in, code, ptr(w), DTYPE_CODE[w.dtype], 0, K, c_out,
                                               ptr(b), ptr(in_maps), ptr(out_maps), host_offsets, ptr(r),
                                               1 if relu else 0, ptr(out), num_out_coords, ptr(ws), nbytes,
                                               stream_ptr(device)),
                  "wcn_sparse_conv_fwd_single")
        return out if out.dtype == in_features.dtype else out.to(in_features.dtype)
    group_start = None
    if not km._out_ascend and num_out_coords > 0:
        # a map whose out_maps does not ascend (transposed convolution, caller-made lists) is
        # re-ordered once and the result kept on the map object
        in_maps, out_maps, groups = _pairs_sorted(km, "out", num_out_coords)
        group_start = ptr(groups)
    elif km._group_start is not None and km._group_start[2] == (K, num_out_coords):
        group_start = ctypes.c_void_p(km._group_start[1])
    ascend = 1
    host_offsets = _host_offsets_of(km)
    iden = -1 if km.identity_map_index is None else int(km.identity_map_index)
    r = None
    if residual is not None:
        if tuple(residual.shape) != (num_out_coords, c_out):
            raise ValueError(f"residual has shape {tuple(residual.shape)}, the output {(num_out_coords, c_out)}")
        require_device(residual, "residual")
        r = as_rows(residual)
    code = DTYPE_CODE[x.dtype]
    if keep_prepared_weight and group_start is not None and num_out_coords > 0:
        tiles = _prepared_weight(weight, make_w, x.dtype, c_in)
        nbytes = L.wcn_conv_prepared_workspace_bytes(num_out_coords, K, c_in, c_out, code)
        ws = workspace(nbytes, device) if nbytes else None
        check(L.wcn_sparse_conv_fwd_prepared(ptr(x), x.shape[0], c_in, code, ptr(tiles),
                                             tiles.numel(), K, c_out, ptr(b), ptr(in_maps), ptr(out_maps),
                                             host_offsets, ptr(_device_offsets_of(km, device)), iden,
                                             group_start, ptr(r), 1 if relu else 0, ptr(out),
                                             num_out_coords, ptr(ws), nbytes, stream_ptr(device)),
              "wcn_sparse_conv_fwd_prepared")
        return out if out.dtype == in_features.dtype else out.to(in_features.dtype)
    num_pairs = int(host_offsets[K])
    nbytes = L.wcn_conv_workspace_bytes(num_out_coords, K, c_in, c_out, code, num_pairs, ascend)
    ws = workspace(nbytes, device)
    w = make_w()
    if residual is not None or relu:
        check(L.wcn_sparse_conv_fwd_fused(ptr(x), x.shape[0], c_in, DTYPE_CODE[x.dtype], ptr(w),
                                          DTYPE_CODE[w.dtype], K, c_out, ptr(b), ptr(in_maps),
                                          ptr(out_maps), host_offsets, iden, ascend, group_start,
                                          ptr(r), 1 if relu else 0, ptr(out), num_out_coords,
                                          ptr(ws), ws.numel(), stream_ptr(device)),
              "wcn_sparse_conv_fwd_fused")
        return out if out.dtype == in_features.dtype else out.to(in_features.dtype)
    check(L.wcn_sparse_conv_fwd(ptr(x), x.shape[0], c_in, DTYPE_CODE[x.dtype], ptr(w),
                                DTYPE_CODE[w.dtype], K, c_out, ptr(b), ptr(in_maps),
                                ptr(out_maps), host_offsets, iden, ascend, group_start,
                                ptr(out), num_out_coords, ptr(ws), ws.numel(), stream_ptr(device)),
          "wcn_sparse_conv_fwd")
    return out if out.dtype == in_features.dtype else out.to(in_features.dtype)


@torch.no_grad()
def sparse_conv_backward(grad_output: Tensor, in_features: Tensor, weight: Tensor,
                         kernel_map: IntSearchResult, compute_dtype: Optional[torch.dtype] = None,
                         need_input_grad: bool = True, need_weight_grad: bool = True):
    """Gradients of the contraction on the GPU (replaces the per-offset loops of
    sparse_conv.py:314-355 / :418-492 / :547-627 and the native GEMMs they call):
    dX[in_k] += dY[out_k] @ W[k]^T ;  dW[k] = X[in_k]^T @ dY[out_k], fp32 accumulation, one
    rounding.  Returns (grad_in_features or None, grad_weight or None) in the dtypes of
    in_features and weight.

    The input gradient walks the map by input row; a map whose in_maps does not ascend inside
    every offset is re-ordered once for that, keeping one pair per (offset, input row).  Where the
    lists hold more (coordinates with repeated rows) the pair with the lowest row is kept and a
    RuntimeWarning says how many were left out: the reference's explicit path keeps one such
    contribution as well (an index assignment without accumulation, sparse_conv.py:350), its
    atomic paths add them up."""
    require_device(grad_output, "grad_output")
    require_device(in_features, "in_features")
    dtype = compute_dtype or in_features.dtype
    if dtype not in DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {dtype}")
    K, c_in, c_out = weight.shape
    if len(kernel_map) != K or in_features.shape[1] != c_in or grad_output.shape[1] != c_out:
        raise ValueError(f"shape mismatch: features {tuple(in_features.shape)}, grad_output "
                         f"{tuple(grad_output.shape)}, weight {tuple(weight.shape)}, "
                         f"{len(kernel_map)} offsets")
    x = in_features.detach().to(dtype).contiguous()
    gy = grad_output.detach().to(dtype).contiguous()
    w = weight.detach()
    if w.dtype != dtype and w.dtype != torch.float32:
        w = w.to(dtype)
    w = w.contiguous()
    km = kernel_map
    n_in, n_out = x.shape[0], gy.shape[0]
    device = x.device
    L = lib()
    host_offsets = _host_offsets_of(km)
    num_pairs = int(host_offsets[K])
    iden = -1 if km.identity_map_index is None else int(km.identity_map_index)
    code = DTYPE_CODE[dtype]
    grad_x = grad_w = None

    if need_input_grad:
        if n_in == 0 or n_out == 0:
            grad_x = torch.zeros_like(x)
        else:
            symmetric = 1 if (km._symmetric and km._out_ascend and n_in == n_out) else 0
            in_maps, out_maps = km.in_maps, km.out_maps
            group_start = None
            if km._single_in and num_pairs == n_in and dtype in (torch.float16, torch.bfloat16) \
                    and L.wcn_conv_single_supported(code, c_out, c_in, K):
                # every input row is in exactly one pair: dX[in] = dY[out] @ W[k]^T, nothing summed, the
                # lists in the order they have
                nbytes = L.wcn_conv_prepared_weight_bytes(K, c_out, c_in, code)
                ws = workspace(nbytes, device)
                grad_x = torch.empty((n_in, c_in), dtype=dtype, device=device)
                check(L.wcn_sparse_conv_fwd_single(ptr(gy), n_out, c_out, code, ptr(w), DTYPE_CODE[w.dtype], 2, K,
                                                   c_in, None, ptr(out_maps), ptr(in_maps), host_offsets, None, 0,
                                                   ptr(grad_x), n_in, ptr(ws), nbytes, stream_ptr(device)),
                      "wcn_sparse_conv_fwd_single")
            elif not symmetric and not km._in_ascend:
                # general map: the lists ascending in input row are made once per map object
                out_maps, in_maps, groups = _pairs_sorted(km, "in", n_in)
                group_start = ptr(groups)
            else:
                gs = km._group_start if symmetric else km._in_group_start
                if gs is not None and gs[2] == (K, n_in):
                    group_start = ctypes.c_void_p(gs[1])
            ascend = 1
            if grad_x is None:
                ws = workspace(L.wcn_conv_workspace_bytes(n_in, K, c_out, c_in, code, num_pairs, ascend),
                               device)
                grad_x = torch.empty((n_in, c_in), dtype=dtype, device=device)
                check(L.wcn_sparse_conv_dgrad(ptr(gy), n_out, c_out, code, ptr(w), DTYPE_CODE[w.dtype], K,
                                              c_in, ptr(in_maps), ptr(out_maps), host_offsets, iden,
                                              symmetric, 1, group_start,
                                              ptr(grad_x), n_in, ptr(ws), ws.numel(), stream_ptr(device)),
                      "wcn_sparse_conv_dgrad")
        grad_x = grad_x.to(in_features.dtype)

    if need_weight_grad:
        grad_w = torch.empty((K, c_in, c_out), dtype=w.dtype, device=device)
        identity_rows = min(n_in, n_out) if iden >= 0 else 0
        ws = workspace(L.wcn_conv_wgrad_workspace_bytes(K, c_in, c_out, num_pairs, identity_rows),
                       device)
        check(L.wcn_sparse_conv_wgrad(ptr(x), n_in, c_in, ptr(gy), n_out, c_out, code,
                                      ptr(km.in_maps), ptr(km.out_maps), host_offsets, K, iden,
                                      ptr(grad_w), DTYPE_CODE[w.dtype], ptr(ws), ws.numel(),
                                      stream_ptr(device)), "wcn_sparse_conv_wgrad")
        grad_w = grad_w.to(weight.dtype)
    return grad_x, grad_w


class UnifiedSpatiallySparseConvFunction(Function):
    """autograd wrapper with the reference's argument list (sparse_conv.py:1321-1482).  The
    algorithm and block-size arguments are accepted and ignored."""

    @staticmethod
    def forward(ctx, in_features, weight, kernel_map, num_out_coords, fwd_algo=None, bwd_algo=None,
                compute_dtype=None, fwd_block_size=None, bwd_block_size=None):
        if num_out_coords == 0 or in_features.shape[0] == 0:
            out = torch.zeros((num_out_coords, weight.shape[-1]), dtype=in_features.dtype,
                              device=in_features.device)
        else:
            out = sparse_conv_forward(in_features, weight, kernel_map, num_out_coords,
                                      compute_dtype=compute_dtype)
        ctx.save_for_backward(in_features, weight)
        ctx.kernel_map = kernel_map
        ctx.compute_dtype = compute_dtype
        return out

    @staticmethod
    def backward(ctx, grad_output):
        in_features, weight = ctx.saved_tensors
        grad_x, grad_w = sparse_conv_backward(grad_output, in_features, weight, ctx.kernel_map,
                                              ctx.compute_dtype,
                                              need_input_grad=ctx.needs_input_grad[0],
                                              need_weight_grad=ctx.needs_input_grad[1])
        return grad_x, grad_w, None, None, None, None, None, None, None


SpatiallySparseConvExplicitGEMMFunction = UnifiedSpatiallySparseConvFunction


# ------------------------------------------------------------------------------------------------
# Output coordinates and kernel map
# ------------------------------------------------------------------------------------------------

def generate_output_coords_and_kernel_map(
    input_sparse_tensor: Voxels,
    kernel_size: Tuple[int, ...],
    kernel_dilation: Tuple[int, ...],
    stride: Tuple[int, ...],
    generative: bool,
    transposed: bool,
    output_spatially_sparse_tensor: Optional[Voxels],
    stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY,
    order=POINT_ORDERING.RANDOM,
) -> Tuple[Tensor, Tensor, IntSearchResult]:
    """Output coordinates (given / strided / same as input), then the kernel map, through the
    cache on the input tensor (reference: sparse_conv.py:1808-1996).  A transposed convolution
    reuses the cached forward map of the matching strided convolution with in/out exchanged."""
    if stride_mode == STRIDED_CONV_MODE.REDUCE_AND_STRIDE and any(s != 1 for s in stride):
        raise ValueError("REDUCE_AND_STRIDE reaches the map builder with stride 1 (the functional "
                         "entry point pools the input by the stride first)")
    in_coords = input_sparse_tensor.batch_indexed_coordinates

    # output coordinates: given, expanded (generative), strided, or the input's (sparse_conv.py:1843-1886)
    if output_spatially_sparse_tensor is not None:
        assert not generative, \
            "Output spatially sparse tensor is not supported with generative convolution"
        out_coords = output_spatially_sparse_tensor.batch_indexed_coordinates
        out_offsets = output_spatially_sparse_tensor.offsets
    elif generative and all(s == 1 for s in stride):
        assert not transposed, "Transposed and generative convolution is not supported yet"
        out_coords, out_offsets = expand_coords(in_coords, kernel_size=kernel_size,
                                                kernel_dilation=kernel_dilation)
    elif any(s != 1 for s in stride):
        out_coords, out_offsets = stride_coords(in_coords, stride, batch_sorted=True)
        if generative:  # the strided voxels are expanded in addition
            out_coords, out_offsets = expand_coords(out_coords, kernel_size=kernel_size,
                                                    kernel_dilation=kernel_dilation)
    else:
        out_coords, out_offsets = in_coords, input_sparse_tensor.offsets

    # optional ordering of the output rows along a space-filling curve (sparse_conv.py:1888-1896)
    if not _is_random_order(order):
        code = encode(out_coords[:, 1:].contiguous(), batch_offsets=out_offsets, order=order,
                      return_perm=True)
        out_coords = take_rows(out_coords, code.perm).contiguous()

    def make_key(is_transposed, in_off, out_off):
        return IntSearchCacheKey(kernel_size=kernel_size, kernel_dilation=kernel_dilation,
                                 transposed=is_transposed, generative=generative,
                                 stride_mode=str(stride_mode), skip_symmetric_kernel_map=False,
                                 in_offsets=in_off, out_offsets=out_off)

    key = make_key(transposed, input_sparse_tensor.offsets, out_offsets)
    cache = input_sparse_tensor.cache
    if cache is not None:
        kernel_map = cache.get(key)
        if kernel_map is not None:
            return out_coords, out_offsets, kernel_map

    # dilated kernels take the offset-based probe (the size-based one asserts dilation 1, as in the
    # reference: torch_discrete.py:445-448)
    method = "offset" if any(int(d) != 1 for d in kernel_dilation) else "size"
    if transposed:
        forward_map = None
        if cache is not None:
            forward_map = cache.get(make_key(False, out_offsets, input_sparse_tensor.offsets))
        if forward_map is None:
            forward_map = generate_kernel_map(out_coords, in_coords, stride, kernel_size,
                                              kernel_dilation, method=method,
                                              skip_symmetric_kernel_map=False)
        kernel_map = IntSearchResult(in_maps=forward_map.out_maps, out_maps=forward_map.in_maps,
                                     offsets=forward_map.offsets)
        kernel_map._in_ascend = forward_map._out_ascend
        kernel_map._in_group_start = forward_map._group_start
        kernel_map._keys_unique = getattr(forward_map, "_keys_unique", False)
        kernel_map._from_builder = getattr(forward_map, "_from_builder", False)
        kernel_map._device_offsets = forward_map._device_offsets
        # kernel as large as the stride, no dilation, a forward map of the builder's over fine voxels
        # without repeats: every fine row has its one parent, at one offset
        kernel_map._single_out = bool(
            tuple(int(k) for k in kernel_size) == tuple(int(v) for v in stride)
            and all(int(d) == 1 for d in kernel_dilation) and not generative
            and kernel_map._from_builder and kernel_map._keys_unique
            and int(forward_map.offsets[-1]) == out_coords.shape[0])
    else:
        kernel_map = generate_kernel_map(in_coords, out_coords, stride, kernel_size,
                                         kernel_dilation, method=method,
                                         skip_symmetric_kernel_map=False)
        # kernel as large as the stride over voxels without repeats: every input row is in one pair
        kernel_map._single_in = bool(
            tuple(int(k) for k in kernel_size) == tuple(int(v) for v in stride)
            and any(int(v) != 1 for v in stride) and all(int(d) == 1 for d in kernel_dilation)
            and not generative and getattr(kernel_map, "_keys_unique", False)
            and int(kernel_map.offsets[-1]) == in_coords.shape[0])

    if input_sparse_tensor.cache is None:
        input_sparse_tensor._extra_attributes["_cache"] = IntSearchCache()
    input_sparse_tensor.cache.put(key, kernel_map)
    return out_coords, out_offsets, kernel_map


# ------------------------------------------------------------------------------------------------
# Public entry point
# ------------------------------------------------------------------------------------------------

def spatially_sparse_conv(
    input_sparse_tensor: Voxels,
    weight: Tensor,
    kernel_size: Union[int, List[int], Tuple[int, ...]],
    stride: Union[int, List[int], Tuple[int, ...]] = 1,
    kernel_dilation: Union[int, List[int], Tuple[int, ...]] = 1,
    bias: Optional[Tensor] = None,
    kernel_matmul_batch_size: int = 2,
    generative: bool = False,
    output_spatially_sparse_tensor: Optional[Voxels] = None,
    transposed: bool = False,
    fwd_algo=SPARSE_CONV_FWD_ALGO_MODE.EXPLICIT_GEMM,
    bwd_algo=SPARSE_CONV_BWD_ALGO_MODE.EXPLICIT_GEMM,
    stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY,
    stride_reduce: str = "max",
    order=POINT_ORDERING.RANDOM,
    compute_dtype: Optional[torch.dtype] = None,
    implicit_matmul_fwd_block_size: Optional[int] = 16,
    implicit_matmul_bwd_block_size: Optional[int] = 16,
    residual: Optional[Union[Tensor, Voxels]] = None,
    relu: bool = False,
    keep_prepared_weight: bool = False,
) -> Voxels:
    """Sparse convolution of a Voxels tensor with weight (K, C_in, C_out)
    (reference: sparse_conv.py:1662-1805).

    `residual` (features of the output's shape, or a Voxels tensor holding them) and `relu` are not
    in the reference: out = act(conv(x) + bias + residual).  Without gradients they are carried out
    in the contraction's epilogue, on the fp32 sums before the one rounding; with gradients (and
    for 1x1x1 kernels) they are the torch operations a caller would write after the call.
    `keep_prepared_weight`: see sparse_conv_forward (used on the path without gradients)."""
    if not isinstance(input_sparse_tensor, Voxels):
        raise TypeError("Native spatially_sparse_conv expects input_sparse_tensor of type Voxels, "
                        f"got {type(input_sparse_tensor)}")
    if output_spatially_sparse_tensor is not None and \
            not isinstance(output_spatially_sparse_tensor, Voxels):
        raise TypeError("Native spatially_sparse_conv expects output_spatially_sparse_tensor of "
                        f"type Voxels or None, got {type(output_spatially_sparse_tensor)}")

    ndim = input_sparse_tensor.num_spatial_dims
    _kernel_size = ntuple(kernel_size, ndim=ndim)
    _kernel_dilation = ntuple(kernel_dilation, ndim=ndim)
    _stride = ntuple(stride, ndim=ndim)

    if isinstance(residual, Voxels):
        residual = residual.feature_tensor

    def after(out_features):  # the unfused form of the two extras
        if residual is not None:
            out_features = out_features + residual.to(out_features.dtype)
        return torch.relu(out_features) if relu else out_features

    if math.prod(_kernel_size) == 1 and math.prod(_stride) == 1:
        out_features = input_sparse_tensor.feature_tensor @ weight[0]
        if bias is not None:
            out_features = out_features + bias.to(out_features.dtype)
        return input_sparse_tensor.replace(batched_features=after(out_features))

    in_tensor_stride = input_sparse_tensor.tensor_stride
    if in_tensor_stride is None:
        in_tensor_stride = ntuple(1, ndim=ndim)

    if transposed and not generative:
        assert output_spatially_sparse_tensor is not None, \
            "Output spatially sparse tensor is required for transposed convolution"

    if not transposed:
        out_tensor_stride = tuple(o * s for o, s in zip(_stride, in_tensor_stride))
    else:
        if output_spatially_sparse_tensor is not None and \
                output_spatially_sparse_tensor.tensor_stride is not None:
            out_tensor_stride = output_spatially_sparse_tensor.tensor_stride
        else:
            out_tensor_stride = ntuple(1, ndim=ndim)
        assert any(o < i for o, i in zip(out_tensor_stride, in_tensor_stride)), \
            "Output stride is larger than input stride"

    if stride_mode == STRIDED_CONV_MODE.REDUCE_AND_STRIDE and any(s != 1 for s in _stride):
        # the input is pooled over stride-sized windows first, the convolution then runs with
        # stride 1 over the pooled voxels (sparse_conv.py:1753-1766)
        from .sparse_pool import sparse_reduce
        input_sparse_tensor = sparse_reduce(input_sparse_tensor, kernel_size=_stride, stride=_stride,
                                            reduction=stride_reduce)
        _stride = ntuple(1, ndim=ndim)

    features = input_sparse_tensor.feature_tensor
    effective_compute_dtype = compute_dtype if compute_dtype is not None else features.dtype

    out_coords, out_offsets, kernel_map = generate_output_coords_and_kernel_map(
        input_sparse_tensor=input_sparse_tensor, kernel_size=_kernel_size,
        kernel_dilation=_kernel_dilation, stride=_stride, generative=generative,
        transposed=transposed, output_spatially_sparse_tensor=output_spatially_sparse_tensor,
        stride_mode=stride_mode, order=order)
    num_out_coords = out_coords.shape[0]

    needs_grad = torch.is_grad_enabled() and (features.requires_grad or weight.requires_grad)
    if needs_grad:
        out_features = UnifiedSpatiallySparseConvFunction.apply(
            features, weight, kernel_map, num_out_coords, fwd_algo, bwd_algo,
            effective_compute_dtype, implicit_matmul_fwd_block_size,
            implicit_matmul_bwd_block_size)
        if bias is not None:
            out_features = out_features + bias.to(out_features.dtype)
        out_features = after(out_features)
    elif num_out_coords == 0 or features.shape[0] == 0:
        out_features = torch.zeros((num_out_coords, weight.shape[-1]), dtype=features.dtype,
                                   device=features.device)
        if bias is not None:
            out_features = out_features + bias.to(features.dtype)
        out_features = after(out_features)
    else:
        # inference: bias, residual and clamp are fused into the contraction's epilogue
        needs_residual_grad = residual is not None and torch.is_grad_enabled() and residual.requires_grad
        fused = not needs_residual_grad
        out_features = sparse_conv_forward(features, weight, kernel_map, num_out_coords, bias=bias,
                                           compute_dtype=effective_compute_dtype,
                                           residual=residual if fused else None,
                                           relu=relu and fused,
                                           keep_prepared_weight=keep_prepared_weight)
        if not fused:
            out_features = after(out_features)

    # The output's coordinate object.  Where the output rows are an existing tensor's (stride 1,
    # or a given output tensor) that tensor's coordinate object is reused, and a newly made one is
    # seeded with the (M, D+1) rows already at hand: either way the batch-indexed rows are not
    # rebuilt by the next layer (the reference rebuilds them in every call, geometry.py:141-142).
    if out_coords is in_coords_of(input_sparse_tensor):
        new_coords = input_sparse_tensor.batched_coordinates
    elif output_spatially_sparse_tensor is not None and \
            out_coords is in_coords_of(output_spatially_sparse_tensor):
        new_coords = output_spatially_sparse_tensor.batched_coordinates
    else:
        new_coords = IntCoords(out_coords[:, 1:], offsets=out_offsets.cpu().int())
        new_coords._batch_indexed = out_coords
    return input_sparse_tensor.replace(
        batched_coordinates=new_coords,
        batched_features=out_features,
        tensor_stride=out_tensor_stride,
    )
