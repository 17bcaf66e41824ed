"""Depthwise sparse convolution over a kernel map (reference:
warpconvnet/nn/functional/sparse_conv_depth.py).

out[m, c] = sum over the pairs (n, m) of offset k of X[n, c] * W[k, c]; weight is (K, C).  The
forward pass, the input gradient and the weight gradient run in the HIP library
(`wcn_sparse_depthwise_fwd` over the pairs grouped by output row, the same call over the
exchanged map for the input gradient, `wcn_sparse_depthwise_wgrad`), with fp32 accumulation and
one rounding.  There is a single algorithm; the `fwd_algo` / `bwd_algo` arguments of the reference
are accepted for call compatibility and do not select anything.
"""
import ctypes
import enum
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ..._lib import DTYPE_CODE, check, lib, ptr, require_device, stream_ptr, workspace
from ...geometry.coords.search.search_results import IntSearchResult
from .sparse_pool import _rows_form


class SPARSE_DEPTHWISE_CONV_FWD_ALGO_MODE(enum.Enum):
    EXPLICIT = "explicit"
    IMPLICIT = "implicit"
    AUTO = "auto"


class SPARSE_DEPTHWISE_CONV_BWD_ALGO_MODE(enum.Enum):
    EXPLICIT = "explicit"
    IMPLICIT = "implicit"
    AUTO = "auto"


def _depthwise(features: Tensor, weight: Tensor, rows: Tensor, km: IntSearchResult, num_rows: int,
               iden: int) -> Tensor:
    L = lib()
    out = torch.empty((num_rows, features.shape[1]), dtype=features.dtype, device=features.device)
    check(L.wcn_sparse_depthwise_fwd(ptr(features), features.shape[0], features.shape[1],
                                     DTYPE_CODE[features.dtype], ptr(weight), DTYPE_CODE[weight.dtype],
                                     ptr(rows), num_rows, len(km), int(km.offsets[-1]), iden, ptr(out),
                                     stream_ptr(features.device)), "wcn_sparse_depthwise_fwd")
    return out


def _prepared(features: Tensor, weight: Tensor, compute_dtype):
    dtype = compute_dtype or features.dtype
    if dtype not in DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {dtype}")
    x = features.detach().to(dtype).contiguous()
    w = weight.detach()
    if w.dtype != dtype and w.dtype != torch.float32:
        w = w.to(dtype)
    return x, w.contiguous()


class UnifiedSpatiallySparseDepthwiseConvFunction(Function):
    """autograd wrapper with the reference's argument list (sparse_conv_depth.py:581-865)."""

    @staticmethod
    def forward(ctx, in_features, weight, kernel_map, num_out_coords, fwd_algo=None, bwd_algo=None,
                compute_dtype=None):
        require_device(in_features, "in_features")
        if weight.ndim != 2 or weight.shape[1] != in_features.shape[1] or weight.shape[0] != len(kernel_map):
            raise ValueError(f"shape mismatch: features {tuple(in_features.shape)}, weight "
                             f"{tuple(weight.shape)}, {len(kernel_map)} offsets")
        x, w = _prepared(in_features, weight, compute_dtype)
        iden = -1 if kernel_map.identity_map_index is None else int(kernel_map.identity_map_index)
        if num_out_coords == 0 or x.shape[0] == 0:
            out = torch.zeros((num_out_coords, x.shape[1]), dtype=x.dtype, device=x.device)
        else:
            rows = _rows_form(kernel_map.in_maps, kernel_map.out_maps, kernel_map, num_out_coords)
            out = _depthwise(x, w, rows, kernel_map, num_out_coords, iden)
        ctx.save_for_backward(in_features, weight)
        ctx.kernel_map, ctx.compute_dtype, ctx.iden = kernel_map, compute_dtype, iden
        return out.to(in_features.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        in_features, weight = ctx.saved_tensors
        km, iden = ctx.kernel_map, ctx.iden
        x, w = _prepared(in_features, weight, ctx.compute_dtype)
        gy = grad_output.detach().to(x.dtype).contiguous()
        n_in, n_out = x.shape[0], gy.shape[0]
        grad_x = grad_w = None
        if ctx.needs_input_grad[0]:
            if n_in == 0 or n_out == 0:
                grad_x = torch.zeros_like(x)
            else:
                rows = _rows_form(km.out_maps, km.in_maps, km, n_in)  # in and out exchanged
                grad_x = _depthwise(gy, w, rows, km, n_in, iden)
            grad_x = grad_x.to(in_features.dtype)
        if ctx.needs_input_grad[1]:
            L = lib()
            K, pairs = len(km), int(km.offsets[-1])
            irows = min(n_in, n_out) if iden >= 0 else 0
            ws = workspace(L.wcn_depthwise_wgrad_workspace_bytes(K, x.shape[1], pairs, irows), x.device)
            host_offsets = (ctypes.c_int64 * (K + 1))(*[int(v) for v in km.offsets.tolist()])
            grad_w = torch.empty_like(w)
            check(L.wcn_sparse_depthwise_wgrad(ptr(x), n_in, ptr(gy), n_out, x.shape[1],
                                               DTYPE_CODE[x.dtype], ptr(km.in_maps), ptr(km.out_maps),
                                               host_offsets, K, iden, ptr(grad_w), DTYPE_CODE[w.dtype],
                                               ptr(ws), ws.numel(), stream_ptr(x.device)),
                  "wcn_sparse_depthwise_wgrad")
            grad_w = grad_w.to(weight.dtype)
        return grad_x, grad_w, None, None, None, None, None


def spatially_sparse_depthwise_conv(in_features: Tensor, weight: Tensor, kernel_map: IntSearchResult,
                                    num_out_coords: int, fwd_algo=None, bwd_algo=None,
                                    compute_dtype: Optional[torch.dtype] = None) -> Tensor:
    """(N, C) features, (K, C) weight, kernel map -> (M, C) features
    (reference: sparse_conv_depth.py:867-910)."""
    return UnifiedSpatiallySparseDepthwiseConvFunction.apply(in_features, weight, kernel_map,
                                                             num_out_coords, fwd_algo, bwd_algo,
                                                             compute_dtype)
