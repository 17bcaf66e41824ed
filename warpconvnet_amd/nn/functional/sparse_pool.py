"""Pooling of sparse voxel tensors over a kernel map (reference:
warpconvnet/nn/functional/sparse_pool.py).

`sparse_reduce` keeps the reference's bookkeeping (strided output coordinates, the kernel-map
cache entry shared with a strided convolution of the same geometry, tensor stride, zeros for
output voxels without any input) and sends the reduction itself to the HIP library: the pairs are
grouped by output row (`wcn_map_rows_build`) and reduced with fp32 accumulation
(`wcn_sparse_pool_fwd`); the gradient runs in the same library (`wcn_sparse_pool_bwd`).
"""
import ctypes
from typing import Optional, Tuple, Union

import torch
from torch import Tensor
from torch.autograd import Function

from ..._lib import DTYPE_CODE, check, lib, ptr, require_device, stream_ptr, workspace
from ...geometry.coords.integer import IntCoords
from ...geometry.coords.ops.stride import stride_coords
from ...geometry.coords.search.cache import IntSearchCache, IntSearchCacheKey
from ...geometry.coords.search.search_results import IntSearchResult
from ...geometry.coords.search.torch_discrete import generate_kernel_map
from ...geometry.types.voxels import Voxels
from ...ops.reductions import REDUCTIONS
from ...utils.ntuple import ntuple
from ...utils.gather import take_rows

_MODE = {REDUCTIONS.SUM: 0, REDUCTIONS.MEAN: 1, REDUCTIONS.MAX: 2, REDUCTIONS.MIN: 3}


def _rows_form(gathered: Tensor, grouping: Tensor, km: IntSearchResult, num_rows: int) -> Tensor:
    """Workspace holding the pairs grouped by `grouping` row (row_ptr / row_in).  It depends on
    the map alone, so it is kept on the map object: the layers and the backward passes that share
    a map share it."""
    kept = km.__dict__.setdefault("_rows_forms", {})
    key = (grouping.data_ptr(), gathered.data_ptr(), num_rows)
    if key not in kept:
        kept[key] = _build_rows_form(gathered, grouping, km, num_rows)
    return kept[key]


def _build_rows_form(gathered: Tensor, grouping: Tensor, km: IntSearchResult, num_rows: int) -> Tensor:
    L = lib()
    K = len(km)
    pairs = int(km.offsets[-1])
    ws = workspace(L.wcn_map_rows_workspace_bytes(num_rows, K, pairs), gathered.device)
    host_offsets = (ctypes.c_int64 * (K + 1))(*[int(v) for v in km.offsets.tolist()])
    check(L.wcn_map_rows_build(ptr(gathered), ptr(grouping), host_offsets, K, num_rows, ptr(ws),
                               ws.numel(), stream_ptr(gathered.device)), "wcn_map_rows_build")
    return ws


class _SparsePoolFunction(Function):
    @staticmethod
    def forward(ctx, features: Tensor, kernel_map: IntSearchResult, num_out: int, mode: int):
        require_device(features, "features")
        if features.dtype not in DTYPE_CODE:
            raise TypeError(f"unsupported feature dtype {features.dtype}")
        x = features.contiguous()
        n_in, channels = x.shape
        L = lib()
        K, pairs = len(kernel_map), int(kernel_map.offsets[-1])
        rows_out = _rows_form(kernel_map.in_maps, kernel_map.out_maps, kernel_map, num_out)
        out = torch.empty((num_out, channels), dtype=x.dtype, device=x.device)
        arg = None
        if mode >= 2:
            arg = torch.empty((num_out, channels), dtype=torch.int32, device=x.device)
        check(L.wcn_sparse_pool_fwd(ptr(x), n_in, channels, DTYPE_CODE[x.dtype], ptr(rows_out), num_out,
                                    K, pairs, mode, ptr(out), ptr(arg), stream_ptr(x.device)),
              "wcn_sparse_pool_fwd")
        ctx.kernel_map, ctx.mode, ctx.n_in, ctx.rows_out, ctx.arg = kernel_map, mode, n_in, rows_out, arg
        return out

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        km, mode, n_in = ctx.kernel_map, ctx.mode, ctx.n_in
        gy = grad_out.contiguous()
        num_out, channels = gy.shape
        L = lib()
        K, pairs = len(km), int(km.offsets[-1])
        rows_in = _rows_form(km.out_maps, km.in_maps, km, n_in)  # the map with in and out exchanged
        grad_in = torch.empty((n_in, channels), dtype=gy.dtype, device=gy.device)
        check(L.wcn_sparse_pool_bwd(ptr(gy), num_out, channels, DTYPE_CODE[gy.dtype], ptr(rows_in),
                                    ptr(ctx.rows_out), n_in, K, pairs, mode, ptr(ctx.arg), ptr(grad_in),
                                    stream_ptr(gy.device)), "wcn_sparse_pool_bwd")
        return grad_in, None, None, None


def sparse_reduce(voxels: Voxels, kernel_size: Union[int, Tuple[int, ...]],
                  stride: Optional[Union[int, Tuple[int, ...]]] = None,
                  reduction: Union[REDUCTIONS, str] = REDUCTIONS.MAX, order="random") -> Voxels:
    """Reduce the features of every strided output voxel's kernel window
    (reference: sparse_pool.py:25-120)."""
    if isinstance(reduction, str):
        reduction = REDUCTIONS(reduction)
    if reduction not in _MODE:
        raise NotImplementedError(f"reduction {reduction.value!r} is not built (min, max, mean, sum are)")
    if stride is None:
        stride = kernel_size
    ndim = voxels.num_spatial_dims
    stride = ntuple(stride, ndim=ndim)
    kernel_size = ntuple(kernel_size, ndim=ndim)
    in_tensor_stride = voxels.stride
    if in_tensor_stride is None:
        in_tensor_stride = ntuple(1, ndim=ndim)
    out_tensor_stride = tuple(o * s for o, s in zip(stride, in_tensor_stride))

    in_coords = voxels.batch_indexed_coordinates
    out_coords, out_offsets = stride_coords(in_coords, stride, order=order, batch_sorted=True)
    from .sparse_conv import STRIDED_CONV_MODE
    key = IntSearchCacheKey(kernel_size=kernel_size, kernel_dilation=ntuple(1, ndim=ndim),
                            transposed=False, generative=False,
                            stride_mode=str(STRIDED_CONV_MODE.STRIDE_ONLY),
                            skip_symmetric_kernel_map=False, in_offsets=voxels.offsets,
                            out_offsets=out_offsets)
    kernel_map = voxels.cache.get(key) if voxels.cache is not None else None
    if kernel_map is None:
        kernel_map = generate_kernel_map(in_coords, out_coords, in_to_out_stride_ratio=stride,
                                         kernel_size=kernel_size,
                                         kernel_dilation=ntuple(1, ndim=ndim),
                                         skip_symmetric_kernel_map=False)
    if voxels.cache is None:
        voxels._extra_attributes["_cache"] = IntSearchCache()
    voxels.cache.put(key, kernel_map)

    out_features = _SparsePoolFunction.apply(voxels.feature_tensor, kernel_map, out_coords.shape[0],
                                             _MODE[reduction])
    new_coords = IntCoords(out_coords[:, 1:], offsets=out_offsets.cpu().int())
    new_coords._batch_indexed = out_coords
    return voxels.replace(batched_coordinates=new_coords, batched_features=out_features,
                          stride=out_tensor_stride)


def sparse_max_pool(voxels: Voxels, kernel_size, stride=None) -> Voxels:
    return sparse_reduce(voxels, kernel_size, stride, reduction=REDUCTIONS.MAX)


def sparse_avg_pool(voxels: Voxels, kernel_size, stride=None) -> Voxels:
    return sparse_reduce(voxels, kernel_size, stride, reduction=REDUCTIONS.MEAN)


def sparse_unpool(pooled_voxels: Voxels, unpooled_voxels: Voxels, kernel_size, stride,
                  concat_unpooled_voxels: bool = False) -> Voxels:
    """Copy every pooled voxel's features back to the fine voxels of its window, through the kernel
    map the pooling left in the cache (reference: sparse_pool.py:145-188: the same torch indexing,
    differentiable by torch)."""
    ndim = pooled_voxels.num_spatial_dims
    stride = ntuple(stride, ndim=ndim)
    kernel_size = ntuple(kernel_size, ndim=ndim)
    from .sparse_conv import STRIDED_CONV_MODE
    key = IntSearchCacheKey(kernel_size=kernel_size, kernel_dilation=ntuple(1, ndim=ndim),
                            transposed=False, generative=False,
                            stride_mode=str(STRIDED_CONV_MODE.STRIDE_ONLY),
                            skip_symmetric_kernel_map=False, in_offsets=unpooled_voxels.offsets,
                            out_offsets=pooled_voxels.offsets)
    assert pooled_voxels.cache is not None
    kernel_map = pooled_voxels.cache.get(key)
    assert kernel_map is not None
    unpooled_maps, pooled_maps = kernel_map.in_maps, kernel_map.out_maps
    perm = torch.argsort(unpooled_maps)
    rep_feats = take_rows(pooled_voxels.feature_tensor, pooled_maps[perm].long())
    if concat_unpooled_voxels:
        rep_feats = torch.cat([unpooled_voxels.feature_tensor, rep_feats], dim=-1)
    return unpooled_voxels.replace(batched_features=rep_feats)
