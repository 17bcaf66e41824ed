"""Kernel-map generation (reference: warpconvnet/geometry/coords/search/torch_discrete.py).

`generate_kernel_map` keeps the reference signature and result type.  The device work is two
calls into the HIP library with a single host read between them:

    wcn_table_build (enqueued, not awaited)
    wcn_kmap_count  (probes + per-offset counts + prefix sums, enqueued)
    wcn_kmap_read_result  <- the only wait: offsets[K+1] and the table status
    wcn_kmap_fill   (writes in_maps / out_maps in the reference's order)

where the reference waits five times and round-trips a dense (K, M) table through HBM
(torch_discrete.py:80-157,301-337).
"""
import ctypes
import os
from typing import Literal, Optional, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor

from ...._lib import ERR_TABLE_OVERFLOW, check, int3, lib, ptr, stream_ptr, workspace
from ....utils.ntuple import ntuple
from .search_results import IntSearchResult
from .torch_hashmap import HashMethod, TorchHashTable, _four_columns


@torch.no_grad()
def kernel_offsets_from_size(kernel_size: Tuple[int, ...], kernel_dilation: Tuple[int, ...],
                             center_offset: Optional[Tuple[int, ...]] = None,
                             device="cpu") -> Tensor:
    """(K, D+1) int32 offsets, batch column 0, last spatial dimension fastest, centre (s-1)//2
    for odd sizes and 0 for even ones, scaled by the dilation (reference: torch_discrete.py:44-77)."""
    assert len(kernel_size) == len(kernel_dilation)
    axes = []
    centres = _kernel_centres(kernel_size, center_offset)
    for size, dil, centre in zip(kernel_size, kernel_dilation, centres):
        axes.append((torch.arange(size, dtype=torch.int32) - centre) * dil)
    grid = torch.meshgrid(*axes, indexing="ij")
    spatial = torch.stack([g.reshape(-1) for g in grid], dim=1)
    batch = torch.zeros(spatial.shape[0], 1, dtype=torch.int32)
    return torch.cat([batch, spatial], dim=1).to(device)


def _kernel_centres(kernel_size, center_offset=None):
    """Index of the zero offset per dimension: (s - 1) // 2 for odd sizes and 0 for even ones,
    unless the caller names it (reference: torch_discrete.py:64-67)."""
    if center_offset is None:
        return [(int(s) - 1) // 2 if int(s) % 2 == 1 else 0 for s in kernel_size]
    assert len(center_offset) == len(kernel_size)
    return [int(c) for c in center_offset]


def _pad_kernel_args(values: Sequence[int], fill: int):
    """The device kernels are written for three spatial dimensions; lower-dimensional problems
    run with size-1 / stride-1 trailing dimensions."""
    values = [int(v) for v in values]
    return values + [fill] * (3 - len(values))


# a map builder's workspace up to this size stays with its map (see _kernel_map_from_table)
_KEEP_WORKSPACE_BYTES = 256 << 20

# pairs per output row of the last map built for (kernel size, stride, size class of the row count):
# sizes the buffers the pairs are emitted into before their number is known
_PAIRS_PER_ROW = {}


@torch.no_grad()
def _kernel_map_from_table(table: TorchHashTable, out_coords: Tensor, kernel_size, stride,
                           identity_map_index: Optional[int], dilation=None,
                           centres=None) -> IntSearchResult:
    """Count, read the offsets, fill.  Handles the device-reported table overflow by rebuilding
    the table with more slots and starting over."""
    device = out_coords.device
    L = lib()
    ks, st = int3(_pad_kernel_args(kernel_size, 1)), int3(_pad_kernel_args(stride, 1))
    K = int(np.prod([int(k) for k in kernel_size]))
    out4 = _four_columns(out_coords)
    M = out4.shape[0]
    ws = workspace(L.wcn_kmap_workspace_bytes(M, K), device)
    # the library writes the result into this host tensor; the ctypes array is a view of it
    offsets64 = torch.empty(K + 1, dtype=torch.int64)
    host_offsets = (ctypes.c_int64 * (K + 1)).from_address(offsets64.data_ptr())
    # The pairs are emitted into buffers of assumed size while the pair count is still on its way
    # to the host (a voxel of a surface-like scene has a handful of neighbours, far from K); the
    # lists handed out are views of these buffers.  More pairs than assumed: the emit pass has
    # written nothing and runs again with exact buffers.
    # Eight per row unless a map of this kernel and size class was built before: then what that
    # one held, with a quarter to spare (the resolutions of a network differ a lot: 4 pairs per
    # voxel of a scene's surface at the finest level, 14 two levels down).
    shape_key = (tuple(int(k) for k in kernel_size), tuple(int(v) for v in stride), M.bit_length())
    per_row = _PAIRS_PER_ROW.get(shape_key, 8.0)
    assumed = min(K * M, max(int(1.25 * per_row * M) + 4096, 1 << 16))
    in_buf = torch.empty(assumed, dtype=torch.int32, device=device)
    out_buf = torch.empty(assumed, dtype=torch.int32, device=device)
    # A coordinate set mapped onto itself can also be probed block by block (WCN_KMAP_PROBE=blocks:
    # the 64 voxels of a block tested against an offset with one AND of occupancy masks, neighbour
    # slots fetched once per block).  Same results; measured a little slower than the row-order
    # probe on the benchmark's scenes, so it is not the default.
    onto_itself = (os.environ.get("WCN_KMAP_PROBE") == "blocks"
                   and dilation is None and all(int(v) == 1 for v in stride)
                   and out4.data_ptr() == table._keys4.data_ptr() and M == table._keys4.shape[0]
                   and bool(L.wcn_kmap_self_supported(ks, M)))

    def fill(capacity, ins, outs):
        if onto_itself:
            check(L.wcn_kmap_fill_self(M, ks, ptr(ws), capacity, ptr(ins), ptr(outs), stream_ptr(device)),
                  "wcn_kmap_fill_self")
        else:
            check(L.wcn_kmap_fill(ptr(raw), n_keys, slots, ptr(out4), M, ks, st, ptr(ws), capacity,
                                  ptr(ins), ptr(outs), stream_ptr(device)), "wcn_kmap_fill")

    while True:
        raw, n_keys, slots = table._raw()
        if onto_itself:
            check(L.wcn_kmap_count_self(ptr(raw), n_keys, slots, ks, ptr(ws), stream_ptr(device)),
                  "wcn_kmap_count_self")
        elif dilation is None:
            check(L.wcn_kmap_count(ptr(raw), n_keys, slots, ptr(out4), M, ks, st, ptr(ws),
                                   stream_ptr(device)), "wcn_kmap_count")
        else:
            check(L.wcn_kmap_count_dilated(ptr(raw), n_keys, slots, ptr(out4), M, ks, st,
                                           int3(_pad_kernel_args(dilation, 1)),
                                           int3(_pad_kernel_args(centres, 0)), ptr(ws),
                                           stream_ptr(device)), "wcn_kmap_count_dilated")
        fill(assumed, in_buf, out_buf)
        # By-product the contraction reuses: the per-64-row group starts of every offset, (K, G + 1)
        # int32, final once the count call's kernels have run.  The workspace begins with the map's
        # K + 1 offsets as int64, which the scan leaves there for the fill pass, and the group starts
        # follow: this head (about K * M / 16 bytes) is what stays with the map, for the kernels
        # that walk the map by groups and for contractions that take their offsets from device
        # memory (wcn_sparse_conv_fwd_prepared).  The probe results behind it are K * M * 4 bytes:
        # where that is more than _KEEP_WORKSPACE_BYTES the head is copied and the workspace goes
        # back to the allocator; below, the map keeps the workspace as it is and the step has no
        # copy in it.  The copy is enqueued here, before the wait for the result, so that nothing
        # stands between that wait and what the caller launches next.
        begin = L.wcn_kmap_group_start(ptr(ws), M, K) - ws.data_ptr()
        kept = ws[:begin + 4 * K * ((M + 63) // 64 + 1)]
        if ws.numel() > _KEEP_WORKSPACE_BYTES:
            kept = kept.clone()
        groups = kept[begin:]
        status = L.wcn_kmap_read_result(ptr(ws), M, K, host_offsets, stream_ptr(device))
        if status == ERR_TABLE_OVERFLOW:
            table._grow()
            continue
        check(status, "wcn_kmap_count")
        table._checked = True
        break
    total = int(host_offsets[K])
    if M > 0:
        _PAIRS_PER_ROW[shape_key] = total / M
    if 2 * total <= assumed and (assumed - total) * 4 > (32 << 20):
        # far fewer pairs than assumed, and more than 32 MiB of each buffer unused: exact copies,
        # so the map does not hold the large buffers (below that the two copy kernels cost more
        # than the memory is worth)
        in_maps, out_maps = in_buf[:total].clone(), out_buf[:total].clone()
    elif total <= assumed:
        in_maps, out_maps = in_buf[:total], out_buf[:total]
    else:
        in_maps = torch.empty(total, dtype=torch.int32, device=device)
        out_maps = torch.empty(total, dtype=torch.int32, device=device)
        fill(total, in_maps, out_maps)
    offsets = offsets64.to(torch.int32)
    result = IntSearchResult(in_maps, out_maps, offsets, identity_map_index=identity_map_index)
    result._host_offsets = host_offsets  # the contraction passes them on as they are
    result._offsets64 = offsets64        # the memory behind that array
    result._out_ascend = True  # pairs ascend in output row inside every offset
    result._group_start = (groups, groups.data_ptr(), (K, M))
    result._device_offsets = kept[:8 * (K + 1)].view(torch.int64)
    result._keys_unique = (L.wcn_kmap_last_table_flags() & 1) == 0
    return result


def _table_of(coords: Tensor, hash_method: HashMethod, device) -> TorchHashTable:
    """The coordinate table of an input tensor, built once per tensor object: the maps of
    different kernels over the same input rows (the 3x3x3 and the strided 2x2x2 map of one
    resolution of a network) share it.  It is kept on the tensor object together with the
    tensor's version counter, so an in-place change of the coordinates rebuilds it.  (The
    reference builds a new table in every call, torch_discrete.py:398-401.)"""
    kept = getattr(coords, "_wcn_table", None)
    if kept is not None and kept[0] == coords._version:
        return kept[1]
    # built from an alias of the tensor (same storage, another Python object): the table keeps its
    # keys alive, and keeping the table on `coords` itself would otherwise close a reference
    # cycle that only the garbage collector could free
    table = TorchHashTable.from_keys(coords.detach(), hash_method=hash_method, device=device,
                                     _defer_check=True)
    try:
        coords._wcn_table = (coords._version, table)
    except AttributeError:
        pass
    return table


@torch.no_grad()
def _kernel_map_more_dims(in_coords: Tensor, out_coords: Tensor, stride, kernel_size, kernel_dilation,
                          kernel_center_offset, hash_method, skip_symmetric_kernel_map) -> IntSearchResult:
    """Kernel maps over more than three spatial dimensions (the reference's offset probe takes up to
    sixteen columns, discrete_kernels.cu:129-180; its size probe is four columns wide like the
    device kernels here).  The dimensions past the third are folded into the batch column: a row
    (b, x, y, z, t, u) becomes ((b T + t - t0) U + u - u0, x, y, z), with T and U wide enough for
    every query, so that a step along t or u is a shift of the batch column and a query that leaves
    the range of the inputs lands on a batch id no input has.  One three-dimensional map per
    combination of offsets along the folded dimensions, over one table of the folded inputs; their
    per-offset lists, put together with the last dimension fastest, are the map (same pairs in the
    same order as a probe of all columns at once)."""
    device = in_coords.device
    D = out_coords.shape[1] - 1
    stride = [int(v) for v in stride]
    ks = [int(v) for v in kernel_size]
    dil = [1] * D if kernel_dilation is None else [int(v) for v in kernel_dilation]
    centres = _kernel_centres(ks, kernel_center_offset)
    steps = [[(i - centres[d]) * dil[d] for i in range(ks[d])] for d in range(D)]  # offsets per dimension
    # ranges of the folded columns over inputs and queries (two small reductions, one read)
    ext_in = in_coords[:, 4:].long()
    ext_out = out_coords[:, 4:].long() * torch.tensor(stride[3:], device=device)
    lows, highs = [], []
    if in_coords.shape[0] and out_coords.shape[0]:
        stats = torch.stack([ext_in.amin(0), ext_in.amax(0), ext_out.amin(0), ext_out.amax(0),
                             in_coords[:, 0].long().amax().expand(D - 3),
                             out_coords[:, 0].long().amax().expand(D - 3)]).cpu()
        batches = int(max(stats[4, 0], stats[5, 0])) + 1
        for e in range(D - 3):
            lows.append(min(int(stats[0, e]), int(stats[2, e]) + min(steps[3 + e])))
            highs.append(max(int(stats[1, e]), int(stats[3, e]) + max(steps[3 + e])))
    else:
        batches = 1
        lows, highs = [0] * (D - 3), [0] * (D - 3)
    widths = [h - l + 1 for l, h in zip(lows, highs)]
    if batches * int(np.prod(widths)) >= 2 ** 31:
        raise ValueError("the range of the dimensions past the third does not fit the batch column "
                         f"({batches} batch items x {widths})")

    def folded(rows, ext, shift):
        b = rows[:, 0].long()
        for e in range(D - 3):
            b = b * widths[e] + (ext[:, e] + shift[e] - lows[e])
        return torch.cat([b.to(torch.int32).unsqueeze(1), rows[:, 1:4]], dim=1).contiguous()

    in3 = folded(in_coords, ext_in, [0] * (D - 3))
    K3 = int(np.prod(ks[:3]))
    combos = [[]]
    for e in range(D - 3):
        combos = [c + [o] for c in combos for o in steps[3 + e]]
    maps = []
    for shift in combos:
        out3 = folded(out_coords, ext_out, shift)
        maps.append(generate_kernel_map(in3, out3, stride[:3], ks[:3], dil[:3], centres[:3],
                                        method="offset", hash_method=hash_method))
    counts = torch.stack([torch.diff(m.offsets) for m in maps], dim=1).reshape(-1)  # (K3, combos) -> k
    offsets = torch.cat([torch.zeros(1, dtype=counts.dtype), counts.cumsum(0)]).to(torch.int32)
    ins = [m.in_maps[int(m.offsets[k]):int(m.offsets[k + 1])] for k in range(K3) for m in maps]
    outs = [m.out_maps[int(m.offsets[k]):int(m.offsets[k + 1])] for k in range(K3) for m in maps]
    K = K3 * len(combos)
    is_odd = all(k % 2 == 1 for k in ks)
    same_count = in_coords.shape[0] == out_coords.shape[0]
    identity_map_index = K // 2 if (is_odd and same_count and centres == _kernel_centres(ks)) else None
    empty = torch.empty(0, dtype=torch.int32, device=device)
    result = IntSearchResult(torch.cat(ins) if ins else empty, torch.cat(outs) if outs else empty,
                             offsets, identity_map_index=identity_map_index)
    result._out_ascend = True
    result._from_builder = True
    result._keys_unique = all(getattr(m, "_keys_unique", False) for m in maps)
    if skip_symmetric_kernel_map and is_odd:
        half = K // 2
        end = int(result.offsets[half])
        result = IntSearchResult(result.in_maps[:end], result.out_maps[:end],
                                 result.offsets[: half + 1].clone(), identity_map_index=identity_map_index)
        result._out_ascend = True
    return result


@torch.no_grad()
def generate_kernel_map(
    batch_indexed_in_coords: Tensor,
    batch_indexed_out_coords: Tensor,
    in_to_out_stride_ratio: Tuple[int, ...],
    kernel_size: Tuple[int, ...],
    kernel_dilation: Optional[Tuple[int, ...]] = None,
    kernel_center_offset: Optional[Tuple[int, ...]] = None,
    method: Literal["offset", "size"] = "size",
    hash_method: HashMethod = HashMethod.CITY,
    skip_symmetric_kernel_map: bool = False,
) -> IntSearchResult:
    """Kernel map between input and output coordinates (reference: torch_discrete.py:365-466).

    For every kernel offset k (enumerated with the last spatial dimension fastest) and output
    row m, the query out[m] * [1, stride] + offset_k is looked up among the inputs; hits become
    pairs (in index, m) stored per offset in ascending m.  `identity_map_index` is K // 2 iff all
    kernel sizes are odd and the input and output row counts agree.
    """
    device = batch_indexed_in_coords.device
    assert device == batch_indexed_out_coords.device
    assert batch_indexed_in_coords.dtype == torch.int32
    assert batch_indexed_out_coords.dtype == torch.int32
    if skip_symmetric_kernel_map:
        assert len(batch_indexed_in_coords) == len(batch_indexed_out_coords), \
            "You can only skip symmetric kernel map if the input and output coordinates are the same."
        assert all(k % 2 == 1 for k in kernel_size), "Kernel size must be odd for symmetric skipping."
    num_spatial_dims = batch_indexed_out_coords.shape[1] - 1
    assert len(in_to_out_stride_ratio) == num_spatial_dims
    assert len(kernel_size) == num_spatial_dims
    if method not in ("size", "offset"):
        raise ValueError(f"Invalid method: {method}. Choose 'query', 'offset', or 'size'.")
    if method == "size":
        assert kernel_dilation is None or all(s == 1 for s in kernel_dilation), \
            "Kernel dilation is not supported with method='size'. Use method='offset' instead."
        assert kernel_center_offset is None, \
            "Custom kernel_center_offset is not supported with method='size'. Use method='offset' instead."
    if num_spatial_dims > 3:
        return _kernel_map_more_dims(batch_indexed_in_coords, batch_indexed_out_coords,
                                     in_to_out_stride_ratio, kernel_size, kernel_dilation,
                                     kernel_center_offset, hash_method, skip_symmetric_kernel_map)

    table = _table_of(batch_indexed_in_coords, hash_method, device)

    is_odd = all(k % 2 == 1 for k in kernel_size)
    same_count = batch_indexed_in_coords.shape[0] == batch_indexed_out_coords.shape[0]
    identity_map_index = int(np.prod(kernel_size)) // 2 if (is_odd and same_count) else None

    stride = ntuple(in_to_out_stride_ratio, ndim=num_spatial_dims)
    dilation = centres = None
    if method == "offset":
        # the reference probes a table of offsets here (torch_discrete.py:428-444); the same
        # queries come out of the size-based probe with scaled and re-centred offsets
        dilation = [1] * num_spatial_dims if kernel_dilation is None else [int(d) for d in kernel_dilation]
        assert len(dilation) == num_spatial_dims and all(d >= 1 for d in dilation)
        centres = _kernel_centres(kernel_size, kernel_center_offset)
        if centres != _kernel_centres(kernel_size):
            identity_map_index = None  # the offset at K // 2 is no longer the zero offset
        elif all(d == 1 for d in dilation):
            dilation = centres = None
    result = _kernel_map_from_table(table, batch_indexed_out_coords, kernel_size, stride,
                                    identity_map_index, dilation, centres)
    same_set = (batch_indexed_in_coords.data_ptr() == batch_indexed_out_coords.data_ptr()
                and batch_indexed_in_coords.shape == batch_indexed_out_coords.shape
                and batch_indexed_in_coords.stride() == batch_indexed_out_coords.stride())
    result._from_builder = True  # pairs come from one lookup per (offset, output row)
    result._symmetric = bool(same_set and is_odd and all(s == 1 for s in stride)
                             and centres is None and getattr(result, "_keys_unique", False))
    if skip_symmetric_kernel_map and is_odd:
        # only the offsets before the centre are kept (torch_discrete.py:286-296)
        half = int(np.prod(kernel_size)) // 2
        end = int(result.offsets[half])
        result = IntSearchResult(result.in_maps[:end], result.out_maps[:end],
                                 result.offsets[: half + 1].clone(),
                                 identity_map_index=identity_map_index)
        result._out_ascend = True
    return result
