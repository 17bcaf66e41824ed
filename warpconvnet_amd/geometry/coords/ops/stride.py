"""Strided (down-sampled) output coordinates (reference:
warpconvnet/geometry/coords/ops/stride.py:17-54 and warpconvnet/utils/unique.py:125-144)."""
import ctypes
from typing import Tuple

import torch
from torch import Tensor

from ...._lib import ERR_TABLE_OVERFLOW, check, int3, lib, ptr, stream_ptr, workspace
from ....utils.ntuple import ntuple
from .batch_index import offsets_from_batch_index
from ..search.torch_hashmap import _four_columns


@torch.no_grad()
def stride_coords(batch_indexed_coords: Tensor, stride: Tuple[int, ...],
                  order="random", batch_sorted: bool = False) -> Tuple[Tensor, Tensor]:
    """Unique rows of floor(coords / [1, *stride]) and their batch offsets.

    One call into the HIP library (floor division, table build over the coarse rows, selection of
    the lowest source row per coarse voxel, order-preserving compaction) and one host read for the
    row count.  Output rows ascend in their representative's source row, so a batch-sorted input
    yields a batch-sorted output (the reference sorts by batch afterwards, stride.py:44-48, with an
    order inside a batch that depends on a thread race; as sets the results are identical).
    Any other `order` sorts the coarse voxels of every batch item along that curve.
    `batch_sorted=True` (not in the reference) vouches that the input's batch column does not
    descend, which makes the batch offsets of the output one device search and one read.
    """
    num_spatial_dims = batch_indexed_coords.shape[1] - 1
    assert len(stride) == num_spatial_dims, \
        (f"Stride must match the number of spatial dimensions. Got {len(stride)} spatial "
         f"dimensions for but coordinates with {num_spatial_dims} spatial dimensions.")
    if all(s == 1 for s in stride):
        return batch_indexed_coords, offsets_from_batch_index(batch_indexed_coords[:, 0], ascending=batch_sorted)
    out, count, bounds = unique_floor_div_rows(batch_indexed_coords, stride, want_bounds=batch_sorted)
    unique_coords = out[:count, : num_spatial_dims + 1]
    if num_spatial_dims != 3:
        unique_coords = unique_coords.contiguous()
    out_offsets = None
    if bounds is not None and count > 0:
        # the library looked the batch items' first rows up behind the compaction and handed them
        # over with the row count: what offsets_from_batch_index(..., ascending=True) computes
        batches = sum(1 for b in bounds if b < count)  # the last batch item with rows, plus one
        if batches < len(bounds):
            out_offsets = torch.tensor(list(bounds[:batches]) + [count], dtype=torch.int64)
    if out_offsets is None:
        out_offsets = offsets_from_batch_index(unique_coords[:, 0], ascending=batch_sorted)
    if str(getattr(order, "name", order)).lower() not in ("random", "point_ordering.random"):
        # The coarse voxels of every batch item along a space-filling curve.  (The reference hands
        # the four-column rows to `encode`, whose code function accepts three columns and raises,
        # stride.py:49-51; the evident intent is the ordering of the spatial columns per batch item.)
        from .serialization import encode
        code = encode(unique_coords[:, 1:].contiguous(), batch_offsets=out_offsets, order=order,
                      return_perm=True)
        unique_coords = unique_coords[code.perm].contiguous()
    return unique_coords, out_offsets


@torch.no_grad()
def unique_floor_div_rows(batch_indexed_coords: Tensor, stride: Tuple[int, ...], want_bounds: bool = False):
    """((n, 4) buffer, M, bounds): the distinct rows of floor(coords / [1, *stride]) in its first M
    rows, ascending in the first source row of each (one library call and one host read).
    `want_bounds`: for an input whose batch column does not descend, bounds[b] (b = 0 .. 1024) is
    the first output row whose batch id is at least b, from the same read; otherwise None."""
    assert batch_indexed_coords.dtype == torch.int32
    num_spatial_dims = batch_indexed_coords.shape[1] - 1
    device = batch_indexed_coords.device
    coords = _four_columns(batch_indexed_coords)
    n = coords.shape[0]
    L = lib()
    strides = list(ntuple(stride, ndim=num_spatial_dims)) + [1] * (3 - num_spatial_dims)
    st = int3(strides)
    out = torch.empty((n, 4), dtype=torch.int32, device=device)
    first = torch.empty(n, dtype=torch.int32, device=device)
    count = ctypes.c_int64(0)
    bounds = (ctypes.c_int64 * 1025)() if want_bounds else None

    def read(ws, slots):
        if want_bounds:
            return L.wcn_stride_unique_read_bounds(ptr(ws), n, slots, ctypes.byref(count), bounds,
                                                   stream_ptr(device))
        return L.wcn_stride_unique_read_count(ptr(ws), n, slots, ctypes.byref(count), stream_ptr(device))

    if all(int(v) in (1, 2, 4) for v in strides) and n > 0:
        # Cells of 1, 2 or 4 voxels per dimension lie inside the 4x4x4 blocks of the table of the
        # fine coordinates (the one this resolution's kernel maps use, kept on the tensor object):
        # the distinct coarse rows come out of that table, no second table is built.
        from ..search.torch_discrete import _table_of
        from ..search.torch_hashmap import HashMethod
        table = _table_of(batch_indexed_coords, HashMethod.CITY, device)
        while True:
            raw, n_keys, slots = table._raw()  # the table's own four-column copy of the rows
            ws = workspace(L.wcn_stride_unique_cells_workspace_bytes(n), device)
            check(L.wcn_stride_unique_cells(ptr(raw), n_keys, slots, ptr(table._keys4), st, ptr(ws), ptr(out),
                                            ptr(first), stream_ptr(device)), "wcn_stride_unique_cells")
            status = read(ws, slots)
            if status == ERR_TABLE_OVERFLOW:
                table._grow()
                continue
            check(status, "wcn_stride_unique_cells")
            table._checked = True
            return out, int(count.value), (list(bounds) if want_bounds else None)

    slots = L.wcn_table_default_capacity(n)
    while True:
        ws = workspace(L.wcn_stride_unique_workspace_bytes(n, slots), device)
        check(L.wcn_stride_unique(ptr(coords), n, st, ptr(ws), slots, ptr(out), ptr(first),
                                  stream_ptr(device)), "wcn_stride_unique")
        status = read(ws, slots)
        if status == ERR_TABLE_OVERFLOW and slots < (1 << 30):
            slots *= 4
            continue
        check(status, "wcn_stride_unique")
        break
    return out, int(count.value), (list(bounds) if want_bounds else None)
