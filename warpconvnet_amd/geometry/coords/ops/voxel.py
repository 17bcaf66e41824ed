"""Voxel down-sampling of points and duplicate removal of voxel coordinates (reference:
warpconvnet/geometry/coords/ops/voxel.py:51-152)."""
import ctypes
from typing import Optional, Tuple

import torch
from torch import Tensor

from ...._lib import check, lib, ptr, require_device, stream_ptr
from ....utils.unique import ToUnique
from .batch_index import batch_index_from_offset
from ..search.torch_hashmap import TorchHashTable


@torch.no_grad()
def voxel_rows(batched_points: Tensor, offsets: Tensor, voxel_size: float) -> Tensor:
    """(N, 4) int32 rows [batch item, floor(p / voxel_size)] of (N, 3) fp32 points on the device:
    `torch.floor(batched_points / voxel_size).int()` with the batch column in front
    (voxel.py:92-95), made by one kernel."""
    require_device(batched_points, "batched_points")
    assert batched_points.ndim == 2 and batched_points.shape[1] == 3, "points must be (N, 3)"
    pts = batched_points.detach().to(torch.float32).contiguous()
    n = pts.shape[0]
    host = [int(v) for v in offsets.tolist()]
    batch = len(host) - 1
    host_offsets = (ctypes.c_int64 * (batch + 1))(*host)
    device_offsets = None
    if batch > 64:  # beyond what the kernel takes by value
        staged = torch.tensor(host, dtype=torch.int64).pin_memory()
        device_offsets = staged.to(pts.device, non_blocking=True)
    rows = torch.empty((n, 4), dtype=torch.int32, device=pts.device)
    check(lib().wcn_voxel_rows(ptr(pts), n, host_offsets, ptr(device_offsets), batch, float(voxel_size),
                               ptr(rows), stream_ptr(pts.device)), "wcn_voxel_rows")
    return rows


def _offsets_of_sorted_batch_column(rows: Tensor, batch_size: int) -> Tensor:
    """CPU offsets (B + 1) of rows whose first column (the batch item) ascends."""
    col = rows[:, 0].contiguous()
    marks = torch.arange(batch_size + 1, device=rows.device, dtype=col.dtype)
    return torch.searchsorted(col, marks).cpu()


@torch.no_grad()
def voxel_downsample_csr_mapping(batched_points: Tensor, offsets: Tensor, voxel_size: float,
                                 unique_method: Optional[str] = None, return_to_orig_indices: bool = False
                                 ) -> Tuple[Tensor, Tensor, Tensor, Tensor, ToUnique]:
    """Distinct voxels of the points in ascending (batch, x, y, z) order with the grouping of the
    points by voxel (voxel.py:51-109):
        unique_coords   (M, 4) int32 rows [batch, x, y, z]  ((M, 3) without the batch column for B = 1)
        unique_offsets  (B + 1) CPU offsets of the voxels
        to_csr_indices  (N) points grouped by voxel, to_csr_offsets (M + 1) the groups
        to_unique       the ToUnique object (to_unique_indices, to_orig_indices ...)."""
    n = len(batched_points)
    batch = len(offsets) - 1
    assert int(offsets[-1]) == n, f"Offsets {offsets} does not match the number of points {n}"
    to_unique = ToUnique(return_to_unique_indices=True, unique_method=unique_method,
                         return_to_orig_indices=return_to_orig_indices)
    unique_rows = to_unique.points_to_unique_voxel_rows(batched_points, offsets, voxel_size)
    to_csr_indices, to_csr_offsets = to_unique.to_csr_indices, to_unique.to_csr_offsets
    if batch == 1:
        unique_offsets = torch.IntTensor([0, len(unique_rows)])
        unique_coords = unique_rows[:, 1:]
    else:
        unique_offsets = _offsets_of_sorted_batch_column(unique_rows, batch)
        unique_coords = unique_rows
    assert len(unique_offsets) == batch + 1
    to_unique.unique_rows = unique_rows  # (M, 4) with the batch column, whatever B is
    return unique_coords, unique_offsets, to_csr_indices, to_csr_offsets, to_unique


@torch.no_grad()
def voxel_downsample_random_indices(batched_points: Tensor, offsets: Tensor,
                                    voxel_size: Optional[float] = None) -> Tuple[Tensor, Tensor]:
    """Sorted indices of one representative per distinct voxel, and the new batch offsets.
    The representative is the lowest row of each voxel (the reference's depends on a race)."""
    n = len(batched_points)
    assert int(offsets[-1]) == n, f"Offsets {offsets} does not match the number of points {n}"
    if (voxel_size is not None and batched_points.is_cuda and batched_points.dtype == torch.float32
            and batched_points.shape[1] == 3):
        keys = voxel_rows(batched_points, offsets, voxel_size)  # one kernel for floor, cast, batch column, cat
    else:
        if voxel_size is not None:
            voxel_coords = torch.floor(batched_points / voxel_size).int()
        else:
            voxel_coords = batched_points.int()
        batch_index = batch_index_from_offset(offsets).to(batched_points.device)
        keys = torch.cat([batch_index.unsqueeze(1).int(), voxel_coords], dim=1)
    table = TorchHashTable(max(16, 2 * n), device=keys.device)
    table.insert(keys)
    unique_indices = table.unique_index.long()
    counts = torch.bincount(keys[unique_indices, 0], minlength=len(offsets) - 1).cpu()
    batch_offsets = torch.cat([counts.new_zeros(1), counts.cumsum(dim=0)])
    return unique_indices, batch_offsets


def _voxel_rows_of(points_or_cells: Tensor, offsets: Tensor, voxel_size: Optional[float]) -> Tensor:
    if voxel_size is not None and points_or_cells.dtype == torch.float32:
        return voxel_rows(points_or_cells, offsets, voxel_size)
    cells = (torch.floor(points_or_cells / voxel_size) if voxel_size is not None else points_or_cells).int()
    batch_index = batch_index_from_offset(offsets).to(cells.device)
    return torch.cat([batch_index.unsqueeze(1).int(), cells], dim=1)


@torch.no_grad()
def voxel_downsample_mapping(up_batched_points: Tensor, up_offsets: Tensor, down_batched_points: Tensor,
                             down_offsets: Tensor, voxel_size: Optional[float] = None,
                             find_nearest_for_invalid: bool = False) -> Tuple[Tensor, Tensor, Tensor]:
    """up_map, down_map, valid with voxel(up[up_map]) == voxel(down[down_map]): every up point is
    looked up in a coordinate table of the down points' voxels (voxel.py:189-258).  Filling the
    misses with the nearest down point needs a nearest-neighbour search and is not built."""
    require_device(up_batched_points, "up_batched_points")
    assert up_batched_points.device == down_batched_points.device, \
        "up_batched_points and down_batched_points must be on the same device"
    if find_nearest_for_invalid:
        raise NotImplementedError("find_nearest_for_invalid needs a nearest-neighbour search, which is not built")
    up_rows = _voxel_rows_of(up_batched_points, up_offsets, voxel_size)
    down_rows = _voxel_rows_of(down_batched_points, down_offsets, voxel_size)
    down_map = TorchHashTable.from_keys(down_rows).search(up_rows)
    valid = down_map >= 0
    return torch.nonzero(valid).squeeze(1), down_map[valid], valid
