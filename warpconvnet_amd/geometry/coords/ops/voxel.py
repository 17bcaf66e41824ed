"""Duplicate removal of voxel coordinates (reference:
warpconvnet/geometry/coords/ops/voxel.py:112-152, used by Voxels.unique())."""
from typing import Optional, Tuple

import torch
from torch import Tensor

from .batch_index import batch_index_from_offset
from ..search.torch_hashmap import TorchHashTable


@torch.no_grad()
def voxel_downsample_random_indices(batched_points: Tensor, offsets: Tensor,
                                    voxel_size: Optional[float] = None) -> Tuple[Tensor, Tensor]:
    """Sorted indices of one representative per distinct voxel, and the new batch offsets.
    The representative is the lowest row of each voxel (the reference's depends on a race)."""
    n = len(batched_points)
    assert int(offsets[-1]) == n, f"Offsets {offsets} does not match the number of points {n}"
    if voxel_size is not None:
        voxel_coords = torch.floor(batched_points / voxel_size).int()
    else:
        voxel_coords = batched_points.int()
    batch_index = batch_index_from_offset(offsets).to(batched_points.device)
    keys = torch.cat([batch_index.unsqueeze(1).int(), voxel_coords], dim=1)
    table = TorchHashTable(max(16, 2 * n), device=keys.device)
    table.insert(keys)
    unique_indices = table.unique_index.long()
    counts = torch.bincount(batch_index[unique_indices], minlength=len(offsets) - 1).cpu()
    batch_offsets = torch.cat([counts.new_zeros(1), counts.cumsum(dim=0)])
    return unique_indices, batch_offsets
