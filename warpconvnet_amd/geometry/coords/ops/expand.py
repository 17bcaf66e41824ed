"""Coordinate expansion for generative convolutions (reference:
warpconvnet/geometry/coords/ops/expand.py:17-64)."""
from typing import Optional, Tuple

import torch
from torch import Tensor

from ..search.torch_discrete import kernel_offsets_from_size
from .stride import unique_floor_div_rows
from ....utils.gather import take_rows


@torch.no_grad()
def expand_coords(batch_indexed_coords: Tensor, kernel_size: Tuple[int, ...],
                  kernel_dilation: Tuple[int, ...],
                  kernel_batch: Optional[int] = None) -> Tuple[Tensor, Tensor]:
    """The input voxels and every voxel a kernel offset reaches from one of them, without
    duplicates, sorted by batch item, with the batch offsets.

    The reference adds the offsets in batches, searching its hash table for the new candidates
    and rebuilding it after each batch; the resulting set does not depend on the batching.  Here
    all candidate rows (the inputs first) go through the library's duplicate removal in one call
    (`wcn_stride_unique` with stride 1: the lowest row of each distinct voxel survives, in row
    order), so the output starts with the input voxels in their order, followed by the new voxels
    in the order the offsets reach them, then stably sorted by batch item.  As a set it is the
    reference's (whose order inside a batch item depends on a thread race).  `kernel_batch` is
    accepted for call compatibility.
    """
    device = batch_indexed_coords.device
    offsets = kernel_offsets_from_size(kernel_size, kernel_dilation).to(device)
    if offsets.shape[1] != batch_indexed_coords.shape[1]:
        raise ValueError("kernel size and coordinates disagree on the number of spatial dimensions")
    shifted = (batch_indexed_coords.unsqueeze(0) + offsets.unsqueeze(1)).reshape(-1, offsets.shape[1])
    rows = torch.cat([batch_indexed_coords, shifted.to(batch_indexed_coords.dtype)], dim=0)
    out, count, _ = unique_floor_div_rows(rows.contiguous(), (1,) * (rows.shape[1] - 1))
    unique = out[:count, : rows.shape[1]]
    order = torch.sort(unique[:, 0], stable=True).indices
    unique = take_rows(unique, order).contiguous()
    counts = torch.bincount(unique[:, 0]).cpu()
    out_offsets = torch.cat([torch.zeros(1, dtype=torch.int32), counts.cumsum(dim=0)], dim=0)
    return unique, out_offsets
