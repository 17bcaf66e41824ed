"""Batch index / offsets conversions (reference: warpconvnet/geometry/coords/ops/batch_index.py)."""
import ctypes

import torch
from torch import Tensor

from ...._lib import check, lib, ptr, stream_ptr

_BY_VALUE_BATCHES = 64  # batch items whose offsets travel with the launch (WCN_VOXEL_MAX_BATCH)


@torch.no_grad()
def batch_index_from_offset(offsets: Tensor) -> Tensor:
    """[0,2,5] -> [0,0,1,1,1] (reference: batch_index.py:22-36)."""
    assert len(offsets) > 1, "offsets must have at least two elements. [0, N] for batch size 1"
    counts = torch.diff(offsets)
    return torch.arange(len(counts), device=offsets.device, dtype=torch.long).repeat_interleave(counts)


@torch.no_grad()
def batch_indexed_coordinates(batched_coords: Tensor, offsets: Tensor) -> Tensor:
    """(N, D) coordinates -> (N, D+1) rows [batch, ...] in the coordinate dtype and device
    (reference: batch_index.py:110-117).  For coordinates on a GPU the batch column is made on
    the device from the B + 1 offsets (sent through pinned memory without waiting for the stream)
    instead of being expanded on the host and copied."""
    if batched_coords.is_cuda:
        n = batched_coords.shape[0]
        host = offsets.tolist()
        batch = len(host) - 1
        if (batched_coords.dtype == torch.int32 and batched_coords.ndim == 2 and n > 0
                and 1 <= batch <= _BY_VALUE_BATCHES and host[0] == 0 and host[-1] == n):
            # one launch of the library instead of arange + searchsorted + cast + cat
            coords = batched_coords.contiguous()
            dims = coords.shape[1]
            rows = torch.empty((n, dims + 1), dtype=torch.int32, device=coords.device)
            host_offsets = (ctypes.c_int64 * (batch + 1))(*[int(v) for v in host])
            check(lib().wcn_batch_indexed_rows(ptr(coords), n, dims, host_offsets, batch, ptr(rows),
                                               stream_ptr(coords.device)), "wcn_batch_indexed_rows")
            return rows
        bounds = offsets[1:].to(dtype=torch.int64, device="cpu")
        staged = torch.empty(bounds.shape, dtype=torch.int64, pin_memory=True)
        staged.copy_(bounds)
        bounds_dev = staged.to(batched_coords.device, non_blocking=True)
        rows = torch.arange(n, device=batched_coords.device, dtype=torch.int64)
        batch_index = torch.searchsorted(bounds_dev, rows, right=True).to(batched_coords.dtype)
    else:
        batch_index = batch_index_from_offset(offsets).to(batched_coords)
    return torch.cat([batch_index.unsqueeze(1), batched_coords], dim=1)


_SORTED_BATCHES = 1024  # batch items a sorted batch column is searched for in one go


@torch.no_grad()
def offsets_from_batch_index(batch_index: Tensor, ascending: bool = False) -> Tensor:
    """[0,0,1,1,2,2,2,3,3] -> [0,2,4,7,9] on the CPU (reference: batch_index.py:143-161).

    `ascending=True` (not in the reference) says that the column does not descend, as the batch
    column of a Voxels object and of everything derived from it: the bounds are then found by a
    search on the device and come to the host in one read, where counting the column costs two
    reductions, a histogram and two waits."""
    n = batch_index.shape[0]
    if ascending and batch_index.is_cuda and n > 0:
        marks = torch.arange(_SORTED_BATCHES + 1, device=batch_index.device, dtype=batch_index.dtype)
        bounds = torch.searchsorted(batch_index.contiguous(), marks).cpu()
        batches = int((bounds < n).sum())  # the last batch item with rows, plus one
        if batches <= _SORTED_BATCHES:
            return torch.cat([bounds[:batches].to(torch.int64), torch.tensor([n], dtype=torch.int64)])
    counts = torch.bincount(batch_index).cpu()
    return torch.cat([torch.zeros(1, dtype=torch.int32), counts.cumsum(dim=0)], dim=0)
