"""Space-filling-curve ordering of voxel coordinates (reference:
warpconvnet/geometry/coords/ops/serialization.py:36-254).

`encode` returns the Morton (Z-order) code of every row and, on request, the permutation that
sorts the rows by code inside every batch item.  The codes come from the HIP library
(`wcn_morton_codes`); the sort itself is torch's (two stable passes: by code, then by batch item).
"""
import ctypes
import enum
from typing import NamedTuple, Optional, Union

import torch
from torch import Tensor

from ...._lib import check, lib, ptr, stream_ptr


class POINT_ORDERING(enum.Enum):
    RANDOM = 0
    MORTON_XYZ = 1
    MORTON_XZY = 2
    MORTON_YXZ = 3
    MORTON_YZX = 4
    MORTON_ZXY = 5
    MORTON_ZYX = 6


STR2POINT_ORDERING = {o.name.lower(): o for o in POINT_ORDERING}

POINT_ORDERING_TO_MORTON_PERMUTATIONS = {
    POINT_ORDERING.MORTON_XYZ: [0, 1, 2],
    POINT_ORDERING.MORTON_XZY: [0, 2, 1],
    POINT_ORDERING.MORTON_YXZ: [1, 0, 2],
    POINT_ORDERING.MORTON_YZX: [1, 2, 0],
    POINT_ORDERING.MORTON_ZXY: [2, 0, 1],
    POINT_ORDERING.MORTON_ZYX: [2, 1, 0],
}


class SerializationResult(NamedTuple):
    codes: Tensor
    perm: Optional[Tensor] = None
    inverse_perm: Optional[Tensor] = None
    counts: Optional[Tensor] = None


def _as_ordering(order) -> POINT_ORDERING:
    if isinstance(order, str):
        return STR2POINT_ORDERING[order.lower()]
    if isinstance(order, POINT_ORDERING):
        return order
    return STR2POINT_ORDERING[str(getattr(order, "name", order)).lower()]


@torch.no_grad()
def morton_code(coords: Tensor, threads_per_block: int = 256,
                order: Union[POINT_ORDERING, str] = POINT_ORDERING.MORTON_XYZ) -> Tensor:
    """int64 Z-order number of every (x, y, z) row, relative to the per-column minimum, the first
    axis of the ordering in the lowest bit of every triple (serialization.py:181-254,
    morton_code.cu:15-58)."""
    order = _as_ordering(order)
    assert order in POINT_ORDERING_TO_MORTON_PERMUTATIONS, f"Order '{order}' not supported for morton code"
    if coords.shape[0] == 0:
        return torch.empty(0, dtype=torch.int64)
    assert coords.shape[1] == 3, "coords must be [N, 3]"
    if not coords.is_cuda:
        raise ValueError(f"coords must be on a GPU device, got {coords.device}")
    c = coords.to(torch.int32).contiguous()
    origin = c.amin(dim=0)  # stays on the device
    axes = (ctypes.c_int32 * 3)(*POINT_ORDERING_TO_MORTON_PERMUTATIONS[order])
    codes = torch.empty(c.shape[0], dtype=torch.int64, device=c.device)
    check(lib().wcn_morton_codes(ptr(c), c.shape[0], 3, 0, ptr(origin), axes, ptr(codes),
                                 stream_ptr(c.device)), "wcn_morton_codes")
    return codes


@torch.no_grad()
def encode(grid_coord: Tensor, batch_offsets: Optional[Tensor] = None,
           order: Union[POINT_ORDERING, str] = POINT_ORDERING.MORTON_XYZ, return_perm: bool = False,
           return_inverse: bool = False, size: Optional[int] = None,
           num_buckets: Optional[int] = None):
    """Codes of the rows and, on request, the permutation sorting them by code inside every batch
    item (sorted = original[perm]) and its inverse (serialization.py:85-178)."""
    order = _as_ordering(order)
    if grid_coord.shape[0] == 0:
        codes = torch.empty(0, dtype=torch.int64)
    elif order in POINT_ORDERING_TO_MORTON_PERMUTATIONS:
        codes = morton_code(grid_coord, order=order)
    elif order == POINT_ORDERING.RANDOM:
        codes = torch.randperm(grid_coord.shape[0], device=grid_coord.device)
    else:
        raise NotImplementedError(f"Order '{order}' not supported at the moment")
    if not return_perm and not return_inverse:
        return codes
    if codes.shape[0] == 0:
        empty = torch.empty(0, dtype=torch.int64)
        return SerializationResult(codes, empty if return_perm else None,
                                   empty if return_inverse else None)
    perm = torch.sort(codes, stable=True).indices
    if batch_offsets is not None and len(batch_offsets) > 2:
        bounds = batch_offsets[1:].to(dtype=torch.int64, device="cpu")
        staged = torch.empty(bounds.shape, dtype=torch.int64, pin_memory=codes.is_cuda)
        staged.copy_(bounds)
        item = torch.searchsorted(staged.to(codes.device, non_blocking=True), perm, right=True)
        perm = perm[torch.sort(item, stable=True).indices]
    inverse = None
    if return_inverse:
        inverse = torch.zeros_like(perm).scatter_(0, perm, torch.arange(len(perm), device=perm.device))
    return SerializationResult(codes, perm, inverse)
