"""Sorted-unique of integer rows with the CSR grouping of the originals
(reference: warpconvnet/utils/unique.py:57-251).

The reference composes torch.unique(dim=0) + a stable argsort + a cumulative sum + a scatter; here
one library call (wcn_unique_rows_csr) packs the rows into 64-bit keys, radix-sorts them once and
writes all results in one pass."""
import ctypes
from typing import Literal, Optional, Tuple

import torch
from torch import Tensor

from .._lib import check, lib, ptr, require_device, stream_ptr, workspace
from .gather import take_rows


def _run_unique(call, n: int, columns: int, dev, want_inverse: bool, want_representatives: bool):
    """Allocates the outputs of one sorted-unique call and trims them to the count it reports.
    `call(workspace, outputs..., count)` is the library call."""
    L = lib()
    ws = workspace(L.wcn_unique_rows_workspace_bytes(n), dev)
    unique_rows = torch.empty((n, columns), dtype=torch.int32, device=dev)
    to_orig = torch.empty(n, dtype=torch.int64, device=dev) if want_inverse else None
    csr_indices = torch.empty(n, dtype=torch.int64, device=dev)
    csr_offsets = torch.empty(n + 1, dtype=torch.int64, device=dev)
    to_unique = torch.empty(n, dtype=torch.int64, device=dev) if want_representatives else None
    count = ctypes.c_int64(0)
    call(ws, unique_rows, to_orig, csr_indices, csr_offsets, to_unique, count)
    m = int(count.value)
    return (unique_rows[:m], to_orig, csr_indices, csr_offsets[:m + 1],
            to_unique[:m] if to_unique is not None else None)


def _unique_rows(x: Tensor, want_inverse: bool, want_representatives: bool):
    require_device(x, "x")
    if x.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"integer rows expected, got {x.dtype}")
    flat = x.ndim == 1
    rows = (x.view(-1, 1) if flat else x)
    if rows.ndim != 2 or not 1 <= rows.shape[1] <= 4:
        raise ValueError(f"expected (N,) or (N, D <= 4) rows, got {tuple(x.shape)}")
    if x.dtype == torch.int64 and rows.numel() > 0:
        lo, hi = torch.aminmax(rows)
        if int(lo) < -(1 << 31) or int(hi) >= (1 << 31):
            raise ValueError("values outside the int32 range are not supported")
    rows32 = rows.to(torch.int32).contiguous()
    n, columns = rows32.shape

    def call(ws, unique_rows, to_orig, csr_indices, csr_offsets, to_unique, count):
        check(lib().wcn_unique_rows_csr(ptr(rows32), n, columns, ptr(ws), ws.numel(), ptr(unique_rows),
                                        ptr(to_orig), ptr(csr_indices), ptr(csr_offsets), ptr(to_unique),
                                        ctypes.byref(count), stream_ptr(rows32.device)),
              "wcn_unique_rows_csr")

    unique, to_orig, csr_indices, csr_offsets, to_unique = _run_unique(
        call, n, columns, rows32.device, want_inverse, want_representatives)
    unique = unique.to(x.dtype)
    if flat:
        unique = unique.view(-1)
    return unique, to_orig, csr_indices, csr_offsets, to_unique


@torch.no_grad()
def unique_torch(x: Tensor, dim: int = 0, stable: bool = False,
                 return_to_unique_indices: bool = False
                 ) -> Tuple[Tensor, Tensor, Tensor, Tensor, Optional[Tensor]]:
    """unique, to_orig_indices, all_to_csr_indices, all_to_csr_offsets, to_unique_indices with
        unique[to_orig_indices] == x
        x[all_to_csr_indices] == repeat_interleave(unique, counts), counts = all_to_csr_offsets.diff()
        x[to_unique_indices] == unique
    for an (N,) or (N, D <= 4) integer tensor on the device (unique.py:57-109).  The grouping is
    always stable (ascending row index inside a group) and the representative is the group's lowest
    row, both of which the reference leaves to chance."""
    assert dim == 0, "rows are compared along dim 0"
    return _unique_rows(x, True, return_to_unique_indices)


def unique_hashmap(bcoords: Tensor):
    """Sorted indices of one representative per distinct row, and the table (unique.py:127-146)."""
    from ..geometry.coords.search.torch_hashmap import TorchHashTable
    assert bcoords.is_cuda, f"Batched coordinates must be on a GPU device, got {bcoords.device}"
    table = TorchHashTable(2 * len(bcoords))
    table.insert(bcoords)
    return table.unique_index, table


class UniqueInfo:
    """Results of one sorted-unique call (unique.py:149-154).  The inverse (`to_orig_indices`) is the
    one output that costs a scatter of N words, and inference never reads it: it is derived from the
    grouping on first access."""

    def __init__(self, to_orig_indices: Optional[Tensor], to_csr_indices: Tensor, to_csr_offsets: Tensor,
                 to_unique_indices: Optional[Tensor]):
        self._to_orig_indices = to_orig_indices
        self.to_csr_indices = to_csr_indices
        self.to_csr_offsets = to_csr_offsets
        self.to_unique_indices = to_unique_indices

    @property
    def to_orig_indices(self) -> Tensor:
        if self._to_orig_indices is None:
            counts = self.to_csr_offsets.diff()
            group = torch.repeat_interleave(torch.arange(len(counts), device=counts.device), counts)
            self._to_orig_indices = torch.empty_like(group).scatter_(0, self.to_csr_indices, group)
        return self._to_orig_indices


class ToUnique:
    """(unique.py:157-251).  "torch" and "ravel" give the same result here: ravelling keeps the
    lexicographic order, and the library packs the rows into one key anyway."""

    unique_info: UniqueInfo

    def __init__(self, unique_method: Optional[Literal["torch", "ravel", "encode"]] = "torch",
                 return_to_unique_indices: bool = False, return_to_orig_indices: bool = False):
        if unique_method is None:
            unique_method = "torch"
        if unique_method == "encode":
            raise NotImplementedError("unique_method 'encode' (order of the Morton codes) is not built")
        # any other name takes the reference's plain torch.unique branch (unique.py:176-177), also
        # the "morton" that its point modules pass by default
        self.unique_method = unique_method
        self.return_to_unique_indices = return_to_unique_indices or unique_method == "ravel"
        # ask the library for the inverse when it is known to be read (gradients, unpooling);
        # otherwise it is derived on first access
        self.return_to_orig_indices = return_to_orig_indices

    def to_unique(self, x: Tensor, dim: int = 0) -> Tensor:
        assert dim == 0, "rows are compared along dim 0"
        unique, to_orig, csr_indices, csr_offsets, to_unique = _unique_rows(
            x, self.return_to_orig_indices, self.return_to_unique_indices)
        self.unique_info = UniqueInfo(to_orig, csr_indices, csr_offsets, to_unique)
        return unique

    @torch.no_grad()
    def points_to_unique_voxel_rows(self, points: Tensor, offsets: Tensor, voxel_size: float) -> Tensor:
        """`to_unique(rows)` for rows = [batch item, floor(points / voxel_size)] without ever storing
        the rows: (M, 4) int32 distinct voxel rows in ascending order."""
        require_device(points, "points")
        assert points.ndim == 2 and points.shape[1] == 3, "points must be (N, 3)"
        pts = points.detach().to(torch.float32).contiguous()
        n = pts.shape[0]
        host = [int(v) for v in offsets.tolist()]
        batch = len(host) - 1
        host_offsets = (ctypes.c_int64 * (batch + 1))(*host)
        device_offsets = None
        if batch > 64:  # beyond what the kernels take by value
            device_offsets = torch.tensor(host, dtype=torch.int64).pin_memory().to(pts.device, non_blocking=True)

        def call(ws, unique_rows, to_orig, csr_indices, csr_offsets, to_unique, count):
            check(lib().wcn_voxelize_points_csr(ptr(pts), n, host_offsets, ptr(device_offsets), batch,
                                                float(voxel_size), ptr(ws), ws.numel(), ptr(unique_rows),
                                                ptr(to_orig), ptr(csr_indices), ptr(csr_offsets),
                                                ptr(to_unique), ctypes.byref(count), stream_ptr(pts.device)),
                  "wcn_voxelize_points_csr")

        unique, to_orig, csr_indices, csr_offsets, to_unique = _run_unique(
            call, n, 4, pts.device, self.return_to_orig_indices, self.return_to_unique_indices)
        self.unique_info = UniqueInfo(to_orig, csr_indices, csr_offsets, to_unique)
        return unique

    def to_unique_csr(self, x: Tensor, dim: int = 0) -> Tuple[Tensor, Tensor, Tensor]:
        unique = self.to_unique(x, dim=dim)
        return unique, self.unique_info.to_csr_indices, self.unique_info.to_csr_offsets

    def to_original(self, unique: Tensor) -> Tensor:
        return take_rows(unique, self.unique_info.to_orig_indices)

    @property
    def to_unique_indices(self) -> Tensor:
        return self.unique_info.to_unique_indices

    @property
    def to_csr_indices(self) -> Tensor:
        return self.unique_info.to_csr_indices

    @property
    def to_csr_offsets(self) -> Tensor:
        return self.unique_info.to_csr_offsets

    @property
    def to_orig_indices(self) -> Tensor:
        return self.unique_info.to_orig_indices
