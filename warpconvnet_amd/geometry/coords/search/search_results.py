"""Kernel-map container (reference: warpconvnet/geometry/coords/search/search_results.py:54-174).

Pairs of all kernel offsets are stored flat: offset k owns in_maps[offsets[k]:offsets[k+1]] and
the matching out_maps slice; offsets live on the CPU.
"""
from typing import List, Literal, Optional, Tuple

import torch
from torch import Tensor


class IntSearchResult:
    in_maps: Tensor
    out_maps: Tensor
    offsets: Tensor
    identity_map_index: Optional[int]

    def __init__(self, in_maps: Tensor, out_maps: Tensor, offsets: Tensor,
                 identity_map_index: Optional[int] = None):
        offsets = offsets.cpu()
        assert in_maps.shape[0] == out_maps.shape[0] == int(offsets[-1])
        self.in_maps = in_maps
        self.out_maps = out_maps
        self.offsets = offsets
        self.identity_map_index = identity_map_index
        # Device-side helpers of the HIP contraction (not part of the reference interface):
        # whether out_maps ascends inside every offset (False: the contraction re-orders the
        # pairs itself) and, from the map builder, (workspace, address, (K, M)) of the table of
        # per-64-row group starts.
        self._out_ascend = False
        self._group_start = None
        self._device_offsets = None  # (K + 1) int64 copy of `offsets` in device memory, when the builder left one
        # For the gradients: whether in_maps ascends inside every offset (the map of a transposed
        # convolution: a forward map with its lists exchanged), the group starts that belong to
        # that order, and whether exchanging in and out turns offset k into offset K - 1 - k
        # (stride-1 map of a duplicate-free coordinate set onto itself).
        self._host_offsets = None  # (K + 1) ctypes int64 array of `offsets`, when the builder left one
        self._in_ascend = False
        self._in_group_start = None
        self._symmetric = False
        # The pair lists re-ordered once for the contraction, kept with the map: ascending in
        # out_maps (`_by_out`, for the forward product over a map whose out_maps does not ascend:
        # the map of a transposed convolution) and ascending in in_maps (`_by_in`, for the input
        # gradient over a map that is not symmetric).  Each is (first list, second list,
        # group-start table, row count) or None until first needed.
        self._by_out = None
        self._by_in = None
        # every output row occurs in exactly one pair (the map of a transposed convolution that
        # undoes a strided one with kernel size = stride over duplicate-free voxels): the
        # contraction then needs neither an order of the pairs nor sums
        self._single_out = False
        # the same for the input rows (the forward map of such a strided convolution): its input
        # gradient is a product of that kind
        self._single_in = False

    @torch.no_grad()
    def __getitem__(self, idx: int) -> Tuple[Tensor, Tensor]:
        start, end = int(self.offsets[idx]), int(self.offsets[idx + 1])
        return self.in_maps[start:end], self.out_maps[start:end]

    def __len__(self) -> int:
        return len(self.offsets) - 1

    def __iter__(self):
        for i in range(len(self)):
            yield self[i]

    def numel(self, i: int) -> int:
        return int(self.offsets[i + 1] - self.offsets[i])

    @torch.no_grad()
    def get_batch(self, start_idx: int, end_idx: int,
                  out_format: Literal["list", "tensor"] = "list"):
        ins: List[Tensor] = []
        outs: List[Tensor] = []
        for i in range(start_idx, end_idx):
            a, b = self[i]
            ins.append(a)
            outs.append(b)
        if out_format == "list":
            return ins, outs
        if out_format != "tensor":
            raise ValueError(f"Invalid output format: {out_format}")
        width = max(len(a) for a in ins)
        in_t = torch.full((len(ins), width), -1, dtype=torch.int64, device=self.in_maps.device)
        out_t = torch.full((len(outs), width), -1, dtype=torch.int64, device=self.out_maps.device)
        for i, (a, b) in enumerate(zip(ins, outs)):
            in_t[i, :len(a)] = a
            out_t[i, :len(b)] = b
        return in_t, out_t

    @torch.no_grad()
    def to_csr(self) -> Tuple[Tensor, Tensor, Tensor]:
        """(in indices sorted by out index, unique out indices, CPU row offsets)."""
        out_sorted, order = torch.sort(self.out_maps)
        unique_out, counts = torch.unique(out_sorted, return_counts=True, sorted=True)
        offsets = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(counts.cpu(), dim=0)])
        return self.in_maps[order], unique_out, offsets

    def clone(self) -> "IntSearchResult":
        return IntSearchResult(self.in_maps.clone(), self.out_maps.clone(), self.offsets.clone(),
                               self.identity_map_index)

    @property
    def device(self):
        return self.in_maps.device

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}(len={len(self)}, iden_map={self.identity_map_index})"


class RealSearchResult:
    """Neighbour lists in CSR form: `neighbor_indices` (N) split by `neighbor_row_splits` (M + 1)
    (reference: search_results.py:14-60; the two-tensor constructor is the one this package uses)."""

    def __init__(self, neighbor_indices: Tensor, neighbor_row_splits: Tensor):
        self.neighbor_indices = neighbor_indices.long()
        self.neighbor_row_splits = neighbor_row_splits.long()
        self.neighbor_distances = None

    def to(self, device):
        self.neighbor_indices = self.neighbor_indices.to(device)
        self.neighbor_row_splits = self.neighbor_row_splits.to(device)
        return self
