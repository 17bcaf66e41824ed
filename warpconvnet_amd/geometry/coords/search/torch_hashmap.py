"""Coordinate hash table on the GPU with the reference's TorchHashTable interface.

Reference: warpconvnet/geometry/coords/search/torch_hashmap.py:35-425 (CuPy launches of
warpconvnet/csrc/hashmap_kernels.cu).  Here the table is the HIP library's block table: slots hold
a 4x4x4-voxel block (packed key, 64-bit occupancy mask, rank base) instead of one voxel each, and
are built and probed by wcn_table_build / wcn_table_query.  Observable behaviour is the same:
`search` returns the row of each query among the inserted keys or -1.  Two deliberate
differences: among duplicate keys the lowest row always wins (the reference's winner depends on
a thread race), and the hash method is accepted and ignored (results never depended on it).
"""
import ctypes
import enum
from typing import Optional, Union

import numpy as np
import torch
from torch import Tensor

from ...._lib import ERR_TABLE_OVERFLOW, WcnError, check, lib, ptr, require_device, stream_ptr, \
    workspace


class HashMethod(enum.Enum):
    FNV1A = 0
    CITY = 1
    MURMUR = 2

    def kernel_suffix(self) -> str:
        return self.name.lower()


def _as_key_tensor(keys, device, what: str) -> Tensor:
    if not isinstance(keys, Tensor):
        try:
            keys = torch.as_tensor(keys, device=device)
        except Exception as e:  # noqa: BLE001
            raise TypeError(f"Could not convert input {what} to a Torch Tensor on device {device}: {e}")
    if keys.device != torch.device(device):
        keys = keys.to(device)
    if keys.dtype != torch.int32:
        if keys.dtype == torch.int64:
            keys = keys.to(dtype=torch.int32)
        else:
            raise TypeError(f"Input {what} must have dtype torch.int32 or compatible, got {keys.dtype}")
    if keys.ndim != 2:
        raise ValueError(f"Input {what} must be 2D, got {keys.ndim} dimensions")
    return keys


def _four_columns(keys: Tensor) -> Tensor:
    """The device table indexes rows of exactly four int32; narrower keys are zero padded."""
    d = keys.shape[1]
    if d == 4:
        return keys.contiguous()
    if d > 4:
        raise ValueError(f"keys with more than 4 columns are not supported, got {d}")
    pad = torch.zeros(keys.shape[0], 4 - d, dtype=torch.int32, device=keys.device)
    return torch.cat([keys, pad], dim=1).contiguous()


class TorchHashTable:
    def __init__(self, capacity: int, hash_method: HashMethod = HashMethod.CITY,
                 device: Union[str, torch.device] = "cuda"):
        if not isinstance(hash_method, HashMethod):
            raise TypeError(f"hash_method must be a HashMethod enum member, got {type(hash_method)}")
        assert capacity > 0
        self._capacity = int(capacity)
        self._hash_method_enum = hash_method
        self._device = torch.device(device)
        self._vector_keys: Optional[Tensor] = None
        self._keys4: Optional[Tensor] = None   # (N, 4) contiguous view the kernels read
        self._table: Optional[Tensor] = None   # opaque device workspace of the block table
        self._slots = 0                        # block-table slot count (power of two)
        self._key_dim = -1
        self._checked = False                  # device-side build status already read back

    # -- properties ----------------------------------------------------------------------------
    @property
    def capacity(self) -> int:
        return self._capacity

    @property
    def hash_method(self) -> HashMethod:
        return self._hash_method_enum

    @property
    def device(self) -> torch.device:
        return self._table.device if self._table is not None else self._device

    @property
    def key_dim(self) -> int:
        return self._key_dim

    # -- build ---------------------------------------------------------------------------------
    def _build(self, slots: int) -> None:
        keys = self._keys4
        n = keys.shape[0]
        L = lib()
        self._slots = int(slots)
        self._table = workspace(L.wcn_table_bytes(n, self._slots), keys.device)
        check(L.wcn_table_build(ptr(keys), n, ptr(self._table), self._slots,
                                stream_ptr(keys.device)), "wcn_table_build")
        self._checked = False

    def _grow(self) -> None:
        """Rebuild with four times the slots (after the device reported an overflow).  More slots
        shorten the probe chains and, up to 2^26 slots, mean more bins during the build; beyond
        that and four slots per key neither changes and the overflow is final."""
        n = self._keys4.shape[0]
        if self._slots >= (1 << 30) or (self._slots >= (1 << 26) and self._slots >= 4 * n):
            raise WcnError(ERR_TABLE_OVERFLOW, "wcn_table_build")
        self._build(self._slots * 4)

    def _ensure_checked(self) -> None:
        """Read the device-side build status once (this waits for the stream)."""
        while not self._checked:
            st = lib().wcn_table_read_status(ptr(self._table), None, stream_ptr(self.device))
            if st == ERR_TABLE_OVERFLOW:
                self._grow()
                continue
            check(st, "wcn_table_build")
            self._checked = True

    def insert(self, vec_keys: Tensor, threads_per_block: int = 256, _defer_check: bool = False):
        """Insert (N, key_dim) int32 keys.  Same argument checks as the reference
        (torch_hashmap.py:102-139): TypeError for non-tensors / non-int32, ValueError for wrong
        rank or a CPU tensor, AssertionError if N exceeds capacity / 2."""
        if not isinstance(vec_keys, Tensor):
            raise TypeError(f"Input vec_keys must be a PyTorch Tensor, got {type(vec_keys)}")
        require_device(vec_keys, "Input vec_keys")
        if vec_keys.ndim != 2:
            raise ValueError(f"Input vec_keys must be 2D, got {vec_keys.ndim} dimensions")
        if vec_keys.dtype != torch.int32:
            raise TypeError(f"Input vec_keys must have dtype torch.int32, got {vec_keys.dtype}")
        assert self._capacity > 0
        assert len(vec_keys) <= self._capacity / 2, \
            f"Number of keys {len(vec_keys)} exceeds capacity/2 ({self._capacity / 2})"
        self._vector_keys = vec_keys.contiguous()
        self._key_dim = vec_keys.shape[1]
        self._keys4 = _four_columns(self._vector_keys)
        self._build(lib().wcn_table_default_capacity(self._keys4.shape[0]))
        if not _defer_check:
            self._ensure_checked()

    @classmethod
    def from_keys(cls, vec_keys: Union[Tensor, np.ndarray],
                  hash_method: HashMethod = HashMethod.CITY,
                  device: Union[str, torch.device] = "cuda", _defer_check: bool = False):
        vec_keys = _as_key_tensor(vec_keys, torch.device(device), "vec_keys")
        obj = cls(capacity=max(16, 2 * len(vec_keys)), hash_method=hash_method, device=vec_keys.device)
        obj.insert(vec_keys, _defer_check=_defer_check)
        return obj

    # -- query ---------------------------------------------------------------------------------
    def search(self, search_keys: Union[Tensor, np.ndarray], threads_per_block: int = 256) -> Tensor:
        if self._table is None or self._vector_keys is None:
            raise RuntimeError("Hash table has not been populated. Call insert() or from_keys() first.")
        search_keys = _as_key_tensor(search_keys, self.device, "search_keys")
        if search_keys.shape[1] != self._key_dim:
            raise ValueError(f"Search keys dimension ({search_keys.shape[1]}) must match "
                             f"inserted keys dimension ({self._key_dim})")
        self._ensure_checked()
        q = _four_columns(search_keys)
        results = torch.empty(q.shape[0], dtype=torch.int32, device=self.device)
        check(lib().wcn_table_query(ptr(self._table), self._keys4.shape[0], self._slots, ptr(q),
                                    q.shape[0], ptr(results), stream_ptr(self.device)),
              "wcn_table_query")
        return results

    @property
    def unique_index(self) -> Tensor:
        """Sorted row indices of the distinct keys (one representative per key)."""
        if self._vector_keys is None:
            raise RuntimeError("Hash table has not been populated. Call insert() or from_keys() first.")
        found = self.search(self._vector_keys)
        return torch.unique(found[found != -1])

    @property
    def vector_keys(self) -> Tensor:
        if self._vector_keys is None:
            raise RuntimeError("Hash table has not been populated. Call insert() or from_keys() first.")
        return self._vector_keys

    @property
    def unique_vector_keys(self) -> Tensor:
        idx = self.unique_index
        if idx.numel() == 0:
            return torch.empty((0, self.key_dim), dtype=torch.int32, device=self.device)
        return self._vector_keys[idx.long()]

    # -- serialisation -------------------------------------------------------------------------
    def to_dict(self) -> dict:
        """Keys and metadata as numpy; the device table is derived data and is rebuilt on load."""
        if self._vector_keys is None:
            raise RuntimeError("Hash table has not been populated. Call insert() or from_keys() first.")
        return {"vector_keys": self._vector_keys.cpu().numpy(), "capacity": self._capacity,
                "hash_method_value": self._hash_method_enum.value, "key_dim": self._key_dim}

    @classmethod
    def from_dict(cls, data: dict, device: Union[str, torch.device] = "cuda"):
        obj = cls(capacity=data["capacity"], hash_method=HashMethod(data["hash_method_value"]),
                  device=device)
        obj.insert(torch.as_tensor(data["vector_keys"], dtype=torch.int32, device=device))
        return obj

    # -- raw handles for the kernel-map builder --------------------------------------------------
    def _raw(self):
        return self._table, self._keys4.shape[0], self._slots
