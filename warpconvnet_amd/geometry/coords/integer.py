"""Integer (voxel) coordinates (reference: warpconvnet/geometry/coords/integer.py:19-110)."""
from typing import List, Optional, Tuple, Union

import torch
from torch import Tensor

from ...utils.ntuple import ntuple
from ..base.coords import Coords
from .ops.batch_index import batch_indexed_coordinates


class IntCoords(Coords):
    def __init__(self, batched_tensor: Union[List[Tensor], Tensor],
                 offsets: Optional[Union[List[int], Tensor]] = None,
                 voxel_size: Optional[float] = None, voxel_origin: Optional[Tensor] = None,
                 tensor_stride: Optional[Union[int, Tuple[int, ...]]] = None,
                 device: Optional[str] = None):
        super().__init__(batched_tensor, offsets, device=device)
        self.voxel_size = voxel_size
        self.voxel_origin = voxel_origin
        self.tensor_stride = None
        if tensor_stride is not None:
            self.tensor_stride = ntuple(tensor_stride, ndim=self.batched_tensor.shape[1])
        self._hashmap = None
        self._batch_indexed: Optional[Tensor] = None

    def check(self):
        super().check()
        assert self.batched_tensor.dtype in (torch.int32, torch.int64), \
            "Discrete coordinates must be integers"

    def to(self, device=None, dtype=None):
        if device is None:
            device = self.device
        return self.__class__(self.batched_tensor.to(device=device), self.offsets,
                              voxel_size=self.voxel_size, voxel_origin=self.voxel_origin,
                              tensor_stride=self.tensor_stride)

    @property
    def stride(self):
        return self.tensor_stride

    def set_tensor_stride(self, tensor_stride: Union[int, Tuple[int, ...]]):
        self.tensor_stride = ntuple(tensor_stride, ndim=self.num_spatial_dims)

    @property
    def batch_indexed_coordinates(self) -> Tensor:
        """(N, D+1) rows [batch, coords].  The reference rebuilds this tensor on every access
        (geometry.py:141-142); coordinates are immutable here, so it is built once."""
        if self._batch_indexed is None:
            self._batch_indexed = batch_indexed_coordinates(self.batched_tensor, self.offsets)
        return self._batch_indexed

    @property
    def hashmap(self):
        from .search.torch_hashmap import TorchHashTable
        if self._hashmap is None:
            self._hashmap = TorchHashTable.from_keys(self.batch_indexed_coordinates)
        return self._hashmap

    def unique(self) -> "IntCoords":
        from .ops.voxel import voxel_downsample_random_indices
        idx, offsets = voxel_downsample_random_indices(self.batched_tensor, self.offsets)
        return self.__class__(self.batched_tensor[idx], offsets)
