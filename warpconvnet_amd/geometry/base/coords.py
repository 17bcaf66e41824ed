"""Coordinate container (reference: warpconvnet/geometry/base/coords.py)."""
from .batched import BatchedTensor


class Coords(BatchedTensor):
    @property
    def num_spatial_dims(self) -> int:
        return self.batched_tensor.shape[1]
