"""Real-valued (point) coordinates (reference: warpconvnet/geometry/coords/real.py:20-44).
Neighbour search and sorting of points are not part of this package."""
from ..base.coords import Coords
from .ops.voxel import voxel_downsample_random_indices
from ...utils.gather import take_rows


class RealCoords(Coords):
    def check(self):
        super().check()
        assert self.batched_tensor.shape[-1] == 3, "Coordinates must have 3 dimensions"

    def voxel_downsample(self, voxel_size: float) -> "RealCoords":
        assert self.device.type != "cpu", "Voxel downsample is only supported on GPU"
        perm, down_offsets = voxel_downsample_random_indices(self.batched_tensor, self.offsets,
                                                             voxel_size=voxel_size)
        return self.__class__(take_rows(self.batched_tensor, perm), offsets=down_offsets)
