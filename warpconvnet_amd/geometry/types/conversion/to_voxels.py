"""Points -> Voxels (reference: warpconvnet/geometry/types/conversion/to_voxels.py:4-24)."""
from typing import Literal, Union


def points_to_voxels(points, voxel_size: float, reduction: Union[str, "REDUCTIONS"] = "random",
                     unique_method: Literal["torch", "ravel"] = "torch", return_to_unique: bool = False):
    from ....nn.functional.point_pool import point_pool
    return point_pool(points, reduction=reduction, downsample_voxel_size=voxel_size,
                      return_type="voxel", unique_method=unique_method,
                      return_to_unique=return_to_unique)
