"""Point pooling modules (reference: warpconvnet/nn/modules/point_pool.py:23-150)."""
from typing import Literal, Optional, Union

import torch.nn as nn

from ...ops.reductions import REDUCTIONS
from ..functional.point_pool import point_pool
from ..functional.point_unpool import FEATURE_UNPOOLING_MODE, point_unpool


class PointPoolBase(nn.Module):
    def __init__(self, reduction: Union[str, REDUCTIONS] = REDUCTIONS.MAX,
                 downsample_max_num_points: Optional[int] = None,
                 downsample_voxel_size: Optional[float] = None,
                 return_type: Literal["point", "voxel"] = "point",
                 unique_method: Literal["torch", "ravel", "morton"] = "torch",
                 avereage_pooled_coordinates: bool = False,
                 return_neighbor_search_result: bool = False):
        super().__init__()
        if isinstance(reduction, str):
            reduction = REDUCTIONS(reduction)
        self.reduction = reduction
        self.downsample_max_num_points = downsample_max_num_points
        self.downsample_voxel_size = downsample_voxel_size
        self.return_type = return_type
        self.return_neighbor_search_result = return_neighbor_search_result
        self.unique_method = unique_method
        self.avereage_pooled_coordinates = avereage_pooled_coordinates

    def forward(self, pc):
        return point_pool(pc=pc, reduction=self.reduction,
                          downsample_max_num_points=self.downsample_max_num_points,
                          downsample_voxel_size=self.downsample_voxel_size,
                          return_type=self.return_type,
                          return_neighbor_search_result=self.return_neighbor_search_result,
                          unique_method=self.unique_method,
                          avereage_pooled_coordinates=self.avereage_pooled_coordinates)


class PointMaxPool(PointPoolBase):
    def __init__(self, **kwargs):
        super().__init__(reduction=REDUCTIONS.MAX, **kwargs)


class PointAvgPool(PointPoolBase):
    def __init__(self, **kwargs):
        super().__init__(reduction=REDUCTIONS.MEAN, **kwargs)


class PointSumPool(PointPoolBase):
    def __init__(self, **kwargs):
        super().__init__(reduction=REDUCTIONS.SUM, **kwargs)


class PointUnpool(nn.Module):
    """(point_pool.py:120-150 of the reference)"""

    def __init__(self, unpooling_mode: Union[str, FEATURE_UNPOOLING_MODE] = FEATURE_UNPOOLING_MODE.REPEAT,
                 concat_unpooled_pc: bool = False):
        super().__init__()
        if isinstance(unpooling_mode, str):
            unpooling_mode = FEATURE_UNPOOLING_MODE(unpooling_mode)
        self.unpooling_mode = unpooling_mode
        self.concat_unpooled_pc = concat_unpooled_pc

    def forward(self, pooled_pc, unpooled_pc, to_unique=None):
        return point_unpool(pooled_pc=pooled_pc, unpooled_pc=unpooled_pc,
                            concat_unpooled_pc=self.concat_unpooled_pc,
                            unpooling_mode=self.unpooling_mode, to_unique=to_unique)


class PointToSparseWrapper(nn.Module):
    """Pool points into voxels, apply a module on the voxels, hand its output back to the points
    (reference: warpconvnet/nn/modules/sparse_pool.py:140-189)."""

    def __init__(self, inner_module: nn.Module, voxel_size: float,
                 reduction: Union[REDUCTIONS, str] = REDUCTIONS.MEAN,
                 unique_method: Literal["morton", "ravel", "torch"] = "morton",
                 concat_unpooled_pc: bool = True):
        super().__init__()
        self.inner_module = inner_module
        self.voxel_size = voxel_size
        self.reduction = reduction
        self.concat_unpooled_pc = concat_unpooled_pc
        self.unique_method = unique_method

    def forward(self, pc):
        from ...geometry.types.voxels import Voxels
        st, to_unique = point_pool(pc, reduction=self.reduction, downsample_voxel_size=self.voxel_size,
                                   return_type="voxel", return_to_unique=True,
                                   unique_method=self.unique_method)
        out_st = self.inner_module(st)
        assert isinstance(out_st, Voxels), "Output of inner module must be a Voxels"
        return point_unpool(out_st.to_point(self.voxel_size), pc,
                            concat_unpooled_pc=self.concat_unpooled_pc, to_unique=to_unique)
