"""Point pooling modules (reference: warpconvnet/nn/modules/point_pool.py:23-150)."""
from typing import Literal, Optional, Union

import torch.nn as nn

from ...ops.reductions import REDUCTIONS
from ..functional.point_pool import point_pool


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
