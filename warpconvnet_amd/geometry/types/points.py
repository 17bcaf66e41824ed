"""Point collections: the front of the voxel path (reference:
warpconvnet/geometry/types/points.py:33-187,301-309).  Construction, voxel down-sampling and the
conversion to Voxels are built; neighbour search, sorting and the encodings are not."""
from typing import List, Optional, Union

import torch
from torch import Tensor

from ...ops.reductions import REDUCTIONS, segment_reduction
from ..base.geometry import Geometry, to_batched_features
from ..coords.ops.voxel import voxel_downsample_csr_mapping, voxel_downsample_random_indices
from ..coords.real import RealCoords
from ..features.cat import CatFeatures
from .conversion.to_voxels import points_to_voxels


class Points(Geometry):
    def __init__(self, batched_coordinates: Union[List[Tensor], Tensor, RealCoords],
                 batched_features: Union[List[Tensor], Tensor, CatFeatures],
                 offsets: Optional[Tensor] = None, device: Optional[str] = None, **kwargs):
        if isinstance(batched_coordinates, list):
            assert isinstance(batched_features, list), \
                "If coords is a list, features must be a list too."
            assert len(batched_coordinates) == len(batched_features)
            assert all(len(c) == len(f) for c, f in zip(batched_coordinates, batched_features)), \
                "All elements in coords and features must have same length"
            batched_coordinates = RealCoords(batched_coordinates, device=device)
        elif isinstance(batched_coordinates, Tensor):
            assert isinstance(batched_features, Tensor) and offsets is not None, \
                "If coordinate is a tensor, features must be a tensor and offsets must be provided."
            batched_coordinates = RealCoords(batched_coordinates, offsets=offsets, device=device)
        if isinstance(batched_features, list):
            batched_features = CatFeatures(batched_features, device=device)
        elif isinstance(batched_features, Tensor):
            batched_features = to_batched_features(batched_features, batched_coordinates.offsets,
                                                   device=device)
        Geometry.__init__(self, batched_coordinates, batched_features, **kwargs)

    @property
    def voxel_size(self):
        return self._extra_attributes.get("voxel_size", None)

    def voxel_downsample(self, voxel_size: float,
                         reduction: Union[REDUCTIONS, str] = REDUCTIONS.RANDOM) -> "Points":
        """One point per occupied voxel: a representative point with its own features (random), or
        a representative point with the reduced features of the voxel (points.py:120-187)."""
        assert self.device.type != "cpu", "Voxel downsample is only supported on GPU"
        if isinstance(reduction, str):
            reduction = REDUCTIONS(reduction)
        extra = self.extra_attributes
        extra["voxel_size"] = voxel_size
        assert isinstance(self.batched_features, CatFeatures), \
            "Voxel downsample is only supported for CatBatchedFeatures"
        if reduction == REDUCTIONS.RANDOM:
            keep, unique_offsets = voxel_downsample_random_indices(
                self.coordinate_tensor, self.offsets, voxel_size=voxel_size)
            return self.__class__(RealCoords(self.coordinate_tensor[keep], offsets=unique_offsets),
                                  CatFeatures(self.feature_tensor[keep], offsets=unique_offsets),
                                  **extra)
        _, unique_offsets, csr_indices, csr_offsets, to_unique = voxel_downsample_csr_mapping(
            self.coordinate_tensor, self.offsets, voxel_size)
        down = segment_reduction(self.feature_tensor, csr_offsets, reduction, indices=csr_indices,
                                 segment_of=lambda: to_unique.to_orig_indices)
        return self.__class__(
            RealCoords(self.coordinate_tensor[to_unique.to_unique_indices], offsets=unique_offsets),
            CatFeatures(down, offsets=unique_offsets), **extra)

    def to_voxels(self, voxel_size: float, reduction: Union[REDUCTIONS, str] = REDUCTIONS.MEAN):
        """(points.py:301-309)"""
        return points_to_voxels(self, voxel_size, reduction)
