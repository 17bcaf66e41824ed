"""Sparse voxel tensor (reference: warpconvnet/geometry/types/voxels.py:23-73,278-303)."""
from typing import List, Optional, Tuple, Union

import torch
from torch import Tensor

from ..base.geometry import Geometry, to_batched_features
from ..coords.integer import IntCoords
from ..coords.ops.voxel import voxel_downsample_random_indices
from ..features.cat import CatFeatures


class Voxels(Geometry):
    def __init__(self, batched_coordinates: Union[List[Tensor], Tensor, IntCoords],
                 batched_features: Union[List[Tensor], Tensor, CatFeatures],
                 offsets: Optional[Tensor] = None, device: Optional[str] = None, **kwargs):
        # tensor_stride / stride live on the coordinates, everything else in the extra attributes
        tensor_stride = kwargs.pop("tensor_stride", None) or kwargs.pop("stride", None)
        if isinstance(batched_coordinates, list):
            assert isinstance(batched_features, list), \
                "If coords is a list, features must be a list too."
            assert len(batched_coordinates) == len(batched_features)
            assert all(len(c) == len(f) for c, f in zip(batched_coordinates, batched_features))
            batched_coordinates = IntCoords(batched_coordinates, device=device,
                                            tensor_stride=tensor_stride)
        elif isinstance(batched_coordinates, Tensor):
            assert isinstance(batched_features, Tensor) and offsets is not None, \
                "If coordinate is a tensor, features must be a tensor and offsets must be provided."
            batched_coordinates = IntCoords(batched_coordinates, offsets=offsets, device=device,
                                            tensor_stride=tensor_stride)
        elif tensor_stride is not None:
            batched_coordinates.set_tensor_stride(tensor_stride)

        if isinstance(batched_features, list):
            batched_features = CatFeatures(batched_features, device=device)
        elif isinstance(batched_features, Tensor):
            batched_features = to_batched_features(batched_features, batched_coordinates.offsets,
                                                   device=device)
        Geometry.__init__(self, batched_coordinates, batched_features, **kwargs)

    # -- path-specific accessors ---------------------------------------------------------------
    @property
    def batch_indexed_coordinates(self) -> Tensor:
        return self.batched_coordinates.batch_indexed_coordinates

    @property
    def coordinate_hashmap(self):
        return self.batched_coordinates.hashmap

    @property
    def voxel_size(self):
        return self._extra_attributes.get("voxel_size", None)

    @property
    def ordering(self):
        return self._extra_attributes.get("ordering", None)

    @property
    def tensor_stride(self) -> Optional[Tuple[int, ...]]:
        return self.batched_coordinates.tensor_stride

    @property
    def stride(self) -> Optional[Tuple[int, ...]]:
        return self.tensor_stride

    def set_tensor_stride(self, tensor_stride):
        self.batched_coordinates.set_tensor_stride(tensor_stride)

    def unique(self) -> "Voxels":
        """Drop duplicate voxels, keeping the lowest row of each (voxels.py:278-287)."""
        idx, batch_offsets = voxel_downsample_random_indices(self.coordinate_tensor, self.offsets)
        coords = IntCoords(self.coordinate_tensor[idx], batch_offsets)
        feats = CatFeatures(self.feature_tensor[idx], batch_offsets)
        return self.__class__(coords, feats, **self.extra_attributes)
