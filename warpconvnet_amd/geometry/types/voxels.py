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

    # -- dense tensors <-> voxel lists (reference: voxels.py:75-226) -----------------------------
    @staticmethod
    def _flat_index(batch_indexed: Tensor, shape) -> Tensor:
        """Row-major position of (b, x, y, ..) rows in a (B, X, Y, ..) array."""
        flat = torch.zeros(batch_indexed.shape[0], dtype=torch.long, device=batch_indexed.device)
        for d, extent in enumerate(shape):
            flat = flat * int(extent) + batch_indexed[:, d].long()
        return flat

    @classmethod
    def from_dense(cls, dense_tensor: Tensor, dense_tensor_channel_dim: int = 1,
                   target_spatial_sparse_tensor: Optional["Voxels"] = None,
                   dense_max_coords: Optional[Tuple[int, ...]] = None, **kwargs) -> "Voxels":
        """Voxels of the non-zero positions of a (B, C, X, Y[, Z]) tensor, in row-major order, or,
        with a target tensor, the dense values at the target's coordinates (shifted so that its
        minimum coordinate is the origin; rows beyond dense_max_coords read as zero)."""
        channels_last = dense_tensor.movedim(dense_tensor_channel_dim, -1)
        grid_shape = channels_last.shape[:-1]  # (B, X, Y, ..)
        flat_features = channels_last.reshape(-1, channels_last.shape[-1])
        if target_spatial_sparse_tensor is None:
            occupied = torch.nonzero(channels_last.abs().sum(dim=-1)).int()  # sorted row-major
            feats = flat_features[cls._flat_index(occupied, grid_shape)]
            counts = torch.bincount(occupied[:, 0], minlength=grid_shape[0]).cpu()
            offsets = torch.cat([counts.new_zeros(1), counts.cumsum(0)])
            return cls(IntCoords(occupied[:, 1:].contiguous(), offsets=offsets),
                       CatFeatures(feats, offsets=offsets), **kwargs)
        target = target_spatial_sparse_tensor
        assert target.num_spatial_dims == len(grid_shape) - 1
        assert target.batch_size == grid_shape[0]
        rows = target.batch_indexed_coordinates.clone()
        rows[:, 1:] -= target.coordinate_tensor.min(dim=0).values.view(1, -1)
        outside = None
        if dense_max_coords is not None:
            limit = torch.as_tensor(dense_max_coords, device=rows.device).view(1, -1)
            outside = (rows[:, 1:] > limit).any(dim=1)
            rows[outside] = 0
        else:
            assert bool((rows[:, 1:].max(dim=0).values.cpu() < torch.tensor(grid_shape[1:])).all()), \
                "Max coords must be aligned with the spatial shape."
        feats = flat_features[cls._flat_index(rows, grid_shape)]
        if outside is not None:
            feats[outside] = 0
        return target.replace(batched_features=feats)

    def to_point(self, voxel_size: Optional[float] = None):
        """Points at the voxels' corners, `coordinates * voxel_size` (times the tensor stride)
        (reference: voxels.py:228-246)."""
        if voxel_size is None:
            assert self.voxel_size is not None, \
                "Voxel size must be provided or the object must have been initialized with a voxel size to convert to point."
            voxel_size = self.voxel_size
        if self.tensor_stride is not None:
            voxel_size = torch.tensor([[voxel_size * s for s in self.tensor_stride]], device=self.device)
        from ..coords.real import RealCoords
        from .points import Points
        return Points(RealCoords(self.coordinate_tensor * voxel_size, self.offsets), self.batched_features)

    def to_dense(self, channel_dim: int = 1, spatial_shape: Optional[Tuple[int, ...]] = None,
                 min_coords: Optional[Tuple[int, ...]] = None,
                 max_coords: Optional[Tuple[int, ...]] = None) -> Tensor:
        """(B, C, X, Y[, Z]) tensor with the features at their voxels and zeros elsewhere.  Without
        arguments the grid is the bounding box of the coordinates; with min_coords and max_coords
        or spatial_shape it is that window and voxels outside it are dropped; spatial_shape alone
        takes the coordinates as they are."""
        rows = self.batch_indexed_coordinates.clone()
        feats = self.batched_features.batched_tensor
        ndim = self.num_spatial_dims
        if spatial_shape is None and min_coords is None:
            if rows.shape[0] == 0:
                spatial_shape = (0,) * ndim
            else:
                low = rows[:, 1:].min(dim=0).values
                spatial_shape = tuple(int(v) for v in (rows[:, 1:].max(dim=0).values - low + 1))
                rows[:, 1:] -= low
        elif min_coords is not None:
            assert max_coords is not None or spatial_shape is not None
            low = torch.as_tensor(min_coords, dtype=rows.dtype, device=rows.device)
            if max_coords is not None:
                assert len(min_coords) == len(max_coords) == ndim
                spatial_shape = tuple(int(b) - int(a) + 1 for a, b in zip(min_coords, max_coords))
            extent = torch.as_tensor(spatial_shape, dtype=rows.dtype, device=rows.device)
            inside = ((rows[:, 1:] >= low) & (rows[:, 1:] < low + extent)).all(dim=1)
            rows, feats = rows[inside], feats[inside]
            rows[:, 1:] -= low
        elif len(spatial_shape) != ndim:
            raise ValueError(f"Provided spatial shape {spatial_shape} must be same length as the "
                             f"number of spatial dimensions {ndim}.")
        spatial_shape = tuple(int(s) for s in spatial_shape)
        dense = torch.zeros((self.batch_size, *spatial_shape, self.num_channels), dtype=feats.dtype,
                            device=feats.device)
        if rows.shape[0] > 0:
            dense.view(-1, self.num_channels)[self._flat_index(rows, (self.batch_size, *spatial_shape))] = feats
        return dense if channel_dim == -1 else dense.movedim(-1, channel_dim)

    def sort(self, ordering=None) -> "Voxels":
        """Rows re-ordered along a Morton curve inside every batch item (voxels.py:246-267)."""
        from ..coords.ops.serialization import POINT_ORDERING, encode
        if ordering is None:
            ordering = POINT_ORDERING.MORTON_XYZ
        if ordering == self.ordering:
            return self
        assert isinstance(self.batched_features, CatFeatures), "Features must be a CatFeatures to sort."
        result = encode(self.coordinate_tensor, batch_offsets=self.offsets, order=ordering,
                        return_perm=True)
        kwargs = self.extra_attributes
        kwargs["ordering"] = ordering
        kwargs["code"] = result.codes
        kwargs.pop("_cache", None)  # kernel maps index rows: they do not survive a re-ordering
        return self.__class__(IntCoords(self.coordinate_tensor[result.perm], self.offsets),
                              CatFeatures(self.feature_tensor[result.perm], self.offsets), **kwargs)

    def unique(self) -> "Voxels":
        """Drop duplicate voxels, keeping the lowest row of each (voxels.py:278-287)."""
        idx, batch_offsets = voxel_downsample_random_indices(self.coordinate_tensor, self.offsets)
        coords = IntCoords(self.coordinate_tensor[idx], batch_offsets)
        feats = CatFeatures(self.feature_tensor[idx], batch_offsets)
        return self.__class__(coords, feats, **self.extra_attributes)
