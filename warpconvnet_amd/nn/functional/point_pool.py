"""Pooling of points into voxels or down-sampled points (reference:
warpconvnet/nn/functional/point_pool.py:31-320).  The voxel-size path is built: points ->
voxel rows -> sorted distinct voxels + grouping (one library call each) -> reduction of the
features per voxel.  The fixed-number-of-points path needs a nearest-neighbour search, which is
not part of this package."""
from typing import Literal, Optional, Union

import torch
from torch import Tensor

from ...geometry.base.geometry import Geometry
from ...geometry.coords.integer import IntCoords
from ...geometry.coords.ops.voxel import (voxel_downsample_csr_mapping,
                                          voxel_downsample_random_indices, voxel_rows)
from ...geometry.coords.real import RealCoords
from ...geometry.coords.search.search_results import RealSearchResult
from ...ops.reductions import REDUCTIONS, segment_reduction
from ...utils.gather import take_rows

__all__ = ["point_pool"]


def _pool_by_random_sample(pc, downsample_voxel_size: Optional[float], return_type: str) -> Geometry:
    """One representative point per voxel with its own features (point_pool.py:73-107)."""
    from ...geometry.types.points import Points
    from ...geometry.types.voxels import Voxels
    keep, unique_offsets = voxel_downsample_random_indices(pc.coordinate_tensor, pc.offsets,
                                                           voxel_size=downsample_voxel_size)
    feats = take_rows(pc.features, keep)
    if return_type == "voxel":
        coords = IntCoords(torch.floor(take_rows(pc.coordinate_tensor, keep) / downsample_voxel_size).int(),
                           offsets=unique_offsets)
        return Voxels(coords, feats, voxel_size=downsample_voxel_size)
    coords = RealCoords(take_rows(pc.coordinate_tensor, keep), offsets=unique_offsets)
    return Points(coords, feats, voxel_size=downsample_voxel_size)


def point_pool(pc, reduction: Union[REDUCTIONS, str], downsample_max_num_points: Optional[int] = None,
               downsample_voxel_size: Optional[float] = None,
               return_type: Literal["point", "voxel"] = "point",
               avereage_pooled_coordinates: bool = False, return_neighbor_search_result: bool = False,
               return_to_unique: bool = False,
               unique_method: Literal["torch", "ravel", "morton"] = "torch"):
    """(point_pool.py:205-320).  Voxels come out in ascending (batch, x, y, z) order, as the
    reference's torch.unique leaves them."""
    from ...geometry.types.points import Points
    from ...geometry.types.voxels import Voxels

    if isinstance(reduction, str):
        reduction = REDUCTIONS(reduction)
    assert downsample_max_num_points is not None or downsample_voxel_size is not None, \
        "Either downsample_num_points or downsample_voxel_size must be provided."
    assert return_type in ["point", "voxel"], "return_type must be either point or voxel."
    if return_type == "voxel":
        assert not avereage_pooled_coordinates, \
            "averaging pooled coordinates is not supported for Voxels return type"
    if downsample_max_num_points is not None:
        raise NotImplementedError(
            "pooling to a fixed number of points needs a nearest-neighbour search, which is not built")
    if reduction == REDUCTIONS.RANDOM:
        assert not return_to_unique, "return_to_unique must be False when reduction is RANDOM."
        assert not return_neighbor_search_result, \
            "return_neighbor_search_result must be False when reduction is RANDOM."
        return _pool_by_random_sample(pc, downsample_voxel_size, return_type)

    feats = pc.feature_tensor
    _, unique_offsets, csr_indices, csr_offsets, to_unique = voxel_downsample_csr_mapping(
        pc.coordinate_tensor, pc.offsets, downsample_voxel_size, unique_method=unique_method,
        return_to_orig_indices=return_to_unique or (feats.requires_grad and torch.is_grad_enabled()))
    down_features = segment_reduction(feats, csr_offsets, reduction, indices=csr_indices,
                                      segment_of=lambda: to_unique.to_orig_indices)
    if return_type == "voxel":
        rows = to_unique.unique_rows  # (M, 4) [batch, x, y, z]: what the convolutions' tables are built from
        coords = IntCoords(rows[:, 1:].contiguous(), offsets=unique_offsets)
        coords._batch_indexed = rows
        out = Voxels(coords, down_features, voxel_size=downsample_voxel_size)
    else:
        if avereage_pooled_coordinates:
            xyz = segment_reduction(pc.coordinate_tensor, csr_offsets, REDUCTIONS.MEAN,
                                    indices=csr_indices, segment_of=lambda: to_unique.to_orig_indices)
        else:
            xyz = take_rows(pc.coordinate_tensor, to_unique.to_unique_indices)
        out = Points(RealCoords(xyz, offsets=unique_offsets), down_features,
                     voxel_size=downsample_voxel_size)
    if return_to_unique:
        return out, to_unique
    if return_neighbor_search_result:
        return out, RealSearchResult(to_unique.to_unique_indices, unique_offsets)
    return out
