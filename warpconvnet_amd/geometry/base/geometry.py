"""Geometry = coordinates + features + free-form extra attributes.

Mirrors warpconvnet/geometry/base/geometry.py:37-347 for what the sparse-convolution path
touches: autocast-aware `feature_tensor`, `replace()` that carries the extra attributes (and with
them the kernel-map cache) over to the new object, `to()`, `half()/float()`.
"""
from typing import Any, Dict, Optional, Union

import torch
from torch import Tensor

from ..features.cat import CatFeatures
from .coords import Coords
from .features import Features


def _autocast_view(t: Tensor) -> Tensor:
    """Under torch.autocast the features are presented in the autocast dtype
    (reference: geometry.py:17-34)."""
    if torch.is_autocast_enabled():
        amp_dtype = torch.get_autocast_dtype("cuda")
        if amp_dtype is not None:
            return t.to(dtype=amp_dtype)
    return t


def to_batched_features(features, offsets, device=None) -> Features:
    """(reference: warpconvnet/geometry/features/ops/convert.py)"""
    if isinstance(features, Features):
        return features.to(device) if device is not None else features
    if isinstance(features, Tensor):
        if features.ndim != 2:
            raise ValueError("only concatenated (N, C) features are supported on this path")
        return CatFeatures(features, offsets, device=device)
    raise TypeError(f"Unsupported features type {type(features)}")


class Geometry:
    batched_coordinates: Coords
    batched_features: Features
    _extra_attributes: Dict[str, Any]

    def __init__(self, batched_coordinates: Union[Coords, Tensor],
                 batched_features: Union[Features, Tensor], **kwargs):
        offsets = kwargs.pop("offsets", None)
        if isinstance(batched_coordinates, Tensor):
            assert offsets is not None, \
                "offsets must be provided when batched_coordinates is a tensor"
            batched_coordinates = Coords(batched_coordinates, offsets)
        self.batched_coordinates = batched_coordinates
        self.batched_features = to_batched_features(batched_features, batched_coordinates.offsets,
                                                    device=kwargs.get("device", None))
        assert batched_coordinates.offsets is self.batched_features.offsets or \
            (batched_coordinates.offsets == self.batched_features.offsets).all()
        if "_extra_attributes" in kwargs:  # flattened, as dataclasses.replace would pass it
            attr = kwargs.pop("_extra_attributes")
            assert isinstance(attr, dict), f"_extra_attributes must be a dictionary, got {attr}"
            kwargs.update(attr)
        self._extra_attributes = kwargs

    # -- tensors -------------------------------------------------------------------------------
    @property
    def coordinate_tensor(self) -> Tensor:
        return self.batched_coordinates.batched_tensor

    @property
    def coordinates(self) -> Tensor:
        return self.batched_coordinates.batched_tensor

    @property
    def feature_tensor(self) -> Tensor:
        return _autocast_view(self.batched_features.batched_tensor)

    @property
    def features(self) -> Tensor:
        return _autocast_view(self.batched_features.batched_tensor)

    @property
    def offsets(self) -> Tensor:
        return self.batched_features.offsets

    @property
    def num_spatial_dims(self) -> int:
        return self.batched_coordinates.num_spatial_dims

    @property
    def device(self):
        return self.batched_features.device

    @property
    def num_channels(self) -> int:
        return self.batched_features.num_channels

    @property
    def batch_size(self) -> int:
        return len(self.offsets) - 1

    @property
    def dtype(self):
        return self.batched_features.dtype

    def __len__(self) -> int:
        return len(self.batched_coordinates)

    # -- extra attributes ----------------------------------------------------------------------
    @property
    def extra_attributes(self) -> Dict[str, Any]:
        return self._extra_attributes.copy()

    @property
    def cache(self):
        return self._extra_attributes.get("_cache")

    # -- functional updates --------------------------------------------------------------------
    def replace(self, batched_coordinates: Optional[Coords] = None,
                batched_features: Optional[Union[Features, Tensor]] = None, **kwargs):
        """New object with coordinates and/or features swapped; extra attributes are carried over
        and updated with kwargs (reference: geometry.py:313-347)."""
        if "_extra_attributes" in kwargs:
            kwargs = {**kwargs.pop("_extra_attributes"), **kwargs}
        assert "batched_features" not in kwargs, "Use features instead of batched_features"
        coords = batched_coordinates if batched_coordinates is not None else self.batched_coordinates
        feats = batched_features if batched_features is not None else self.batched_features
        if isinstance(feats, Tensor):
            feats = to_batched_features(feats, coords.offsets)
        return self.__class__(coords, feats, **{**self._extra_attributes, **kwargs})

    def to(self, device=None, dtype: Optional[torch.dtype] = None):
        if device is None:
            device = self.device
        return self.__class__(self.batched_coordinates.to(device=device),
                              self.batched_features.to(device=device, dtype=dtype),
                              **self._extra_attributes)

    def _map_features(self, fn):
        return self.replace(batched_features=fn(self.feature_tensor))

    def half(self):
        return self._map_features(lambda x: x.half())

    def float(self):
        return self._map_features(lambda x: x.float())

    def double(self):
        return self._map_features(lambda x: x.double())

    def equal_shape(self, value: "Geometry") -> bool:
        return self.batched_coordinates.equal_shape(value.batched_coordinates) and \
            self.batched_features.equal_shape(value.batched_features)

    def __repr__(self) -> str:
        extras = {k: v for k, v in self._extra_attributes.items() if v is not None}
        tail = "".join(f", {k}={v}" for k, v in extras.items())
        return (f"{self.__class__.__name__}(offsets={self.offsets.tolist()}, "
                f"feature_shape={tuple(self.feature_tensor.shape)}, "
                f"coords_shape={tuple(self.batched_coordinates.shape)}, device={self.device}, "
                f"dtype={self.feature_tensor.dtype}{tail})")
