"""Unpooling of pooled features back onto the points they came from (reference:
warpconvnet/nn/functional/point_unpool.py:15-66).  With the ToUnique object of the pooling this is
a gather through its inverse; without it the reference runs a nearest-neighbour search, which is
not part of this package."""
import enum
from typing import Optional, Union

import torch

from ...utils.unique import ToUnique


class FEATURE_UNPOOLING_MODE(enum.Enum):
    REPEAT = "repeat"


def point_unpool(pooled_pc, unpooled_pc, concat_unpooled_pc: bool,
                 unpooling_mode: Optional[Union[str, FEATURE_UNPOOLING_MODE]] = FEATURE_UNPOOLING_MODE.REPEAT,
                 to_unique: Optional[ToUnique] = None):
    """Every point of `unpooled_pc` receives the features of the pooled row it was reduced into."""
    if isinstance(unpooling_mode, str):
        unpooling_mode = FEATURE_UNPOOLING_MODE(unpooling_mode)
    if unpooling_mode != FEATURE_UNPOOLING_MODE.REPEAT:
        raise NotImplementedError(f"Unpooling mode {unpooling_mode} not implemented")
    if to_unique is None:
        raise NotImplementedError("unpooling without the pooling's ToUnique object needs a "
                                  "nearest-neighbour search, which is not built")
    features = to_unique.to_original(pooled_pc.features)
    if concat_unpooled_pc:
        features = torch.cat((features, unpooled_pc.feature_tensor), dim=-1)
    return unpooled_pc.replace(batched_features=features)
