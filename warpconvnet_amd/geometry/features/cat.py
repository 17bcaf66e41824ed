"""Concatenated features (N, C) (reference: warpconvnet/geometry/features/cat.py:12-34)."""
from ..base.features import Features


class CatFeatures(Features):
    def check(self):
        super().check()
        assert self.batched_tensor.ndim == 2, "Batched tensor must be 2D"

    def to_cat(self) -> "CatFeatures":
        return self
