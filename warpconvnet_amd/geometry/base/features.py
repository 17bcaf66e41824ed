"""Feature container base (reference: warpconvnet/geometry/base/features.py)."""
from .batched import BatchedTensor


class Features(BatchedTensor):
    @property
    def num_channels(self) -> int:
        return self.batched_tensor.shape[-1]

    @property
    def is_cat(self) -> bool:
        return True

    @property
    def is_pad(self) -> bool:
        return False
