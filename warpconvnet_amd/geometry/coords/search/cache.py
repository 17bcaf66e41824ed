"""Per-tensor kernel-map cache (reference: warpconvnet/geometry/coords/search/cache.py:84-153).

The key is what the reference keys on: kernel size, dilation, transposed, generative, stride
mode, skip-symmetric flag and the input / output batch offsets.
"""
from typing import Optional, Sequence, Tuple

from torch import Tensor

from .search_results import IntSearchResult


def _seq_hash(values: Sequence[int]) -> int:
    h = 0x345678
    for v in values:
        h = ((h * 1000003) ^ hash(int(v))) & 0xFFFFFFFFFFFFFFFF
    return h


class IntSearchCacheKey:
    def __init__(self, kernel_size: Tuple[int, ...], kernel_dilation: Tuple[int, ...],
                 transposed: bool, generative: bool, stride_mode: str,
                 skip_symmetric_kernel_map: bool, in_offsets: Tensor, out_offsets: Tensor):
        self.kernel_size = tuple(kernel_size)
        self.kernel_dilation = tuple(kernel_dilation)
        self.transposed = bool(transposed)
        self.generative = bool(generative)
        self.stride_mode = str(stride_mode)
        self.skip_symmetric_kernel_map = bool(skip_symmetric_kernel_map)
        self.in_offsets = in_offsets.detach().cpu().int()
        self.out_offsets = out_offsets.detach().cpu().int()

    def _scalars(self):
        return (self.kernel_size, self.kernel_dilation, self.transposed, self.generative,
                self.stride_mode, self.skip_symmetric_kernel_map)

    def __hash__(self) -> int:
        return hash((self._scalars(), _seq_hash(self.in_offsets.tolist()),
                     _seq_hash(self.out_offsets.tolist())))

    def __eq__(self, other) -> bool:
        return (isinstance(other, IntSearchCacheKey) and self._scalars() == other._scalars()
                and self.in_offsets.equal(other.in_offsets)
                and self.out_offsets.equal(other.out_offsets))

    def __repr__(self) -> str:
        return (f"IntSearchCacheKey(kernel_size={self.kernel_size}, "
                f"kernel_dilation={self.kernel_dilation}, transposed={self.transposed}, "
                f"generative={self.generative}, stride_mode={self.stride_mode}, "
                f"skip_symmetric_kernel_map={self.skip_symmetric_kernel_map}, "
                f"num_in={int(self.in_offsets[-1])}, num_out={int(self.out_offsets[-1])})")


class IntSearchCache(dict):
    def get(self, key: IntSearchCacheKey) -> Optional[IntSearchResult]:
        return super().get(key, None)

    def put(self, key: IntSearchCacheKey, value: IntSearchResult) -> None:
        super().__setitem__(key, value)

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}({len(self)} keys)"
