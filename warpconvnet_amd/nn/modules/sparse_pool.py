"""Pooling modules over sparse voxel tensors (reference: warpconvnet/nn/modules/sparse_pool.py)."""
from typing import Literal

import torch.nn as nn

from ...geometry.types.voxels import Voxels
from ..functional.sparse_pool import sparse_reduce, sparse_unpool


class SparsePool(nn.Module):
    """Reduce the features of a Voxels object over a strided kernel window
    (reference: sparse_pool.py:18-51).  min, max, mean and sum are built."""

    def __init__(self, kernel_size: int, stride: int,
                 reduce: Literal["max", "min", "mean", "sum", "random"] = "max"):
        super().__init__()
        self.kernel_size = kernel_size
        self.stride = stride
        self.reduce = reduce

    def __repr__(self):
        return (f"{self.__class__.__name__}(kernel_size={self.kernel_size}, stride={self.stride}, "
                f"reduce={self.reduce})")

    def forward(self, st: Voxels) -> Voxels:
        return sparse_reduce(st, self.kernel_size, self.stride, self.reduce)


class SparseMaxPool(SparsePool):
    def __init__(self, kernel_size: int, stride: int):
        super().__init__(kernel_size, stride, "max")


class SparseMinPool(SparsePool):
    def __init__(self, kernel_size: int, stride: int):
        super().__init__(kernel_size, stride, "min")


class SparseAvgPool(SparsePool):
    def __init__(self, kernel_size: int, stride: int):
        super().__init__(kernel_size, stride, "mean")


class SparseUnpool(nn.Module):
    """Copy pooled features back to the voxels they were pooled from (reference:
    sparse_pool.py:111-141)."""

    def __init__(self, kernel_size: int, stride: int, concat_unpooled_st: bool = True):
        super().__init__()
        self.kernel_size = kernel_size
        self.stride = stride
        self.concat_unpooled_st = concat_unpooled_st

    def forward(self, st: Voxels, unpooled_st: Voxels) -> Voxels:
        return sparse_unpool(st, unpooled_st, self.kernel_size, self.stride, self.concat_unpooled_st)
