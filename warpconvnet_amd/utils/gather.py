"""Rows of a tensor picked by an index tensor, `src[index]`, for index tensors of any length.

With PyTorch 2.10.0+rocm7.0 on an MI355X, `src[index]` and `torch.index_select(src, 0, index)` return
wrong rows for the last 2^26 of more than 2^26 indices when a row of `src` is 16 bytes ((M, 4) int32
or fp32: a batch-indexed coordinate array), although both operands are intact and the same gather
column by column is right; rows of 4, 32 bytes and more were not affected.  Coordinate sets of that
size fit this GPU's memory many times over, so the gathers of rows in this package go through here:
up to 2^25 indices at a time."""
import torch
from torch import Tensor

_PIECE = 1 << 25


def take_rows(src: Tensor, index: Tensor) -> Tensor:
    if index.dtype == torch.bool or index.ndim != 1 or index.numel() <= _PIECE or src.ndim < 2:
        return src[index]
    return torch.cat([src[index[lo:lo + _PIECE]] for lo in range(0, index.numel(), _PIECE)], dim=0)
