"""Tuple normalisation helper (reference: warpconvnet/utils/ntuple.py)."""
from typing import List, Tuple, Union

import torch


def ntuple(x: Union[int, List[int], Tuple[int, ...], torch.Tensor], ndim: int) -> Tuple[int, ...]:
    """An int becomes (x,)*ndim; lists and tensors become tuples; the length must be ndim."""
    if isinstance(x, torch.Tensor):
        x = tuple(int(v) for v in x.reshape(-1).cpu().tolist())
    elif isinstance(x, int):
        x = (x,) * ndim
    elif isinstance(x, list):
        x = tuple(x)
    assert isinstance(x, tuple) and len(x) == ndim, x
    return x
