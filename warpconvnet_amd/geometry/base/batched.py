"""Concatenated variable-length batch: one (N, C) tensor plus CPU offsets (B+1).

Mirrors the part of warpconvnet/geometry/base/batched.py:14-120 the sparse-convolution path
uses: construction from a list or a pre-concatenated tensor, offsets kept on the CPU, `.to()`.
"""
from typing import List, Optional, Sequence, Union

import torch
from torch import Tensor


def _cat_list(tensors: Sequence[Tensor]):
    offsets = [0]
    for t in tensors:
        offsets.append(offsets[-1] + int(t.shape[0]))
    return torch.cat(list(tensors), dim=0), torch.LongTensor(offsets)


class BatchedTensor:
    batched_tensor: Tensor
    offsets: Tensor  # (B+1,) CPU int tensor

    def __init__(self, batched_tensor: Union[List[Tensor], Tensor],
                 offsets: Optional[Union[List[int], Tensor]] = None,
                 device: Optional[str] = None):
        if isinstance(batched_tensor, (list, tuple)):
            assert offsets is None, "If batched_tensors is a list, offsets must be None."
            batched_tensor, offsets = _cat_list(batched_tensor)
        else:
            assert isinstance(batched_tensor, Tensor), "Batched tensor must be a tensor or a list"
            if offsets is None:
                offsets = [0, batched_tensor.shape[0]]
        if isinstance(offsets, (list, tuple)):
            offsets = torch.LongTensor(list(offsets))
        elif isinstance(offsets, Tensor):
            # a CPU tensor outside autograd is taken as it is: the coordinates and features of one
            # geometry then share one offsets object, which later checks recognise at once
            if offsets.is_cuda or offsets.requires_grad:
                offsets = offsets.detach().cpu()
        else:
            raise ValueError(f"Invalid offsets type {type(offsets)}")
        if device is not None:
            batched_tensor = batched_tensor.to(device)
        self.offsets = offsets
        self.batched_tensor = batched_tensor
        self.check()

    def check(self):
        assert self.offsets.dtype in (torch.int32, torch.int64) and not self.offsets.is_cuda, \
            f"Offsets must be a cpu IntTensor or cpu LongTensor, got {self.offsets}"
        assert not self.offsets.requires_grad, "Offsets must not require grad"
        assert isinstance(self.batched_tensor, Tensor)
        assert int(self.offsets[-1]) == self.batched_tensor.shape[0], \
            f"Offsets {self.offsets.tolist()} do not match {self.batched_tensor.shape[0]} rows"

    @property
    def batch_size(self) -> int:
        return len(self.offsets) - 1

    @property
    def device(self):
        return self.batched_tensor.device

    @property
    def dtype(self):
        return self.batched_tensor.dtype

    @property
    def shape(self):
        return self.batched_tensor.shape

    def __len__(self) -> int:
        return self.batched_tensor.shape[0]

    def __getitem__(self, idx: int) -> Tensor:
        return self.batched_tensor[int(self.offsets[idx]):int(self.offsets[idx + 1])]

    def to(self, device=None, dtype: Optional[torch.dtype] = None):
        if device is None:
            device = self.device
        return self.__class__(self.batched_tensor.to(device=device, dtype=dtype), self.offsets)

    def equal_shape(self, value: "BatchedTensor") -> bool:
        return bool((self.offsets == value.offsets).all()) and \
            self.batched_tensor.shape[1:] == value.batched_tensor.shape[1:]

    def __repr__(self) -> str:
        return f"{self.__class__.__name__}(offsets={self.offsets.tolist()}, shape={tuple(self.shape)})"
