"""Sparse convolution modules (reference: warpconvnet/nn/modules/sparse_conv.py:30-374)."""
import math
from typing import List, Optional, Tuple, Union

import numpy as np
import torch
import torch.nn as nn
from torch.nn.init import calculate_gain

from ...geometry.types.voxels import Voxels
from ...utils.ntuple import ntuple
from ..functional.sparse_conv import POINT_ORDERING, SPARSE_CONV_BWD_ALGO_MODE, \
    SPARSE_CONV_FWD_ALGO_MODE, STRIDED_CONV_MODE, spatially_sparse_conv


class SpatiallySparseConv(nn.Module):
    """Parameters: weight (prod(kernel_size), C_in, C_out), bias (C_out) or None, the layout of
    the reference's state dict.  Algorithm-selection arguments are stored and ignored."""

    def __init__(self, in_channels: int, out_channels: int,
                 kernel_size: Union[int, List[int], Tuple[int, ...]],
                 stride: Union[int, List[int], Tuple[int, ...]] = 1,
                 dilation: Union[int, List[int], Tuple[int, ...]] = 1, bias: bool = True,
                 transposed: bool = False, generative: bool = False,
                 kernel_matmul_batch_size: int = 2, num_spatial_dims: Optional[int] = 3,
                 fwd_algo=None, bwd_algo=None,
                 stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY,
                 order=POINT_ORDERING.RANDOM, compute_dtype: Optional[torch.dtype] = None,
                 implicit_matmul_fwd_block_size: Optional[int] = None,
                 implicit_matmul_bwd_block_size: Optional[int] = None):
        super().__init__()
        self.num_spatial_dims = num_spatial_dims
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = ntuple(kernel_size, ndim=num_spatial_dims)
        self.stride = ntuple(stride, ndim=num_spatial_dims)
        self.dilation = ntuple(dilation, ndim=num_spatial_dims)
        self.transposed = transposed
        self.generative = generative
        self.kernel_matmul_batch_size = kernel_matmul_batch_size
        self.stride_mode = stride_mode
        self.order = order
        self.compute_dtype = compute_dtype
        self.fwd_algo = fwd_algo if fwd_algo is not None else SPARSE_CONV_FWD_ALGO_MODE.AUTO
        self.bwd_algo = bwd_algo if bwd_algo is not None else SPARSE_CONV_BWD_ALGO_MODE.AUTO
        self.implicit_matmul_fwd_block_size = implicit_matmul_fwd_block_size
        self.implicit_matmul_bwd_block_size = implicit_matmul_bwd_block_size

        self.weight = nn.Parameter(torch.randn(int(np.prod(self.kernel_size)), in_channels,
                                               out_channels))
        if bias:
            self.bias = nn.Parameter(torch.randn(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def _fan_in_out(self) -> Tuple[int, int]:
        volume = int(np.prod(self.kernel_size))
        return self.in_channels * volume, self.out_channels * volume

    @torch.no_grad()
    def reset_parameters(self):
        """Kaiming-uniform with a = sqrt(5): bound = sqrt(D) * gain / sqrt(fan), fan = C_in * K
        (C_out * K when transposed); bias uniform in +-1/sqrt(fan_in) (reference :159-191)."""
        fan_in, fan_out = self._fan_in_out()
        fan = fan_out if self.transposed else fan_in
        gain = calculate_gain("leaky_relu", math.sqrt(5))
        bound = math.sqrt(self.num_spatial_dims) * gain / math.sqrt(fan)
        self.weight.uniform_(-bound, bound)
        if self.bias is not None and fan_in > 0:
            b = 1.0 / math.sqrt(fan_in)
            self.bias.uniform_(-b, b)

    def extra_repr(self) -> str:
        s = f"in_channels={self.in_channels}, out_channels={self.out_channels}, kernel_size={self.kernel_size}"
        if any(v != 1 for v in self.stride):
            s += f", stride={self.stride}"
        if any(v != 1 for v in self.dilation):
            s += f", dilation={self.dilation}"
        if self.transposed:
            s += ", transposed=True"
        if self.generative:
            s += ", generative=True"
        if self.bias is None:
            s += ", bias=False"
        return s

    # Set on an instance (or the class) whose weight stays the same between calls, or changes only in
    # ways its version counter sees: the kernels' tiles of the weight are then kept with the
    # parameter instead of being made by one more kernel in every call (see sparse_conv_forward).
    keep_prepared_weight = False

    def forward(self, input_sparse_tensor: Voxels,
                output_spatially_sparse_tensor: Optional[Voxels] = None, *,
                residual=None, relu: bool = False) -> Voxels:
        """`residual` and `relu` (keyword only, not in the reference): act(conv(x) + residual), done
        in the convolution's epilogue where no gradient is asked for."""
        return spatially_sparse_conv(
            input_sparse_tensor, weight=self.weight, kernel_size=self.kernel_size,
            stride=self.stride, kernel_dilation=self.dilation, bias=self.bias,
            kernel_matmul_batch_size=self.kernel_matmul_batch_size, generative=self.generative,
            output_spatially_sparse_tensor=output_spatially_sparse_tensor,
            transposed=self.transposed, fwd_algo=self.fwd_algo, bwd_algo=self.bwd_algo,
            stride_mode=self.stride_mode, order=self.order, compute_dtype=self.compute_dtype,
            implicit_matmul_fwd_block_size=self.implicit_matmul_fwd_block_size,
            implicit_matmul_bwd_block_size=self.implicit_matmul_bwd_block_size,
            residual=residual, relu=relu, keep_prepared_weight=self.keep_prepared_weight)


class SparseConv2d(SpatiallySparseConv):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, dilation=1, bias=True,
                 transposed=False, generative: bool = False,
                 stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY, fwd_algo=None,
                 bwd_algo=None, kernel_matmul_batch_size: int = 2, order=POINT_ORDERING.RANDOM,
                 compute_dtype: Optional[torch.dtype] = None):
        super().__init__(in_channels, out_channels, kernel_size, stride=stride, dilation=dilation,
                         bias=bias, transposed=transposed, generative=generative,
                         kernel_matmul_batch_size=kernel_matmul_batch_size, num_spatial_dims=2,
                         fwd_algo=fwd_algo, bwd_algo=bwd_algo, stride_mode=stride_mode,
                         order=order, compute_dtype=compute_dtype)


class SparseConv3d(SpatiallySparseConv):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, dilation=1, bias=True,
                 transposed=False, generative: bool = False,
                 stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY, fwd_algo=None,
                 bwd_algo=None, kernel_matmul_batch_size: int = 2, order=POINT_ORDERING.RANDOM,
                 compute_dtype: Optional[torch.dtype] = None):
        super().__init__(in_channels, out_channels, kernel_size, stride=stride, dilation=dilation,
                         bias=bias, transposed=transposed, generative=generative,
                         kernel_matmul_batch_size=kernel_matmul_batch_size, num_spatial_dims=3,
                         fwd_algo=fwd_algo, bwd_algo=bwd_algo, stride_mode=stride_mode,
                         order=order, compute_dtype=compute_dtype)
