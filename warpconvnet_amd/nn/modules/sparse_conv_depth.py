"""Depthwise sparse convolution modules (reference: warpconvnet/nn/modules/sparse_conv_depth.py)."""
import math
from typing import Optional, Tuple, Union

import numpy as np
import torch
import torch.nn as nn
from torch.nn.init import calculate_gain

from ...geometry.coords.integer import IntCoords
from ...geometry.types.voxels import Voxels
from ...utils.ntuple import ntuple
from ..functional.sparse_conv import (POINT_ORDERING, STRIDED_CONV_MODE,
                                      generate_output_coords_and_kernel_map, in_coords_of)
from ..functional.sparse_conv_depth import spatially_sparse_depthwise_conv


class SpatiallySparseDepthwiseConv(nn.Module):
    """One (K,) kernel per channel; weight (K, C), optional bias (C,)
    (reference: sparse_conv_depth.py:34-255)."""

    def __init__(self, channels: int, kernel_size: Union[int, Tuple[int, ...]],
                 stride: Union[int, Tuple[int, ...]] = 1, dilation: Union[int, Tuple[int, ...]] = 1,
                 bias: bool = True, transposed: bool = False, generative: bool = False,
                 num_spatial_dims: int = 3, fwd_algo=None, bwd_algo=None,
                 stride_mode: STRIDED_CONV_MODE = STRIDED_CONV_MODE.STRIDE_ONLY,
                 order=POINT_ORDERING.RANDOM, compute_dtype: Optional[torch.dtype] = None):
        super().__init__()
        self.num_spatial_dims = num_spatial_dims
        self.channels = self.in_channels = self.out_channels = channels
        self.kernel_size = ntuple(kernel_size, ndim=num_spatial_dims)
        self.stride = ntuple(stride, ndim=num_spatial_dims)
        self.dilation = ntuple(dilation, ndim=num_spatial_dims)
        self.transposed = transposed
        self.generative = generative
        self.fwd_algo, self.bwd_algo = fwd_algo, bwd_algo
        self.stride_mode = stride_mode
        self.order = order
        self.compute_dtype = compute_dtype
        self.weight = nn.Parameter(torch.randn(int(np.prod(self.kernel_size)), channels))
        self.bias = nn.Parameter(torch.randn(channels)) if bias else None
        self.reset_parameters()

    def __repr__(self):
        out = f"{self.__class__.__name__}(channels={self.channels}, kernel_size={self.kernel_size}"
        if self.stride != (1,) * self.num_spatial_dims:
            out += f", stride={self.stride}"
        if self.transposed:
            out += f", transposed={self.transposed}"
        if self.bias is None:
            out += ", bias=False"
        return out + ")"

    @torch.no_grad()
    def reset_parameters(self):
        """Uniform in +-sqrt(D) * gain / sqrt(K) (sparse_conv_depth.py:144-181: fan = kernel volume)."""
        fan = int(np.prod(self.kernel_size))
        std = calculate_gain("leaky_relu", math.sqrt(5)) / math.sqrt(fan)
        bound = math.sqrt(self.num_spatial_dims) * std
        self.weight.uniform_(-bound, bound)
        if self.bias is not None:
            b = 1 / math.sqrt(fan) if fan > 0 else 0
            self.bias.uniform_(-b, b)

    def forward(self, input_sparse_tensor: Voxels,
                output_spatially_sparse_tensor: Optional[Voxels] = None) -> Voxels:
        out_coords, out_offsets, kernel_map = generate_output_coords_and_kernel_map(
            input_sparse_tensor=input_sparse_tensor, kernel_size=self.kernel_size,
            kernel_dilation=self.dilation, stride=self.stride, generative=self.generative,
            transposed=self.transposed, output_spatially_sparse_tensor=output_spatially_sparse_tensor,
            stride_mode=self.stride_mode, order=self.order)
        features = spatially_sparse_depthwise_conv(
            input_sparse_tensor.feature_tensor, self.weight, kernel_map, out_coords.shape[0],
            fwd_algo=self.fwd_algo, bwd_algo=self.bwd_algo, compute_dtype=self.compute_dtype)
        if self.bias is not None:
            features = features + self.bias.to(features.dtype)
        in_stride = input_sparse_tensor.tensor_stride or (1,) * self.num_spatial_dims
        if not self.transposed:
            out_stride = tuple(o * s for o, s in zip(self.stride, in_stride))
        elif output_spatially_sparse_tensor is not None and \
                output_spatially_sparse_tensor.tensor_stride is not None:
            out_stride = output_spatially_sparse_tensor.tensor_stride
        else:
            out_stride = (1,) * self.num_spatial_dims
        if out_coords is in_coords_of(input_sparse_tensor):
            coords = input_sparse_tensor.batched_coordinates
        elif output_spatially_sparse_tensor is not None:
            coords = output_spatially_sparse_tensor.batched_coordinates
        else:
            coords = IntCoords(out_coords[:, 1:], offsets=out_offsets.cpu().int())
            coords._batch_indexed = out_coords
        return input_sparse_tensor.replace(batched_coordinates=coords, batched_features=features,
                                           tensor_stride=out_stride)


class SparseDepthwiseConv2d(SpatiallySparseDepthwiseConv):
    def __init__(self, channels, kernel_size, stride=1, dilation=1, bias=True, transposed=False,
                 generative=False, **kw):
        super().__init__(channels, kernel_size, stride=stride, dilation=dilation, bias=bias,
                         transposed=transposed, generative=generative, num_spatial_dims=2, **kw)


class SparseDepthwiseConv3d(SpatiallySparseDepthwiseConv):
    def __init__(self, channels, kernel_size, stride=1, dilation=1, bias=True, transposed=False,
                 generative=False, **kw):
        super().__init__(channels, kernel_size, stride=stride, dilation=dilation, bias=bias,
                         transposed=transposed, generative=generative, num_spatial_dims=3, **kw)
