"""Torch-CPU restatement of the reference's explicit gather-GEMM-scatter forward and backward.

TEST INFRASTRUCTURE ONLY (parity checker and the benchmark's cpu_baseline leg).

Follows warpconvnet/nn/functional/sparse_conv.py:281-311 operation by operation, so that the
rounding of a low-precision run (the running output is rounded to the compute dtype after every
kernel offset) is reproduced by torch itself:

    X, W cast to compute_dtype (if given)
    out = X @ W[iden]                      if the map carries an identity index
          zeros(M, C_out, dtype of X)      otherwise
    for k in range(K), skipping iden and empty offsets, in k order:
        out[out_map_k] += X[in_map_k] @ W[k]
    return out cast back to the dtype X came in with

The bias add and the output container are applied by the caller (sparse_conv.py:1794-1805).

`explicit_gemm_backward` follows sparse_conv.py:314-355 the same way.  It is pinned by torch's
automatic differentiation of `explicit_gemm_forward` (tests/test_oracle_pins.py), which in turn
is pinned by the dense-cube conv3d identity and the pairwise brute force.
"""
from typing import Optional

import torch


def explicit_gemm_forward(in_features: torch.Tensor, weight: torch.Tensor, in_maps: torch.Tensor,
                          out_maps: torch.Tensor, offsets, identity_map_index: Optional[int],
                          num_out_coords: int,
                          compute_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    x = in_features if compute_dtype is None else in_features.to(compute_dtype)
    w = weight if compute_dtype is None else weight.to(compute_dtype)
    offs = [int(o) for o in offsets]
    num_offsets = len(offs) - 1
    if identity_map_index is not None:
        out = torch.matmul(x, w[identity_map_index])
    else:
        out = torch.zeros(num_out_coords, w.shape[-1], dtype=x.dtype, device=x.device)
    for k in range(num_offsets):
        if k == identity_map_index:
            continue
        lo, hi = offs[k], offs[k + 1]
        if hi == lo:
            continue
        rows_in = in_maps[lo:hi].long()
        rows_out = out_maps[lo:hi].long()
        out[rows_out] += torch.matmul(x[rows_in], w[k])
    return out.to(dtype=in_features.dtype)


def explicit_gemm_backward(grad_output: torch.Tensor, in_features: torch.Tensor,
                           weight: torch.Tensor, in_maps: torch.Tensor, out_maps: torch.Tensor,
                           offsets, identity_map_index: Optional[int],
                           compute_dtype: Optional[torch.dtype] = None):
    """(grad_in_features, grad_weight):
        dX = dY @ W[iden]^T, dW[iden] = X^T @ dY     if the map carries an identity index
        for k != iden, non-empty, in k order:
            dX[in_map_k] += dY[out_map_k] @ W[k]^T ;  dW[k] += X[in_map_k]^T @ dY[out_map_k]
    computed in compute_dtype (else the dtype of X), returned in the dtypes of X and W."""
    dtype = compute_dtype if compute_dtype is not None else in_features.dtype
    x = in_features.to(dtype)
    w = weight.to(dtype)
    gy = grad_output.to(dtype)
    offs = [int(o) for o in offsets]
    grad_w = torch.zeros_like(w)
    if identity_map_index is not None:
        grad_x = torch.matmul(gy, w[identity_map_index].T)
        grad_w[identity_map_index] = torch.matmul(x.T, gy)
    else:
        grad_x = torch.zeros_like(x)
    for k in range(len(offs) - 1):
        if k == identity_map_index:
            continue
        lo, hi = offs[k], offs[k + 1]
        if hi == lo:
            continue
        rows_in = in_maps[lo:hi].long()
        rows_out = out_maps[lo:hi].long()
        g = gy[rows_out]
        grad_x[rows_in] += torch.matmul(g, w[k].T)
        grad_w[k] += torch.matmul(x[rows_in].T, g)
    return grad_x.to(in_features.dtype), grad_w.to(weight.dtype)


def explicit_depthwise_forward(in_features: torch.Tensor, weight: torch.Tensor, in_maps: torch.Tensor,
                               out_maps: torch.Tensor, offsets, identity_map_index: Optional[int],
                               num_out_coords: int,
                               compute_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Depthwise convolution, weight (K, C), following
    warpconvnet/nn/functional/sparse_conv_depth.py:151-182 operation by operation:
        out = X * W[iden]                       if the map carries an identity index, else zeros
        for k != iden, non-empty, in k order:   out[out_map_k] += X[in_map_k] * W[k]
    Written with differentiable torch operations: the gradients the parity tests compare against
    are autograd's.  Pinned in tests/test_oracle_pins.py by conv3d with groups = C on a dense cube."""
    x = in_features if compute_dtype is None else in_features.to(compute_dtype)
    w = weight if compute_dtype is None else weight.to(compute_dtype)
    offs = [int(o) for o in offsets]
    if identity_map_index is not None:
        out = x * w[identity_map_index].unsqueeze(0)
    else:
        out = torch.zeros(num_out_coords, w.shape[-1], dtype=x.dtype, device=x.device)
    for k in range(len(offs) - 1):
        if k == identity_map_index:
            continue
        lo, hi = offs[k], offs[k + 1]
        if hi == lo:
            continue
        out = out.index_add(0, out_maps[lo:hi].long(), x[in_maps[lo:hi].long()] * w[k].unsqueeze(0))
    return out.to(dtype=in_features.dtype)
