"""Shared helpers of the parity tests."""
import numpy as np
import torch


def canonical_pairs(in_maps, out_maps, offsets):
    """(k, out, in) triples sorted lexicographically: the canonical form of a kernel map."""
    in_maps = np.asarray(in_maps, dtype=np.int64)
    out_maps = np.asarray(out_maps, dtype=np.int64)
    offsets = np.asarray(offsets, dtype=np.int64)
    k = np.repeat(np.arange(len(offsets) - 1), np.diff(offsets))
    order = np.lexsort((in_maps, out_maps, k))
    return np.stack([k[order], out_maps[order], in_maps[order]], axis=1)


def sort_rows(a):
    a = np.asarray(a)
    return a[np.lexsort(a.T[::-1])]


def rel_err(a, b):
    """max|a-b| / max|b| per tensor (the relative error the feature tolerance is stated in)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def elementwise_rel_err(a, b):
    """max of |a-b| / (|b| + 1e-6) over entries with |b| > 1e-3 max|b| (the form the reference's
    native GEMM tests print, tests/csrc/test_cutlass_gemm.py:24-26)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    mask = np.abs(b) > 1e-3 * np.abs(b).max()
    return float((np.abs(a - b)[mask] / (np.abs(b)[mask] + 1e-6)).max())


def kaiming_weight(K, c_in, c_out, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    std = (2.0 / (c_in * K)) ** 0.5
    return (torch.randn(K, c_in, c_out, generator=g) * std).to(dtype)


def normal_features(n, c, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed + 1)
    return torch.randn(n, c, generator=g).to(dtype)
