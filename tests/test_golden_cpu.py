"""The oracle against the committed golden fixtures (and the fixtures against a brute-force
restatement, so a regenerated fixture cannot silently drift)."""
import glob
import os

import numpy as np
import pytest

from test_oracle_pins import brute_force_kernel_map

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def test_fixtures_present():
    assert len(GOLDEN) >= 4


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p) for p in GOLDEN])
def test_oracle_reproduces_fixture(oracle, path):
    g = np.load(path)
    ksize, stride = tuple(g["kernel_size"]), tuple(g["stride"])
    im, om, off, iden = oracle.kernel_map(g["in_coords"], g["out_coords"], ksize, stride)
    assert np.array_equal(im, g["in_maps"]) and np.array_equal(om, g["out_maps"])
    assert np.array_equal(off, g["offsets"])
    assert (-1 if iden is None else iden) == int(g["identity"])
    out = oracle.explicit_conv_f64(g["features"], g["weight"], im, om, off, iden, len(g["out_coords"]))
    assert np.abs(out - g["out_features_f64"]).max() < 1e-12
    bf = brute_force_kernel_map(g["in_coords"], g["out_coords"], ksize, stride)
    assert np.array_equal(bf[0], g["in_maps"]) and np.array_equal(bf[1], g["out_maps"])
    assert np.array_equal(bf[2], g["offsets"])
    # the stored gradients: reproduced by the backward restatement, and equal to a pair-by-pair
    # brute force (dX[in] += dY[out] W[k]^T, dW[k] += X[in]^T dY[out] over every pair of the map)
    import torch
    from oracle.explicit_conv import explicit_gemm_backward
    x, w, gy = (g["features"].astype(np.float64), g["weight"].astype(np.float64),
                g["grad_out"].astype(np.float64))
    gx, gw = explicit_gemm_backward(torch.from_numpy(gy), torch.from_numpy(x), torch.from_numpy(w),
                                    torch.from_numpy(im), torch.from_numpy(om), off, iden)
    assert np.abs(gx.numpy() - g["grad_features_f64"]).max() < 1e-12
    assert np.abs(gw.numpy() - g["grad_weight_f64"]).max() < 1e-12
    want_x, want_w = np.zeros_like(x), np.zeros_like(w)
    for k in range(len(off) - 1):
        for p in range(off[k], off[k + 1]):
            want_x[im[p]] += gy[om[p]] @ w[k].T
            want_w[k] += np.outer(x[im[p]], gy[om[p]])
    assert np.abs(want_x - g["grad_features_f64"]).max() < 1e-10
    assert np.abs(want_w - g["grad_weight_f64"]).max() < 1e-10
