"""Writes the small golden fixtures of the parity tests from the CPU oracle.

    python tests/golden/make_golden.py

The reference keeps no stored vectors for this path (its tests are property checks), and its
Python cannot be imported here (it needs CuPy, the compiled CUDA extension and Warp), so the
fixtures are produced by this repository's own oracle after the pins in
tests/test_oracle_pins.py passed.  Each .npz holds inputs and expected outputs only.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import torch  # noqa: E402

from oracle import cpu_oracle  # noqa: E402
from oracle.explicit_conv import explicit_gemm_backward  # noqa: E402
from warpconvnet_amd.utils import synthetic  # noqa: E402


def case(name, coords, ksize, stride, c_in, c_out, seed):
    rng = np.random.default_rng(seed)
    batches = int(coords[:, 0].max()) + 1
    if any(s != 1 for s in stride):
        out_coords, first, out_offsets = cpu_oracle.stride_coords(coords, stride, batches)
    else:
        out_coords, first = coords, np.arange(len(coords), dtype=np.int32)
        out_offsets = np.concatenate([[0], np.cumsum(np.bincount(coords[:, 0], minlength=batches))])
    im, om, off, iden = cpu_oracle.kernel_map(coords, out_coords, ksize, stride)
    K = int(np.prod(ksize))
    x = rng.normal(size=(len(coords), c_in)).astype(np.float32)
    w = (rng.normal(size=(K, c_in, c_out)) * np.sqrt(2.0 / (c_in * K))).astype(np.float32)
    out = cpu_oracle.explicit_conv_f64(x, w, im, om, off, iden, len(out_coords))
    # gradients of sum(out * grad_out): the torch restatement of the reference's explicit backward
    # (sparse_conv.py:314-355) in float64
    gy = rng.normal(size=(len(out_coords), c_out)).astype(np.float32)
    gx, gw = explicit_gemm_backward(torch.from_numpy(gy).double(), torch.from_numpy(x).double(),
                                    torch.from_numpy(w).double(), torch.from_numpy(im),
                                    torch.from_numpy(om), off, iden)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), in_coords=coords, kernel_size=np.array(ksize),
                        stride=np.array(stride), out_coords=out_coords, out_first_index=first,
                        out_offsets=np.asarray(out_offsets, np.int64), in_maps=im, out_maps=om,
                        offsets=off, identity=np.array(-1 if iden is None else iden),
                        features=x, weight=w, out_features_f64=out, grad_out=gy,
                        grad_features_f64=gx.numpy(), grad_weight_f64=gw.numpy())


if __name__ == "__main__":
    case("k3s1_spheres", synthetic.batch_indexed([synthetic.spheres_scene(3, 400, 0.08)]),
         (3, 3, 3), (1, 1, 1), 8, 12, 0)
    case("k2s2_cloud", synthetic.random_cloud(4, 300, 10, batch_size=2), (2, 2, 2), (2, 2, 2), 6, 10, 1)
    case("k3s2_cloud", synthetic.random_cloud(5, 300, 10, batch_size=2), (3, 3, 3), (2, 2, 2), 5, 7, 2)
    case("k5s1_cloud", synthetic.random_cloud(6, 200, 8, batch_size=1), (5, 5, 5), (1, 1, 1), 4, 4, 3)
    print(sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
