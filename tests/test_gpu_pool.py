"""GPU parity of the pooling over a kernel map (wcn_map_rows_build / wcn_sparse_pool_fwd / _bwd)
against the torch restatement of the reference's sparse_reduce (oracle/pool.py) and its
gradients as torch differentiates them.  Tolerances: 1e-5 (fp32), 1e-2 (fp16 / bf16) relative;
max / min are selections and must be exact."""
import numpy as np
import pytest
import torch

from helpers import normal_features, rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _voxels(items, feats):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    offsets = np.zeros(len(items) + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    coords = torch.as_tensor(np.concatenate(items, axis=0), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats, offsets=torch.as_tensor(offsets))


@pytest.mark.parametrize("reduction", ["max", "min", "mean", "sum"])
@pytest.mark.parametrize("dtype,channels,ksize,stride", [
    (torch.float32, 32, 2, 2), (torch.float16, 64, 3, 2), (torch.bfloat16, 24, 2, 2),
    (torch.float32, 7, 3, 2)])
def test_pool_forward_and_gradient(oracle, reduction, dtype, channels, ksize, stride):
    from oracle.pool import pool_over_map
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_reduce
    items = [synthetic.indoor_scene(seed=70 + b, n_target=5000, voxel_size=0.05) for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), channels, seed=2, dtype=dtype)
    xd = x.to(DEV).requires_grad_(True)
    out = sparse_reduce(_voxels(items, xd), ksize, stride, reduction)
    out_bc = out.batch_indexed_coordinates.cpu().numpy()
    assert out.tensor_stride == (stride,) * 3 and out.feature_tensor.dtype == dtype
    im, om, off, _ = oracle.kernel_map(bc, out_bc, (ksize,) * 3, (stride,) * 3)
    x64 = x.double().requires_grad_(True)
    want = pool_over_map(x64, torch.as_tensor(im), torch.as_tensor(om), len(out_bc), reduction)
    got = out.feature_tensor.detach().double().cpu()
    if reduction in ("max", "min"):
        assert torch.equal(got, want.detach())
    else:
        assert rel_err(got.numpy(), want.detach().numpy()) <= TOL[dtype]
    gy = normal_features(len(out_bc), channels, seed=3, dtype=dtype)
    out.feature_tensor.backward(gy.to(DEV))
    if reduction in ("max", "min"):
        # The gradient goes to the one input row that supplied the extremum (torch_scatter's
        # segment_csr, which the reference uses, does the same; torch's own scatter_reduce splits
        # it among equal values, which 16-bit features do produce).  Among equals this library
        # takes the first pair in kernel-offset order: restated here row by row.
        xs = x.double().numpy() * (1.0 if reduction == "max" else -1.0)
        want_gx = np.zeros_like(xs)
        order = np.argsort(om, kind="stable")  # pairs of a row in kernel-offset order
        rows_in, rows_out = im[order], om[order]
        bounds = np.searchsorted(rows_out, np.arange(len(out_bc) + 1))
        g64 = gy.double().numpy()
        cols = np.arange(channels)
        for m in range(len(out_bc)):
            cand = rows_in[bounds[m]:bounds[m + 1]]
            if len(cand):
                winner = cand[np.argmax(xs[cand], axis=0)]
                want_gx[winner, cols] += g64[m]
    else:
        (want_gx,) = torch.autograd.grad(want, x64, gy.double())
        want_gx = want_gx.numpy()
    assert xd.grad.dtype == dtype
    assert rel_err(xd.grad.double().cpu().numpy(), want_gx) <= TOL[dtype]


def test_pool_dense_cube_equals_torch_pooling():
    """kernel = stride = 2 over a full cube: max_pool3d / avg_pool3d of the dense tensor."""
    from warpconvnet_amd.nn.modules.sparse_pool import SparseAvgPool, SparseMaxPool
    S, C = 12, 16
    g = torch.Generator().manual_seed(6)
    dense = torch.randn(1, C, S, S, S, generator=g)
    grid = torch.stack(torch.meshgrid(torch.arange(S), torch.arange(S), torch.arange(S), indexing="ij"), -1)
    xyz = grid.reshape(-1, 3)[torch.randperm(S**3, generator=g)]
    feats = dense[0, :, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T.contiguous()
    vox = _voxels([xyz.numpy().astype(np.int32)], feats.to(DEV))
    for module, fn in ((SparseMaxPool(2, 2), torch.nn.functional.max_pool3d),
                       (SparseAvgPool(2, 2), torch.nn.functional.avg_pool3d)):
        out = module(vox)
        c = out.coordinate_tensor.cpu().long()
        want = fn(dense, 2)[0][:, c[:, 0], c[:, 1], c[:, 2]].T
        assert rel_err(out.feature_tensor.cpu().numpy(), want.numpy()) <= 1e-6


def test_unpool_returns_features_to_their_windows():
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_max_pool, sparse_unpool
    items = [synthetic.random_cloud(80, 4000, 20)[:, 1:]]
    x = normal_features(len(items[0]), 8, seed=1)
    fine = _voxels(items, x.to(DEV))
    pooled = sparse_max_pool(fine, 2, 2)
    back = sparse_unpool(pooled, fine, 2, 2, concat_unpooled_voxels=True)
    assert back.feature_tensor.shape == (len(x), 16)
    assert torch.equal(back.feature_tensor[:, :8].cpu(), x)
    # every fine voxel received the maximum of its 2x2x2 window, which is at least its own value
    assert (back.feature_tensor[:, 8:].cpu() >= x).all()
    coarse_of = {tuple(c): i for i, c in enumerate(pooled.coordinate_tensor.cpu().numpy().tolist())}
    idx = [coarse_of[tuple(c)] for c in (fine.coordinate_tensor.cpu().numpy() // 2).tolist()]
    assert torch.equal(back.feature_tensor[:, 8:].cpu(), pooled.feature_tensor.cpu()[idx])


def test_pool_at_benchmark_size():
    """4 x 250k voxels, 64 channels fp16, 2x2x2 stride 2: mean pooling of ones is one, the sum
    counts the window's voxels (all fine voxels are counted exactly once), max is bounded by both."""
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_reduce
    items, _ = synthetic.indoor_batch(4, 250_000)
    n = sum(len(i) for i in items)
    ones = torch.ones(n, 64, dtype=torch.float16, device=DEV)
    vox = _voxels(items, ones)
    assert torch.equal(sparse_reduce(vox, 2, 2, "mean").feature_tensor,
                       torch.ones_like(sparse_reduce(vox, 2, 2, "max").feature_tensor))
    counts = sparse_reduce(vox, 2, 2, "sum").feature_tensor
    assert int(counts[:, 0].float().sum()) == n and float(counts.max()) <= 8 and float(counts.min()) >= 1


def test_reduce_and_stride_convolution(oracle):
    """stride_mode=REDUCE_AND_STRIDE: max pooling over stride-sized windows, then the convolution
    with stride 1 over the pooled voxels (reference: sparse_conv.py:1753-1766)."""
    from helpers import kaiming_weight
    from warpconvnet_amd.nn.functional.sparse_conv import STRIDED_CONV_MODE, spatially_sparse_conv
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_max_pool
    items = [synthetic.random_cloud(140 + b, 3000, 24)[:, 1:] for b in range(2)]
    x = normal_features(sum(len(i) for i in items), 16, seed=5)
    w = kaiming_weight(27, 16, 24, seed=6).to(DEV)
    fine = _voxels(items, x.to(DEV))
    got = spatially_sparse_conv(fine, w, 3, stride=2, stride_mode=STRIDED_CONV_MODE.REDUCE_AND_STRIDE)
    pooled = sparse_max_pool(_voxels(items, x.to(DEV)), 2, 2)
    want = spatially_sparse_conv(pooled, w, 3)
    assert got.tensor_stride == (2, 2, 2)
    assert torch.equal(got.coordinate_tensor, want.coordinate_tensor)
    assert torch.equal(got.feature_tensor, want.feature_tensor)
    # and against the oracle chain
    from oracle.pool import pool_over_map
    bc = synthetic.batch_indexed(items)
    pc = pooled.batch_indexed_coordinates.cpu().numpy()
    im, om, off, _ = oracle.kernel_map(bc, pc, (2, 2, 2), (2, 2, 2))
    px = pool_over_map(x.double(), torch.as_tensor(im), torch.as_tensor(om), len(pc), "max")
    im, om, off, iden = oracle.kernel_map(pc, pc, (3, 3, 3))
    ref = oracle.explicit_conv_f64(px.numpy(), w.double().cpu().numpy(), im, om, off, iden, len(pc))
    assert rel_err(got.feature_tensor.cpu().numpy(), ref) <= 1e-5
