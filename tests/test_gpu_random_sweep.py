"""Seeded random sweep over what the fixed cases pin one at a time: batch sizes, voxel counts from one
to twelve thousand per item (tiny, just below / at / above a 64-row group), sparse to nearly full
boxes, coordinates far from the origin and negative, kernel sizes 1 to 5 per axis, strides 1 to 3 per
axis, channel counts on and off the kernels' tile widths, the three element types.  Every case:
strided coordinates and kernel map bit for bit against the C oracle, features (with a bias, a
residual and a ReLU in the epilogue now and then) against its double-precision gather-GEMM-scatter
within the tolerances of test_gpu_conv.py; a second sweep does the same for the two gradients, a
third for the pooling reductions and the depthwise convolution over the maps, a fourth for maps
over one to five spatial dimensions with dilated kernels against a dictionary look-up, a fifth for
points -> voxels against the restatement of the reference's voxelisation."""
import numpy as np
import pytest
import torch

from helpers import kaiming_weight, normal_features, rel_err, sort_rows
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}
COUNTS = (1, 7, 63, 64, 65, 500, 3000, 12000)
EXTENTS = (4, 12, 30, 80)
SHIFTS = (0, -17, 1000, -(1 << 20))
CHANNELS = (1, 3, 8, 13, 16, 24, 32, 40, 64, 96, 128, 160)
DTYPES = (torch.float16, torch.bfloat16, torch.float32)


def _case(seed):
    rng = np.random.default_rng(1000 + seed)
    batch = int(rng.integers(1, 5))
    extent = int(rng.choice(EXTENTS))
    items = []
    for _ in range(batch):
        n = min(int(rng.choice(COUNTS)), extent ** 3)
        cells = rng.choice(extent ** 3, size=n, replace=False)
        c = np.stack([cells // (extent * extent), cells // extent % extent, cells % extent], axis=1)
        items.append((c + rng.choice(SHIFTS, size=3)).astype(np.int32))
    ksize = tuple(int(k) for k in rng.integers(1, 6, size=3))
    stride = (1, 1, 1) if rng.random() < 0.5 else tuple(int(s) for s in rng.integers(1, 4, size=3))
    c_in, c_out = int(rng.choice(CHANNELS)), int(rng.choice(CHANNELS))
    dtype = DTYPES[int(rng.integers(0, 3))]
    epilogue = (rng.random() < 0.5, rng.random() < 0.3, rng.random() < 0.3)  # bias, residual, ReLU
    return synthetic.batch_indexed(items), batch, ksize, stride, c_in, c_out, dtype, epilogue


@pytest.mark.parametrize("seed", range(160))
def test_random_case_against_the_oracle(oracle, seed):
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    in_coords, batch, ksize, stride, c_in, c_out, dtype, (with_bias, with_residual, relu) = _case(seed)
    print(f"seed {seed}: {len(in_coords)} voxels in {batch} items, kernel {ksize}, stride {stride}, "
          f"{c_in} -> {c_out} {dtype}, bias {with_bias}, residual {with_residual}, relu {relu}", flush=True)
    dev_in = torch.as_tensor(in_coords, device=DEV)
    if any(s != 1 for s in stride):
        out_dev, off_dev = stride_coords(dev_in, stride)
        out_coords = out_dev.cpu().numpy()
        ref_out, _, ref_off = oracle.stride_coords(in_coords, stride, batch)
        assert np.array_equal(out_coords, ref_out)
        assert np.array_equal(off_dev.numpy().astype(np.int64), ref_off)
    else:
        out_coords = in_coords
    km = generate_kernel_map(dev_in, torch.as_tensor(out_coords, device=DEV), stride, ksize)
    im, om, off, iden = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    assert km.identity_map_index == iden
    assert np.array_equal(km.offsets.numpy().astype(np.int64), off)
    assert np.array_equal(km.in_maps.cpu().numpy(), im)
    assert np.array_equal(km.out_maps.cpu().numpy(), om)
    K = ksize[0] * ksize[1] * ksize[2]
    x = normal_features(len(in_coords), c_in, seed=seed, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=seed + 1, dtype=dtype)
    bias = normal_features(1, c_out, seed=seed + 2, dtype=dtype)[0] if with_bias else None
    residual = normal_features(len(out_coords), c_out, seed=seed + 3, dtype=dtype) if with_residual else None
    got = sparse_conv_forward(x.to(DEV), w.to(DEV), km, len(out_coords),
                              bias=None if bias is None else bias.to(DEV),
                              residual=None if residual is None else residual.to(DEV), relu=relu)
    want = oracle.explicit_conv_f64(x.double().numpy(), w.double().numpy(), im, om, off, iden, len(out_coords))
    if bias is not None:
        want = want + bias.double().numpy()
    if residual is not None:
        want = want + residual.double().numpy()
    if relu:
        want = np.maximum(want, 0.0)
    assert got.shape == want.shape and got.dtype == dtype
    if np.abs(want).max() > 0:
        assert rel_err(got.float().cpu().numpy(), want) <= TOL[dtype]
    else:
        assert not bool(got.any())


@pytest.mark.parametrize("seed", range(60))
def test_random_case_gradients_against_the_oracle(oracle, seed):
    """Both gradients of the contraction over the same random cases (strided maps included, whose
    exchanged lists have to be re-ordered for the input gradient), against the torch-CPU restatement
    of the reference's explicit backward in float64."""
    from oracle.explicit_conv import explicit_gemm_backward
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward
    in_coords, batch, ksize, stride, c_in, c_out, dtype, _ = _case(500 + seed)
    print(f"seed {seed}: {len(in_coords)} voxels in {batch} items, kernel {ksize}, stride {stride}, "
          f"{c_in} -> {c_out} {dtype}", flush=True)
    dev_in = torch.as_tensor(in_coords, device=DEV)
    if any(s != 1 for s in stride):
        out_coords = stride_coords(dev_in, stride)[0].cpu().numpy()
    else:
        out_coords = in_coords
    km = generate_kernel_map(dev_in, torch.as_tensor(out_coords, device=DEV), stride, ksize)
    im, om, off, iden = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
    K = ksize[0] * ksize[1] * ksize[2]
    x = normal_features(len(in_coords), c_in, seed=seed, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=seed + 1, dtype=dtype)
    gy = normal_features(len(out_coords), c_out, seed=seed + 2, dtype=dtype)
    gx, gw = sparse_conv_backward(gy.to(DEV), x.to(DEV), w.to(DEV), km)
    want_x, want_w = explicit_gemm_backward(gy.double(), x.double(), w.double(), torch.as_tensor(im),
                                            torch.as_tensor(om), off, iden)
    assert gx.dtype == dtype and gw.dtype == dtype
    for got, want in ((gx, want_x), (gw, want_w)):
        if float(want.abs().max()) > 0:
            assert rel_err(got.float().cpu().numpy(), want.numpy()) <= TOL[dtype]
        else:
            assert not bool(got.any())


@pytest.mark.parametrize("seed", range(40))
def test_random_case_pooling_and_depthwise_against_the_oracle(oracle, seed):
    """The consumers of a kernel map over the same random cases: the four pooling reductions against
    the torch restatement of the reference's sparse_reduce (selections exact, sums within the
    tolerance), the depthwise convolution and its two gradients against the float64 restatement of
    the reference's explicit depthwise path."""
    from oracle.explicit_conv import explicit_depthwise_forward
    from oracle.pool import pool_over_map
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_reduce
    in_coords, batch, ksize, stride, channels, _, dtype, _ = _case(900 + seed)
    print(f"seed {seed}: {len(in_coords)} voxels in {batch} items, kernel {ksize}, stride {stride}, "
          f"{channels} channels {dtype}", flush=True)
    n = len(in_coords)
    x = normal_features(n, channels, seed=seed, dtype=dtype)
    # pooling through the public functional (it strides the coordinates and builds the map itself)
    counts = np.bincount(in_coords[:, 0], minlength=batch)
    offsets = torch.as_tensor(np.concatenate([[0], np.cumsum(counts)]))
    voxels = Voxels(torch.as_tensor(in_coords[:, 1:].copy(), device=DEV), x.to(DEV), offsets=offsets)
    for reduction in ("max", "min", "mean", "sum"):
        out = sparse_reduce(voxels, ksize, stride, reduction)
        out_bc = out.batch_indexed_coordinates.cpu().numpy()
        im, om, off, _ = oracle.kernel_map(in_coords, out_bc, ksize, stride)
        want = pool_over_map(x.double(), torch.as_tensor(im), torch.as_tensor(om), len(out_bc), reduction)
        got = out.feature_tensor.double().cpu()
        if reduction in ("max", "min"):
            assert torch.equal(got, want)
        else:
            assert rel_err(got.numpy(), want.numpy()) <= TOL[dtype]
    # depthwise convolution over the map of the same geometry
    dev_in = torch.as_tensor(in_coords, device=DEV)
    out_coords = stride_coords(dev_in, stride)[0].cpu().numpy() if any(s != 1 for s in stride) else in_coords
    km = generate_kernel_map(dev_in, torch.as_tensor(out_coords, device=DEV), stride, ksize)
    im, om, off, iden = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    K = ksize[0] * ksize[1] * ksize[2]
    w = (torch.randn(K, channels, generator=torch.Generator().manual_seed(seed)) * (1.0 / K) ** 0.5).to(dtype)
    xd, wd = x.to(DEV).requires_grad_(True), w.to(DEV).requires_grad_(True)
    got = spatially_sparse_depthwise_conv(xd, wd, km, len(out_coords))
    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    want = explicit_depthwise_forward(x64, w64, torch.as_tensor(im), torch.as_tensor(om), off, iden,
                                      len(out_coords))
    assert got.dtype == dtype
    if float(want.detach().abs().max()) > 0:
        assert rel_err(got.detach().double().cpu().numpy(), want.detach().numpy()) <= TOL[dtype]
        gy = normal_features(len(out_coords), channels, seed=seed + 5, dtype=dtype)
        got.backward(gy.to(DEV))
        want_gx, want_gw = torch.autograd.grad(want, (x64, w64), gy.double())
        for g, wg in ((xd.grad, want_gx), (wd.grad, want_gw)):
            if float(wg.abs().max()) > 0:
                assert rel_err(g.double().cpu().numpy(), wg.numpy()) <= TOL[dtype]


def _brute_force_map(in_rows, out_rows, stride, ksize, dilation):
    """Kernel map over any number of columns by dictionary look-up: offsets enumerated with the last
    dimension fastest and centred as the reference centres them (odd sizes about the middle, even
    sizes from zero), pairs of an offset in ascending output row."""
    import itertools
    D = len(ksize)
    where = {tuple(r): i for i, r in enumerate(in_rows.tolist())}
    centres = [(k - 1) // 2 if k % 2 == 1 else 0 for k in ksize]
    ins, outs, offsets = [], [], [0]
    for idx in itertools.product(*[range(k) for k in ksize]):
        off = [(i - c) * d for i, c, d in zip(idx, centres, dilation)]
        for m, r in enumerate(out_rows.tolist()):
            hit = where.get((r[0],) + tuple(r[1 + d] * stride[d] + off[d] for d in range(D)))
            if hit is not None:
                ins.append(hit)
                outs.append(m)
        offsets.append(len(ins))
    return np.array(ins, np.int32), np.array(outs, np.int32), np.array(offsets, np.int64)


@pytest.mark.parametrize("seed", range(40))
def test_random_case_dimensions_and_dilation_against_brute_force(seed):
    """One to five spatial dimensions, dilated kernels, strides: the map against a dictionary
    look-up over all columns (the C oracle restates the three-dimensional probe only)."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    rng = np.random.default_rng(7000 + seed)
    D = int(rng.integers(1, 6))
    extent = int(rng.choice((3, 6, 10, 16)))
    n = int(rng.choice((1, 5, 64, 65, 400, 1500)))
    rows = rng.integers(-extent // 2, extent // 2 + 1, size=(n, D + 1)).astype(np.int32)
    rows[:, 0] = rng.integers(0, 3, size=n)
    rows = np.unique(rows, axis=0)
    rng.shuffle(rows)
    top = 5 if D <= 3 else 3
    ksize = tuple(int(k) for k in rng.integers(1, top + 1, size=D))
    dilated = rng.random() < 0.5
    dilation = tuple(int(d) for d in rng.integers(1, 4, size=D)) if dilated else (1,) * D
    stride = tuple(int(s) for s in rng.integers(1, 3, size=D)) if rng.random() < 0.4 else (1,) * D
    print(f"seed {seed}: {len(rows)} rows, {D} dimensions, kernel {ksize}, stride {stride}, dilation {dilation}",
          flush=True)
    if any(s != 1 for s in stride):
        coarse = rows.copy()
        coarse[:, 1:] = np.floor_divide(rows[:, 1:], np.array(stride, dtype=np.int32))
        out_rows = np.unique(coarse, axis=0)
    else:
        out_rows = rows
    dev = lambda a: torch.as_tensor(np.ascontiguousarray(a), device=DEV)
    km = generate_kernel_map(dev(rows), dev(out_rows), stride, ksize,
                             kernel_dilation=dilation if dilated else None,
                             method="offset" if dilated else "size")
    want_in, want_out, want_off = _brute_force_map(rows, out_rows, stride, ksize, dilation)
    assert np.array_equal(km.offsets.numpy().astype(np.int64), want_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), want_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), want_out)


@pytest.mark.parametrize("seed", range(30))
def test_random_case_points_to_voxels_against_the_oracle(seed):
    """Points -> voxels over random batches (ragged and empty items, clouds far from the origin and
    below zero, voxel sizes from millimetres to metres, 1 to 70 feature channels, every reduction the
    front-end builds): coordinates and offsets bit for bit, selections exact, sums within 1e-5."""
    from oracle import voxelize
    from warpconvnet_amd.geometry.types.points import Points
    rng = np.random.default_rng(9000 + seed)
    batch = int(rng.integers(1, 6))
    counts = [int(rng.choice((0, 1, 2, 63, 65, 1000, 20000))) for _ in range(batch)]
    if sum(counts) == 0:
        counts[0] = 5
    span = float(rng.choice((0.05, 1.0, 30.0)))
    centre = rng.choice((0.0, -50.0, 1000.0), size=3)
    pts = ((rng.random((sum(counts), 3)) - 0.5) * span + centre).astype(np.float32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    voxel_size = float(rng.choice((0.002, 0.02, 0.1, 0.75)))
    channels = int(rng.choice((1, 3, 7, 16, 33, 70)))
    reduction = str(rng.choice(("mean", "max", "sum", "min")))
    print(f"seed {seed}: items {counts}, span {span}, centre {centre.tolist()}, voxel {voxel_size}, "
          f"{channels} channels, {reduction}", flush=True)
    feats = normal_features(len(pts), channels, seed=seed)
    pc = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets))
    st = pc.to_voxels(voxel_size, reduction=reduction)
    coords, vfeats, voffsets = voxelize.points_to_voxels(pts, feats.double().numpy(), offsets, voxel_size,
                                                         reduction)
    assert np.array_equal(st.coordinate_tensor.cpu().numpy(), coords)
    assert np.array_equal(st.offsets.numpy(), voffsets)
    got = st.feature_tensor.double().cpu().numpy()
    if reduction in ("max", "min"):
        assert np.array_equal(got, vfeats)
    else:
        assert rel_err(got, vfeats) <= 1e-5
