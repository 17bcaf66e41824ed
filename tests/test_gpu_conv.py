"""GPU parity of the feature contraction and of the public convolution entry points.

Yardsticks: the C oracle's double-precision explicit gather-GEMM-scatter, and the torch-CPU
restatement of the reference's explicit path in the reference's own operation order (which
reproduces its per-offset rounding in low precision).
Tolerances (max|a-b| / max|b| per tensor): 1e-5 for fp32, 1e-2 for fp16 / bf16.
"""
import numpy as np
import pytest
import torch

from helpers import elementwise_rel_err, kaiming_weight, normal_features, rel_err
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}
# Entry by entry, |a - b| / (|b| + 1e-6) over the entries above a thousandth of the largest (the form
# the reference's native GEMM tests print, tests/csrc/test_cutlass_gemm.py:24-26).  16-bit results
# are correctly rounded sums, so the tensor-wide bound holds per entry as well.  An fp32 sum of a few
# hundred to a few thousand products carries an absolute error of some 1e-7 of the largest entry
# (measured: 1.4e-7 to 9.7e-7), which is up to 1e-3 of an entry a thousand times smaller.
ELEM_TOL = {torch.float32: 1e-3, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _dev_i32(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.int32, device=DEV)


def _voxels(items, feats, **kw):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    offsets = np.zeros(len(items) + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    coords = torch.as_tensor(np.concatenate(items, axis=0), dtype=torch.int32, device=DEV)
    return Voxels(coords, feats.to(DEV), offsets=torch.as_tensor(offsets), **kw)


def _oracle_out(oracle, x, w, in_coords, out_coords, ksize, stride, bias=None):
    im, om, off, iden = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    out = oracle.explicit_conv_f64(x.double().numpy(), w.double().numpy(), im, om, off, iden,
                                   len(out_coords))
    if bias is not None:
        out = out + bias.double().numpy()
    return out, (im, om, off, iden)


CONV_CASES = [
    # name, dtype, c_in, c_out, voxels per item, batch, kernel
    ("f32_32_32", torch.float32, 32, 32, 6000, 2, (3, 3, 3)),
    ("f16_64_64", torch.float16, 64, 64, 6000, 2, (3, 3, 3)),
    ("bf16_96_128", torch.bfloat16, 96, 128, 4000, 1, (3, 3, 3)),
    ("f32_7_13", torch.float32, 7, 13, 3000, 2, (3, 3, 3)),     # the reference's odd channel counts
    ("f16_16_13", torch.float16, 16, 13, 3000, 1, (3, 3, 3)),
    ("f16_3_32", torch.float16, 3, 32, 3000, 1, (3, 3, 3)),      # network stem
    ("f16_256_256", torch.float16, 256, 256, 1500, 1, (3, 3, 3)),
    # rows of several 128-byte slices: fp32 slices of 32 channels, a last slice that is partly there,
    # a map of a single tile, and column groups of 32 output channels
    ("f32_128_64", torch.float32, 128, 64, 3000, 2, (3, 3, 3)),
    ("f16_160_96", torch.float16, 160, 96, 3000, 1, (3, 3, 3)),
    ("f32_40_24", torch.float32, 40, 24, 2500, 1, (3, 3, 3)),
    ("bf16_192_32_tiny", torch.bfloat16, 192, 32, 40, 1, (3, 3, 3)),
    ("f16_128_128_k2", torch.float16, 128, 128, 3000, 1, (2, 2, 2)),
    ("f16_16_16_k5", torch.float16, 16, 16, 3000, 1, (5, 5, 5)),
    ("bf16_40_72_k2", torch.bfloat16, 40, 72, 3000, 1, (2, 2, 2)),
    # fp32 rows that are not a whole 128-byte slice under more than 64 offsets: the pair-packed
    # kernel's eight-wave instance
    ("f32_24_40_k5", torch.float32, 24, 40, 2500, 1, (5, 5, 5)),
    # wide rows on both sides and at least 96 tiles of 256 output rows: the output-stationary kernel
    # (sums in registers), with and without an identity offset, last tile partly filled; tiles of
    # 192 rows (four 48-row waves, whose rows span two 64-row groups) and, for the map of 51,000
    # rows, of 256 rows (eight 32-row waves)
    ("f16_128_128_rows", torch.float16, 128, 128, 13000, 2, (3, 3, 3)),
    ("bf16_256_128_rows", torch.bfloat16, 256, 128, 12500, 2, (3, 3, 3)),
    ("f16_128_256_rows_k2", torch.float16, 128, 256, 13000, 2, (2, 2, 2)),
    ("bf16_128_128_rows_tall", torch.bfloat16, 128, 128, 17000, 3, (3, 3, 3)),
    ("f16_256_128_rows_k1", torch.float16, 256, 128, 13000, 2, (1, 1, 1)),   # pointwise: the identity offset alone
]


@pytest.mark.parametrize("name,dtype,c_in,c_out,n,batch,ksize", CONV_CASES,
                         ids=[c[0] for c in CONV_CASES])
def test_conv_stride1_matches_oracle(oracle, name, dtype, c_in, c_out, n, batch, ksize):
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    from oracle.explicit_conv import explicit_gemm_forward
    items = [synthetic.random_cloud(10 + b, n, 26)[:, 1:] for b in range(batch)]
    bc = synthetic.batch_indexed(items)
    K = int(np.prod(ksize))
    x = normal_features(len(bc), c_in, seed=3, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=4, dtype=dtype)
    bias = (torch.randn(c_out, generator=torch.Generator().manual_seed(5)) * 0.1).to(dtype)
    vox = _voxels(items, x)
    out = spatially_sparse_conv(vox, w.to(DEV), ksize, bias=bias.to(DEV))
    assert out.feature_tensor.dtype == dtype and out.feature_tensor.shape == (len(bc), c_out)
    assert torch.equal(out.coordinate_tensor, vox.coordinate_tensor)
    got = out.feature_tensor.float().cpu().numpy()
    want, (im, om, off, iden) = _oracle_out(oracle, x, w, bc, bc, ksize, (1, 1, 1), bias)
    assert rel_err(got, want) <= TOL[dtype], name
    # and entry by entry, in the form the reference's native GEMM tests print
    # (tests/csrc/test_cutlass_gemm.py:24-26), over the entries above a thousandth of the largest
    # (a 1x1x1 kernel is a torch matmul followed by a torch add, as in the reference,
    # sparse_conv.py:1715-1721: two roundings, felt where product and bias cancel)
    assert elementwise_rel_err(got, want) <= (5e-2 if K == 1 else ELEM_TOL[dtype]), name
    # the reference's own operation order (per-offset rounding) on the CPU, same tolerance
    ref = explicit_gemm_forward(x.float() if dtype != torch.float32 else x, w.float(),
                                torch.as_tensor(im), torch.as_tensor(om), off, iden, len(bc))
    ref = ref.double().numpy() + bias.double().numpy()
    assert rel_err(got, ref) <= TOL[dtype], name


NARROW_CASES = [
    # name, dtype, c_in, c_out, kernel, voxels (0: a full 14^3 cube, runs of up to 64 pairs), extent
    ("bf16_32_32", torch.bfloat16, 32, 32, (3, 3, 3), 9000, 26),          # twelve waves: 54 KB of weights
    ("f16_24_32", torch.float16, 24, 32, (3, 3, 3), 5000, 22),            # the last quarter of the k-step is padding
    ("bf16_8_16", torch.bfloat16, 8, 16, (3, 3, 3), 5000, 22),            # 16-channel k-step, one block of output channels
    ("f16_12_20", torch.float16, 12, 20, (3, 3, 3), 5000, 22),            # output rows that are not whole 16-byte vectors
    ("f16_16_16_k5", torch.float16, 16, 16, (5, 5, 5), 4000, 24),         # more than 64 offsets, 16-channel k-step
    ("f16_32_16_k357", torch.float16, 32, 16, (3, 5, 7), 4000, 24),       # 105 offsets of 32 channels: 105 KB of weights
    ("bf16_16_16_k2", torch.bfloat16, 16, 16, (2, 2, 2), 5000, 22),       # no identity offset
    ("f16_16_32_cube", torch.float16, 16, 32, (3, 3, 3), 0, 14),          # every run full: four blocks per offset and group
    ("bf16_32_32_sparse", torch.bfloat16, 32, 32, (3, 3, 3), 3000, 60),   # nearly every run empty
]


@pytest.mark.parametrize("name,dtype,c_in,c_out,ksize,n,extent", NARROW_CASES, ids=[c[0] for c in NARROW_CASES])
def test_narrow_layers_take_the_group_kernel_and_match_the_oracle(oracle, name, dtype, c_in, c_out, ksize, n, extent):
    """16-bit rows of at most 32 channels on both sides: a wave per group of 64 output rows, all weight
    tiles in LDS (conv_fwd_group).  Every instance of the kernel, against the fp64 oracle."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    if n == 0:
        xs, ys, zs = np.meshgrid(np.arange(extent), np.arange(extent), np.arange(extent), indexing="ij")
        cube = np.stack([xs, ys, zs], axis=-1).reshape(-1, 3).astype(np.int32)
        items = [cube[np.random.default_rng(1).permutation(len(cube))]]
    else:
        items = [synthetic.random_cloud(70 + b, n, extent)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    K = int(np.prod(ksize))
    x = normal_features(len(bc), c_in, seed=21, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=22, dtype=dtype)
    bias = (torch.randn(c_out, generator=torch.Generator().manual_seed(23)) * 0.1).to(dtype)
    out = spatially_sparse_conv(_voxels(items, x), w.to(DEV), ksize, bias=bias.to(DEV))
    assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_group<"), lib().wcn_conv_last_kernel()
    got = out.feature_tensor.float().cpu().numpy()
    want, _ = _oracle_out(oracle, x, w, bc, bc, ksize, (1, 1, 1), bias)
    assert rel_err(got, want) <= TOL[dtype], name
    assert elementwise_rel_err(got, want) <= ELEM_TOL[dtype], name
    # the same call again: the additions of a row happen in a fixed order
    again = spatially_sparse_conv(_voxels(items, x), w.to(DEV), ksize, bias=bias.to(DEV))
    assert torch.equal(out.feature_tensor, again.feature_tensor)


FUSED_CASES = [
    # name, dtype, c_in, c_out, voxels, extent, kernel whose launcher takes it
    ("group", torch.bfloat16, 32, 32, 6000, 24, "conv_fwd_group"),
    ("pack", torch.float16, 64, 64, 6000, 24, "conv_fwd_pack"),
    ("pack_f32", torch.float32, 32, 24, 4000, 22, "conv_fwd_pack"),
    ("dense", torch.bfloat16, 128, 128, 30000, 64, "conv_fwd_dense"),
    ("ring_split", torch.float16, 256, 256, 1500, 16, "conv_fwd_ring"),
    ("odd_widths", torch.float32, 7, 13, 3000, 20, "conv_fwd"),  # whichever kernel takes the padded rows
]


@pytest.mark.parametrize("name,dtype,c_in,c_out,n,extent,kernel", FUSED_CASES, ids=[c[0] for c in FUSED_CASES])
def test_residual_and_relu_in_the_epilogue(oracle, name, dtype, c_in, c_out, n, extent, kernel):
    """act(conv + bias + residual) with the two extras inside the contraction (every kernel's epilogue)
    against the fp64 oracle, and against the same call followed by the two torch operations."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(80, n, extent)[:, 1:]]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), c_in, seed=31, dtype=dtype)
    w = kaiming_weight(27, c_in, c_out, seed=32, dtype=dtype)
    bias = (torch.randn(c_out, generator=torch.Generator().manual_seed(33)) * 0.1).to(dtype)
    res = normal_features(len(bc), c_out, seed=34, dtype=dtype)
    vox = _voxels(items, x)
    want, _ = _oracle_out(oracle, x, w, bc, bc, (3, 3, 3), (1, 1, 1), bias)
    for residual, relu in ((res, True), (res, False), (None, True)):
        out = spatially_sparse_conv(vox, w.to(DEV), 3, bias=bias.to(DEV),
                                    residual=None if residual is None else residual.to(DEV), relu=relu)
        assert lib().wcn_conv_last_kernel().decode().startswith(kernel), lib().wcn_conv_last_kernel()
        ref = want + (0 if residual is None else residual.double().numpy())
        ref = np.maximum(ref, 0.0) if relu else ref
        got = out.feature_tensor.float().cpu().numpy()
        assert rel_err(got, ref) <= TOL[dtype], (name, relu)
        if relu:
            assert (got >= 0).all()
    # with gradients asked for, the extras are torch operations behind the same interface
    xg = x.to(DEV).requires_grad_(True)
    out = spatially_sparse_conv(_voxels(items, xg), w.to(DEV), 3, bias=bias.to(DEV), residual=res.to(DEV), relu=True)
    out.feature_tensor.sum().backward()
    assert xg.grad is not None and rel_err(out.feature_tensor.float().detach().cpu().numpy(),
                                           np.maximum(want + res.double().numpy(), 0.0)) <= 2 * TOL[dtype]


@pytest.mark.parametrize("name,dtype,c_in,c_out,n,extent,kernel", FUSED_CASES, ids=[c[0] for c in FUSED_CASES])
def test_prepared_weight_tiles_give_the_same_bits(name, dtype, c_in, c_out, n, extent, kernel):
    """keep_prepared_weight: the tiles of the weight made once and kept on the tensor
    (wcn_conv_prepare_weight + wcn_sparse_conv_fwd_prepared) against the call that makes them every
    time, bit for bit, through every kernel; the tiles follow a change of the weight."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(81, n, extent)[:, 1:]]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), c_in, seed=41, dtype=dtype)
    w = kaiming_weight(27, c_in, c_out, seed=42, dtype=dtype).to(DEV)
    bias = (torch.randn(c_out, generator=torch.Generator().manual_seed(43)) * 0.1).to(dtype).to(DEV)
    res = normal_features(len(bc), c_out, seed=44, dtype=dtype).to(DEV)
    vox = _voxels(items, x)
    for residual, relu in ((None, False), (res, True)):
        plain = spatially_sparse_conv(vox, w, 3, bias=bias, residual=residual, relu=relu).feature_tensor
        for _ in range(2):  # the second call finds the tiles
            kept = spatially_sparse_conv(vox, w, 3, bias=bias, residual=residual, relu=relu,
                                         keep_prepared_weight=True).feature_tensor
            assert lib().wcn_conv_last_kernel().decode().startswith(kernel), lib().wcn_conv_last_kernel()
            assert torch.equal(plain, kept), (name, relu)
    tiles = w._wcn_prepared[1]
    w.mul_(0.5)  # the version counter moves: new tiles
    plain = spatially_sparse_conv(vox, w, 3, bias=bias).feature_tensor
    kept = spatially_sparse_conv(vox, w, 3, bias=bias, keep_prepared_weight=True).feature_tensor
    assert w._wcn_prepared[1] is not tiles and torch.equal(plain, kept)


def test_prepared_weight_tiles_over_an_exchanged_map_and_fp32_master_weights():
    """The transposed convolution's map (lists re-ordered by the library, offsets copied to the device
    on first use) and a float32 weight under bfloat16 features, both with kept tiles."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    items = [synthetic.random_cloud(24 + b, 5000, 30)[:, 1:] for b in range(2)]
    x = normal_features(sum(len(i) for i in items), 32, seed=9, dtype=torch.bfloat16)
    fine = _voxels(items, x)
    down = SparseConv3d(32, 64, 2, stride=2, bias=False).to(DEV)  # float32 parameters
    up = SparseConv3d(64, 32, 2, stride=2, bias=True, transposed=True).to(DEV)
    with torch.no_grad():
        coarse = down(fine)
        back = up(coarse, fine)
        down.keep_prepared_weight = up.keep_prepared_weight = True
        for _ in range(2):
            coarse_kept = down(fine)
            back_kept = up(coarse_kept, fine)
            assert torch.equal(coarse.feature_tensor, coarse_kept.feature_tensor)
            assert torch.equal(back.feature_tensor, back_kept.feature_tensor)
    assert hasattr(down.weight, "_wcn_prepared") and hasattr(up.weight, "_wcn_prepared")


def test_conv_dense_cube_equals_conv3d():
    """Textbook anchor: on a fully occupied cube with zero padding the sparse convolution is
    torch.nn.functional.conv3d (cross-correlation), W[k] <-> weight[:, :, i, j, kk].T with
    k = (i * 3 + j) * 3 + kk."""
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    S, c_in, c_out = 12, 8, 16
    g = torch.Generator().manual_seed(0)
    dense = torch.randn(1, c_in, S, S, S, generator=g)
    w = torch.randn(27, c_in, c_out, generator=g) * 0.2
    xs, ys, zs = torch.meshgrid(torch.arange(S), torch.arange(S), torch.arange(S), indexing="ij")
    coords = torch.stack([xs, ys, zs], dim=-1).reshape(-1, 3).int()
    perm = torch.randperm(len(coords), generator=g)
    coords = coords[perm]
    feats = dense[0, :, coords[:, 0].long(), coords[:, 1].long(), coords[:, 2].long()].T.contiguous()
    vox = _voxels([coords.numpy()], feats)
    out = spatially_sparse_conv(vox, w.to(DEV), 3).feature_tensor.cpu()
    w5 = w.reshape(3, 3, 3, c_in, c_out).permute(4, 3, 0, 1, 2).contiguous()
    want = torch.nn.functional.conv3d(dense, w5, padding=1)[0]
    want = want[:, coords[:, 0].long(), coords[:, 1].long(), coords[:, 2].long()].T
    assert rel_err(out.numpy(), want.numpy()) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_strided_then_transposed_pair(oracle, dtype):
    """2x2x2 stride-2 down convolution followed by its transposed convolution back onto the
    fine coordinates; the second reuses the cached map with in/out exchanged."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    items = [synthetic.random_cloud(20 + b, 5000, 30)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), 24, seed=7, dtype=dtype)
    fine = _voxels(items, x)
    down = SparseConv3d(24, 40, 2, stride=2, bias=False).to(DEV)
    up = SparseConv3d(40, 24, 2, stride=2, bias=True, transposed=True).to(DEV)
    with torch.no_grad():
        coarse = down(fine)
        assert coarse.tensor_stride == (2, 2, 2)
        assert fine.cache is not None and len(fine.cache) == 1
        back = up(coarse, fine)
        assert len(fine.cache) == 2  # transposed entry added, no new device map build
    assert back.tensor_stride in (None, (1, 1, 1))
    assert torch.equal(back.coordinate_tensor, fine.coordinate_tensor)
    # oracle: forward map fine->coarse, then the same map with in/out exchanged
    coarse_bc = coarse.batch_indexed_coordinates.cpu().numpy()
    wd = down.weight.detach().cpu()
    wu = up.weight.detach().cpu()
    im, om, off, iden = oracle.kernel_map(bc, coarse_bc, (2, 2, 2), (2, 2, 2))
    assert iden is None
    xd = x.to(dtype).double().numpy()
    mid = oracle.explicit_conv_f64(xd, wd.to(dtype).double().numpy(), im, om, off, None,
                                   len(coarse_bc))
    assert rel_err(coarse.feature_tensor.float().cpu().numpy(), mid) <= TOL[dtype]
    mid_in = coarse.feature_tensor.double().cpu().numpy()  # what the GPU fed the second conv
    want = oracle.explicit_conv_f64(mid_in, wu.to(dtype).double().numpy(), om, im, off, None,
                                    len(bc)) + up.bias.detach().to(dtype).double().cpu().numpy()
    assert rel_err(back.feature_tensor.float().cpu().numpy(), want) <= TOL[dtype]


SINGLE_CASES = [
    # name, dtype, coarse channels, fine channels, kernel = stride, voxels per item
    ("bf16_32_32", torch.bfloat16, 32, 32, (2, 2, 2), 6000),
    ("f16_64_32", torch.float16, 64, 32, (2, 2, 2), 6000),
    ("bf16_128_96", torch.bfloat16, 128, 96, (2, 2, 2), 6000),
    ("f16_256_128", torch.float16, 256, 128, (2, 2, 2), 3000),
    ("bf16_96_200", torch.bfloat16, 96, 200, (2, 1, 2), 5000),   # 25 channel blocks: the last column group partly there
    ("f16_192_8_k4", torch.float16, 192, 8, (4, 4, 4), 5000),    # 64 offsets, most of them with a handful of pairs
]


@pytest.mark.parametrize("name,dtype,c_coarse,c_fine,ks,n", SINGLE_CASES, ids=[c[0] for c in SINGLE_CASES])
def test_transposed_convolution_with_one_pair_per_output_row(oracle, name, dtype, c_coarse, c_fine, ks, n):
    """The transposed convolution that undoes a strided one with kernel = stride: every fine voxel has one
    parent, so nothing is summed and the exchanged lists are used as they are (conv_fwd_single).  Against
    the fp64 oracle, against the general path over the re-ordered lists, with residual and clamp in the
    epilogue and with kept weight tiles."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import (generate_output_coords_and_kernel_map,
                                                         spatially_sparse_conv)
    items = [synthetic.random_cloud(40 + b, n, 36)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    fine = _voxels(items, normal_features(len(bc), 8, seed=3, dtype=dtype))
    wd = kaiming_weight(int(np.prod(ks)), 8, c_coarse, seed=4, dtype=dtype).to(DEV)
    wu = kaiming_weight(int(np.prod(ks)), c_coarse, c_fine, seed=5, dtype=dtype).to(DEV)
    bias = (torch.randn(c_fine, generator=torch.Generator().manual_seed(6)) * 0.1).to(dtype).to(DEV)
    res = normal_features(len(bc), c_fine, seed=7, dtype=dtype).to(DEV)
    with torch.no_grad():
        coarse = spatially_sparse_conv(fine, wd, ks, stride=ks)
        coarse = coarse.replace(batched_features=normal_features(len(coarse.feature_tensor), c_coarse, seed=8, dtype=dtype).to(DEV))
        back = spatially_sparse_conv(coarse, wu, ks, stride=ks, bias=bias, transposed=True,
                                     output_spatially_sparse_tensor=fine)
        assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_single<"), lib().wcn_conv_last_kernel()
        _, _, km = generate_output_coords_and_kernel_map(coarse, ks, (1,) * 3, ks, False, True, fine)
        assert km._single_out and km._by_out is None  # no re-ordered lists were made
        # oracle: the forward map with its lists exchanged
        coarse_bc = coarse.batch_indexed_coordinates.cpu().numpy()
        im, om, off, _ = oracle.kernel_map(bc, coarse_bc, ks, ks)
        want = oracle.explicit_conv_f64(coarse.feature_tensor.double().cpu().numpy(), wu.double().cpu().numpy(),
                                        om, im, off, None, len(bc)) + bias.double().cpu().numpy()
        got = back.feature_tensor.float().cpu().numpy()
        assert rel_err(got, want) <= TOL[dtype] and elementwise_rel_err(got, want) <= 5e-2  # one product per entry
        # residual, clamp and kept tiles
        fused = spatially_sparse_conv(coarse, wu, ks, stride=ks, bias=bias, transposed=True,
                                      output_spatially_sparse_tensor=fine, residual=res, relu=True)
        ref = np.maximum(want + res.double().cpu().numpy(), 0.0)
        assert rel_err(fused.feature_tensor.float().cpu().numpy(), ref) <= TOL[dtype]
        kept = spatially_sparse_conv(coarse, wu, ks, stride=ks, bias=bias, transposed=True,
                                     output_spatially_sparse_tensor=fine, keep_prepared_weight=True)
        assert torch.equal(kept.feature_tensor, back.feature_tensor)
        # the general path over the same map (lists re-ordered, sums in LDS): same result up to rounding
        km._single_out = False
        general = spatially_sparse_conv(coarse, wu, ks, stride=ks, bias=bias, transposed=True,
                                        output_spatially_sparse_tensor=fine)
        assert not lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_single<")
        assert rel_err(general.feature_tensor.float().cpu().numpy(), want) <= TOL[dtype]
        km._single_out = True


def test_transposed_convolution_onto_voxels_without_a_parent_takes_the_general_path(oracle):
    """An output tensor with voxels that no coarse voxel covers: fewer pairs than output rows, so the map
    is not of the one-pair-per-row kind; those rows get the bias alone."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    dtype = torch.bfloat16
    items = [synthetic.random_cloud(61, 5000, 30)[:, 1:]]
    fine = _voxels(items, normal_features(len(items[0]), 8, seed=3, dtype=dtype))
    far = (items[0][:400] + np.array([64, 64, 64], dtype=items[0].dtype))  # a second cloud no coarse voxel covers
    wider_items = [np.concatenate([items[0], far])]
    wider = _voxels(wider_items, normal_features(len(wider_items[0]), 8, seed=4, dtype=dtype))
    wd = kaiming_weight(8, 8, 64, seed=5, dtype=dtype).to(DEV)
    wu = kaiming_weight(8, 64, 32, seed=6, dtype=dtype).to(DEV)
    bias = (torch.randn(32, generator=torch.Generator().manual_seed(7)) * 0.1).to(dtype).to(DEV)
    with torch.no_grad():
        coarse = spatially_sparse_conv(fine, wd, 2, stride=2)
        back = spatially_sparse_conv(coarse, wu, 2, stride=2, bias=bias, transposed=True,
                                     output_spatially_sparse_tensor=wider)
    assert not lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_single<")
    bc_w = synthetic.batch_indexed(wider_items)
    coarse_bc = coarse.batch_indexed_coordinates.cpu().numpy()
    im, om, off, _ = oracle.kernel_map(bc_w, coarse_bc, (2, 2, 2), (2, 2, 2))
    assert int(off[-1]) == len(items[0]) < len(bc_w)
    want = oracle.explicit_conv_f64(coarse.feature_tensor.double().cpu().numpy(), wu.double().cpu().numpy(),
                                    om, im, off, None, len(bc_w)) + bias.double().cpu().numpy()
    got = back.feature_tensor.float().cpu().numpy()
    assert rel_err(got, want) <= TOL[dtype]
    assert np.allclose(got[len(items[0]):], bias.float().cpu().numpy(), atol=1e-6)


def test_pair_lists_are_reordered_once_and_kept_on_the_map(oracle):
    """The map of a transposed convolution does not ascend in output row: its re-ordered lists
    are made on the first product and the very same tensors serve the second one."""
    import ctypes
    from warpconvnet_amd._lib import check, lib, ptr, stream_ptr, workspace
    from warpconvnet_amd.nn.functional.sparse_conv import (generate_output_coords_and_kernel_map,
                                                         spatially_sparse_conv)
    items = [synthetic.random_cloud(40 + b, 6000, 32)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), 16, seed=11)
    fine = _voxels(items, x)
    w = kaiming_weight(8, 16, 32, seed=12)
    coarse = spatially_sparse_conv(fine, w.to(DEV), 2, stride=2)
    wt = kaiming_weight(8, 32, 16, seed=13).to(DEV)
    first = spatially_sparse_conv(coarse, wt, 2, stride=2, transposed=True,
                                  output_spatially_sparse_tensor=fine)
    _, _, km = generate_output_coords_and_kernel_map(
        coarse, (2, 2, 2), (1, 1, 1), (2, 2, 2), False, True, output_spatially_sparse_tensor=fine)
    assert km._by_out is not None and not km._out_ascend
    kept = km._by_out
    second = spatially_sparse_conv(coarse, wt, 2, stride=2, transposed=True,
                                   output_spatially_sparse_tensor=fine)
    assert km._by_out is kept
    assert torch.equal(first.feature_tensor, second.feature_tensor)
    # the kept lists: same pairs per offset, ascending output rows, group starts by definition
    K = len(km)
    off = km.offsets.tolist()
    gi, go, groups = (t.cpu().numpy() for t in kept[:3])
    im, om = km.in_maps.cpu().numpy(), km.out_maps.cpu().numpy()
    M = len(bc)
    G = (M + 63) // 64
    groups = groups.reshape(K, G + 1)
    for k in range(K):
        a, b = off[k], off[k + 1]
        assert np.all(np.diff(go[a:b]) > 0)
        order = np.argsort(om[a:b], kind="stable")
        assert np.array_equal(go[a:b], om[a:b][order]) and np.array_equal(gi[a:b], im[a:b][order])
        assert np.array_equal(groups[k], np.searchsorted(go[a:b], 64 * np.arange(G + 1)))

    # direct call with duplicate (offset, output row) pairs: the lowest input row is kept
    L = lib()
    in_l = torch.tensor([9, 3, 7, 5, 1, 8], dtype=torch.int32, device=DEV)
    out_l = torch.tensor([2, 2, 0, 2, 1, 1], dtype=torch.int32, device=DEV)  # offset 0: rows 2,2,0,2; offset 1: 1,1
    host_off = (ctypes.c_int64 * 3)(0, 4, 6)
    for _ in range(3):
        ins = torch.full((6,), -7, dtype=torch.int32, device=DEV)
        outs = torch.full((6,), -7, dtype=torch.int32, device=DEV)
        gs = torch.empty(2 * 2, dtype=torch.int32, device=DEV)
        ws = workspace(L.wcn_pairs_sort_workspace_bytes(3, 2, 6), torch.device(DEV))
        check(L.wcn_pairs_sort_by_out(ptr(in_l), ptr(out_l), host_off, 2, 3, ptr(ins), ptr(outs), ptr(gs),
                                      ptr(ws), ws.numel(), stream_ptr(torch.device(DEV))), "sort")
        assert gs.tolist() == [0, 2, 0, 1]
        assert ins.tolist()[:2] == [7, 3] and outs.tolist()[:2] == [0, 2]
        assert ins.tolist()[4] == 1 and outs.tolist()[4] == 1

    # through the operator interface such lists are refused: the reference's scatter would add up
    # all three pairs of (offset 0, row 2), the device contraction takes one pair per offset and row
    from warpconvnet_amd.geometry.coords.search.search_results import IntSearchResult
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    repeated = IntSearchResult(in_l, out_l, torch.tensor([0, 4, 6], dtype=torch.int32))
    feats = torch.randn(10, 16, device=DEV)
    weights = torch.randn(2, 16, 16, device=DEV)
    with pytest.raises(ValueError, match="repeat an"):
        sparse_conv_forward(feats, weights, repeated, 3)
    # the same lists without the repeats pass, out of order as they are
    clean = IntSearchResult(in_l[[2, 4, 0]], out_l[[2, 4, 0]], torch.tensor([0, 2, 3], dtype=torch.int32))
    got = sparse_conv_forward(feats, weights, clean, 3)
    want = torch.zeros(3, 16, device=DEV)
    want[0] += feats[7] @ weights[0]
    want[1] += feats[1] @ weights[0]
    want[2] += feats[9] @ weights[1]
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
    # and with kept weight tiles: a caller's map has no offsets in device memory yet (they are copied
    # there on first use and kept on the map object)
    assert clean._device_offsets is None
    kept = sparse_conv_forward(feats, weights, clean, 3, keep_prepared_weight=True)
    assert torch.equal(got, kept) and clean._device_offsets.tolist() == [0, 2, 3]


def test_transposed_adjoint_identity():
    """<conv(x), y> == <x, conv_T(y)> when the transposed weights are W[k]^T on the same map."""
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(30, 4000, 28)[:, 1:]]
    x = normal_features(len(items[0]), 16, seed=1)
    fine = _voxels(items, x)
    w = kaiming_weight(8, 16, 24, seed=2)
    coarse = spatially_sparse_conv(fine, w.to(DEV), 2, stride=2)
    y = normal_features(len(coarse), 24, seed=3).to(DEV)
    back = spatially_sparse_conv(coarse.replace(batched_features=y), w.transpose(1, 2).contiguous().to(DEV),
                                 2, stride=2, transposed=True, output_spatially_sparse_tensor=fine)
    lhs = (coarse.feature_tensor.double() * y.double()).sum().item()
    rhs = (fine.feature_tensor.double() * back.feature_tensor.double()).sum().item()
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), 1.0)


def test_conv_linearity_and_determinism():
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(40, 5000, 28)[:, 1:]]
    n = len(items[0])
    a = normal_features(n, 32, seed=1)
    b = normal_features(n, 32, seed=2)
    w = kaiming_weight(27, 32, 48, seed=3).to(DEV)
    fa = spatially_sparse_conv(_voxels(items, a), w, 3).feature_tensor
    fb = spatially_sparse_conv(_voxels(items, b), w, 3).feature_tensor
    fab = spatially_sparse_conv(_voxels(items, 2 * a - 3 * b), w, 3).feature_tensor
    assert rel_err((2 * fa - 3 * fb).cpu().numpy(), fab.cpu().numpy()) <= 1e-5
    again = spatially_sparse_conv(_voxels(items, a), w, 3).feature_tensor
    assert torch.equal(fa, again)  # no atomics: bitwise reproducible
    # the same for rows of several slices (their products are added slice by slice, in order)
    wide = normal_features(n, 192, seed=4, dtype=torch.float16)
    ww = kaiming_weight(27, 192, 64, seed=5, dtype=torch.float16).to(DEV)
    first = spatially_sparse_conv(_voxels(items, wide), ww, 3).feature_tensor
    assert torch.equal(first, spatially_sparse_conv(_voxels(items, wide), ww, 3).feature_tensor)


def test_one_by_one_shortcut_and_errors():
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(50, 500, 20)[:, 1:]]
    x = normal_features(len(items[0]), 8, seed=1)
    vox = _voxels(items, x)
    w = kaiming_weight(1, 8, 4, seed=2).to(DEV)
    out = spatially_sparse_conv(vox, w, 1)
    assert torch.allclose(out.feature_tensor, vox.feature_tensor @ w[0])
    with pytest.raises(TypeError):
        spatially_sparse_conv(x, w, 3)
    with pytest.raises(AssertionError):
        spatially_sparse_conv(vox, kaiming_weight(8, 8, 4).to(DEV), 2, stride=2, transposed=True)


def test_module_autocast_and_backward():
    """AMP view of the features (reference: tests/nn/test_sparse_conv.py:527-585) and gradients
    of the autograd Function against the torch-CPU restatement."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    from oracle.explicit_conv import explicit_gemm_forward
    items = [synthetic.random_cloud(60, 2000, 22)[:, 1:]]
    x = normal_features(len(items[0]), 16, seed=1)
    conv = SparseConv3d(16, 32, 3).to(DEV)
    with torch.autocast("cuda", dtype=torch.float16):
        out = conv(_voxels(items, x))
    assert out.batched_features.batched_tensor.dtype == torch.float16
    # gradients
    xg = x.clone().to(DEV).requires_grad_(True)
    vox = _voxels(items, xg.detach())
    vox.batched_features.batched_tensor = xg
    out = conv(vox)
    out.feature_tensor.square().sum().backward()
    bc = synthetic.batch_indexed(items)
    from oracle import cpu_oracle
    im, om, off, iden = cpu_oracle.kernel_map(bc, bc, (3, 3, 3))
    xc = x.clone().requires_grad_(True)
    wc = conv.weight.detach().cpu().clone().requires_grad_(True)
    ref = explicit_gemm_forward(xc, wc, torch.as_tensor(im), torch.as_tensor(om), off, iden,
                                len(bc)) + conv.bias.detach().cpu()
    ref.square().sum().backward()
    assert rel_err(xg.grad.cpu().numpy(), xc.grad.numpy()) <= 1e-4
    assert rel_err(conv.weight.grad.cpu().numpy(), wc.grad.numpy()) <= 1e-4


@pytest.mark.parametrize("dtype,c_in,c_out", [(torch.float32, 7, 13), (torch.float16, 3, 32),
                                               (torch.bfloat16, 13, 7)])
def test_c_abi_with_rows_that_are_not_16_byte_vectors(oracle, dtype, c_in, c_out):
    """wcn_sparse_conv_fwd called directly with channel counts whose rows are not whole 16-byte
    vectors: the library's general kernel (the Python entry points pad such inputs instead)."""
    import ctypes
    from warpconvnet_amd._lib import DTYPE_CODE, check, lib, ptr, stream_ptr, workspace
    bc = synthetic.random_cloud(70, 4000, 22, batch_size=2)
    n = len(bc)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    x = normal_features(n, c_in, seed=1, dtype=dtype)
    w = kaiming_weight(27, c_in, c_out, seed=2, dtype=dtype)
    L = lib()
    code = DTYPE_CODE[dtype]
    ws = workspace(L.wcn_conv_workspace_bytes(n, 27, c_in, c_out, code, len(im), 1), DEV)
    out = torch.empty(n, c_out, dtype=dtype, device=DEV)
    xd, wd = x.to(DEV), w.to(DEV)
    imd, omd = _dev_i32(im), _dev_i32(om)
    offs = (ctypes.c_int64 * 28)(*[int(v) for v in off])
    check(L.wcn_sparse_conv_fwd(ptr(xd), n, c_in, code, ptr(wd), code, 27, c_out, None, ptr(imd),
                                ptr(omd), offs, iden, 1, None, ptr(out), n, ptr(ws), ws.numel(),
                                stream_ptr(torch.device(DEV))), "wcn_sparse_conv_fwd")
    want = oracle.explicit_conv_f64(x.double().numpy(), w.double().numpy(), im, om, off, iden, n)
    assert rel_err(out.float().cpu().numpy(), want) <= TOL[dtype]


def test_two_dimensional_convolution(oracle):
    """SparseConv2d on (N, 2) coordinates, forward and gradients: the device kernels run it as a
    3-D problem with a size-1 third dimension; the oracle sees the same rows with z = 0."""
    from oracle.explicit_conv import explicit_gemm_backward
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv2d
    rng = np.random.default_rng(7)
    xy = np.unique(rng.integers(-40, 40, size=(5000, 2)), axis=0).astype(np.int32)
    rng.shuffle(xy)
    n = len(xy)
    offsets = torch.tensor([0, n // 3, n])
    x = normal_features(n, 16, seed=4)
    torch.manual_seed(1)
    down = SparseConv2d(16, 24, 3, stride=2, bias=False).to(DEV)
    same = SparseConv2d(16, 24, 3, bias=False).to(DEV)
    xd = x.to(DEV).requires_grad_(True)
    vox = Voxels(torch.as_tensor(xy, device=DEV), xd, offsets=offsets)
    batch = np.repeat([0, 1], [n // 3, n - n // 3]).astype(np.int32)
    bc = np.concatenate([batch[:, None], xy, np.zeros((n, 1), np.int32)], axis=1)

    y = same(vox)
    assert y.coordinate_tensor.shape == (n, 2)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 1))
    w = same.weight.detach().cpu()
    want = oracle.explicit_conv_f64(x.double().numpy(), w.double().numpy(), im, om, off, iden, n)
    assert rel_err(y.feature_tensor.detach().cpu().numpy(), want) <= 1e-5
    gy = normal_features(n, 24, seed=5)
    y.feature_tensor.backward(gy.to(DEV))
    want_x, want_w = explicit_gemm_backward(gy.double(), x.double(), w.double(), torch.as_tensor(im),
                                            torch.as_tensor(om), off, iden)
    assert rel_err(xd.grad.cpu().numpy(), want_x.numpy()) <= 1e-5
    assert rel_err(same.weight.grad.cpu().numpy(), want_w.numpy()) <= 1e-5

    z = down(vox)
    out_bc = z.batch_indexed_coordinates.cpu().numpy()
    assert out_bc.shape[1] == 3 and z.tensor_stride == (2, 2)
    out4 = np.concatenate([out_bc, np.zeros((len(out_bc), 1), np.int32)], axis=1)
    want_set, _, _ = oracle.stride_coords(bc, (2, 2, 1), 2)
    assert np.array_equal(out4[np.lexsort(out4.T[::-1])], want_set[np.lexsort(want_set.T[::-1])])
    im, om, off, iden = oracle.kernel_map(bc, out4, (3, 3, 1), (2, 2, 1))
    want = oracle.explicit_conv_f64(x.double().numpy(), down.weight.detach().double().cpu().numpy(), im, om,
                                    off, iden, len(out4))
    assert rel_err(z.feature_tensor.detach().cpu().numpy(), want) <= 1e-5


def test_generative_convolution_expands_the_coordinates(oracle):
    """generative=True: the output voxels are the inputs plus everything a kernel offset reaches
    (reference: coords/ops/expand.py:17-64, sparse_conv.py:1852-1870), as a set equal to numpy's
    unique over all shifted rows; features against the oracle over those output rows."""
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(120 + b, 1500, 30)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), 16, seed=1)
    w = kaiming_weight(27, 16, 24, seed=2)
    out = spatially_sparse_conv(_voxels(items, x), w.to(DEV), 3, generative=True)
    out_bc = out.batch_indexed_coordinates.cpu().numpy()
    offs = oracle.kernel_offsets((3, 3, 3))
    want_set = np.unique((bc[None, :, :] + offs[:, None, :]).reshape(-1, 4), axis=0)
    assert len(out_bc) == len(want_set) > len(bc)
    assert np.array_equal(out_bc[np.lexsort(out_bc.T[::-1])], want_set)
    assert (np.diff(out_bc[:, 0]) >= 0).all()                      # batch items stay contiguous
    assert out.offsets.tolist() == [0, int((out_bc[:, 0] == 0).sum()), len(out_bc)]
    want, _ = _oracle_out(oracle, x, w, bc, out_bc, (3, 3, 3), (1, 1, 1))
    assert rel_err(out.feature_tensor.cpu().numpy(), want) <= 1e-5
    # strided and generative: the strided voxels are expanded
    out2 = spatially_sparse_conv(_voxels(items, x), w.to(DEV), 3, stride=2, generative=True)
    out2_bc = out2.batch_indexed_coordinates.cpu().numpy()
    coarse = oracle.stride_coords(bc, (2, 2, 2), 2)[0]
    want_set2 = np.unique((coarse[None, :, :] + offs[:, None, :]).reshape(-1, 4), axis=0)
    assert np.array_equal(out2_bc[np.lexsort(out2_bc.T[::-1])], want_set2)
    want2, _ = _oracle_out(oracle, x, w, bc, out2_bc, (3, 3, 3), (2, 2, 2))
    assert rel_err(out2.feature_tensor.cpu().numpy(), want2) <= 1e-5


def test_morton_ordered_output(oracle):
    """order=MORTON_XYZ: the output rows of a strided convolution are sorted along the curve inside
    every batch item (sparse_conv.py:1888-1896); features follow their voxels."""
    from warpconvnet_amd.geometry.coords.ops.serialization import POINT_ORDERING, morton_code
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    items = [synthetic.random_cloud(130 + b, 3000, 30)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), 8, seed=3)
    w = kaiming_weight(8, 8, 8, seed=4)
    out = spatially_sparse_conv(_voxels(items, x), w.to(DEV), 2, stride=2, order=POINT_ORDERING.MORTON_XYZ)
    out_bc = out.batch_indexed_coordinates
    codes = morton_code(out_bc[:, 1:].contiguous()).cpu().numpy()
    b = out_bc[:, 0].cpu().numpy()
    assert (np.diff(b) >= 0).all()
    for item in (0, 1):
        assert (np.diff(codes[b == item]) > 0).all()
    want, _ = _oracle_out(oracle, x, w, bc, out_bc.cpu().numpy(), (2, 2, 2), (2, 2, 2))
    assert rel_err(out.feature_tensor.cpu().numpy(), want) <= 1e-5


def test_dilated_convolution_matches_oracle(oracle):
    """SparseConv3d(dilation=2): the map comes from the offset-based probe, the features match the
    fp64 oracle over the oracle's dilated map."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    items = [synthetic.random_cloud(50 + b, 5000, 28)[:, 1:] for b in range(2)]
    bc = synthetic.batch_indexed(items)
    x = normal_features(len(bc), 16, seed=8)
    vox = _voxels(items, x)
    torch.manual_seed(2)
    conv = SparseConv3d(16, 24, 3, dilation=2, bias=True).to(DEV)
    with torch.no_grad():
        y = conv(vox)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3), dilation=(2, 2, 2))
    want = oracle.explicit_conv_f64(x.double().numpy(), conv.weight.detach().double().cpu().numpy(), im, om,
                                    off, iden, len(bc)) + conv.bias.detach().double().cpu().numpy()
    assert rel_err(y.feature_tensor.cpu().numpy(), want) <= 1e-5
    km = next(iter(vox.cache.values()))
    assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)


CHOICE_CASES = [
    # name, dtype, c_in, c_out, voxels, kernel: shapes the wide-row, narrow-row and pair-packed kernels take by default
    ("f16_16_16", torch.float16, 16, 16, 6000, (3, 3, 3)),
    ("bf16_32_32_k5", torch.bfloat16, 32, 32, 3000, (5, 5, 5)),
    ("f16_64_64", torch.float16, 64, 64, 6000, (3, 3, 3)),
    ("f32_32_32", torch.float32, 32, 32, 6000, (3, 3, 3)),
    ("f16_128_128_rows", torch.float16, 128, 128, 26000, (3, 3, 3)),
    ("bf16_160_96", torch.bfloat16, 160, 96, 3000, (3, 3, 3)),
]


@pytest.mark.parametrize("name,dtype,c_in,c_out,n,ksize", CHOICE_CASES, ids=[c[0] for c in CHOICE_CASES])
def test_the_kernels_behind_the_environment_switch_agree(oracle, monkeypatch, name, dtype, c_in, c_out, n, ksize):
    """WCN_CONV_KERNEL=ring keeps every shape on the ring kernel (the documented fallback),
    WCN_CONV_KERNEL=pack skips the kernels for narrow and for wide rows: all three choices against
    the oracle, and against each other within two roundings of the element type."""
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    bc = synthetic.random_cloud(77, n, 30)
    c = torch.as_tensor(bc, device=DEV)
    km = generate_kernel_map(c, c, (1, 1, 1), ksize)
    K = int(np.prod(ksize))
    x = normal_features(len(bc), c_in, seed=11, dtype=dtype)
    w = kaiming_weight(K, c_in, c_out, seed=12, dtype=dtype)
    want, _ = _oracle_out(oracle, x, w, bc, bc, ksize, (1, 1, 1))
    results, kernels = {}, {}
    for choice in ("", "pack", "ring"):
        if choice:
            monkeypatch.setenv("WCN_CONV_KERNEL", choice)
        else:
            monkeypatch.delenv("WCN_CONV_KERNEL", raising=False)
        got = sparse_conv_forward(x.to(DEV), w.to(DEV), km, len(bc))
        kernels[choice] = lib().wcn_conv_last_kernel().decode()
        results[choice] = got.float().cpu().numpy()
        assert rel_err(results[choice], want) <= TOL[dtype], (name, choice, kernels[choice])
    assert kernels["ring"].startswith(("conv_fwd_ring<", "conv_fwd<")), kernels
    assert kernels["pack"].startswith(("conv_fwd_pack<", "conv_fwd_ring<", "conv_fwd<")), kernels
    for choice in ("pack", "ring"):
        assert rel_err(results[choice], results[""]) <= 2 * TOL[dtype]
