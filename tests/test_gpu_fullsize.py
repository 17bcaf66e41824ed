"""The benchmark configurations at (or near) their full sizes, checked through properties that do
not need the CPU oracle to finish: identity weights, neighbour sums against torch index_add, the
explicit per-offset algorithm written with plain torch fp32 operations on the GPU, and the map
invariants of the strided / transposed pair."""
import numpy as np
import pytest
import torch

from helpers import elementwise_rel_err, kaiming_weight, oracle_kernel_map_by_item, rel_err, sort_rows
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def torch_explicit_fp32(x, w, km, num_out):
    """Plain torch fp32 restatement of the per-offset gather-GEMM-scatter on the GPU."""
    out = torch.zeros(num_out, w.shape[-1], dtype=torch.float32, device=x.device)
    xf, wf = x.float(), w.float()
    for k in range(len(km)):
        im, om = km[k]
        if im.numel():
            out.index_add_(0, om.long(), xf[im.long()] @ wf[k])
    return out


@pytest.fixture(scope="module")
def scenes():
    items, _ = synthetic.indoor_batch(4, 250_000)
    return torch.as_tensor(synthetic.batch_indexed(items), device=DEV)


def test_cfg2_full_size_identity_and_neighbour_sum(scenes):
    """3x3x3, 64 -> 64, fp16, 4 x 250k voxels."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    n = scenes.shape[0]
    km = generate_kernel_map(scenes, scenes, (1, 1, 1), (3, 3, 3))
    x = torch.randn(n, 64, generator=torch.Generator().manual_seed(0)).half().to(DEV)
    eye = torch.eye(64, dtype=torch.float16, device=DEV)
    w = torch.zeros(27, 64, 64, dtype=torch.float16, device=DEV)
    w[13] = eye
    assert torch.equal(sparse_conv_forward(x, w, km, n), x)          # centre tap only: a copy
    w[:] = eye                                                       # all taps: neighbour sum
    want = torch.zeros(n, 64, dtype=torch.float32, device=DEV)
    want.index_add_(0, km.out_maps.long(), x.float()[km.in_maps.long()])
    got = sparse_conv_forward(x, w, km, n)
    assert rel_err(got.float().cpu().numpy(), want.cpu().numpy()) <= 1e-2
    w = kaiming_weight(27, 64, 64, seed=1, dtype=torch.float16).to(DEV)
    got = sparse_conv_forward(x, w, km, n)
    assert rel_err(got.float().cpu().numpy(), torch_explicit_fp32(x, w, km, n).cpu().numpy()) <= 1e-2
    assert torch.equal(got, sparse_conv_forward(x, w, km, n))        # bitwise reproducible


def test_cfg3_strided_and_transposed_full_size(scenes):
    """2x2x2 stride-2 96 -> 128 and its transposed 128 -> 96, bf16."""
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    n = scenes.shape[0]
    offsets = torch.tensor([0, 250_000, 500_000, 750_000, 1_000_000])
    x = torch.randn(n, 96, generator=torch.Generator().manual_seed(2)).bfloat16().to(DEV)
    fine = Voxels(scenes[:, 1:].contiguous(), x, offsets=offsets)
    wd = kaiming_weight(8, 96, 128, seed=3, dtype=torch.bfloat16).to(DEV)
    wu = kaiming_weight(8, 128, 96, seed=4, dtype=torch.bfloat16).to(DEV)
    coarse = spatially_sparse_conv(fine, wd, 2, stride=2)
    km = next(iter(fine.cache.values()))
    assert int(km.offsets[-1]) == n and n // 8 <= len(coarse) < n
    assert torch.equal(torch.sort(km.in_maps).values, torch.arange(n, dtype=torch.int32, device=DEV))
    want = torch_explicit_fp32(x, wd, km, len(coarse))
    assert rel_err(coarse.feature_tensor.float().cpu().numpy(), want.cpu().numpy()) <= 1e-2
    back = spatially_sparse_conv(coarse, wu, 2, stride=2, transposed=True,
                                 output_spatially_sparse_tensor=fine)
    assert len(fine.cache) == 2
    from warpconvnet_amd.geometry.coords.search.search_results import IntSearchResult
    swapped = IntSearchResult(km.out_maps, km.in_maps, km.offsets)
    want = torch_explicit_fp32(coarse.feature_tensor, wu, swapped, n)
    assert rel_err(back.feature_tensor.float().cpu().numpy(), want.cpu().numpy()) <= 1e-2


def test_cfg5a_5x5x5_map_bound(scenes):
    """5x5x5 (125 offsets), 16 -> 16, fp16, 1M voxels."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    n = scenes.shape[0]
    km = generate_kernel_map(scenes, scenes, (1, 1, 1), (5, 5, 5))
    assert km.identity_map_index == 62 and len(km) == 125
    i62, o62 = km[62]
    ar = torch.arange(n, dtype=torch.int32, device=DEV)
    assert torch.equal(i62, ar) and torch.equal(o62, ar)
    counts = torch.diff(km.offsets)
    assert torch.equal(counts, counts.flip(0))
    for k in (0, 31, 61):  # (i, j) in map_k  <=>  (j, i) in map_{124-k}
        a_in, a_out = km[k]
        b_in, b_out = km[124 - k]
        assert (torch.diff(a_out) > 0).all()
        order = torch.argsort(b_in)
        assert torch.equal(b_in[order], a_out) and torch.equal(b_out[order], a_in)
    x = torch.randn(n, 16, generator=torch.Generator().manual_seed(5)).half().to(DEV)
    w = kaiming_weight(125, 16, 16, seed=6, dtype=torch.float16).to(DEV)
    got = sparse_conv_forward(x, w, km, n)
    assert rel_err(got.float().cpu().numpy(), torch_explicit_fp32(x, w, km, n).cpu().numpy()) <= 1e-2


def _assert_same_map(km, ref):
    ref_in, ref_out, ref_off, ref_iden = ref
    assert km.identity_map_index == ref_iden
    assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), ref_out)


@pytest.mark.parametrize("ksize", [(3, 3, 3), (5, 5, 5)], ids=["cfg2_3x3x3", "cfg5a_5x5x5"])
def test_full_size_map_equals_the_oracle_bit_for_bit(oracle, scenes, ksize):
    """The 1,000,000-voxel maps of the benchmark configurations against the C oracle, in native
    order (offsets in k order, ascending output row inside an offset: discrete_kernels.cu:183-213),
    from both probe passes."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    host = scenes.cpu().numpy()
    ref = oracle_kernel_map_by_item(oracle, host, host, ksize)
    _assert_same_map(generate_kernel_map(scenes, scenes, (1, 1, 1), ksize), ref)
    mp = pytest.MonkeyPatch()
    try:
        mp.setenv("WCN_KMAP_PROBE", "blocks")
        again = scenes.view(-1, 4)  # another tensor object: a table of its own
        _assert_same_map(generate_kernel_map(again, again, (1, 1, 1), ksize), ref)
    finally:
        mp.undo()


def test_full_size_strided_coordinates_and_map_equal_the_oracle(oracle, scenes):
    """cfg3: the strided coordinates of 4 x 250k voxels (as a set, and in this implementation's
    documented order: ascending first source row) and the 2x2x2 stride-2 map onto them."""
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    host = scenes.cpu().numpy()
    coarse, offs = stride_coords(scenes, (2, 2, 2))
    ref_coarse, _, ref_offs = oracle.stride_coords(host, (2, 2, 2), 4)
    got = coarse.cpu().numpy()
    assert np.array_equal(sort_rows(got), sort_rows(ref_coarse))
    assert np.array_equal(got, ref_coarse)
    assert np.array_equal(offs.numpy().astype(np.int64), ref_offs)
    ref = oracle_kernel_map_by_item(oracle, host, ref_coarse, (2, 2, 2), (2, 2, 2))
    _assert_same_map(generate_kernel_map(scenes, coarse, (2, 2, 2), (2, 2, 2)), ref)


def test_cfg5b_wide_channels_small_map():
    """3x3x3, 256 -> 256, fp16, ~50k voxels from a 16 cm voxelisation of the same scenes; checked
    against the torch-CPU restatement of the reference's explicit path."""
    from oracle import cpu_oracle
    from oracle.explicit_conv import explicit_gemm_forward
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    items = [synthetic.indoor_scene(b, None, 0.16) for b in range(4)]
    bc = synthetic.batch_indexed(items)
    n = len(bc)
    assert 30_000 < n < 80_000
    coords = torch.as_tensor(bc, device=DEV)
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    im, om, off, iden = cpu_oracle.kernel_map(bc, bc, (3, 3, 3))
    assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
    x = torch.randn(n, 256, generator=torch.Generator().manual_seed(7)).half()
    w = kaiming_weight(27, 256, 256, seed=8, dtype=torch.float16)
    got = sparse_conv_forward(x.to(DEV), w.to(DEV), km, n)
    want = explicit_gemm_forward(x, w, torch.as_tensor(im), torch.as_tensor(om), off, iden, n,
                                 compute_dtype=torch.float32)
    assert rel_err(got.float().cpu().numpy(), want.float().numpy()) <= 1e-2


def test_cfg1_spheres_fp32_contraction_matches_oracle(oracle):
    """configs[0] at its own size: 3x3x3, 32 -> 32, fp32, ~100k voxels on 3 spheres at 1 cm.  The
    kernel map is the oracle's bit for bit and the contraction matches the fp64 oracle <= 1e-5."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    from helpers import normal_features
    bc = synthetic.batch_indexed([synthetic.spheres_scene(0, 100_000, 0.01)])
    n = len(bc)
    assert n == 100_000
    coords = torch.as_tensor(bc, device=DEV)
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
    assert np.array_equal(km.offsets.numpy().astype(np.int64), off) and km.identity_map_index == iden == 13
    x = normal_features(n, 32, seed=21)
    w = kaiming_weight(27, 32, 32, seed=22)
    got = sparse_conv_forward(x.to(DEV), w.to(DEV), km, n)
    want = oracle.explicit_conv_f64(x.double().numpy(), w.double().numpy(), im, om, off, iden, n)
    assert rel_err(got.cpu().numpy(), want) <= 1e-5
