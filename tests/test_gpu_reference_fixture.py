"""The reference's own standard fixture (tests/nn/test_sparse_conv.py:35-47: three clouds of
torch.randint(1e5, 1e6) points, coordinates (rand(N, 3) / 0.01).int() in [0, 100)^3, 16 channels,
.unique()) through the two convolutions its tests run on it: 3x3x3 stride 2, 16 -> 13, fp32 with
bias (:184-223) and 3x3x3 stride 1; maps bit for bit against the oracle, features against the
fp64 oracle.  The occupancy (11 to 22 % of the cells) is several times that of a surface scan."""
import numpy as np
import pytest
import torch

from helpers import elementwise_rel_err, oracle_kernel_map_by_item, rel_err, sort_rows

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def setup_voxels():
    from warpconvnet_amd.geometry.types.voxels import Voxels
    torch.manual_seed(0)
    B, min_N, max_N, C = 3, 100000, 1000000, 16
    Ns = torch.randint(min_N, max_N, (B,))
    voxel_size = 0.01
    coords = [(torch.rand((N, 3)) / voxel_size).int() for N in Ns]
    features = [torch.rand((N, C)) for N in Ns]
    return Voxels(coords, features, device=DEV).unique()


def _host_rows(vox):
    from warpconvnet_amd.geometry.coords.ops.batch_index import batch_indexed_coordinates
    return batch_indexed_coordinates(vox.coordinate_tensor, vox.offsets).cpu().numpy()


def test_fixture_is_what_the_reference_builds(setup_voxels):
    vox = setup_voxels
    rows = _host_rows(vox)
    assert vox.num_channels == 16 and vox.batch_size == 3
    assert rows[:, 1:].min() >= 0 and rows[:, 1:].max() < 100
    assert len(np.unique(rows, axis=0)) == len(rows)  # .unique() left no repeated voxel
    per_item = np.diff(vox.offsets.numpy())
    assert (per_item > 100_000 * 0.9).all() and (per_item < 1_000_000).all()


def test_stride2_16_to_13_fp32_with_bias(oracle, setup_voxels):
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    vox = setup_voxels
    g = torch.Generator().manual_seed(1)
    weights = torch.randn(27, 16, 13, generator=g)
    bias = torch.randn(13, generator=g)
    out = spatially_sparse_conv(vox, weight=weights.to(DEV), bias=bias.to(DEV), kernel_size=(3, 3, 3),
                                stride=(2, 2, 2))
    assert out.num_channels == 13
    rows, out_rows = _host_rows(vox), _host_rows(out)
    ref_coarse, _, ref_offs = oracle.stride_coords(rows, (2, 2, 2), 3)
    assert np.array_equal(sort_rows(out_rows), sort_rows(ref_coarse))
    assert np.array_equal(out_rows, ref_coarse)  # this implementation's order: ascending first source row
    assert np.array_equal(out.offsets.numpy().astype(np.int64), ref_offs)
    km = next(iter(vox.cache.values()))
    ref_in, ref_out, ref_off, ref_iden = oracle_kernel_map_by_item(oracle, rows, ref_coarse, (3, 3, 3), (2, 2, 2))
    assert km.identity_map_index == ref_iden
    assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), ref_out)
    want = oracle.explicit_conv_f64(vox.feature_tensor.double().cpu().numpy(), weights.double().numpy(),
                                    ref_in, ref_out, ref_off, ref_iden, len(ref_coarse)) + bias.double().numpy()
    got = out.feature_tensor.cpu().numpy()
    assert rel_err(got, want) <= 1e-5
    assert elementwise_rel_err(got, want) <= 1e-3  # see tests/test_gpu_conv.py on this bound


@pytest.mark.parametrize("dtype,c_out", [(torch.float16, 16), (torch.float32, 13)], ids=["f16_16_16", "f32_16_13"])
def test_stride1_same_coordinates(oracle, setup_voxels, dtype, c_out):
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    vox = setup_voxels
    x = vox.feature_tensor.to(dtype)
    from warpconvnet_amd.geometry.types.voxels import Voxels
    vin = Voxels(vox.coordinate_tensor, x, offsets=vox.offsets)  # a map cache of its own
    g = torch.Generator().manual_seed(2)
    weights = (torch.randn(27, 16, c_out, generator=g) * (2.0 / (16 * 27)) ** 0.5).to(dtype)
    out = spatially_sparse_conv(vin, weight=weights.to(DEV), kernel_size=(3, 3, 3))
    rows = _host_rows(vox)
    km = next(iter(vin.cache.values()))
    ref_in, ref_out, ref_off, ref_iden = oracle_kernel_map_by_item(oracle, rows, rows, (3, 3, 3))
    assert km.identity_map_index == ref_iden == 13
    assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), ref_out)
    want = oracle.explicit_conv_f64(x.double().cpu().numpy(), weights.double().numpy(), ref_in, ref_out, ref_off,
                                    ref_iden, len(rows))
    got = out.feature_tensor.float().cpu().numpy()
    assert rel_err(got, want) <= (1e-2 if dtype == torch.float16 else 1e-5)
    assert elementwise_rel_err(got, want) <= (1e-2 if dtype == torch.float16 else 1e-3)
