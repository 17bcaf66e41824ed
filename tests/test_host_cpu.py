"""Host-side logic and the C-ABI surface, without a GPU: containers, cache keys, argument
checks, and that libwcn_hip.so loads and exports every symbol include/wcn_hip.h declares."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI -----------------------------------------------------------------------------------

def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "wcn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wcn_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from warpconvnet_amd._lib import SIGNATURES, lib
    handle = lib()
    declared = _declared_symbols()
    assert len(declared) >= 18
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in include/wcn_hip.h but not exported"
    assert sorted(SIGNATURES) == declared, "ctypes binding and header disagree"


def test_size_queries_and_status_strings():
    from warpconvnet_amd._lib import lib
    L = lib()
    assert L.wcn_version() >= 100
    for code in range(0, -7, -1):
        assert L.wcn_status_string(code).decode() not in ("", "unknown status")
    assert L.wcn_status_string(-99).decode() == "unknown status"
    for n in (0, 1, 1000, 10**6, 10**8):
        cap = L.wcn_table_default_capacity(n)
        assert cap >= 1024 and cap & (cap - 1) == 0 and cap >= n // 2
        assert L.wcn_table_bytes(n, cap) >= 256 + 32 * cap + 8 * n
    assert L.wcn_kmap_workspace_bytes(10**6, 27) >= 27 * (10**6 // 64 + 1) * 4
    assert L.wcn_kmap_workspace_bytes(10, 0) == 0 and L.wcn_kmap_workspace_bytes(10, 5000) == 0
    assert L.wcn_conv_workspace_bytes(1000, 27, 64, 64, 1, 5000, 1) >= 27 * 64 * 64 * 2
    assert L.wcn_conv_workspace_bytes(1000, 27, 64, 64, 1, 5000, 0) >= 27 * 64 * 64 * 2 + 8 * 5000 + 4 * 1000 + 8 * 27 * 16
    assert L.wcn_conv_workspace_bytes(1000, 27, 64, 64, 7, 0, 1) == 0
    assert L.wcn_stride_unique_workspace_bytes(1000, 1024) > 16 * 1000


def test_entry_points_reject_bad_arguments_before_touching_the_device():
    from warpconvnet_amd._lib import lib
    L = lib()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    three = (ctypes.c_int32 * 3)(3, 3, 3)
    bad = (ctypes.c_int32 * 3)(3, 0, 3)
    assert L.wcn_table_build(fake, 10, null, 1024, null) == -1
    assert L.wcn_table_build(fake, 10, fake, 1000, null) == -1      # capacity not a power of two
    assert L.wcn_table_build(fake, -1, fake, 1024, null) == -1
    assert L.wcn_table_query(fake, 10, 1000, fake, 5, fake, null) == -1
    assert L.wcn_kmap_count(fake, 10, 1024, fake, 5, bad, three, fake, null) == -1
    assert L.wcn_kmap_count(fake, 10, 1024, fake, 5, three, three, null, null) == -1
    big = (ctypes.c_int32 * 3)(11, 11, 11)                             # 1331 offsets > 1024
    assert L.wcn_kmap_count(fake, 10, 1024, fake, 5, big, three, fake, null) == -1
    assert L.wcn_kmap_fill(fake, 10, 1024, fake, 5, bad, three, fake, 100, fake, fake, null) == -1
    assert L.wcn_kmap_fill(fake, 10, 1024, fake, 5, three, three, fake, 100, null, null, null) == -1
    assert L.wcn_kmap_fill(fake, 10, 1024, fake, 5, three, three, fake, -1, fake, fake, null) == -1
    assert L.wcn_stride_unique(fake, 10, bad, fake, 1024, fake, fake, null) == -1
    one = (ctypes.c_int32 * 3)(1, 1, 1)
    zero = (ctypes.c_int32 * 3)(0, 0, 0)
    assert L.wcn_kmap_count_dilated(fake, 10, 1024, fake, 5, three, three, zero, one, fake, null) == -1  # dilation 0
    assert L.wcn_kmap_count_dilated(fake, 10, 1024, fake, 5, bad, three, one, one, fake, null) == -1
    assert L.wcn_kmap_count_dilated(fake, 10, 1024, fake, 5, three, three, one, one, null, null) == -1
    offs = (ctypes.c_int64 * 28)(*([0] * 28))
    assert L.wcn_pairs_sort_workspace_bytes(1000, 27, 5000) >= 4 * 1000 + 8 * 27 * 16   # row bits + per-group masks
    assert L.wcn_pairs_sort_workspace_bytes(1000, 0, 5000) == 0
    assert L.wcn_pairs_sort_by_out(fake, fake, offs, 27, 10, fake, fake, null, fake, 1 << 20, null) == -1   # no group table
    assert L.wcn_pairs_sort_by_out(fake, fake, None, 27, 10, fake, fake, fake, fake, 1 << 20, null) == -1
    assert L.wcn_pairs_sort_by_out(fake, fake, offs, 27, 10, fake, fake, fake, fake, 16, null) == -6         # workspace too small
    too_many = (ctypes.c_int64 * 201)(*([0] * 201))
    assert L.wcn_sparse_conv_fwd_static(fake, 10, 64, 1, fake, 1, 200, 64, null, fake, fake, too_many, -1, 1,
                                        null, fake, 10, null) == -1                                       # > 127 offsets
    assert L.wcn_sparse_conv_fwd_static(fake, 10, 64, 1, fake, 1, 27, 64, null, fake, fake, offs, -1, 1,
                                        null, fake, 10_000_000, null) == -6                               # beyond the 4 MiB array

    def conv(dtype=1, wdtype=1, ws_bytes=1 << 30, ascend=1, gs=null, offsets=offs):
        return L.wcn_sparse_conv_fwd(fake, 10, 64, dtype, fake, wdtype, 27, 64, null, fake, fake,
                                     offsets, -1, ascend, gs, fake, 10, fake, ws_bytes, null)

    # weight tiles made ahead of the call
    assert L.wcn_conv_prepared_weight_bytes(27, 64, 64, 1) >= 27 * 64 * 64 * 2
    assert L.wcn_conv_prepared_weight_bytes(27, 3, 20, 2) >= 27 * 32 * 32 * 2    # channels padded to whole tiles
    assert L.wcn_conv_prepared_weight_bytes(0, 64, 64, 1) == 0 and L.wcn_conv_prepared_weight_bytes(27, 64, 64, 5) == 0
    assert L.wcn_conv_prepared_workspace_bytes(1_000_000, 27, 64, 64, 1) == 0   # no split of input-channel slices
    assert L.wcn_conv_prepared_workspace_bytes(1500, 27, 256, 256, 1) >= 4 * 4 * 1500 * 256
    assert L.wcn_conv_prepare_weight(fake, 1, 27, 64, 64, 1, null, 1 << 20, null) == -1
    assert L.wcn_conv_prepare_weight(fake, 2, 27, 64, 64, 1, fake, 1 << 20, null) == -1   # bf16 weight, f16 tiles
    assert L.wcn_conv_prepare_weight(fake, 1, 27, 64, 64, 1, fake, 16, null) == -6

    def prepared(tile_bytes=1 << 20, dev_offsets=fake, gs=fake, ws=null, ws_bytes=0, c=64, n=10, residual=null, out=fake):
        return L.wcn_sparse_conv_fwd_prepared(fake, 10, c, 1, fake, tile_bytes, 27, c, null, fake, fake, offs,
                                              dev_offsets, -1, gs, residual, 0, out, n, ws, ws_bytes, null)

    assert prepared(dev_offsets=null) == -1          # the offsets have to be in device memory as well
    assert prepared(gs=null) == -1                   # and the group starts come with the map
    assert prepared(tile_bytes=16) == -6
    assert prepared(c=256, n=1500, tile_bytes=1 << 23) == -6   # this shape splits slices: partial sums need room
    assert prepared(residual=fake, out=fake) == -1   # the residual may not be the output buffer
    # one pair per output row
    assert L.wcn_conv_single_supported(1, 128, 96, 8) == 1 and L.wcn_conv_single_supported(2, 32, 8, 64) == 1
    assert L.wcn_conv_single_supported(0, 128, 96, 8) == 0      # fp32 features
    assert L.wcn_conv_single_supported(1, 40, 96, 8) == 0       # rows that are not whole 32-channel steps
    assert L.wcn_conv_single_supported(1, 160, 96, 8) == 0      # no instance for five steps
    assert L.wcn_conv_single_supported(1, 128, 260, 8) == 0 and L.wcn_conv_single_supported(1, 128, 96, 65) == 0
    eight = (ctypes.c_int64 * 9)(0, 1, 2, 3, 4, 5, 6, 7, 10)

    def single(num_out=10, offsets=eight, c_in=128, ws=fake, ws_bytes=1 << 20, prepared=0, residual=null, out=fake):
        return L.wcn_sparse_conv_fwd_single(fake, 10, c_in, 1, fake, 1, prepared, 8, 96, null, fake, fake, offsets,
                                            residual, 0, out, num_out, ws, ws_bytes, null)

    assert single(num_out=11) == -1                  # as many pairs as output rows, or it is not this kind of map
    assert single(c_in=40) == -1
    assert single(ws_bytes=16) == -6                 # room for the weight tiles
    assert single(offsets=None) == -1
    assert single(residual=fake, out=fake) == -1
    assert conv(dtype=9) == -1
    assert conv(wdtype=2) == -1                      # f16 features with bf16 weights
    assert conv(ws_bytes=16) == -6                   # workspace too small
    assert conv(ascend=0, gs=fake) == -1             # group starts need ascending pairs
    assert conv(offsets=None) == -1
    offs[3] = 5
    assert conv() == -1                              # offsets not monotone


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from warpconvnet_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


# ---- containers ------------------------------------------------------------------------------

def _voxels(**kw):
    from warpconvnet_amd.geometry.types.voxels import Voxels
    g = torch.Generator().manual_seed(0)
    coords = [torch.randint(0, 50, (n, 3), generator=g, dtype=torch.int32) for n in (11, 7, 5)]
    feats = [torch.randn(len(c), 6, generator=g) for c in coords]
    return Voxels(coords, feats, **kw), coords, feats


def test_voxels_construction_offsets_and_batch_index():
    """reference: tests/types/test_voxels.py:30-46."""
    vox, coords, feats = _voxels(voxel_size=0.02)
    assert vox.batch_size == 3 and len(vox) == 23 and vox.num_channels == 6
    assert vox.offsets.tolist() == [0, 11, 18, 23] and not vox.offsets.is_cuda
    assert vox.num_spatial_dims == 3 and vox.voxel_size == 0.02 and vox.tensor_stride is None
    bc = vox.batch_indexed_coordinates
    assert bc.shape == (23, 4) and bc.dtype == torch.int32
    assert bc[:, 0].tolist() == [0] * 11 + [1] * 7 + [2] * 5
    assert torch.equal(bc[:, 1:], torch.cat(coords))
    assert torch.equal(vox.feature_tensor, torch.cat(feats))
    from warpconvnet_amd.geometry.types.voxels import Voxels
    again = Voxels(torch.cat(coords), torch.cat(feats), offsets=vox.offsets)
    assert torch.equal(again.coordinate_tensor, vox.coordinate_tensor)
    with pytest.raises(AssertionError):
        Voxels(torch.cat(coords), torch.cat(feats))  # tensor input needs offsets
    with pytest.raises(AssertionError):
        Voxels(torch.cat(coords).float(), torch.cat(feats), offsets=vox.offsets)


def test_voxels_replace_keeps_extra_attributes_and_cache():
    """reference: tests/types/test_voxels.py:189-239 and geometry.py:313-347."""
    from warpconvnet_amd.geometry.coords.search.cache import IntSearchCache
    vox, _, _ = _voxels(voxel_size=0.05, custom="x", tensor_stride=2)
    assert vox.tensor_stride == (2, 2, 2) and vox.stride == (2, 2, 2)
    vox._extra_attributes["_cache"] = IntSearchCache()
    new = vox.replace(batched_features=vox.feature_tensor * 2)
    assert new.extra_attributes["custom"] == "x" and new.voxel_size == 0.05
    assert new.cache is vox.cache
    assert new.tensor_stride == (2, 2, 2)
    assert torch.equal(new.feature_tensor, vox.feature_tensor * 2)
    newer = new.replace(tensor_stride=(4, 4, 4), voxel_size=0.1)
    assert newer.tensor_stride == (4, 4, 4) and newer.voxel_size == 0.1
    half = vox.half()
    assert half.feature_tensor.dtype == torch.float16 and half.extra_attributes["custom"] == "x"
    assert vox.to(dtype=torch.float64).dtype == torch.float64


def test_int_search_result_and_cache_key():
    from warpconvnet_amd.geometry.coords.search.cache import IntSearchCache, IntSearchCacheKey
    from warpconvnet_amd.geometry.coords.search.search_results import IntSearchResult
    km = IntSearchResult(torch.tensor([5, 6, 7, 8], dtype=torch.int32),
                         torch.tensor([0, 1, 0, 2], dtype=torch.int32),
                         torch.tensor([0, 2, 2, 4], dtype=torch.int32), identity_map_index=1)
    assert len(km) == 3 and km.numel(0) == 2 and km.numel(1) == 0
    assert km[2][0].tolist() == [7, 8] and km[2][1].tolist() == [0, 2]
    assert [a.tolist() for a, _ in km] == [[5, 6], [], [7, 8]]
    ins, outs = km.get_batch(0, 3, out_format="tensor")
    assert ins.tolist() == [[5, 6], [-1, -1], [7, 8]]
    with pytest.raises(AssertionError):
        IntSearchResult(km.in_maps, km.out_maps, torch.tensor([0, 2, 3]))
    clone = km.clone()
    assert clone.identity_map_index == 1 and torch.equal(clone.in_maps, km.in_maps)

    def key(**kw):
        base = dict(kernel_size=(3, 3, 3), kernel_dilation=(1, 1, 1), transposed=False,
                    generative=False, stride_mode="stride_only", skip_symmetric_kernel_map=False,
                    in_offsets=torch.tensor([0, 4, 9]), out_offsets=torch.tensor([0, 4, 9]))
        base.update(kw)
        return IntSearchCacheKey(**base)

    cache = IntSearchCache()
    cache.put(key(), km)
    assert cache.get(key()) is km and hash(key()) == hash(key())
    assert cache.get(key(transposed=True)) is None
    assert cache.get(key(kernel_size=(2, 2, 2))) is None
    assert cache.get(key(out_offsets=torch.tensor([0, 3, 9]))) is None


def test_ntuple_and_offsets_helpers():
    from warpconvnet_amd.geometry.coords.ops.batch_index import batch_index_from_offset, \
        batch_indexed_coordinates, offsets_from_batch_index
    from warpconvnet_amd.utils.ntuple import ntuple
    assert ntuple(3, 3) == (3, 3, 3) and ntuple([1, 2, 3], 3) == (1, 2, 3)
    assert ntuple(torch.tensor([2, 2]), 2) == (2, 2)
    with pytest.raises(AssertionError):
        ntuple((1, 2), 3)
    off = torch.tensor([0, 2, 2, 5])
    assert batch_index_from_offset(off).tolist() == [0, 0, 2, 2, 2]
    assert offsets_from_batch_index(torch.tensor([0, 0, 1, 1, 2, 2, 2, 3, 3])).tolist() == [0, 2, 4, 7, 9]
    bc = batch_indexed_coordinates(torch.arange(15, dtype=torch.int32).reshape(5, 3), off)
    assert bc.dtype == torch.int32 and bc[:, 0].tolist() == [0, 0, 2, 2, 2]


def test_kernel_offsets_from_size_matches_oracle(oracle):
    from warpconvnet_amd.geometry.coords.search.torch_discrete import kernel_offsets_from_size
    for ks, dil in (((3, 3, 3), (1, 1, 1)), ((2, 2, 2), (1, 1, 1)), ((3, 2, 5), (1, 2, 3))):
        assert np.array_equal(kernel_offsets_from_size(ks, dil).numpy(), oracle.kernel_offsets(ks, dil))


def test_reference_import_path_resolves_to_the_same_modules():
    """`warpconvnet.*` (the reference's package name) names the very modules of this package."""
    import importlib
    import warpconvnet  # noqa: F401
    for rel in ("nn.modules.sparse_conv", "nn.functional.sparse_conv", "geometry.types.voxels",
                "geometry.coords.search.torch_discrete", "geometry.coords.ops.stride"):
        m = importlib.import_module("warpconvnet." + rel)
        assert m is importlib.import_module("warpconvnet_amd." + rel)
        # the alias leaves the module's own spec in place (relative imports inside it go by it)
        assert m.__spec__.name == m.__name__ == "warpconvnet_amd." + rel
        assert m.__spec__.parent == m.__package__
    from warpconvnet.nn.modules.sparse_conv import SparseConv3d
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d as ours
    assert SparseConv3d is ours
    with pytest.raises(ModuleNotFoundError):
        importlib.import_module("warpconvnet.nn.modules.attention")


def test_thread_release_without_any_call_is_a_no_op():
    from warpconvnet_amd._lib import lib
    assert lib().wcn_thread_release() == 0
    assert lib().wcn_thread_release() == 0


# ---- module / functional argument handling -----------------------------------------------------

def test_module_parameters_and_init_bound():
    """weight (K, C_in, C_out) uniform within sqrt(3) * sqrt(2 / (1 + 5)) / sqrt(C_in * K)
    (reference: nn/modules/sparse_conv.py:136,159-191)."""
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv2d, SparseConv3d, SpatiallySparseConv
    torch.manual_seed(0)
    m = SparseConv3d(16, 32, 3)
    assert tuple(m.weight.shape) == (27, 16, 32) and tuple(m.bias.shape) == (32,)
    bound = math.sqrt(3) * math.sqrt(2.0 / 6.0) / math.sqrt(16 * 27)
    assert m.weight.abs().max().item() <= bound and m.weight.abs().max().item() > 0.9 * bound
    assert m.bias.abs().max().item() <= 1 / math.sqrt(16 * 27)
    assert list(m.state_dict()) == ["weight", "bias"]
    t = SparseConv3d(16, 32, 2, stride=2, transposed=True, bias=False)
    assert t.bias is None and tuple(t.weight.shape) == (8, 16, 32) and t.stride == (2, 2, 2)
    assert t.weight.abs().max().item() <= math.sqrt(3) * math.sqrt(2.0 / 6.0) / math.sqrt(32 * 8)
    assert SparseConv2d(4, 4, 3).kernel_size == (3, 3)
    assert SpatiallySparseConv(4, 4, (3, 1, 3), fwd_algo="explicit_gemm").kernel_size == (3, 1, 3)
    assert "kernel_size=(3, 3, 3)" in repr(m)


def test_functional_type_errors_and_cpu_guard():
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import HashMethod, TorchHashTable
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    vox, _, _ = _voxels()
    w = torch.randn(27, 6, 4)
    with pytest.raises(TypeError):
        spatially_sparse_conv(vox.feature_tensor, w, 3)
    with pytest.raises(TypeError):
        spatially_sparse_conv(vox, w, 3, output_spatially_sparse_tensor=vox.feature_tensor)
    # 1x1 shortcut is plain torch and works anywhere
    out = spatially_sparse_conv(vox, torch.randn(1, 6, 4), 1, bias=torch.ones(4))
    assert out.feature_tensor.shape == (23, 4)
    table = TorchHashTable(64)
    with pytest.raises(ValueError):
        table.insert(torch.zeros(4, 4, dtype=torch.int32))           # CPU tensor
    with pytest.raises(TypeError):
        table.insert(np.zeros((4, 4), dtype=np.int32))
    with pytest.raises(TypeError):
        TorchHashTable(64, hash_method="city")
    with pytest.raises(RuntimeError):
        table.search(torch.zeros(1, 4, dtype=torch.int32))
    assert HashMethod.CITY.kernel_suffix() == "city"
    with pytest.raises(ValueError):                                   # no silent CPU fallback
        from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
        from warpconvnet_amd.geometry.coords.search.search_results import IntSearchResult
        km = IntSearchResult(torch.zeros(0, dtype=torch.int32), torch.zeros(0, dtype=torch.int32),
                             torch.zeros(28, dtype=torch.int32))
        sparse_conv_forward(vox.feature_tensor, w, km, 23)


def test_synthetic_scenes_are_seeded_and_unique():
    from warpconvnet_amd.utils import synthetic
    a = synthetic.indoor_scene(3, 5000)
    b = synthetic.indoor_scene(3, 5000)
    assert np.array_equal(a, b) and a.dtype == np.int32 and a.shape == (5000, 3)
    assert len(np.unique(a, axis=0)) == 5000
    s = synthetic.spheres_scene(1, 3000)
    assert len(np.unique(s, axis=0)) == 3000
    bc = synthetic.batch_indexed([a, s])
    assert bc.shape == (8000, 4) and (np.diff(bc[:, 0]) >= 0).all()


def test_voxels_dense_round_trip():
    """from_dense / to_dense (reference: tests/types/test_voxels.py:241-267 round trip)."""
    from warpconvnet_amd.geometry.types.voxels import Voxels
    g = torch.Generator().manual_seed(0)
    dense = torch.randn(2, 3, 5, 6, 4, generator=g)
    dense = dense * (torch.rand(2, 1, 5, 6, 4, generator=g) < 0.3)  # ~30 % occupied
    vox = Voxels.from_dense(dense)
    occupied = int((dense.abs().sum(1) > 0).sum())
    assert len(vox) == occupied and vox.num_channels == 3 and vox.batch_size == 2
    assert vox.offsets.tolist() == [0, int((dense[0].abs().sum(0) > 0).sum()), occupied]
    bc = vox.batch_indexed_coordinates
    assert torch.equal(dense[bc[:, 0].long(), :, bc[:, 1].long(), bc[:, 2].long(), bc[:, 3].long()],
                       vox.feature_tensor)
    # back onto the same grid
    back = vox.to_dense(channel_dim=1, min_coords=(0, 0, 0), max_coords=(4, 5, 3))
    assert torch.equal(back, dense)
    assert torch.equal(vox.to_dense(channel_dim=1, spatial_shape=(5, 6, 4)), dense)
    # bounding-box form: the grid starts at the minimum coordinate
    lo = vox.coordinate_tensor.min(0).values.tolist()
    hi = vox.coordinate_tensor.max(0).values.tolist()
    box = vox.to_dense(channel_dim=-1)
    assert box.shape == (2, hi[0] - lo[0] + 1, hi[1] - lo[1] + 1, hi[2] - lo[2] + 1, 3)
    assert torch.equal(box.movedim(-1, 1), dense[:, :, lo[0]:hi[0] + 1, lo[1]:hi[1] + 1, lo[2]:hi[2] + 1])
    # a window drops what lies outside
    win = vox.to_dense(channel_dim=1, min_coords=(1, 1, 1), spatial_shape=(3, 3, 2))
    assert torch.equal(win, dense[:, :, 1:4, 1:4, 1:3])
    # dense values read back at a target tensor's coordinates (shifted to its minimum)
    other = torch.randn(2, 7, 5, 6, 4, generator=g)
    shifted = torch.zeros_like(other)
    shifted[:, :, :5 - lo[0], :6 - lo[1], :4 - lo[2]] = other[:, :, lo[0]:, lo[1]:, lo[2]:]
    picked = Voxels.from_dense(shifted, target_spatial_sparse_tensor=vox)
    assert torch.equal(picked.feature_tensor,
                       other[bc[:, 0].long(), :, bc[:, 1].long(), bc[:, 2].long(), bc[:, 3].long()])
    # two spatial dimensions
    d2 = torch.randn(1, 2, 4, 4, generator=g) * (torch.rand(1, 1, 4, 4, generator=g) < 0.5)
    assert torch.equal(Voxels.from_dense(d2).to_dense(spatial_shape=(4, 4)), d2)


def test_voxelisation_entry_points_reject_bad_arguments():
    from warpconvnet_amd._lib import lib
    L = lib()
    null = ctypes.c_void_p(0)
    fake = ctypes.c_void_p(4096)  # never dereferenced: validation fails first
    count = ctypes.c_int64(7)
    ok = (ctypes.c_int64 * 3)(0, 4, 10)
    assert L.wcn_unique_rows_workspace_bytes(-1) == 0 and L.wcn_unique_rows_workspace_bytes(1 << 31) == 0
    small, large = L.wcn_unique_rows_workspace_bytes(1000), L.wcn_unique_rows_workspace_bytes(10**6)
    assert small >= 256 + 1000 * 28 and large >= 256 + 10**6 * 28
    assert L.wcn_unique_rows_csr(fake, 10, 5, fake, 1 << 30, null, null, null, null, null, ctypes.byref(count), null) == -1
    assert L.wcn_unique_rows_csr(fake, 10, 0, fake, 1 << 30, null, null, null, null, null, ctypes.byref(count), null) == -1
    assert L.wcn_unique_rows_csr(fake, 10, 4, fake, 1 << 30, null, null, null, null, null, None, null) == -1
    assert L.wcn_unique_rows_csr(null, 10, 4, fake, 1 << 30, null, null, null, null, null, ctypes.byref(count), null) == -1
    assert L.wcn_unique_rows_csr(fake, 10, 4, fake, 64, null, null, null, null, null, ctypes.byref(count), null) == -6
    assert count.value == 0
    for offsets, batch, size in ((ok, 2, 0.0), (ok, 2, -1.0), ((ctypes.c_int64 * 3)(0, 4, 9), 2, 0.1),
                                 ((ctypes.c_int64 * 3)(1, 4, 10), 2, 0.1), ((ctypes.c_int64 * 3)(0, 11, 10), 2, 0.1),
                                 (ok, 0, 0.1), (None, 2, 0.1)):
        assert L.wcn_voxel_rows(fake, 10, offsets, null, batch, size, fake, null) == -1
        assert L.wcn_voxelize_points_csr(fake, 10, offsets, null, batch, size, fake, 1 << 30, null, null, null,
                                         null, null, ctypes.byref(count), null) == -1
    for offsets, rows, dims, batch in ((ok, 10, 0, 2), (ok, 9, 3, 2), (ok, 10, 3, 0), (None, 10, 3, 2),
                                       ((ctypes.c_int64 * 3)(1, 4, 10), 10, 3, 2),
                                       ((ctypes.c_int64 * 3)(0, 11, 10), 10, 3, 2), (ok, -1, 3, 2)):
        assert L.wcn_batch_indexed_rows(fake, rows, dims, offsets, batch, fake, null) == -1
    assert L.wcn_batch_indexed_rows(null, 10, 3, ok, 2, fake, null) == -1
    assert L.wcn_batch_indexed_rows(null, 0, 3, (ctypes.c_int64 * 2)(0, 0), 1, null, null) == 0  # nothing to do
    many = (ctypes.c_int64 * 102)(*range(0, 102))  # 101 batch items: the offsets must also be on the device
    assert L.wcn_batch_indexed_rows(fake, 101, 3, many, 101, fake, null) == -1  # more than travel with a launch
    assert L.wcn_voxel_rows(fake, 101, many, null, 101, 0.1, fake, null) == -1
    assert L.wcn_voxelize_points_csr(fake, 10, ok, null, 2, 0.1, fake, 64, null, null, null, null, null,
                                     ctypes.byref(count), null) == -6
    offs = (ctypes.c_int64 * 2)(0, 5)
    assert L.wcn_segment_reduce(fake, 5, 8, 7, offs, null, 5, 1, 0, fake, null, null) == -1     # dtype
    assert L.wcn_segment_reduce(fake, 5, 8, 0, offs, null, 5, 1, 4, fake, null, null) == -1     # mode
    assert L.wcn_segment_reduce(fake, 5, 0, 0, offs, null, 5, 1, 0, fake, null, null) == -1     # channels
    assert L.wcn_segment_reduce(fake, 5, 8, 0, None, null, 5, 1, 0, fake, null, null) == -1
    assert L.wcn_segment_reduce(fake, 5, 8, 0, offs, null, 5, 0, 0, null, null, null) == 0      # nothing to do
    assert L.wcn_segment_reduce_bwd(fake, 1, 8, 0, offs, fake, 5, 2, null, fake, null) == -1  # max without argmax
    assert L.wcn_segment_reduce_bwd(fake, 1, 8, 0, offs, null, 5, 0, null, fake, null) == -1  # no segment ids


def test_points_reductions_and_unique_host_logic():
    import torch
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.nn.functional.point_pool import point_pool
    from warpconvnet_amd.ops.reductions import REDUCTIONS, row_reduction
    from warpconvnet_amd.utils.unique import ToUnique, UniqueInfo
    import warpconvnet_amd.nn.functional.sparse_pool as sparse_pool
    assert sparse_pool.REDUCTIONS is REDUCTIONS  # one enum for both pooling paths
    coords = [torch.rand(5, 3), torch.rand(7, 3)]
    feats = [torch.rand(5, 4), torch.rand(7, 4)]
    pc = Points(coords, feats)
    assert len(pc) == 12 and pc.batch_size == 2 and pc.offsets.tolist() == [0, 5, 12] and pc.num_channels == 4
    assert Points(torch.cat(coords), torch.cat(feats), offsets=torch.tensor([0, 5, 12])).equal_shape(pc)
    with pytest.raises(AssertionError):
        Points(torch.rand(5, 2), torch.rand(5, 4), offsets=torch.tensor([0, 5]))  # not 3-D
    with pytest.raises(AssertionError):
        Points(coords, feats[:1])
    with pytest.raises(AssertionError):
        point_pool(pc, "mean")  # neither a voxel size nor a point count
    with pytest.raises(AssertionError):
        point_pool(pc, "mean", downsample_voxel_size=0.1, return_type="grid")
    with pytest.raises(AssertionError):
        point_pool(pc, "mean", downsample_voxel_size=0.1, return_type="voxel", avereage_pooled_coordinates=True)
    with pytest.raises(NotImplementedError):
        point_pool(pc, "mean", downsample_max_num_points=4)
    with pytest.raises(AssertionError):
        point_pool(pc, "random", downsample_voxel_size=0.1, return_to_unique=True)
    with pytest.raises((ValueError, RuntimeError)):
        point_pool(pc, "mean", downsample_voxel_size=0.1)  # CPU tensors: the library path refuses them
    with pytest.raises(NotImplementedError):
        ToUnique(unique_method="encode")
    assert ToUnique(unique_method="morton").unique_method == "morton"  # the point modules' default
    with pytest.raises(AssertionError):
        row_reduction(torch.rand(5, 2), torch.tensor([0, 2, 4]), "sum")  # splits do not cover the rows
    with pytest.raises(ValueError):
        REDUCTIONS("median")
    # the inverse is derived from the grouping on first access
    info = UniqueInfo(None, torch.tensor([2, 0, 3, 1, 4]), torch.tensor([0, 2, 3, 5]), None)
    assert info.to_orig_indices.tolist() == [0, 2, 0, 1, 2]
    assert info.to_orig_indices is info.to_orig_indices


def test_take_rows_in_pieces_equals_plain_indexing(monkeypatch):
    from warpconvnet_amd.utils import gather
    g = torch.Generator().manual_seed(0)
    src = torch.randn(50, 4, generator=g, requires_grad=True)
    index = torch.randint(0, 50, (1000,), generator=g)
    whole = gather.take_rows(src, index)
    monkeypatch.setattr(gather, "_PIECE", 64)
    pieces = gather.take_rows(src, index)
    assert torch.equal(pieces, src[index]) and torch.equal(pieces, whole)
    pieces.sum().backward()  # the gradient counts how often every row was picked
    assert torch.equal(src.grad[:, 0], torch.bincount(index, minlength=50).float())
    mask = torch.arange(50) % 2 == 0
    assert torch.equal(gather.take_rows(src, mask), src[mask])
    assert torch.equal(gather.take_rows(src[:, 0], index), src[:, 0][index])
