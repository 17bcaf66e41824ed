"""GPU parity of the integer stages (table, kernel map, strided coordinates) against the CPU
oracle.  Bit-exact: indices and coordinates must be identical."""
import numpy as np
import pytest
import torch

from helpers import canonical_pairs, sort_rows
from warpconvnet_amd.utils import synthetic

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.int32, device=DEV)


def test_table_finds_every_key_and_rejects_absent_keys(oracle):
    """Invariant of the reference's own test (tests/coords/test_torch_hashmap.py:35-69)."""
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import HashMethod, TorchHashTable
    rng = np.random.default_rng(0)
    keys = np.unique(rng.integers(-1000, 1000, size=(65536, 4)).astype(np.int32), axis=0)
    rng.shuffle(keys)
    for method in HashMethod:
        table = TorchHashTable.from_keys(_dev(keys), hash_method=method, device=DEV)
        got = table.search(_dev(keys)).cpu().numpy()
        assert np.array_equal(got, np.arange(len(keys), dtype=np.int32))
        absent = keys + np.array([0, 5000, 0, 0], dtype=np.int32)
        assert (table.search(_dev(absent)).cpu().numpy() == -1).all()
    # mixed queries against the oracle's restatement of the reference table
    q = np.concatenate([keys[:1000], absent[:1000], keys[-7:] + np.array([0, 0, 0, 1], np.int32)])
    ref = oracle.HashTable(keys).search(q)
    assert np.array_equal(table.search(_dev(q)).cpu().numpy(), ref)


def test_table_duplicates_lowest_row_wins():
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import TorchHashTable
    rng = np.random.default_rng(1)
    base = rng.integers(0, 50, size=(5000, 4)).astype(np.int32)  # many duplicates
    table = TorchHashTable.from_keys(_dev(base), device=DEV)
    got = table.search(_dev(base)).cpu().numpy()
    first = {}
    for i, r in enumerate(map(tuple, base.tolist())):
        first.setdefault(r, i)
    want = np.array([first[tuple(r)] for r in base.tolist()], dtype=np.int32)
    assert np.array_equal(got, want)
    assert np.array_equal(table.unique_index.cpu().numpy(), np.unique(want))


def test_table_sparse_keys_force_a_rebuild():
    """Isolated voxels put one key in every block: the default slot count overflows on the
    device and the host retries with more slots; results stay exact."""
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import TorchHashTable
    rng = np.random.default_rng(2)
    keys = np.unique(rng.integers(0, 1 << 20, size=(200000, 4)).astype(np.int32), axis=0)
    keys[:, 0] %= 8
    keys = np.unique(keys, axis=0)
    table = TorchHashTable.from_keys(_dev(keys), device=DEV)
    got = table.search(_dev(keys)).cpu().numpy()
    assert np.array_equal(got, np.arange(len(keys), dtype=np.int32))


def test_table_extreme_coordinates_report_range_error():
    from warpconvnet_amd._lib import WcnError
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import TorchHashTable
    keys = np.array([[0, -2**31, -2**31, -2**31], [2**31 - 1, 2**31 - 1, 2**31 - 1, 2**31 - 1]],
                    dtype=np.int32)
    with pytest.raises(WcnError):
        TorchHashTable.from_keys(_dev(keys), device=DEV)
    # a wide but packable range works, negative coordinates included
    keys = np.array([[0, -2**20, 5, 7], [3, 2**20, -9, 2**15], [1, 0, 0, 0]], dtype=np.int32)
    table = TorchHashTable.from_keys(_dev(keys), device=DEV)
    assert table.search(_dev(keys)).cpu().tolist() == [0, 1, 2]


CASES = [
    # name, coords generator, kernel, stride
    ("cloud_k3", lambda: synthetic.random_cloud(0, 20000, 40, batch_size=3), (3, 3, 3), (1, 1, 1)),
    ("cloud_k2s2", lambda: synthetic.random_cloud(1, 20000, 40, batch_size=2), (2, 2, 2), (2, 2, 2)),
    ("cloud_k3s2", lambda: synthetic.random_cloud(2, 20000, 40, batch_size=2), (3, 3, 3), (2, 2, 2)),
    ("cloud_k5", lambda: synthetic.random_cloud(3, 5000, 24, batch_size=1), (5, 5, 5), (1, 1, 1)),
    ("cloud_k323", lambda: synthetic.random_cloud(4, 5000, 24, batch_size=2), (3, 2, 3), (1, 2, 1)),
    ("spheres_k3", lambda: synthetic.batch_indexed([synthetic.spheres_scene(0, 100_000)]),
     (3, 3, 3), (1, 1, 1)),
    ("indoor_k3", lambda: synthetic.batch_indexed(synthetic.indoor_batch(2, 60_000)[0]),
     (3, 3, 3), (1, 1, 1)),
]


@pytest.mark.parametrize("name,gen,ksize,stride", CASES, ids=[c[0] for c in CASES])
def test_kernel_map_bit_exact(oracle, name, gen, ksize, stride):
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    in_coords = gen()
    batches = int(in_coords[:, 0].max()) + 1
    if any(s != 1 for s in stride):
        out_dev, off_dev = stride_coords(_dev(in_coords), stride)
        out_coords = out_dev.cpu().numpy()
        # strided coordinates: same set as the oracle, same batch offsets
        ref_out, _, ref_off = oracle.stride_coords(in_coords, stride, batches)
        assert np.array_equal(sort_rows(out_coords), sort_rows(ref_out))
        assert np.array_equal(off_dev.numpy().astype(np.int64), ref_off)
        # and in this implementation's documented order: ascending first source row
        assert np.array_equal(out_coords, ref_out)
    else:
        out_coords = in_coords
    km = generate_kernel_map(_dev(in_coords), _dev(out_coords), stride, ksize)
    ref_in, ref_out_map, ref_off, ref_iden = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    assert km.identity_map_index == ref_iden
    assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
    # native order equals the reference's (ascending output row inside every offset) ...
    assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), ref_out_map)
    # ... and therefore also after the canonical sort
    assert np.array_equal(canonical_pairs(km.in_maps.cpu(), km.out_maps.cpu(), km.offsets),
                          canonical_pairs(ref_in, ref_out_map, ref_off))


BLOCK_CASES = [c for c in CASES if all(s == 1 for s in c[3]) and c[2] in ((3, 3, 3), (5, 5, 5))]


@pytest.mark.parametrize("name,gen,ksize,stride", BLOCK_CASES, ids=[c[0] for c in BLOCK_CASES])
def test_kernel_map_probed_block_by_block_bit_exact(oracle, monkeypatch, name, gen, ksize, stride):
    """The other probe pass for a coordinate set mapped onto itself (WCN_KMAP_PROBE=blocks: hit masks
    of whole 4x4x4 blocks from ANDs of shifted occupancy masks): the same map, bit for bit in native
    order, with its group starts; also with repeated input rows (against the row-order probe: among
    repeated keys the reference's winner is a race, here the lowest row) and with 27 pairs per voxel
    (more than the emit pass assumes)."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    coords = gen()
    variants = [(coords, True)]
    if name == "cloud_k3":
        rng = np.random.default_rng(5)
        variants.append((np.concatenate([coords, coords[rng.integers(0, len(coords), 3000)]]), False))
        cube = np.stack(np.meshgrid(*[np.arange(14)] * 3, indexing="ij"), axis=-1).reshape(-1, 3)
        variants.append((synthetic.batch_indexed([cube.astype(np.int32) - 5]), True))
    for c, unique in variants:
        monkeypatch.setenv("WCN_KMAP_PROBE", "blocks")
        same = _dev(c)
        km = generate_kernel_map(same, same, stride, ksize)
        if unique:
            ref_in, ref_out_map, ref_off, ref_iden = oracle.kernel_map(c, c, ksize, stride)
        else:
            monkeypatch.setenv("WCN_KMAP_PROBE", "rows")
            other = _dev(c)
            by_rows = generate_kernel_map(other, other, stride, ksize)
            ref_in, ref_out_map = by_rows.in_maps.cpu().numpy(), by_rows.out_maps.cpu().numpy()
            ref_off, ref_iden = by_rows.offsets.numpy().astype(np.int64), by_rows.identity_map_index
        assert km.identity_map_index == ref_iden
        assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
        assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
        assert np.array_equal(km.out_maps.cpu().numpy(), ref_out_map)
        groups, _, (K, M) = km._group_start
        gs = groups.view(torch.int32).cpu().numpy().reshape(K, -1)
        bounds = np.arange(0, 64 * (gs.shape[1] - 1), 64)
        want = np.stack([np.searchsorted(ref_out_map[ref_off[k]:ref_off[k + 1]], bounds) for k in range(K)])
        assert np.array_equal(gs[:, :-1], want)
        assert np.array_equal(gs[:, -1], np.diff(ref_off))


DILATED = [
    ("k3_d2", (3, 3, 3), (1, 1, 1), (2, 2, 2), None),
    ("k3_d123", (3, 3, 3), (1, 1, 1), (1, 2, 3), None),
    ("k2s2_d212", (2, 2, 2), (2, 2, 2), (2, 1, 2), None),
    ("k3_centre", (3, 3, 3), (1, 1, 1), (1, 1, 1), (0, 2, 1)),
    ("k323_d231_centre", (3, 2, 3), (1, 1, 1), (2, 3, 1), (1, 1, 0)),
    ("k5_d2", (5, 5, 5), (1, 1, 1), (2, 2, 2), None),
]


@pytest.mark.parametrize("name,ksize,stride,dilation,centre", DILATED, ids=[c[0] for c in DILATED])
def test_dilated_kernel_map_bit_exact(oracle, name, ksize, stride, dilation, centre):
    """method="offset": dilated and re-centred kernels, bit-exact in native order against the oracle's
    offset-table probe (itself pinned by a dictionary brute force)."""
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    in_coords = synthetic.random_cloud(31, 20000, 40, batch_size=2)
    if any(s != 1 for s in stride):
        out_coords = stride_coords(_dev(in_coords), stride)[0].cpu().numpy()
    else:
        out_coords = in_coords
    km = generate_kernel_map(_dev(in_coords), _dev(out_coords), stride, ksize, kernel_dilation=dilation,
                             kernel_center_offset=centre, method="offset")
    ref_in, ref_out, ref_off, ref_iden = oracle.kernel_map(in_coords, out_coords, ksize, stride,
                                                           dilation=dilation, center_offset=centre)
    assert int(ref_off[-1]) > 0
    assert np.array_equal(km.offsets.numpy().astype(np.int64), ref_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), ref_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), ref_out)
    assert km.identity_map_index == (None if centre is not None else ref_iden)


def test_ordered_stride_coords():
    """stride_coords with a Morton ordering: the same set of coarse voxels, batch items contiguous,
    Morton codes ascending inside every batch item."""
    from warpconvnet_amd.geometry.coords.ops.serialization import POINT_ORDERING, morton_code
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    in_coords = synthetic.random_cloud(33, 30000, 48, batch_size=3)
    plain, plain_off = stride_coords(_dev(in_coords), (2, 2, 2))
    ordered, off = stride_coords(_dev(in_coords), (2, 2, 2), order=POINT_ORDERING.MORTON_XYZ)
    assert torch.equal(off, plain_off)
    assert np.array_equal(sort_rows(ordered.cpu().numpy()), sort_rows(plain.cpu().numpy()))
    assert bool((torch.diff(ordered[:, 0]) >= 0).all())
    codes = morton_code(ordered[:, 1:].contiguous(), order=POINT_ORDERING.MORTON_XYZ)
    for b in range(3):
        seg = codes[int(off[b]):int(off[b + 1])]
        assert bool((torch.diff(seg) >= 0).all())


def test_batch_offsets_of_an_ascending_column_by_search():
    """The search for the bounds of an ascending batch column gives what counting gives, with batch
    items that have no rows in the middle, and falls back to counting beyond its limit of items."""
    from warpconvnet_amd.geometry.coords.ops import batch_index as bi
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    col = torch.tensor([0, 0, 1, 1, 1, 4, 4, 7], dtype=torch.int32, device=DEV)
    counted = bi.offsets_from_batch_index(col)
    assert counted.tolist() == [0, 2, 5, 5, 5, 7, 7, 7, 8]
    assert bi.offsets_from_batch_index(col, ascending=True).tolist() == counted.tolist()
    many = torch.arange(0, 3000, dtype=torch.int32, device=DEV).repeat_interleave(2)  # more items than searched for
    assert bi.offsets_from_batch_index(many, ascending=True).tolist() == bi.offsets_from_batch_index(many).tolist()
    in_coords = synthetic.random_cloud(34, 20000, 40, batch_size=4)
    a, a_off = stride_coords(_dev(in_coords), (2, 2, 2))
    b, b_off = stride_coords(_dev(in_coords), (2, 2, 2), batch_sorted=True)
    assert torch.equal(a, b) and a_off.tolist() == b_off.tolist()
    # batch items without rows in the middle: the bounds the library hands over with the row count
    gaps = in_coords.copy()
    gaps[:, 0] = np.array([0, 2, 5, 6])[gaps[:, 0]]
    a, a_off = stride_coords(_dev(gaps), (2, 2, 2))
    b, b_off = stride_coords(_dev(gaps), (2, 2, 2), batch_sorted=True)
    assert torch.equal(a, b) and a_off.tolist() == b_off.tolist() and len(b_off) == 8
    assert b_off[2] == b_off[1] and b_off[-1] == len(b)


def test_kernel_map_invariants_full_size():
    """Size-independent properties at the benchmark's size (4 x 250k voxels, 3x3x3):
    identity row, offset symmetry, duplicate-free rows."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    items, _ = synthetic.indoor_batch(4, 250_000)
    coords = _dev(synthetic.batch_indexed(items))
    n = coords.shape[0]
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    assert km.identity_map_index == 13
    i13, o13 = km[13]
    ar = torch.arange(n, dtype=torch.int32, device=DEV)
    assert torch.equal(i13, ar) and torch.equal(o13, ar)
    counts = torch.diff(km.offsets)
    assert torch.equal(counts, counts.flip(0))  # |map_k| == |map_{K-1-k}|
    for k in (0, 5, 12):
        a_in, a_out = km[k]
        b_in, b_out = km[26 - k]
        assert (torch.diff(a_out) > 0).all()
        # (i, j) in map_k  <=>  (j, i) in map_{K-1-k}
        order = torch.argsort(b_in)
        assert torch.equal(b_in[order], a_out) and torch.equal(b_out[order], a_in)


def test_kernel_map_stride2_every_fine_voxel_once():
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    items, _ = synthetic.indoor_batch(2, 100_000)
    fine = _dev(synthetic.batch_indexed(items))
    coarse, offsets = stride_coords(fine, (2, 2, 2))
    assert int(offsets[-1]) == coarse.shape[0] < fine.shape[0]
    km = generate_kernel_map(fine, coarse, (2, 2, 2), (2, 2, 2))
    assert km.identity_map_index is None
    assert int(km.offsets[-1]) == fine.shape[0]
    assert torch.equal(torch.sort(km.in_maps).values,
                       torch.arange(fine.shape[0], dtype=torch.int32, device=DEV))


def test_kernel_map_skip_symmetric_prefix():
    """reference: tests/nn/test_sparse_conv.py:137-181."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    coords = _dev(synthetic.random_cloud(5, 10000, 30, batch_size=2))
    full = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3), kernel_dilation=(1, 1, 1))
    skip = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3), kernel_dilation=(1, 1, 1),
                               skip_symmetric_kernel_map=True)
    assert skip.identity_map_index == 13
    n = len(skip.offsets)
    assert torch.equal(full.offsets[:n], skip.offsets)
    assert torch.equal(full.in_maps[: int(full.offsets[n - 1])], skip.in_maps)
    assert torch.equal(full.out_maps[: int(full.offsets[n - 1])], skip.out_maps)


def test_empty_and_tiny_inputs():
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    one = _dev(np.array([[0, 3, 4, 5]], dtype=np.int32))
    km = generate_kernel_map(one, one, (1, 1, 1), (3, 3, 3))
    assert km.offsets.tolist() == [0] * 14 + [1] * 14
    assert km.in_maps.tolist() == [0] and km.out_maps.tolist() == [0]
    none = torch.empty((0, 4), dtype=torch.int32, device=DEV)
    km = generate_kernel_map(one, none, (1, 1, 1), (3, 3, 3))
    assert int(km.offsets[-1]) == 0 and len(km) == 27


def test_golden_fixtures_on_gpu():
    """Committed fixtures: strided coordinates, kernel map (bit-exact), fp32 features and gradients."""
    import glob
    import os
    from helpers import rel_err
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward, sparse_conv_forward
    paths = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))
    assert len(paths) >= 4
    for path in paths:
        g = np.load(path)
        ksize, stride = tuple(int(v) for v in g["kernel_size"]), tuple(int(v) for v in g["stride"])
        in_dev = _dev(g["in_coords"])
        if any(s != 1 for s in stride):
            out_dev, offsets = stride_coords(in_dev, stride)
            assert np.array_equal(out_dev.cpu().numpy(), g["out_coords"])
            assert np.array_equal(offsets.numpy().astype(np.int64), g["out_offsets"])
        else:
            out_dev = in_dev
        km = generate_kernel_map(in_dev, out_dev, stride, ksize)
        assert np.array_equal(km.in_maps.cpu().numpy(), g["in_maps"]), path
        assert np.array_equal(km.out_maps.cpu().numpy(), g["out_maps"]), path
        assert np.array_equal(km.offsets.numpy().astype(np.int64), g["offsets"]), path
        assert (-1 if km.identity_map_index is None else km.identity_map_index) == int(g["identity"])
        out = sparse_conv_forward(torch.as_tensor(g["features"], device=DEV),
                                  torch.as_tensor(g["weight"], device=DEV), km, len(g["out_coords"]))
        assert rel_err(out.cpu().numpy(), g["out_features_f64"]) <= 1e-5, path
        gx, gw = sparse_conv_backward(torch.as_tensor(g["grad_out"], device=DEV),
                                      torch.as_tensor(g["features"], device=DEV),
                                      torch.as_tensor(g["weight"], device=DEV), km)
        assert rel_err(gx.cpu().numpy(), g["grad_features_f64"]) <= 1e-5, path
        assert rel_err(gw.cpu().numpy(), g["grad_weight_f64"]) <= 1e-5, path


def test_maps_over_one_tensor_share_its_table(oracle):
    """The coordinate table is kept on the input tensor object: a second map over the same rows
    reuses it, an in-place change of the rows rebuilds it, and the maps are the oracle's either way."""
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    bc = synthetic.random_cloud(90, 5000, 24, batch_size=2)
    c = torch.as_tensor(bc, device=DEV)
    km3 = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    table = c._wcn_table[1]
    coarse, _ = stride_coords(c, (2, 2, 2))
    km2 = generate_kernel_map(c, coarse, (2, 2, 2), (2, 2, 2))
    assert c._wcn_table[1] is table
    for km, out, ks, st in ((km3, bc, (3, 3, 3), (1, 1, 1)), (km2, coarse.cpu().numpy(), (2, 2, 2), (2, 2, 2))):
        im, om, off, _ = oracle.kernel_map(bc, out, ks, st)
        assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
        assert np.array_equal(km.offsets.numpy(), off)
    c[:, 1] += 3  # in place: the kept table no longer describes the rows
    km3b = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
    assert c._wcn_table[1] is not table
    assert torch.equal(km3b.in_maps, km3.in_maps) and torch.equal(km3b.offsets, km3.offsets)  # a pure shift
    q = torch.as_tensor(bc[:50], device=DEV)
    q[:, 1] += 3
    assert torch.equal(c._wcn_table[1].search(q).cpu(), torch.arange(50, dtype=torch.int32))


def _morton_numpy(xyz, axes):
    """Bit-by-bit restatement: bit i of the axis in position p goes to bit 3 i + p."""
    rel = (xyz - xyz.min(0)).astype(np.uint64)
    code = np.zeros(len(xyz), dtype=np.uint64)
    for pos, axis in enumerate(axes):
        for bit in range(21):
            code |= ((rel[:, axis] >> np.uint64(bit)) & np.uint64(1)) << np.uint64(3 * bit + pos)
    return code.astype(np.int64)


def test_morton_codes_and_sort():
    """encode / morton_code / Voxels.sort (reference: serialization.py:85-254, voxels.py:246-267):
    codes against a bit-by-bit restatement for every axis order, the permutation sorts by code
    inside every batch item, the inverse restores the order, features travel with their voxels."""
    from warpconvnet_amd.geometry.coords.ops.serialization import (POINT_ORDERING,
                                                                   POINT_ORDERING_TO_MORTON_PERMUTATIONS,
                                                                   encode, morton_code)
    from warpconvnet_amd.geometry.types.voxels import Voxels
    rng = np.random.default_rng(3)
    xyz = np.unique(rng.integers(-3000, 900_000, size=(20_000, 3)), axis=0).astype(np.int32)
    rng.shuffle(xyz)
    dev = torch.as_tensor(xyz, device=DEV)
    for order, axes in POINT_ORDERING_TO_MORTON_PERMUTATIONS.items():
        assert np.array_equal(morton_code(dev, order=order).cpu().numpy(), _morton_numpy(xyz, axes)), order
    n = len(xyz)
    offsets = torch.tensor([0, n // 4, n // 2, n])
    res = encode(dev, batch_offsets=offsets, order="morton_xyz", return_perm=True, return_inverse=True)
    codes, perm = res.codes.cpu().numpy(), res.perm.cpu().numpy()
    assert np.array_equal(np.sort(perm), np.arange(n))
    for lo, hi in zip(offsets[:-1].tolist(), offsets[1:].tolist()):
        seg = perm[lo:hi]
        assert seg.min() >= lo and seg.max() < hi              # rows stay in their batch item
        assert (np.diff(codes[seg]) > 0).all()                 # ascending (codes of distinct voxels differ)
    assert np.array_equal(perm[res.inverse_perm.cpu().numpy()], np.arange(n))
    feats = torch.arange(n, dtype=torch.float32, device=DEV).unsqueeze(1)
    vox = Voxels(dev, feats, offsets=offsets)
    s = vox.sort(POINT_ORDERING.MORTON_XYZ)
    assert s.ordering == POINT_ORDERING.MORTON_XYZ and s.sort(POINT_ORDERING.MORTON_XYZ) is s
    assert torch.equal(s.coordinate_tensor, dev[res.perm]) and torch.equal(s.feature_tensor[:, 0].long(), res.perm)
    assert encode(torch.empty(0, 3, dtype=torch.int32), return_perm=True).perm.numel() == 0


def test_kernel_map_with_more_pairs_than_assumed(oracle):
    """A dense cube has ~27 pairs per voxel, more than the buffers the emit pass is first enqueued
    into hold: that pass must leave them untouched and the second, exact one produce the map."""
    from warpconvnet_amd.geometry.coords.search import torch_discrete
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    S = 24
    g = np.stack(np.meshgrid(np.arange(S), np.arange(S), np.arange(S), indexing="ij"), -1).reshape(-1, 3)
    rng = np.random.default_rng(0)
    rng.shuffle(g)
    bc = np.concatenate([np.zeros((len(g), 1), np.int32), g.astype(np.int32)], axis=1)
    im, om, off, iden = oracle.kernel_map(bc, bc, (3, 3, 3))
    torch_discrete._PAIRS_PER_ROW.clear()  # nothing remembered: eight pairs per row are assumed
    for attempt in range(2):               # the second build sizes its buffers by what the first one held
        km = generate_kernel_map(_dev(bc), _dev(bc), (1, 1, 1), (3, 3, 3))
        assert int(km.offsets[-1]) == len(im) > 8 * len(bc)
        assert np.array_equal(km.in_maps.cpu().numpy(), im) and np.array_equal(km.out_maps.cpu().numpy(), om)
        assert np.array_equal(km.offsets.numpy().astype(np.int64), off)
    assert max(torch_discrete._PAIRS_PER_ROW.values()) > 8


def _brute_force_map(in_rows, out_rows, stride, ksize, dilation=None):
    """Kernel map over any number of columns by dictionary look-up: offsets enumerated with the last
    dimension fastest, pairs of an offset in ascending output row (what the reference's offset probe
    over all columns yields, discrete_kernels.cu:129-180)."""
    import itertools
    D = len(ksize)
    dilation = dilation or [1] * D
    where = {tuple(r): i for i, r in enumerate(in_rows.tolist())}
    centres = [(k - 1) // 2 if k % 2 == 1 else 0 for k in ksize]
    ins, outs, offsets = [], [], [0]
    for idx in itertools.product(*[range(k) for k in ksize]):
        off = [(i - c) * d for i, c, d in zip(idx, centres, dilation)]
        for m, r in enumerate(out_rows.tolist()):
            q = (r[0],) + tuple(r[1 + d] * stride[d] + off[d] for d in range(D))
            hit = where.get(q)
            if hit is not None:
                ins.append(hit)
                outs.append(m)
        offsets.append(len(ins))
    return np.array(ins, np.int32), np.array(outs, np.int32), np.array(offsets, np.int64)


MORE_DIMS = [
    # name, columns past the batch, rows, extent, kernel, stride, dilation
    ("4d_k3", 4, 3000, 9, (3, 3, 3, 3), (1, 1, 1, 1), None),
    ("4d_k2s2", 4, 3000, 10, (2, 2, 2, 2), (2, 2, 2, 2), None),
    ("4d_mixed_dilated", 4, 2000, 12, (3, 1, 2, 3), (1, 1, 1, 1), (1, 1, 2, 2)),
    ("5d", 5, 2500, 6, (3, 3, 1, 2, 3), (1, 1, 1, 1, 1), None),
]


@pytest.mark.parametrize("name,D,n,extent,ksize,stride,dilation", MORE_DIMS, ids=[c[0] for c in MORE_DIMS])
def test_kernel_map_over_more_than_three_dimensions(name, D, n, extent, ksize, stride, dilation):
    """Four and five spatial dimensions (folded into the batch column for the device kernels) against
    a dictionary look-up over all columns: same pairs, same order, negative coordinates included."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    rng = np.random.default_rng(len(name))
    rows = rng.integers(-extent // 2, extent // 2 + 1, size=(n, D + 1)).astype(np.int32)
    rows[:, 0] = rng.integers(0, 3, size=n)
    rows = np.unique(rows, axis=0)
    rng.shuffle(rows)
    if any(s != 1 for s in stride):
        coarse = rows.copy()
        coarse[:, 1:] = np.floor_divide(rows[:, 1:], np.array(stride, dtype=np.int32))
        out_rows = np.unique(coarse, axis=0)
    else:
        out_rows = rows
    km = generate_kernel_map(_dev(rows), _dev(out_rows), stride, ksize, kernel_dilation=dilation,
                             method="offset" if dilation else "size")
    want_in, want_out, want_off = _brute_force_map(rows, out_rows, stride, ksize, dilation)
    assert np.array_equal(km.offsets.numpy().astype(np.int64), want_off)
    assert np.array_equal(km.in_maps.cpu().numpy(), want_in)
    assert np.array_equal(km.out_maps.cpu().numpy(), want_out)
    all_odd = all(k % 2 == 1 for k in ksize)
    assert km.identity_map_index == (int(np.prod(ksize)) // 2 if all_odd and len(rows) == len(out_rows) else None)
    if km.identity_map_index is not None:
        i, o = km[km.identity_map_index]
        assert torch.equal(i, o) and len(i) == len(rows)


@pytest.mark.parametrize("stride", [(2, 2, 2), (4, 4, 4), (4, 2, 1), (1, 1, 2), (3, 2, 2)],
                         ids=["s2", "s4", "s421", "s112", "s322_other_path"])
def test_strided_coordinates_with_negative_coordinates_and_repeated_rows(oracle, stride):
    """Strides of 1, 2, 4 take the distinct coarse rows out of the table of the fine rows (cells inside
    4x4x4 blocks); any other stride builds a table over the coarse rows.  Both against the oracle, in
    this implementation's order (ascending first source row), with coordinates on both sides of zero
    and with fine rows that repeat."""
    from warpconvnet_amd.geometry.coords.ops.stride import stride_coords
    rng = np.random.default_rng(sum(stride))
    rows = rng.integers(-37, 41, size=(30000, 4)).astype(np.int32)
    rows[:, 0] = np.sort(rng.integers(0, 3, size=len(rows)))
    rows = np.concatenate([rows, rows[rng.integers(0, len(rows), 2000)]])  # repeats, batch column no longer sorted
    for batch_sorted in (False, True):
        use = rows[np.argsort(rows[:, 0], kind="stable")] if batch_sorted else rows
        got, got_off = stride_coords(_dev(use), stride, batch_sorted=batch_sorted)
        ref_out, _, ref_off = oracle.stride_coords(use, stride, 3)
        if batch_sorted:  # same rows in the same order, same offsets
            assert np.array_equal(got.cpu().numpy(), ref_out), stride
            assert np.array_equal(got_off.numpy().astype(np.int64), ref_off)
        else:             # the oracle orders by batch item afterwards, as the reference does
            assert np.array_equal(sort_rows(got.cpu().numpy()), sort_rows(ref_out)), stride
            assert np.array_equal(got_off.numpy().astype(np.int64), ref_off)


@pytest.mark.parametrize("dims", [1, 2, 3, 4])
@pytest.mark.parametrize("counts", [(5,), (3, 0, 4, 0), (0, 0, 7), tuple(range(64)), tuple([2] * 65)],
                         ids=["one_item", "empty_items", "leading_empty", "64_items", "65_items"])
def test_batch_indexed_coordinates_against_the_formula(dims, counts):
    """[batch item, coordinates] rows against the reference's formula, the batch column expanded
    from the offsets with repeat_interleave (batch_index.py:22-36, 110-117); 65 batch items are
    beyond what travels with the library's launch and take the torch path."""
    from warpconvnet_amd.geometry.coords.ops.batch_index import batch_indexed_coordinates
    g = torch.Generator().manual_seed(len(counts) * 10 + dims)
    n = sum(counts)
    coords = torch.randint(-50, 50, (n, dims), generator=g, dtype=torch.int32)
    offsets = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int64)
    got = batch_indexed_coordinates(coords.cuda(), offsets)
    batch = torch.arange(len(counts)).repeat_interleave(torch.tensor(counts))
    want = torch.cat([batch.to(torch.int32).unsqueeze(1), coords], dim=1)
    assert got.dtype == torch.int32 and got.shape == want.shape
    assert torch.equal(got.cpu(), want)


def test_steps_from_several_host_threads_on_their_own_streams():
    """The library's state between its calls (the mailbox the pair counts arrive in, the pending
    result, the table flags) is per thread: four threads, each on a stream of its own, build maps of
    different scenes and run the contraction over them at the same time, and every thread gets what
    the main thread got for its scene, bit for bit."""
    import threading
    from helpers import kaiming_weight
    from warpconvnet_amd._lib import lib
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    w = kaiming_weight(27, 64, 64, seed=3, dtype=torch.float16).to(DEV)
    scenes = []
    for t in range(4):
        bc = synthetic.batch_indexed([synthetic.indoor_scene(40 + t, 60_000 + 7_000 * t, 0.02)])
        c = torch.as_tensor(bc, device=DEV)
        x = torch.randn(len(bc), 64, generator=torch.Generator().manual_seed(t)).half().to(DEV)
        km = generate_kernel_map(c, c, (1, 1, 1), (3, 3, 3))
        scenes.append((c, x, km.in_maps.clone(), km.out_maps.clone(), km.offsets.clone(),
                       sparse_conv_forward(x, w, km, len(bc))))
    torch.cuda.synchronize()
    failures = []

    def work(t):
        c, x, want_in, want_out, want_offsets, want = scenes[t]
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for _ in range(15):
                    cold = c.view(-1, 4)  # a new tensor object: table and map are built again
                    km = generate_kernel_map(cold, cold, (1, 1, 1), (3, 3, 3))
                    # the weight's tiles are made once, on the stream of whichever thread comes
                    # first, and the other threads' streams wait for them
                    out = sparse_conv_forward(x, w, km, c.shape[0], keep_prepared_weight=True)
                    if not (torch.equal(km.offsets, want_offsets) and torch.equal(km.in_maps, want_in)
                            and torch.equal(km.out_maps, want_out) and torch.equal(out, want)):
                        failures.append(t)
        except Exception as e:  # a thread's exception would otherwise be lost
            failures.append((t, repr(e)))
        torch.cuda.synchronize()
        lib().wcn_thread_release()  # the thread's pinned mailbox and events

    threads = [threading.Thread(target=work, args=(t,)) for t in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    assert failures == []
