"""Pins of the CPU oracle: every oracle function is checked here against something that does
not share its code - a library routine, a published known answer, a brute-force restatement with
Python dicts, or an invariant the mathematics fixes.  No GPU needed."""
import itertools

import numpy as np
import pytest
import torch

from helpers import canonical_pairs, sort_rows
from warpconvnet_amd.utils import synthetic


# ---- hash functions --------------------------------------------------------------------------

def test_murmur_matches_library_murmur3_32(oracle):
    """The reference's Murmur variant (seed 0x9747B28C, 4-byte blocks, length finaliser) is the
    standard MurmurHash3_x86_32 of the little-endian bytes: published vector and sklearn."""
    from sklearn.utils import murmurhash3_32
    assert oracle.hash32([0x74736574], oracle.HASH_MURMUR) == 0x704B81DC  # "test"
    rng = np.random.default_rng(0)
    for dim in (1, 2, 4, 7):
        for _ in range(20):
            key = rng.integers(-2**31, 2**31, size=dim).astype(np.int32)
            want = murmurhash3_32(key.astype("<i4").tobytes(), seed=0x9747B28C, positive=True)
            assert oracle.hash32(key, oracle.HASH_MURMUR) == want


def test_city_mix_is_fmix32_chain(oracle):
    """City variant: h <- fmix32(h + k * 0x9E3779B9).  fmix32(s) is what murmur3_32 returns for
    the empty string with seed s, so the chain is rebuilt from the library routine."""
    from sklearn.utils import murmurhash3_32
    assert oracle.hash32([0, 0, 0, 0], oracle.HASH_CITY) == 0
    rng = np.random.default_rng(1)
    for _ in range(50):
        key = rng.integers(-2**31, 2**31, size=4).astype(np.int32)
        h = 0
        for k in key.astype(np.int64):
            h = murmurhash3_32(b"", seed=int((h + (int(k) % 2**32) * 0x9E3779B9) % 2**32),
                               positive=True)
        assert oracle.hash32(key, oracle.HASH_CITY) == h


def test_fnv1a_published_vectors(oracle):
    """With every word below 256 the word-wise FNV-1a equals the byte-wise FNV-1a-32 whose
    published test vectors are used here."""
    assert oracle.hash32(list(b"a"), oracle.HASH_FNV1A) == 0xE40C292C
    assert oracle.hash32(list(b"foobar"), oracle.HASH_FNV1A) == 0xBF9CF968


def test_slot_is_nonnegative_signed_modulo(oracle):
    lib = oracle.lib()
    import ctypes
    rng = np.random.default_rng(2)
    for _ in range(200):
        key = rng.integers(-2**31, 2**31, size=4).astype(np.int32)
        cap = int(rng.integers(1, 100000))
        h = oracle.hash32(key, oracle.HASH_CITY)
        signed = h - 2**32 if h >= 2**31 else h
        got = lib.wcn_oracle_hash_slot(key.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), 4, cap, 1)
        assert got == signed % cap  # Python's % is the mathematical modulo


# ---- table -----------------------------------------------------------------------------------

@pytest.mark.parametrize("method", [0, 1, 2])
def test_table_search_invariants(oracle, method):
    """tests/coords/test_torch_hashmap.py:35-69 of the reference: all inserted keys are found at
    their own row, keys from a disjoint range are absent."""
    rng = np.random.default_rng(3)
    keys = np.unique(rng.integers(-500, 500, size=(20000, 4)).astype(np.int32), axis=0)
    rng.shuffle(keys)
    table = oracle.HashTable(keys, method=method)
    assert table.dropped == 0
    assert np.array_equal(table.search(keys), np.arange(len(keys), dtype=np.int32))
    assert (table.search(keys + np.array([0, 2000, 0, 0], np.int32)) == -1).all()
    lookup = {tuple(r): i for i, r in enumerate(keys.tolist())}
    q = rng.integers(-500, 500, size=(5000, 4)).astype(np.int32)
    want = np.array([lookup.get(tuple(r), -1) for r in q.tolist()], dtype=np.int32)
    assert np.array_equal(table.search(q), want)


# ---- kernel map ------------------------------------------------------------------------------

def brute_force_kernel_map(in_coords, out_coords, ksize, stride, dilation=(1, 1, 1), centre=None):
    """Independent restatement: a Python dict of coordinate tuples, offsets from itertools."""
    lookup = {}
    for i, r in enumerate(map(tuple, in_coords.tolist())):
        lookup.setdefault(r, i)
    if centre is None:
        centre = [s // 2 if s % 2 == 1 else 0 for s in ksize]
    ins, outs, offsets = [], [], [0]
    for i, j, k in itertools.product(range(ksize[0]), range(ksize[1]), range(ksize[2])):
        for m, (b, x, y, z) in enumerate(out_coords.tolist()):
            q = (b, x * stride[0] + (i - centre[0]) * dilation[0], y * stride[1] + (j - centre[1]) * dilation[1],
                 z * stride[2] + (k - centre[2]) * dilation[2])
            hit = lookup.get(q)
            if hit is not None:
                ins.append(hit)
                outs.append(m)
        offsets.append(len(ins))
    return np.array(ins, np.int32), np.array(outs, np.int32), np.array(offsets, np.int64)


KMAP_CASES = [((3, 3, 3), (1, 1, 1)), ((2, 2, 2), (2, 2, 2)), ((3, 3, 3), (2, 2, 2)),
              ((5, 5, 5), (1, 1, 1)), ((3, 2, 1), (1, 2, 1)), ((4, 4, 4), (1, 1, 1))]


@pytest.mark.parametrize("ksize,stride", KMAP_CASES)
def test_kernel_map_equals_brute_force(oracle, ksize, stride):
    in_coords = synthetic.random_cloud(7, 1500, 14, batch_size=2)
    if any(s != 1 for s in stride):
        out_coords = np.unique(np.concatenate(
            [in_coords[:, :1], np.floor_divide(in_coords[:, 1:], np.array(stride))], axis=1), axis=0)
    else:
        out_coords = in_coords
    got = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    want = brute_force_kernel_map(in_coords, out_coords, ksize, stride)
    for g, w in zip(got[:3], want):
        assert np.array_equal(g, w)
    odd = all(k % 2 == 1 for k in ksize)
    assert got[3] == (int(np.prod(ksize)) // 2 if odd and len(in_coords) == len(out_coords) else None)


DILATED_CASES = [((3, 3, 3), (1, 1, 1), (2, 2, 2), None), ((3, 3, 3), (1, 1, 1), (1, 2, 3), None),
                 ((2, 2, 2), (2, 2, 2), (2, 1, 2), None), ((3, 3, 3), (1, 1, 1), (1, 1, 1), (0, 2, 1)),
                 ((3, 2, 3), (1, 1, 1), (2, 3, 1), (1, 1, 0))]


@pytest.mark.parametrize("ksize,stride,dilation,centre", DILATED_CASES)
def test_dilated_kernel_map_equals_brute_force(oracle, ksize, stride, dilation, centre):
    """The offset-table probe (dilation, custom centre): every offset, scale and sign is fixed by the
    dictionary brute force; with dilation 1 and the default centre it is the size-based map."""
    in_coords = synthetic.random_cloud(9, 1500, 14, batch_size=2)
    if any(s != 1 for s in stride):
        out_coords = np.unique(np.concatenate(
            [in_coords[:, :1], np.floor_divide(in_coords[:, 1:], np.array(stride))], axis=1), axis=0)
    else:
        out_coords = in_coords
    got = oracle.kernel_map(in_coords, out_coords, ksize, stride, dilation=dilation, center_offset=centre)
    want = brute_force_kernel_map(in_coords, out_coords, ksize, stride, dilation, centre)
    for g, w in zip(got[:3], want):
        assert np.array_equal(g, w)
    assert int(want[2][-1]) > 0
    plain = oracle.kernel_map(in_coords, out_coords, ksize, stride)
    same = oracle.kernel_map(in_coords, out_coords, ksize, stride, dilation=(1, 1, 1))
    for g, w in zip(same[:3], plain[:3]):
        assert np.array_equal(g, w)


@pytest.mark.parametrize("method", [0, 1, 2])
def test_kernel_map_does_not_depend_on_hash(oracle, method):
    coords = synthetic.random_cloud(8, 3000, 18)
    a = oracle.kernel_map(coords, coords, (3, 3, 3), method=method)
    b = oracle.kernel_map(coords, coords, (3, 3, 3), method=1)
    for x, y in zip(a[:3], b[:3]):
        assert np.array_equal(x, y)


def test_kernel_map_invariants(oracle):
    coords = synthetic.batch_indexed([synthetic.spheres_scene(1, 20000)])
    im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
    n = len(coords)
    assert iden == 13
    assert np.array_equal(im[off[13]:off[14]], np.arange(n)) and np.array_equal(om[off[13]:off[14]], np.arange(n))
    counts = np.diff(off)
    assert np.array_equal(counts, counts[::-1])
    for k in range(13):
        a = np.stack([im[off[k]:off[k + 1]], om[off[k]:off[k + 1]]], 1)
        b = np.stack([om[off[26 - k]:off[27 - k]], im[off[26 - k]:off[27 - k]]], 1)
        assert np.array_equal(sort_rows(a), sort_rows(b))
        assert (np.diff(om[off[k]:off[k + 1]]) > 0).all()
        assert len(np.unique(im[off[k]:off[k + 1]])) == counts[k]


def test_kernel_map_dense_cube_closed_form(oracle):
    """A full S^3 cube in raster order: the neighbour of voxel (x,y,z) at offset (dx,dy,dz) is
    row ((x+dx)*S + y+dy)*S + z+dz when inside the cube."""
    S = 7
    g = np.stack(np.meshgrid(np.arange(S), np.arange(S), np.arange(S), indexing="ij"), -1).reshape(-1, 3)
    coords = np.concatenate([np.zeros((S**3, 1), np.int32), g.astype(np.int32)], 1)
    im, om, off, _ = oracle.kernel_map(coords, coords, (3, 3, 3))
    k = 0
    for dx, dy, dz in itertools.product((-1, 0, 1), repeat=3):
        nb = g + np.array([dx, dy, dz])
        ok = ((nb >= 0) & (nb < S)).all(1)
        rows = np.nonzero(ok)[0]
        want_in = (nb[ok, 0] * S + nb[ok, 1]) * S + nb[ok, 2]
        assert np.array_equal(om[off[k]:off[k + 1]], rows)
        assert np.array_equal(im[off[k]:off[k + 1]], want_in)
        k += 1


def test_stride2_kernel2_partitions_the_fine_voxels(oracle):
    fine = synthetic.random_cloud(9, 4000, 20, batch_size=2)
    coarse, first, offsets = oracle.stride_coords(fine, (2, 2, 2), 2)
    im, om, off, iden = oracle.kernel_map(fine, coarse, (2, 2, 2), (2, 2, 2))
    assert iden is None and off[-1] == len(fine)
    assert np.array_equal(np.sort(im), np.arange(len(fine)))
    # every pair links a fine voxel to the coarse voxel that contains it
    assert np.array_equal(np.floor_divide(fine[im][:, 1:], 2), coarse[om][:, 1:])


def test_kernel_offsets_table(oracle):
    """torch_discrete.py:44-77: last dimension fastest, centre (s-1)//2 odd / 0 even, dilation."""
    got = oracle.kernel_offsets((3, 2, 3), (1, 1, 2))
    want = [(0, i - 1, j, (k - 1) * 2) for i, j, k in itertools.product(range(3), range(2), range(3))]
    assert got.tolist() == [list(w) for w in want]


# ---- strided coordinates ---------------------------------------------------------------------

@pytest.mark.parametrize("stride", [(2, 2, 2), (2, 1, 4), (3, 3, 3)])
def test_stride_coords_equals_numpy_unique(oracle, stride):
    coords = synthetic.random_cloud(10, 5000, 40, batch_size=3)
    coords[:, 1:] -= 17  # negative coordinates exercise floor (not truncation)
    out, first, offsets = oracle.stride_coords(coords, stride, 3)
    disc = np.concatenate([coords[:, :1], np.floor_divide(coords[:, 1:], np.array(stride))], 1)
    uniq, first_idx = np.unique(disc, axis=0, return_index=True)
    assert np.array_equal(sort_rows(out), uniq)                    # same set as the library routine
    assert np.array_equal(np.sort(first), np.sort(first_idx))      # lowest row represents a voxel
    assert np.array_equal(out, disc[first])
    assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(np.bincount(out[:, 0], minlength=3))]))
    assert (np.diff(out[:, 0]) >= 0).all()


# ---- explicit gather-GEMM-scatter ------------------------------------------------------------

def test_conv_f64_dense_cube_equals_conv3d(oracle):
    S, c_in, c_out = 6, 5, 4
    g = torch.Generator().manual_seed(0)
    dense = torch.randn(1, c_in, S, S, S, generator=g, dtype=torch.float64)
    w = torch.randn(27, c_in, c_out, generator=g, dtype=torch.float64)
    grid = torch.stack(torch.meshgrid(torch.arange(S), torch.arange(S), torch.arange(S), indexing="ij"), -1)
    xyz = grid.reshape(-1, 3)[torch.randperm(S**3, generator=g)]
    coords = np.concatenate([np.zeros((S**3, 1), np.int32), xyz.numpy().astype(np.int32)], 1)
    feats = dense[0, :, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T.contiguous()
    im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
    got = oracle.explicit_conv_f64(feats.numpy(), w.numpy(), im, om, off, iden, len(coords))
    w5 = w.reshape(3, 3, 3, c_in, c_out).permute(4, 3, 0, 1, 2).contiguous()
    want = torch.nn.functional.conv3d(dense, w5, padding=1)[0][:, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T
    assert np.abs(got - want.numpy()).max() < 1e-12


def test_conv_f64_equals_pairwise_brute_force(oracle):
    rng = np.random.default_rng(5)
    coords = synthetic.random_cloud(11, 60, 6)
    n = len(coords)
    x = rng.normal(size=(n, 3))
    w = rng.normal(size=(27, 3, 2))
    im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
    want = np.zeros((n, 2))
    for k in range(27):
        for p in range(off[k], off[k + 1]):
            want[om[p]] += x[im[p]] @ w[k]
    assert np.abs(oracle.explicit_conv_f64(x, w, im, om, off, iden, n) - want).max() < 1e-12
    # without the identity shortcut the result is the same, because map row 13 is the identity
    assert np.abs(oracle.explicit_conv_f64(x, w, im, om, off, None, n) - want).max() < 1e-12


def test_torch_restatement_agrees_with_c_oracle(oracle):
    from oracle.explicit_conv import explicit_gemm_forward
    coords = synthetic.random_cloud(12, 3000, 18, batch_size=2)
    n = len(coords)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(n, 16, generator=g, dtype=torch.float64)
    w = torch.randn(27, 16, 24, generator=g, dtype=torch.float64)
    im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
    a = explicit_gemm_forward(x, w, torch.as_tensor(im), torch.as_tensor(om), off, iden, n).numpy()
    b = oracle.explicit_conv_f64(x.numpy(), w.numpy(), im, om, off, iden, n)
    assert np.abs(a - b).max() < 1e-11
    # low-precision run: rounded after every offset, still within the stated feature tolerance
    h = explicit_gemm_forward(x.to(torch.bfloat16), w.to(torch.bfloat16), torch.as_tensor(im),
                              torch.as_tensor(om), off, iden, n, compute_dtype=torch.float32)
    assert h.dtype == torch.bfloat16
    ref = oracle.explicit_conv_f64(x.to(torch.bfloat16).double().numpy(), w.to(torch.bfloat16).double().numpy(), im, om, off, iden, n)
    assert np.abs(h.double().numpy() - ref).max() / np.abs(ref).max() < 1e-2


@pytest.mark.parametrize("case", ["same_coords", "strided", "transposed"])
def test_backward_restatement_equals_autograd_of_the_forward(oracle, case):
    """The forward restatement is pinned above (dense-cube conv3d identity, pairwise brute force);
    torch differentiates it by itself, which pins the hand-written backward formulas (a dropped
    transpose, exchanged maps or a missed identity branch all fail here)."""
    from oracle.explicit_conv import explicit_gemm_backward, explicit_gemm_forward
    coords = synthetic.random_cloud(21, 700, 12, batch_size=2)
    if case == "same_coords":
        im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
        n_in = n_out = len(coords)
    else:
        coarse = oracle.stride_coords(coords, (2, 2, 2), 2)[0]
        im, om, off, iden = oracle.kernel_map(coords, coarse, (2, 2, 2), (2, 2, 2))
        n_in, n_out = len(coords), len(coarse)
        if case == "transposed":
            im, om, n_in, n_out = om, im, n_out, n_in
    K = len(off) - 1
    g = torch.Generator().manual_seed(3)
    x = torch.randn(n_in, 5, generator=g, dtype=torch.float64, requires_grad=True)
    w = torch.randn(K, 5, 7, generator=g, dtype=torch.float64, requires_grad=True)
    gy = torch.randn(n_out, 7, generator=g, dtype=torch.float64)
    im_t, om_t = torch.as_tensor(im), torch.as_tensor(om)
    out = explicit_gemm_forward(x, w, im_t, om_t, off, iden, n_out)
    want_x, want_w = torch.autograd.grad(out, (x, w), gy)
    got_x, got_w = explicit_gemm_backward(gy, x.detach(), w.detach(), im_t, om_t, off, iden)
    assert (got_x - want_x).abs().max() < 1e-10
    assert (got_w - want_w).abs().max() < 1e-10
    assert want_w.abs().max() > 0 and want_x.abs().max() > 0


# ---- pooling over a kernel map ----------------------------------------------------------------

def test_pool_dense_cube_equals_torch_pooling(oracle):
    """kernel = stride = 2 over a full 8^3 cube: the sparse pooling of the voxel list is
    max_pool3d / avg_pool3d of the dense tensor."""
    from oracle.pool import pool_over_map
    S, C = 8, 5
    g = torch.Generator().manual_seed(2)
    dense = torch.randn(1, C, S, S, S, generator=g, dtype=torch.float64)
    grid = torch.stack(torch.meshgrid(torch.arange(S), torch.arange(S), torch.arange(S), indexing="ij"), -1)
    xyz = grid.reshape(-1, 3)[torch.randperm(S**3, generator=g)]
    coords = np.concatenate([np.zeros((S**3, 1), np.int32), xyz.numpy().astype(np.int32)], 1)
    feats = dense[0, :, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T.contiguous()
    coarse = oracle.stride_coords(coords, (2, 2, 2), 1)[0]
    im, om, off, _ = oracle.kernel_map(coords, coarse, (2, 2, 2), (2, 2, 2))
    cx, cy, cz = coarse[:, 1], coarse[:, 2], coarse[:, 3]
    for name, fn in (("max", torch.nn.functional.max_pool3d), ("mean", torch.nn.functional.avg_pool3d)):
        got = pool_over_map(feats, torch.as_tensor(im), torch.as_tensor(om), len(coarse), name)
        want = fn(dense, 2)[0][:, cx, cy, cz].T
        assert (got - want).abs().max() < 1e-12, name


def test_pool_equals_row_by_row_brute_force(oracle):
    from oracle.pool import pool_over_map
    coords = synthetic.random_cloud(31, 400, 9, batch_size=2)
    coarse = oracle.stride_coords(coords, (2, 2, 2), 2)[0]
    im, om, off, _ = oracle.kernel_map(coords, coarse, (3, 3, 3), (2, 2, 2))  # overlapping windows
    x = torch.randn(len(coords), 3, generator=torch.Generator().manual_seed(4), dtype=torch.float64)
    rows = [[] for _ in range(len(coarse))]
    for i, m in zip(im, om):
        rows[m].append(int(i))
    assert any(len(r) > 4 for r in rows)
    ops = {"sum": lambda t: t.sum(0), "mean": lambda t: t.mean(0), "max": lambda t: t.max(0).values,
           "min": lambda t: t.min(0).values}
    for name, op in ops.items():
        want = torch.stack([op(x[r]) if r else torch.zeros(3, dtype=torch.float64) for r in rows])
        got = pool_over_map(x, torch.as_tensor(im), torch.as_tensor(om), len(coarse), name)
        assert (got - want).abs().max() < 1e-12, name


def test_depthwise_dense_cube_equals_grouped_conv3d(oracle):
    from oracle.explicit_conv import explicit_depthwise_forward
    S, C = 6, 5
    g = torch.Generator().manual_seed(8)
    dense = torch.randn(1, C, S, S, S, generator=g, dtype=torch.float64)
    w = torch.randn(27, C, generator=g, dtype=torch.float64)
    grid = torch.stack(torch.meshgrid(torch.arange(S), torch.arange(S), torch.arange(S), indexing="ij"), -1)
    xyz = grid.reshape(-1, 3)[torch.randperm(S**3, generator=g)]
    coords = np.concatenate([np.zeros((S**3, 1), np.int32), xyz.numpy().astype(np.int32)], 1)
    feats = dense[0, :, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T.contiguous()
    im, om, off, iden = oracle.kernel_map(coords, coords, (3, 3, 3))
    w5 = w.reshape(3, 3, 3, C).permute(3, 0, 1, 2).unsqueeze(1).contiguous()  # (C, 1, 3, 3, 3)
    want = torch.nn.functional.conv3d(dense, w5, padding=1, groups=C)[0][:, xyz[:, 0], xyz[:, 1], xyz[:, 2]].T
    for use_iden in (iden, None):  # with and without the identity shortcut
        got = explicit_depthwise_forward(feats, w, torch.as_tensor(im), torch.as_tensor(om), off,
                                         use_iden, len(coords))
        assert (got - want).abs().max() < 1e-12


# ---- point -> voxel front-end (oracle/voxelize.py) ------------------------------------------------
def _cloud_points(seed, n, batch, extent=1.0):
    rng = np.random.default_rng(seed)
    sizes = rng.multinomial(n - batch, np.ones(batch) / batch) + 1
    offsets = np.concatenate([[0], np.cumsum(sizes)])
    pts = ((rng.random((n, 3)) - 0.3) * extent).astype(np.float32)  # negative coordinates included
    return pts, offsets


def test_voxelize_equals_dictionary_brute_force():
    from oracle import voxelize
    pts, offsets = _cloud_points(5, 700, 3)
    feats = np.random.default_rng(6).standard_normal((700, 5))
    vs = 0.26
    rows = voxelize.voxel_rows(pts, offsets, vs)
    # the rows themselves: python floats, one point at a time
    inv = float(np.float32(1.0 / vs))
    for i in (0, 1, 350, 699):
        b = int(np.searchsorted(offsets, i, side="right") - 1)
        cell = [int(np.floor(np.float32(np.float32(v) * np.float32(inv)))) for v in pts[i]]
        assert rows[i].tolist() == [b] + cell
    groups = {}
    for i, r in enumerate(map(tuple, rows.tolist())):
        groups.setdefault(r, []).append(i)
    keys = sorted(groups)  # tuples compare lexicographically
    assert any(len(g) > 3 for g in groups.values()) and len(keys) > 100
    unique, to_orig, csr_indices, csr_offsets, to_unique = voxelize.unique_rows_csr(rows)
    assert unique.tolist() == [list(k) for k in keys]
    assert csr_indices.tolist() == [i for k in keys for i in groups[k]]
    assert csr_offsets.tolist() == [0] + list(np.cumsum([len(groups[k]) for k in keys]))
    assert to_unique.tolist() == [groups[k][0] for k in keys]
    assert all(keys[to_orig[i]] == tuple(rows[i]) for i in range(len(rows)))
    ops = {"sum": lambda a: a.sum(0), "mean": lambda a: a.mean(0), "max": lambda a: a.max(0),
           "min": lambda a: a.min(0)}
    for name, op in ops.items():
        want = np.stack([op(feats[groups[k]]) for k in keys])
        got = voxelize.segment_reduce(feats, csr_offsets, name, indices=csr_indices)
        assert np.abs(got - want).max() < 1e-12, name
    coords, vfeats, voffsets = voxelize.points_to_voxels(pts, feats, offsets, vs, "mean")
    assert coords.tolist() == [list(k[1:]) for k in keys]
    assert voffsets.tolist() == [sum(k[0] < b for k in keys) for b in range(4)]
    assert np.abs(vfeats - np.stack([feats[groups[k]].mean(0) for k in keys])).max() < 1e-12


def test_voxelize_lattice_closed_form():
    """c copies (jittered inside the cell) of every cell centre of an S^3 lattice, shuffled: S^3
    voxels in lexicographic order, c points each, mean feature = the cell's own value."""
    from oracle import voxelize
    S, c, vs = 5, 3, 0.25
    rng = np.random.default_rng(9)
    cells = np.stack(np.meshgrid(np.arange(S), np.arange(S), np.arange(S), indexing="ij"), -1).reshape(-1, 3) - 2
    cell_of_point = np.repeat(np.arange(S**3), c)
    rng.shuffle(cell_of_point)
    pts = ((cells[cell_of_point] + 0.5 + (rng.random((S**3 * c, 3)) - 0.5) * 0.8) * vs).astype(np.float32)
    value = rng.standard_normal((S**3, 2))
    feats = value[cell_of_point]
    coords, vfeats, voffsets = voxelize.points_to_voxels(pts, feats, [0, len(pts)], vs, "mean")
    assert coords.tolist() == cells.tolist()  # meshgrid 'ij' order is the lexicographic order
    assert voffsets.tolist() == [0, S**3]
    assert np.abs(vfeats - value).max() < 1e-12
    summed = voxelize.points_to_voxels(pts, feats, [0, len(pts)], vs, "sum")[1]
    assert np.abs(summed - c * value).max() < 1e-12


def test_unique_identities_of_the_reference_test():
    """tests/test_unique.py:21-35 of the reference: x == unique[to_orig] and x[csr_indices] sorted."""
    from oracle import voxelize
    x = np.random.default_rng(0).integers(0, 5, (10, 1))
    unique, to_orig, csr_indices, csr_offsets, to_unique = voxelize.unique_rows_csr(x)
    assert (unique[to_orig] == x).all()
    assert (np.sort(x[csr_indices], axis=0) == x[csr_indices]).all()
    assert (x[to_unique] == unique).all()
    assert np.diff(csr_offsets).sum() == len(x)


def test_device_division_differs_from_true_division_only_at_cell_borders():
    from oracle import voxelize
    rng = np.random.default_rng(3)
    vs = 0.02
    k = rng.integers(-2000, 2000, (4000, 3))
    on_border = (k * np.float32(vs)).astype(np.float32)  # products rounded to float: within an ulp of a border
    a = voxelize.voxel_rows(on_border, [0, 4000], vs, device_division=True)
    b = voxelize.voxel_rows(on_border, [0, 4000], vs, device_division=False)
    assert np.abs(a - b).max() == 1 and (a != b).any()
    inside = ((k + 0.5) * vs).astype(np.float32)
    a = voxelize.voxel_rows(inside, [0, 4000], vs, device_division=True)
    b = voxelize.voxel_rows(inside, [0, 4000], vs, device_division=False)
    assert (a == b).all() and (a[:, 1:] == k).all()
