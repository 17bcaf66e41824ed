"""GPU parity of the point -> voxel front-end (wcn_voxel_rows, wcn_unique_rows_csr,
wcn_segment_reduce / _bwd) against oracle/voxelize.py and against torch's own device ops, which
are what the reference composes.  Index work is bit-exact; reduced features are within 1e-5
(fp32) / 1e-2 (fp16, bf16) relative; max / min are selections and exact."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import normal_features, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _points(seed, n, batch, extent=4.0):
    rng = np.random.default_rng(seed)
    sizes = rng.multinomial(n - batch, np.ones(batch) / batch) + 1
    offsets = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    pts = ((rng.random((n, 3)) - 0.3) * extent).astype(np.float32)
    return pts, offsets


# ---- voxel rows --------------------------------------------------------------------------------
@pytest.mark.parametrize("voxel_size", [0.02, 0.025, 0.1, 0.3])
def test_voxel_rows_equal_torch_device_op_and_oracle(voxel_size):
    from oracle import voxelize
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_rows
    pts, offsets = _points(1, 200_000, 3)
    rng = np.random.default_rng(2)
    k = rng.integers(-3000, 3000, (50_000, 3))
    border = (k * np.float32(voxel_size)).astype(np.float32)  # within an ulp of a cell border
    pts[:50_000] = border
    d = torch.as_tensor(pts, device=DEV)
    got = voxel_rows(d, torch.as_tensor(offsets), voxel_size).cpu().numpy()
    torch_cells = torch.floor(d / voxel_size).int().cpu().numpy()  # voxel.py:92 on the device
    assert np.array_equal(got[:, 1:], torch_cells)
    assert np.array_equal(got, voxelize.voxel_rows(pts, offsets, voxel_size, device_division=True))
    assert np.array_equal(got[:, 0], np.repeat(np.arange(3), np.diff(offsets)))


def test_voxel_rows_many_batch_items_and_bad_arguments():
    from warpconvnet_amd._lib import lib, ptr, stream_ptr
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_rows
    pts, offsets = _points(3, 30_000, 100)  # more items than the kernel takes by value
    got = voxel_rows(torch.as_tensor(pts, device=DEV), torch.as_tensor(offsets), 0.05).cpu().numpy()
    assert np.array_equal(got[:, 0], np.repeat(np.arange(100), np.diff(offsets)))
    L = lib()
    d = torch.as_tensor(pts, device=DEV)
    rows = torch.empty((len(pts), 4), dtype=torch.int32, device=DEV)
    bad = (ctypes.c_int64 * 2)(0, len(pts) - 1)  # offsets that do not end at N
    assert L.wcn_voxel_rows(ptr(d), len(pts), bad, None, 1, 0.05, ptr(rows), stream_ptr(d.device)) == -1
    ok = (ctypes.c_int64 * 2)(0, len(pts))
    assert L.wcn_voxel_rows(ptr(d), len(pts), ok, None, 1, 0.0, ptr(rows), stream_ptr(d.device)) == -1
    assert L.wcn_voxel_rows(ptr(d), len(pts), ok, None, 1, 0.05, ptr(rows), stream_ptr(d.device)) == 0
    torch.cuda.synchronize()


# ---- sorted unique + CSR -------------------------------------------------------------------------
def _check_unique(rows_np, dtype=torch.int32):
    from oracle import voxelize
    from warpconvnet_amd.utils.unique import unique_torch
    x = torch.as_tensor(rows_np, dtype=dtype, device=DEV)
    unique, to_orig, csr_indices, csr_offsets, to_unique = unique_torch(
        x, return_to_unique_indices=True)
    want = voxelize.unique_rows_csr(rows_np.reshape(len(rows_np), -1))
    assert unique.dtype == dtype and to_orig.dtype == torch.int64 and csr_offsets.dtype == torch.int64
    got_unique = unique.cpu().numpy().reshape(len(want[0]), -1)
    assert np.array_equal(got_unique, want[0])
    assert np.array_equal(to_orig.cpu().numpy(), want[1])
    assert np.array_equal(csr_indices.cpu().numpy(), want[2])
    assert np.array_equal(csr_offsets.cpu().numpy(), want[3])
    assert np.array_equal(to_unique.cpu().numpy(), want[4])
    return unique


@pytest.mark.parametrize("case", ["voxels4", "three_columns", "one_column", "flat_int64", "all_equal",
                                  "single_row", "wide_ranges", "one_full_range_column"])
def test_unique_rows_equal_oracle(case):
    rng = np.random.default_rng(11)
    if case == "voxels4":
        rows = np.concatenate([rng.integers(0, 3, (60_000, 1)), rng.integers(-20, 20, (60_000, 3))], 1)
    elif case == "three_columns":
        rows = rng.integers(-7, 9, (20_000, 3))
    elif case == "one_column":
        rows = rng.integers(0, 5, (10, 1))  # the size of the reference's own test
    elif case == "flat_int64":
        rows = rng.integers(-1000, 1000, (30_000,))
    elif case == "all_equal":
        rows = np.tile(np.array([[3, -4, 5, 6]]), (1000, 1))
    elif case == "single_row":
        rows = np.array([[0, 7, -7, 1]])
    elif case == "wide_ranges":  # 2 + 21 + 21 + 20 = 64 key bits
        rows = np.concatenate([rng.integers(0, 4, (40_000, 1)), rng.integers(-2**20, 2**20, (40_000, 2)),
                               rng.integers(0, 2**20, (40_000, 1))], 1)
        rows[:20_000] = rows[20_000:]  # every row twice
        rows[0] = [3, 2**20 - 1, 2**20 - 1, 2**20 - 1]
        rows[1] = [0, -2**20, -2**20, 0]
    else:
        rows = rng.integers(-2**31, 2**31, (5000, 1))
        rows[:100] = rows[100:200]
        rows[0], rows[1] = -2**31, 2**31 - 1
    dtype = torch.int64 if case == "flat_int64" else torch.int32
    _check_unique(rows.astype(np.int64 if case == "flat_int64" else np.int32), dtype)


def test_unique_rows_empty_and_range_error():
    from warpconvnet_amd._lib import WcnError
    from warpconvnet_amd.utils.unique import unique_torch
    empty = torch.empty((0, 4), dtype=torch.int32, device=DEV)
    unique, to_orig, csr_indices, csr_offsets, to_unique = unique_torch(empty, return_to_unique_indices=True)
    assert unique.shape == (0, 4) and len(to_orig) == 0 and csr_offsets.tolist() == [0] and len(to_unique) == 0
    rng = np.random.default_rng(0)
    wide = torch.as_tensor(rng.integers(-2**31, 2**31, (1000, 4)).astype(np.int32), device=DEV)
    with pytest.raises(WcnError) as e:  # 4 x 32 bits do not pack into one key
        unique_torch(wide)
    assert e.value.status == -4


def test_unique_rows_equal_torch_unique_at_full_size():
    """1 M rows against the ops the reference composes, run by torch on the same device
    (unique.py:84-100)."""
    from warpconvnet_amd.utils.unique import ToUnique
    g = torch.Generator(device=DEV).manual_seed(0)
    x = torch.randint(0, 1000, (1_000_000, 3), device=DEV, generator=g, dtype=torch.int32)  # test_unique.py:41
    x[:, 0] %= 8
    tu = ToUnique(return_to_unique_indices=True)
    unique, csr_indices, csr_offsets = tu.to_unique_csr(x)
    want_unique, inverse, counts = torch.unique(x, dim=0, sorted=True, return_inverse=True, return_counts=True)
    assert torch.equal(unique, want_unique)
    assert torch.equal(tu.to_orig_indices, inverse)
    assert torch.equal(csr_indices, inverse.argsort(stable=True))
    assert torch.equal(csr_offsets[1:], counts.cumsum(0)) and int(csr_offsets[0]) == 0
    assert torch.equal(x[tu.to_unique_indices], unique)
    assert torch.equal(tu.to_original(unique), x)
    # idempotence: the distinct rows are their own distinct rows, each in a group of its own
    again, idx2, off2 = ToUnique().to_unique_csr(unique)
    assert torch.equal(again, unique) and torch.equal(idx2, torch.arange(len(unique), device=DEV))
    assert torch.equal(off2, torch.arange(len(unique) + 1, device=DEV))


# ---- reductions over the groups -------------------------------------------------------------------
@pytest.mark.parametrize("reduction", ["sum", "mean", "max", "min"])
@pytest.mark.parametrize("dtype,channels", [(torch.float32, 7), (torch.float16, 32), (torch.bfloat16, 3),
                                            (torch.float32, 64)])
def test_segment_reduction_and_gradient(reduction, dtype, channels):
    from oracle import voxelize
    from warpconvnet_amd.ops.reductions import segment_reduction
    from warpconvnet_amd.utils.unique import unique_torch
    rng = np.random.default_rng(5)
    rows = rng.integers(0, 12, (30_000, 3)).astype(np.int32)
    x = normal_features(len(rows), channels, seed=1, dtype=dtype)
    _, to_orig, csr_indices, csr_offsets, _ = unique_torch(torch.as_tensor(rows, device=DEV))
    xd = x.to(DEV).requires_grad_(True)
    out = segment_reduction(xd, csr_offsets, reduction, indices=csr_indices, segment_of=to_orig)
    want = voxelize.segment_reduce(x.double().numpy(), csr_offsets.cpu().numpy(), reduction,
                                   indices=csr_indices.cpu().numpy())
    got = out.detach().double().cpu().numpy()
    assert out.dtype == dtype
    if reduction in ("max", "min"):
        assert np.array_equal(got, want)
    else:
        assert rel_err(got, want) <= TOL[dtype]
    # gradient: every point belongs to one voxel
    gy = normal_features(len(want), channels, seed=2, dtype=dtype)
    out.backward(gy.to(DEV))
    seg = to_orig.cpu().numpy()
    g64 = gy.double().numpy()
    if reduction == "sum":
        want_gx = g64[seg]
    elif reduction == "mean":
        counts = np.diff(csr_offsets.cpu().numpy())
        want_gx = g64[seg] / counts[seg][:, None]
    else:
        # the first point (lowest index) among equal extrema takes the gradient, as
        # torch_scatter.segment_csr's arg output does
        xs = x.double().numpy() * (1.0 if reduction == "max" else -1.0)
        order = csr_indices.cpu().numpy()
        offs = csr_offsets.cpu().numpy()
        want_gx = np.zeros_like(xs)
        for u in range(len(offs) - 1):
            members = order[offs[u]:offs[u + 1]]
            winner = members[np.argmax(xs[members], axis=0)]  # argmax returns the first maximum
            want_gx[winner, np.arange(channels)] = g64[u]
    got_gx = xd.grad.double().cpu().numpy()
    if reduction == "mean":
        assert rel_err(got_gx, want_gx) <= TOL[dtype]
    else:
        assert np.array_equal(got_gx, want_gx)
    # the same call without the caller's inverse derives it from the grouping
    xd2 = x.to(DEV).requires_grad_(True)
    segment_reduction(xd2, csr_offsets, reduction, indices=csr_indices).backward(gy.to(DEV))
    assert torch.equal(xd2.grad, xd.grad)


def test_row_reduction_consecutive_segments_var_std_random():
    from oracle import voxelize
    from warpconvnet_amd.ops.reductions import REDUCTIONS, row_reduction
    rng = np.random.default_rng(8)
    counts = rng.integers(0, 6, 5000)  # empty segments included
    counts[0] = 0
    splits = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    x = normal_features(int(splits[-1]), 16, seed=4)
    xd = x.to(DEV)
    sd = torch.as_tensor(splits, device=DEV)
    for name in ("sum", "mean", "max", "min"):
        got = row_reduction(xd, sd, name).double().cpu().numpy()
        want = voxelize.segment_reduce(x.double().numpy(), splits, name)
        assert rel_err(got, want) <= 1e-5, name
        assert np.all(got[counts == 0] == 0)
    mean = voxelize.segment_reduce(x.double().numpy(), splits, "mean")
    var = voxelize.segment_reduce(x.double().numpy() ** 2, splits, "mean") - mean ** 2  # reductions.py:27-34
    assert rel_err(row_reduction(xd, sd, REDUCTIONS.VAR).double().cpu().numpy(), var) <= 1e-5
    got_std = row_reduction(xd, sd, "std").double().cpu().numpy()
    # the difference of two fp32 means cancels; the square root magnifies that for small variances
    assert rel_err(got_std[counts > 1], np.sqrt(var + 1e-6)[counts > 1]) <= 1e-4
    filled = torch.as_tensor(counts > 0, device=DEV)
    keep = torch.as_tensor(splits[:-1][counts > 0], device=DEV)
    nonempty = torch.as_tensor(np.concatenate([splits[:-1][counts > 0], splits[-1:]]), device=DEV)
    picked = row_reduction(xd, nonempty, "random")  # one row of every segment
    lo = row_reduction(xd, nonempty, "min")
    hi = row_reduction(xd, nonempty, "max")
    assert picked.shape == lo.shape and bool(((picked >= lo) & (picked <= hi)).all())
    assert int(filled.sum()) == len(keep)


# ---- Points -> Voxels ---------------------------------------------------------------------------
@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("reduction", ["mean", "max", "sum"])
def test_points_to_voxels_equal_oracle(batch, reduction):
    from oracle import voxelize
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.geometry.types.voxels import Voxels
    pts, offsets = _points(21, 120_000, batch)
    feats = normal_features(len(pts), 7, seed=3)  # C = 7 as in the reference's tests
    pc = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets))
    st = pc.to_voxels(0.1, reduction=reduction)
    coords, vfeats, voffsets = voxelize.points_to_voxels(pts, feats.double().numpy(), offsets, 0.1, reduction)
    assert isinstance(st, Voxels) and st.voxel_size == 0.1
    assert st.coordinate_tensor.dtype == torch.int32
    assert np.array_equal(st.coordinate_tensor.cpu().numpy(), coords)
    assert np.array_equal(st.offsets.numpy(), voffsets)
    got = st.feature_tensor.double().cpu().numpy()
    if reduction == "max":
        assert np.array_equal(got, vfeats)
    else:
        assert rel_err(got, vfeats) <= 1e-5
    bi = st.batch_indexed_coordinates.cpu().numpy()
    assert np.array_equal(bi[:, 1:], coords)
    assert np.array_equal(bi[:, 0], np.repeat(np.arange(batch), np.diff(voffsets)))
    assert len(coords) < len(pts)


def test_voxels_from_points_feed_the_convolution():
    """The voxels made from points carry their (M, 4) rows; a convolution over them gives what it
    gives over the same voxels built from plain tensors."""
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    pts, offsets = _points(31, 60_000, 2)
    feats = normal_features(len(pts), 16, seed=5)
    st = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets)).to_voxels(0.1)
    plain = Voxels(st.coordinate_tensor.clone(), st.feature_tensor.clone(), offsets=st.offsets.clone())
    torch.manual_seed(0)
    conv = SparseConv3d(16, 32, kernel_size=3).to(DEV)
    assert torch.equal(conv(st).feature_tensor, conv(plain).feature_tensor)


def test_point_pool_variants():
    from oracle import voxelize
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.nn.functional.point_pool import point_pool
    from warpconvnet_amd.nn.modules.point_pool import PointMaxPool, PointSumPool
    B, C = 3, 7
    pts, offsets = _points(41, 20_000, B, extent=1.0)  # test_point_pool.py:20-29: unit cube, C = 7
    feats = normal_features(len(pts), C, seed=6)
    pc = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets))
    rows = voxelize.voxel_rows(pts, offsets, 0.1)
    unique, _, csr_indices, csr_offsets, to_unique = voxelize.unique_rows_csr(rows)

    out = PointMaxPool(downsample_voxel_size=0.1, return_type="point")(pc)  # test_point_pool.py:32-50
    assert isinstance(out, Points) and out.num_channels == C and len(out) < len(pc) and out.voxel_size == 0.1
    assert np.array_equal(out.coordinate_tensor.cpu().numpy(), pts[to_unique])
    want = voxelize.segment_reduce(feats.double().numpy(), csr_offsets, "max", indices=csr_indices)
    assert np.array_equal(out.feature_tensor.double().cpu().numpy(), want)

    out, found = PointSumPool(downsample_voxel_size=0.1, return_type="point",
                              return_neighbor_search_result=True)(pc)  # test_point_pool.py:73-92
    assert np.array_equal(found.neighbor_indices.cpu().numpy(), to_unique)
    assert np.array_equal(found.neighbor_row_splits.cpu().numpy(), out.offsets.numpy())

    out, tu = point_pool(pc, "mean", downsample_voxel_size=0.1, return_type="point",
                         avereage_pooled_coordinates=True, return_to_unique=True)
    centre = voxelize.segment_reduce(pts.astype(np.float64), csr_offsets, "mean", indices=csr_indices)
    assert rel_err(out.coordinate_tensor.double().cpu().numpy(), centre) <= 1e-5
    assert np.array_equal(tu.to_csr_indices.cpu().numpy(), csr_indices)

    # random: one point per voxel with its own features, in ascending point order
    out = point_pool(pc, "random", downsample_voxel_size=0.1, return_type="voxel")
    assert len(out) == len(unique)
    got_rows = np.concatenate([np.repeat(np.arange(B), np.diff(out.offsets.numpy()))[:, None],
                               out.coordinate_tensor.cpu().numpy()], 1)
    assert np.array_equal(np.unique(got_rows, axis=0), unique)
    down = pc.voxel_downsample(0.1)  # test_points.py:110-120
    assert down.coordinate_tensor.shape[1] == 3 and len(down) == len(unique)
    assert down.feature_tensor.shape[0] == down.coordinate_tensor.shape[0]
    reduced = pc.voxel_downsample(0.1, reduction="mean")
    mean = voxelize.segment_reduce(feats.double().numpy(), csr_offsets, "mean", indices=csr_indices)
    assert rel_err(reduced.feature_tensor.double().cpu().numpy(), mean) <= 1e-5
    with pytest.raises(NotImplementedError):
        point_pool(pc, "mean", downsample_max_num_points=100)


def test_points_to_voxels_full_size_properties():
    """4 M points (4 scenes) -> voxels of 2 cm: properties that do not need the oracle."""
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_downsample_csr_mapping
    from warpconvnet_amd.ops.reductions import segment_reduction
    g = torch.Generator(device=DEV).manual_seed(1)
    n = 4_000_000
    pts = torch.rand((n, 3), device=DEV, generator=g) * torch.tensor([8.0, 8.0, 0.1], device=DEV)
    offsets = torch.tensor([0, 1_000_000, 2_000_000, 3_000_000, n])
    unique, voffsets, csr_indices, csr_offsets, tu = voxel_downsample_csr_mapping(pts, offsets, 0.02)
    m = len(unique)
    assert unique.shape[1] == 4 and int(voffsets[-1]) == m and int(csr_offsets[-1]) == n
    key = ((unique[:, 0].long() * 1024 + unique[:, 1].long()) * 1024 + unique[:, 2].long()) * 1024 + unique[:, 3].long()
    assert bool((key[1:] > key[:-1]).all())  # strictly ascending: sorted and distinct
    assert torch.equal(torch.sort(csr_indices).values, torch.arange(n, device=DEV))  # a permutation
    cells = torch.floor(pts / 0.02).int()
    assert torch.equal(unique[tu.to_orig_indices][:, 1:], cells)
    assert torch.equal(cells[tu.to_unique_indices], unique[:, 1:])
    counts = csr_offsets.diff()
    assert int(counts.min()) >= 1
    ones = torch.ones((n, 4), device=DEV)
    assert torch.equal(segment_reduction(ones, csr_offsets, "sum", indices=csr_indices)[:, 0], counts.float())
    # sum over voxels of the per-voxel sums = sum over points (integers, exact in fp32 up to 2^24)
    marks = (torch.arange(n, device=DEV) % 3).float().view(-1, 1).expand(-1, 4).contiguous()
    per_voxel = segment_reduction(marks, csr_offsets, "sum", indices=csr_indices)
    assert float(per_voxel[:, 0].double().sum()) == float(marks[:, 0].double().sum())


def test_fused_points_call_equals_rows_then_unique_and_gradient_flows():
    """wcn_voxelize_points_csr = wcn_voxel_rows + wcn_unique_rows_csr; the inverse, derived on
    demand, equals the one the library writes; the gradient of to_voxels reaches the points'
    features."""
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_rows
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.utils.unique import ToUnique, unique_torch
    pts, offsets = _points(51, 150_000, 3)
    d = torch.as_tensor(pts, device=DEV)
    off = torch.as_tensor(offsets)
    fused = ToUnique(return_to_unique_indices=True)
    unique = fused.points_to_unique_voxel_rows(d, off, 0.07)
    want = unique_torch(voxel_rows(d, off, 0.07), return_to_unique_indices=True)
    assert torch.equal(unique, want[0])
    assert torch.equal(fused.to_orig_indices, want[1])  # derived from the grouping
    assert torch.equal(fused.to_csr_indices, want[2])
    assert torch.equal(fused.to_csr_offsets, want[3])
    assert torch.equal(fused.to_unique_indices, want[4])

    feats = normal_features(len(pts), 8, seed=9).to(DEV).requires_grad_(True)
    st = Points(d, feats, offsets=off).to_voxels(0.07, reduction="mean")
    gy = normal_features(len(st), 8, seed=10)
    st.feature_tensor.backward(gy.to(DEV))
    seg = want[1].cpu().numpy()
    counts = np.diff(want[3].cpu().numpy())
    want_gx = gy.double().numpy()[seg] / counts[seg][:, None]
    assert rel_err(feats.grad.double().cpu().numpy(), want_gx) <= 1e-5


def test_voxel_downsample_mapping():
    """tests/coords/test_voxel_ops.py:34-75 of the reference: every point maps to the voxel (or the
    down-sampled point) of its own cell; points outside every occupied cell are reported invalid."""
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_downsample_mapping
    from warpconvnet_amd.geometry.types.points import Points
    pts, offsets = _points(61, 90_000, 3, extent=1.0)
    feats = normal_features(len(pts), 7, seed=7)
    pc = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets))
    vs = 0.025
    down = pc.voxel_downsample(vs)
    up_map, down_map, valid = voxel_downsample_mapping(pc.coordinate_tensor, pc.offsets,
                                                       down.coordinate_tensor, down.offsets, vs)
    assert bool(valid.all()) and len(up_map) == len(pts)
    assert torch.equal(torch.floor(pc.coordinate_tensor[up_map] / vs),
                       torch.floor(down.coordinate_tensor[down_map] / vs))
    st = pc.to_voxels(vs)
    up_cells = torch.floor(pc.coordinate_tensor / vs).int()
    up_map, down_map, valid = voxel_downsample_mapping(up_cells, pc.offsets, st.coordinate_tensor, st.offsets)
    assert bool(valid.all())
    assert torch.equal(up_cells[up_map], st.coordinate_tensor[down_map.long()])
    # batch items must match too
    up_batch = torch.as_tensor(np.repeat(np.arange(3), np.diff(offsets)), device=DEV)
    down_batch = torch.as_tensor(np.repeat(np.arange(3), np.diff(st.offsets.numpy())), device=DEV)
    assert torch.equal(up_batch[up_map], down_batch[down_map.long()])
    moved = up_cells.clone()
    moved[:100] += 10_000  # far outside
    _, _, valid = voxel_downsample_mapping(moved, pc.offsets, st.coordinate_tensor, st.offsets)
    assert int((~valid).sum()) == 100 and not bool(valid[:100].any())


def test_point_to_sparse_wrapper_and_unpool():
    """Points -> voxels (mean) -> 3x3x3 convolution -> back onto the points: every point receives
    the output row of its own voxel, concatenated with its own features
    (reference: nn/modules/sparse_pool.py:172-189; its default unique_method "morton" takes the
    plain torch.unique branch of ToUnique)."""
    from oracle import voxelize
    from warpconvnet_amd.geometry.types.points import Points
    from warpconvnet_amd.nn.functional.point_pool import point_pool
    from warpconvnet_amd.nn.modules.point_pool import PointMaxPool, PointToSparseWrapper, PointUnpool
    from warpconvnet_amd.nn.modules.sparse_conv import SparseConv3d
    pts, offsets = _points(71, 50_000, 2, extent=2.0)
    feats = normal_features(len(pts), 16, seed=8)
    pc = Points(torch.as_tensor(pts, device=DEV), feats.to(DEV), offsets=torch.as_tensor(offsets))
    torch.manual_seed(1)
    conv = SparseConv3d(16, 32, kernel_size=3).to(DEV)
    out = PointToSparseWrapper(conv, voxel_size=0.1, concat_unpooled_pc=True)(pc)
    assert isinstance(out, Points) and len(out) == len(pc) and out.num_channels == 32 + 16
    assert torch.equal(out.coordinate_tensor, pc.coordinate_tensor)
    st, tu = point_pool(pc, "mean", downsample_voxel_size=0.1, return_type="voxel", return_to_unique=True)
    want_rows = conv(st).feature_tensor
    rows = voxelize.voxel_rows(pts, offsets, 0.1)
    inverse = voxelize.unique_rows_csr(rows)[1]
    assert np.array_equal(tu.to_orig_indices.cpu().numpy(), inverse)
    assert torch.equal(out.feature_tensor[:, :32], want_rows[torch.as_tensor(inverse, device=DEV)])
    assert torch.equal(out.feature_tensor[:, 32:], pc.feature_tensor)
    # module form (test_point_pool.py:95-121 of the reference, with the pooling's ToUnique handed over)
    pooled, tu = point_pool(pc, "max", downsample_voxel_size=0.1, return_to_unique=True)
    back = PointUnpool(concat_unpooled_pc=False)(pooled, pc, to_unique=tu)
    assert len(back) == len(pc) and back.num_channels == pooled.num_channels
    assert torch.equal(back.feature_tensor, pooled.feature_tensor[tu.to_orig_indices])
    assert bool((back.feature_tensor >= pc.feature_tensor).all())  # a maximum over a set containing the point
    with pytest.raises(NotImplementedError):
        PointUnpool()(PointMaxPool(downsample_voxel_size=0.1)(pc), pc)  # needs a nearest-neighbour search
