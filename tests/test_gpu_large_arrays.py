"""Feature arrays of more than 2^31 elements (and more than 4 GiB): the sizes 288 GB of HBM invite.
Row indices stay below 2^31, but `row * channels` and the byte offsets behind it do not, so every
address in the kernels has to be formed in 64 bits.  The CPU oracle does not finish at these sizes:
sampled output rows (the first, the last, and those either side of element 2^31) are checked against
plain torch fp32 operations over the same map, the maps themselves against their invariants."""
import math

import pytest
import torch

from helpers import kaiming_weight
from warpconvnet_amd._lib import lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def _enough_memory():
    """The cases here take up to some 60 GB of device memory."""
    free, _ = torch.cuda.mem_get_info(0)
    if free < (96 << 30):
        pytest.skip(f"{free >> 30} GiB of device memory free; these cases are sized for an MI355X")
    yield
    torch.cuda.empty_cache()


def _random_voxels(n, extent, seed):
    """n distinct voxels of an extent^3 box in random order, four batch items of n / 4 rows."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    return _voxels_of_cells(torch.randperm(extent ** 3, generator=g, device=DEV)[:n], extent)


def _scattered_voxels(n, gap, extent, seed):
    """n distinct voxels, one in every run of `gap` cells of an extent^3 box, in random order: with
    a large gap nearly every voxel is alone in its 4x4x4 block."""
    assert n * gap <= extent ** 3
    g = torch.Generator(device=DEV).manual_seed(seed)
    cells = torch.arange(n, device=DEV) * gap + torch.randint(0, gap, (n,), generator=g, device=DEV)
    return _voxels_of_cells(cells[torch.randperm(n, generator=g, device=DEV)], extent)


def _voxels_of_cells(cells, extent):
    n = cells.numel()
    rows = torch.empty((n, 4), dtype=torch.int32, device=DEV)
    rows[:, 0] = (torch.arange(n, device=DEV) * 4 // n).to(torch.int32)
    rows[:, 1] = (cells // (extent * extent)).to(torch.int32)
    rows[:, 2] = (cells // extent % extent).to(torch.int32)
    rows[:, 3] = (cells % extent).to(torch.int32)
    return rows


def _sample_rows(n, channels):
    edge = (1 << 31) // channels  # the row that holds element 2^31, where the array is that long
    parts = [torch.arange(0, 256), torch.arange(n - 256, n)]
    if 512 < edge < n - 512:
        parts.insert(1, torch.arange(edge - 128, edge + 128))
    return torch.cat(parts).to(DEV)


def _sampled_scatter(src, w_of, km, from_rows, to_rows, picks, n_to, width):
    """sum over pairs whose `to` row is in picks of src[from] @ w_of(k), in fp32, as (len(picks), width)."""
    place = torch.full((n_to,), -1, dtype=torch.int64, device=DEV)
    place[picks] = torch.arange(len(picks), device=DEV)
    out = torch.zeros(len(picks), width, dtype=torch.float32, device=DEV)
    for k in range(len(km)):
        im, om = km[k]
        f, t = (im, om) if from_rows == "in" else (om, im)
        where = place[t.long()]
        keep = where >= 0
        if bool(keep.any()):
            out.index_add_(0, where[keep], src[f[keep].long()].float() @ w_of(k))
    return out


def _check_map(km, n):
    offs = km.offsets.cpu()
    assert int(offs[-1]) == km.in_maps.numel() == km.out_maps.numel()
    assert int(km.in_maps.min()) >= 0 and int(km.in_maps.max()) < n
    assert int(km.out_maps.min()) >= 0 and int(km.out_maps.max()) < n
    centre = len(km) // 2
    im, om = km[centre]
    assert im.numel() == n and torch.equal(im, om)  # every voxel meets itself once at the centre offset
    for k in (0, len(km) - 1):
        a, b = km[k]
        assert bool((b[1:] > b[:-1]).all())           # output rows ascend inside an offset


def _check_pair_count(km, n, extent):
    """Voxels drawn uniformly from the box, a quarter of them per batch item: a voxel meets itself
    and, in each of the other directions, another voxel of its item with the item's density (a
    little less at the faces of the box)."""
    expected = n + (len(km) - 1) * n * (n / 4) / extent ** 3
    assert 0.98 * expected < km.in_maps.numel() < 1.005 * expected


def _close(got, want, tol=1e-2):
    scale = float(want.abs().max())
    return float((got.float() - want).abs().max()) <= tol * scale


def test_wide_rows_beyond_two_to_the_31_elements():
    """3x3x3, 256 -> 256, fp16, 8.5 M voxels: 2.18 G elements and 4.35 GB per feature array (the
    output-stationary kernel for wide rows), with both gradients."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_backward, sparse_conv_forward
    n, c = 8_500_000, 256
    assert n * c > (1 << 31)
    coords = _random_voxels(n, 400, seed=3)
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    _check_map(km, n)
    _check_pair_count(km, n, 400)
    g = torch.Generator(device=DEV).manual_seed(4)
    x = torch.randn(n, c, generator=g, device=DEV, dtype=torch.float16)
    w = kaiming_weight(27, c, c, seed=5, dtype=torch.float16).to(DEV)
    picks = _sample_rows(n, c)
    got = sparse_conv_forward(x, w, km, n)
    assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_dense<"), lib().wcn_conv_last_kernel()
    want = _sampled_scatter(x, lambda k: w[k].float(), km, "in", "out", picks, n, c)
    assert _close(got[picks], want)
    gy = torch.randn(n, c, generator=g, device=DEV, dtype=torch.float16)
    gx, gw = sparse_conv_backward(gy, x, w, km)
    want = _sampled_scatter(gy, lambda k: w[k].float().t(), km, "out", "in", picks, n, c)
    assert _close(gx[picks], want)
    del want, gx
    want = torch.stack([x[km[k][0].long()].float().t() @ gy[km[k][1].long()].float() for k in range(27)])
    assert _close(gw, want)


def test_one_slice_rows_beyond_two_to_the_31_elements():
    """3x3x3, 64 -> 64, fp16, 34 M voxels: 2.18 G elements per feature array (the pair-packed
    kernel of the headline configuration) over a map of some 150 M pairs."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    n, c = 34_000_000, 64
    assert n * c > (1 << 31)
    coords = _random_voxels(n, 640, seed=6)
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    _check_map(km, n)
    g = torch.Generator(device=DEV).manual_seed(7)
    x = torch.randn(n, c, generator=g, device=DEV, dtype=torch.float16)
    w = kaiming_weight(27, c, c, seed=8, dtype=torch.float16).to(DEV)
    picks = _sample_rows(n, c)
    got = sparse_conv_forward(x, w, km, n)
    assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_pack<"), lib().wcn_conv_last_kernel()
    want = _sampled_scatter(x, lambda k: w[k].float(), km, "in", "out", picks, n, c)
    assert _close(got[picks], want)
    _check_pair_count(km, n, 640)
    eye = torch.zeros(27, c, c, dtype=torch.float16, device=DEV)
    eye[13] = torch.eye(c, dtype=torch.float16, device=DEV)
    assert torch.equal(sparse_conv_forward(x, eye, km, n), x)  # centre tap only: a copy of every row


def test_table_of_scattered_voxels_with_many_bins():
    """12 M voxels that are nearly all alone in their block: 12 M blocks, which the build sorts into
    more bins than its small form has (an LDS counter per bin, a bin's blocks in an LDS table).
    Every voxel is found again at its own row, absent neighbours are not found, and the map of the
    set onto itself holds the centre pairs and little else."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.geometry.coords.search.torch_hashmap import TorchHashTable
    n = 12_000_000
    coords = _scattered_voxels(n, 500, 1900, seed=9)
    table = TorchHashTable.from_keys(coords)
    assert lib().wcn_table_default_capacity(n) // 2048 > 4096  # more bins than the small form takes
    found = table.search(coords)
    assert torch.equal(found.long(), torch.arange(n, device=DEV))
    shifted = coords.clone()
    shifted[:, 1] += 2000  # outside the box of the set
    assert int((table.search(shifted) >= 0).sum()) == 0
    km = generate_kernel_map(coords, coords, (1, 1, 1), (3, 3, 3))
    _check_map(km, n)
    pairs = km.in_maps.numel()
    assert n <= pairs < n + n // 10
    # every pair joins two voxels one step apart, in the direction of its offset
    for k in (0, 5, 26):
        im, om = km[k]
        if im.numel():
            d = coords[im.long()] - coords[om.long()]
            want = torch.tensor([0, k // 9 - 1, k // 3 % 3 - 1, k % 3 - 1], dtype=torch.int32, device=DEV)
            assert bool((d == want).all())


def test_down_and_up_sampling_beyond_two_to_the_31_elements():
    """2x2x2 stride 2, 64 -> 128, and its transposed 128 -> 64 back onto the fine voxels, fp16, 34 M
    fine voxels: the coarse array (some 30 M rows of 128) and the fine ones are beyond 2^31
    elements; the up-sampling takes the kernel for maps with one pair per output row."""
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.functional.sparse_conv import spatially_sparse_conv
    n = 34_000_000
    rows = _random_voxels(n, 640, seed=10)
    g = torch.Generator(device=DEV).manual_seed(11)
    x = torch.randn(n, 64, generator=g, device=DEV, dtype=torch.float16)
    offsets = torch.tensor([0, n // 4, n // 2, 3 * n // 4, n])
    fine = Voxels(rows[:, 1:].contiguous(), x, offsets=offsets)
    wd = kaiming_weight(8, 64, 128, seed=12, dtype=torch.float16).to(DEV)
    wu = kaiming_weight(8, 128, 64, seed=13, dtype=torch.float16).to(DEV)
    coarse = spatially_sparse_conv(fine, wd, 2, stride=2)
    m = len(coarse)
    assert m * 128 > (1 << 31)
    km = next(iter(fine.cache.values()))
    assert int(km.offsets[-1]) == n
    assert torch.equal(torch.sort(km.in_maps).values, torch.arange(n, dtype=torch.int32, device=DEV))
    assert int(km.out_maps.max()) == m - 1
    picks = _sample_rows(m, 128)
    want = _sampled_scatter(x, lambda k: wd[k].float(), km, "in", "out", picks, m, 128)
    assert _close(coarse.feature_tensor[picks], want)
    back = spatially_sparse_conv(coarse, wu, 2, stride=2, transposed=True, output_spatially_sparse_tensor=fine)
    assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_single<"), lib().wcn_conv_last_kernel()
    picks = _sample_rows(n, 64)
    want = _sampled_scatter(coarse.feature_tensor, lambda k: wu[k].float(), km, "out", "in", picks, n, 64)
    assert _close(back.feature_tensor[picks], want)


def test_map_of_125_offsets_over_20_million_voxels():
    """5x5x5 over 20 M voxels: offsets x voxels = 2.5 G entries of parked rows (10 GB), 16 -> 16 fp16
    over the map's 99 M pairs (the kernel for narrow rows takes up to 2^24 input rows; beyond that
    the pair-packed kernel runs)."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.nn.functional.sparse_conv import sparse_conv_forward
    n = 20_000_000
    assert 125 * n > (1 << 31)
    coords = _random_voxels(n, 540, seed=14)
    km = generate_kernel_map(coords, coords, (1, 1, 1), (5, 5, 5))
    assert len(km) == 125 and km.identity_map_index == 62
    _check_map(km, n)
    _check_pair_count(km, n, 540)
    counts = torch.diff(km.offsets)
    assert torch.equal(counts, counts.flip(0))
    for k in (0, 57, 124):  # every pair joins two voxels of one item, apart by its offset
        im, om = km[k]
        d = coords[im.long()] - coords[om.long()]
        want = torch.tensor([0, k // 25 - 2, k // 5 % 5 - 2, k % 5 - 2], dtype=torch.int32, device=DEV)
        assert im.numel() > 0 and bool((d == want).all())
    g = torch.Generator(device=DEV).manual_seed(15)
    x = torch.randn(n, 16, generator=g, device=DEV, dtype=torch.float16)
    w = kaiming_weight(125, 16, 16, seed=16, dtype=torch.float16).to(DEV)
    got = sparse_conv_forward(x, w, km, n)
    assert lib().wcn_conv_last_kernel().decode().startswith("conv_fwd_pack<"), lib().wcn_conv_last_kernel()
    picks = _sample_rows(n, 16)
    want = _sampled_scatter(x, lambda k: w[k].float(), km, "in", "out", picks, n, 16)
    assert _close(got[picks], want)


def test_pooling_and_depthwise_beyond_two_to_the_31_elements():
    """34 M voxels x 64 channels fp16 through the depthwise 3x3x3 convolution (centre tap: a copy;
    all taps one: the neighbours' sum on sampled rows) and through 2x2x2 stride-2 pooling (the sum of
    ones counts every fine voxel once, the mean of ones is one, the maximum on sampled coarse rows)."""
    from warpconvnet_amd.geometry.coords.search.torch_discrete import generate_kernel_map
    from warpconvnet_amd.geometry.types.voxels import Voxels
    from warpconvnet_amd.nn.functional.sparse_conv_depth import spatially_sparse_depthwise_conv
    from warpconvnet_amd.nn.functional.sparse_pool import sparse_reduce
    n, c = 34_000_000, 64
    rows = _random_voxels(n, 640, seed=17)
    g = torch.Generator(device=DEV).manual_seed(18)
    x = torch.randn(n, c, generator=g, device=DEV, dtype=torch.float16)
    km = generate_kernel_map(rows, rows, (1, 1, 1), (3, 3, 3))
    w = torch.zeros(27, c, dtype=torch.float16, device=DEV)
    w[13] = 1
    assert torch.equal(spatially_sparse_depthwise_conv(x, w, km, n), x)
    w[:] = 1
    got = spatially_sparse_depthwise_conv(x, w, km, n)
    picks = _sample_rows(n, c)
    eye = torch.eye(c, dtype=torch.float32, device=DEV)
    want = _sampled_scatter(x, lambda k: eye, km, "in", "out", picks, n, c)
    assert _close(got[picks], want)
    del got, km

    offsets = torch.tensor([0, n // 4, n // 2, 3 * n // 4, n])
    fine = Voxels(rows[:, 1:].contiguous(), x, offsets=offsets)
    top = sparse_reduce(fine, 2, 2, "max")
    m = len(top)
    pool_map = next(iter(fine.cache.values()))
    assert int(pool_map.offsets[-1]) == n and int(pool_map.out_maps.max()) == m - 1
    picks = _sample_rows(m, c)
    place = torch.full((m,), -1, dtype=torch.int64, device=DEV)
    place[picks] = torch.arange(len(picks), device=DEV)
    where = place[pool_map.out_maps.long()]
    keep = where >= 0
    want = torch.full((len(picks), c), float("-inf"), device=DEV)
    want.scatter_reduce_(0, where[keep][:, None].expand(-1, c), x[pool_map.in_maps[keep].long()].float(), "amax")
    assert torch.equal(top.feature_tensor[picks].float(), want)
    ones = fine.replace(batched_features=torch.ones_like(x))
    counts = sparse_reduce(ones, 2, 2, "sum").feature_tensor
    assert int(counts[:, 0].double().sum()) == n and float(counts.max()) <= 8 and float(counts.min()) >= 1
    assert bool((sparse_reduce(ones, 2, 2, "mean").feature_tensor == 1).all())


def test_points_to_voxels_of_120_million_points():
    """120 M points (4 items) -> some 104 M voxels of 2 cm, and the per-voxel sums of 32 fp32 features
    per point (3.84 G elements): sorted distinct voxels, the grouping a permutation of the points,
    every point in the group of its own cell, exact sums of small integers."""
    from warpconvnet_amd.geometry.coords.ops.voxel import voxel_downsample_csr_mapping
    from warpconvnet_amd.ops.reductions import segment_reduction
    from warpconvnet_amd.utils.gather import take_rows
    g = torch.Generator(device=DEV).manual_seed(19)
    n, c = 120_000_000, 32
    assert n * c > (1 << 31)
    pts = torch.rand((n, 3), device=DEV, generator=g) * torch.tensor([20.0, 20.0, 2.0], device=DEV)
    offsets = torch.tensor([0, n // 4, n // 2, 3 * n // 4, n])
    unique, voffsets, csr_indices, csr_offsets, tu = voxel_downsample_csr_mapping(pts, offsets, 0.02)
    m = len(unique)
    expected = 4 * 1e8 * (1 - math.exp(-(n / 4) / 1e8))  # occupied cells of 10^8 per item, uniform points
    assert 0.995 * expected < m < 1.005 * expected
    assert unique.shape[1] == 4 and int(voffsets[-1]) == m and int(csr_offsets[-1]) == n
    key = ((unique[:, 0].long() * 1024 + unique[:, 1].long()) * 1024 + unique[:, 2].long()) * 1024 + unique[:, 3].long()
    assert bool((key[1:] > key[:-1]).all())  # strictly ascending: sorted and distinct
    del key
    assert torch.equal(torch.sort(csr_indices).values, torch.arange(n, device=DEV))  # a permutation
    cells = torch.floor(pts / 0.02).int()
    # rows are picked with the package's take_rows: `unique[index]` itself returns wrong rows for the
    # last 2^26 of more than 2^26 indices into 16-byte rows with this PyTorch build
    assert torch.equal(tu.to_original(unique)[:, 1:], cells)
    by_column = torch.stack([unique[:, j].contiguous()[tu.to_orig_indices] for j in range(4)], dim=1)
    assert torch.equal(take_rows(unique, tu.to_orig_indices), by_column)
    del by_column
    assert torch.equal(take_rows(cells, tu.to_unique_indices), unique[:, 1:])
    del cells
    counts = csr_offsets.diff()
    assert int(counts.min()) >= 1
    marks = ((torch.arange(n, device=DEV).view(-1, 1) + torch.arange(c, device=DEV).view(1, -1)) % 3).float()
    per_voxel = segment_reduction(marks, csr_offsets, "sum", indices=csr_indices)
    assert per_voxel.shape == (m, c)
    for col in (0, c - 1):  # integers, exact in fp32 per voxel and in fp64 over all of them
        assert float(per_voxel[:, col].double().sum()) == float(marks[:, col].double().sum())
    last = csr_indices[int(csr_offsets[m - 1]):]   # the last voxel's points: beyond element 2^31 of `marks`
    assert torch.equal(per_voxel[m - 1], marks[last].sum(dim=0))
