"""Shared helpers of the parity tests."""
import numpy as np
import torch


def canonical_pairs(in_maps, out_maps, offsets):
    """(k, out, in) triples sorted lexicographically: the canonical form of a kernel map."""
    in_maps = np.asarray(in_maps, dtype=np.int64)
    out_maps = np.asarray(out_maps, dtype=np.int64)
    offsets = np.asarray(offsets, dtype=np.int64)
    k = np.repeat(np.arange(len(offsets) - 1), np.diff(offsets))
    order = np.lexsort((in_maps, out_maps, k))
    return np.stack([k[order], out_maps[order], in_maps[order]], axis=1)


def sort_rows(a):
    a = np.asarray(a)
    return a[np.lexsort(a.T[::-1])]


def rel_err(a, b):
    """max|a-b| / max|b| per tensor (the relative error the feature tolerance is stated in)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def elementwise_rel_err(a, b):
    """max of |a-b| / (|b| + 1e-6) over entries with |b| > 1e-3 max|b| (the form the reference's
    native GEMM tests print, tests/csrc/test_cutlass_gemm.py:24-26)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    mask = np.abs(b) > 1e-3 * np.abs(b).max()
    return float((np.abs(a - b)[mask] / (np.abs(b)[mask] + 1e-6)).max())


def kaiming_weight(K, c_in, c_out, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    std = (2.0 / (c_in * K)) ** 0.5
    return (torch.randn(K, c_in, c_out, generator=g) * std).to(dtype)


def normal_features(n, c, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed + 1)
    return torch.randn(n, c, generator=g).to(dtype)


def oracle_kernel_map_by_item(oracle, in_coords, out_coords, kernel_size, stride=(1, 1, 1), threads=16):
    """The C oracle's kernel map of batch-sorted coordinates, one batch item per host thread (a pair
    never crosses items; the C code releases the interpreter lock), merged into one map in the
    reference's order: offsets in k order, ascending output row inside an offset."""
    from concurrent.futures import ThreadPoolExecutor
    in_coords, out_coords = np.asarray(in_coords), np.asarray(out_coords)

    def cuts(c):
        assert (np.diff(c[:, 0]) >= 0).all(), "coordinates must be sorted by batch item"
        return np.searchsorted(c[:, 0], np.arange(int(max(in_coords[:, 0].max(), out_coords[:, 0].max())) + 2))

    ci, co = cuts(in_coords), cuts(out_coords)
    parts = [(np.ascontiguousarray(in_coords[ci[b]:ci[b + 1]]), np.ascontiguousarray(out_coords[co[b]:co[b + 1]]))
             for b in range(len(ci) - 1)]
    with ThreadPoolExecutor(max_workers=max(1, min(threads, len(parts)))) as pool:
        maps = list(pool.map(lambda p: oracle.kernel_map(p[0], p[1], kernel_size, stride), parts))
    K = len(maps[0][2]) - 1
    ins, outs, off = [], [], [0]
    for k in range(K):
        for b, (im, om, o, _) in enumerate(maps):
            ins.append(im[o[k]:o[k + 1]] + ci[b])
            outs.append(om[o[k]:o[k + 1]] + co[b])
        off.append(off[-1] + sum(int(m[2][k + 1] - m[2][k]) for m in maps))
    odd = all(int(k) % 2 == 1 for k in kernel_size)
    iden = K // 2 if odd and len(in_coords) == len(out_coords) else None
    return (np.concatenate(ins).astype(np.int32), np.concatenate(outs).astype(np.int32),
            np.asarray(off, dtype=np.int64), iden)
