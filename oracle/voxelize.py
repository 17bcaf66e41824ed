"""CPU restatement of the reference's point -> voxel front-end.

TEST INFRASTRUCTURE ONLY.

* `voxel_rows`: warpconvnet/geometry/coords/ops/voxel.py:92-95 (`torch.floor(points /
  voxel_size).int()` with the batch index of `batch_index_from_offset` in front).  The reference
  runs this on the device, where torch divides a float tensor by a host scalar as a multiplication
  with the scalar's reciprocal (reciprocal taken in double, rounded to float); `device_division=False`
  gives the true float32 division torch's CPU kernel does.  The two differ for points within an
  ulp of a voxel boundary.  Which one the device op does is pinned by the GPU test that compares the
  library's rows with torch's own device result bit for bit.
* `unique_rows_csr`: warpconvnet/utils/unique.py:57-109 (`torch.unique(dim=0, sorted=True,
  return_inverse=True, return_counts=True)`, stable argsort of the inverse, cumulative sum of the
  counts) with numpy's unique / argsort, which have the same definitions.  `to_unique` is the lowest
  row of every group; the reference's scatter with repeated indices (unique.py:96-100) leaves the
  choice among a group's rows open.
* `segment_reduce`: warpconvnet/ops/reductions.py:36-72.  Its torch_scatter.segment_csr
  (torch_scatter 2.1.x, not installed here) is documented as out[i] = reduce(src[indptr[i] :
  indptr[i + 1]]) with 0 for empty segments; restated with numpy ufunc.reduceat in float64.
* `points_to_voxels`: warpconvnet/nn/functional/point_pool.py:281-313 for return_type="voxel".

Pinned in tests/test_oracle_pins.py by a dictionary-based brute force, by a lattice with a known
number of points per cell (closed form) and by the identities the reference's own test asserts
(tests/test_unique.py:21-35).
"""
import numpy as np


def voxel_rows(points: np.ndarray, offsets, voxel_size: float, device_division: bool = True) -> np.ndarray:
    pts = np.asarray(points, dtype=np.float32)
    if device_division:
        q = pts * np.float32(1.0 / float(voxel_size))
    else:
        q = pts / np.float32(voxel_size)
    cells = np.floor(q).astype(np.int32)
    counts = np.diff(np.asarray(offsets, dtype=np.int64))
    batch = np.repeat(np.arange(len(counts), dtype=np.int32), counts)
    return np.concatenate([batch[:, None], cells], axis=1)


def unique_rows_csr(rows: np.ndarray):
    """unique (M, D), to_orig (N), csr_indices (N), csr_offsets (M + 1), to_unique (M)."""
    rows = np.asarray(rows)
    unique, inverse, counts = np.unique(rows, axis=0, return_inverse=True, return_counts=True)
    inverse = inverse.reshape(-1).astype(np.int64)
    csr_indices = np.argsort(inverse, kind="stable").astype(np.int64)
    csr_offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    to_unique = csr_indices[csr_offsets[:-1]] if len(counts) else np.zeros(0, np.int64)
    return unique, inverse, csr_indices, csr_offsets, to_unique


_UFUNC = {"sum": np.add, "mean": np.add, "max": np.maximum, "min": np.minimum}


def segment_reduce(features: np.ndarray, offsets: np.ndarray, reduction: str, indices=None) -> np.ndarray:
    x = np.asarray(features, dtype=np.float64)
    if indices is not None:
        x = x[np.asarray(indices)]
    offsets = np.asarray(offsets, dtype=np.int64)
    m = len(offsets) - 1
    out = np.zeros((m, x.shape[1]), dtype=np.float64)
    counts = np.diff(offsets)
    filled = counts > 0
    if filled.any():
        # reduceat reads up to the next start, so only the starts of non-empty segments are passed
        out[filled] = _UFUNC[reduction].reduceat(x, offsets[:-1][filled], axis=0)
    if reduction == "mean":
        out[filled] /= counts[filled][:, None]
    return out


def points_to_voxels(points, features, offsets, voxel_size: float, reduction: str):
    """coords (M, 3) int32, features (M, C) float64, voxel offsets (B + 1)."""
    rows = voxel_rows(points, offsets, voxel_size)
    unique, _, csr_indices, csr_offsets, _ = unique_rows_csr(rows)
    feats = segment_reduce(features, csr_offsets, reduction, indices=csr_indices)
    batch = len(offsets) - 1
    voxel_offsets = np.searchsorted(unique[:, 0], np.arange(batch + 1)).astype(np.int64)
    return unique[:, 1:], feats, voxel_offsets
