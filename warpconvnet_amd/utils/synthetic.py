"""Seeded synthetic voxel scenes for the benchmark configurations and the parity tests.

All generators are numpy-only, deterministic for a given seed, and return int32 voxel coordinates
deduplicated by first occurrence (so the row order is the random sampling order, which is the
hardest case for the gather side of the convolution).
"""
from typing import List, Tuple

import numpy as np


def _dedup_first_occurrence(vox: np.ndarray) -> np.ndarray:
    _, first = np.unique(vox, axis=0, return_index=True)
    return vox[np.sort(first)]


def _sample_until(sample_points, voxel_size: float, n_target: int, rng, batch: int = 1 << 18):
    """Draw surface points until n_target distinct voxels exist; keep the first n_target."""
    chunks: List[np.ndarray] = []
    vox = np.empty((0, 3), dtype=np.int32)
    for _ in range(64):
        pts = sample_points(rng, batch)
        chunks.append(np.floor(pts / voxel_size).astype(np.int32))
        vox = _dedup_first_occurrence(np.concatenate(chunks, axis=0))
        chunks = [vox]
        if n_target is not None and len(vox) >= n_target:
            return np.ascontiguousarray(vox[:n_target])
    return np.ascontiguousarray(vox)


def spheres_scene(seed: int = 0, n_target: int = 100_000, voxel_size: float = 0.01) -> np.ndarray:
    """Points uniform on the surfaces of 3 spheres (centres U[-1,1]^3 m, radii U[0.3,1.0] m)."""
    rng = np.random.default_rng(seed)
    centres = rng.uniform(-1.0, 1.0, size=(3, 3))
    radii = rng.uniform(0.3, 1.0, size=3)
    area = radii ** 2

    def sample(r, n):
        which = r.choice(3, size=n, p=area / area.sum())
        d = r.normal(size=(n, 3))
        d /= np.linalg.norm(d, axis=1, keepdims=True)
        return centres[which] + d * radii[which, None]

    return _sample_until(sample, voxel_size, n_target, rng)


def _indoor_rectangles(rng) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Axis-aligned rectangles (origin, edge u, edge v) of a room: floor, 4 walls, 10-30 boxes."""
    origin, eu, ev = [], [], []

    def rect(o, u, v):
        origin.append(o)
        eu.append(u)
        ev.append(v)

    ext = 8.0
    h = rng.uniform(2.5, 3.0)
    rect([0, 0, 0], [ext, 0, 0], [0, ext, 0])  # floor
    rect([0, 0, 0], [ext, 0, 0], [0, 0, h])  # walls
    rect([0, ext, 0], [ext, 0, 0], [0, 0, h])
    rect([0, 0, 0], [0, ext, 0], [0, 0, h])
    rect([ext, 0, 0], [0, ext, 0], [0, 0, h])
    for _ in range(int(rng.integers(10, 31))):
        e = rng.uniform(0.3, 2.0, size=3)
        p = np.array([rng.uniform(0, ext - e[0]), rng.uniform(0, ext - e[1]), 0.0])
        x, y, z = e
        rect(p + [0, 0, z], [x, 0, 0], [0, y, 0])  # top
        rect(p, [x, 0, 0], [0, 0, z])  # 4 sides
        rect(p + [0, y, 0], [x, 0, 0], [0, 0, z])
        rect(p, [0, y, 0], [0, 0, z])
        rect(p + [x, 0, 0], [0, y, 0], [0, 0, z])
    return np.array(origin, float), np.array(eu, float), np.array(ev, float)


def indoor_scene(seed: int = 0, n_target: int = 250_000, voxel_size: float = 0.02) -> np.ndarray:
    """Floor plane, 4 walls and 10-30 random axis-aligned boxes, surface-sampled by area."""
    rng = np.random.default_rng(seed)
    origin, eu, ev = _indoor_rectangles(rng)
    area = np.linalg.norm(np.cross(eu, ev), axis=1)
    prob = area / area.sum()

    def sample(r, n):
        which = r.choice(len(prob), size=n, p=prob)
        a = r.uniform(size=(n, 1))
        b = r.uniform(size=(n, 1))
        return origin[which] + a * eu[which] + b * ev[which]

    return _sample_until(sample, voxel_size, n_target, rng)


def indoor_batch(batch_size: int = 4, n_per_item: int = 250_000, voxel_size: float = 0.02,
                 seed: int = 0):
    """List of per-item (N_i, 3) int32 coordinate arrays and the (B+1,) offsets."""
    items = [indoor_scene(seed * 1000 + b, n_per_item, voxel_size) for b in range(batch_size)]
    offsets = np.zeros(batch_size + 1, dtype=np.int64)
    offsets[1:] = np.cumsum([len(i) for i in items])
    return items, offsets


def batch_indexed(items) -> np.ndarray:
    """Concatenate per-item (N_i, 3) coordinates into (N, 4) rows [batch, x, y, z]."""
    rows = [np.concatenate([np.full((len(c), 1), b, dtype=np.int32), c], axis=1)
            for b, c in enumerate(items)]
    return np.ascontiguousarray(np.concatenate(rows, axis=0), dtype=np.int32)


def random_cloud(seed: int, n: int, extent: int, batch_size: int = 1) -> np.ndarray:
    """(N, 4) batch-indexed unique voxels uniformly random in [0, extent)^3, batch-sorted."""
    rng = np.random.default_rng(seed)
    items = []
    for _ in range(batch_size):
        c = rng.integers(0, extent, size=(n, 3)).astype(np.int32)
        items.append(_dedup_first_occurrence(c))
    return batch_indexed(items)
