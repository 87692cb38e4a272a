"""Seeded synthetic point clouds for the five benchmark configurations.

Every generator returns int32 voxel coordinates ``[N, 4] = (b, x, y, z)`` that are
unique, non-negative (shifted by the cloud minimum as ``check_fwd.py:51`` does),
floor-quantised like ``script/utils.py:43`` and ordered like the reference's
``sparse_quantize`` + ``sparse_collate`` pipeline leaves them
(``script/utils.py:45-48, 167-196``): ascending by (b, x, y, z).

Only numpy is used so the same arrays feed the CPU oracle, the fixtures and the
GPU path.
"""
from __future__ import annotations

import numpy as np

COORD_BOUND = 3259  # backend/hash.cuh:503 (_BOUND of the base-3259 coordinate code)


def voxelize(points: np.ndarray, voxel: float, batch: int = 0) -> np.ndarray:
    """floor(points / voxel) after shifting by the minimum; unique; sorted (x,y,z)."""
    pts = points - points.min(axis=0, keepdims=True)
    q = np.floor(pts / voxel).astype(np.int64)
    q = np.unique(q, axis=0)  # lexicographic == ravel_hash order of script/utils.py:18-30
    assert q.min() >= 0 and q.max() < COORD_BOUND, (q.min(), q.max())
    b = np.full((q.shape[0], 1), batch, dtype=np.int64)
    return np.concatenate([b, q], axis=1).astype(np.int32)


def sphere_plane_cloud(seed: int = 1, n_sphere: int = 21000, n_plane: int = 7300,
                       voxel: float = 0.02) -> np.ndarray:
    """Config 1: unit-sphere surface samples plus a z=0 patch over [-1,1]^2."""
    rng = np.random.default_rng(seed)
    s = rng.standard_normal((n_sphere, 3))
    s /= np.linalg.norm(s, axis=1, keepdims=True)
    p = np.zeros((n_plane, 3))
    p[:, :2] = rng.uniform(-1.0, 1.0, size=(n_plane, 2))
    return voxelize(np.concatenate([s, p], axis=0), voxel)


def lidar_cloud(seed: int = 2, rings: int = 64, azimuths: int = 2048,
                n_ground: int = 19500, voxel: float = 0.1,
                half_extent: float = 50.0) -> np.ndarray:
    """Config 2: 64 elevation rings (-25..+3 deg) x 2048 azimuth steps with
    per-ray range U(2, 50) m, plus ground-plane samples at z = -1.7 m."""
    rng = np.random.default_rng(seed)
    elev = np.deg2rad(np.linspace(-25.0, 3.0, rings))
    azim = np.linspace(0.0, 2.0 * np.pi, azimuths, endpoint=False)
    e, a = np.meshgrid(elev, azim, indexing="ij")
    r = rng.uniform(2.0, 50.0, size=e.shape)
    xyz = np.stack([r * np.cos(e) * np.cos(a), r * np.cos(e) * np.sin(a), r * np.sin(e)], axis=-1)
    g = np.empty((n_ground, 3))
    g[:, :2] = rng.uniform(-half_extent, half_extent, size=(n_ground, 2))
    g[:, 2] = -1.7
    return voxelize(np.concatenate([xyz.reshape(-1, 3), g], axis=0), voxel)


def lidar_cloud_100k(seed: int = 2) -> np.ndarray:
    """Config 4 input: the config-2 generator with counts tuned to ~100k voxels."""
    return lidar_cloud(seed=seed, rings=64, azimuths=1344, n_ground=14000)


def _box_surface(rng, lo, hi, n):
    """n points uniformly spread over the six faces of the box [lo, hi]."""
    lo = np.asarray(lo, dtype=np.float64)
    hi = np.asarray(hi, dtype=np.float64)
    ext = hi - lo
    areas = np.array([ext[1] * ext[2], ext[1] * ext[2], ext[0] * ext[2],
                      ext[0] * ext[2], ext[0] * ext[1], ext[0] * ext[1]])
    face = rng.choice(6, size=n, p=areas / areas.sum())
    pts = lo + rng.uniform(size=(n, 3)) * ext
    axis = face // 2
    side = face % 2
    pts[np.arange(n), axis] = np.where(side == 0, lo[axis], hi[axis])
    return pts


def indoor_scene(rng, n_room: int = 120000, n_box: int = 2500) -> np.ndarray:
    """One 8 x 8 x 3 m room (four walls + floor) plus 20 axis-aligned boxes."""
    room = _box_surface(rng, (0, 0, 0), (8, 8, 3), n_room)
    room = room[room[:, 2] < 3.0 - 1e-9]  # no ceiling
    parts = [room]
    for _ in range(20):
        size = rng.uniform(0.3, 1.5, size=3)
        lo = np.array([rng.uniform(0.2, 7.8 - size[0]), rng.uniform(0.2, 7.8 - size[1]), 0.0])
        parts.append(_box_surface(rng, lo, lo + size, n_box))
    return np.concatenate(parts, axis=0)


def indoor_batch(seed: int = 5, scenes: int = 8, voxel: float = 0.02,
                 n_room: int = 120000, n_box: int = 2500) -> np.ndarray:
    """Config 5: ``scenes`` rooms collated with the batch index in column 0."""
    rng = np.random.default_rng(seed)
    out = [voxelize(indoor_scene(rng, n_room, n_box), voxel, batch=b) for b in range(scenes)]
    return np.concatenate(out, axis=0)


def random_cloud(seed: int, n: int, extent: int, batches: int = 1) -> np.ndarray:
    """Small dense-ish random cloud for unit tests (unique, sorted by (b,x,y,z))."""
    rng = np.random.default_rng(seed)
    c = np.stack([rng.integers(0, batches, n), rng.integers(0, extent, n),
                  rng.integers(0, extent, n), rng.integers(0, extent, n)], axis=1)
    return np.unique(c, axis=0).astype(np.int32)


def features(seed: int, n: int, c: int, dtype=np.float32) -> np.ndarray:
    rng = np.random.default_rng(seed + 1000)
    return rng.standard_normal((n, c)).astype(dtype)


def weights(seed: int, kv: int, c_in: int, c_out: int, dtype=np.float32) -> np.ndarray:
    rng = np.random.default_rng(seed + 2000)
    w = rng.standard_normal((kv, c_in, c_out)) / np.sqrt(kv * c_in)
    return w.astype(dtype)
