"""Seeded synthetic point clouds for tests and benchmarks.

All generators draw from ``numpy.random.Generator(PCG64(seed))``, build float64
geometry, quantise with ``floor(p / voxel)`` to int32 and return UNSORTED unique
voxels (a seeded shuffle is applied so no caller can rely on sortedness).  When
more voxels than ``target`` come out, a seeded random subset of exactly
``target`` rows is kept.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np

__all__ = ["planes_and_spheres", "lidar_scan", "indoor_room", "uniform_random",
           "make_cloud", "CONFIG_SEEDS"]

CONFIG_SEEDS = {1: 1001, 2: 1002, 3: 1003, 4: 1004, 5: 1005}


_BIAS = 1 << 20


def _unique_voxels(vox: np.ndarray) -> np.ndarray:
    """Distinct rows of an int32 [N,3] array with |coordinate| < 2^20 (fast path
    over one packed int64 key instead of a row-wise unique)."""
    v = vox.astype(np.int64) + _BIAS
    key = np.unique((v[:, 0] << 42) | (v[:, 1] << 21) | v[:, 2])
    out = np.empty((key.shape[0], 3), dtype=np.int32)
    out[:, 0] = (key >> 42) - _BIAS
    out[:, 1] = ((key >> 21) & ((1 << 21) - 1)) - _BIAS
    out[:, 2] = (key & ((1 << 21) - 1)) - _BIAS
    return out


def _finish(points: np.ndarray, voxel: float, target: Optional[int],
            rng: np.random.Generator) -> np.ndarray:
    vox = np.floor(points / voxel).astype(np.int32)
    vox = _unique_voxels(vox)
    perm = rng.permutation(vox.shape[0])
    if target is not None and vox.shape[0] > target:
        perm = perm[:target]
    return np.ascontiguousarray(vox[perm])


def uniform_random(n: int, extent: int, seed: int, ndim: int = 3,
                   lo: int = 0) -> np.ndarray:
    """``n`` distinct uniformly random voxels in ``[lo, lo+extent)^ndim``."""
    rng = np.random.default_rng(np.random.PCG64(seed))
    total = extent ** ndim
    if n > total:
        raise ValueError("more points requested than cells available")
    if total <= 8 * n + 1024:
        flat = rng.permutation(total)[:n]
    else:
        flat = np.unique(rng.integers(0, total, size=int(n * 1.2) + 64))
        while flat.shape[0] < n:
            flat = np.unique(np.concatenate(
                [flat, rng.integers(0, total, size=n)]))
        flat = rng.permutation(flat)[:n]
    out = np.empty((n, ndim), dtype=np.int32)
    for d in range(ndim - 1, -1, -1):
        out[:, d] = flat % extent + lo
        flat = flat // extent
    return out


def planes_and_spheres(target: int = 20000, grid: int = 128, seed: int = 1001
                       ) -> np.ndarray:
    """4 random planes and 2 random spheres in a ``grid^3`` cube, voxel 1.0."""
    rng = np.random.default_rng(np.random.PCG64(seed))
    per = max(64, int(target * 1.6) // 6)
    chunks = []
    for _ in range(4):
        normal = rng.normal(size=3)
        normal /= np.linalg.norm(normal)
        origin = rng.uniform(0.25 * grid, 0.75 * grid, size=3)
        helper = np.eye(3)[np.argmin(np.abs(normal))]
        u = np.cross(normal, helper)
        u /= np.linalg.norm(u)
        v = np.cross(normal, u)
        ab = rng.uniform(-grid, grid, size=(per * 4, 2))
        p = origin + ab[:, :1] * u + ab[:, 1:] * v
        keep = np.all((p >= 0) & (p < grid), axis=1)
        chunks.append(p[keep][:per * 2])
    for _ in range(2):
        centre = rng.uniform(0.25 * grid, 0.75 * grid, size=3)
        radius = rng.uniform(10.0, 30.0) * grid / 128.0
        d = rng.normal(size=(per * 2, 3))
        d /= np.linalg.norm(d, axis=1, keepdims=True)
        p = centre + radius * d
        keep = np.all((p >= 0) & (p < grid), axis=1)
        chunks.append(p[keep])
    return _finish(np.concatenate(chunks), 1.0, target, rng)


def _cast_sweep(sensor: np.ndarray, yaw0: float, boxes_lo: np.ndarray,
                boxes_hi: np.ndarray, max_range: float, rings: int,
                azimuths: int) -> np.ndarray:
    """One revolution: nearest hit of every ray on the ground plane z=0 or on an
    axis-aligned box (slab test); rays without a hit within range are dropped."""
    elev = np.deg2rad(np.linspace(-24.8, 2.0, rings))
    azim = yaw0 + np.linspace(0.0, 2.0 * np.pi, azimuths, endpoint=False)
    ce, se = np.cos(elev)[:, None], np.sin(elev)[:, None]
    d = np.stack([ce * np.cos(azim)[None, :], ce * np.sin(azim)[None, :],
                  np.broadcast_to(se, (rings, azimuths))], axis=-1).reshape(-1, 3)
    t_best = np.full(d.shape[0], np.inf)
    down = d[:, 2] < -1e-9
    t_best[down] = -sensor[2] / d[down, 2]
    with np.errstate(divide="ignore", invalid="ignore"):
        inv = 1.0 / d
        for lo, hi in zip(boxes_lo, boxes_hi):
            t0 = (lo - sensor) * inv
            t1 = (hi - sensor) * inv
            tn = np.nanmax(np.minimum(t0, t1), axis=1)
            tf = np.nanmin(np.maximum(t0, t1), axis=1)
            hit = (tf >= tn) & (tn > 1e-6)
            t_best = np.where(hit & (tn < t_best), tn, t_best)
    ok = np.isfinite(t_best) & (t_best <= max_range)
    return sensor + d[ok] * t_best[ok, None]


def lidar_scan(target: int = 200000, seed: int = 1002, voxel: float = 0.05,
               max_range: float = 50.0, rings: int = 64, azimuths: int = 2048,
               trajectory: float = 0.0, shift_to_positive: bool = False,
               max_sweeps: int = 400, grid_limit: Optional[int] = None
               ) -> Tuple[np.ndarray, int]:
    """Rotating-LiDAR scan of a ground plane and 30 random boxes.

    Sweeps are merged until at least ``1.1 * target`` unique voxels exist: with
    ``trajectory == 0`` the sensor is jittered by at most 0.5 m around the origin,
    otherwise it advances along a straight line of that length.  With
    ``grid_limit`` voxels whose x or y falls outside a window of that many
    cells around the median are dropped, so the shifted cloud fits a
    ``grid_limit``-wide grid.  Returns ``(voxels, sweeps_used)``.
    """
    rng = np.random.default_rng(np.random.PCG64(seed))
    r = max_range * np.sqrt(rng.uniform(0.0, 1.0, size=30))
    a = rng.uniform(0.0, 2.0 * np.pi, size=30)
    size = np.stack([rng.uniform(1, 6, 30), rng.uniform(1, 6, 30),
                     rng.uniform(1, 4, 30)], axis=1)
    centre = np.stack([r * np.cos(a), r * np.sin(a), size[:, 2] / 2], axis=1)
    boxes_lo, boxes_hi = centre - size / 2, centre + size / 2
    # keep the sensor outside every box
    near = np.all((boxes_lo[:, :2] < 1.5) & (boxes_hi[:, :2] > -1.5), axis=1)
    boxes_lo, boxes_hi = boxes_lo[~near], boxes_hi[~near]
    want = int(target * 1.1)
    vox = np.zeros((0, 3), dtype=np.int32)
    sweeps = 0
    while vox.shape[0] < want and sweeps < max_sweeps:
        if trajectory > 0.0:
            steps = max(2, int(trajectory / 0.25))
            pos = np.array([trajectory * (sweeps % steps) / steps - trajectory / 2,
                            rng.uniform(-0.2, 0.2), 1.8])
        elif sweeps == 0:
            pos = np.array([0.0, 0.0, 1.8])
        else:
            pos = np.array([rng.uniform(-0.5, 0.5), rng.uniform(-0.5, 0.5), 1.8])
        yaw0 = rng.uniform(0.0, 2.0 * np.pi / azimuths) if sweeps else 0.0
        pts = _cast_sweep(pos, yaw0, boxes_lo, boxes_hi, max_range, rings, azimuths)
        new = np.floor(pts / voxel).astype(np.int32)
        vox = _unique_voxels(np.concatenate([vox, new]))
        sweeps += 1
        if grid_limit is not None:
            centred = vox - np.median(vox, axis=0).astype(np.int32) + grid_limit // 2
            inside = np.all((centred[:, :2] >= 0) & (centred[:, :2] < grid_limit), axis=1)
            vox = vox[inside]
    if shift_to_positive:
        vox = vox - vox.min(axis=0, keepdims=True)
    perm = rng.permutation(vox.shape[0])
    if vox.shape[0] > target:
        perm = perm[:target]
    return np.ascontiguousarray(vox[perm]), sweeps


def indoor_room(target: int = 150000, seed: int = 1003, voxel: float = 0.02
                ) -> np.ndarray:
    """8 x 6 x 3 m room: 6 bounding planes plus 40 boxes / vertical cylinders,
    all surface-sampled."""
    rng = np.random.default_rng(np.random.PCG64(seed))
    room = np.array([8.0, 6.0, 3.0])
    budget = int(target * 2.2)
    chunks = []
    areas = []
    faces = []
    for axis in range(3):
        for side in (0.0, room[axis]):
            others = [k for k in range(3) if k != axis]
            areas.append(room[others[0]] * room[others[1]])
            faces.append((axis, side, others))
    areas = np.asarray(areas)
    wall_budget = int(budget * 0.7)
    for (axis, side, others), area in zip(faces, areas):
        n = int(wall_budget * area / areas.sum())
        p = np.empty((n, 3))
        p[:, axis] = side if side == 0.0 else side - 1e-6
        p[:, others[0]] = rng.uniform(0, room[others[0]], n)
        p[:, others[1]] = rng.uniform(0, room[others[1]], n)
        chunks.append(p)
    per = max(16, (budget - wall_budget) // 40)
    for k in range(40):
        dims = rng.uniform(0.2, 1.5, size=3)
        base = np.array([rng.uniform(0, room[0] - dims[0]),
                         rng.uniform(0, room[1] - dims[1]), 0.0])
        if k % 2 == 0:      # box: pick a face per sample, proportional to area
            fa = np.array([dims[1] * dims[2], dims[0] * dims[2], dims[0] * dims[1]])
            axis = rng.choice(3, size=per, p=fa / fa.sum())
            p = rng.uniform(0, 1, size=(per, 3)) * dims
            side = rng.integers(0, 2, size=per)
            p[np.arange(per), axis] = side * dims[axis] * (1 - 1e-9)
            chunks.append(base + p)
        else:               # vertical cylinder: lateral surface + top disc
            radius, height = dims[0] / 2, dims[2]
            n_side = int(per * 0.8)
            th = rng.uniform(0, 2 * np.pi, n_side)
            side_p = np.stack([radius * np.cos(th), radius * np.sin(th),
                               rng.uniform(0, height, n_side)], axis=1)
            n_top = per - n_side
            rr = radius * np.sqrt(rng.uniform(0, 1, n_top))
            th = rng.uniform(0, 2 * np.pi, n_top)
            top_p = np.stack([rr * np.cos(th), rr * np.sin(th),
                              np.full(n_top, height)], axis=1)
            c = base + np.array([radius, radius, 0.0])
            chunks.append(c + np.concatenate([side_p, top_p]))
    pts = np.concatenate(chunks)
    pts = np.clip(pts, 0.0, room - 1e-6)
    return _finish(pts, voxel, target, rng)


def make_cloud(config: int, scale: float = 1.0):
    """Voxels of BASELINE configuration ``config`` (1..5), optionally scaled down
    in voxel count for tests.  Returns a dict with ``coords`` (unsorted unique
    int32 [N,3]), ``batch_dims`` (None or int32 [B+1]) and a ``note``."""
    seed = CONFIG_SEEDS[config]
    if config == 1:
        c = planes_and_spheres(int(20000 * scale), 128, seed)
        return {"coords": c, "batch_dims": None, "note": "4 planes + 2 spheres, 128^3"}
    if config == 2:
        c, sweeps = lidar_scan(int(200000 * scale), seed)
        return {"coords": c, "batch_dims": None,
                "note": f"rotating LiDAR, 5 cm voxels, {sweeps} sweeps"}
    if config == 3:
        c = indoor_room(int(150000 * scale), seed)
        return {"coords": c, "batch_dims": None, "note": "indoor room, 2 cm voxels"}
    if config == 4:
        a, s0 = lidar_scan(int(100000 * scale), 1004)
        b, s1 = lidar_scan(int(100000 * scale), 2004)
        bd = np.array([0, a.shape[0], a.shape[0] + b.shape[0]], dtype=np.int32)
        return {"coords": np.concatenate([a, b]), "batch_dims": bd,
                "note": f"2 LiDAR scans ({s0}+{s1} sweeps)"}
    if config == 5:
        c, sweeps = lidar_scan(int(1000000 * scale), seed, trajectory=20.0,
                               shift_to_positive=True, grid_limit=2048)
        return {"coords": c, "batch_dims": None,
                "note": f"merged LiDAR sweeps along 20 m ({sweeps} sweeps), shifted to >= 0"}
    raise ValueError(f"unknown config {config}")
