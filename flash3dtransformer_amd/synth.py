"""Synthetic point clouds for benchmarks and tests (numpy, seeded; no dataset is needed).

uniform_cube  points ~ U[0, side)^3
lidar_sweep   a spinning-LiDAR-like sweep: 64 elevation rings from -25 deg to +2 deg, 2048 azimuth
              steps, rays cast from the origin against a ground plane z = -1.7 m and random
              axis-aligned boxes, ranges kept in [2, 80] m, then thinned to the requested size with
              acceptance proportional to 1/r^2.
"""
import numpy as np


def uniform_cube(n: int, side: float = 51.2, seed: int = 1001) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.uniform(0.0, side, (n, 3)).astype(np.float32)


def _ray_box(dirs, lo, hi):
    """slab test for rays from the origin; returns hit distance (inf when missed)"""
    with np.errstate(divide="ignore", invalid="ignore"):
        t1 = lo[None, :] / dirs
        t2 = hi[None, :] / dirs
    tmin = np.nanmax(np.minimum(t1, t2), axis=1)
    tmax = np.nanmin(np.maximum(t1, t2), axis=1)
    hit = (tmax >= np.maximum(tmin, 0.0)) & (tmin > 0.0)
    return np.where(hit, tmin, np.inf)


def lidar_sweep(n_points: int = 120_000, seed: int = 1004, n_rings: int = 64, n_azimuth: int = 2048,
                n_boxes: int = 30, oversample: int = 4) -> np.ndarray:
    """float32 [n_points, 4]: x, y, z, intensity ~ U[0, 1)"""
    rng = np.random.default_rng(seed)
    elev = np.deg2rad(np.linspace(-25.0, 2.0, n_rings))
    centres = rng.uniform(-60.0, 60.0, (n_boxes, 2))
    sizes = rng.uniform(1.0, 6.0, (n_boxes, 3))
    ground = -1.7
    pts = []
    for _ in range(oversample):
        az = (np.arange(n_azimuth) + rng.uniform(0.0, 1.0, n_azimuth)) * (2.0 * np.pi / n_azimuth)
        e, a = np.meshgrid(elev, az, indexing="ij")
        e = e + rng.normal(0.0, np.deg2rad(0.05), e.shape)
        dirs = np.stack([np.cos(e) * np.cos(a), np.cos(e) * np.sin(a), np.sin(e)], axis=-1).reshape(-1, 3)
        with np.errstate(divide="ignore"):
            t = np.where(dirs[:, 2] < 0, ground / dirs[:, 2], np.inf)
        for c, s in zip(centres, sizes):
            lo = np.array([c[0] - s[0] / 2, c[1] - s[1] / 2, ground])
            hi = np.array([c[0] + s[0] / 2, c[1] + s[1] / 2, ground + s[2]])
            t = np.minimum(t, _ray_box(dirs, lo, hi))
        keep = (t >= 2.0) & (t <= 80.0)
        pts.append(dirs[keep] * t[keep, None])
    pts = np.concatenate(pts, axis=0)
    r2 = (pts ** 2).sum(1)
    w = 1.0 / r2
    w /= w.sum()
    if pts.shape[0] < n_points:
        raise ValueError(f"only {pts.shape[0]} returns for {n_points} requested points; raise `oversample`")
    # weighted sampling without replacement (Efraimidis-Spirakis keys), O(n log n) and seed-stable
    keys = rng.uniform(0.0, 1.0, pts.shape[0]) ** (1.0 / (w * pts.shape[0]))
    idx = np.sort(np.argpartition(-keys, n_points - 1)[:n_points])   # keep sweep (ring-major) order
    out = np.empty((n_points, 4), dtype=np.float32)
    out[:, :3] = pts[idx]
    out[:, 3] = rng.uniform(0.0, 1.0, n_points)
    return out


def batch_of(clouds):
    """list of [n_i, >=3] arrays -> (fp16 xyz [N, 3], uint32 inclusive cumulative sizes [B])"""
    xyz = np.concatenate([c[:, :3] for c in clouds], axis=0).astype(np.float16)
    seps = np.cumsum([c.shape[0] for c in clouds]).astype(np.uint32)
    return np.ascontiguousarray(xyz), seps
