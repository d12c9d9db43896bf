"""Seeded synthetic inputs for tests and benchmarks (numpy only).

  uniform_voxels       unique voxels drawn uniformly from a box
  lidar_scan_voxels    a spinning multi-beam sensor ray-cast against a ground plane
                       and random axis-aligned boxes, quantised to voxels
  multisweep_voxels    several sweeps of such a sensor merged in a fixed metric range
  sphere_shell_voxels  one-voxel-thick shells of random spheres (dense neighbourhoods)
"""
from typing import Tuple

import numpy as np

__all__ = ["uniform_voxels", "lidar_scan_voxels", "multisweep_voxels", "sphere_shell_voxels"]


def uniform_voxels(n: int, extent: int = 128, seed: int = 0, batch: int = 1) -> np.ndarray:
    """int32 [batch*n, 4] rows (b, x, y, z), unique per sample."""
    rng = np.random.default_rng(seed)
    out = []
    for b in range(batch):
        flat = rng.choice(extent ** 3, size=n, replace=False)
        xyz = np.stack(np.unravel_index(flat, (extent,) * 3), 1)
        out.append(np.concatenate([np.full((n, 1), b), xyz], 1))
    return np.concatenate(out, 0).astype(np.int32)


def _raycast(origin, dirs, boxes_lo, boxes_hi, rmin, rmax):
    """Nearest hit of each ray with the plane z = 0 and a set of boxes; nan if none."""
    with np.errstate(divide="ignore", invalid="ignore"):
        t_ground = np.where(dirs[:, 2] < 0, -origin[2] / dirs[:, 2], np.inf)
        best = t_ground
        inv = 1.0 / dirs
        for lo, hi in zip(boxes_lo, boxes_hi):
            t0 = (lo - origin) * inv
            t1 = (hi - origin) * inv
            tn = np.minimum(t0, t1).max(1)
            tf = np.maximum(t0, t1).min(1)
            hit = (tn <= tf) & (tf > 0)
            t = np.where(hit, np.where(tn > 0, tn, tf), np.inf)
            best = np.minimum(best, t)
    ok = np.isfinite(best) & (best >= rmin) & (best <= rmax)
    return origin + dirs[ok] * best[ok, None]


def _sensor_dirs(n_beams, elev_lo_deg, elev_hi_deg, n_azimuth):
    elev = np.deg2rad(np.linspace(elev_lo_deg, elev_hi_deg, n_beams))
    azim = np.linspace(0, 2 * np.pi, n_azimuth, endpoint=False)
    e, a = np.meshgrid(elev, azim, indexing="ij")
    return np.stack([np.cos(e) * np.cos(a), np.cos(e) * np.sin(a), np.sin(e)], -1).reshape(-1, 3)


def _random_boxes(rng, n_boxes, r_lo, r_hi):
    radius = rng.uniform(r_lo, r_hi, n_boxes)
    angle = rng.uniform(0, 2 * np.pi, n_boxes)
    centre = np.stack([radius * np.cos(angle), radius * np.sin(angle)], 1)
    size = np.stack([rng.uniform(1.5, 5, n_boxes), rng.uniform(1.5, 5, n_boxes),
                     rng.uniform(1, 3, n_boxes)], 1)
    lo = np.concatenate([centre - size[:, :2] / 2, np.zeros((n_boxes, 1))], 1)
    hi = np.concatenate([centre + size[:, :2] / 2, size[:, 2:]], 1)
    return lo, hi


def lidar_scan_voxels(seed: int = 1, voxel: float = 0.05, n_beams: int = 64, n_azimuth: int = 2048,
                      n_boxes: int = 30, range_noise: float = 0.02) -> np.ndarray:
    """A 64-beam spinning sensor 1.8 m above a ground plane with `n_boxes` boxes in
    5-60 m, ranges 2-70 m (about 120k returns), Gaussian range noise of
    `range_noise` metres, quantised at `voxel` metres, shifted to non-negative
    coordinates and de-duplicated (sorted).  About 90k voxels with the defaults."""
    rng = np.random.default_rng(seed)
    origin = np.array([0.0, 0.0, 1.8])
    dirs = _sensor_dirs(n_beams, -24.8, 2.0, n_azimuth)
    lo, hi = _random_boxes(rng, n_boxes, 5.0, 60.0)
    pts = _raycast(origin, dirs, lo, hi, 2.0, 70.0)
    if range_noise > 0:
        ray = pts - origin
        rng_m = np.linalg.norm(ray, axis=1, keepdims=True)
        pts = origin + ray / rng_m * (rng_m + rng.normal(0, range_noise, rng_m.shape))
    vox = np.floor(pts / voxel).astype(np.int64)
    vox -= vox.min(0)
    vox = np.unique(vox, axis=0)
    return np.concatenate([np.zeros((len(vox), 1), np.int64), vox], 1).astype(np.int32)


def multisweep_voxels(seed: int = 2, batch: int = 2, target: int = 250_000, max_sweeps: int = 80,
                      n_azimuth: int = 2180, range_noise: float = 0.03) -> Tuple[np.ndarray, tuple]:
    """Per sample: sweeps of a 32-beam sensor (the ego moves 0.5 m per sweep past 40 boxes,
    Gaussian range noise of `range_noise` metres) are merged inside +-54 m x +-54 m x [-5, 3] m
    and voxelised at (0.075, 0.075, 0.2) m until the sample holds `target` voxels (or
    `max_sweeps` were merged).  Rows are (b, z, y, x) in a
    (41, 1440, 1440) grid, the layout detection backbones use.
    Returns (coords, spatial_range)."""
    rng = np.random.default_rng(seed)
    dirs = _sensor_dirs(32, -30.0, 10.0, n_azimuth)
    grid = (41, 1440, 1440)
    out = []
    for b in range(batch):
        lo, hi = _random_boxes(rng, 40, 4.0, 52.0)
        keys = np.zeros(0, np.int64)
        for s in range(max_sweeps):
            origin = np.array([0.5 * s, 0.0, 1.8])
            d = dirs + rng.normal(0, 0.002, dirs.shape)
            d /= np.linalg.norm(d, axis=1, keepdims=True)
            p = _raycast(origin, d, lo, hi, 1.0, 75.0)
            if range_noise > 0:
                ray = p - origin
                rng_m = np.linalg.norm(ray, axis=1, keepdims=True)
                p = origin + ray / rng_m * (rng_m + rng.normal(0, range_noise, rng_m.shape))
            p[:, 2] -= 1.8  # sensor frame: the ground lies near z = -1.8, inside [-5, 3]
            keep = (np.abs(p[:, 0]) < 54) & (np.abs(p[:, 1]) < 54) & (p[:, 2] > -5) & (p[:, 2] < 3)
            p = p[keep]
            ix = np.floor((p[:, 0] + 54) / 0.075).astype(np.int64)
            iy = np.floor((p[:, 1] + 54) / 0.075).astype(np.int64)
            iz = np.floor((p[:, 2] + 5) / 0.2).astype(np.int64)
            ok = (iz < grid[0]) & (iy < grid[1]) & (ix < grid[2])
            keys = np.union1d(keys, ((iz * grid[1] + iy) * grid[2] + ix)[ok])
            if len(keys) >= target:
                break
        zyx = np.stack([keys // (grid[1] * grid[2]), (keys // grid[2]) % grid[1], keys % grid[2]], 1)
        out.append(np.concatenate([np.full((len(zyx), 1), b), zyx], 1))
    return np.concatenate(out, 0).astype(np.int32), (batch,) + grid


def sphere_shell_voxels(seed: int = 3, extent: int = 512, n_spheres: int = 200,
                        target: int = 1_000_000) -> np.ndarray:
    """One-voxel-thick shells (round(|p - c|) == r) of random spheres, radii 10-60,
    clipped to the grid; spheres are added until about `target` voxels exist."""
    rng = np.random.default_rng(seed)
    centres = rng.uniform(0, extent, (n_spheres, 3))
    radii = rng.integers(10, 61, n_spheres)
    keys = np.zeros(0, np.int64)
    for c, r in zip(centres, radii):
        lo = np.maximum(np.floor(c - r - 1).astype(np.int64), 0)
        hi = np.minimum(np.ceil(c + r + 2).astype(np.int64), extent)
        gx, gy, gz = np.meshgrid(*[np.arange(lo[a], hi[a]) for a in range(3)], indexing="ij")
        dist = np.sqrt((gx - c[0]) ** 2 + (gy - c[1]) ** 2 + (gz - c[2]) ** 2)
        on = np.rint(dist) == r
        k = (gx[on] * extent + gy[on]) * extent + gz[on]
        keys = np.union1d(keys, k)
        if len(keys) >= target:
            break
    xyz = np.stack([keys // (extent * extent), (keys // extent) % extent, keys % extent], 1)
    return np.concatenate([np.zeros((len(xyz), 1), np.int64), xyz], 1).astype(np.int32)
