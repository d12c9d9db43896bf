"""Shared input generators and brute-force definitions for the tests.

The brute-force builders below are written from the mathematical definition of
a (strided / transposed) convolution over a set of voxels, with python dicts and
loops, so that they share no code or formula layout with oracle/oracle.c.
"""
import itertools

import numpy as np


def random_coords(rng, n, shape, batch=1):
    """n unique voxels per sample, uniformly in the box `shape`; rows (b,x,y,z)."""
    shape = tuple(shape)
    out = []
    for b in range(batch):
        flat = rng.choice(int(np.prod(shape)), size=n, replace=False)
        xyz = np.stack(np.unravel_index(flat, shape), 1)
        out.append(np.concatenate([np.full((n, 1), b), xyz], 1))
    return np.concatenate(out, 0).astype(np.int32)


def digits(k, ks, odd):
    """Per-axis digit (cx,cy,cz) of flat kernel index k: x fastest for an odd
    kernel volume, z fastest for an even one."""
    if odd:
        cx = k % ks[0]
        cy = (k // ks[0]) % ks[1]
        cz = k // (ks[0] * ks[1])
    else:
        cz = k % ks[2]
        cy = (k // ks[2]) % ks[1]
        cx = k // (ks[2] * ks[1])
    return cx, cy, cz


def brute_conv_map(in_coords, out_coords, ks, stride, pad_eff):
    """map[o,k] = i  iff  in[i] == out[o]*stride - pad_eff + digit(k) (same batch)."""
    ks = tuple(ks)
    kvol = int(np.prod(ks))
    odd = kvol % 2 == 1
    where = {tuple(int(v) for v in c): i for i, c in enumerate(in_coords)}
    n_pad = (len(out_coords) + 127) // 128 * 128
    m = np.full((n_pad, kvol), -1, np.int32)
    for o, c in enumerate(out_coords):
        for k in range(kvol):
            d = digits(k, ks, odd)
            q = (int(c[0]),) + tuple(int(c[a + 1]) * stride[a] - pad_eff[a] + d[a] for a in range(3))
            m[o, k] = where.get(q, -1)
    return m


def brute_downsample_coords(in_coords, ks, stride, pad, cmax):
    """All outputs o (0 <= o <= cmax per spatial axis) whose receptive field
    {o*s - pad + c, 0 <= c < ks} contains an input voxel; lexicographic order."""
    outs = set()
    for c in in_coords:
        per_axis = []
        for a in range(3):
            cand = []
            for d in range(ks[a]):
                v = int(c[a + 1]) + pad[a] - d
                if v % stride[a] == 0 and 0 <= v // stride[a] <= cmax[a + 1]:
                    cand.append(v // stride[a])
            per_axis.append(cand)
        for xyz in itertools.product(*per_axis):
            outs.add((int(c[0]),) + xyz)
    return np.array(sorted(outs), np.int32).reshape(-1, 4)


def conv_closed_form(x, w, m, n_out):
    """float64 sum_k X[map[:,k]] W[k] with numpy fancy indexing."""
    x = np.asarray(x, np.float64)
    w = np.asarray(w, np.float64)
    y = np.zeros((n_out, w.shape[2]))
    for k in range(w.shape[0]):
        idx = m[:n_out, k]
        ok = idx >= 0
        y[ok] += x[idx[ok]] @ w[k]
    return y


def rel_rms(a, b):
    """max |a-b| relative to the RMS of b."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    rms = np.sqrt(np.mean(b * b)) + 1e-30
    return float(np.max(np.abs(a - b)) / rms)


def lidar_like_coords(rng, n_target, extent=(400, 400, 40)):
    """A cheap surface-like point set (ground sheet + boxes) for medium-size tests."""
    X, Y, Z = extent
    n_g = n_target * 2
    gx = rng.integers(0, X, n_g)
    gy = rng.integers(0, Y, n_g)
    gz = (2 + 1.5 * np.sin(gx / 37.0) + 1.5 * np.cos(gy / 23.0)).astype(np.int64)
    pts = [np.stack([gx, gy, gz], 1)]
    for _ in range(20):
        cx, cy = rng.integers(20, X - 20), rng.integers(20, Y - 20)
        sx, sy, sz = rng.integers(4, 16), rng.integers(4, 16), rng.integers(4, min(24, Z - 6))
        m = 400
        fx = rng.integers(cx - sx, cx + sx + 1, m)
        fz = rng.integers(3, 3 + sz, m)
        pts.append(np.stack([fx, np.full(m, cy - sy), fz], 1))
        pts.append(np.stack([fx, np.full(m, cy + sy), fz], 1))
    p = np.concatenate(pts, 0)
    p = p[(p[:, 0] >= 0) & (p[:, 0] < X) & (p[:, 1] >= 0) & (p[:, 1] < Y) & (p[:, 2] >= 0) & (p[:, 2] < Z)]
    p = np.unique(p, axis=0)
    if len(p) > n_target:
        p = p[np.sort(rng.choice(len(p), n_target, replace=False))]
    return np.concatenate([np.zeros((len(p), 1), np.int64), p], 1).astype(np.int32)
