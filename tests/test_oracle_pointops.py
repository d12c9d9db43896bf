"""Pins the oracle's point-voxel operators: golden vectors written by the reference's own
compiled CPU sources (tests/golden/pointops_cpu.npz, hash_cpu.npz), numpy closed forms,
adjoint identities."""
import os

import numpy as np

import oracle

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _fold60(h):
    h = h.astype(np.uint64)
    return ((h >> np.uint64(60)) ^ (h & np.uint64(0xFFFFFFFFFFFFFFF))).astype(np.int64)


def test_gpu_hash_folds_to_the_reference_cpu_hash():
    g = np.load(os.path.join(GOLD, "hash_cpu.npz"))
    np.testing.assert_array_equal(_fold60(oracle.hash_gpu(g["rows"])), g["hash"])
    # known answer: FNV-1a of the four little-endian-independent words 0,1,2,3
    h = np.uint64(14695981039346656037)
    with np.errstate(over="ignore"):
        for v in (0, 1, 2, 3):
            h = (h ^ np.uint64(v)) * np.uint64(1099511628211)
    assert oracle.hash_gpu([[0, 1, 2, 3]])[0] == np.int64(h)
    # negative coordinates hash as their 32-bit two's complement
    a = oracle.hash_gpu([[0, -1, 5, 7]])[0]
    h = np.uint64(14695981039346656037)
    with np.errstate(over="ignore"):
        for v in (0, 0xFFFFFFFF, 5, 7):
            h = (h ^ np.uint64(v)) * np.uint64(1099511628211)
    assert a == np.int64(h)


def test_kernel_hash_is_the_hash_of_the_shifted_rows():
    rng = np.random.default_rng(0)
    rows = rng.integers(0, 500, (40, 4)).astype(np.int32)
    offs = oracle.kernel_offsets(3)
    got = oracle.kernel_hash_gpu(rows, offs)
    assert got.shape == (27, 40)
    for k in (0, 5, 13, 26):
        shifted = rows.copy()
        shifted[:, 1:] += offs[k]          # the batch column is not shifted
        np.testing.assert_array_equal(got[k], oracle.hash_gpu(shifted))
    np.testing.assert_array_equal(got[13], oracle.hash_gpu(rows))  # centre offset


def test_count_voxelize_devoxelize_against_the_compiled_reference():
    g = np.load(os.path.join(GOLD, "pointops_cpu.npz"))
    idx, n_vox = g["idx"], int(g["n_vox"])
    np.testing.assert_array_equal(oracle.count(idx, n_vox), g["counts"])
    np.testing.assert_array_equal(oracle.count(idx, n_vox), np.bincount(idx[idx >= 0], minlength=n_vox))
    valid = idx >= 0
    np.testing.assert_allclose(oracle.voxelize_forward(g["pts"][valid], idx[valid], g["counts"]), g["vox"],
                               rtol=1e-5, atol=1e-6)
    # points with an index outside the voxels contribute nothing (the GPU kernels' guard)
    np.testing.assert_allclose(oracle.voxelize_forward(g["pts"], idx, g["counts"]), g["vox"],
                               rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.voxelize_backward(g["top"], idx[valid], g["counts"], valid.sum()),
                               g["vox_bwd"], rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.devoxelize_forward(g["vfeat"], g["corner"], g["wts"]), g["devox"],
                               rtol=1e-5, atol=1e-5)


def test_voxelize_closed_forms_and_adjoint():
    rng = np.random.default_rng(1)
    n, n1, c = 500, 120, 7
    idx = rng.integers(-2, n1 + 3, n).astype(np.int32)       # some below 0, some past the end
    ok = (idx >= 0) & (idx < n1)
    counts = np.bincount(idx[ok], minlength=n1).astype(np.int32)
    counts[5] = 0                                             # a voxel declared empty is skipped
    x = rng.standard_normal((n, c)).astype(np.float32)
    want = np.zeros((n1, c))
    use = ok & (counts[np.clip(idx, 0, n1 - 1)] > 0)
    np.add.at(want, idx[use], x[use] / counts[idx[use]][:, None])
    np.testing.assert_allclose(oracle.voxelize_forward(x, idx, counts), want, rtol=1e-5, atol=1e-6)
    g = rng.standard_normal((n1, c)).astype(np.float32)
    back = oracle.voxelize_backward(g, idx, counts, n)
    assert (back[~use] == 0).all()
    # adjoint: <voxelize(x), g> == <x, voxelize_backward(g)>
    lhs = (oracle.voxelize_forward(x, idx, counts).astype(np.float64) * g).sum()
    rhs = (x.astype(np.float64) * back).sum()
    assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))


def test_devoxelize_closed_forms_and_adjoint():
    rng = np.random.default_rng(2)
    n, n_vox, c = 400, 150, 6
    corner = rng.integers(-1, n_vox, (n, 8)).astype(np.int32)
    w = rng.uniform(0, 1, (n, 8)).astype(np.float32)
    f = rng.standard_normal((n_vox, c)).astype(np.float32)
    gathered = np.where(corner[..., None] >= 0, f[np.clip(corner, 0, None)], 0.0)
    want = np.einsum("nk,nkc->nc", w.astype(np.float64), gathered)
    np.testing.assert_allclose(oracle.devoxelize_forward(f, corner, w), want, rtol=1e-5, atol=1e-5)
    g = rng.standard_normal((n, c)).astype(np.float32)
    want_b = np.zeros((n_vox, c))
    for k in range(8):
        ok = corner[:, k] >= 0
        np.add.at(want_b, corner[ok, k], w[ok, k][:, None].astype(np.float64) * g[ok])
    back = oracle.devoxelize_backward(g, corner, w, n_vox)
    np.testing.assert_allclose(back, want_b, rtol=1e-5, atol=1e-5)
    lhs = (oracle.devoxelize_forward(f, corner, w).astype(np.float64) * g).sum()
    rhs = (f.astype(np.float64) * back).sum()
    assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))


def test_to_dense_round_trip():
    rng = np.random.default_rng(3)
    rng_shape = (2, 6, 5, 4)
    cells = np.stack(np.unravel_index(rng.choice(np.prod(rng_shape), 70, replace=False), rng_shape), 1)
    coords = cells.astype(np.int32)
    feats = rng.standard_normal((70, 3)).astype(np.float32)
    dense = oracle.to_dense_forward(feats, coords, rng_shape)
    assert dense.shape == rng_shape + (3,)
    want = np.zeros(rng_shape + (3,), np.float32)
    want[coords[:, 0], coords[:, 1], coords[:, 2], coords[:, 3]] = feats
    np.testing.assert_array_equal(dense, want)
    np.testing.assert_array_equal(oracle.to_dense_backward(dense, coords, rng_shape), feats)
