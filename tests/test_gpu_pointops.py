"""GPU parity of the point-voxel operators against the CPU oracle: hashes, counts, dense copies
and index look-ups bit-exact; voxelize / devoxelize within 1e-5 (fp32), 1e-2 (fp16), 3e-2
(bf16) relative to the RMS of the expected values (fp32 sums; the oracle gets the inputs
already rounded to the I/O type).  Also the point-voxel round trip of an SPVCNN-style model."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 3e-2}


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd.nn import functional as F
    return ts, backend, F


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def _f32(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("n", [0, 1, 255, 5000, 200000])
def test_sphash_matches_oracle(mods, n):
    _, _, F = mods
    rng = np.random.default_rng(n)
    rows = rng.integers(-1000, 100000, (n, 4)).astype(np.int32)
    got = F.sphash(dev(rows))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.hash_gpu(rows))
    if n in (0, 200000):
        return
    offs = oracle.kernel_offsets(3)
    got = F.sphash(dev(rows), dev(offs))
    assert got.shape == (27, n)
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.kernel_hash_gpu(rows, offs))


def test_sphashquery_finds_rows_and_reports_missing(mods):
    _, _, F = mods
    rng = np.random.default_rng(0)
    coords = random_coords(rng, 6000, (40, 40, 20), batch=2)
    ref_hash = F.sphash(dev(coords))
    pick = rng.integers(0, len(coords), (700, 3))
    queries = coords[pick]                                    # [700, 3, 4], all present
    queries[::7, 0, 1] += 1000                                # some absent
    q_hash = F.sphash(dev(queries.reshape(-1, 4))).view(700, 3)
    got = F.sphashquery(q_hash, ref_hash).cpu().numpy()
    lut = {tuple(c): i for i, c in enumerate(coords.tolist())}
    want = np.array([[lut.get(tuple(r), -1) for r in q] for q in queries.tolist()])
    assert got.shape == (700, 3) and got.dtype == np.int32
    np.testing.assert_array_equal(got, want)
    assert (got[::7, 0] == -1).all()


@pytest.mark.parametrize("n,num", [(0, 5), (1, 1), (1000, 37), (300000, 90000)])
def test_spcount_matches_oracle(mods, n, num):
    _, _, F = mods
    rng = np.random.default_rng(n)
    idx = rng.integers(-3, num, n).astype(np.int32)
    got = F.spcount(dev(idx), num)
    assert got.dtype == torch.int32 and got.shape == (num,)
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.count(idx, num))


@pytest.mark.parametrize("c", [1, 4, 5, 16, 64, 96])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_spvoxelize_forward_backward(mods, c, dtype):
    _, _, F = mods
    rng = np.random.default_rng(c)
    n, n1 = 7000, 1500
    idx = rng.integers(-2, n1 + 2, n).astype(np.int32)
    counts = oracle.count(idx, n1)
    counts[3] = 0
    x = dev(rng.standard_normal((n, c)).astype(np.float32), dtype).requires_grad_(True)
    y = F.spvoxelize(x, dev(idx), dev(counts))
    assert y.shape == (n1, c) and y.dtype == dtype
    want = oracle.voxelize_forward(_f32(x), idx, counts)
    assert rel_rms(_f32(y), want) < TOL[dtype]
    # the points of a voxel are added in a fixed order: bit-identical from run to run, also
    # with the grouping rebuilt from a fresh copy of the indices
    assert torch.equal(y, F.spvoxelize(x.detach(), dev(idx), dev(counts)))
    g = dev(rng.standard_normal((n1, c)).astype(np.float32), dtype)
    y.backward(g)
    want_g = oracle.voxelize_backward(_f32(g), idx, counts, n)
    assert x.grad.shape == (n, c)
    assert rel_rms(_f32(x.grad), want_g) < TOL[dtype]


@pytest.mark.parametrize("c", [1, 4, 6, 32, 96])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_spdevoxelize_forward_backward(mods, c, dtype):
    _, _, F = mods
    rng = np.random.default_rng(c + 100)
    n, n_vox = 6000, 2000
    corner = rng.integers(-1, n_vox, (n, 8)).astype(np.int32)
    w = rng.uniform(0, 1, (n, 8)).astype(np.float32)
    f = dev(rng.standard_normal((n_vox, c)).astype(np.float32), dtype).requires_grad_(True)
    y = F.spdevoxelize(f, dev(corner), dev(w))
    assert y.shape == (n, c) and y.dtype == dtype
    assert rel_rms(_f32(y), oracle.devoxelize_forward(_f32(f), corner, w)) < TOL[dtype]
    g = dev(rng.standard_normal((n, c)).astype(np.float32), dtype)
    y.backward(g)
    want_g = oracle.devoxelize_backward(_f32(g), corner, w, n_vox)
    assert f.grad.shape == (n_vox, c)
    assert rel_rms(_f32(f.grad), want_g) < TOL[dtype]
    from torchsparse_amd import backend
    assert torch.equal(f.grad, backend.devoxelize_backward_cuda(g, dev(corner), dev(w), n_vox))


@pytest.mark.parametrize("m,groups", [(0, 4), (1, 1), (1000, 7), (50000, 20000), (300000, 100)])
def test_group_by_index_is_a_stable_sort(mods, m, groups):
    _, backend, _ = mods
    rng = np.random.default_rng(m)
    idx = rng.integers(-2, groups + 2, m).astype(np.int32)
    order, starts = backend.group_by_index(dev(idx), groups)
    starts = starts.cpu().numpy()
    valid = np.nonzero((idx >= 0) & (idx < groups))[0]
    want_order = valid[np.argsort(idx[valid], kind="stable")]
    np.testing.assert_array_equal(order.cpu().numpy()[:len(want_order)], want_order)
    np.testing.assert_array_equal(starts, np.searchsorted(np.sort(idx[valid]), np.arange(groups + 1)))
    # an in-place change of the indices invalidates the cached grouping
    t = dev(idx)
    backend.group_by_index(t, groups)
    if m:
        t.fill_(0)
        _, s2 = backend.group_by_index(t, groups)
        assert s2.cpu().numpy().tolist() == [0] + [m] * groups


def test_calc_ti_weights_are_the_trilinear_weights(mods):
    _, _, F = mods
    rng = np.random.default_rng(5)
    pts = rng.uniform(0, 20, (500, 3)).astype(np.float32)
    idx_query = rng.integers(-1, 50, (500, 8))
    idx_query[idx_query.max(1) < 0, 0] = 0                     # at least one corner exists
    for scale in (1, 2):
        w = F.calc_ti_weights(dev(pts), dev(idx_query), scale=scale).cpu().numpy()
        low = np.floor(pts / scale) * scale
        t = (pts - low) / scale                                # fraction along each axis
        want = np.zeros((500, 8))
        for corner in range(8):
            bits = [(corner >> 2) & 1, (corner >> 1) & 1, corner & 1]
            want[:, corner] = np.prod([t[:, a] if bits[a] else 1 - t[:, a] for a in range(3)], axis=0)
        want[idx_query == -1] = 0
        want /= want.sum(1, keepdims=True) + 1e-8
        np.testing.assert_allclose(w, want, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(w.sum(1), 1.0, atol=1e-4)


@pytest.mark.parametrize("c", [3, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_to_dense_forward_backward(mods, c, dtype):
    ts, _, _ = mods
    rng = np.random.default_rng(c)
    shape = (2, 9, 8, 7)
    coords = random_coords(rng, 300, shape[1:], batch=2)
    feats = dev(rng.standard_normal((len(coords), c)).astype(np.float32), dtype).requires_grad_(True)
    x = ts.SparseTensor(feats, dev(coords), spatial_range=shape)
    dense = x.dense()
    assert dense.shape == shape + (c,)
    np.testing.assert_array_equal(_f32(dense), oracle.to_dense_forward(_f32(feats), coords, shape))
    g = dev(rng.standard_normal(shape + (c,)).astype(np.float32), dtype)
    dense.backward(g)
    np.testing.assert_array_equal(_f32(feats.grad), oracle.to_dense_backward(_f32(g), coords, shape))


def test_point_voxel_round_trip(mods):
    """The initial_voxelize / voxel_to_point recipe of point-voxel networks: hash the floored
    points, find their voxel among the unique ones, average into voxels, interpolate back."""
    ts, _, F = mods
    rng = np.random.default_rng(9)
    pts = rng.uniform(0, 30, (20000, 3)).astype(np.float32)
    pc = np.concatenate([np.zeros((len(pts), 1), np.int32), np.floor(pts).astype(np.int32)], 1)
    pc_hash = F.sphash(dev(pc))
    sparse_hash = torch.unique(pc_hash)
    idx_query = F.sphashquery(pc_hash, sparse_hash)
    assert (idx_query >= 0).all()
    counts = F.spcount(idx_query, len(sparse_hash))
    assert int(counts.sum()) == len(pts)
    feats = dev(rng.standard_normal((len(pts), 16)).astype(np.float32))
    vox = F.spvoxelize(feats, idx_query, counts)
    want = oracle.voxelize_forward(_f32(feats), idx_query.cpu().numpy(), counts.cpu().numpy())
    assert rel_rms(_f32(vox), want) < 1e-5
    # a constant field survives voxelize -> devoxelize with full weights on one corner
    ones = torch.ones(len(pts), 4, device="cuda")
    v1 = F.spvoxelize(ones, idx_query, counts)
    corner = torch.full((len(pts), 8), -1, device="cuda", dtype=torch.int32)
    corner[:, 0] = idx_query
    w = torch.zeros(len(pts), 8, device="cuda")
    w[:, 0] = 1
    back = F.spdevoxelize(v1, corner, w)
    assert torch.allclose(back, ones, atol=1e-5)
