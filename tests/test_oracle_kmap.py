"""Pins the integer part of the CPU oracle (kernel maps and derived products)
against brute force, invariants and numpy library routines."""
import numpy as np
import pytest

import oracle
from helpers import brute_conv_map, brute_downsample_coords, random_coords

RNG = np.random.default_rng


def test_kernel_offsets_literal_tables():
    # nn/utils/kernel.py:21-35 written out by hand
    k3 = [(x, y, z) for z in (-1, 0, 1) for y in (-1, 0, 1) for x in (-1, 0, 1)]
    assert oracle.kernel_offsets(3).tolist() == [list(t) for t in k3]
    k2 = [(x, y, z) for x in (0, 1) for y in (0, 1) for z in (0, 1)]
    assert oracle.kernel_offsets(2).tolist() == [list(t) for t in k2]
    assert oracle.kernel_offsets((3, 1, 1)).tolist() == [[-1, 0, 0], [0, 0, 0], [1, 0, 0]]
    assert oracle.kernel_offsets((1, 3, 1)).tolist() == [[0, -1, 0], [0, 0, 0], [0, 1, 0]]
    # even size 4 spans -1..2 (python floor division), stride and dilation scale it
    assert sorted(set(oracle.kernel_offsets(4)[:, 0].tolist())) == [-1, 0, 1, 2]
    assert oracle.kernel_offsets(3, stride=2, dilation=3)[0].tolist() == [-6, -6, -6]


@pytest.mark.parametrize("ks", [3, 2, 5, (3, 1, 1), (1, 3, 1), (2, 3, 3), (3, 5, 3)])
@pytest.mark.parametrize("batch", [1, 3])
def test_kmap_subm_bruteforce(ks, batch):
    rng = RNG(10)
    coords = random_coords(rng, 60, (7, 6, 5), batch)
    coords = coords[rng.permutation(len(coords))]
    ks3 = (ks,) * 3 if isinstance(ks, int) else ks
    kvol = int(np.prod(ks3))
    odd = kvol % 2 == 1
    got = oracle.kmap_subm(coords, ks3)
    pad_eff = [(k - 1) // 2 if odd else 0 for k in ks3]
    want = brute_conv_map(coords, coords, ks3, (1, 1, 1), pad_eff)
    np.testing.assert_array_equal(got, want)
    n = len(coords)
    assert (got[n:] == -1).all()
    if odd:
        assert (got[:n, kvol // 2] == np.arange(n)).all()
        o, k = np.nonzero(got[:n] >= 0)
        assert (got[got[o, k], kvol - 1 - k] == o).all()  # symmetry


@pytest.mark.parametrize("ks,stride,pad", [
    (2, 2, 0), (3, 2, 1), (3, 3, 1), (5, 2, 2), (5, 3, 2), (2, 3, 0), (3, 2, 0),
    ((3, 1, 1), (2, 1, 1), (0, 0, 0)), ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((1, 3, 1), (1, 2, 1), 0)])
@pytest.mark.parametrize("with_range", [False, True])
def test_kmap_downsample_bruteforce(ks, stride, pad, with_range):
    rng = RNG(11)
    shape = (9, 8, 7)
    coords = random_coords(rng, 70, shape, batch=2)
    coords = coords[rng.permutation(len(coords))]
    ks3 = (ks,) * 3 if isinstance(ks, int) else tuple(ks)
    st3 = (stride,) * 3 if isinstance(stride, int) else tuple(stride)
    pd3 = (pad,) * 3 if isinstance(pad, int) else tuple(pad)
    sr = None
    if with_range:  # build_kmap.py:65-72
        sr = (2,) + tuple((shape[a] + 2 * pd3[a] - (ks3[a] - 1) - 1) // st3[a] + 1 for a in range(3))
    omap, ocoords = oracle.kmap_downsample(coords, ks3, st3, pd3, spatial_range=sr)
    _, cmax = oracle.downsample_bounds(coords, ks3, st3, pd3, sr)
    want_coords = brute_downsample_coords(coords, ks3, st3, pd3, cmax)
    np.testing.assert_array_equal(ocoords, want_coords)
    want = brute_conv_map(coords, want_coords, ks3, st3, pd3)
    np.testing.assert_array_equal(omap, want)
    # every (input, offset) appears at most once
    n_out = len(ocoords)
    for k in range(omap.shape[1]):
        col = omap[:n_out, k]
        col = col[col >= 0]
        assert len(np.unique(col)) == len(col)
    # strictly ascending lexicographic order
    key = ((ocoords[:, 0].astype(np.int64) * 1000 + ocoords[:, 1]) * 1000 + ocoords[:, 2]) * 1000 + ocoords[:, 3]
    assert (np.diff(key) > 0).all()


def test_downsample_k_equals_s_is_floor_unique():
    # kmap/downsample.py:34-37: for k == s the output set is unique(coords // s)
    rng = RNG(12)
    coords = random_coords(rng, 300, (20, 18, 16), batch=2)
    _, ocoords = oracle.kmap_downsample(coords, 2, 2, 0)
    c = coords.copy()
    c[:, 1:] //= 2
    np.testing.assert_array_equal(ocoords, np.unique(c, axis=0))
    np.testing.assert_array_equal(oracle.spdownsample_floor(coords, 2), np.unique(c, axis=0))


def test_downsample_k_equals_s_drops_inputs_at_an_even_maximum():
    # kmap/func/hashmap_on_the_fly.py:27-37 derives the output bound from the input maximum as
    # (max + 2 pad - (k - 1)) // stride: with k = s = 2 an input whose coordinate is the (even)
    # maximum of its axis maps to max / 2, one past that bound, and gets no output.  A strided
    # map therefore does NOT give every input a pair, and its transposed map has empty rows.
    coords = np.array([[0, 0, 0, 0], [0, 3, 5, 1], [0, 6, 2, 1], [0, 6, 5, 0]], np.int32)  # max x = 6
    omap, ocoords = oracle.kmap_downsample(coords, 2, 2, 0)
    np.testing.assert_array_equal(ocoords, [[0, 0, 0, 0], [0, 1, 2, 0]])
    assert sorted(omap[omap >= 0].tolist()) == [0, 1]
    t = oracle.transpose_map(omap, len(coords))
    assert ((t[:4] >= 0).sum(1) == [1, 1, 0, 0]).all()
    # an odd maximum on every axis keeps all of them
    coords[:, 1:] += np.array([1, 0, 0], np.int32)
    omap, _ = oracle.kmap_downsample(coords, 2, 2, 0)
    assert (omap >= 0).sum() == 4


@pytest.mark.parametrize("ks,stride", [(2, 2), (3, 2), (3, 1), (2, 1), (5, 3)])
def test_lookup_coords_bruteforce(ks, stride):
    rng = RNG(13)
    coords = random_coords(rng, 80, (8, 8, 8), batch=2)
    ocoords = oracle.spdownsample_floor(coords, stride)
    got = oracle.lookup_coords(coords, ocoords, ks, stride)
    odd = ks % 2 == 1
    want = brute_conv_map(coords, ocoords, (ks,) * 3, (stride,) * 3, [(ks - 1) // 2] * 3)
    np.testing.assert_array_equal(got, want)
    assert odd or (ks - 1) // 2 == 0


def test_transpose_map_inverse_relation():
    rng = RNG(14)
    coords = random_coords(rng, 200, (12, 12, 12))
    omap, ocoords = oracle.kmap_downsample(coords, 2, 2, 0)
    t = oracle.transpose_map(omap, len(coords))
    assert t.shape == (oracle.ceil128(len(coords)), 8)
    rel = {(int(o), int(k), int(omap[o, k])) for o, k in zip(*np.nonzero(omap >= 0))}
    rel_t = {(int(t[i, k]), int(k), int(i)) for i, k in zip(*np.nonzero(t >= 0))}
    assert rel == rel_t
    # k == s: every fine voxel has exactly one coarse parent
    assert ((t[: len(coords)] >= 0).sum(1) == 1).all()


@pytest.mark.parametrize("kvol,split", [(27, 1), (27, 3), (8, 1), (8, 2), (125, 5), (27, 2)])
def test_bitmask_reorder_reduce_definitions(kvol, split):
    rng = RNG(15)
    n, n_pad = 300, 384
    m = np.full((n_pad, kvol), -1, np.int32)
    m[:n] = np.where(rng.random((n, kvol)) < 0.3, rng.integers(0, n, (n, kvol)), -1)
    bm = oracle.derive_bitmask(m, split, n)
    L = -(-kvol // split)
    for s in range(split):
        cols = m[:n, s * L:min(kvol, (s + 1) * L)] >= 0
        want = (cols.astype(np.int64) << np.arange(cols.shape[1])).sum(1)
        np.testing.assert_array_equal(bm[s, :n].astype(np.int64) & 0xFFFFFFFF, want & 0xFFFFFFFF)
        assert (bm[s, n:] == -1).all()
    loc = np.argsort(-bm.astype(np.int64), axis=1, kind="stable").astype(np.int32)
    srt = np.take_along_axis(bm, loc, 1)
    assert (np.diff(srt.astype(np.int64), axis=1) <= 0).all()
    ro = oracle.reorder_map(m, loc)
    for c in range(kvol):
        np.testing.assert_array_equal(ro[:, c], m[loc[c // L], c])
    red = oracle.reduce_bitmask(srt, 128)
    want = np.bitwise_or.reduce(srt.reshape(split, -1, 128), axis=2)
    np.testing.assert_array_equal(red, want)
    red64 = oracle.reduce_bitmask(srt, 64)
    np.testing.assert_array_equal(red64, np.bitwise_or.reduce(srt.reshape(split, -1, 64), axis=2))


def test_pair_lists_masks_scans():
    rng = RNG(16)
    coords = random_coords(rng, 500, (14, 14, 14))
    for omap, n_in, n_out in [
        (oracle.kmap_subm(coords, 3), 500, 500),
        oracle.kmap_downsample(coords, 2, 2, 0)[:1] + (500, None),
        oracle.kmap_downsample(coords, 3, 2, 1)[:1] + (500, None),
    ]:
        if n_out is None:
            n_out = int((omap >= 0).any(1).sum())
        nbmaps, nbsizes = oracle.pair_lists(omap)
        # the reference's recipe (hashmap_on_the_fly.py:138-141) with numpy
        res = np.ascontiguousarray(omap.T)
        want_sizes = (res != -1).sum(1)
        k_idx, o_idx = np.nonzero(res != -1)
        want = np.stack([res[k_idx, o_idx], o_idx], 1)
        np.testing.assert_array_equal(nbsizes, want_sizes)
        np.testing.assert_array_equal(nbmaps, want)
        assert nbsizes.sum() == (omap >= 0).sum()
        im, om = oracle.build_masks(n_in, n_out, nbmaps, nbsizes)
        kvol = omap.shape[1]
        base = np.concatenate([[0], np.cumsum(nbsizes)])
        subm_odd = n_in == n_out and kvol % 2 == 1
        for k in range(kvol):
            seg = nbmaps[base[k]:base[k + 1]]
            if subm_odd and k == kvol // 2:
                assert (im[k * n_in:(k + 1) * n_in] == -1).all()
                continue
            pos = np.arange(len(seg))
            np.testing.assert_array_equal(im[k * n_in + seg[:, 0]], pos)
            np.testing.assert_array_equal(om[k * n_out + seg[:, 1]], pos)
            assert (im[k * n_in:(k + 1) * n_in] >= 0).sum() == len(seg)
            assert (om[k * n_out:(k + 1) * n_out] >= 0).sum() == len(seg)
        a, q = oracle.exclusive_scan_quantified(nbsizes)
        np.testing.assert_array_equal(a, base)
        np.testing.assert_array_equal(q, np.concatenate([[0], np.cumsum((nbsizes + 127) // 128 * 128)]))


def test_empty_and_single_voxel():
    one = np.array([[0, 3, 3, 3]], np.int32)
    m = oracle.kmap_subm(one, 3)
    assert m.shape == (128, 27) and m[0, 13] == 0 and (m >= 0).sum() == 1
    omap, oc = oracle.kmap_downsample(one, 2, 2, 0)
    assert oc.tolist() == [[0, 1, 1, 1]] and (omap >= 0).sum() == 1
    empty = np.zeros((0, 4), np.int32)
    m = oracle.kmap_subm(empty, 3, coords_max=[0, 0, 0, 0])
    assert m.shape == (0, 27)


def test_hash_golden_value_and_dictionary():
    # value produced by the compiled reference hash_cpu (backend/hash/hash_cpu.cpp)
    assert int(oracle.hash_cpu([[0, 1, 2, 3]])[0]) == 321218472033932309
    rng = RNG(17)
    tgt = rng.integers(1, 1 << 60, 1000)
    qry = np.concatenate([tgt[::3], rng.integers(1, 1 << 60, 100)])
    got = oracle.hash_query_cpu(qry, tgt, np.arange(1000))
    d = {}
    for i, t in enumerate(tgt.tolist()):
        d.setdefault(t, i + 1)
    want = np.array([d.get(q, 0) for q in qry.tolist()])
    np.testing.assert_array_equal(got, want)


def test_cpu_backend_recipe_equals_exact_map():
    rng = RNG(18)
    coords = random_coords(rng, 2000, (30, 30, 30), batch=2)
    nb, sz = oracle.kmap_cpu_backend(coords, 3)
    want_nb, want_sz = oracle.pair_lists(oracle.kmap_subm(coords, 3))
    np.testing.assert_array_equal(sz, want_sz)
    np.testing.assert_array_equal(nb, want_nb)


def test_negative_lower_bound_follows_the_torch_expression():
    """hashmap_on_the_fly.py:39-43 stores a true division into an int tensor; the oracle's
    bound must round the same way (toward zero), checked by evaluating that expression."""
    import torch
    rng = np.random.default_rng(11)
    for _ in range(20):
        coords = rng.integers(-40, 40, (50, 4)).astype(np.int32)
        ks = rng.integers(1, 5, 3)
        st = rng.integers(1, 4, 3)
        pd = rng.integers(0, 3, 3)
        cmin_t = torch.from_numpy(coords).min(0).values
        cmin_t[1:] = torch.div(cmin_t[1:] - 2 * torch.from_numpy(pd) + (torch.from_numpy(ks) - 1),
                               torch.from_numpy(st))
        got, _ = oracle.downsample_bounds(coords, ks, st, pd, allow_negative=True)
        np.testing.assert_array_equal(got, cmin_t.numpy())
    # with the flag off the bound is zero and negative candidates are dropped
    got, _ = oracle.downsample_bounds(coords, ks, st, pd)
    assert got.tolist() == [0, 0, 0, 0]


def test_strided_outputs_at_negative_coordinates_are_the_valid_candidates():
    """Brute force over every (input, offset): the output set with allow_negative is exactly
    the candidates inside [coords_min, coords_max]."""
    rng = np.random.default_rng(12)
    coords = np.unique(rng.integers(-9, 9, (120, 4)).astype(np.int32), axis=0)
    coords[:, 0] = np.abs(coords[:, 0]) % 2
    coords = np.unique(coords, axis=0)
    for ks, st, pd in [(2, 2, 0), (3, 2, 1), (3, 1, 1), (2, 3, 0)]:
        cmin, cmax = oracle.downsample_bounds(coords, ks, st, pd, allow_negative=True)
        want = set()
        for b, x, y, z in coords.tolist():
            for dx in range(ks):
                for dy in range(ks):
                    for dz in range(ks):
                        num = (x + pd - dx, y + pd - dy, z + pd - dz)
                        if any(v % st for v in num):
                            continue
                        o = tuple(v // st for v in num)
                        if all(cmin[a + 1] <= o[a] <= cmax[a + 1] for a in range(3)):
                            want.add((b,) + o)
        _, out = oracle.kmap_downsample(coords, ks, st, pd, allow_negative=True)
        assert [tuple(r) for r in out.tolist()] == sorted(want)


@pytest.mark.parametrize("ks,st", [(3, 2), (3, 1), (3, 3), (5, 2)])
def test_generative_map_equals_dense_transposed_convolution(ks, st):
    """y[o] = sum_k x[i] W[k] with i*s = o + offset_k is conv_transpose3d with the kernel
    flipped and padding (ks-1)/2; inputs are kept away from the border so that the clamp of
    the generated coordinates does not act."""
    import torch
    rng = np.random.default_rng(ks * 10 + st)
    ext = 6
    cells = np.stack(np.unravel_index(rng.choice(ext ** 3, 40, replace=False), (ext,) * 3), 1)
    coords = np.concatenate([np.zeros((40, 1), np.int32), cells.astype(np.int32) + 2], 1)
    big = (ext + 4) * st + ks
    omap, out_coords = oracle.kmap_generative(coords, ks, st, (1, big, big, big))
    cin, cout = 3, 4
    x = rng.standard_normal((40, cin)).astype(np.float32)
    w = rng.standard_normal((ks ** 3, cin, cout)).astype(np.float32)
    y = oracle.conv_implicit_gemm(x, w, omap, len(out_coords))
    dense = torch.zeros(1, cin, ext + 4, ext + 4, ext + 4, dtype=torch.float64)
    dense[0, :, coords[:, 1], coords[:, 2], coords[:, 3]] = torch.from_numpy(x.T).double()
    # weight k applies to offset (dx,dy,dz), x fastest; conv_transpose3d wants [cin, cout, kx, ky, kz]
    wt = torch.from_numpy(w).double().reshape(ks, ks, ks, cin, cout).permute(3, 4, 2, 1, 0)
    wt = torch.flip(wt, dims=(2, 3, 4))
    full = torch.nn.functional.conv_transpose3d(dense, wt, stride=st, padding=(ks - 1) // 2)[0]
    got = np.zeros(tuple(full.shape[1:]) + (cout,))
    got[out_coords[:, 1], out_coords[:, 2], out_coords[:, 3]] = y
    np.testing.assert_allclose(got, full.permute(1, 2, 3, 0).numpy(), rtol=1e-4, atol=1e-4)


def test_generative_coordinates_are_clamped_and_unique():
    coords = np.array([[0, 0, 0, 0], [0, 3, 3, 3], [1, 3, 0, 1]], np.int32)
    out = oracle.upsample_generative_coords(coords, 3, 2, (2, 6, 6, 6))
    assert out[:, 1:].min() == 0 and out[:, 1:].max() == 5
    assert len(np.unique(out, axis=0)) == len(out)
    key = ((out[:, 0].astype(np.int64) * 8 + out[:, 1]) * 8 + out[:, 2]) * 8 + out[:, 3]
    assert (np.diff(key) > 0).all()
    # voxel (0,0,0): offsets -1..1 around 0 clamp to {0,1}^3 -> 8 cells of batch 0 near the origin
    near = out[(out[:, 0] == 0) & (out[:, 1:] <= 1).all(1)]
    assert len(near) == 8
