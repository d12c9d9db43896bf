"""Seeded random sweeps against the oracle: combinations of sizes (1 to 50k voxels), batches,
per-axis kernel sizes / strides / paddings, channel counts, dtypes, dataflows and sort settings
that the hand-picked cases of the other files do not enumerate.  Maps bit-exact; convolutions
to the tolerance of their dtype (relative to the RMS of the expected output)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 3e-2}


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend, nn as spnn
    from torchsparse_amd.nn import functional as F
    return ts, backend, spnn, F


def rel_rms(a, b):
    return float(np.sqrt(((a - b) ** 2).mean()) / (np.sqrt((b ** 2).mean()) + 1e-12))


def _f32(t):
    return t.detach().float().cpu().numpy()


def _cloud(rng, n, batch):
    ext = max(4, int(round((n * rng.uniform(3, 30)) ** (1 / 3))))
    shape = (ext, ext + 1, max(3, ext // 2))
    while np.prod(shape) < n:
        shape = tuple(s * 2 for s in shape)
    return random_coords(rng, n, shape, batch), shape


@pytest.mark.parametrize("seed", range(6))
def test_single_convolutions(mods, seed):
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(1000 + seed)
    for case in range(12):
        n = int(rng.choice([1, 7, 100, 1000, 5000, 17000, 33000]))
        coords, _ = _cloud(rng, n, int(rng.choice([1, 2, 3])))
        n = len(coords)
        ks = tuple(int(v) for v in rng.choice([1, 2, 3], 3)) if rng.random() < 0.5 else (3, 3, 3)
        if all(k == 1 for k in ks):
            ks = (3, 1, 1)
        stride = int(rng.choice([1, 1, 2]))
        cin = int(rng.choice([1, 4, 5, 8, 16, 32, 48, 64, 96, 128, 200, 256]))
        cout = int(rng.choice([3, 16, 19, 32, 64, 96, 128, 160, 256]))
        dtype = [torch.float16, torch.float32, torch.bfloat16][int(rng.integers(0, 3))]
        flow = ["ImplicitGEMM", "ImplicitGEMM", "GatherScatter", "FetchOnDemand"][int(rng.integers(0, 4))]
        ifsort = bool(rng.integers(0, 2)) and flow == "ImplicitGEMM"
        kvol = int(np.prod(ks))
        split = int(rng.integers(1, 4))
        while (split - 1) * -(-kvol // split) >= kvol:
            split -= 1
        pad = tuple((k - 1) // 2 for k in ks) if stride == 1 else (0, 0, 0)
        what = f"seed {seed} case {case}: n={n} ks={ks} s={stride} {cin}->{cout} {dtype} {flow} sort={ifsort}/{split}"
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow, cfg.ifsort, cfg.split_mask_num = getattr(F.Dataflow, flow), ifsort, split
        x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
        w = torch.from_numpy((rng.standard_normal((kvol, cin, cout)) / np.sqrt(cin * kvol)).astype(np.float32))
        w = w.to("cuda", dtype)
        bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
        relu = bool(case % 2)
        with torch.no_grad():
            out = F.conv3d(ts.SparseTensor(x, torch.from_numpy(coords).cuda()), w, ks, bias=bias, stride=stride,
                           padding=pad, config=cfg, activation="relu" if relu else None)
        if stride == 1:
            omap, ocoords = oracle.kmap_subm(coords, ks), coords
        else:
            omap, ocoords = oracle.kmap_downsample(coords, ks, (stride,) * 3, pad)
        n_out = len(ocoords)
        assert np.array_equal(out.coords.cpu().numpy(), ocoords), what
        assert out.feats.shape == (n_out, cout), what
        if n_out == 0:
            continue
        want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap, n_out) + _f32(bias)
        if relu:
            want = np.maximum(want, 0)
        assert rel_rms(_f32(out.feats), want) < TOL[dtype], what


@pytest.mark.parametrize("seed", range(4))
def test_strided_submanifold_transposed_chains_with_backward(mods, seed):
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(2000 + seed)
    for case in range(8):
        n = int(rng.choice([1, 2, 30, 500, 3000, 12000]))
        coords, _ = _cloud(rng, n, int(rng.choice([1, 2])))
        n = len(coords)
        k = int(rng.choice([2, 3]))
        pad = int(rng.choice([0, 1])) if k == 3 else 0
        c0, c1, c2 = (int(rng.choice(v)) for v in ([4, 8, 16, 24, 32], [8, 16, 40, 64], [8, 16, 32]))
        flow = ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"][int(rng.integers(0, 3))]
        ifsort = bool(rng.integers(0, 2)) and flow == "ImplicitGEMM"
        mode = ["hashmap_on_the_fly", "hashmap"][int(rng.integers(0, 2))]
        what = f"seed {seed} case {case}: n={n} k={k} pad={pad} {c0}->{c1}->{c1}->{c2} {flow} sort={ifsort} {mode}"
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow, cfg.ifsort = getattr(F.Dataflow, flow), ifsort
        cfg.split_mask_num = cfg.split_mask_num_bwd = 2
        cfg.kmap_mode = mode
        torch.manual_seed(case)
        down = spnn.Conv3d(c0, c1, k, stride=2, padding=pad, config=cfg).cuda().train()
        mid = spnn.Conv3d(c1, c1, 3, config=cfg).cuda().train()
        up = spnn.Conv3d(c1, c2, k, stride=2, padding=pad, transposed=True, config=cfg).cuda().train()
        x = torch.from_numpy(rng.standard_normal((n, c0)).astype(np.float32)).cuda().requires_grad_(True)
        y1 = down(ts.SparseTensor(x, torch.from_numpy(coords).cuda()))
        if mode == "hashmap":
            oc = (oracle.spdownsample_floor(coords, 2) if k == 2 else
                  oracle.kmap_downsample(coords, (k,) * 3, (2,) * 3, (pad,) * 3)[1])
            omap = oracle.lookup_coords(coords, oc, k, 2)
        else:
            omap, oc = oracle.kmap_downsample(coords, (k,) * 3, (2,) * 3, (pad,) * 3)
        n1 = len(oc)
        assert np.array_equal(y1.coords.cpu().numpy(), oc), what
        if n1 == 0:
            continue
        y3 = up(mid(y1))
        assert torch.equal(y3.coords.cpu(), torch.from_numpy(coords)), what
        g = torch.from_numpy(rng.standard_normal(tuple(y3.feats.shape)).astype(np.float32)).cuda()
        (y3.feats * g).sum().backward()
        smap = oracle.kmap_subm(oc, 3)
        tmap = oracle.transpose_map(omap[:n1], n)
        a1 = oracle.conv_implicit_gemm(_f32(x), _f32(down.kernel), omap, n1)
        a2 = oracle.conv_implicit_gemm(a1, _f32(mid.kernel), smap, n1)
        a3 = oracle.conv_implicit_gemm(a2, _f32(up.kernel), tmap, n)
        d2, dw_up = oracle.conv_backward_implicit_gemm(a2, _f32(up.kernel), tmap, _f32(g))
        d1, dw_mid = oracle.conv_backward_implicit_gemm(a1, _f32(mid.kernel), smap, d2)
        dx, dw_down = oracle.conv_backward_implicit_gemm(_f32(x), _f32(down.kernel), omap, d1)
        for name, got, want in (("out", y3.feats, a3), ("dx", x.grad, dx), ("dw_down", down.kernel.grad, dw_down),
                                ("dw_mid", mid.kernel.grad, dw_mid), ("dw_up", up.kernel.grad, dw_up)):
            assert rel_rms(_f32(got), want) < 1e-4, (what, name)


@pytest.mark.parametrize("seed", range(5))
def test_kernel_maps_of_arbitrary_geometry(mods, seed):
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(3000 + seed)
    for case in range(16):
        n = int(rng.choice([1, 5, 200, 2000, 20000, 50000]))
        batch = int(rng.choice([1, 2, 4]))
        coords, shape = _cloud(rng, n, batch)
        n = len(coords)
        ks = tuple(int(v) for v in rng.choice([1, 2, 3, 5], 3))
        if np.prod(ks) > 64 and rng.random() < 0.7:
            ks = (3, 3, 3)
        st = tuple(int(v) for v in rng.choice([1, 2, 3], 3))
        if rng.random() < 0.35:
            st = (1, 1, 1)
        pd = tuple(int(v) for v in rng.choice([0, 1, 2], 3))
        subm = all(s == 1 for s in st)
        neg = bool(rng.random() < 0.25)
        c = coords.copy()
        if neg:
            c[:, 1:] -= np.array(shape, np.int32) // 2
        sr = None
        if not subm and not neg and rng.random() < 0.5:
            sr = (batch,) + tuple(int(v) for v in (np.array(shape) + rng.integers(0, 3, 3)))
        what = f"seed {seed} case {case}: n={n} b={batch} ks={ks} st={st} pd={pd} range={sr} neg={neg}"
        ts.tensor.set_allow_negative_coordinates(neg)
        try:
            # geometries with more than two outputs per input on average overflow the first table
            # and are built again with room for every candidate
            kmap = F.build_kernel_map(torch.from_numpy(c).cuda(), n, ks, st, pd, mode="hashmap_on_the_fly",
                                      spatial_range=sr)
        finally:
            ts.tensor.set_allow_negative_coordinates(False)
        if subm:
            shifted = c.copy()
            shifted[:, 1:] -= c[:, 1:].min(0)  # the map is translation invariant; the oracle ravels from 0
            want_map, want_coords = oracle.kmap_subm(shifted, ks), c
        else:
            strided = None if sr is None else (sr[0],) + tuple(
                (sr[1 + a] + 2 * pd[a] - (ks[a] - 1) - 1) // st[a] + 1 for a in range(3))
            want_map, want_coords = oracle.kmap_downsample(c, ks, st, pd, spatial_range=strided, allow_negative=neg)
        n_out = len(want_coords)
        got_c, got_m = kmap["coords"].cpu().numpy(), kmap["out_in_map"].cpu().numpy()
        assert np.array_equal(got_c, want_coords), what
        assert got_m.shape == ((n_out + 127) // 128 * 128, int(np.prod(ks))), what
        assert np.array_equal(got_m[:n_out], want_map[:n_out]) and (got_m[n_out:] == -1).all(), what
        if n_out == 0:
            continue
        t = backend.convert_transposed_out_in_map(kmap["out_in_map"], (n + 127) // 128 * 128, n_out).cpu().numpy()
        assert np.array_equal(t[:n], oracle.transpose_map(want_map[:n_out], n)[:n]), what
        pl = backend.pair_lists(kmap["out_in_map"], n, n_out, want_inter=True, want_planar=True)
        nb, sz = oracle.pair_lists(want_map[:n_out])
        assert np.array_equal(pl["nbsizes"].cpu().numpy(), sz), what
        assert np.array_equal(pl["nbmaps_inter"].cpu().numpy(), nb), what


@pytest.mark.parametrize("seed", range(4))
def test_chains_of_equal_strided_layers(mods, seed):
    """One to four equal strided layers, each on the previous one's output coordinates, three
    passes: the later passes take the levels that the first call of the chain computed ahead
    through the occupancy bitmaps.  Coordinates, their order and the output tables against the
    oracle, level by level."""
    from torchsparse_amd import backend
    rng = np.random.default_rng(4000 + seed)
    for _ in range(6):
        ks = tuple(int(v) for v in rng.integers(1, 6, 3))
        st = tuple(int(v) for v in rng.integers(1, 4, 3))
        if all(s == 1 for s in st):
            st = (2, st[1], st[2])
        pd = tuple(int(v) for v in rng.integers(0, 3, 3))
        n = int(rng.choice([1, 7, 300, 5000, 40000]))
        ext = tuple(int(v) for v in rng.choice([3, 17, 64, 300, 2000], 3))
        batch = int(rng.integers(1, 4))
        cols = [rng.integers(0, batch, n)] + [rng.integers(0, e, n) for e in ext]
        coords = np.unique(np.stack(cols, 1).astype(np.int32), axis=0)
        coords = coords[rng.permutation(len(coords))]
        want, c = [], coords
        for _ in range(int(rng.integers(1, 5))):
            c = oracle.kmap_downsample(c, ks, st, pd)[1]
            want.append(c)
            if len(c) == 0:
                break
        for rep in range(3):
            c = torch.from_numpy(coords).cuda()
            for level, w in enumerate(want):
                out, table = backend.downsample_coords(c, ks, st, pd)
                rows = table.query_bxyz(out, (1, 1, 1), (1, 1, 1), (0, 0, 0))[:out.shape[0], 0]
                case = f"ks={ks} st={st} pd={pd} n={len(coords)} ext={ext} pass={rep} level={level}"
                np.testing.assert_array_equal(out.cpu().numpy(), w, err_msg=case)
                np.testing.assert_array_equal(rows.cpu().numpy(), np.arange(len(w)), err_msg=case)
                c = out
