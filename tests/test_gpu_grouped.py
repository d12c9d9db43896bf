"""GPU parity of the grouped form of the implicit-GEMM dataflow (tsmi_map_group_rows,
tsmi_conv_implicit_gemm_grouped): the rows of a 3x3x3 map counting-sorted, inside windows, by the
kernel planes they use, and the convolution over that copy with its tiles started heaviest first.

The grouping is integer work: checked exactly against a numpy restatement of its definition (the
order of rows with equal keys and of tiles with equally many offsets is not fixed, so sets and
sortedness are compared, not raw positions).  The convolution computes the sums of the plain
implicit GEMM row by row: compared bit for bit with it, and with the CPU oracle at 1e-2 (fp16) /
3e-2 (bf16) / 1e-4 (fp32) of the RMS of the oracle's output."""
import numpy as np
import pytest
import torch

import oracle
from helpers import lidar_like_coords, random_coords, rel_rms

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-2, torch.bfloat16: 3e-2, torch.float32: 1e-4}


@pytest.fixture(scope="module")
def mods():
    from torchsparse_amd import backend
    from torchsparse_amd.nn import functional as F
    return backend, F


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def _has_copy(backend, omap):
    """Whether the library holds a grouped copy of this very tensor (ids of dead tensors recur)."""
    hit = backend._grouped_of.get(id(omap))
    return hit is not None and hit[0]() is omap


def _keys(valid):
    """Sort key of every row of a [n, 27] validity matrix: rank of the number of offsets its
    occupied outer planes span << 6 | plane bits (the first digit of an offset runs fastest)."""
    k = np.arange(27)
    digit = (k % 3, (k // 3) % 3, k // 9)
    planes = np.zeros(len(valid), np.int64)
    for axis in range(3):
        planes |= valid[:, digit[axis] == 0].any(1).astype(np.int64) << (2 * axis)
        planes |= valid[:, digit[axis] == 2].any(1).astype(np.int64) << (2 * axis + 1)
    ext = [1 + ((planes >> (2 * a)) & 1) + ((planes >> (2 * a + 1)) & 1) for a in range(3)]
    span = ext[0] * ext[1] * ext[2]
    rank = np.searchsorted(np.array([1, 2, 3, 4, 6, 8, 9, 12, 18, 27]), span)
    return (rank << 6) | planes


def _check_grouping(backend, omap_np, n_rows, window):
    g = backend.grouped_map(dev(omap_np), n_rows, window)
    padded = -(-n_rows // window) * window
    assert g.padded == padded
    grouped, row_of = g.grouped.cpu().numpy(), g.row_of.cpu().numpy()
    masks64, order64, order128 = g.masks64.cpu().numpy(), g.order64.cpu().numpy(), g.order128.cpu().numpy()
    assert grouped.shape == (padded, 27) and row_of.shape == (padded,)
    valid = omap_np[:n_rows] >= 0
    key = _keys(valid)
    bits = (valid.astype(np.int64) << np.arange(27)).sum(1)
    for w0 in range(0, padded, window):
        rows = row_of[w0:w0 + window]
        real = rows[rows >= 0]
        # every row of the window once, the padding positions behind them
        np.testing.assert_array_equal(np.sort(real), np.arange(w0, min(w0 + window, n_rows)))
        assert (rows[len(real):] == -1).all()
        assert (np.diff(key[real]) >= 0).all()  # keys ascend inside the window
    ok = row_of >= 0
    np.testing.assert_array_equal(grouped[ok], omap_np[row_of[ok]])
    assert (grouped[~ok] == -1).all()
    # unions of the offsets of every 64 positions
    pos_bits = np.where(ok, bits[np.maximum(row_of, 0)], 0)
    want64 = np.bitwise_or.reduce(pos_bits.reshape(-1, 64), axis=1)
    np.testing.assert_array_equal(masks64.astype(np.int64), want64)
    want128 = np.bitwise_or.reduce(pos_bits.reshape(-1, 128), axis=1)
    for order, want in ((order64, want64), (order128, want128)):
        t = len(want)
        run = -(-t // 8)
        assert order.shape == (8 * run,)
        cost = np.array([bin(int(v)).count("1") for v in want])
        listed = order[order >= 0]
        np.testing.assert_array_equal(np.sort(listed), np.arange(t))  # every tile once
        for c in range(8):
            mine = order[c::8]
            tiles = mine[mine >= 0]
            assert (mine[len(tiles):] == -1).all()
            # the tiles of run c, heaviest first
            np.testing.assert_array_equal(np.sort(tiles), np.arange(c * run, min((c + 1) * run, t)))
            assert (np.diff(cost[tiles]) <= 0).all()
    return g


@pytest.mark.parametrize("n,window", [(1, 128), (127, 128), (128, 128), (129, 256), (5000, 1024),
                                      (20000, 8192), (8192, 8192), (8193, 8192), (30000, 4096)])
def test_rows_are_grouped_by_the_planes_they_use(mods, n, window):
    backend, F = mods
    rng = np.random.default_rng(n + window)
    coords = lidar_like_coords(rng, n) if n >= 5000 else random_coords(rng, n, (12, 12, 6))
    coords = coords[np.lexsort((coords[:, 3], coords[:, 2], coords[:, 1], coords[:, 0]))]
    omap = oracle.kmap_subm(coords, 3)
    _check_grouping(backend, omap, len(coords), window)


def test_grouping_refuses_other_maps_and_windows(mods):
    backend, F = mods
    omap = dev(np.full((256, 8), -1, np.int32))
    with pytest.raises(ValueError, match="3x3x3"):
        backend.grouped_map(omap, 200)
    omap = dev(np.full((256, 27), -1, np.int32))
    for window in (0, 64, 200, 8192 + 128):
        with pytest.raises(ValueError, match="window"):
            backend.grouped_map(omap, 200, window)
    with pytest.raises(ValueError, match="rows"):
        backend.grouped_map(omap, 300)


@pytest.mark.parametrize("cin,cout,dtype", [(32, 32, torch.float16), (96, 96, torch.float16),
                                            (128, 96, torch.float16), (64, 64, torch.bfloat16),
                                            (16, 48, torch.float16), (32, 32, torch.float32),
                                            (256, 256, torch.float16), (24, 40, torch.float16)])
def test_grouped_convolution_equals_the_plain_one_and_the_oracle(mods, cin, cout, dtype, monkeypatch):
    backend, F = mods
    rng = np.random.default_rng(cin * 1000 + cout)
    n_target = 70000 if cout >= 128 else 36000  # 256 columns: only maps of 65536 rows or more are grouped
    coords = lidar_like_coords(rng, n_target, extent=(700, 700, 40))
    coords = coords[np.lexsort((coords[:, 3], coords[:, 2], coords[:, 1], coords[:, 0]))]
    n = len(coords)
    assert n >= (65536 if cout >= 128 else 32768)
    omap_np = oracle.kmap_subm(coords, 3)
    omap = dev(omap_np)
    torch.manual_seed(cin + cout)
    x = torch.randn(n, cin, device="cuda", dtype=dtype)
    w = (torch.randn(27, cin, cout, device="cuda") * (2.0 / (27 * cin)) ** 0.5).to(dtype)
    bias = torch.randn(cout, device="cuda", dtype=dtype)
    res = torch.randn(n, cout, device="cuda", dtype=dtype)
    monkeypatch.setattr(backend, "igemm_group_rows", "always")
    assert backend._grouping_pays(x, 27, cin, cout, n, omap)
    got = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout, bias=bias, residual=res, relu=True)
    assert _has_copy(backend, omap)  # the grouped copy was built and kept with the map
    monkeypatch.setattr(backend, "igemm_group_rows", False)
    plain = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout, bias=bias, residual=res, relu=True)
    assert torch.equal(got, plain)
    f = lambda t: t.detach().float().cpu().numpy()  # noqa: E731
    want = oracle.conv_implicit_gemm(f(x), f(w), omap_np, n) + f(bias)[None, :] + f(res)
    want = np.maximum(want, 0)
    assert rel_rms(f(got), want) < TOL[dtype]


def test_scan_layers_run_over_the_grouped_map(mods, monkeypatch):
    """The public module on the benchmark scan's first level: the same features with and without the
    grouping, and fewer kernel offsets per row tile with it."""
    backend, F = mods
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    coords = torch.from_numpy(lidar_scan_voxels(seed=1)).cuda()
    n = coords.shape[0]
    torch.manual_seed(3)
    layer = spnn.Conv3d(32, 48, 3).cuda().half()
    x = torch.randn(n, 32, device="cuda", dtype=torch.float16)
    monkeypatch.setattr(backend, "igemm_group_rows", "always")
    with torch.no_grad():
        a = layer(ts.SparseTensor(x, coords))
        omap = a._caches.kmaps[((1, 1, 1), (3, 3, 3), (1, 1, 1), (1, 1, 1))]["out_in_map"]
        assert _has_copy(backend, omap)
        g = backend.grouped_map(omap, n)
        monkeypatch.setattr(backend, "igemm_group_rows", False)
        b = layer(ts.SparseTensor(x, coords))
    assert torch.equal(a.feats, b.feats)
    # offsets a 128-row tile multiplies: the union over its rows, grouped against coordinate order
    valid = (omap[:n] >= 0).cpu().numpy()
    pad = (-n) % 128
    natural = np.concatenate([valid, np.zeros((pad, 27), bool)]).reshape(-1, 128, 27).any(1).sum(1).mean()
    masks = g.masks64.cpu().numpy().astype(np.int64)
    grouped = np.array([bin(int(a | b)).count("1") for a, b in zip(masks[0::2], masks[1::2])]).mean()
    assert natural > 24 and grouped < 0.6 * natural


def test_a_map_is_grouped_once_it_has_been_used_often_enough(mods, monkeypatch):
    """With the default setting the copy is built at the group_after_uses-th eligible layer over the
    same map tensor, not before; every call computes the same features."""
    backend, F = mods
    rng = np.random.default_rng(77)
    coords = lidar_like_coords(rng, 36000, extent=(700, 700, 40))
    n = len(coords)
    omap = dev(oracle.kmap_subm(coords, 3))
    x = torch.randn(n, 32, device="cuda", dtype=torch.float16)
    w = torch.randn(27, 32, 32, device="cuda", dtype=torch.float16) * 0.05
    monkeypatch.setattr(backend, "igemm_group_rows", True)
    monkeypatch.setattr(backend, "group_after_uses", 4)
    outs = []
    for use in range(1, 7):
        outs.append(backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, 32))
        assert _has_copy(backend, omap) == (use >= 4)
    for y in outs[1:]:
        assert torch.equal(y, outs[0])
