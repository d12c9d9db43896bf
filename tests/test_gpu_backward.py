"""GPU parity of the convolution backward (input and weight gradients) against the CPU
oracle.  Tolerances relative to the RMS of the expected gradient: 1e-4 fp32, 1e-2 fp16,
3e-2 bf16 (fp32 accumulation; the oracle gets the inputs already rounded to the I/O type)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 3e-2}


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    return ts, backend, spnn, F


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def _f32(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("cin,cout", [(32, 32), (64, 96), (96, 64), (128, 128), (16, 40), (5, 7), (4, 32), (200, 72)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_wgrad_and_dgrad_kernels_match_oracle(mods, cin, cout, dtype):
    _, backend, _, F = mods
    rng = np.random.default_rng(cin * 100 + cout)
    coords = random_coords(rng, 1800, (22, 20, 12))
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
    w = torch.from_numpy(rng.uniform(-0.1, 0.1, (27, cin, cout)).astype(np.float32)).to("cuda", dtype)
    dy = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    map_bwd = backend.convert_transposed_out_in_map(omap, (n + 127) // 128 * 128, n)
    dw = backend.conv_backward_wgrad_implicit_gemm_cuda(dy, x, map_bwd, n)
    dx = backend.conv_forward_implicit_gemm_cuda(dy, w.transpose(1, 2).contiguous(), map_bwd, n, cin)
    want_dx, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), _f32(w), omap.cpu().numpy(), _f32(dy))
    assert dw.shape == (27, cin, cout) and dw.dtype == dtype
    assert rel_rms(_f32(dw), want_dw) < TOL[dtype]
    assert rel_rms(_f32(dx), want_dx) < TOL[dtype]


@pytest.mark.parametrize("n", [1, 31, 32, 33, 500, 5000])
def test_wgrad_ragged_row_counts(mods, n):
    _, backend, _, F = mods
    rng = np.random.default_rng(n)
    coords = random_coords(rng, n, (30, 30, 10))
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    x = torch.from_numpy(rng.standard_normal((n, 24)).astype(np.float32)).cuda()
    dy = torch.from_numpy(rng.standard_normal((n, 40)).astype(np.float32)).cuda()
    w = np.zeros((27, 24, 40), np.float32)
    map_bwd = backend.convert_transposed_out_in_map(omap, (n + 127) // 128 * 128, n)
    dw = backend.conv_backward_wgrad_implicit_gemm_cuda(dy, x, map_bwd, n)
    _, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), w, omap.cpu().numpy(), _f32(dy))
    assert rel_rms(_f32(dw), want_dw) < 1e-4


def _expected_pair_lists(omap, n_rows):
    """Per offset: (map value, row) for every row with an entry, ascending rows, padded
    with (-1, -1) to a multiple of 32."""
    pairs, seg = [], [0]
    for k in range(omap.shape[1]):
        rows = np.nonzero(omap[:n_rows, k] >= 0)[0]
        blk = np.full(((len(rows) + 31) // 32 * 32, 2), -1, np.int32)
        blk[:len(rows), 0] = omap[rows, k]
        blk[:len(rows), 1] = rows
        pairs.append(blk)
        seg.append(seg[-1] + len(blk) // 32)
    return np.concatenate(pairs), np.array(seg, np.int32)


@pytest.mark.parametrize("n,geom", [(1, (3, 1, 1)), (33, (3, 1, 1)), (700, (3, 1, 1)), (5000, (3, 1, 1)),
                                    (3000, (2, 2, 0)), (3000, (3, 2, 1)), (400, (5, 1, 2))])
def test_wgrad_pair_lists_are_exact(mods, n, geom):
    _, backend, _, F = mods
    rng = np.random.default_rng(n + geom[0])
    coords = random_coords(rng, n, (30, 30, 10))
    kmap = F.build_kernel_map(dev(coords), len(coords), *geom, mode="hashmap_on_the_fly")
    n_out = kmap["sizes"][1]
    omap = kmap["out_in_map"].cpu().numpy()
    got = backend.wgrad_pair_lists(kmap["out_in_map"], n_out)
    want_pairs, want_seg = _expected_pair_lists(omap, n_out)
    np.testing.assert_array_equal(got["seg_steps"].cpu().numpy(), want_seg)
    np.testing.assert_array_equal(got["nbsizes"].cpu().numpy(), (omap[:n_out] >= 0).sum(0))
    np.testing.assert_array_equal(got["pairs"].cpu().numpy()[:len(want_pairs)], want_pairs)
    assert got["pairs"].shape[0] >= len(want_pairs)


@pytest.mark.parametrize("cin,cout", [(32, 32), (64, 96), (96, 64), (128, 128), (16, 40), (8, 8), (200, 72),
                                      (256, 160), (384, 32)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_wgrad_over_pair_lists_matches_oracle(mods, cin, cout, dtype):
    _, backend, _, F = mods
    rng = np.random.default_rng(cin * 100 + cout)
    coords = random_coords(rng, 1800, (22, 20, 12))
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
    dy = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    lists = backend.wgrad_pair_lists(omap, n)
    assert backend.wgrad_pairs_supported(x, dy)
    dw = backend.conv_backward_wgrad_pairs_cuda(dy, x, lists, 0)
    w = np.zeros((27, cin, cout), np.float32)
    _, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), w, omap.cpu().numpy(), _f32(dy))
    assert dw.shape == (27, cin, cout) and dw.dtype == dtype
    assert rel_rms(_f32(dw), want_dw) < TOL[dtype]
    # the same lists with the roles of the two columns exchanged: the transposed gradient
    dw_t = backend.conv_backward_wgrad_pairs_cuda(x, dy, lists, 1)
    assert rel_rms(_f32(dw_t), want_dw.transpose(0, 2, 1)) < TOL[dtype]
    # and the same sums as the map form, run twice: bit-identical results
    again = backend.conv_backward_wgrad_pairs_cuda(dy, x, lists, 0)
    assert torch.equal(dw, again)


@pytest.mark.parametrize("n,geom", [(1, (3, 1, 1)), (31, (3, 1, 1)), (257, (3, 1, 1)), (9000, (3, 1, 1)),
                                    (4000, (2, 2, 0)), (300, (5, 1, 2))])
def test_wgrad_over_pair_lists_row_counts_and_geometries(mods, n, geom):
    """Few rows (ranges without work), strided maps (n_in != n_out), a 125-offset kernel."""
    _, backend, _, F = mods
    rng = np.random.default_rng(n)
    coords = random_coords(rng, n, (30, 30, 10))
    n_in = len(coords)
    kmap = F.build_kernel_map(dev(coords), n_in, *geom, mode="hashmap_on_the_fly")
    n_out = kmap["sizes"][1]
    omap = kmap["out_in_map"]
    x = torch.from_numpy(rng.standard_normal((n_in, 24)).astype(np.float32)).cuda()
    dy = torch.from_numpy(rng.standard_normal((n_out, 40)).astype(np.float32)).cuda()
    dw = backend.conv_backward_wgrad_pairs_cuda(dy, x, backend.wgrad_pair_lists(omap, n_out), 0)
    w = np.zeros((omap.shape[1], 24, 40), np.float32)
    _, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), w, omap.cpu().numpy()[:n_out], _f32(dy))
    assert rel_rms(_f32(dw), want_dw) < 1e-4


def test_wgrad_over_pair_lists_rejects_odd_widths(mods):
    _, backend, _, F = mods
    rng = np.random.default_rng(0)
    coords = random_coords(rng, 200, (10, 10, 10))
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    lists = backend.wgrad_pair_lists(kmap["out_in_map"], n)
    x = torch.randn(n, 5, device="cuda", dtype=torch.float16)
    dy = torch.randn(n, 16, device="cuda", dtype=torch.float16)
    assert not backend.wgrad_pairs_supported(x, dy)
    with pytest.raises(ValueError, match="multiples of"):
        backend.conv_backward_wgrad_pairs_cuda(dy, x, lists, 0)


@pytest.mark.parametrize("geom", [(3, 1, 1), (2, 2, 0), (3, 2, 1)])
@pytest.mark.parametrize("transpose", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_backward_over_gather_scatter_pair_lists(mods, geom, transpose, dtype):
    """conv_backward_gather_scatter_cuda fills both gradients in place from the dataflow's
    own pair lists; the oracle's pair-list backward is the reference CPU kernel's restatement."""
    _, backend, _, F = mods
    rng = np.random.default_rng(sum(geom) + transpose)
    coords = random_coords(rng, 1500, (20, 18, 12))
    n_in = len(coords)
    kmap = F.build_kernel_map(dev(coords), n_in, *geom, mode="hashmap_on_the_fly",
                              dataflow=F.Dataflow.GatherScatter)
    n_out = kmap["sizes"][1]
    kvol, cin, cout = kmap["out_in_map"].shape[1], 24, 40
    n_x, n_y = (n_out, n_in) if transpose else (n_in, n_out)
    x = torch.from_numpy(rng.standard_normal((n_x, cin)).astype(np.float32)).to("cuda", dtype)
    dy = torch.from_numpy(rng.standard_normal((n_y, cout)).astype(np.float32)).to("cuda", dtype)
    w = torch.from_numpy(rng.uniform(-0.1, 0.1, (kvol, cin, cout)).astype(np.float32)).to("cuda", dtype)
    nbmaps = kmap["nbmaps"].int()
    dx, dw = torch.empty(0, device="cuda", dtype=dtype), torch.empty(0, device="cuda", dtype=dtype)
    backend.conv_backward_gather_scatter_cuda(x, dx, dy, w, dw, nbmaps, kmap["nbsizes"].cpu(), transpose)
    want_dx, want_dw = oracle.conv_backward_gather_scatter(
        _f32(x), _f32(w), nbmaps.cpu().numpy(), kmap["nbsizes"].cpu().numpy(), _f32(dy), transpose)
    assert dx.shape == x.shape and dw.shape == w.shape
    assert rel_rms(_f32(dx), want_dx) < TOL[dtype]
    assert rel_rms(_f32(dw), want_dw) < TOL[dtype]


@pytest.mark.parametrize("ifsort", [False, True])
def test_training_kernel_map_holds_the_backward_products(mods, ifsort):
    _, backend, _, F = mods
    rng = np.random.default_rng(3)
    coords = random_coords(rng, 2500, (20, 18, 12))
    n_in = len(coords)
    kmap = F.build_kernel_map(dev(coords), n_in, 3, 2, 1, mode="hashmap_on_the_fly", training=True,
                              ifsort=ifsort, split_mask_num=1, split_mask_num_bwd=3)
    n_out = kmap["sizes"][1]
    omap = kmap["out_in_map"].cpu().numpy()
    bwd = kmap["out_in_map_bwd"].cpu().numpy()
    assert bwd.shape == ((n_in + 127) // 128 * 128, 27)
    want = np.full_like(bwd, -1)
    rows, ks = np.nonzero(omap[:n_out] >= 0)
    want[omap[rows, ks], ks] = rows
    np.testing.assert_array_equal(bwd, want)
    if not ifsort:
        assert kmap["reorder_out_in_map_bwd"] is None
        return
    loc = kmap["reorder_loc_bwd"].cpu().numpy()
    assert loc.shape == (3, bwd.shape[0])
    for s in range(3):
        assert sorted(loc[s].tolist()) == list(range(bwd.shape[0]))
    ro = kmap["reorder_out_in_map_bwd"].cpu().numpy()
    for s in range(3):
        np.testing.assert_array_equal(ro[:, s * 9:(s + 1) * 9], bwd[loc[s]][:, s * 9:(s + 1) * 9])
    assert kmap["reduced_sorted_mask_bwd_wgrad"].shape == (3, (bwd.shape[0] - 1) // 64 + 1)
    assert kmap["reduced_sorted_mask_bwd_dgrad"].shape == (3, (bwd.shape[0] - 1) // 128 + 1)


@pytest.mark.parametrize("geom", [(3, 1, 1), (2, 2, 0), (3, 2, 1), (2, 1, 0)])
@pytest.mark.parametrize("flow", ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"])
def test_autograd_through_conv3d_matches_oracle(mods, geom, flow):
    """loss = sum(conv(x) * g): x.grad and kernel.grad for every dataflow and geometry,
    including the bias gradient."""
    ts, backend, spnn, F = mods
    k, s, pad = geom
    rng = np.random.default_rng(k * 10 + s)
    coords = random_coords(rng, 900, (16, 14, 10))
    n = len(coords)
    cin, cout = 16, 24
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).cuda().requires_grad_(True)
    torch.manual_seed(k)
    layer = spnn.Conv3d(cin, cout, k, stride=s, padding=pad, bias=True).cuda()
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = getattr(F.Dataflow, flow)
    layer._config = cfg
    inp = ts.SparseTensor(x, dev(coords))
    out = F.conv3d(inp, layer.kernel, kernel_size=k, bias=layer.bias, stride=s, padding=pad, config=cfg)
    g = torch.from_numpy(rng.standard_normal(tuple(out.feats.shape)).astype(np.float32)).cuda()
    (out.feats * g).sum().backward()
    if s == 1:
        omap = oracle.kmap_subm(coords, k)
    else:
        omap, _ = oracle.kmap_downsample(coords, k, s, pad)
    want_dx, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), _f32(layer.kernel), omap, _f32(g))
    assert rel_rms(_f32(x.grad), want_dx) < 1e-4
    assert rel_rms(_f32(layer.kernel.grad), want_dw) < 1e-4
    assert rel_rms(_f32(layer.bias.grad), _f32(g).sum(0)) < 1e-4


def test_autograd_through_transposed_conv_and_relu_residual(mods):
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(11)
    coords = random_coords(rng, 1200, (20, 18, 10))
    n = len(coords)
    torch.manual_seed(0)
    down = spnn.Conv3d(8, 12, 2, stride=2).cuda()
    up = spnn.Conv3d(12, 6, 2, stride=2, transposed=True).cuda()
    x = torch.from_numpy(rng.standard_normal((n, 8)).astype(np.float32)).cuda().requires_grad_(True)
    res = torch.from_numpy(rng.standard_normal((n, 6)).astype(np.float32)).cuda().requires_grad_(True)
    inp = ts.SparseTensor(x, dev(coords))
    mid = down(inp)
    out = F.conv3d(mid, up.kernel, kernel_size=2, stride=2, transposed=True, residual=res, activation="relu")
    g = torch.from_numpy(rng.standard_normal((n, 6)).astype(np.float32)).cuda()
    (out.feats * g).sum().backward()
    # oracle: chain rule by hand
    omap, ocoords = oracle.kmap_downsample(coords, 2, 2, 0)
    n_mid = len(ocoords)
    mid_np = oracle.conv_implicit_gemm(_f32(x), _f32(down.kernel), omap, n_mid)
    tmap = oracle.transpose_map(omap[:n_mid], n)
    pre = oracle.conv_implicit_gemm(mid_np, _f32(up.kernel), tmap, n) + _f32(res)
    gpre = _f32(g) * (pre > 0)
    dmid, dw_up = oracle.conv_backward_implicit_gemm(mid_np, _f32(up.kernel), tmap, gpre)
    dx, dw_down = oracle.conv_backward_implicit_gemm(_f32(x), _f32(down.kernel), omap, dmid)
    assert rel_rms(_f32(res.grad), gpre) < 1e-4
    assert rel_rms(_f32(up.kernel.grad), dw_up) < 1e-4
    assert rel_rms(_f32(down.kernel.grad), dw_down) < 1e-4
    assert rel_rms(_f32(x.grad), dx) < 1e-4


@pytest.mark.parametrize("flow", ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"])
def test_only_bias_and_residual_trainable(mods, flow):
    """Frozen features and kernel, trainable bias and residual: the reference adds both with
    torch ops, so both get a gradient (d loss / d bias = column sums of the ReLU-masked g)."""
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(3)
    coords = random_coords(rng, 700, (14, 12, 9))
    n = len(coords)
    torch.manual_seed(2)
    layer = spnn.Conv3d(16, 8, 3, bias=True).cuda()
    layer.kernel.requires_grad_(False)
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = getattr(F.Dataflow, flow)
    x = torch.from_numpy(rng.standard_normal((n, 16)).astype(np.float32)).cuda()
    res = torch.from_numpy(rng.standard_normal((n, 8)).astype(np.float32)).cuda().requires_grad_(True)
    out = F.conv3d(ts.SparseTensor(x, dev(coords)), layer.kernel, kernel_size=3, bias=layer.bias,
                   residual=res, activation="relu", config=cfg)
    g = torch.from_numpy(rng.standard_normal((n, 8)).astype(np.float32)).cuda()
    (out.feats * g).sum().backward()
    pre = oracle.conv_implicit_gemm(_f32(x), _f32(layer.kernel), oracle.kmap_subm(coords, 3), n) \
        + _f32(layer.bias) + _f32(res)
    assert rel_rms(_f32(out.feats), np.maximum(pre, 0)) < 1e-4
    gpre = _f32(g) * (pre > 0)
    assert layer.kernel.grad is None
    assert rel_rms(_f32(res.grad), gpre) < 1e-4
    assert rel_rms(_f32(layer.bias.grad), gpre.sum(0)) < 1e-4


@pytest.mark.parametrize("geom", [(3, 1, 1), (2, 2, 0), (3, 2, 1)])
@pytest.mark.parametrize("splits", [(1, 1), (3, 2)])
@pytest.mark.parametrize("cin,cout", [(16, 24), (32, 64)])
def test_sorted_configuration_runs_the_input_gradient_over_sorted_products(mods, geom, splits, cin, cout,
                                                                           monkeypatch):
    """ifsort: the input gradient goes through the mask-sorted transposed map (both the packed
    and the as-stored weight forms) and equals the oracle's; a transposed convolution uses
    the strided map's forward sort products."""
    ts, backend, spnn, F = mods
    k, s, pad = geom
    calls = []
    real = backend.conv_dgrad_implicit_gemm_sorted_cuda
    monkeypatch.setattr(backend, "conv_dgrad_implicit_gemm_sorted_cuda",
                        lambda *a, **kw: (calls.append(a[2].shape), real(*a, **kw))[1])
    rng = np.random.default_rng(k * 7 + s)
    coords = random_coords(rng, 1500, (18, 14, 12))
    n = len(coords)
    cfg = F.conv_config.get_default_conv_config()
    cfg.ifsort, cfg.split_mask_num, cfg.split_mask_num_bwd = True, splits[0], splits[1]
    torch.manual_seed(k)
    layer = spnn.Conv3d(cin, cout, k, stride=s, padding=pad).cuda()
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).cuda().requires_grad_(True)
    out = F.conv3d(ts.SparseTensor(x, dev(coords)), layer.kernel, kernel_size=k, stride=s, padding=pad,
                   config=cfg, training=True)
    g = torch.from_numpy(rng.standard_normal(tuple(out.feats.shape)).astype(np.float32)).cuda()
    if s == 1:
        omap = oracle.kmap_subm(coords, k)
        (out.feats * g).sum().backward()
        want_dx, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), _f32(layer.kernel), omap, _f32(g))
        assert len(calls) == 1
    else:
        # strided convolution followed by its transposed twin on the same (sorted) map
        up = spnn.Conv3d(cout, cin, k, stride=s, transposed=True).cuda()
        back = F.conv3d(out, up.kernel, kernel_size=k, stride=s, padding=pad, transposed=True, config=cfg,
                        training=True)
        g = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).cuda()
        (back.feats * g).sum().backward()
        omap, ocoords = oracle.kmap_downsample(coords, k, s, pad)
        n_mid = len(ocoords)
        mid = oracle.conv_implicit_gemm(_f32(x), _f32(layer.kernel), omap, n_mid)
        tmap = oracle.transpose_map(omap[:n_mid], n)
        dmid, dw_up = oracle.conv_backward_implicit_gemm(mid, _f32(up.kernel), tmap, _f32(g))
        want_dx, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), _f32(layer.kernel), omap, dmid)
        assert rel_rms(_f32(up.kernel.grad), dw_up) < 1e-4
        assert len(calls) == 2
    assert rel_rms(_f32(x.grad), want_dx) < 1e-4
    assert rel_rms(_f32(layer.kernel.grad), want_dw) < 1e-4
