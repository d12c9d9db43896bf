"""Parity of the two headline workloads at their own size: the synthetic 64-beam scan
(lidar_scan_voxels(seed=1), 89,834 voxels).

  layer sweep   the five single layers (submanifold k3 at 32/64/128 channels, strided k2 s2
                64->128, transposed k2 s2 128->64) in fp16, for the three dataflows: kernel
                maps, output coordinates and pair lists bit-exact against the oracle,
                outputs within 1e-2 of RMS of the oracle's double-accumulated sums.
  network       the MinkUNet forward exactly as bench.py runs it (inference form, a fresh
                SparseTensor per forward, the second forward so that the strided levels
                computed ahead are the ones used): all nine kernel maps and five coordinate
                levels bit-exact, every sparse convolution against the oracle fed that
                layer's own fp16 input, and the 19-class output against the whole network
                evaluated on the CPU in fp32 from the unfused parameters.

The method is the reference's tests/python/test_single_layer_conv.py:111-220 (same seeded
inputs through both implementations, outputs compared), at the size the benchmark runs."""
import copy

import numpy as np
import pytest
import torch

import oracle
from helpers import rel_rms

pytestmark = pytest.mark.gpu

FP16_TOL = 1e-2  # max |got - want| / RMS(want), fp16 storage, fp32 accumulation


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    return ts, backend, spnn, F


def _scan_tables(coords):
    """The coordinate levels and kernel maps of a scan as the oracle builds them."""
    levels = {1: coords}
    down = {}
    for s in (1, 2, 4, 8):
        omap, oc = oracle.kmap_downsample(levels[s], 2, 2, 0)
        down[s] = omap
        levels[2 * s] = oc
    subm = {s: oracle.kmap_subm(c, 3) for s, c in levels.items()}
    up = {s: oracle.transpose_map(down[s], levels[s].shape[0]) for s in down}
    return {"levels": levels, "down": down, "subm": subm, "up": up}


@pytest.fixture(scope="module")
def scan():
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    coords = lidar_scan_voxels(seed=1)
    assert 85_000 < coords.shape[0] < 100_000
    return _scan_tables(coords)


def _f32(t):
    return t.detach().float().cpu().numpy()


def _key(level, k, s):
    return ((level,) * 3, (k,) * 3, (s,) * 3, (1, 1, 1))


def _check_pair_products(F, flow, kmap, want_map, n_in, n_out, subm):
    """The pair lists, sizes, masks and scans a pair-list dataflow works from."""
    nb, sz = oracle.pair_lists(want_map[:n_out])
    np.testing.assert_array_equal(kmap["nbsizes"].cpu().numpy(), sz)
    got = kmap["nbmaps"].cpu().numpy()
    if flow == F.Dataflow.FetchOnDemand:
        np.testing.assert_array_equal(got, nb.T)
    else:
        np.testing.assert_array_equal(got, nb)
    a, q = oracle.exclusive_scan_quantified(sz)
    np.testing.assert_array_equal(kmap["nbaddrs"].cpu().numpy(), a)
    np.testing.assert_array_equal(kmap["qnbaddrs"].cpu().numpy(), q)
    im, om = oracle.build_masks(n_in, n_out, nb, sz)
    got_im, got_om = kmap["input_mask"].cpu().numpy(), kmap["output_mask"].cpu().numpy()
    kvol = len(sz)
    if subm:  # the identity offset is left out of both masks, as in the reference
        c = kvol // 2
        assert (got_im[c * n_in:(c + 1) * n_in] == -1).all()
        assert (got_om[c * n_out:(c + 1) * n_out] == -1).all()
        im[c * n_in:(c + 1) * n_in] = -1
        om[c * n_out:(c + 1) * n_out] = -1
    np.testing.assert_array_equal(got_im, im)
    np.testing.assert_array_equal(got_om, om)


SWEEP = [("subm", 32, 32), ("subm", 64, 64), ("subm", 128, 128), ("down", 64, 128), ("up", 128, 64)]


@pytest.mark.parametrize("kind,cin,cout", SWEEP)
def test_layer_sweep_on_the_scan(mods, scan, kind, cin, cout):
    ts, backend, spnn, F = mods
    coords_np = scan["levels"][1]
    n = coords_np.shape[0]
    coords = torch.from_numpy(coords_np).cuda()
    torch.manual_seed(cin * 1000 + cout)
    if kind == "subm":
        want_map, n_in, n_out = scan["subm"][1], n, n
    elif kind == "down":
        want_map, n_in, n_out = scan["down"][1], n, scan["levels"][2].shape[0]
    else:
        want_map, n_in, n_out = scan["up"][1], scan["levels"][2].shape[0], n
    x = torch.randn(n_in, cin, device="cuda", dtype=torch.float16)
    want = None
    for flow in (F.Dataflow.ImplicitGEMM, F.Dataflow.GatherScatter, F.Dataflow.FetchOnDemand):
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow = flow
        torch.manual_seed(7)
        if kind == "subm":
            layer = spnn.Conv3d(cin, cout, 3, config=cfg).cuda().half()
            inp = ts.SparseTensor(x, coords)
        elif kind == "down":
            layer = spnn.Conv3d(cin, cout, 2, stride=2, config=cfg).cuda().half()
            inp = ts.SparseTensor(x, coords)
        else:
            layer = spnn.Conv3d(cin, cout, 2, stride=2, transposed=True, config=cfg).cuda().half()
            lower = spnn.Conv3d(1, 1, 2, stride=2, config=cfg).cuda().half()
            mid = lower(ts.SparseTensor(torch.zeros(n, 1, device="cuda", dtype=torch.float16), coords))
            assert np.array_equal(mid.coords.cpu().numpy(), scan["levels"][2])
            inp = ts.SparseTensor(x, mid.coords, stride=mid.stride)
            inp._caches = mid._caches
        with torch.no_grad():
            out = layer(inp)
        # --- integer products: bit-exact
        if kind == "subm":
            kmap = inp._caches.kmaps[_key(1, 3, 1)]
            np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)
            assert torch.equal(out.coords, coords) and out.stride == (1, 1, 1)
        elif kind == "down":
            kmap = inp._caches.kmaps[_key(1, 2, 2)]
            np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want_map)
            np.testing.assert_array_equal(out.coords.cpu().numpy(), scan["levels"][2])
            assert out.stride == (2, 2, 2)
        else:
            kmap = inp._caches.kmaps[_key(1, 2, 2)]
            np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), scan["down"][1])
            if flow == F.Dataflow.ImplicitGEMM:
                np.testing.assert_array_equal(kmap["out_in_map_t"].cpu().numpy(), want_map)
            assert torch.equal(out.coords, coords) and out.stride == (1, 1, 1)
        if flow != F.Dataflow.ImplicitGEMM:
            # the pair lists are those of the strided map; a transposed layer reads them mirrored
            fwd_map = scan["down"][1] if kind == "up" else want_map
            sizes = (n, scan["levels"][2].shape[0]) if kind != "subm" else (n, n)
            _check_pair_products(F, flow, kmap, fwd_map, sizes[0], sizes[1], kind == "subm")
        # --- features
        if want is None:
            want = oracle.conv_implicit_gemm(_f32(x), _f32(layer.kernel), want_map, n_out)
        assert out.feats.shape == (n_out, cout) and out.feats.dtype == torch.float16
        err = rel_rms(_f32(out.feats), want)
        assert err < FP16_TOL, (kind, cin, cout, flow, err)


# ----------------------------------------------------------------------------- the network


def _randomise_norms(model, seed):
    g = torch.Generator().manual_seed(seed)
    for m in model.modules():
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.1)
            m.running_var.copy_(torch.rand(m.num_features, generator=g) * 0.5 + 0.25)
            m.weight.data.copy_(torch.rand(m.num_features, generator=g) + 0.75)
            m.bias.data.copy_(torch.randn(m.num_features, generator=g) * 0.1)


class _OracleNet:
    """The unfused network evaluated on the CPU: convolutions by the oracle over the oracle's
    maps (fp32 in and out, double accumulation), BatchNorm in evaluation mode and ReLU in
    numpy float32.  Parameters are the fp16 model's, widened."""

    def __init__(self, scan, spnn):
        self.scan, self.spnn = scan, spnn

    def conv(self, mod, x, level):
        w = _f32(mod.kernel)
        ks, st = mod.kernel_size, mod.stride
        if ks == (1, 1, 1):
            y = (x.astype(np.float64) @ w.astype(np.float64)).astype(np.float32)
            out_level = level
        elif mod.transposed:
            out_level = level // st[0]
            m = self.scan["up"][out_level]
            y = oracle.conv_implicit_gemm(x, w, m, self.scan["levels"][out_level].shape[0])
        elif st == (1, 1, 1):
            out_level = level
            y = oracle.conv_implicit_gemm(x, w, self.scan["subm"][level], x.shape[0])
        else:
            out_level = level * st[0]
            y = oracle.conv_implicit_gemm(x, w, self.scan["down"][level],
                                          self.scan["levels"][out_level].shape[0])
        if mod.bias is not None:
            y = y + _f32(mod.bias)
        return y, out_level

    def run(self, mod, x, level):
        from torchsparse_amd.backbones.modules.blocks import SparseResBlock
        spnn = self.spnn
        if isinstance(mod, spnn.Conv3d):
            return self.conv(mod, x, level)
        if isinstance(mod, torch.nn.BatchNorm1d):
            g = _f32(mod.weight) / np.sqrt(_f32(mod.running_var) + mod.eps)
            return (x - _f32(mod.running_mean)) * g + _f32(mod.bias), level
        if isinstance(mod, spnn.ReLU):
            return np.maximum(x, 0), level
        if isinstance(mod, torch.nn.Identity):
            return x, level
        if isinstance(mod, torch.nn.Sequential):
            for child in mod:
                x, level = self.run(child, x, level)
            return x, level
        if isinstance(mod, SparseResBlock):
            a, la = self.run(mod.main, x, level)
            b, _ = self.run(mod.shortcut, x, level)
            return np.maximum(a + b, 0), la
        raise TypeError(type(mod))

    def forward(self, net, head, x):
        skips = [self.run(net.stem, x, 1)]
        for enc in net.encoders:
            skips.append(self.run(enc, *skips[-1]))
        y, level = skips[-1]
        for i, dec in enumerate(net.decoders):
            u, level = self.run(dec["upsample"], y, level)
            assert level == skips[3 - i][1]
            y, level = self.run(dec["fuse"], np.concatenate([u, skips[3 - i][0]], 1), level)
        logits = y.astype(np.float64) @ _f32(head.weight).T.astype(np.float64) + _f32(head.bias)
        return logits.astype(np.float32), y


def test_minkunet_forward_on_the_scan(mods, scan):
    ts, backend, spnn, F = mods
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    coords_np = scan["levels"][1]
    n = coords_np.shape[0]
    coords = torch.from_numpy(coords_np).cuda()
    torch.manual_seed(0)
    feats = torch.randn(n, 4, device="cuda", dtype=torch.float16)
    unfused = SparseResUNet42(in_channels=4).eval()
    _randomise_norms(unfused, 3)
    unfused = unfused.cuda().half()
    model = fuse_inference(copy.deepcopy(unfused))
    head = torch.nn.Linear(96, 19).cuda().half().eval()
    assert backend.downsample_through_grid and backend.downsample_chain_ahead  # bench.py's path

    records = []

    def hook(mod, args, kwargs, output):
        x = args[0]
        res = kwargs.get("residual")
        records.append({"mod": mod, "level": x.stride[0], "x": x.feats.clone(),
                        "res": None if res is None else res.clone(), "y": output.feats.clone(),
                        "out_level": output.stride[0]})

    def step():
        with torch.no_grad():
            x = ts.SparseTensor(feats, coords)
            outs = model(x)
            return x, outs, head(outs[-1].feats)

    backend.release_scratch()
    step()  # the first forward learns the chain of strided layers ...
    step()  # ... the second computes levels 2, 3, 4 ahead in its first strided call ...
    handles = [m.register_forward_hook(hook, with_kwargs=True)
               for m in model.modules() if isinstance(m, spnn.Conv3d)]
    inp, outs, logits = step()  # ... the third queues that call's first half when the stem's map is built
    for h in handles:
        h.remove()
    state, = backend._stream_states.values()
    assert state.ahead_hits == 6, state.ahead_hits  # per forward one strided call computed, three answered ahead
    assert state.lookahead_hits == 1 and state.pending is None  # bench.py's steady state
    # ... and builds the four strided maps and the submanifold maps of levels 2 - 16 on the second
    # stream as soon as the row counts are known (the maps compared below are those)
    assert state.maps_ahead_hits == 8, state.maps_ahead_hits
    assert state.transposed_hits == 0  # (asked for in this forward for the first time: see the end)
    # ... queued behind the chain before its counts had reached the host (the counts stay on the device)
    assert state.maps_early_hits == 1, state.maps_early_hits

    # --- the nine kernel maps and the coordinate levels, bit-exact
    caches = inp._caches
    assert len(caches.kmaps) == 9
    for s in (1, 2, 4, 8, 16):
        got = caches.kmaps[_key(s, 3, 1)]
        np.testing.assert_array_equal(got["out_in_map"].cpu().numpy(), scan["subm"][s])
        np.testing.assert_array_equal(caches.cmaps[(s,) * 3][0].cpu().numpy(), scan["levels"][s])
    for s in (1, 2, 4, 8):
        got = caches.kmaps[_key(s, 2, 2)]
        np.testing.assert_array_equal(got["out_in_map"].cpu().numpy(), scan["down"][s])
        np.testing.assert_array_equal(got["coords"].cpu().numpy(), scan["levels"][2 * s])
        np.testing.assert_array_equal(got["out_in_map_t"].cpu().numpy(), scan["up"][s])
        assert got["sizes"] == (scan["levels"][s].shape[0], scan["levels"][2 * s].shape[0])
    torch.cuda.synchronize()
    for s in (2, 4, 8, 16):
        want = scan["subm"][s][:scan["levels"][s].shape[0]]
        assert backend.map_density(caches.kmaps[_key(s, 3, 1)]["out_in_map"]) == (want >= 0).mean()
    assert backend.map_density(caches.kmaps[_key(1, 3, 1)]["out_in_map"]) is None  # (built before the chain is known)
    for i, out in enumerate(outs):
        level = (1, 2, 4, 8, 16, 8, 4, 2, 1)[i]
        assert out.stride == (level,) * 3
        np.testing.assert_array_equal(out.coords.cpu().numpy(), scan["levels"][level])

    # --- every convolution of the forward against the oracle fed the same fp16 input
    assert len(records) == 49 and sum(r["mod"].kernel_size != (1, 1, 1) for r in records) == 42
    ref = _OracleNet(scan, spnn)
    worst = 0.0
    for i, r in enumerate(records):
        mod = r["mod"]
        want, out_level = ref.conv(mod, _f32(r["x"]), r["level"])
        assert out_level == r["out_level"]
        if r["res"] is not None:
            want = want + _f32(r["res"])
        if mod.activation == "relu":
            want = np.maximum(want, 0)
        got = _f32(r["y"])
        if mod.transposed:  # placed into the left-hand columns of the buffer its level concatenates in
            assert got.shape[1] > want.shape[1]
            got = got[:, :want.shape[1]]
        err = rel_rms(got, want)
        worst = max(worst, err)
        assert err < FP16_TOL, (i, mod, r["level"], err)

    # --- the network output against the fp32 evaluation of the unfused network.  fp16 rounding
    # of 49 layers of activations accumulates: 3e-2 of RMS end to end (each layer alone: 1e-2).
    want_logits, want_last = ref.forward(unfused, head, _f32(feats))
    assert logits.shape == (n, 19)
    e_last = rel_rms(_f32(outs[-1].feats), want_last)
    e_logits = rel_rms(_f32(logits), want_logits)
    print(f"per-layer worst {worst:.2e}, last features {e_last:.2e}, logits {e_logits:.2e}")
    assert e_last < 3e-2 and e_logits < 3e-2, (e_last, e_logits)
    # the forward measured by the benchmark is deterministic: a third run gives the same bits
    inp3, outs3, logits3 = step()
    assert torch.equal(logits3, logits) and torch.equal(outs3[-1].feats, outs[-1].feats)
    # ... in which the launch of the maps queued ahead has also stored the transposed maps of the
    # four strided ones (the forward before asked for them): still the oracle's
    assert state.transposed_hits == 4, state.transposed_hits
    # ... and the pair segments of the three deep maps behind them, on the second stream
    assert state.segments_hits == 3, state.segments_hits
    step()
    assert state.segments_hits == 6 and state.transposed_hits == 8  # ... in every forward from then on
    for s in (1, 2, 4, 8):
        np.testing.assert_array_equal(inp3._caches.kmaps[_key(s, 2, 2)]["out_in_map_t"].cpu().numpy(), scan["up"][s])


def _check_maps(caches, outs, tables):
    """All nine kernel maps and the coordinate levels of one forward, bit for bit."""
    assert len(caches.kmaps) == 9
    for s in (1, 2, 4, 8, 16):
        np.testing.assert_array_equal(caches.kmaps[_key(s, 3, 1)]["out_in_map"].cpu().numpy(), tables["subm"][s])
        np.testing.assert_array_equal(caches.cmaps[(s,) * 3][0].cpu().numpy(), tables["levels"][s])
    for s in (1, 2, 4, 8):
        got = caches.kmaps[_key(s, 2, 2)]
        np.testing.assert_array_equal(got["out_in_map"].cpu().numpy(), tables["down"][s])
        np.testing.assert_array_equal(got["coords"].cpu().numpy(), tables["levels"][2 * s])
        np.testing.assert_array_equal(got["out_in_map_t"].cpu().numpy(), tables["up"][s])
    for i, out in enumerate(outs):
        level = (1, 2, 4, 8, 16, 8, 4, 2, 1)[i]
        np.testing.assert_array_equal(out.coords.cpu().numpy(), tables["levels"][level])


def test_minkunet_over_alternating_scans(mods, scan):
    """One fused model over scan A, scan B (another scene, other row counts at every level), scan A
    again, each as a new coordinate tensor: what the first scan left behind (the levels computed
    ahead, the maps queued ahead, the learnt chain of strided layers, cached buffers sized for A)
    must not reach B's result, nor B's reach A's.  Every forward: the nine maps and five levels bit
    for bit against the oracle's for THAT scan, and the output against the whole network evaluated
    on the CPU (3e-2 of RMS end to end, as in the test above); A's output after B equals A's
    output before B bit for bit."""
    ts, backend, spnn, F = mods
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    tables = {"A": scan, "B": _scan_tables(lidar_scan_voxels(seed=7, n_azimuth=1500, n_boxes=18))}
    sizes = {k: [t["levels"][s].shape[0] for s in (1, 2, 4, 8, 16)] for k, t in tables.items()}
    assert all(a != b for a, b in zip(sizes["A"], sizes["B"])), sizes
    assert sizes["B"][0] > 40_000
    unfused = SparseResUNet42(in_channels=4).eval()
    _randomise_norms(unfused, 3)
    unfused = unfused.cuda().half()
    model = fuse_inference(copy.deepcopy(unfused))
    head = torch.nn.Linear(96, 19).cuda().half().eval()
    torch.manual_seed(11)
    feats = {k: torch.randn(sizes[k][0], 4, device="cuda", dtype=torch.float16) for k in tables}
    want = {}
    for k, t in tables.items():
        want[k] = _OracleNet(t, spnn).forward(unfused, head, _f32(feats[k]))[0]

    def step(k):
        with torch.no_grad():
            x = ts.SparseTensor(feats[k], torch.from_numpy(tables[k]["levels"][1]).cuda())
            outs = model(x)
            return x, outs, head(outs[-1].feats)

    backend.release_scratch()
    logits = {}
    for turn, k in enumerate("AAABABBA"):
        x, outs, got = step(k)
        _check_maps(x._caches, outs, tables[k])
        assert got.shape == (sizes[k][0], 19)
        err = rel_rms(_f32(got), want[k])
        assert err < 3e-2, (turn, k, err)
        if k in logits:
            assert torch.equal(got, logits[k]), (turn, k)
        logits[k] = got
    state, = backend._stream_states.values()
    # from the third forward on the maps are queued before the counts of their levels are known on
    # the host, with room for an eighth more rows than the forward before had: enough for A after
    # A, B after B and B (the smaller scan) after A; A after B outgrows it, twice, and has its
    # maps queued once the counts are there
    assert sizes["A"][1] > sizes["B"][1] + sizes["B"][1] // 8 + 1024, sizes
    assert state.maps_early_hits == 4, state.maps_early_hits


def test_minkunet_over_small_clouds_of_changing_size(mods):
    """The look-ahead machinery (chain on the second stream, maps queued with the row counts still
    on the device and room for an eighth more rows than the forward before) over clouds of a few
    hundred voxels whose sizes jump up and down from one forward to the next, several batches among
    them: every forward's nine maps and five levels bit for bit the oracle's, every output that of
    the same cloud when it was first seen (to 2e-3 of its RMS: the form a wide layer takes may differ)."""
    ts, backend, spnn, F = mods
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from helpers import random_coords
    rng = np.random.default_rng(21)

    def cloud(n, shape, batch):
        c = random_coords(rng, n, shape, batch)
        return c[np.lexsort((c[:, 3], c[:, 2], c[:, 1], c[:, 0]))]
    clouds = [cloud(300, (64, 64, 32), 1), cloud(2500, (96, 96, 32), 2), cloud(120, (48, 48, 32), 1),
              cloud(4000, (128, 96, 48), 3)]
    tables = [_scan_tables(c) for c in clouds]
    assert all(t["levels"][16].shape[0] > 0 for t in tables)
    torch.manual_seed(8)
    model = fuse_inference(SparseResUNet42(in_channels=4).eval().cuda().half())
    feats = [torch.randn(len(c), 4, device="cuda", dtype=torch.float16) for c in clouds]
    backend.release_scratch()
    first = {}
    for turn, k in enumerate([0, 0, 0, 1, 1, 2, 3, 3, 0, 2, 1, 3]):
        with torch.no_grad():
            x = ts.SparseTensor(feats[k], torch.from_numpy(clouds[k]).cuda())
            outs = model(x)
        _check_maps(x._caches, outs, tables[k])
        got = _f32(outs[-1].feats)
        if k in first:
            # (not bit for bit: once a map's pairs have been counted - from the third forward on - a
            # wide layer may take the other of its two forms, which rounds its sums differently)
            assert rel_rms(got, first[k]) < 2e-3, (turn, k)
        else:
            first[k] = got
    state, = backend._stream_states.values()
    assert state.maps_early_hits >= 4, state.maps_early_hits  # (forwards whose levels fit the room given)
    torch.cuda.synchronize()


def test_new_tensors_whose_rows_do_not_ascend_between_tensors_whose_rows_do(mods):
    """What is queued ahead of a new tensor's verdict (its strided chain, the maps over the chain's
    levels, the map over the rows themselves) is queued for any tensor; rows that turn out not to
    ascend take the table builders, the queued chain serves them all the same, the map searched
    over them is dropped.  Shuffled and sorted clouds in turn through one U-Net: the submanifold
    map and the first strided map of every forward bit for bit the oracle's for THAT order of rows,
    outputs those of the same forwards with nothing queued ahead of the verdict."""
    ts, backend, spnn, F = mods
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    rows = lidar_scan_voxels(seed=5, n_azimuth=700, n_boxes=8)
    rng = np.random.default_rng(6)
    perm = rng.permutation(len(rows))
    clouds = {"s": rows, "u": rows[perm]}
    torch.manual_seed(9)
    model = fuse_inference(SparseResUNet42(in_channels=4).eval().cuda().half())
    base = torch.randn(len(rows), 4, device="cuda", dtype=torch.float16)
    feats = {"s": base, "u": base[torch.from_numpy(perm).cuda()]}
    want_maps = {k: (oracle.kmap_subm(c, 3), oracle.kmap_downsample(c, 2, 2, 0)) for k, c in clouds.items()}
    order = "sssuusuussus"

    def sweep():
        outs = []
        backend.release_scratch()
        for k in order:
            with torch.no_grad():
                x = ts.SparseTensor(feats[k], torch.from_numpy(clouds[k]).cuda())
                y = model(x)[-1].feats
            kmaps = x._caches.kmaps
            np.testing.assert_array_equal(kmaps[_key(1, 3, 1)]["out_in_map"].cpu().numpy(), want_maps[k][0])
            np.testing.assert_array_equal(kmaps[_key(1, 2, 2)]["out_in_map"].cpu().numpy(), want_maps[k][1][0])
            np.testing.assert_array_equal(kmaps[_key(1, 2, 2)]["coords"].cpu().numpy(), want_maps[k][1][1])
            outs.append(_f32(y))
        return outs

    backend.coords_check_overlap = False
    try:
        plain = sweep()
    finally:
        backend.coords_check_overlap = True
    ahead = sweep()
    for turn, (a, b) in enumerate(zip(ahead, plain)):
        assert rel_rms(a, b) < 2e-3, (turn, order[turn])
    # the same cloud in the other order of rows: the same features, row for row
    assert rel_rms(ahead[3], ahead[0][perm]) < 2e-3
    assert not backend._root_maps
    torch.cuda.synchronize()
