"""The benchmark configurations at their full sizes.

The 20k-voxel fp32 layer is small enough for the CPU oracle to check every output.
The detection backbone (two merged multi-sweep samples) and the ~1M-voxel 256->256
layer are checked through properties that do not need a full CPU run: map symmetry,
sortedness and uniqueness of generated coordinates, batch independence, linearity,
and oracle values on a random sample of output rows."""
import numpy as np
import pytest
import torch

import oracle
from helpers import rel_rms

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    from torchsparse_amd.utils import synthetic
    return ts, backend, spnn, F, synthetic


def _rows_expected(x, w, omap_rows):
    """sum_k X[map[i,k]] W[k] for the given map rows, float64 accumulation."""
    out = np.zeros((omap_rows.shape[0], w.shape[2]), dtype=np.float64)
    for k in range(w.shape[0]):
        m = omap_rows[:, k]
        ok = m >= 0
        if ok.any():
            out[ok] += x[m[ok]].astype(np.float64) @ w[k].astype(np.float64)
    return out


def test_single_layer_20k_voxels_fp32_matches_oracle(mods):
    ts, backend, spnn, F, synthetic = mods
    coords = synthetic.uniform_voxels(20000, extent=128, seed=0)
    rng = np.random.default_rng(0)
    feats = rng.standard_normal((20000, 32)).astype(np.float32)
    torch.manual_seed(0)
    layer = spnn.Conv3d(32, 32, 3).cuda()
    x = ts.SparseTensor(torch.from_numpy(feats).cuda(), torch.from_numpy(coords).cuda())
    for flow in (F.Dataflow.ImplicitGEMM, F.Dataflow.GatherScatter, F.Dataflow.FetchOnDemand):
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow = flow
        xi = ts.SparseTensor(x.feats, x.coords)
        y = F.conv3d(xi, layer.kernel, kernel_size=3, padding=1, config=cfg)
        want_map = oracle.kmap_subm(coords, (3, 3, 3))
        key = ((1, 1, 1), (3, 3, 3), (1, 1, 1), (1, 1, 1))
        if flow == F.Dataflow.ImplicitGEMM:
            got_map = xi._caches.kmaps[key]["out_in_map"].cpu().numpy()
            np.testing.assert_array_equal(got_map[:20000], want_map[:20000])
            assert (got_map[20000:] == -1).all() and got_map.shape[0] == 20096
        want = oracle.conv_implicit_gemm(feats, layer.kernel.detach().cpu().numpy(), want_map, 20000)
        assert rel_rms(y.feats.detach().cpu().numpy(), want) < 1e-4, flow
        assert torch.equal(y.coords, x.coords)


def test_detection_backbone_batch_of_two(mods):
    ts, backend, spnn, F, synthetic = mods
    from torchsparse_amd.backbones import VoxelResBackBone8x
    coords_np, spatial_range = synthetic.multisweep_voxels(seed=2)
    n = coords_np.shape[0]
    per_sample = np.bincount(coords_np[:, 0])
    assert len(per_sample) == 2 and per_sample.min() >= 240_000 and n >= 450_000  # ~250k voxels per sample
    torch.manual_seed(1)
    net = VoxelResBackBone8x(in_channels=5).cuda().half().eval()
    feats = torch.randn(n, 5, device="cuda", dtype=torch.float16)
    coords = torch.from_numpy(coords_np).cuda()
    with torch.no_grad():
        both = net(ts.SparseTensor(feats, coords, spatial_range=spatial_range))
        singles = []
        for b in (0, 1):
            sel = coords[:, 0] == b
            c = coords[sel].clone()
            c[:, 0] = 0
            singles.append(net(ts.SparseTensor(feats[sel], c, spatial_range=(1,) + tuple(spatial_range[1:]))))
    for name, out in both.items():
        oc = out.coords.cpu().numpy()
        # generated coordinates: unique, ascending (b, x, y, z) for the strided levels
        assert len(np.unique(oc, axis=0)) == len(oc)
        if name != "x_conv1":
            key = ((oc[:, 0].astype(np.int64) << 54) | (oc[:, 1].astype(np.int64) << 36)
                   | (oc[:, 2].astype(np.int64) << 18) | oc[:, 3].astype(np.int64))
            assert (np.diff(key) > 0).all(), name
        # batch independence: sample b of the batched run == the run on sample b alone
        for b in (0, 1):
            sel = out.coords[:, 0] == b
            got_c = out.coords[sel].clone()
            got_c[:, 0] = 0
            assert torch.equal(got_c, singles[b][name].coords), name
            got, want = out.feats[sel].float().cpu().numpy(), singles[b][name].feats.float().cpu().numpy()
            # same sums; tile shapes and offset splits (so fp16 roundings of the
            # intermediate activations) differ between the two problem sizes
            assert rel_rms(got, want) < 1e-2, (name, b)
    # one strided map of the batched input against the oracle, exactly
    kmap = F.build_kernel_map(coords, n, 3, 2, 1, mode="hashmap_on_the_fly",
                              spatial_range=spatial_range)
    strided = (spatial_range[0],) + tuple((v + 2 - 2 - 1) // 2 + 1 for v in spatial_range[1:])
    assert tuple(kmap["spatial_range"]) == strided
    want_map, want_coords = oracle.kmap_downsample(coords_np, (3, 3, 3), (2, 2, 2), (1, 1, 1),
                                                   spatial_range=strided)
    np.testing.assert_array_equal(kmap["coords"].cpu().numpy(), want_coords)
    got = kmap["out_in_map"].cpu().numpy()
    np.testing.assert_array_equal(got[:len(want_coords)], want_map[:len(want_coords)])


def test_million_voxel_256_channel_layer(mods):
    ts, backend, spnn, F, synthetic = mods
    coords_np = synthetic.sphere_shell_voxels(seed=3)
    n = coords_np.shape[0]
    assert n > 900000
    coords = torch.from_numpy(coords_np).cuda()
    kmap = F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    assert omap.shape == ((n + 127) // 128 * 128, 27)
    m = omap[:n]
    # map properties: centre is the identity, and j is i's neighbour at offset k iff i is
    # j's neighbour at the mirrored offset 26-k
    assert torch.equal(m[:, 13], torch.arange(n, device="cuda", dtype=torch.int32))
    for k in (0, 5, 12):
        i = torch.nonzero(m[:, k] >= 0).squeeze(1)
        j = m[i, k].long()
        assert torch.equal(m[j, 26 - k].long(), i)
    assert (omap[n:] == -1).all()
    # a sample of rows against a dictionary of the coordinates
    rng = np.random.default_rng(5)
    rows = rng.choice(n, 3000, replace=False)
    lut = {tuple(c): i for i, c in enumerate(coords_np.tolist())}
    offs = oracle.kernel_offsets((3, 3, 3))
    got_rows = m[torch.from_numpy(rows).cuda()].cpu().numpy()
    for r, g in zip(rows[:300], got_rows[:300]):
        b, x, y, z = coords_np[r]
        want = [lut.get((b, x + o[0], y + o[1], z + o[2]), -1) for o in offs]
        assert g.tolist() == want

    torch.manual_seed(2)
    x1 = torch.randn(n, 256, device="cuda", dtype=torch.float16)
    w = (torch.rand(27, 256, 256, device="cuda") * 2 - 1).mul_(1 / np.sqrt(256 * 27)).half()
    y1 = backend.conv_forward_implicit_gemm_cuda(x1, w, omap, n, 256)
    # sampled rows against a float64 evaluation of the definition
    want = _rows_expected(x1.float().cpu().numpy(), w.float().cpu().numpy(), got_rows)
    got = y1[torch.from_numpy(rows).cuda()].float().cpu().numpy()
    assert rel_rms(got, want) < 1e-2
    # the same layer over the row-sorted map (the 128 x 256 tiles of a large 256-channel layer
    # in both modes): the rows are the same sums
    ks = F.build_kernel_map(coords, n, 3, 1, 1, mode="hashmap_on_the_fly", ifsort=True)
    ys = backend.conv_forward_implicit_gemm_sorted_cuda(x1, w, ks["reorder_out_in_map"], ks["reduced_sorted_mask"],
                                                        ks["reorder_loc"], n, 256)
    assert rel_rms(ys.float().cpu().numpy(), y1.float().cpu().numpy()) < 1e-3
    del ys, ks
    # linearity in the features (power-of-two scale: exact in fp16)
    x2 = torch.randn(n, 256, device="cuda", dtype=torch.float16)
    y2 = backend.conv_forward_implicit_gemm_cuda(x2, w, omap, n, 256)
    y12 = backend.conv_forward_implicit_gemm_cuda((2 * x1 + x2), w, omap, n, 256)
    lin = 2 * y1.float() + y2.float()
    assert rel_rms(y12.float().cpu().numpy(), lin.cpu().numpy()) < 1e-2
    # weight gradient at this size: the pair-list kernel against an fp32 GEMM of the gathered
    # rows (hipBLASLt through torch: an independent implementation) for a few offsets, and
    # the input gradient's adjoint identity <conv(x), g> = <x, dgrad(g)>
    g1 = torch.randn(n, 256, device="cuda", dtype=torch.float16)
    lists = backend.wgrad_pair_lists(omap, n)
    dw = backend.conv_backward_wgrad_pairs_cuda(g1, x1, lists, 0)
    assert dw.shape == (27, 256, 256)
    for k in (0, 13, 22):
        out_rows = torch.nonzero(m[:, k] >= 0).squeeze(1)
        in_rows = m[out_rows, k].long()
        want_k = x1[in_rows].float().t() @ g1[out_rows].float()
        assert rel_rms(dw[k].float().cpu().numpy(), want_k.cpu().numpy()) < 1e-2, k
    assert torch.equal(dw, backend.conv_backward_wgrad_pairs_cuda(g1, x1, lists, 0))
    map_bwd = backend.convert_transposed_out_in_map(omap, omap.shape[0], n)
    dx = backend.conv_forward_implicit_gemm_cuda(g1, w.transpose(1, 2).contiguous(), map_bwd, n, 256)
    lhs = (y1.float() * g1.float()).sum().item()
    rhs = (x1.float() * dx.float()).sum().item()
    assert abs(lhs - rhs) < 2e-2 * max(abs(lhs), (y1.float().norm() * g1.float().norm()).item() * 1e-2)
    # the three dataflows agree at this size
    cfg_rows = torch.from_numpy(rows).cuda()
    for flow in (F.Dataflow.FetchOnDemand, F.Dataflow.GatherScatter):
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow = flow
        xi = ts.SparseTensor(x1, coords)
        y = F.conv3d(xi, w, kernel_size=3, padding=1, config=cfg).feats
        assert rel_rms(y[cfg_rows].float().cpu().numpy(), want) < 1e-2, flow


def _strided(spatial_range, ks, st, pd):
    return (spatial_range[0],) + tuple((spatial_range[a + 1] + 2 * pd[a] - (ks[a] - 1) - 1) // st[a] + 1
                                       for a in range(3))


def test_detection_backbone_every_layer_against_the_oracle(mods):
    """The fused detection backbone on one multi-sweep sample cropped to at most 80k voxels: every
    kernel map (the submanifold maps of the four levels, the three k3 s2 maps with paddings 1, 1
    and (0, 1, 1), the (3, 1, 1) s(2, 1, 1) map) and every generated coordinate level bit for bit
    against the oracle, and every convolution's output against oracle.conv_implicit_gemm fed that
    layer's own fp16 input, bias, shortcut and ReLU included: 1e-2 of the RMS of the oracle's output
    (fp16 storage, fp32 accumulation)."""
    ts, backend, spnn, F, synthetic = mods
    import copy
    from torchsparse_amd.backbones import VoxelResBackBone8x
    from torchsparse_amd.nn.utils import fuse_inference
    coords_np, spatial_range = synthetic.multisweep_voxels(seed=2)
    coords_np = coords_np[coords_np[:, 0] == 0]
    half = 720
    while True:  # a centred square window of the (y, x) plane holding at most 80k voxels
        sel = (np.abs(coords_np[:, 2] - 720) < half) & (np.abs(coords_np[:, 3] - 720) < half)
        if sel.sum() <= 80_000:
            break
        half -= 20
    coords_np = np.ascontiguousarray(coords_np[sel])
    n = coords_np.shape[0]
    assert 40_000 <= n <= 80_000, n
    spatial_range = (1,) + tuple(spatial_range[1:])
    torch.manual_seed(4)
    net = VoxelResBackBone8x(in_channels=5).eval()
    g = torch.Generator().manual_seed(5)
    for m in net.modules():
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.copy_(torch.randn(m.num_features, generator=g) * 0.1)
            m.running_var.copy_(torch.rand(m.num_features, generator=g) * 0.5 + 0.25)
            m.weight.data.copy_(torch.rand(m.num_features, generator=g) + 0.75)
            m.bias.data.copy_(torch.randn(m.num_features, generator=g) * 0.1)
    net = fuse_inference(copy.deepcopy(net.cuda().half()))
    assert not any(isinstance(m, torch.nn.BatchNorm1d) for m in net.modules())  # all folded
    feats = torch.randn(n, 5, device="cuda", dtype=torch.float16)
    coords = torch.from_numpy(coords_np).cuda()

    records = []

    def hook(mod, args, kwargs, output):
        x = args[0]
        res = kwargs.get("residual")
        records.append({"mod": mod, "stride": x.stride, "range": x.spatial_range, "x": x.feats.clone(),
                        "coords": x.coords, "res": None if res is None else res.clone(),
                        "y": output.feats.clone(), "out_coords": output.coords,
                        "out_range": output.spatial_range})

    handles = [m.register_forward_hook(hook, with_kwargs=True)
               for m in net.modules() if isinstance(m, spnn.Conv3d)]
    with torch.no_grad():
        inp = ts.SparseTensor(feats, coords, spatial_range=spatial_range)
        outs = net(inp)
    for h in handles:
        h.remove()
    # 1 stem + 2 blocks x 2, then three stages of (strided + 2 blocks x 2), then the output layer
    assert len(records) == 1 + 4 + 3 * 5 + 1

    f32 = lambda t: t.detach().float().cpu().numpy()  # noqa: E731
    maps = {}  # (input level, kernel, stride) -> (oracle map, oracle output coordinates)
    strided_seen = []
    worst = 0.0
    for i, r in enumerate(records):
        mod = r["mod"]
        ks, st, pd = mod.kernel_size, mod.stride, mod.padding
        c_in = r["coords"].cpu().numpy()
        key = (r["stride"], ks, st)
        if key not in maps:
            if st == (1, 1, 1):
                maps[key] = (oracle.kmap_subm(c_in, ks), c_in)
            else:
                out_range = _strided(r["range"], ks, st, pd)
                assert tuple(r["out_range"]) == out_range
                maps[key] = oracle.kmap_downsample(c_in, ks, st, pd, spatial_range=out_range)
                strided_seen.append((ks, st, pd))
            want_map, want_coords = maps[key]
            got = inp._caches.kmaps[(r["stride"], ks, st, (1, 1, 1))]
            n_out = want_coords.shape[0]
            got_map = got["out_in_map"].cpu().numpy()
            np.testing.assert_array_equal(got_map[:n_out], want_map[:n_out])
            assert (got_map[n_out:] == -1).all()
            np.testing.assert_array_equal(r["out_coords"].cpu().numpy(), want_coords)
        want_map, want_coords = maps[key]
        n_out = want_coords.shape[0]
        want = oracle.conv_implicit_gemm(f32(r["x"]), f32(mod.kernel), want_map, n_out)
        if mod.bias is not None:
            want = want + f32(mod.bias)
        if r["res"] is not None:
            want = want + f32(r["res"])
        if mod.activation == "relu":
            want = np.maximum(want, 0)
        assert r["y"].shape == want.shape
        err = rel_rms(f32(r["y"]), want)
        worst = max(worst, err)
        assert err < 1e-2, (i, ks, st, pd, err)
    assert strided_seen == [((3, 3, 3), (2, 2, 2), (1, 1, 1)), ((3, 3, 3), (2, 2, 2), (1, 1, 1)),
                            ((3, 3, 3), (2, 2, 2), (0, 1, 1)), ((3, 1, 1), (2, 1, 1), (0, 0, 0))]
    assert len(maps) == 8  # four submanifold maps (levels 1, 2, 4, 8) and the four strided ones
    assert outs["out"].coords.shape[0] == maps[((8, 8, 8), (3, 1, 1), (2, 1, 1))][1].shape[0]
    print(f"{n} voxels, worst layer {worst:.2e}")


def test_two_networks_alternating_on_one_stream():
    """A U-Net and a detection backbone take turns on one stream, each forward over a new coordinate
    tensor: what the library learnt from one network (its strided chain, the maps it asks for, the
    map over the caller's rows queued ahead of the check's verdict) must not reach the other's
    results.  Every output bit for bit the one the same network gave on its first forward."""
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd.backbones import SparseResUNet42, VoxelResBackBone8x
    from torchsparse_amd.nn.utils import fuse_inference
    from torchsparse_amd.utils import synthetic
    torch.manual_seed(0)
    rows_u = synthetic.lidar_scan_voxels(seed=1)
    rows_d, range_d = synthetic.multisweep_voxels(seed=2)
    rows_d = rows_d[:120000]
    rows_d = rows_d[np.lexsort((rows_d[:, 3], rows_d[:, 2], rows_d[:, 1], rows_d[:, 0]))]
    unet = fuse_inference(SparseResUNet42(in_channels=4).eval().cuda().half())
    det = fuse_inference(VoxelResBackBone8x(in_channels=5).eval().cuda().half())
    feats_u = torch.randn(len(rows_u), 4, device="cuda", dtype=torch.float16)
    feats_d = torch.randn(len(rows_d), 5, device="cuda", dtype=torch.float16)

    def run(kind):
        with torch.no_grad():
            if kind == "U":
                return unet(ts.SparseTensor(feats_u, torch.from_numpy(rows_u).cuda()))[-1].feats.clone()
            out = det(ts.SparseTensor(feats_d, torch.from_numpy(rows_d).cuda(), spatial_range=range_d))
            return out["out"].feats.clone()

    backend.release_scratch()
    first = {}
    for turn, kind in enumerate("UUUDDDUDUDDUUUDU"):
        got = run(kind)
        if kind in first:
            assert torch.equal(got, first[kind]), (turn, kind)
        else:
            first[kind] = got
    state, = backend._stream_states.values()
    assert state.lookahead_hits >= 2  # (the U-Net's chain was queued ahead again after the other network's turns)
    torch.cuda.synchronize()
