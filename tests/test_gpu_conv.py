"""GPU parity of the convolution dataflows against the CPU oracle.

Tolerances (relative to the RMS of the expected output): 1e-4 for fp32, 1e-2 for
fp16 / bf16 with fp32 accumulation — the bar the north star sets.  The oracle is fed
the inputs already rounded to the I/O type, so only accumulation order and the final
rounding differ."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import lidar_like_coords, random_coords, rel_rms

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 3e-2}
GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    return ts, backend, spnn, F


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def _case(rng, n, cin, cout, kvol, dtype, wscale=None):
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
    bound = wscale or 1.0 / np.sqrt(cin * kvol)
    w = torch.from_numpy(rng.uniform(-bound, bound, (kvol, cin, cout)).astype(np.float32)).to("cuda", dtype)
    return x, w


def _f32(t):
    return t.detach().float().cpu().numpy()


CHANNELS = [(32, 32), (64, 64), (128, 128), (4, 32), (5, 16), (16, 16), (96, 96), (128, 96),
            (24, 40), (32, 19), (7, 3), (192, 256), (96, 160), (64, 128), (256, 130)]


@pytest.mark.parametrize("cin,cout", CHANNELS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
def test_implicit_gemm_matches_oracle(mods, cin, cout, dtype):
    _, backend, _, F = mods
    rng = np.random.default_rng(cin * 1000 + cout)
    coords = random_coords(rng, 1500, (20, 20, 12))
    kmap = F.build_kernel_map(dev(coords), len(coords), 3, 1, 1, mode="hashmap_on_the_fly")
    x, w = _case(rng, len(coords), cin, cout, 27, dtype)
    y = backend.conv_forward_implicit_gemm_cuda(x, w, kmap["out_in_map"], len(coords), cout)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), kmap["out_in_map"].cpu().numpy(), len(coords))
    assert y.dtype == dtype and y.shape == (len(coords), cout)
    assert rel_rms(_f32(y), want) < TOL[dtype]


@pytest.mark.parametrize("n", [1, 15, 16, 17, 63, 64, 65, 129, 255, 257, 700])
def test_implicit_gemm_ragged_row_counts(mods, n):
    _, backend, _, F = mods
    rng = np.random.default_rng(n)
    coords = random_coords(rng, n, (9, 9, 9))
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    x, w = _case(rng, n, 32, 64, 27, torch.float16)
    bias = torch.from_numpy(rng.standard_normal(64).astype(np.float32)).to("cuda", torch.float16)
    y = backend.conv_forward_implicit_gemm_cuda(x, w, kmap["out_in_map"], n, 64, bias=bias)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), kmap["out_in_map"].cpu().numpy(), n) + _f32(bias)
    assert rel_rms(_f32(y), want) < 1e-2


@pytest.mark.parametrize("cin,cout", [(1, 16), (3, 20), (4, 32), (5, 16), (8, 64), (8, 8), (6, 48), (4, 96)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n,ks", [(1, 3), (127, 3), (129, 3), (3000, 3), (900, 2), (700, (3, 1, 3)), (500, 5)])
def test_few_input_channels_all_row_counts_and_kernels(mods, cin, cout, dtype, n, ks):
    """Layers of at most 8 input channels (16-bit types, up to 64 output channels, kernel
    volumes up to 64) run the densely packed kernel; wider outputs and 5^3 kernels the general
    one.  Bias, residual and ReLU included; compared with the oracle and, for the epilogue,
    with the same sums formed by torch."""
    _, backend, _, F = mods
    rng = np.random.default_rng(cin * 100 + cout + n)
    coords = random_coords(rng, n, (20, 18, 12))
    stride = 1
    kmap = F.build_kernel_map(dev(coords), n, ks, stride, 0, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    x, w = _case(rng, n, cin, cout, omap.shape[1], dtype)
    y = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap.cpu().numpy(), n)
    assert y.shape == (n, cout) and y.dtype == dtype
    assert rel_rms(_f32(y), want) < TOL[dtype]
    bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
    res = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    y2 = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout, bias=bias, residual=res, relu=True)
    want2 = np.maximum(want + _f32(bias) + _f32(res), 0)
    assert rel_rms(_f32(y2), want2) < TOL[dtype]


@pytest.mark.parametrize("geom", [(3, 1, 1), (2, 2, 0), (3, 2, 1), (5, 1, 2), (2, 1, 0)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_all_dataflows_agree_with_oracle(mods, geom, dtype):
    ts, _, _, F = mods
    ks, stride, pad = geom
    rng = np.random.default_rng(7 + ks * 10 + stride)
    coords = random_coords(rng, 2000, (24, 24, 12), batch=2)
    cin, cout = 32, 48
    x, w = _case(rng, len(coords), cin, cout, ks ** 3, dtype)
    bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
    if stride == 1:
        omap, n_out = oracle.kmap_subm(coords, ks), len(coords)
    else:
        omap, oc = oracle.kmap_downsample(coords, ks, stride, pad)
        n_out = len(oc)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap, n_out) + _f32(bias)
    configs = []
    for dataflow in (F.Dataflow.ImplicitGEMM, F.Dataflow.GatherScatter, F.Dataflow.FetchOnDemand):
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow = dataflow
        configs.append(cfg)
    for split in (1, 3, 5):
        length = -(-ks ** 3 // split)
        if length > 32 or (split - 1) * length >= ks ** 3:  # 32 offsets per mask word, no empty split
            continue
        cfg = F.conv_config.get_default_conv_config()
        cfg.ifsort, cfg.split_mask_num = True, split
        configs.append(cfg)
    for cfg in configs:
        inp = ts.SparseTensor(x, dev(coords))
        out = F.conv3d(inp, w, ks, bias=bias, stride=stride, padding=pad, config=cfg)
        assert out.feats.shape == (n_out, cout)
        assert rel_rms(_f32(out.feats), want) < TOL[dtype], cfg
        assert out.stride == (stride,) * 3


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_transposed_all_dataflows(mods, dtype):
    ts, _, spnn, F = mods
    rng = np.random.default_rng(33)
    coords = random_coords(rng, 3000, (32, 32, 16))
    omap, oc = oracle.kmap_downsample(coords, 2, 2, 0)
    map_t = oracle.transpose_map(omap, len(coords))
    cin, cout = 64, 32
    for dataflow, ifsort, split in [(F.Dataflow.ImplicitGEMM, False, 1), (F.Dataflow.ImplicitGEMM, True, 1),
                                    (F.Dataflow.ImplicitGEMM, True, 2), (F.Dataflow.GatherScatter, False, 1),
                                    (F.Dataflow.FetchOnDemand, False, 1)]:
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow, cfg.ifsort, cfg.split_mask_num = dataflow, ifsort, split
        down = spnn.Conv3d(8, cin, 2, stride=2, config=cfg).to("cuda", dtype)
        up = spnn.Conv3d(cin, cout, 2, stride=2, transposed=True, config=cfg).to("cuda", dtype)
        x0 = torch.from_numpy(rng.standard_normal((len(coords), 8)).astype(np.float32)).to("cuda", dtype)
        mid = down(ts.SparseTensor(x0, dev(coords)))
        np.testing.assert_array_equal(mid.coords.cpu().numpy(), oc)
        out = up(mid)
        assert out.stride == (1, 1, 1) and out.coords.data_ptr() == mid._caches.cmaps[(1, 1, 1)][0].data_ptr()
        want = oracle.conv_implicit_gemm(_f32(mid.feats), _f32(up.kernel), map_t, len(coords))
        assert rel_rms(_f32(out.feats), want) < TOL[dtype], (dataflow, ifsort, split)


def test_golden_reference_cpu_vectors(mods):
    """The fixtures written by the compiled reference CPU convolution."""
    _, backend, _, F = mods
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    for name in ("subm3", "down2", "down3", "up2"):
        x, w, y = g[name + "_x"], g[name + "_w"], g[name + "_y"]
        omap = g[name + "_map"]
        if name == "up2":
            omap = oracle.transpose_map(omap, y.shape[0])
        got = backend.conv_forward_implicit_gemm_cuda(dev(x, torch.float32), dev(w, torch.float32),
                                                      dev(omap), y.shape[0], w.shape[2])
        assert rel_rms(_f32(got), y) < 1e-4, name


def _dense_reference(coords, feats, filters, k, s, shape):
    dense = torch.zeros(1, feats.shape[1], *shape, dtype=torch.float64)
    for c, f in zip(coords, feats):
        dense[0, :, c[1], c[2], c[3]] = torch.from_numpy(f.astype(np.float64))
    f_t = torch.from_numpy(filters.astype(np.float64))
    if k % 2 == 1:
        weight, pad = f_t.permute(4, 3, 2, 1, 0).contiguous(), (k - 1) // 2
    else:
        weight, pad = f_t.permute(4, 3, 0, 1, 2).contiguous(), 0
        dense = torch.nn.functional.pad(dense, (0, k - 1) * 3)
    return torch.nn.functional.conv3d(dense, weight, stride=s, padding=pad).numpy()


@pytest.mark.parametrize("kmap_mode", ["hashmap_on_the_fly", "hashmap"])
def test_single_layer_vs_dense_conv(mods, kmap_mode):
    """The reference's own unit test (tests/test.py:11-41): fp16, 20 voxels in 5^3,
    IC16 -> OC32, k in {2,3,5} x s in {1,2,3}; mean |diff| <= 1e-4 and max relative
    diff <= 1e-2 on average over the cases."""
    ts, _, spnn, F = mods
    acc_adiff = acc_rdiff = 0.0
    count = 0
    for k in (2, 3, 5):
        for s in (1, 2, 3):
            rng = np.random.default_rng(0)
            shape, IC, OC = (5, 5, 5), 16, 32
            coords = random_coords(rng, 20, shape)
            feats = rng.uniform(-1, 1, (20, IC)).astype(np.float16)
            filters = rng.uniform(-1, 1, (k, k, k, IC, OC)).astype(np.float16)
            cfg = F.conv_config.get_default_conv_config()
            cfg.kmap_mode = kmap_mode
            pad = (k - 1) // 2 if k % 2 == 1 else 0
            layer = spnn.Conv3d(IC, OC, k, s, pad, config=cfg).to("cuda").half()
            layer.kernel.data[:] = torch.from_numpy(filters.reshape(-1, IC, OC)).cuda()
            out = layer(ts.SparseTensor(dev(feats, torch.float16), dev(coords)))
            oc = out.coords.cpu().numpy()
            ref = _dense_reference(coords, feats.astype(np.float32), filters.astype(np.float32), k, s, shape)
            want = np.stack([ref[0, :, c[1], c[2], c[3]] for c in oc])
            got = _f32(out.feats)
            assert rel_rms(got, want) <= 1e-2, (k, s)  # the per-case bound: fp16 storage, fp32 sums
            acc_adiff += np.abs(got - want).sum() / want.size
            acc_rdiff += np.abs(got - want).max() / np.abs(got).mean()
            count += 1
    assert acc_adiff / count <= 1e-2  # fp16 rounding of sums of ~2000 unit-scale products
    assert acc_rdiff / count <= 1e-2


def test_pointwise_and_module_init(mods):
    ts, _, spnn, F = mods
    torch.manual_seed(0)
    layer = spnn.Conv3d(32, 64, 1, bias=True).to("cuda")
    assert layer.kernel.shape == (32, 64)
    assert float(layer.kernel.detach().abs().max()) <= 1 / np.sqrt(32) + 1e-6
    x = torch.randn(100, 32, device="cuda")
    coords = dev(random_coords(np.random.default_rng(1), 100, (8, 8, 8)))
    out = layer(ts.SparseTensor(x, coords))
    torch.testing.assert_close(out.feats, x @ layer.kernel + layer.bias)
    strided_pw = spnn.Conv3d(8, 8, 1, stride=2)
    assert strided_pw.kernel.shape == (1, 8, 8)
    assert spnn.Conv3d(4, 4, 3, padding=0).padding == (1, 1, 1)
    assert spnn.Conv3d(4, 4, 3, stride=2, padding=0).padding == (0, 0, 0)
    assert spnn.Conv3d(4, 4, (3, 1, 1), stride=(2, 1, 1), padding=0).padding == (0, 0, 0)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,cin,cout", [(0, 16, 8), (1, 32, 64), (100, 32, 64), (4097, 128, 96), (3000, 384, 256),
                                        (2500, 96, 19), (700, 5, 7)])
def test_pointwise_convolution_without_autograd_runs_the_fused_kernel(mods, dtype, n, cin, cout, monkeypatch):
    """Outside autograd a 1x1x1 convolution goes through the implicit-GEMM kernels over the
    identity map with bias, residual and ReLU in the epilogue; same result as the fp32 product."""
    ts, backend, spnn, F = mods
    calls = []
    real = backend.conv_pointwise_cuda
    monkeypatch.setattr(backend, "conv_pointwise_cuda", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    rng = np.random.default_rng(n + cin)
    coords = dev(random_coords(rng, n, (20, 20, 12))) if n else torch.zeros((0, 4), dtype=torch.int32, device="cuda")
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
    torch.manual_seed(cin)
    layer = spnn.Conv3d(cin, cout, 1, bias=True).to("cuda", dtype)
    layer.bias.data.normal_()
    res = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    with torch.no_grad():
        plain = layer(ts.SparseTensor(x, coords))
        fused = F.conv3d(ts.SparseTensor(x, coords), layer.kernel, 1, bias=layer.bias, residual=res,
                         activation="relu")
    assert len(calls) == 2 and plain.feats.shape == (n, cout) and plain.feats.dtype == dtype
    if n == 0:
        return
    want = x.float() @ layer.kernel.float() + layer.bias.float()
    assert rel_rms(_f32(plain.feats), _f32(want)) < TOL[dtype]
    assert rel_rms(_f32(fused.feats), _f32(torch.relu(want + res.float()))) < TOL[dtype]
    # with autograd the product stays torch's, and its gradients flow
    out = layer(ts.SparseTensor(x, coords))
    assert len(calls) == 2 and out.feats.requires_grad
    assert rel_rms(_f32(out.feats.detach()), _f32(want)) < TOL[dtype]


@pytest.mark.parametrize("flow", ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"])
@pytest.mark.parametrize("ifsort", [False, True])
def test_strided_convolution_without_outputs(mods, flow, ifsort):
    """A voxel at the origin has no output under kernel 3, stride 2, padding 0 (the output
    range is empty): every dataflow, sorted or not, returns an empty tensor and the gradients
    of an empty output are zero."""
    ts, backend, spnn, F = mods
    if ifsort and flow != "ImplicitGEMM":
        pytest.skip("pair-list dataflows never sort")
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow, cfg.ifsort, cfg.split_mask_num = getattr(F.Dataflow, flow), ifsort, 3
    coords = torch.tensor([[0, 0, 0, 0], [1, 1, 0, 1]], dtype=torch.int32, device="cuda")
    layer = spnn.Conv3d(8, 16, 3, stride=2, padding=0, bias=True, config=cfg).cuda().half()
    x = torch.randn(2, 8, device="cuda", dtype=torch.float16)
    with torch.no_grad():
        out = layer(ts.SparseTensor(x, coords))
    assert out.feats.shape == (0, 16) and out.coords.shape == (0, 4)
    xg = x.clone().requires_grad_(True)
    out = layer(ts.SparseTensor(xg, coords))
    out.feats.sum().backward()
    assert out.feats.shape == (0, 16)
    assert float(xg.grad.abs().max()) == 0.0 and float(layer.kernel.grad.abs().max()) == 0.0


@pytest.mark.parametrize("flow", ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"])
@pytest.mark.parametrize("n", [1, 2])
def test_strided_convolution_with_as_many_outputs_as_inputs(mods, flow, n):
    """Kernel 3, stride 2, padding 1 on one or two voxels gives as many outputs as inputs, but
    the centre offset is not the identity: the pair-list dataflows must not take the map for a
    submanifold one (the reference tells by the sizes and odd volume alone)."""
    ts, backend, spnn, F = mods
    coords = np.array([[0, 2, 3, 1], [0, 2, 3, 2]][:n], np.int32)
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = getattr(F.Dataflow, flow)
    torch.manual_seed(n)
    layer = spnn.Conv3d(8, 16, 3, stride=2, padding=1, config=cfg).cuda()
    x = torch.randn(n, 8, device="cuda", requires_grad=True)
    out = layer(ts.SparseTensor(x, dev(coords)))
    omap, ocoords = oracle.kmap_downsample(coords, 3, 2, 1)
    assert len(ocoords) == n and np.array_equal(out.coords.cpu().numpy(), ocoords)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(layer.kernel), omap, n)
    assert rel_rms(_f32(out.feats), want) < 1e-4
    g = torch.randn_like(out.feats)
    (out.feats * g).sum().backward()
    want_dx, want_dw = oracle.conv_backward_implicit_gemm(_f32(x), _f32(layer.kernel), omap, _f32(g))
    assert rel_rms(_f32(x.grad), want_dx) < 1e-4
    assert rel_rms(_f32(layer.kernel.grad), want_dw) < 1e-4


def test_kmap_cache_and_errors(mods):
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(5)
    coords = dev(random_coords(rng, 500, (12, 12, 12)))
    x = torch.randn(500, 16, device="cuda").half()
    conv_a = spnn.Conv3d(16, 16, 3).cuda().half()
    conv_b = spnn.Conv3d(16, 8, 3).cuda().half()
    inp = ts.SparseTensor(x, coords)
    y = conv_a(inp)
    assert len(inp._caches.kmaps) == 1 and y._caches is inp._caches
    z = conv_b(y)
    assert len(inp._caches.kmaps) == 1 and z.feats.shape == (500, 8)
    with pytest.raises(ValueError, match="mismatch"):
        conv_b(z)
    up = spnn.Conv3d(16, 16, 2, stride=2, transposed=True).cuda().half()
    with pytest.raises(ValueError, match="kernel map"):
        up(y)
    with pytest.raises(ValueError, match="unsupported dataflow"):
        F.conv3d(inp, conv_a.kernel, 3, config=dict(F.conv_config.get_default_conv_config(), dataflow="bogus"))
    with pytest.raises(RuntimeError, match="GPU"):
        backend.conv_forward_implicit_gemm_cuda(x.cpu(), conv_a.kernel.cpu(), torch.zeros(1), 1, 16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("n", [300, 5000])
def test_fused_epilogue_bias_residual_relu(mods, dtype, n):
    """y = relu(conv + bias + residual) in every dataflow (small n takes the offset-split path)."""
    ts, backend, _, F = mods
    rng = np.random.default_rng(n)
    coords = random_coords(rng, n, (30, 30, 10))
    cin, cout = 64, 128
    x, w = _case(rng, n, cin, cout, 27, dtype)
    bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
    res = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    omap = oracle.kmap_subm(coords, 3)
    want = np.maximum(oracle.conv_implicit_gemm(_f32(x), _f32(w), omap, n) + _f32(bias) + _f32(res), 0)
    for dataflow, ifsort in [(F.Dataflow.ImplicitGEMM, False), (F.Dataflow.ImplicitGEMM, True),
                             (F.Dataflow.GatherScatter, False), (F.Dataflow.FetchOnDemand, False)]:
        cfg = F.conv_config.get_default_conv_config()
        cfg.dataflow, cfg.ifsort = dataflow, ifsort
        out = F.conv3d(ts.SparseTensor(x, dev(coords)), w, 3, bias=bias, padding=1, config=cfg,
                       residual=res, activation="relu")
        assert rel_rms(_f32(out.feats), want) < TOL[dtype], (dataflow, ifsort)
    with pytest.raises(ValueError, match="activation"):
        F.conv3d(ts.SparseTensor(x, dev(coords)), w, 3, activation="gelu")


def test_fuse_inference_matches_unfused_unet(mods):
    """BatchNorm folding + fused ReLU / shortcut add leave the network function unchanged."""
    ts, _, _, F = mods
    from torchsparse_amd.backbones import SparseResUNet42
    from torchsparse_amd.nn.utils import fuse_inference
    import copy
    torch.manual_seed(1)
    rng = np.random.default_rng(11)
    coords = dev(random_coords(rng, 6000, (48, 48, 16)))
    x = torch.randn(6000, 4, device="cuda")
    model = SparseResUNet42(in_channels=4).cuda().eval()
    for m in model.modules():  # non-trivial norm statistics
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.normal_(0, 0.3)
            m.running_var.uniform_(0.5, 1.5)
            m.weight.data.uniform_(0.5, 1.5)
            m.bias.data.normal_(0, 0.2)
    fused = fuse_inference(copy.deepcopy(model))
    with torch.no_grad():
        ref = model(ts.SparseTensor(x, coords))
        got = fused(ts.SparseTensor(x, coords))
        assert len(ref) == len(got) == 9
        for a, b in zip(ref, got):
            assert a.coords.data_ptr() != 0 and torch.equal(a.coords, b.coords)
            assert rel_rms(_f32(b.feats), _f32(a.feats)) < 1e-3
        # and in half precision, against the fp32 network
        got16 = copy.deepcopy(fused).half()(ts.SparseTensor(x.half(), coords))
        assert rel_rms(_f32(got16[-1].feats), _f32(ref[-1].feats)) < 3e-2


def test_fuse_inference_matches_unfused_detection_backbone(mods):
    """The detection backbone's basic blocks (two biased convolutions, identity shortcut)
    fold the same way: every stage output of the fused network equals the unfused one's."""
    ts, _, _, F = mods
    from torchsparse_amd.backbones import VoxelResBackBone8x
    from torchsparse_amd.backbones.detection import SparseBasicBlock
    from torchsparse_amd.nn.utils import fuse_inference
    import copy
    torch.manual_seed(2)
    rng = np.random.default_rng(12)
    coords = dev(random_coords(rng, 7000, (33, 48, 48)))
    x = torch.randn(7000, 5, device="cuda")
    model = VoxelResBackBone8x(in_channels=5).cuda().eval()
    for m in model.modules():
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.normal_(0, 0.3)
            m.running_var.uniform_(0.5, 1.5)
            m.weight.data.uniform_(0.5, 1.5)
            m.bias.data.normal_(0, 0.2)
    fused = fuse_inference(copy.deepcopy(model))
    blocks = [m for m in fused.modules() if isinstance(m, SparseBasicBlock)]
    assert len(blocks) == 8 and all(b._fused_tail for b in blocks)
    assert not any(isinstance(m, torch.nn.BatchNorm1d) for m in fused.modules())
    with torch.no_grad():
        ref = model(ts.SparseTensor(x, coords, spatial_range=(1, 33, 48, 48)))
        got = fused(ts.SparseTensor(x, coords, spatial_range=(1, 33, 48, 48)))
    assert set(ref) == set(got)
    for name in ref:
        assert torch.equal(ref[name].coords, got[name].coords), name
        assert rel_rms(_f32(got[name].feats), _f32(ref[name].feats)) < 1e-3, name


@pytest.mark.parametrize("cin,cout", [(64, 64), (128, 128), (96, 160), (256, 256)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_offset_split_sums_in_kernel_equal_second_launch(mods, cin, cout, dtype):
    """Small maps split the kernel offsets over several workgroups.  With tile counters
    the last workgroup of a tile adds the partial sums; without, a second launch does.
    Both add in split order, so the results are bit-identical; the counters are left
    zero, and a second call on the same counters gives the same result."""
    _, backend, _, F = mods
    rng = np.random.default_rng(cin + cout)
    coords = random_coords(rng, 4000, (24, 24, 16))
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, 3, 1, 1, mode="hashmap_on_the_fly")
    omap = kmap["out_in_map"]
    x, w = _case(rng, n, cin, cout, 27, dtype)
    wp = backend.pack_weights(w)
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    C, ptr = backend._C, backend._ptr
    ws_elems = C.tsmi_conv_workspace_elems(n, n, 27, 1, cin, cout, code, 0)
    assert ws_elems > 0  # this size is split
    ws = torch.empty(ws_elems, dtype=torch.float32, device="cuda")
    counters = torch.zeros(4096, dtype=torch.int32, device="cuda")
    bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
    outs = []
    for cnt in (None, counters, counters):
        y = torch.full((n, cout), float("nan"), dtype=dtype, device="cuda")
        backend._check(C.tsmi_conv_implicit_gemm(backend._stream(), ptr(x), ptr(wp), ptr(omap), omap.shape[0],
                                                 n, 27, cin, cout, code, ptr(bias), None, 1, ptr(ws),
                                                 ws_elems, ptr(cnt), 4096, ptr(y)))
        outs.append(y)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    assert int(counters.abs().sum().item()) == 0
    want = np.maximum(oracle.conv_implicit_gemm(_f32(x), _f32(w), omap.cpu().numpy(), n) + _f32(bias), 0)
    assert rel_rms(_f32(outs[1]), want) < TOL[dtype]


def test_short_path_of_cached_map_layers_equals_conv3d(mods):
    """Conv3d.forward takes a short host path (F.conv3d_cached) for inference calls whose map is
    cached; it must return what F.conv3d returns, bit for bit (same kernels, same arguments), for
    submanifold, strided, transposed and 1x1x1 layers with bias, residual and fused ReLU, and
    must step aside whenever a gradient is wanted."""
    ts, backend, spnn, F = mods
    rng = np.random.default_rng(31)
    coords = dev(random_coords(rng, 2500, (20, 20, 12)))
    x = ts.SparseTensor(torch.randn(2500, 32, device="cuda", dtype=torch.float16), coords)
    down = spnn.Conv3d(32, 64, 2, stride=2, bias=True).cuda().half().eval()
    subm = spnn.Conv3d(64, 64, 3, bias=True).cuda().half().eval()
    point = spnn.Conv3d(64, 48, 1, bias=True).cuda().half().eval()
    up = spnn.Conv3d(48, 32, 2, stride=2, transposed=True).cuda().half().eval()
    subm.activation = "relu"

    def general(layer, inp, residual=None):
        return F.conv3d(inp, weight=layer.kernel, kernel_size=layer.kernel_size, bias=layer.bias,
                        stride=layer.stride, padding=layer.padding, dilation=layer.dilation,
                        transposed=layer.transposed, generative=layer.generative, config=layer._config,
                        training=False, residual=residual, activation=layer.activation)

    with torch.no_grad():
        mid = down(x)            # first call builds the map (general path) ...
        res = torch.randn(mid.feats.shape[0], 64, device="cuda", dtype=torch.float16)
        for layer, inp, r in ((down, x, None), (subm, mid, None), (subm, mid, res)):
            general(layer, inp, r)  # ... and the maps are cached from here on
            assert F.conv3d_cached(inp, layer.kernel, layer.bias, layer.kernel_size, layer.stride,
                                   (1, 1, 1), layer.transposed, layer._config, r, layer.activation) is not None
            a, b = layer(inp, residual=r) if r is not None else layer(inp), general(layer, inp, r)
            assert torch.equal(a.feats, b.feats) and a.coords is b.coords and a.stride == b.stride
            assert a._caches is inp._caches
        p1, p2 = point(subm(mid)), general(point, general(subm, mid))
        assert torch.equal(p1.feats, p2.feats) and p1.stride == (2, 2, 2)
        general(up, p2)  # builds the transposed map
        u1, u2 = up(p1), general(up, p2)
        assert torch.equal(u1.feats, u2.feats) and u1.stride == (1, 1, 1) and u1.coords is x.coords
    # a gradient is wanted: the short path declines and autograd gets its graph
    xg = ts.SparseTensor(mid.feats.clone().requires_grad_(True), mid.coords, stride=mid.stride)
    xg._caches = mid._caches
    assert F.conv3d_cached(xg, subm.kernel, subm.bias, subm.kernel_size, subm.stride, (1, 1, 1), False,
                           None, None, "relu") is None
    out = subm(xg)
    out.feats.float().sum().backward()
    assert xg.feats.grad is not None and subm.kernel.grad is not None
    # sorted mode and the other dataflows: not the short path's case
    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = F.Dataflow.GatherScatter
    with torch.no_grad():
        assert F.conv3d_cached(mid, subm.kernel, subm.bias, subm.kernel_size, subm.stride, (1, 1, 1), False,
                               cfg, None, "relu") is None


@pytest.mark.parametrize("n,cin,cout,dtype,how", [
    (40000, 32, 32, torch.float16, "plain"), (5000, 64, 64, torch.float16, "plain"),
    (3000, 256, 256, torch.float16, "plain"), (3000, 256, 256, torch.float16, "segments"),
    (40000, 96, 96, torch.bfloat16, "grouped"), (9000, 16, 24, torch.float32, "plain"),
    (2000, 4, 32, torch.float16, "plain"), (6000, 128, 96, torch.float16, "transposed")])
def test_results_placed_into_column_slices_equal_the_dense_ones(n, cin, cout, dtype, how, monkeypatch):
    """out= / also=: the launch writes its rows into a column slice of a wider buffer (and a
    second time into another) - bit for bit the rows of the dense result, nothing outside the
    slices touched; bias, residual and ReLU included."""
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    rng = np.random.default_rng(n + cin)
    coords_np = lidar_like_coords(rng, n)
    coords_np = coords_np[np.lexsort((coords_np[:, 3], coords_np[:, 2], coords_np[:, 1], coords_np[:, 0]))]
    coords = torch.from_numpy(coords_np).cuda()
    n = coords.shape[0]
    torch.manual_seed(n)
    if how == "grouped":
        monkeypatch.setattr(backend, "igemm_group_rows", "always")
        monkeypatch.setattr(backend, "group_min_rows", 1024)
    if how == "transposed":
        down = spnn.Conv3d(8, cin, 2, stride=2).cuda().to(dtype).eval()
        layer = spnn.Conv3d(cin, cout, 2, stride=2, transposed=True, bias=True).cuda().to(dtype).eval()
        with torch.no_grad():
            x = down(ts.SparseTensor(torch.randn(n, 8, device="cuda", dtype=dtype), coords))
        n_out = n
    else:
        layer = spnn.Conv3d(cin, cout, 3, bias=True).cuda().to(dtype).eval()
        if how == "segments":
            monkeypatch.setattr(backend, "igemm_through_segments", "always")
        x = ts.SparseTensor(torch.randn(n, cin, device="cuda", dtype=dtype), coords)
        n_out = n
    layer.activation = "relu"
    res = torch.randn(n_out, cout, device="cuda", dtype=dtype)
    with torch.no_grad():
        want = layer(x, residual=res).feats
        wide = torch.full((n_out, 8 + cout + 16), 7.0, device="cuda", dtype=dtype)
        second = torch.full((n_out, cout + 8), 5.0, device="cuda", dtype=dtype)
        got = layer(x, residual=res, out=wide[:, 8:8 + cout], also=second[:, :cout])
    assert got.feats.data_ptr() == wide[:, 8:].data_ptr() and got.feats.shape == (n_out, cout)
    assert torch.equal(got.feats, want) and torch.equal(second[:, :cout], want)
    assert (wide[:, :8] == 7).all() and (wide[:, 8 + cout:] == 7).all() and (second[:, cout:] == 5).all()
    assert torch.equal(got.coords, x.coords if how != "transposed" else coords)
    # the same through column slices named without a view
    with torch.no_grad():
        wide2 = torch.full((n_out, 8 + cout + 16), 7.0, device="cuda", dtype=dtype)
        second2 = torch.full((n_out, cout + 8), 5.0, device="cuda", dtype=dtype)
        got2 = layer(x, residual=res, out=backend.ColumnSlice(wide2, 8, cout), also=backend.ColumnSlice(second2, 0, cout))
    assert got2.feats is wide2 and torch.equal(wide2, wide) and torch.equal(second2, second)
    with pytest.raises(ValueError):
        backend.ColumnSlice(wide2, 3, cout)
    # misplaced views are refused
    with torch.no_grad():
        with pytest.raises(ValueError, match="placed"):
            layer(x, out=wide[:, 3:3 + cout])
        with pytest.raises(ValueError, match="placed"):
            layer(x, also=second[:-1, :cout])


def test_placed_results_through_paths_that_copy():
    """out= / also= where the launch does not place its rows itself: another dataflow, a call
    that records gradients, a 1x1x1 layer, the unfused residual block.  The values are copied into
    the slices and the returned tensor is the slice (or the slice's buffer)."""
    import torchsparse_amd as ts
    from torchsparse_amd import backend
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.backbones.modules.blocks import SparseResBlock
    from torchsparse_amd.nn import functional as F
    rng = np.random.default_rng(5)
    coords_np = lidar_like_coords(rng, 3000)
    coords_np = coords_np[np.lexsort((coords_np[:, 3], coords_np[:, 2], coords_np[:, 1], coords_np[:, 0]))]
    coords = torch.from_numpy(coords_np).cuda()
    n = coords.shape[0]
    torch.manual_seed(5)
    feats = torch.randn(n, 16, device="cuda", dtype=torch.float16)

    def slices():
        wide = torch.full((n, 48), 7.0, device="cuda", dtype=torch.float16)
        second = torch.full((n, 40), 5.0, device="cuda", dtype=torch.float16)
        return wide, second

    cfg = F.conv_config.get_default_conv_config()
    cfg.dataflow = F.Dataflow.GatherScatter
    layer = spnn.Conv3d(16, 32, 3, bias=True, config=cfg).cuda().half().eval()
    with torch.no_grad():
        want = layer(ts.SparseTensor(feats, coords)).feats
        wide, second = slices()
        got = layer(ts.SparseTensor(feats, coords), out=wide[:, 8:40], also=backend.ColumnSlice(second, 8, 32))
    assert torch.equal(got.feats, want) and torch.equal(second[:, 8:], want) and (wide[:, :8] == 7).all()
    # gradients recorded: the autograd function computes, the slices receive copies
    layer2 = spnn.Conv3d(16, 32, 3).cuda().half()
    x = ts.SparseTensor(feats.clone().requires_grad_(True), coords)
    want = layer2(x).feats.detach()
    wide, second = slices()
    got = layer2(ts.SparseTensor(feats.clone().requires_grad_(True), coords), out=backend.ColumnSlice(wide, 16, 32))
    assert got.feats is wide and torch.equal(wide[:, 16:], want)
    # a 1x1x1 layer
    point = spnn.Conv3d(16, 32, 1).cuda().half().eval()
    with torch.no_grad():
        want = point(ts.SparseTensor(feats, coords)).feats
        wide, second = slices()
        got = point(ts.SparseTensor(feats, coords), also=second[:, :32])
    assert torch.equal(got.feats, want) and torch.equal(second[:, :32], want) and (second[:, 32:] == 5).all()
    # the residual block before fuse_inference
    block = SparseResBlock(16, 32, 3).cuda().half().eval()
    with torch.no_grad():
        want = block(ts.SparseTensor(feats, coords)).feats
        wide, second = slices()
        got = block(ts.SparseTensor(feats, coords), also=backend.ColumnSlice(wide, 8, 32))
    assert torch.equal(got.feats, want) and torch.equal(wide[:, 8:40], want) and (wide[:, 40:] == 7).all()
