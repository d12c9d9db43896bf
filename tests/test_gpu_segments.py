"""GPU parity of the pair-segment form of the implicit-GEMM dataflow (tsmi_pair_segments,
tsmi_conv_implicit_gemm_segments) against the CPU oracle.

Integer products are compared exactly (counts per offset, the place of every pair, the input
row stored at that place); the order of the pairs inside a segment is not fixed, so it is the
relation between the two arrays that is checked, not their raw contents.  Features: 1e-2
(fp16) / 3e-2 (bf16) of the RMS of the oracle's output, which is fed the inputs already
rounded to the I/O type."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-2, torch.bfloat16: 3e-2}


@pytest.fixture(scope="module")
def mods():
    from torchsparse_amd import backend
    from torchsparse_amd.nn import functional as F
    return backend, F


def dev(a, dtype=torch.int32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dtype)


def _f32(t):
    return t.detach().float().cpu().numpy()


def _check_segments(backend, omap_np, n_rows):
    omap = dev(omap_np)
    counts, in_rows, pos, seg_rows = backend.pair_segments(omap, n_rows)
    counts, in_rows, pos = counts.cpu().numpy(), in_rows.cpu().numpy(), pos.cpu().numpy()
    kvol = omap_np.shape[1]
    assert seg_rows >= n_rows and seg_rows % 64 == 0
    assert in_rows.shape == (kvol, seg_rows) and pos.shape == (kvol, n_rows)
    m = omap_np[:n_rows]
    np.testing.assert_array_equal(counts, (m >= 0).sum(0))
    for k in range(kvol):
        has = m[:, k] >= 0
        assert (pos[k][~has] == -1).all()
        places = pos[k][has]
        # the places of an offset's pairs are 0 .. count-1, each once
        np.testing.assert_array_equal(np.sort(places), np.arange(counts[k]))
        np.testing.assert_array_equal(in_rows[k][places], m[has, k])


@pytest.mark.parametrize("ks,stride,n", [(3, 1, 2500), (3, 1, 1), (2, 2, 3000), ((3, 1, 3), 1, 700),
                                         (5, 1, 400), (3, 2, 2000)])
def test_pair_segments_hold_every_pair_once(mods, ks, stride, n):
    backend, F = mods
    rng = np.random.default_rng(n + 17)
    coords = random_coords(rng, n, (24, 20, 12))
    if stride == 1:
        omap = oracle.kmap_subm(coords, ks)
        n_rows = n
    else:
        pad = 0 if ks == 2 else 1
        omap, out_coords = oracle.kmap_downsample(coords, ks, stride, pad)
        n_rows = len(out_coords)
    _check_segments(backend, omap, n_rows)


def test_pair_segments_of_offsets_without_pairs(mods):
    backend, _ = mods
    # isolated voxels: only the centre offset has pairs
    coords = np.array([[0, 4 * i, 0, 0] for i in range(130)], np.int32)
    omap = oracle.kmap_subm(coords, 3)
    assert (omap[:130] >= 0).sum() == 130
    _check_segments(backend, omap, 130)


def test_pair_segments_are_built_once_per_map(mods):
    backend, _ = mods
    rng = np.random.default_rng(5)
    omap = dev(oracle.kmap_subm(random_coords(rng, 300, (10, 10, 10)), 3))
    a = backend.pair_segments(omap, 300)
    assert backend.pair_segments(omap, 300) is a
    assert backend.pair_segments(omap, 256) is not a  # another row count: rebuilt
    with pytest.raises(ValueError):
        backend.pair_segments(omap, omap.shape[0] + 1)


SHAPES = [(3000, 128, 128), (2100, 256, 256), (1300, 192, 128), (777, 384, 256), (1500, 128, 136),
          (64, 256, 128), (1, 128, 128)]


@pytest.mark.parametrize("n,cin,cout", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_convolution_over_segments_matches_oracle(mods, n, cin, cout, dtype):
    backend, F = mods
    rng = np.random.default_rng(n + cin + cout)
    coords = random_coords(rng, n, (22, 18, 12))
    omap_np = oracle.kmap_subm(coords, 3)
    omap = dev(omap_np)
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).to("cuda", dtype)
    bound = 1.0 / np.sqrt(cin * 27)
    w = torch.from_numpy(rng.uniform(-bound, bound, (27, cin, cout)).astype(np.float32)).to("cuda", dtype)
    assert backend._C.tsmi_conv_segments_supported(27, cin, cout, backend._dtype_code(x)) == 1
    wp = backend.pack_weights(w)
    y = backend.conv_implicit_gemm_segments(x, wp, 27, cin, cout, omap, n)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap_np, n)
    assert y.dtype == dtype and y.shape == (n, cout)
    assert rel_rms(_f32(y), want) < TOL[dtype]
    # epilogue: bias, residual and ReLU
    bias = torch.from_numpy(rng.standard_normal(cout).astype(np.float32)).to("cuda", dtype)
    res = torch.from_numpy(rng.standard_normal((n, cout)).astype(np.float32)).to("cuda", dtype)
    y2 = backend.conv_implicit_gemm_segments(x, wp, 27, cin, cout, omap, n, bias, res, True)
    want2 = np.maximum(want + _f32(bias)[None, :] + _f32(res), 0)
    assert rel_rms(_f32(y2), want2) < TOL[dtype]


def test_segments_and_dense_pass_agree_through_the_public_call(mods):
    """conv_forward_implicit_gemm_cuda takes the segment form for small, wide layers; switched
    off it runs the dense pass.  Both against the oracle, and close to each other."""
    backend, F = mods
    rng = np.random.default_rng(99)
    n, cin, cout = 4000, 256, 256
    coords = random_coords(rng, n, (30, 30, 10))
    omap_np = oracle.kmap_subm(coords, 3)
    omap = dev(omap_np)
    x = torch.from_numpy(rng.standard_normal((n, cin)).astype(np.float32)).cuda().half()
    w = torch.from_numpy(rng.uniform(-0.01, 0.01, (27, cin, cout)).astype(np.float32)).cuda().half()
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap_np, n)
    keep = backend.igemm_through_segments
    try:
        backend.igemm_through_segments = True  # the default: only maps known to be thin
        assert not backend._segments_pay(x, 27, cin, cout, n, omap)
        backend.hint_sparse_map(omap)
        assert backend._segments_pay(x, 27, cin, cout, n, omap)
        seg = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout)
        assert id(omap) in backend._segments_of  # the segment form ran (and kept its lists)
        other = omap.clone()  # an unmarked map of the same content: dense, unless told "always"
        assert not backend._segments_pay(x, 27, cin, cout, n, other)
        backend.igemm_through_segments = "always"
        assert backend._segments_pay(x, 27, cin, cout, n, other)
        backend.igemm_through_segments = False
        assert not backend._segments_pay(x, 27, cin, cout, n, omap)
        dense = backend.conv_forward_implicit_gemm_cuda(x, w, omap, n, cout)
    finally:
        backend.igemm_through_segments = keep
    assert rel_rms(_f32(seg), want) < 1e-2 and rel_rms(_f32(dense), want) < 1e-2
    assert rel_rms(_f32(seg), _f32(dense)) < 1e-2


def test_strided_and_transposed_maps_over_segments(mods):
    """A strided map (K_vol 8, fewer outputs than inputs) and its transposed map (every row at
    most one pair), called directly."""
    backend, F = mods
    rng = np.random.default_rng(321)
    coords = random_coords(rng, 5000, (40, 30, 12))
    omap_np, out_coords = oracle.kmap_downsample(coords, 2, 2, 0)
    n_in, n_out = len(coords), len(out_coords)
    cin, cout = 128, 256
    x = torch.from_numpy(rng.standard_normal((n_in, cin)).astype(np.float32)).cuda().half()
    w = torch.from_numpy(rng.uniform(-0.03, 0.03, (8, cin, cout)).astype(np.float32)).cuda().half()
    y = backend.conv_implicit_gemm_segments(x, backend.pack_weights(w), 8, cin, cout, dev(omap_np), n_out)
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap_np, n_out)
    assert rel_rms(_f32(y), want) < 1e-2
    map_t = oracle.transpose_map(omap_np, n_in)
    xt = torch.from_numpy(rng.standard_normal((n_out, cout)).astype(np.float32)).cuda().half()
    wt = torch.from_numpy(rng.uniform(-0.03, 0.03, (8, cout, cin)).astype(np.float32)).cuda().half()
    yt = backend.conv_implicit_gemm_segments(xt, backend.pack_weights(wt), 8, cout, cin, dev(map_t), n_in)
    want_t = oracle.conv_implicit_gemm(_f32(xt), _f32(wt), map_t, n_in)
    assert rel_rms(_f32(yt), want_t) < 1e-2


def test_shapes_without_a_variant_are_refused_and_fall_back(mods):
    backend, F = mods
    code = 1  # fp16
    for kvol, cin, cout in ((27, 96, 128), (27, 64, 128), (27, 512, 128), (125, 128, 128), (27, 128, 130)):
        assert backend._C.tsmi_conv_segments_supported(kvol, cin, cout, code) == 0, (kvol, cin, cout)
    assert backend._C.tsmi_conv_segments_supported(27, 128, 128, 0) == 0  # fp32: the dense pass only
    rng = np.random.default_rng(8)
    n = 500
    coords = random_coords(rng, n, (12, 12, 8))
    omap_np = oracle.kmap_subm(coords, 3)
    x = torch.from_numpy(rng.standard_normal((n, 96)).astype(np.float32)).cuda().half()
    w = torch.from_numpy(rng.uniform(-0.02, 0.02, (27, 96, 128)).astype(np.float32)).cuda().half()
    with pytest.raises(ValueError):
        backend.conv_implicit_gemm_segments(x, backend.pack_weights(w), 27, 96, 128, dev(omap_np), n)
    assert not backend._segments_pay(x, 27, 96, 128, n, dev(omap_np))
    y = backend.conv_forward_implicit_gemm_cuda(x, w, dev(omap_np), n, 128)  # the dense pass
    want = oracle.conv_implicit_gemm(_f32(x), _f32(w), omap_np, n)
    assert rel_rms(_f32(y), want) < 1e-2


def test_maps_over_thinned_rows_are_marked_sparse_and_solid_ones_are_not(mods):
    """build_kernel_map marks the submanifold map of a level that a kernel = stride layer
    produced when the level kept at least 0.3 rows per input row (surfaces, scattered voxels);
    a solid volume keeps 1/8 and stays with the dense pass."""
    backend, F = mods
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    rng = np.random.default_rng(77)
    scattered = random_coords(rng, 3000, (60, 60, 40))
    g = np.stack(np.meshgrid(np.arange(16), np.arange(16), np.arange(12), indexing="ij"), -1).reshape(-1, 3)
    solid = np.concatenate([np.zeros((len(g), 1), np.int64), g], 1).astype(np.int32)
    for coords_np, marked in ((scattered, True), (solid, False)):
        order = np.lexsort((coords_np[:, 3], coords_np[:, 2], coords_np[:, 1], coords_np[:, 0]))
        coords = dev(coords_np[order])
        x = ts.SparseTensor(torch.zeros(len(coords_np), 4, device="cuda", dtype=torch.float16), coords)
        down = spnn.Conv3d(4, 128, 2, stride=2).cuda().half().eval()
        deep = spnn.Conv3d(128, 256, 3).cuda().half().eval()
        with torch.no_grad():
            mid = down(x)
            thinning = backend.level_thinning(mid.coords)
            assert thinning is not None and abs(thinning - mid.coords.shape[0] / len(coords_np)) < 1e-9
            assert (thinning >= 0.3) == marked
            out = deep(mid)
        omap = mid._caches.kmaps[((2, 2, 2), (3, 3, 3), (1, 1, 1), (1, 1, 1))]["out_in_map"]
        hit = backend._sparse_maps.get(id(omap))
        assert (hit is not None and hit() is omap) == marked
        assert backend._segments_pay(mid.feats, 27, 128, 256, mid.feats.shape[0], omap) == marked
        want = oracle.conv_implicit_gemm(_f32(mid.feats), _f32(deep.kernel), omap.cpu().numpy(), mid.feats.shape[0])
        assert rel_rms(_f32(out.feats), want) < 1e-2
    assert backend.level_thinning(dev(scattered)) is None  # a caller's own rows: nothing known


def test_the_form_of_a_wide_layer_follows_the_measured_density_of_its_map(mods):
    """Maps queued ahead of their use count their pairs; once the count is on the host the
    implicit-GEMM dataflow takes the pair form for a wide, small layer where at most
    segments_max_density of the map's entries are pairs.  A solid volume (more than half of the
    entries) and a surface scan (a quarter or less): the measured density equals the oracle's,
    decides the form, and the form taken is the quicker of the two on the device (medians of
    20 timed calls each; the slower form is slower by 25 % and more on both, the test allows
    the taken one 15 %)."""
    backend, F = mods
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.utils.synthetic import lidar_scan_voxels
    g = np.stack(np.meshgrid(np.arange(64), np.arange(64), np.arange(32), indexing="ij"), -1).reshape(-1, 3)
    solid = np.concatenate([np.zeros((len(g), 1), np.int64), g], 1).astype(np.int32)
    thin = lidar_scan_voxels(seed=1)[::2].copy()  # (every other voxel of the benchmark's scan)
    torch.manual_seed(9)
    net = torch.nn.ModuleList([spnn.Conv3d(16, 128, 2, stride=2), spnn.Conv3d(128, 256, 3),
                               spnn.Conv3d(256, 256, 2, stride=2), spnn.Conv3d(256, 256, 3),
                               spnn.Conv3d(4, 16, 3)]).cuda().half().eval()
    key2 = ((2, 2, 2), (3, 3, 3), (1, 1, 1), (1, 1, 1))

    def median_us(fn):
        ts_ = []
        for _ in range(20):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            b.synchronize()
            ts_.append(a.elapsed_time(b) * 1e3)
        return float(np.median(ts_))

    for coords_np, dense in ((solid, True), (thin, False)):
        coords_np = coords_np[np.lexsort((coords_np[:, 3], coords_np[:, 2], coords_np[:, 1], coords_np[:, 0]))]
        base = dev(coords_np)
        feats = torch.randn(len(coords_np), 4, device="cuda", dtype=torch.float16)
        backend.release_scratch()
        with torch.no_grad():
            # (a submanifold layer first, as in a network: the chain of the two strided layers starts
            # beside it once it has been learnt, and the maps over its levels are queued ahead)
            for _ in range(5):
                x = ts.SparseTensor(feats, base.clone())
                mid = net[1](net[0](net[4](x)))
                net[3](net[2](mid))
        torch.cuda.synchronize()
        omap = x._caches.kmaps[key2]["out_in_map"]
        n2 = mid.feats.shape[0]
        want = oracle.kmap_subm(mid.coords.cpu().numpy(), 3)[:n2]
        density = backend.map_density(omap)
        assert density is not None and density == (want >= 0).mean()
        assert (density >= 0.5) if dense else (density <= 0.25), density
        assert 4000 < n2 < 65536
        assert backend._segments_pay(mid.feats, 27, 128, 256, n2, omap) == (not dense)
        xin = torch.randn(n2, 128, device="cuda", dtype=torch.float16)
        wp = backend.pack_weights(net[1].kernel)
        pair = median_us(lambda: backend.conv_implicit_gemm_segments(xin, wp, 27, 128, 256, omap, n2))
        try:
            backend.igemm_through_segments = False
            plain = median_us(lambda: backend._implicit_gemm(xin, wp, 27, 128, 256, omap, n2))
        finally:
            backend.igemm_through_segments = True
        taken, other = (plain, pair) if dense else (pair, plain)
        print(f"density {density:.3f}: pair form {pair:.1f} us, dense pass {plain:.1f} us")
        assert taken <= 1.15 * other, (density, pair, plain)
