"""Pins the floating-point part of the CPU oracle: golden vectors written by the
compiled reference CPU convolution, dense torch.nn.Conv3d / ConvTranspose3d
equivalence (the method of the reference's tests/python/test_single_layer_conv.py),
and the float64 closed form."""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import conv_closed_form, random_coords, rel_rms

GOLD = os.path.join(os.path.dirname(__file__), "golden")


@pytest.mark.parametrize("name", ["subm3", "down2", "up2", "down3"])
@pytest.mark.parametrize("variant", [0, 1])
def test_gather_scatter_matches_reference_golden(name, variant):
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    x, w, y = g[name + "_x"], g[name + "_w"], g[name + "_y"]
    got = oracle.conv_gather_scatter(x, w, g[name + "_nbmaps"], g[name + "_nbsizes"], y.shape[0],
                                     transpose=bool(g[name + "_transpose"]), variant=variant)
    assert rel_rms(got, y) < 1e-5  # fp32 tolerance: summation order differs from ATen's mm


@pytest.mark.parametrize("name", ["subm3", "down2", "down3"])
def test_implicit_gemm_matches_reference_golden(name):
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    y = g[name + "_y"]
    got = oracle.conv_implicit_gemm(g[name + "_x"], g[name + "_w"], g[name + "_map"], y.shape[0])
    assert rel_rms(got, y) < 1e-5


def test_transposed_closed_form_matches_reference_golden():
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    y = g["up2_y"]
    map_t = oracle.transpose_map(g["up2_map"], y.shape[0])
    got = oracle.conv_implicit_gemm(g["up2_x"], g["up2_w"], map_t, y.shape[0])
    assert rel_rms(got, y) < 1e-5


def test_hash_matches_reference_golden():
    g = np.load(os.path.join(GOLD, "hash_cpu.npz"))
    np.testing.assert_array_equal(oracle.hash_cpu(g["rows"]), g["hash"])
    np.testing.assert_array_equal(oracle.kernel_hash_cpu(g["rows"], g["offsets"]), g["kernel_hash"])


def test_gather_scatter_channel_mismatch_raises():
    with pytest.raises(ValueError, match="mismatch"):
        oracle.conv_gather_scatter(np.zeros((4, 3)), np.zeros((27, 5, 2)), np.zeros((0, 2)),
                                   np.zeros(27), 4)


def test_identity_map_reduces_to_matmul():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((256, 16)).astype(np.float32)
    w = rng.standard_normal((1, 16, 8)).astype(np.float32)
    m = np.arange(256, dtype=np.int32)[:, None]
    np.testing.assert_allclose(oracle.conv_implicit_gemm(x, w, m, 256), x.astype(np.float64) @ w[0],
                               rtol=1e-6, atol=1e-6)


def _dense_reference(coords, feats, filters, k, s, shape, transposed=False):
    """Dense torch conv of the scattered input, float64 on CPU.  Weight permutation
    and far-end padding as in tests/python/test_single_layer_conv.py:186-203."""
    B = int(coords[:, 0].max()) + 1
    cin = feats.shape[1]
    dense = torch.zeros(B, cin, *shape, dtype=torch.float64)
    for c, f in zip(coords, feats):
        dense[c[0], :, c[1], c[2], c[3]] = torch.from_numpy(f.astype(np.float64))
    f_t = torch.from_numpy(filters.astype(np.float64))
    if k % 2 == 1:
        weight = f_t.permute(4, 3, 2, 1, 0).contiguous()
        pad = (k - 1) // 2
    else:
        weight = f_t.permute(4, 3, 0, 1, 2).contiguous()
        pad = 0
        dense = torch.nn.functional.pad(dense, (0, k - 1) * 3)
    return torch.nn.functional.conv3d(dense, weight, stride=s, padding=pad).numpy()


@pytest.mark.parametrize("k", [2, 3, 5])
@pytest.mark.parametrize("s", [1, 2, 3])
@pytest.mark.parametrize("mode", ["hashmap_on_the_fly", "hashmap"])
def test_dense_conv_equivalence(k, s, mode):
    """k in {2,3,5} x s in {1,2,3} in both kmap modes, as tests/test.py:11-38."""
    rng = np.random.default_rng(0)
    shape, IC, OC = (5, 5, 5), 16, 32
    coords = random_coords(rng, 20, shape)
    feats = rng.uniform(-1, 1, (20, IC)).astype(np.float32)
    filters = rng.uniform(-1, 1, (k, k, k, IC, OC)).astype(np.float32)
    w = filters.reshape(-1, IC, OC)
    pad = (k - 1) // 2 if k % 2 == 1 else 0
    if s == 1:
        omap, ocoords = oracle.kmap_subm(coords, k, coords_max=[0, 4, 4, 4]), coords
    elif mode == "hashmap_on_the_fly":
        sr = (1,) + tuple((shape[a] + 2 * pad - (k - 1) - 1) // s + 1 for a in range(3))
        omap, ocoords = oracle.kmap_downsample(coords, k, s, pad, spatial_range=sr)
    else:
        if s == k:
            ocoords = oracle.spdownsample_floor(coords, s)
        else:
            sr = (1,) + tuple((shape[a] + 2 * pad - (k - 1) - 1) // s + 1 for a in range(3))
            ocoords = oracle.kmap_downsample(coords, k, s, pad, spatial_range=sr)[1]
        omap = oracle.lookup_coords(coords, ocoords, k, s)
    y = oracle.conv_implicit_gemm(feats, w, omap, len(ocoords))
    ref = _dense_reference(coords, feats, filters, k, s, shape)
    want = np.stack([ref[c[0], :, c[1], c[2], c[3]] for c in ocoords])
    assert rel_rms(y, want) < 1e-5
    # pair-list dataflow gives the same numbers
    nbmaps, nbsizes = oracle.pair_lists(omap)
    y2 = oracle.conv_gather_scatter(feats, w, nbmaps, nbsizes, len(ocoords))
    assert rel_rms(y2, want) < 1e-5
    if s > 1 and mode == "hashmap_on_the_fly":
        # output set = dense occupancy (any input in the receptive field), inside the bound
        occ = _dense_reference(coords, np.ones((20, 1), np.float32), np.ones((k, k, k, 1, 1), np.float32),
                               k, s, shape)[0, 0]
        lim = [(shape[a] + 2 * pad - (k - 1) - 1) // s + 1 for a in range(3)]
        occ = occ[:lim[0], :lim[1], :lim[2]]
        want_set = {(0,) + tuple(int(v) for v in p) for p in np.argwhere(occ > 0)}
        assert {tuple(int(v) for v in c) for c in ocoords} == want_set


def test_transposed_equals_dense_conv_transpose():
    rng = np.random.default_rng(5)
    shape, IC, OC = (8, 8, 8), 6, 5
    coords = random_coords(rng, 60, shape)
    omap, ocoords = oracle.kmap_downsample(coords, 2, 2, 0)
    x = rng.standard_normal((len(ocoords), IC)).astype(np.float32)
    filters = rng.uniform(-1, 1, (2, 2, 2, IC, OC)).astype(np.float32)
    map_t = oracle.transpose_map(omap, len(coords))
    y = oracle.conv_implicit_gemm(x, filters.reshape(-1, IC, OC), map_t, len(coords))
    dense = torch.zeros(1, IC, 4, 4, 4, dtype=torch.float64)
    for c, f in zip(ocoords, x):
        dense[0, :, c[1], c[2], c[3]] = torch.from_numpy(f.astype(np.float64))
    wt = torch.from_numpy(filters.astype(np.float64)).permute(3, 4, 0, 1, 2).contiguous()
    ref = torch.nn.functional.conv_transpose3d(dense, wt, stride=2).numpy()
    want = np.stack([ref[0, :, c[1], c[2], c[3]] for c in coords])
    assert rel_rms(y, want) < 1e-5
    # the pair-list form with swapped roles agrees
    nbmaps, nbsizes = oracle.pair_lists(omap)
    y2 = oracle.conv_gather_scatter(x, filters.reshape(-1, IC, OC), nbmaps, nbsizes, len(coords),
                                    transpose=True)
    assert rel_rms(y2, want) < 1e-5


def test_closed_form_float64():
    rng = np.random.default_rng(6)
    coords = random_coords(rng, 3000, (40, 40, 12))
    omap = oracle.kmap_subm(coords, 3)
    x = rng.standard_normal((3000, 24)).astype(np.float32)
    w = rng.uniform(-0.1, 0.1, (27, 24, 40)).astype(np.float32)
    y = oracle.conv_implicit_gemm(x, w, omap, 3000)
    assert rel_rms(y, conv_closed_form(x, w, omap, 3000)) < 1e-6


# ------------------------------------------------------------------ backward

@pytest.mark.parametrize("name", ["subm3", "down2", "up2", "down3"])
def test_backward_gather_scatter_matches_reference_golden(name):
    """conv_backward_gather_scatter_cpu of the compiled reference
    (convolution_gather_scatter_cpu.cpp:111-188) on the golden cases."""
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    b = np.load(os.path.join(GOLD, "conv_gs_bwd_cpu.npz"))
    dx, dw = oracle.conv_backward_gather_scatter(g[name + "_x"], g[name + "_w"], g[name + "_nbmaps"],
                                                 g[name + "_nbsizes"], b[name + "_dy"],
                                                 bool(g[name + "_transpose"]))
    assert rel_rms(dx, b[name + "_dx"]) < 1e-5  # the reference sums in fp32
    assert rel_rms(dw, b[name + "_dw"]) < 1e-5  # the reference sums in fp32


@pytest.mark.parametrize("name", ["subm3", "down2", "down3"])
def test_backward_from_map_equals_backward_from_pairs(name):
    g = np.load(os.path.join(GOLD, "conv_gs_cpu.npz"))
    b = np.load(os.path.join(GOLD, "conv_gs_bwd_cpu.npz"))
    dx, dw = oracle.conv_backward_implicit_gemm(g[name + "_x"], g[name + "_w"], g[name + "_map"],
                                                b[name + "_dy"])
    assert rel_rms(dx, b[name + "_dx"]) < 1e-5  # the reference sums in fp32
    assert rel_rms(dw, b[name + "_dw"]) < 1e-5  # the reference sums in fp32


@pytest.mark.parametrize("k,s", [(3, 1), (2, 2), (3, 2)])
def test_backward_equals_autograd_of_dense_conv(k, s):
    """Gradients of the dense nn.functional.conv3d equivalent, restricted to the active
    voxels (the reference's own test method, tests/python/test_single_layer_conv.py)."""
    rng = np.random.default_rng(5)
    shape, IC, OC = (6, 5, 4), 6, 5
    coords = random_coords(rng, 30, shape)
    feats = rng.uniform(-1, 1, (30, IC)).astype(np.float32)
    filters = rng.uniform(-1, 1, (k, k, k, IC, OC)).astype(np.float32)
    w = filters.reshape(-1, IC, OC)
    pad = (k - 1) // 2 if k % 2 == 1 else 0
    if s == 1:
        omap, ocoords = oracle.kmap_subm(coords, k, coords_max=[0] + [v - 1 for v in shape]), coords
    else:
        sr = (1,) + tuple((shape[a] + 2 * pad - (k - 1) - 1) // s + 1 for a in range(3))
        omap, ocoords = oracle.kmap_downsample(coords, k, s, pad, spatial_range=sr)
    dy = rng.standard_normal((len(ocoords), OC)).astype(np.float32)
    dx, dw = oracle.conv_backward_implicit_gemm(feats, w, omap, dy)

    dense = torch.zeros(1, IC, *shape, dtype=torch.float64)
    for c, f in zip(coords, feats):
        dense[0, :, c[1], c[2], c[3]] = torch.from_numpy(f.astype(np.float64))
    dense.requires_grad_(True)
    f_t = torch.from_numpy(filters.astype(np.float64)).requires_grad_(True)
    if k % 2 == 1:
        weight, xin = f_t.permute(4, 3, 2, 1, 0), dense
    else:
        weight, xin = f_t.permute(4, 3, 0, 1, 2), torch.nn.functional.pad(dense, (0, k - 1) * 3)
    out = torch.nn.functional.conv3d(xin, weight, stride=s, padding=pad)
    gout = torch.zeros_like(out)
    for c, g in zip(ocoords, dy):
        gout[0, :, c[1], c[2], c[3]] = torch.from_numpy(g.astype(np.float64))
    out.backward(gout)
    want_dx = np.stack([dense.grad[0, :, c[1], c[2], c[3]].numpy() for c in coords])
    want_dw = f_t.grad.numpy().reshape(-1, IC, OC)
    assert rel_rms(dx, want_dx) < 1e-5
    assert rel_rms(dw, want_dw) < 1e-5


def test_backward_is_the_derivative_of_the_oracle_forward():
    rng = np.random.default_rng(6)
    coords = random_coords(rng, 40, (5, 5, 5))
    omap = oracle.kmap_subm(coords, 3)
    x = rng.standard_normal((40, 3)).astype(np.float32)
    w = rng.standard_normal((27, 3, 4)).astype(np.float32)
    dy = rng.standard_normal((40, 4)).astype(np.float32)
    dx, dw = oracle.conv_backward_implicit_gemm(x, w, omap, dy)
    # the forward is bilinear: <dy, conv(x + e, w)> - <dy, conv(x, w)> = <dx, e> exactly
    e = rng.standard_normal(x.shape).astype(np.float32)
    lhs = (dy * (oracle.conv_implicit_gemm(x + e, w, omap, 40) - oracle.conv_implicit_gemm(x, w, omap, 40))).sum()
    assert abs(lhs - (dx * e).sum()) < 1e-3 * max(1.0, abs(lhs))
    ew = rng.standard_normal(w.shape).astype(np.float32)
    lhs = (dy * (oracle.conv_implicit_gemm(x, w + ew, omap, 40) - oracle.conv_implicit_gemm(x, w, omap, 40))).sum()
    assert abs(lhs - (dw * ew).sum()) < 1e-3 * max(1.0, abs(lhs))
