"""Generative transposed convolution (conv.py:162-204, kmap/upsample.py): generated output
coordinates and the map bit-exact against the oracle, features within the conv tolerance."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu


@pytest.fixture()
def mods():
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    yield ts, spnn, F


def _hashmap_config(F, flow="ImplicitGEMM"):
    """Generative convolutions need kmap_mode "hashmap" in the layer's config (conv.py:47)."""
    cfg = F.conv_config.get_default_conv_config()
    cfg.kmap_mode = "hashmap"
    cfg.dataflow = getattr(F.Dataflow, flow)
    return cfg


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("ks,st,rng_shape", [(3, 2, (2, 40, 36, 24)), (2, 2, (2, 40, 36, 24)),
                                            (3, 1, (2, 20, 18, 12)), ((3, 1, 2), (2, 1, 2), (2, 25, 18, 20)),
                                            (5, 2, (2, 12, 12, 12))])
def test_generated_coordinates_match_oracle(mods, ks, st, rng_shape):
    _, _, F = mods
    rng = np.random.default_rng(0)
    coords = random_coords(rng, 1500, (20, 18, 12), batch=2)
    got = F.spupsample_generative(dev(coords), st, ks, 0, rng_shape).cpu().numpy()
    np.testing.assert_array_equal(got, oracle.upsample_generative_coords(coords, ks, st, rng_shape))


@pytest.mark.parametrize("flow", ["ImplicitGEMM", "GatherScatter", "FetchOnDemand"])
@pytest.mark.parametrize("ks,st", [(3, 2), (2, 2)])
def test_generative_convolution_matches_oracle(mods, flow, ks, st):
    ts, spnn, F = mods
    rng = np.random.default_rng(1)
    coords = random_coords(rng, 1200, (16, 14, 10), batch=2)
    n = len(coords)
    # the reference clamps to the STRIDED range of the input (build_kmap.py:65-74): make it
    # large enough that the upsampled coordinates fit
    in_range = (2, 80, 80, 80)
    cfg = _hashmap_config(F, flow)
    torch.manual_seed(2)
    layer = spnn.Conv3d(8, 16, ks, stride=st, transposed=True, generative=True, bias=True, config=cfg).cuda()
    x = rng.standard_normal((n, 8)).astype(np.float32)
    inp = ts.SparseTensor(dev(x), dev(coords), stride=2, spatial_range=in_range)
    inp._caches.kmaps["stale"] = 1
    with torch.no_grad():
        out = layer(inp)
    pad = layer.padding
    new_range = (2,) + tuple((in_range[a + 1] + 2 * pad[a] - (layer.kernel_size[a] - 1) - 1) // st + 1
                             for a in range(3))
    want_map, want_coords = oracle.kmap_generative(coords, ks, st, new_range)
    np.testing.assert_array_equal(out.coords.cpu().numpy(), want_coords)
    assert out.stride == (2 // st,) * 3 and tuple(out.spatial_range) == new_range
    want = oracle.conv_implicit_gemm(x, layer.kernel.detach().cpu().numpy(), want_map, len(want_coords))
    want = want + layer.bias.detach().cpu().numpy()
    assert rel_rms(out.feats.cpu().numpy(), want) < 1e-4
    # the new level is registered, the maps and tables of the old levels are dropped
    assert out._caches is inp._caches and out._caches.kmaps == {} and out._caches.hashmaps == {}
    assert torch.equal(out._caches.cmaps[out.stride][0], out.coords)
    # a submanifold convolution runs on the generated tensor
    with torch.no_grad():
        nxt = spnn.Conv3d(16, 16, 3, config=cfg).cuda()(out)
    assert nxt.feats.shape == (len(want_coords), 16)


def test_generative_gradients_match_oracle(mods):
    ts, spnn, F = mods
    rng = np.random.default_rng(3)
    coords = random_coords(rng, 600, (12, 12, 8))
    x = rng.standard_normal((len(coords), 8)).astype(np.float32)
    layer = spnn.Conv3d(8, 8, 3, stride=2, transposed=True, generative=True, config=_hashmap_config(F)).cuda()
    xt = dev(x).requires_grad_(True)
    out = layer(ts.SparseTensor(xt, dev(coords), stride=2, spatial_range=(1, 60, 60, 60)))
    g = rng.standard_normal(tuple(out.feats.shape)).astype(np.float32)
    out.feats.backward(dev(g))
    pad = layer.padding
    new_range = (1,) + tuple((60 + 2 * pad[a] - 2 - 1) // 2 + 1 for a in range(3))
    omap, oc = oracle.kmap_generative(coords, 3, 2, new_range)
    want_dx, want_dw = oracle.conv_backward_implicit_gemm(x, layer.kernel.detach().cpu().numpy(), omap, g)
    assert rel_rms(xt.grad.cpu().numpy(), want_dx) < 1e-4
    assert rel_rms(layer.kernel.grad.cpu().numpy(), want_dw) < 1e-4


def test_generative_needs_hashmap_mode_and_a_spatial_range(mods):
    ts, spnn, F = mods
    coords = dev(random_coords(np.random.default_rng(4), 100, (8, 8, 8)))
    x = torch.randn(len(coords), 4, device="cuda")
    layer = spnn.Conv3d(4, 4, 2, stride=2, transposed=True, generative=True, config=_hashmap_config(F)).cuda()
    with pytest.raises(AssertionError, match="spatial range"):
        layer(ts.SparseTensor(x, coords, stride=2))
    on_the_fly = spnn.Conv3d(4, 4, 2, stride=2, transposed=True, generative=True).cuda()
    with pytest.raises(ValueError, match="generative"):
        on_the_fly(ts.SparseTensor(x, coords, stride=2, spatial_range=(1, 32, 32, 32)))
