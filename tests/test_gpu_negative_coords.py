"""Negative voxel coordinates (tensor.set_allow_negative_coordinates, tensor.py:16-26):
kernel maps and output coordinates bit-exact against the oracle, which restates the
reference's coords_min rule (hashmap_on_the_fly.py:39-43)."""
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
    from torchsparse_amd import tensor
    from torchsparse_amd.nn import functional as F
    yield ts, spnn, F, tensor
    tensor.set_allow_negative_coordinates(False)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _shifted(rng, n, extent, shift):
    coords = random_coords(rng, n, extent, batch=2)
    coords[:, 1:] -= np.asarray(shift, np.int32)
    return coords


@pytest.mark.parametrize("ks", [3, 2, (3, 1, 5)])
def test_submanifold_map_with_negative_coordinates(mods, ks):
    _, _, F, _ = mods
    rng = np.random.default_rng(0)
    coords = _shifted(rng, 3000, (30, 25, 20), (17, 40, 9))
    assert coords[:, 1:].min() < 0
    n = len(coords)
    kmap = F.build_kernel_map(dev(coords), n, ks, 1, 0, mode="hashmap_on_the_fly")
    want = oracle.kmap_subm(coords, ks, coords_min=coords.min(0), coords_max=coords.max(0))
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy(), want)
    # a map depends on coordinate differences only
    moved = coords.copy()
    moved[:, 1:] += np.array([1000, -3000, 77], np.int32)
    again = F.build_kernel_map(dev(moved), n, ks, 1, 0, mode="hashmap_on_the_fly")
    assert torch.equal(again["out_in_map"], kmap["out_in_map"])


@pytest.mark.parametrize("geom", [(2, 2, 0), (3, 2, 1), (3, 2, 0), ((3, 2, 2), (2, 2, 1), (1, 0, 0))])
@pytest.mark.parametrize("flag", [True, False])
def test_strided_map_with_negative_coordinates(mods, geom, flag):
    _, _, F, tensor = mods
    ks, st, pad = geom
    rng = np.random.default_rng(1)
    coords = _shifted(rng, 2500, (28, 26, 22), (13, 11, 6))
    tensor.set_allow_negative_coordinates(flag)
    assert tensor.get_allow_negative_coordinates() == flag
    kmap = F.build_kernel_map(dev(coords), len(coords), ks, st, pad, mode="hashmap_on_the_fly")
    want_map, want_coords = oracle.kmap_downsample(coords, ks, st, pad, allow_negative=flag)
    got_coords = kmap["coords"].cpu().numpy()
    np.testing.assert_array_equal(got_coords, want_coords)
    np.testing.assert_array_equal(kmap["out_in_map"].cpu().numpy()[:len(want_coords)],
                                  want_map[:len(want_coords)])
    if flag:
        assert got_coords[:, 1:].min() < 0
    else:
        # outputs below zero are dropped, as in the reference
        assert len(got_coords) > 0 and got_coords[:, 1:].min() >= 0


def test_network_on_negative_coordinates_matches_oracle(mods):
    ts, spnn, F, tensor = mods
    tensor.set_allow_negative_coordinates(True)
    rng = np.random.default_rng(2)
    coords = _shifted(rng, 2000, (24, 24, 16), (12, 12, 8))
    x = rng.standard_normal((len(coords), 16)).astype(np.float32)
    torch.manual_seed(0)
    subm = spnn.Conv3d(16, 32, 3).cuda()
    down = spnn.Conv3d(32, 32, 2, stride=2).cuda()
    up = spnn.Conv3d(32, 16, 2, stride=2, transposed=True).cuda()
    with torch.no_grad():
        a = subm(ts.SparseTensor(dev(x), dev(coords)))
        b = down(a)
        c = up(b)
    m1 = oracle.kmap_subm(coords, 3, coords_min=coords.min(0), coords_max=coords.max(0))
    want_a = oracle.conv_implicit_gemm(x, subm.kernel.detach().cpu().numpy(), m1, len(coords))
    assert rel_rms(a.feats.cpu().numpy(), want_a) < 1e-4
    m2, c2 = oracle.kmap_downsample(coords, 2, 2, 0, allow_negative=True)
    np.testing.assert_array_equal(b.coords.cpu().numpy(), c2)
    want_b = oracle.conv_implicit_gemm(want_a, down.kernel.detach().cpu().numpy(), m2, len(c2))
    assert rel_rms(b.feats.cpu().numpy(), want_b) < 1e-4
    assert torch.equal(c.coords, a.coords) and c.feats.shape == (len(coords), 16)
    m2t = oracle.transpose_map(m2, len(coords))
    want_c = oracle.conv_implicit_gemm(want_b, up.kernel.detach().cpu().numpy(), m2t, len(coords))
    assert rel_rms(c.feats.cpu().numpy(), want_c) < 1e-4
