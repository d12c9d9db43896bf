"""SpConv -> kernel-layout converter (the reference's examples/converter.py).  The layout
rule is pinned against the offset table (row k of a converted kernel must be the SpConv
weight at get_kernel_offsets(size)[k]) and, on the GPU, against torch's dense Conv3d."""
import numpy as np
import pytest
import torch

from torchsparse_amd.nn.utils.kernel import get_kernel_offsets
from torchsparse_amd.utils import convert_weights as cw

SIZES = [(3, 3, 3), (2, 2, 2), (5, 5, 5), (3, 1, 1), (1, 3, 3), (3, 3, 1), (1, 1, 3), (2, 2, 1), (1, 1, 1)]


def _spconv_weights(size, cin, cout, seed=0):
    g = torch.Generator().manual_seed(seed)
    v1 = torch.randn(*size, cin, cout, generator=g)
    v2 = v1.permute(4, 0, 1, 2, 3).contiguous()  # [Cout, kx, ky, kz, Cin], same filter
    return v1, v2


@pytest.mark.parametrize("size", SIZES)
def test_rows_follow_the_offset_table(size):
    cin, cout = 3, 5
    v1, v2 = _spconv_weights(size, cin, cout)
    k1, w1 = cw.convert_weights_v1("a.b.weight", {"a.b.weight": v1})
    k2, w2 = cw.convert_weights_v2("a.b.weight", {"a.b.weight": v2})
    assert k1 == k2 == "a.b.kernel"
    assert torch.equal(w1, w2)
    kvol = int(np.prod(size))
    if kvol == 1:
        assert w1.shape == (cin, cout) and torch.equal(w1, v1[0, 0, 0])
        return
    assert w1.shape == (kvol, cin, cout) and w1.is_contiguous()
    offsets = get_kernel_offsets(size).numpy()
    lo = [-(s // 2) + (1 if s % 2 == 0 else 0) for s in size]  # first offset per axis: 3 -> -1, 2 -> 0
    for k, (dx, dy, dz) in enumerate(offsets):
        assert torch.equal(w1[k], v1[dx - lo[0], dy - lo[1], dz - lo[2]]), (size, k)


def test_state_dict_and_checkpoint(tmp_path):
    v1, v2 = _spconv_weights((3, 3, 3), 4, 6)
    dense5d = torch.randn(6, 4, 3, 3, 3)  # a dense Conv3d weight: 5-d, must be left alone when keys are given

    class SubMConv3d(torch.nn.Module):  # stands for SpConv's class: matched by name
        def __init__(self):
            super().__init__()
            self.weight = torch.nn.Parameter(v2.clone())

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = SubMConv3d()
            self.dense = torch.nn.Conv3d(4, 6, 3)
            self.bn = torch.nn.BatchNorm1d(6)

    net = Net()
    assert list(cw.sparse_conv_weight_keys(net)) == ["conv.weight"]
    sd = {"conv.weight": v2, "dense.weight": dense5d, "bn.weight": torch.ones(6)}
    out = cw.convert_state_dict(sd, cw.sparse_conv_weight_keys(net))
    assert set(out) == {"conv.kernel", "dense.weight", "bn.weight"}
    assert torch.equal(out["dense.weight"], dense5d)
    assert torch.equal(out["conv.kernel"], cw.convert_weights_v1("w.weight", {"w.weight": v1})[1])
    # without keys every 5-d weight is taken for a sparse convolution weight
    assert set(cw.convert_state_dict(sd)) == {"conv.kernel", "dense.kernel", "bn.weight"}
    for field, legacy, w in (("state_dict", False, v2), ("model_state", True, v1)):
        before, after = tmp_path / f"{field}.pth", tmp_path / f"{field}_ts.pth"
        torch.save({field: {"conv.weight": w, "bn.weight": torch.ones(6)}, "epoch": 3}, before)
        cw.convert_model_weights(str(before), str(after), net, legacy=legacy)
        got = torch.load(after, weights_only=True)
        assert got["epoch"] == 3 and set(got[field]) == {"conv.kernel", "bn.weight"}
        assert torch.equal(got[field]["conv.kernel"], out["conv.kernel"])
    torch.save({"weights": {}}, tmp_path / "bad.pth")
    with pytest.raises(ValueError):
        cw.convert_model_weights(str(tmp_path / "bad.pth"), str(tmp_path / "x.pth"))
    with pytest.raises(ValueError):
        cw.convert_weights_v2("w.weight", {"w.weight": torch.zeros(3, 3)})


@pytest.mark.gpu
@pytest.mark.parametrize("size,stride", [((3, 3, 3), 1), ((5, 5, 5), 1), ((3, 1, 3), 1), ((1, 3, 1), 1),
                                         ((2, 2, 2), 2)])
def test_converted_kernel_matches_dense_conv3d(size, stride):
    """A converted SpConv filter applied by the sparse convolution equals torch's Conv3d
    with the same filter [Cout, Cin, kx, ky, kz] on the densified input (fp32, 1e-4 of RMS)."""
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    rng = np.random.default_rng(3)
    shape, cin, cout, n = (8, 6, 10), 8, 16, 150
    flat = rng.choice(int(np.prod(shape)), n, replace=False)
    xyz = np.stack(np.unravel_index(flat, shape), 1).astype(np.int32)
    coords = np.concatenate([np.zeros((n, 1), np.int32), xyz], 1)
    feats = rng.standard_normal((n, cin)).astype(np.float32)
    _, v2 = _spconv_weights(size, cin, cout, seed=5)
    _, kernel = cw.convert_weights_v2("c.weight", {"c.weight": v2})
    pad = tuple((k - 1) // 2 for k in size) if stride == 1 else 0
    layer = spnn.Conv3d(cin, cout, size, stride, pad).cuda()
    assert layer.kernel.shape == kernel.shape
    layer.kernel.data.copy_(kernel)
    with torch.no_grad():
        out = layer(ts.SparseTensor(torch.from_numpy(feats).cuda(), torch.from_numpy(coords).cuda()))
    dense = torch.zeros(1, cin, *shape, dtype=torch.float64)
    dense[0, :, xyz[:, 0], xyz[:, 1], xyz[:, 2]] = torch.from_numpy(feats.T.astype(np.float64))
    ref = torch.nn.functional.conv3d(dense, v2.permute(0, 4, 1, 2, 3).double(), stride=stride, padding=pad)
    oc = out.coords.cpu().numpy()
    want = ref[0][:, oc[:, 1], oc[:, 2], oc[:, 3]].T.numpy()
    got = out.feats.float().cpu().numpy()
    assert np.abs(got - want).max() <= 1e-4 * np.sqrt((want ** 2).mean())
    if stride == 1:
        assert np.array_equal(oc, coords)
