"""``torchsparse_amd.install_as("torchsparse")``: code written against the reference's import
block (backbones/unet.py:5-9 — ``import torchsparse``, ``from torchsparse import nn as spnn``,
``from torchsparse.nn import functional as F``, ``from torchsparse.utils...``) runs unchanged
and gets THIS package's module objects.  The small U-Net below is written for this test
against those names only; on the GPU its output is compared with the same network evaluated
layer by layer through the oracle."""
import numpy as np
import pytest
import torch

import torchsparse_amd

torchsparse_amd.install_as("torchsparse")

import torchsparse  # noqa: E402
import torchsparse.nn as spnn  # noqa: E402
from torchsparse import SparseTensor  # noqa: E402
from torchsparse.nn import functional as F  # noqa: E402
from torchsparse.utils.collate import sparse_collate_fn  # noqa: E402
from torchsparse.utils.quantize import sparse_quantize  # noqa: E402


class TinyUNet(torch.nn.Module):
    """stem -> strided -> submanifold -> transposed -> concat with the stem -> head."""

    def __init__(self, cin=4, width=16, classes=5):
        super().__init__()
        self.stem = torch.nn.Sequential(spnn.Conv3d(cin, width, 3), spnn.BatchNorm(width), spnn.ReLU(True))
        self.down = torch.nn.Sequential(spnn.Conv3d(width, 2 * width, 2, stride=2), spnn.BatchNorm(2 * width),
                                        spnn.ReLU(True))
        self.mid = torch.nn.Sequential(spnn.Conv3d(2 * width, 2 * width, 3), spnn.BatchNorm(2 * width),
                                       spnn.ReLU(True))
        self.up = torch.nn.Sequential(spnn.Conv3d(2 * width, width, 2, stride=2, transposed=True),
                                      spnn.BatchNorm(width), spnn.ReLU(True))
        self.head = spnn.Conv3d(2 * width, classes, 1)

    def forward(self, x):
        a = self.stem(x)
        b = self.up(self.mid(self.down(a)))
        return self.head(torchsparse.cat([b, a]))


def test_alias_gives_the_same_module_objects():
    import torchsparse.backends
    import importlib
    cc = importlib.import_module("torchsparse.nn.functional.conv.conv_config")
    cc_amd = importlib.import_module("torchsparse_amd.nn.functional.conv.conv_config")
    assert torchsparse is torchsparse_amd and spnn is torchsparse_amd.nn
    assert F is torchsparse_amd.nn.functional and cc is cc_amd
    assert torchsparse.backends is torchsparse_amd.backends
    assert SparseTensor is torchsparse_amd.SparseTensor
    from torchsparse.backbones import SparseResUNet42  # noqa: F401
    from torchsparse.utils.tune import tune
    assert torchsparse.tune is tune
    with pytest.raises(ImportError):
        import torchsparse.no_such_module  # noqa: F401
    torchsparse_amd.install_as("torchsparse")  # a second call changes nothing
    import sys
    sys.modules["_tsmi_other_pkg"] = np
    try:
        with pytest.raises(ImportError):
            torchsparse_amd.install_as("_tsmi_other_pkg")
    finally:
        del sys.modules["_tsmi_other_pkg"]


def test_sparse_quantize_against_a_dictionary_of_voxels():
    rng = np.random.default_rng(0)
    pts = rng.uniform(-3, 5, size=(4000, 3))
    for vs in (0.5, (0.25, 0.5, 1.0)):
        coords, index, inverse = sparse_quantize(pts, vs, return_index=True, return_inverse=True)
        size = np.array(vs if isinstance(vs, tuple) else (vs,) * 3)
        first = {}
        for i, p in enumerate(pts):
            first.setdefault(tuple(int(v) for v in np.floor(p / size)), i)
        want = sorted(first)  # ascending (x, y, z)
        assert coords.dtype == np.int32 and [tuple(c) for c in coords] == want
        assert [first[v] for v in want] == list(index)
        vox = np.floor(pts / size).astype(np.int32)
        assert np.array_equal(coords[inverse], vox)
        assert np.array_equal(sparse_quantize(pts, vs), coords)
    assert sparse_quantize(np.zeros((0, 3)), 1.0).shape == (0, 3)


def test_sparse_collate_fn_batches_dicts():
    samples = []
    for b, n in enumerate((5, 3)):
        c = torch.arange(3 * n, dtype=torch.int32).reshape(n, 3) + b
        samples.append({"input": SparseTensor(torch.full((n, 2), float(b)), c), "label": np.array([b, b + 1]),
                        "t": torch.tensor([b]), "name": f"s{b}", "nested": {"k": np.array([b])}})
    out = sparse_collate_fn(samples)
    st = out["input"]
    assert st.coords.shape == (8, 4) and st.coords.dtype == torch.int32
    assert st.coords[:, 0].tolist() == [0] * 5 + [1] * 3
    assert torch.equal(st.coords[5:, 1:], samples[1]["input"].coords)
    assert st.feats[:, 0].tolist() == [0.0] * 5 + [1.0] * 3
    assert out["label"].tolist() == [[0, 1], [1, 2]] and out["t"].tolist() == [[0], [1]]
    assert out["name"] == ["s0", "s1"] and out["nested"]["k"].tolist() == [[0], [1]]
    assert sparse_collate_fn([1, 2]) == [1, 2]


@pytest.mark.gpu
def test_network_written_against_the_reference_names_matches_the_oracle():
    import oracle
    from helpers import random_coords, rel_rms
    rng = np.random.default_rng(11)
    pts = rng.uniform(0, 40, size=(30000, 3))
    vox = sparse_quantize(pts, 1.0)
    coords_np = np.concatenate([np.zeros((len(vox), 1), np.int32), vox], 1)
    n = coords_np.shape[0]
    torch.manual_seed(5)
    model = TinyUNet().cuda().eval()
    for m in model.modules():  # non-trivial running statistics
        if isinstance(m, spnn.BatchNorm):
            m.running_mean.normal_(0, 0.2)
            m.running_var.uniform_(0.5, 1.5)
    feats = torch.randn(n, 4, device="cuda")
    with torch.no_grad():
        got = model(SparseTensor(feats, torch.from_numpy(coords_np).cuda())).feats.cpu().numpy()

    def bn_relu(y, bn):
        g, b = bn.weight.detach().cpu().numpy(), bn.bias.detach().cpu().numpy()
        mu, var = bn.running_mean.cpu().numpy(), bn.running_var.cpu().numpy()
        return np.maximum((y - mu) / np.sqrt(var + bn.eps) * g + b, 0)

    def w(seq):
        return seq[0].kernel.detach().cpu().numpy().astype(np.float32)

    m_subm1 = oracle.kmap_subm(coords_np, 3)
    m_down, c2 = oracle.kmap_downsample(coords_np, 2, 2, 0)
    m_subm2 = oracle.kmap_subm(c2, 3)
    m_up = oracle.transpose_map(m_down, n)
    x = feats.cpu().numpy()
    a = bn_relu(oracle.conv_implicit_gemm(x, w(model.stem), m_subm1, n), model.stem[1])
    d = bn_relu(oracle.conv_implicit_gemm(a, w(model.down), m_down, c2.shape[0]), model.down[1])
    d = bn_relu(oracle.conv_implicit_gemm(d, w(model.mid), m_subm2, c2.shape[0]), model.mid[1])
    b = bn_relu(oracle.conv_implicit_gemm(d, w(model.up), m_up, n), model.up[1])
    want = np.concatenate([b, a], 1) @ model.head.kernel.detach().cpu().numpy()
    assert got.shape == want.shape
    assert rel_rms(got, want) <= 1e-4  # fp32 end to end
