"""The per-group tuner: it must leave a model that computes the function the oracle computes,
choose only among the candidates (each of which computes that function too), persist its
choice and reload it (the reference's utils/tune.py:373-654)."""
import numpy as np
import pytest
import torch

import oracle
from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu


def _net(spnn):
    from torch import nn
    return nn.Sequential(
        spnn.Conv3d(8, 16, 3), spnn.ReLU(True),
        spnn.Conv3d(16, 16, 3), spnn.ReLU(True),
        spnn.Conv3d(16, 128, 2, stride=2), spnn.ReLU(True),
        spnn.Conv3d(128, 192, 3), spnn.ReLU(True),  # (wide enough for the pair-segment form)
        spnn.Conv3d(192, 16, 2, stride=2, transposed=True))


def _samples(ts, n_samples, seed=0):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n_samples):
        coords = random_coords(rng, 4000, (24, 24, 12))
        feats = rng.standard_normal((len(coords), 8)).astype(np.float32)
        out.append({"input": ts.SparseTensor(torch.from_numpy(feats), torch.from_numpy(coords))})
    return out


def _oracle_net(model, spnn, feats, coords):
    """The network of _net evaluated layer by layer on the CPU: the oracle's maps and its
    double-accumulated convolution, fed the parameters as stored (fp16 values, fp32 arithmetic
    between the layers)."""
    w = [m.kernel.detach().float().cpu().numpy() for m in model.modules() if isinstance(m, spnn.Conv3d)]
    n = coords.shape[0]
    subm1 = oracle.kmap_subm(coords, 3)
    down, c2 = oracle.kmap_downsample(coords, 2, 2, 0)
    subm2 = oracle.kmap_subm(c2, 3)
    up = oracle.transpose_map(down, n)
    x = np.maximum(oracle.conv_implicit_gemm(feats, w[0], subm1, n), 0)
    x = np.maximum(oracle.conv_implicit_gemm(x, w[1], subm1, n), 0)
    x = np.maximum(oracle.conv_implicit_gemm(x, w[2], down, c2.shape[0]), 0)
    x = np.maximum(oracle.conv_implicit_gemm(x, w[3], subm2, c2.shape[0]), 0)
    return oracle.conv_implicit_gemm(x, w[4], up, n)


def test_every_candidate_configuration_matches_the_oracle():
    """Each configuration the tuner may time — unsorted (as the library decides, and with the
    pair-segment form of the wide layer forced on and off), sorted with 1 to 4 mask splits,
    fetch-on-demand, gather-scatter — set on every group at once, against the oracle."""
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    from torchsparse_amd.utils import tune as T
    torch.manual_seed(1)
    model = _net(spnn).cuda().half()
    probe = _samples(ts, 1, seed=4)[0]["input"]
    coords = probe.coords.numpy()
    x16 = probe.feats.half()
    want = _oracle_net(model, spnn, x16.float().numpy(), coords)
    names = [name for name, _ in T._conv_modules(model)]
    flows = [F.Dataflow.ImplicitGEMM, F.Dataflow.FetchOnDemand, F.Dataflow.GatherScatter]
    cands = T._candidates(flows, tune_with_bwd=True)
    assert len(cands) == 9
    from torchsparse_amd import backend
    for cand in cands:
        T._set_configs(model, names, cand)
        backend._segments_of.clear()
        torch.cuda.synchronize()
        backend.release_scratch()  # (and what the forward before asked to be built ahead of this one)
        with torch.no_grad():
            got = model(ts.SparseTensor(x16.cuda(), probe.coords.cuda())).feats.float().cpu().numpy()
        # the wide layer ran over pair segments exactly when the candidate forces that form
        assert bool(backend._segments_of) == (cand.get("pair_segments") is True), cand
        assert rel_rms(got, want) < 2e-2, cand  # five fp16 layers deep: 1e-2 per layer does not compound past this


@pytest.mark.parametrize("with_bwd", [False, True])
def test_tune_keeps_the_function_and_persists_the_choice(tmp_path, with_bwd):
    import torchsparse_amd as ts
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.nn import functional as F
    from torchsparse_amd.utils.tune import tune
    torch.manual_seed(0)
    model = _net(spnn).cuda().half()
    samples = _samples(ts, 3)
    probe = samples[0]["input"].cuda().half()
    with torch.no_grad():
        before = model(ts.SparseTensor(probe.feats, probe.coords)).feats.float().cpu().numpy()
    flows = [F.Dataflow.ImplicitGEMM, F.Dataflow.FetchOnDemand, F.Dataflow.GatherScatter]
    chosen = tune(model, samples, n_samples=2, collect_fn=lambda d: d["input"], enable_fp16=True,
                  save_dir=str(tmp_path), tune_tag="t", dataflow_range=flows, dataflow_prune=with_bwd,
                  tune_with_bwd=with_bwd, verbose=False)
    # groups: subm k3 at stride 1, k2s2 (shared by the strided and the transposed layer), subm k3 at stride 2
    assert len(chosen) == 3
    for cfg in chosen.values():
        assert cfg["dataflow"] in flows and cfg["split_mask_num"] in (1, 2, 3, 4)
        assert cfg["ifsort"] in (False, True)
    layers = [m for m in model.modules() if isinstance(m, spnn.Conv3d)]
    assert layers[0]._config["dataflow"] == layers[1]._config["dataflow"]      # same group
    assert layers[2]._config["dataflow"] == layers[4]._config["dataflow"]      # same map
    assert layers[2]._config["ifsort"] == layers[4]._config["ifsort"]
    with torch.no_grad():
        after = model(ts.SparseTensor(probe.feats, probe.coords)).feats.float().cpu().numpy()
    assert rel_rms(after, before) < 1e-2
    want = _oracle_net(model, spnn, probe.feats.float().cpu().numpy(), probe.coords.cpu().numpy())
    assert rel_rms(after, want) < 2e-2  # the tuned model against the oracle, five fp16 layers deep
    # a second model picks the stored choice up without measuring anything
    again = _net(spnn).cuda().half()
    loaded = tune(again, [], save_dir=str(tmp_path), tune_tag="t", dataflow_range=flows, verbose=False)
    assert loaded == chosen
    for a, b in zip([m for m in again.modules() if isinstance(m, spnn.Conv3d)], layers):
        for key in ("dataflow", "ifsort", "split_mask_num", "split_mask_num_bwd"):
            assert a._config[key] == b._config[key]


def test_tune_needs_a_sample(tmp_path):
    import torchsparse_amd as ts  # noqa: F401
    from torchsparse_amd import nn as spnn
    from torchsparse_amd.utils.tune import tune
    with pytest.raises(ValueError, match="no sample"):
        tune(_net(spnn).cuda(), [], save_dir=str(tmp_path), tune_tag="none", verbose=False)
