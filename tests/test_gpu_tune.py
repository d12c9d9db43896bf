"""The per-group tuner: it must leave a model that computes the same function, choose only
among the candidates, persist its choice and reload it."""
import numpy as np
import pytest
import torch

from helpers import random_coords, rel_rms

pytestmark = pytest.mark.gpu


def _net(spnn):
    from torch import nn
    return nn.Sequential(
        spnn.Conv3d(8, 16, 3), spnn.ReLU(True),
        spnn.Conv3d(16, 16, 3), spnn.ReLU(True),
        spnn.Conv3d(16, 32, 2, stride=2), spnn.ReLU(True),
        spnn.Conv3d(32, 32, 3), spnn.ReLU(True),
        spnn.Conv3d(32, 16, 2, stride=2, transposed=True))


def _samples(ts, n_samples, seed=0):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n_samples):
        coords = random_coords(rng, 4000, (24, 24, 12))
        feats = rng.standard_normal((len(coords), 8)).astype(np.float32)
        out.append({"input": ts.SparseTensor(torch.from_numpy(feats), torch.from_numpy(coords))})
    return out


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
