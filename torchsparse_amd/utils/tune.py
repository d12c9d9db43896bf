"""Per-group tuner of the convolution configuration (the reference's utils/tune.py:373-654).

Layers that share a kernel map — same fine tensor stride, kernel size, stride and dilation —
form a group and must share dataflow and sort settings, because the map is built once per
group with the products of one configuration.  ``tune`` runs the model on a few samples,
times every candidate configuration of every group (all other groups at the default), keeps
the fastest per group, writes the choice to ``save_dir/tune_tag`` and sets it on the model's
``Conv3d`` modules.

Candidates per dataflow:
  ImplicitGEMM   unsorted (small wide layers over pair segments where the library knows the map
                 to be thin; then the same with that form forced on and forced off), and sorted
                 with 1 to 4 mask splits
  FetchOnDemand  one candidate (fusion does not change this implementation's kernels)
  GatherScatter  one candidate (epsilon / mm_thresh only steer grouping in the reference and
                 change neither results nor launches here, utils/tune.py:322-352 sweeps them)

The timed region is the whole model call on the stream with a cleared tensor cache, as in
the reference (utils/tune.py:87-110): the cost of building a group's map products counts
against the configuration that needs them.  Times are HIP-event times, the per-candidate
figure is the median over the samples of the faster of two runs; the first candidate in the order above that is
within 2 % of the fastest wins.  The choice is stored with plain types only (dataflow by
name) and read back with ``torch.load(weights_only=True)``."""
import os
from collections import defaultdict
from typing import Any, Callable, Dict, Iterable, List, Tuple

import torch
from torch import nn

import torchsparse_amd
from torchsparse_amd import SparseTensor
from torchsparse_amd.nn import functional as F
from torchsparse_amd.utils import make_ntuple

__all__ = ["tune"]

_TUNED_KEYS = ("epsilon", "mm_thresh", "split_mask_num", "split_mask_num_bwd", "dataflow", "ifsort",
               "FOD_fusion", "pair_segments")


def _map_tensors(x, fn):
    if isinstance(x, dict):
        return {k: _map_tensors(v, fn) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return type(x)(_map_tensors(v, fn) for v in x)
    if isinstance(x, SparseTensor):
        y = fn(x)
        return y if isinstance(y, SparseTensor) else x
    return x


def _clear_caches(inputs) -> None:
    def clear(t: SparseTensor):
        t._caches.cmaps.clear()
        t._caches.kmaps.clear()
        t._caches.hashmaps.clear()
    _map_tensors(inputs, clear)


def _conv_modules(model: nn.Module):
    from torchsparse_amd.nn import Conv3d
    return [(name, m) for name, m in model.named_modules()
            if isinstance(m, Conv3d) and m.kernel.dim() == 3]


def _groups_of(model: nn.Module, inputs) -> Dict[str, Tuple[Any, ...]]:
    """One forward with hooks: layer name -> key of the kernel map it uses."""
    name_to_group: Dict[str, Tuple[Any, ...]] = {}

    def record(module, args, output, name):
        stride = args[0].stride
        if module.transposed:
            ms = make_ntuple(module.stride, ndim=3)
            stride = tuple(stride[a] // ms[a] for a in range(3))
        name_to_group[name] = (tuple(stride), tuple(make_ntuple(module.kernel_size, ndim=3)),
                               tuple(make_ntuple(module.stride, ndim=3)),
                               tuple(make_ntuple(module.dilation, ndim=3)))

    handles = [m.register_forward_hook(lambda mod, a, o, name=name: record(mod, a, o, name))
               for name, m in _conv_modules(model)]
    try:
        model(inputs)
    finally:
        for h in handles:
            h.remove()
    return name_to_group


def _candidates(dataflow_range: List, tune_with_bwd: bool) -> List[Dict]:
    out = []
    if F.Dataflow.ImplicitGEMM in dataflow_range:
        out.append(dict(dataflow=F.Dataflow.ImplicitGEMM, ifsort=False, split_mask_num=1,
                        split_mask_num_bwd=1))
        # small, wide layers over pair segments, forced on and off (the default decides from what
        # the library knows of the map; layers without a variant run the same either way)
        for forced in (True, False):
            out.append(dict(dataflow=F.Dataflow.ImplicitGEMM, ifsort=False, split_mask_num=1,
                            split_mask_num_bwd=1, pair_segments=forced))
        for split in range(1, 5):
            out.append(dict(dataflow=F.Dataflow.ImplicitGEMM, ifsort=True, split_mask_num=split,
                            split_mask_num_bwd=split if tune_with_bwd else 1))
    if F.Dataflow.FetchOnDemand in dataflow_range:
        out.append(dict(dataflow=F.Dataflow.FetchOnDemand, ifsort=False, split_mask_num=1,
                        split_mask_num_bwd=1))
    if F.Dataflow.GatherScatter in dataflow_range:
        out.append(dict(dataflow=F.Dataflow.GatherScatter, ifsort=False, split_mask_num=1,
                        split_mask_num_bwd=1))
    return out


def _set_configs(model: nn.Module, names, overrides: Dict) -> None:
    """Default configuration on every convolution, `overrides` on the layers in `names`."""
    names = set(names)
    for name, m in _conv_modules(model):
        cfg = F.conv_config.get_default_conv_config().copy()
        if name in names:
            for k, v in overrides.items():
                cfg[k] = v
        m._config = cfg


def _time_call(model: nn.Module, inputs, with_backward: bool, runs: int = 2) -> float:
    """Milliseconds of one call with cleared caches: the faster of `runs` runs, so that what a
    configuration change leaves behind for the first run after it (allocator pools sized for
    the previous candidate, kernels not yet loaded) does not count against the candidate."""
    best = float("inf")
    for _ in range(runs):
        _clear_caches(inputs)
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        out = model(inputs)
        if with_backward:
            feats = out.feats if isinstance(out, SparseTensor) else out
            if isinstance(feats, (list, tuple)):
                feats = feats[-1].feats if isinstance(feats[-1], SparseTensor) else feats[-1]
            feats.backward(torch.randn_like(feats) * 1e-3)
        stop.record()
        stop.synchronize()
        best = min(best, start.elapsed_time(stop))
    return best


def _median(values: List[float]) -> float:
    v = sorted(values)
    return v[len(v) // 2]


def tune(model: nn.Module, data_loader: Iterable, n_samples: int = 100,
         collect_fn: Callable = lambda data: data, enable_fp16: bool = False,
         save_dir: str = ".torchsparse-tune", tune_tag: str = "temp", force_retune: bool = False,
         dataflow_range: List = (F.Dataflow.ImplicitGEMM,), dataflow_prune: bool = False,
         tune_with_bwd: bool = False, verbose: bool = True, skip_warning: bool = False) -> Dict:
    """Choose, per kernel-map group, the fastest convolution configuration for ``model`` on
    samples of ``data_loader`` (``model(collect_fn(sample))``) and set it on the model.
    Returns the chosen group configurations.  ``dataflow_prune`` first picks each group's
    dataflow from one representative candidate per dataflow, then tunes only inside it."""
    if not torchsparse_amd.backends.benchmark:
        if not skip_warning and verbose:
            print("Warning: to use tuning, torchsparse.backends.benchmark is automatically set to be true.")
        torchsparse_amd.backends.benchmark = True
    dataflow_range = list(dataflow_range)
    path = os.path.join(save_dir, tune_tag)

    def prepare(sample):
        inputs = collect_fn(sample)
        if enable_fp16:
            inputs = _map_tensors(inputs, lambda t: t.half())
        return _map_tensors(inputs, lambda t: t.cuda())

    if os.path.exists(path) and not force_retune:
        if verbose:
            print("Load existing tuned group configs")
        name_to_group, stored = torch.load(path, weights_only=True)
        group_configs = {g: dict(c, dataflow=F.Dataflow[c["dataflow"]]) for g, c in stored.items()}
    else:
        model = model.cuda()
        if enable_fp16:
            model = model.half()
        saved = {name: m._config for name, m in _conv_modules(model)}
        times: Dict[Tuple, Dict[int, List[float]]] = defaultdict(lambda: defaultdict(list))
        name_to_group: Dict[str, Tuple[Any, ...]] = {}
        group_to_names: Dict[Tuple, List[str]] = defaultdict(list)
        candidates = _candidates(dataflow_range, tune_with_bwd)
        allowed: Dict[Tuple, List[int]] = {}
        count = 0
        for sample in data_loader:
            inputs = prepare(sample)
            ctx = torch.enable_grad() if tune_with_bwd else torch.no_grad()
            with ctx:
                if count == 0:
                    _set_configs(model, (), {})
                    name_to_group = _groups_of(model, inputs)
                    for name, g in name_to_group.items():
                        group_to_names[g].append(name)
                    for _ in range(3):  # warm-up: code objects, allocator pools
                        _time_call(model, inputs, tune_with_bwd)
                    if dataflow_prune and len(dataflow_range) > 1:
                        # one representative per dataflow: its first candidate
                        first = {}
                        for i, c in enumerate(candidates):
                            first.setdefault(c["dataflow"], i)
                        for g, names in group_to_names.items():
                            best = None
                            for flow, i in first.items():
                                _set_configs(model, names, candidates[i])
                                t = _time_call(model, inputs, tune_with_bwd)
                                if best is None or t < best[0]:
                                    best = (t, flow)
                            allowed[g] = [i for i, c in enumerate(candidates) if c["dataflow"] == best[1]]
                for g, names in group_to_names.items():
                    for i in allowed.get(g, range(len(candidates))):
                        _set_configs(model, names, candidates[i])
                        times[g][i].append(_time_call(model, inputs, tune_with_bwd))
            count += 1
            if count >= n_samples:
                break
        if count == 0:
            raise ValueError("tune: the data loader yielded no sample")
        group_configs = {}
        for g, per_candidate in times.items():
            # the first (simplest) candidate within 2 % of the fastest: differences below the
            # timing noise must not switch a group to a configuration with more map products
            fastest = min(_median(t) for t in per_candidate.values())
            best_i = min(i for i, t in per_candidate.items() if _median(t) <= 1.02 * fastest)
            cfg = F.conv_config.get_default_conv_config().copy()
            for k, v in candidates[best_i].items():
                cfg[k] = v
            group_configs[g] = {k: cfg[k] for k in _TUNED_KEYS}
            if verbose:
                ms = {i: round(_median(t), 3) for i, t in per_candidate.items()}
                print(f"group {g}: candidate times (ms) {ms} -> {candidates[best_i]}")
        for name, m in _conv_modules(model):
            m._config = saved[name]
        if verbose:
            print("Save tuned group configs to", path)
        os.makedirs(save_dir, exist_ok=True)
        # plain types only (the dataflow by name), so that the file loads without unpickling code
        torch.save((name_to_group, {g: dict(c, dataflow=c["dataflow"].name)
                                    for g, c in group_configs.items()}), path)

    for name, m in _conv_modules(model):
        g = name_to_group.get(name)
        if g is None or g not in group_configs:
            continue
        cfg = m._config
        if cfg is None:
            glb = F.conv_config.get_global_conv_config()
            cfg = glb.copy() if glb is not None else F.conv_config.get_default_conv_config().copy()
        else:
            cfg = cfg.copy()
        for k in _TUNED_KEYS:
            cfg[k] = group_configs[g][k]
        m._config = cfg
    return group_configs
