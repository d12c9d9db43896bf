"""Batching of samples for a data loader (the reference's utils/collate.py:11-60).

``sparse_collate`` joins SparseTensors with [N, 3] coordinates into one with [sum N, 4]
coordinates whose first column is the sample's position in the list; ``sparse_collate_fn``
applies it to the SparseTensor entries of a list of (possibly nested) dicts, stacks arrays and
tensors, and leaves everything else as a list."""
from typing import Any, List

import numpy as np
import torch

from ..tensor import SparseTensor

__all__ = ["sparse_collate", "sparse_collate_fn"]


def _as_tensor(v):
    return torch.tensor(v) if isinstance(v, np.ndarray) else v


def sparse_collate(inputs: List[SparseTensor]) -> SparseTensor:
    stride = inputs[0].stride
    rows, feats = [], []
    for b, sample in enumerate(inputs):
        sample.coords, sample.feats = _as_tensor(sample.coords), _as_tensor(sample.feats)
        if not isinstance(sample.coords, torch.Tensor):
            raise AssertionError(type(sample.coords))
        if not isinstance(sample.feats, torch.Tensor):
            raise AssertionError(type(sample.feats))
        if sample.stride != stride:
            raise AssertionError((sample.stride, stride))
        c = sample.coords
        rows.append(torch.cat((c.new_full((c.shape[0], 1), b, dtype=torch.int), c), dim=1))
        feats.append(sample.feats)
    return SparseTensor(coords=torch.cat(rows, dim=0), feats=torch.cat(feats, dim=0), stride=stride)


def sparse_collate_fn(inputs: List[Any]) -> Any:
    if not isinstance(inputs[0], dict):
        return inputs
    out = {}
    for name, first in inputs[0].items():
        column = [sample[name] for sample in inputs]
        if isinstance(first, dict):
            out[name] = sparse_collate_fn(column)
        elif isinstance(first, np.ndarray):
            out[name] = torch.stack([torch.tensor(v) for v in column], dim=0)
        elif isinstance(first, torch.Tensor):
            out[name] = torch.stack(column, dim=0)
        elif isinstance(first, SparseTensor):
            out[name] = sparse_collate(column)
        else:
            out[name] = column
    return out
