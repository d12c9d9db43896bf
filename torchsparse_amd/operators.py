"""Tensor-level operators (the reference's torchsparse/operators.py:12-16)."""
from typing import List

import torch

from .tensor import SparseTensor

__all__ = ["cat"]


def cat(inputs: List[SparseTensor]) -> SparseTensor:
    """Channel-wise concatenation of tensors that share coordinates (and row order)."""
    head = inputs[0]
    out = SparseTensor(feats=torch.cat([t.feats for t in inputs], dim=1), coords=head.coords,
                       stride=head.stride)
    out._caches = head._caches
    return out
