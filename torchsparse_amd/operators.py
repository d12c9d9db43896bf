"""Tensor-level operators (the reference's torchsparse/operators.py:12-16)."""
from typing import List

import torch

from .tensor import SparseTensor

__all__ = ["cat"]


def cat(inputs: List[SparseTensor]) -> SparseTensor:
    """Channel-wise concatenation of tensors that share coordinates (and row order)."""
    if inputs[0].feats.is_cuda:
        from . import backend
        backend.flush_launches()  # (the inputs may be results of convolutions still with the launch thread)
    head = inputs[0]
    out = SparseTensor(feats=torch.cat([t.feats for t in inputs], dim=1), coords=head.coords,
                       stride=head.stride)
    out._caches = head._caches
    return out
