from typing import Callable

import torch

from ...tensor import SparseTensor

__all__ = ["fapply"]


def fapply(input: SparseTensor, fn: Callable[..., torch.Tensor], *args, **kwargs) -> SparseTensor:
    """Apply a dense op to the features; coordinates, stride and caches carry over
    (the reference's nn/utils/apply.py:10-22)."""
    return input._like(fn(input.feats, *args, **kwargs))
