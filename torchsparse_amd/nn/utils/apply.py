from typing import Callable

import torch

from ...tensor import SparseTensor

__all__ = ["fapply"]


def fapply(input: SparseTensor, fn: Callable[..., torch.Tensor], *args, **kwargs) -> SparseTensor:
    """Apply a dense op to the features; coordinates, stride and caches carry over
    (the reference's nn/utils/apply.py:10-22)."""
    if input.feats.is_cuda:
        from torchsparse_amd import backend
        backend.flush_launches()  # (the features may be the result of a convolution still with the launch thread)
    return input._like(fn(input.feats, *args, **kwargs))
