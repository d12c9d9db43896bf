"""Small argument helpers (the reference's torchsparse/utils/utils.py)."""
from functools import lru_cache
from typing import Tuple

import torch

__all__ = ["make_ntuple", "make_tensor", "make_divisible"]


def make_ntuple(x, ndim: int) -> Tuple[int, ...]:
    """int -> (x,)*ndim; list / tuple / tensor -> tuple of python ints of length ndim."""
    if type(x) is tuple and len(x) == ndim:
        return x
    if isinstance(x, torch.Tensor):
        x = x.reshape(-1).tolist()
    if isinstance(x, (list, tuple)):
        out = tuple(int(v) for v in x)
    else:
        out = (int(x),) * ndim
    assert len(out) == ndim, x
    return out


@lru_cache()
def make_tensor(x: Tuple[int, ...], dtype: torch.dtype, device) -> torch.Tensor:
    return torch.tensor(x, dtype=dtype, device=device)


def make_divisible(x: int, divisor: int) -> int:
    return -(-x // divisor) * divisor
