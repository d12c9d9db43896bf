from torch.nn import functional as _F

from ...tensor import SparseTensor
from ..utils import fapply

__all__ = ["relu", "silu", "leaky_relu"]


def relu(input: SparseTensor, inplace: bool = True) -> SparseTensor:
    return fapply(input, _F.relu, inplace=inplace)


def silu(input: SparseTensor, inplace: bool = True) -> SparseTensor:
    return fapply(input, _F.silu, inplace=inplace)


def leaky_relu(input: SparseTensor, negative_slope: float = 0.1, inplace: bool = True) -> SparseTensor:
    return fapply(input, _F.leaky_relu, negative_slope=negative_slope, inplace=inplace)
