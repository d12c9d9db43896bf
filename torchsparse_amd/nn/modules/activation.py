from torch import nn

from ...tensor import SparseTensor
from ..utils import fapply

__all__ = ["ReLU", "LeakyReLU", "SiLU"]


def _on_feats(base):
    """A dense activation module that acts on SparseTensor.feats."""

    class _Wrapped(base):
        def forward(self, input: SparseTensor) -> SparseTensor:
            return fapply(input, super().forward)

    _Wrapped.__name__ = _Wrapped.__qualname__ = base.__name__
    return _Wrapped


ReLU = _on_feats(nn.ReLU)
LeakyReLU = _on_feats(nn.LeakyReLU)
SiLU = _on_feats(nn.SiLU)
