import math
from typing import Dict, List, Tuple, Union

import torch
from torch import nn

from ...tensor import SparseTensor
from ...utils import make_ntuple
from .. import functional as F

__all__ = ["Conv3d"]


class Conv3d(nn.Module):
    """Sparse 3-D convolution layer (the reference's nn/modules/conv.py:22-110).

    Parameters keep the reference's names and shapes so its checkpoints load:
    ``kernel`` is [K_vol, Cin, Cout] (or [Cin, Cout] for a 1x1x1 stride-1 layer),
    ``bias`` is [Cout] or absent.  On an axis with an odd kernel size and stride 1
    the padding is forced to (k-1)//2 (conv.py:42-48); elsewhere the user's value
    is kept."""

    def __init__(self, in_channels: int, out_channels: int,
                 kernel_size: Union[int, List[int], Tuple[int, ...]] = 3,
                 stride: Union[int, List[int], Tuple[int, ...]] = 1,
                 padding: Union[int, Tuple[int, ...]] = 0, dilation: int = 1, bias: bool = False,
                 transposed: bool = False, generative: bool = False, config: Dict = None) -> None:
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size = make_ntuple(kernel_size, ndim=3)
        self.stride = make_ntuple(stride, ndim=3)
        self.dilation = dilation
        self._dilation3 = make_ntuple(dilation, ndim=3)
        user_pad = make_ntuple(padding, ndim=3)
        self.padding = tuple((k - 1) // 2 if (k % 2 == 1 and s == 1) else p
                             for k, s, p in zip(self.kernel_size, self.stride, user_pad))
        self.transposed, self.generative = transposed, generative
        if generative:
            assert transposed
        self._config = config
        self.activation = None  # "relu" once a following ReLU has been fused in (see nn.utils.fuse)
        self.kernel_volume = self.kernel_size[0] * self.kernel_size[1] * self.kernel_size[2]
        pointwise = self.kernel_volume == 1 and self.stride == (1, 1, 1)
        shape = (in_channels, out_channels) if pointwise else (self.kernel_volume, in_channels, out_channels)
        self.kernel = nn.Parameter(torch.zeros(*shape))
        if bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self) -> None:
        fan = (self.out_channels if self.transposed else self.in_channels) * self.kernel_volume
        bound = 1.0 / math.sqrt(fan)
        with torch.no_grad():
            self.kernel.uniform_(-bound, bound)
            if self.bias is not None:
                self.bias.uniform_(-bound, bound)

    def extra_repr(self) -> str:
        parts = [f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}"]
        if self.stride != (1, 1, 1):
            parts.append(f"stride={self.stride}")
        if self.dilation != 1:
            parts.append(f"dilation={self.dilation}")
        if self.bias is None:
            parts.append("bias=False")
        if self.transposed:
            parts.append("transposed=True")
        if self.generative:
            parts.append("generative=True")
        return ", ".join(parts)

    def forward(self, input: SparseTensor, residual: torch.Tensor = None, out: torch.Tensor = None,
                also: torch.Tensor = None) -> SparseTensor:
        """``residual``: added before the activation; ``out`` / ``also``: where the result is
        written instead of a new tensor / a second time (functional.conv3d)."""
        if not self.training and not self.generative and self.activation in (None, "relu"):
            # a layer whose map is already cached, in inference: the short way (None: not that case)
            dilation = getattr(self, "_dilation3", None) or make_ntuple(self.dilation, ndim=3)
            params = self._parameters  # (plain dictionary look-ups: Module.__getattr__ costs 0.4 us each)
            done = F.conv3d_cached(input, params["kernel"], params["bias"], self.kernel_size, self.stride,
                                   dilation, self.transposed, self._config, residual, self.activation, out, also)
            if done is not None:
                return done
        return F.conv3d(input, weight=self.kernel, kernel_size=self.kernel_size, bias=self.bias,
                        stride=self.stride, padding=self.padding, dilation=self.dilation,
                        transposed=self.transposed, generative=self.generative,
                        config=self._config, training=self.training, residual=residual,
                        activation=self.activation, out=out, also=also)
