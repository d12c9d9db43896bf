"""Building blocks of the sparse backbones.  Sub-module names and order follow the
reference (backbones/modules/blocks.py) so its state dicts load unchanged:
ConvBlock / ConvTransposeBlock are Sequential(conv, norm, relu) with indices 0-2;
ResBlock has ``main`` (conv, norm, relu, conv, norm), ``shortcut`` and ``relu``."""
from typing import List, Tuple, Union

import numpy as np
from torch import nn

from ... import nn as spnn
from ...nn.utils.fuse import call_module
from ...tensor import SparseTensor

__all__ = ["SparseConvBlock", "SparseConvTransposeBlock", "SparseResBlock"]

_Size = Union[int, List[int], Tuple[int, ...]]


def _conv_bn(cin: int, cout: int, kernel_size: _Size, act: bool, **conv_kwargs):
    layers = [spnn.Conv3d(cin, cout, kernel_size, **conv_kwargs), spnn.BatchNorm(cout)]
    if act:
        layers.append(spnn.ReLU(True))
    return layers


class _Chain(nn.Sequential):
    """nn.Sequential that skips nn.Identity children (what nn.utils.fuse_inference leaves in
    place of folded norms and activations) instead of calling them."""

    def forward(self, x):
        for m in self._modules.values():
            if m.__class__ is not nn.Identity:
                x = call_module(m, x)
        return x


class SparseConvBlock(_Chain):
    def __init__(self, in_channels: int, out_channels: int, kernel_size: _Size, stride: _Size = 1,
                 dilation: int = 1) -> None:
        super().__init__(*_conv_bn(in_channels, out_channels, kernel_size, True, stride=stride,
                                   dilation=dilation))


class SparseConvTransposeBlock(_Chain):
    def __init__(self, in_channels: int, out_channels: int, kernel_size: _Size, stride: _Size = 1,
                 dilation: int = 1) -> None:
        super().__init__(*_conv_bn(in_channels, out_channels, kernel_size, True, stride=stride,
                                   dilation=dilation, transposed=True))


class SparseResBlock(nn.Module):
    """relu(main(x) + shortcut(x)); the shortcut is a 1x1x1 conv + norm when the
    channel count or the stride changes, the identity otherwise."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size: _Size, stride: _Size = 1,
                 dilation: int = 1) -> None:
        super().__init__()
        self.main = nn.Sequential(
            *_conv_bn(in_channels, out_channels, kernel_size, True, stride=stride, dilation=dilation),
            *_conv_bn(out_channels, out_channels, kernel_size, False, dilation=dilation))
        if in_channels != out_channels or int(np.prod(stride)) != 1:
            self.shortcut = nn.Sequential(*_conv_bn(in_channels, out_channels, 1, False, stride=stride))
        else:
            self.shortcut = nn.Identity()
        self.relu = spnn.ReLU(True)

    def forward(self, x: SparseTensor, also=None) -> SparseTensor:
        """``also``: a [N, out_channels] view the block's result is written into as well (the
        place a later concatenation wants it)."""
        if getattr(self, "_fused_tail", False):
            # after nn.utils.fuse_inference(): norms are folded into the convolutions and the
            # shortcut add + ReLU run in the epilogue of the block's last convolution
            layers = self.__dict__.get("_fused_layers")
            if layers is None:  # the convolutions of `main` (its folded norms are placeholders)
                layers = self.__dict__["_fused_layers"] = tuple(
                    m for m in list(self.main)[:-1] if not isinstance(m, nn.Identity))
            shortcut = self._modules["shortcut"]
            residual = x.feats if shortcut.__class__ is nn.Identity else call_module(shortcut, x).feats
            y = x
            for layer in layers[:-1]:
                y = call_module(layer, y)
            if also is None:
                return call_module(layers[-1], y, residual=residual)
            return call_module(layers[-1], y, residual=residual, also=also)
        out = self.relu(self.main(x) + self.shortcut(x))
        if also is not None:
            if not hasattr(also, "copy_"):  # a backend.ColumnSlice
                first = (also.ptr - also.buffer.data_ptr()) // also.buffer.element_size()
                also = also.buffer[:, first:first + also.cols]
            also.copy_(out.feats)
        return out
