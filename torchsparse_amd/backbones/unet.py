"""Sparse residual U-Net (the MinkUNet-shaped network; the reference's
backbones/unet.py).  Module names (stem, encoders.N, decoders.N.upsample / .fuse)
match the reference so its checkpoints load."""
from typing import List

from torch import nn

from .. import nn as spnn
from ..operators import cat
from ..tensor import SparseTensor
from .modules import SparseConvBlock, SparseConvTransposeBlock, SparseResBlock

__all__ = ["SparseResUNet", "SparseResUNet42"]


class SparseResUNet(nn.Module):
    """stem (two k3 conv blocks) -> 4 x [k2 s2 down, 2 res blocks] -> 4 x [k2 s2
    transposed up, concat with the skip of the same stride, 2 res blocks].
    forward() returns the feature pyramid [stem, enc0..enc3, dec0..dec3]."""

    def __init__(self, stem_channels: int, encoder_channels: List[int], decoder_channels: List[int], *,
                 in_channels: int = 4, width_multiplier: float = 1.0) -> None:
        super().__init__()
        assert len(encoder_channels) == 4 and len(decoder_channels) == 4
        self.stem_channels, self.encoder_channels = stem_channels, encoder_channels
        self.decoder_channels, self.in_channels = decoder_channels, in_channels
        self.width_multiplier = width_multiplier
        nc = [int(width_multiplier * c) for c in [stem_channels] + encoder_channels + decoder_channels]

        self.stem = nn.Sequential(
            spnn.Conv3d(in_channels, nc[0], 3), spnn.BatchNorm(nc[0]), spnn.ReLU(True),
            spnn.Conv3d(nc[0], nc[0], 3), spnn.BatchNorm(nc[0]), spnn.ReLU(True))
        self.encoders = nn.ModuleList(
            nn.Sequential(SparseConvBlock(nc[i], nc[i], 2, stride=2),
                          SparseResBlock(nc[i], nc[i + 1], 3),
                          SparseResBlock(nc[i + 1], nc[i + 1], 3))
            for i in range(4))
        self.decoders = nn.ModuleList(
            nn.ModuleDict({
                "upsample": SparseConvTransposeBlock(nc[i + 4], nc[i + 5], 2, stride=2),
                "fuse": nn.Sequential(SparseResBlock(nc[i + 5] + nc[3 - i], nc[i + 5], 3),
                                      SparseResBlock(nc[i + 5], nc[i + 5], 3)),
            }) for i in range(4))

    def forward(self, x: SparseTensor) -> List[SparseTensor]:
        skips = [self.stem(x)]
        for enc in self.encoders:
            skips.append(enc(skips[-1]))
        outputs = list(skips)
        y = skips[-1]
        for i, dec in enumerate(self.decoders):
            y = dec["fuse"](cat([dec["upsample"](y), skips[3 - i]]))
            outputs.append(y)
        return outputs


class SparseResUNet42(SparseResUNet):
    def __init__(self, **kwargs) -> None:
        super().__init__(stem_channels=32, encoder_channels=[32, 64, 128, 256],
                         decoder_channels=[256, 128, 96, 96], **kwargs)
