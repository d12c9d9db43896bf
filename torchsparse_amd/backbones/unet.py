"""Sparse residual U-Net (the MinkUNet-shaped network; the reference's
backbones/unet.py).  Module names (stem, encoders.N, decoders.N.upsample / .fuse)
match the reference so its checkpoints load."""
from typing import List

import torch
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
        if not self.training and x.feats.is_cuda and not torch.is_grad_enabled():
            # inference: the convolution calls go through the library's launch thread
            from .. import backend
            with backend.launch_region():
                return self._forward(x)
        return self._forward(x)

    def _forward(self, x: SparseTensor) -> List[SparseTensor]:
        plan = self.__dict__.get("_placed_plan")
        if plan is None:
            plan = self.__dict__["_placed_plan"] = self._plan_placement()
        if plan and not self.training and x.feats.is_cuda:
            return self._forward_placed(x, plan)
        skips = [self.stem(x)]
        for enc in self.encoders:
            skips.append(enc(skips[-1]))
        outputs = list(skips)
        y = skips[-1]
        for i, dec in enumerate(self.decoders):
            y = dec["fuse"](cat([dec["upsample"](y), skips[3 - i]]))
            outputs.append(y)
        return outputs

    # In inference form (nn.utils.fuse_inference: norms folded, activations in the convolutions'
    # epilogues) the concatenations of the decoder cost nothing: the buffer [N, C_up + C_skip] of
    # a level is allocated when the level's skip is produced, the layer that produces the skip
    # writes it into the right-hand columns as well, and the transposed convolution of the decoder
    # writes its rows into the left-hand ones.

    def _plan_placement(self):
        """Per skip level (stem, encoders 0-2): (layers before the last, the last layer, the
        transposed convolution that returns to the level, its channels, the skip's channels);
        () when the model is not in inference form or a channel count does not fit."""
        from .modules.blocks import SparseResBlock
        stages = [self.stem] + list(self.encoders)[:3]
        plan = []
        for j, stage in enumerate(stages):
            layers = [m for m in stage if not isinstance(m, nn.Identity)]
            up = [m for m in self.decoders[3 - j]["upsample"] if not isinstance(m, nn.Identity)]
            last = layers[-1]
            if len(up) != 1 or not isinstance(up[0], spnn.Conv3d):
                return ()
            if isinstance(last, SparseResBlock):
                if not getattr(last, "_fused_tail", False):
                    return ()
                c_skip = last.main[0].out_channels
            elif isinstance(last, spnn.Conv3d):
                c_skip = last.out_channels
            else:
                return ()
            if any(isinstance(m, spnn.BatchNorm) for m in stage.modules()):
                return ()
            c_up = up[0].out_channels
            if c_up % 8 or c_skip % 8:
                return ()
            plan.append((tuple(layers[:-1]), last, up[0], c_up, c_skip))
        return tuple(plan)

    def _forward_placed(self, x: SparseTensor, plan) -> List[SparseTensor]:
        from ..backend import ColumnSlice
        from ..nn.utils.fuse import call_module
        skips, buffers = [], []
        y = x
        for before, last, _, c_up, c_skip in plan:
            for m in before:
                y = call_module(m, y)
            buf = y.feats.new_empty(y.feats.shape[0], c_up + c_skip)
            y = call_module(last, y, also=ColumnSlice(buf, c_up, c_skip))
            skips.append(y)
            buffers.append(buf)
        y = call_module(self.encoders[3], y)
        outputs = skips + [y]
        for i, dec in enumerate(self.decoders):
            _, _, up, c_up, _ = plan[3 - i]
            buf = buffers[3 - i]
            # (the result tensor of a call placed through a ColumnSlice is the whole buffer)
            y = call_module(dec["fuse"], call_module(up, y, out=ColumnSlice(buf, 0, c_up)))
            outputs.append(y)
        return outputs


class SparseResUNet42(SparseResUNet):
    def __init__(self, **kwargs) -> None:
        super().__init__(stem_channels=32, encoder_channels=[32, 64, 128, 256],
                         decoder_channels=[256, 128, 96, 96], **kwargs)
