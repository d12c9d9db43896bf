"""VoxelResBackBone8x-style sparse detection backbone: the layer shapes OpenPCDet
plugs sparse convolutions into (the reference's
examples/openpcdet/pcdet_plugin/models/backbones_3d/backbone3d.py:39-80 and
backbone_voxel_next.py:57-138).  Coordinates are (b, z, y, x)."""
from typing import Dict

import torch
from torch import nn

from .. import nn as spnn
from ..nn.utils.fuse import call_module
from ..tensor import SparseTensor

__all__ = ["SparseBasicBlock", "VoxelResBackBone8x"]


class SparseBasicBlock(nn.Module):
    """Two submanifold k3 convs with bias, norm after each, identity shortcut."""

    def __init__(self, channels: int) -> None:
        super().__init__()
        self.conv1 = spnn.Conv3d(channels, channels, 3, bias=True)
        self.bn1 = spnn.BatchNorm(channels, eps=1e-3, momentum=0.01)
        self.relu = spnn.ReLU(True)
        self.conv2 = spnn.Conv3d(channels, channels, 3, bias=True)
        self.bn2 = spnn.BatchNorm(channels, eps=1e-3, momentum=0.01)

    def forward(self, x: SparseTensor) -> SparseTensor:
        if getattr(self, "_fused_tail", False):
            # after nn.utils.fuse_inference(): norms folded into the convolutions, ReLU and
            # the shortcut add in their epilogues
            mods = self._modules
            return call_module(mods["conv2"], call_module(mods["conv1"], x), residual=x.feats)
        out = self.bn2(self.conv2(self.relu(self.bn1(self.conv1(x)))))
        return self.relu(out + x)


def _block(cin, cout, kernel_size, stride=1, padding=0):
    return nn.Sequential(spnn.Conv3d(cin, cout, kernel_size, stride=stride, padding=padding),
                         spnn.BatchNorm(cout, eps=1e-3, momentum=0.01), spnn.ReLU(True))


class VoxelResBackBone8x(nn.Module):
    def __init__(self, in_channels: int = 5) -> None:
        super().__init__()
        self.conv_input = _block(in_channels, 16, 3)
        self.conv1 = nn.Sequential(SparseBasicBlock(16), SparseBasicBlock(16))
        self.conv2 = nn.Sequential(_block(16, 32, 3, 2, 1), SparseBasicBlock(32), SparseBasicBlock(32))
        self.conv3 = nn.Sequential(_block(32, 64, 3, 2, 1), SparseBasicBlock(64), SparseBasicBlock(64))
        self.conv4 = nn.Sequential(_block(64, 128, 3, 2, (0, 1, 1)), SparseBasicBlock(128),
                                   SparseBasicBlock(128))
        self.conv_out = _block(128, 128, (3, 1, 1), (2, 1, 1), 0)

    def forward(self, x: SparseTensor) -> Dict[str, SparseTensor]:
        if not self.training and x.feats.is_cuda and not torch.is_grad_enabled():
            # inference: the convolution calls go through the library's launch thread
            from .. import backend
            with backend.launch_region():
                return self._forward(x)
        return self._forward(x)

    def _forward(self, x: SparseTensor) -> Dict[str, SparseTensor]:
        x = self.conv_input(x)
        c1 = self.conv1(x)
        c2 = self.conv2(c1)
        c3 = self.conv3(c2)
        c4 = self.conv4(c3)
        return {"x_conv1": c1, "x_conv2": c2, "x_conv3": c3, "x_conv4": c4, "out": self.conv_out(c4)}
