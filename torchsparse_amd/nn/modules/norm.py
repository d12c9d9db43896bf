import torch
from torch import nn

from ...tensor import SparseTensor
from ..utils import fapply

__all__ = ["BatchNorm", "GroupNorm", "InstanceNorm"]


class BatchNorm(nn.BatchNorm1d):
    """BatchNorm1d over the voxel axis of SparseTensor.feats."""

    def forward(self, input: SparseTensor) -> SparseTensor:
        return fapply(input, super().forward)


class InstanceNorm(nn.InstanceNorm1d):
    def forward(self, input: SparseTensor) -> SparseTensor:
        return fapply(input, super().forward)


class GroupNorm(nn.GroupNorm):
    """GroupNorm applied per batch sample (rows are grouped by coords[:, 0])."""

    def forward(self, input: SparseTensor) -> SparseTensor:
        feats, batch_col = input.feats, input.coords[:, 0]
        out = torch.zeros_like(feats)
        for b in range(int(batch_col.max().item()) + 1):
            rows = batch_col == b
            sample = feats[rows].t().unsqueeze(0)  # [1, C, n_b]
            out[rows] = super().forward(sample).squeeze(0).t()
        return input._like(out)
