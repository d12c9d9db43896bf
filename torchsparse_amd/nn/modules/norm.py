import torch
from torch import nn

from ...tensor import SparseTensor
from ..utils import fapply

__all__ = ["BatchNorm", "GroupNorm", "InstanceNorm"]


class _BatchNormTrain(torch.autograd.Function):
    """Training-mode batch norm of feats [N, C] on the library's kernels (statistics, running
    statistics, output; backward) — torch's channels-last kernels spend ~50 us per call on the
    column sums of a 90k-row matrix that a streaming pass reads in a tenth of that."""

    @staticmethod
    def forward(ctx, x, weight, bias, running_mean, running_var, momentum, eps):
        from ... import backend
        y, mean, invstd = backend.bn_forward_train(x, weight, bias, running_mean, running_var, momentum, eps)
        ctx.save_for_backward(x, weight, mean, invstd)
        ctx.has_bias = bias is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        from ... import backend
        x, weight, mean, invstd = ctx.saved_tensors
        dx, dweight, dbias = backend.bn_backward(dy.contiguous(), x, weight, mean, invstd)
        return (dx, dweight if weight is not None else None, dbias if ctx.has_bias else None,
                None, None, None, None)


class BatchNorm(nn.BatchNorm1d):
    """BatchNorm1d over the voxel axis of SparseTensor.feats (nn/modules/norm.py:13-17).  In
    training mode on the GPU the statistics, the output and the backward run on this library's
    kernels; everything else (evaluation mode, CPU tensors, channel counts that are not a
    multiple of 16 bytes, cumulative averaging with momentum=None) goes through torch."""

    def forward(self, input: SparseTensor) -> SparseTensor:
        from ... import backend
        x = input.feats
        if (self.training and self.momentum is not None
                and backend.bn_supported(x, self.weight, self.bias, self.running_mean, self.running_var)
                and (self.bias is None or self.weight is not None)):
            if self.num_batches_tracked is not None:
                self.num_batches_tracked.add_(1)
            rm = self.running_mean if self.track_running_stats else None
            rv = self.running_var if self.track_running_stats else None
            return input._like(_BatchNormTrain.apply(x, self.weight, self.bias, rm, rv, self.momentum, self.eps))
        return fapply(input, super().forward)


class InstanceNorm(nn.InstanceNorm1d):
    def forward(self, input: SparseTensor) -> SparseTensor:
        return fapply(input, super().forward)


class GroupNorm(nn.GroupNorm):
    """GroupNorm applied per batch sample (rows are grouped by coords[:, 0])."""

    def forward(self, input: SparseTensor) -> SparseTensor:
        feats, batch_col = input.feats, input.coords[:, 0]
        if feats.is_cuda:
            from ... import backend
            backend.flush_launches()
        out = torch.zeros_like(feats)
        for b in range(int(batch_col.max().item()) + 1):
            rows = batch_col == b
            sample = feats[rows].t().unsqueeze(0)  # [1, C, n_b]
            out[rows] = super().forward(sample).squeeze(0).t()
        return input._like(out)
