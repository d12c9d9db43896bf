"""spvoxelize: mean of the point features falling into each voxel, differentiable
(the reference's nn/functional/voxelize.py:11-59)."""
import torch
from torch.autograd import Function

from torchsparse_amd import backend

__all__ = ["spvoxelize"]


class VoxelizeFunction(Function):
    @staticmethod
    def forward(ctx, feats: torch.Tensor, coords: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
        feats = feats.contiguous()
        coords = coords.contiguous().int()
        counts = counts.contiguous().int()
        out = backend.voxelize_forward_cuda(feats, coords, counts)
        ctx.for_backwards = (coords, counts, feats.shape[0])
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        coords, counts, n = ctx.for_backwards
        return backend.voxelize_backward_cuda(grad_output.contiguous(), coords, counts, n), None, None


def spvoxelize(feats: torch.Tensor, coords: torch.Tensor, counts: torch.Tensor) -> torch.Tensor:
    """[len(counts), C]: out[v] = sum of feats[i] with coords[i] == v, divided by counts[v]."""
    return VoxelizeFunction.apply(feats, coords, counts)
