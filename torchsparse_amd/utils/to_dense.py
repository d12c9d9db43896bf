"""to_dense: sparse rows into a dense [B, X, Y, Z, C] tensor, differentiable
(the reference's utils/to_dense.py:13-64)."""
from typing import Tuple

import torch
from torch.autograd import Function

__all__ = ["to_dense"]


class ToDenseFunction(Function):
    @staticmethod
    def forward(ctx, feats: torch.Tensor, coords: torch.Tensor, spatial_range: Tuple[int]) -> torch.Tensor:
        feats = feats.contiguous()
        coords = coords.contiguous().int()
        spatial_range = tuple(int(v) for v in spatial_range)
        out = torch.zeros(spatial_range + (feats.size(1),), dtype=feats.dtype, device=feats.device)
        from torchsparse_amd import backend  # needs the built library: imported on use
        backend.to_dense_forward_cuda(feats, coords, spatial_range, out)
        ctx.for_backwards = (coords, spatial_range)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        coords, spatial_range = ctx.for_backwards
        grad_output = grad_output.contiguous()
        grad = torch.empty(coords.size(0), grad_output.size(-1), dtype=grad_output.dtype,
                           device=grad_output.device)
        from torchsparse_amd import backend
        backend.to_dense_backward_cuda(grad_output, coords, spatial_range, grad)
        return grad, None, None


def to_dense(feats: torch.Tensor, coords: torch.Tensor, spatial_range: Tuple[int]) -> torch.Tensor:
    return ToDenseFunction.apply(feats, coords, spatial_range)
