"""spdevoxelize: trilinear interpolation of voxel features at points, differentiable, and the
interpolation weights (the reference's nn/functional/devoxelize.py:11-101)."""
import torch
from torch.autograd import Function

from torchsparse_amd import backend

__all__ = ["spdevoxelize", "calc_ti_weights"]


def calc_ti_weights(coords: torch.Tensor, idx_query: torch.Tensor, scale: float = 1) -> torch.Tensor:
    """[N, 8] trilinear weights of float points ``coords`` [N, 3] with respect to the 8 corners
    of their cell of edge ``scale`` (corner order: x slowest, z fastest, low before high);
    corners that do not exist (idx_query == -1) get weight 0 and the rest is renormalised."""
    with torch.no_grad():
        p = coords
        low = torch.floor(p / scale) * scale if scale != 1 else torch.floor(p)
        frac_hi = (p - low).float()            # distance to the low corner, per axis
        frac_lo = (low + scale - p).float()    # distance to the high corner
        cols = []
        for corner in range(8):
            w = torch.ones(p.shape[0], device=p.device, dtype=torch.float32)
            for axis in range(3):
                high = (corner >> (2 - axis)) & 1
                w = w * (frac_hi[:, axis] if high else frac_lo[:, axis])
            cols.append(w.view(-1, 1))
        w = torch.cat(cols, dim=1)
        if scale != 1:
            w /= scale ** 3
        w[idx_query == -1] = 0
        w /= torch.sum(w, dim=1).unsqueeze(1) + 1e-8
    return w


class DevoxelizeFunction(Function):
    @staticmethod
    def forward(ctx, feats: torch.Tensor, coords: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
        feats = feats.contiguous()
        coords = coords.contiguous().int()
        weights = weights.contiguous().float()
        out = backend.devoxelize_forward_cuda(feats, coords, weights)
        ctx.for_backwards = (coords, weights, feats.shape[0])
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        coords, weights, n = ctx.for_backwards
        return backend.devoxelize_backward_cuda(grad_output.contiguous(), coords, weights, n), None, None


def spdevoxelize(feats: torch.Tensor, coords: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """[N, C]: out[i] = sum_k weights[i,k] * feats[coords[i,k]] over the 8 corner voxel indices
    ``coords`` int [N, 8] (-1 = absent)."""
    return DevoxelizeFunction.apply(feats, coords, weights)
