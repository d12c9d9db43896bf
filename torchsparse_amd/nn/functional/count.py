"""spcount: occurrences of every voxel index (the reference's nn/functional/count.py:8-16)."""
import torch

from torchsparse_amd import backend

__all__ = ["spcount"]


def spcount(coords: torch.Tensor, num: int) -> torch.Tensor:
    """int32 [num] with out[v] = number of entries of ``coords`` (voxel indices) equal to v;
    negative entries are skipped."""
    idx = coords.contiguous()
    if idx.dtype != torch.int32:
        idx = idx.int()
    return backend.count_cuda(idx, int(num))
