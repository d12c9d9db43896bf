"""sphash: 64-bit hashes of integer coordinates (the reference's nn/functional/hash.py:10-39)."""
from typing import Optional

import torch

from torchsparse_amd import backend

__all__ = ["sphash"]


def sphash(coords: torch.Tensor, offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """int64 [N] hashes of int32 [N,4] rows (batch, x, y, z); with ``offsets`` int32 [K,3] the
    [K,N] hashes of the rows shifted by every offset (the batch field is not shifted)."""
    assert coords.dtype == torch.int, coords.dtype
    assert coords.ndim == 2 and coords.shape[1] == 4, coords.shape
    coords = coords.contiguous()
    if offsets is None:
        return backend.hash_cuda(coords)
    assert offsets.dtype == torch.int, offsets.dtype
    assert offsets.ndim == 2 and offsets.shape[1] == 3, offsets.shape
    return backend.kernel_hash_cuda(coords, offsets.contiguous())
