import torch

from torchsparse_amd import backend

__all__ = ["convert_transposed_out_in_map"]


def convert_transposed_out_in_map(out_in_map: torch.Tensor, size: int) -> torch.Tensor:
    """int32 [size, K_vol] with out_in_map_t[in, k] = out, -1 elsewhere
    (the reference's nn/functional/conv/hash/query.py:47-55)."""
    return backend.convert_transposed_out_in_map(out_in_map, size)
