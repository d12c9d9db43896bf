"""sphashquery: position of each query hash among the reference hashes
(the reference's nn/functional/query.py:8-37)."""
import torch

from torchsparse_amd import backend

__all__ = ["sphashquery"]


def sphashquery(queries: torch.Tensor, references: torch.Tensor) -> torch.Tensor:
    """For every int64 query the index i with references[i] == query, or -1; the result has
    the shape of ``queries``."""
    references = references.contiguous()
    sizes = queries.size()
    flat = queries.contiguous().view(-1)
    table = backend.GPUHashTable(backend.hash_capacity(references.shape[0]), device=references.device)
    table.insert_vals(references)
    out = table.lookup_vals(flat).to(torch.int64) - 1
    return out.view(*sizes)
