"""sphashquery: position of each query hash among the reference hashes
(the reference's nn/functional/query.py:8-37)."""
import torch

from torchsparse_amd import backend

__all__ = ["sphashquery"]


def sphashquery(queries: torch.Tensor, references: torch.Tensor) -> torch.Tensor:
    """For every int64 query the index i with references[i] == query, or -1; int32, shaped
    like ``queries`` (the reference's GPU path returns int32 as well,
    hashmap/hashmap_cuda.cuh:298-300)."""
    references = references.contiguous()
    sizes = queries.size()
    flat = queries.contiguous().view(-1)
    table = backend.GPUHashTable(backend.hash_capacity(references.shape[0]), device=references.device)
    table.insert_vals(references)
    out = table.lookup_vals(flat).sub_(1)
    return out.view(*sizes)
