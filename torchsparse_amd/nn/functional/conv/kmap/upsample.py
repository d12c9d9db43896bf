from typing import Optional, Tuple, Union

import torch

from torchsparse_amd import backend
from torchsparse_amd.utils import make_ntuple

__all__ = ["spupsample_generative"]


def spupsample_generative(_coords: torch.Tensor, stride: Union[int, Tuple[int, ...]] = 2,
                          kernel_size: Union[int, Tuple[int, ...]] = 2, padding=0,
                          spatial_range: Optional[Tuple[int]] = None, return_table: bool = False):
    """Output coordinates of a generative transposed convolution: every input coordinate times
    the stride, shifted by every kernel offset (-ks//2+1 .. ks//2 per axis), clamped to
    [0, spatial_range - 1], unique, ascending in (b, x, y, z)
    (the reference's nn/functional/conv/kmap/upsample.py:12-41; ``padding`` is not used there
    either).  One launch inserts the candidates into a hash table of the outputs; the unique
    coordinates are its sorted occupied slots."""
    stride, kernel_size = make_ntuple(stride, ndim=3), make_ntuple(kernel_size, ndim=3)
    assert spatial_range is not None, "spatial range must be specified in generative mode"
    host_max = tuple(int(x) - 1 for x in spatial_range[1:])
    out, table = backend.downsample_coords(_coords.contiguous(), kernel_size, stride, (0, 0, 0),
                                           host_max, mode=3)
    return (out, table) if return_table else out
