from typing import Optional, Tuple, Union

import torch

from torchsparse_amd import backend
from torchsparse_amd.utils import make_ntuple

__all__ = ["spdownsample"]


def spdownsample(_coords: torch.Tensor, stride: Union[int, Tuple[int, ...]] = 2,
                 kernel_size: Union[int, Tuple[int, ...]] = 2, padding=0,
                 spatial_range: Optional[Tuple[int]] = None, downsample_mode: str = "spconv",
                 return_table: bool = False):
    """Output coordinates of a strided convolution, ascending in (b, x, y, z)
    (the reference's nn/functional/conv/kmap/downsample.py:11-79).

    When every axis has stride 1 or stride == kernel size, or in "minkowski" mode,
    the outputs are unique(floor(coords / stride)); otherwise every
    (coords + padding - c) / stride, 0 <= c < kernel size, that divides exactly and
    lies inside the output range (spatial_range, already strided, or the range
    derived from the largest input coordinate)."""
    assert downsample_mode in ("spconv", "minkowski")
    stride, kernel_size, padding = (make_ntuple(v, ndim=3) for v in (stride, kernel_size, padding))
    coords = _coords.contiguous()
    if all(s in (1, k) for s, k in zip(stride, kernel_size)) or downsample_mode == "minkowski":
        out, table = backend.downsample_coords(coords, kernel_size, stride, padding, None, mode=1)
    else:
        host_max = None if spatial_range is None else tuple(x - 1 for x in spatial_range[1:])
        from torchsparse_amd.tensor import get_allow_negative_coordinates
        out, table = backend.downsample_coords(coords, kernel_size, stride, padding, host_max, mode=0,
                                               allow_negative=get_allow_negative_coordinates())
    return (out, table) if return_table else out
