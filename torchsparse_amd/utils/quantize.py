"""Voxelisation of a point cloud on the host (the reference's utils/quantize.py:10-54).

``sparse_quantize`` floors ``coords / voxel_size`` to int32 and keeps one point per voxel: the
first in input order.  Voxels come out in ascending (x, y, z) order, which is the order the
reference's ravelled hash plus ``np.unique`` gives."""
from typing import List, Tuple, Union

import numpy as np

__all__ = ["sparse_quantize", "ravel_hash"]


def ravel_hash(x: np.ndarray) -> np.ndarray:
    """uint64 key of every row: the row's offset from the column minima, ravelled over the
    extents (first column most significant) — utils/quantize.py:10-22."""
    if x.ndim != 2:
        raise AssertionError(x.shape)
    if x.shape[0] == 0:
        return np.zeros(0, dtype=np.uint64)
    rel = (x - x.min(axis=0)).astype(np.uint64)
    extent = rel.max(axis=0) + np.uint64(1)
    key = rel[:, 0].copy()
    for col in range(1, x.shape[1]):
        key = key * extent[col] + rel[:, col]
    return key


def sparse_quantize(coords, voxel_size: Union[float, Tuple[float, ...]] = 1, *,
                    return_index: bool = False, return_inverse: bool = False) -> List[np.ndarray]:
    if isinstance(voxel_size, (float, int)):
        voxel_size = (voxel_size,) * 3
    if not (isinstance(voxel_size, tuple) and len(voxel_size) == 3):
        raise AssertionError(voxel_size)
    voxels = np.floor(np.asarray(coords) / np.asarray(voxel_size)).astype(np.int32)
    _, index, inverse = np.unique(ravel_hash(voxels), return_index=True, return_inverse=True)
    out = [voxels[index]]
    if return_index:
        out.append(index)
    if return_inverse:
        out.append(inverse)
    return out[0] if len(out) == 1 else out
