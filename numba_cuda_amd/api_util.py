"""Argument normalisation shared by the array constructors (reference:
numba_cuda/numba/cuda/api_util.py:11-51)."""

import numpy as np

from numba_cuda_amd.cudadrv import dummyarray


def prepare_shape_strides_dtype(shape, strides, dtype, order):
    """-> (shape tuple, strides tuple, np.dtype); missing strides are filled in
    for the given order ("C" or "F")."""
    dtype = np.dtype(dtype)
    if isinstance(shape, (float, np.floating)) or (
            isinstance(shape, np.ndarray) and np.issubdtype(shape.dtype, np.floating)):
        raise TypeError("shape must be an integer or tuple of integers")
    shape = (shape,) if isinstance(shape, (int, np.integer)) else tuple(shape)
    if isinstance(strides, (int, np.integer)):
        strides = (strides,)
    elif not strides:
        strides = _fill_stride_by_order(shape, dtype, order)
    else:
        strides = tuple(strides)
    return shape, strides, dtype


def _fill_stride_by_order(shape, dtype, order):
    if order == "C":
        return dummyarray.c_strides(shape, dtype.itemsize)
    if order == "F":
        return dummyarray.f_strides(shape, dtype.itemsize)
    raise ValueError("must be either C/F order")
