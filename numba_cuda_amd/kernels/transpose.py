"""2-d transpose on the device (drop-in for
numba_cuda/numba/cuda/kernels/transpose.py:10-65)."""

import numpy as np

from numba_cuda_amd.cudadrv import devicearray
from numba_cuda_amd.cudadrv import driver as _driver


def transpose(a, b=None):
    """Store the transpose of `a` into `b` and return `b`; `b` is allocated
    (C-contiguous, on `a`'s stream) when not given.

    `a` may be a host ndarray or a device array of any dtype and strides.  Unlike
    the reference, a `b` of the wrong shape or dtype is an error instead of being
    silently clipped.
    """
    stream = getattr(a, "stream", 0)
    if a.ndim != 2:
        raise ValueError("transpose needs a 2-d array, got %d-d" % a.ndim)
    rows, cols = a.shape
    itemsize = a.dtype.itemsize

    host_b = None
    if b is None:
        b = devicearray.DeviceNDArray((cols, rows), (itemsize * rows, itemsize), dtype=a.dtype,
                                      stream=stream)
    else:
        if tuple(b.shape) != (cols, rows):
            raise ValueError("incompatible shape: transpose of %s does not fit %s" % (a.shape, b.shape))
        if b.dtype != a.dtype:
            raise TypeError("incompatible dtype: %s vs. %s" % (a.dtype, b.dtype))
        if not _driver.is_device_memory(b):
            host_b = b
            b = devicearray.from_array_like(np.asarray(b), stream=stream)
    if not _driver.is_device_memory(a):
        a, _ = devicearray.auto_device(a, stream=stream)

    if a.size:
        _driver.driver.nbh_transpose(a.device_ctypes_pointer.value, b.device_ctypes_pointer.value,
                                     rows, cols, a.strides[0], a.strides[1], b.strides[0], b.strides[1],
                                     itemsize, _driver._stream_handle(stream) or None)
    if host_b is not None:
        b.copy_to_host(host_b, stream=stream)
        return host_b
    return b
