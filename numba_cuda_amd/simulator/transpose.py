"""transpose(a, b=None) in the CPU mode (the reference runs its tile kernel through the
simulator, numba_cuda/numba/cuda/kernels/transpose.py:10-65; the result is b[j, i] = a[i, j])."""

import numpy as np

from numba_cuda_amd.simulator.hostarray import device_array


def transpose(a, b=None):
    if a.ndim != 2:
        raise ValueError("transpose needs a 2D array, got %dD" % a.ndim)
    if b is None:
        rows, cols = a.shape
        b = device_array((cols, rows), dtype=a.dtype, stream=getattr(a, "stream", 0))
    np.copyto(getattr(b, "_ary", b), np.transpose(getattr(a, "_ary", a)))
    return b
