"""The CUDA array interface as the reference's suite pins it
(numba_cuda/numba/cuda/tests/cudapy/test_cuda_array_interface.py), restated with the
lines each case follows; cases that launch @cuda.jit kernels or ufuncs have no
counterpart (:66-133, :380-470).  Run on the fake library and on the GPU."""
import gc
from unittest.mock import patch

import numpy as np
import pytest

from numba_cuda_amd.core import config
from numba_cuda_amd.cudadrv import driver


class ForeignArray:
    """An array "from another library": only the interface dict is visible
    (reference testing.py:374-383)."""

    def __init__(self, arr):
        self._arr = arr
        self.__cuda_array_interface__ = arr.__cuda_array_interface__


def import_and_ownership(cuda):
    # :23-64
    h = np.arange(10)
    assert not cuda.is_cuda_array(h)
    d = cuda.to_device(h)
    assert cuda.is_cuda_array(d)
    foreign = ForeignArray(d)
    assert cuda.is_cuda_array(foreign)
    wrapped = cuda.as_cuda_array(foreign)
    assert cuda.is_cuda_array(wrapped)
    np.testing.assert_array_equal(wrapped.copy_to_host(), h)
    np.testing.assert_array_equal(d.copy_to_host(), h)
    assert wrapped.device_ctypes_pointer.value == d.device_ctypes_pointer.value
    deallocs = cuda.current_context().memory_manager.deallocations
    del d, foreign, wrapped
    gc.collect()
    deallocs.clear()
    assert len(deallocs) == 0
    d = cuda.to_device(np.arange(100))
    converted = cuda.as_cuda_array(d)
    del d
    gc.collect()
    assert len(deallocs) == 0                 # the import keeps the allocation alive
    np.testing.assert_equal(converted.copy_to_host(), np.arange(100))
    del converted
    gc.collect()
    # the default manager queues the free; a pooling manager takes the block back at once
    queued = type(cuda.current_context().memory_manager) is driver.NumbaCUDAMemoryManager
    assert len(deallocs) == (1 if queued else 0)
    deallocs.clear()


def views_of_an_imported_array(cuda):
    # :135-195
    h = np.random.default_rng(5).random(10)
    c = cuda.to_device(h)
    arr = cuda.as_cuda_array(c)
    for key in (slice(None), slice(None, 5), slice(None, None, 2)):
        np.testing.assert_array_equal(arr[key].copy_to_host(), h[key])
    strided = cuda.as_cuda_array(c[::2])
    np.testing.assert_array_equal(strided.copy_to_host(), h[::2])
    assert arr[::2].shape == strided.shape and arr[::2].strides == strided.strides
    assert arr[::2].dtype.itemsize == strided.dtype.itemsize and arr[::2].alloc_size == strided.alloc_size
    assert arr[::2].nbytes == strided.size * strided.dtype.itemsize
    arr[:5] = np.pi
    np.testing.assert_array_equal(c.copy_to_host(), np.concatenate((np.full(5, np.pi), h[5:])))
    arr[:5] = arr[5:]
    np.testing.assert_array_equal(c.copy_to_host(), np.concatenate((h[5:], h[5:])))
    arr[:] = cuda.to_device(h)
    np.testing.assert_array_equal(c.copy_to_host(), h)
    arr[::2] = np.pi
    np.testing.assert_array_equal(c.copy_to_host()[::2], np.full(5, np.pi))
    np.testing.assert_array_equal(c.copy_to_host()[1::2], h[1::2])


def negative_strides_masks_and_empties(cuda):
    # :197-258
    h = np.random.default_rng(6).random(10)
    c = cuda.to_device(h)
    h_face, c_face = h.__array_interface__, c.__cuda_array_interface__
    h_rev, c_rev = h[::-1].__array_interface__, c[::-1].__cuda_array_interface__
    assert h_rev["data"][0] - h_face["data"][0] == c_rev["data"][0] - c_face["data"][0]
    assert h_rev["shape"] == c_rev["shape"] and h_rev["strides"] == c_rev["strides"]
    with pytest.raises(NotImplementedError, match="D->H copy not implemented for negative strides"):
        c[::-1].copy_to_host()
    masked = c.__cuda_array_interface__.copy()
    masked["mask"] = cuda.to_device(np.ones(10, dtype=bool))
    with pytest.raises(NotImplementedError, match="Masked arrays are not supported"):
        cuda.from_cuda_array_interface(masked)
    assert cuda.device_array(0).__cuda_array_interface__["data"][0] == 0


def strides_in_the_interface(cuda):
    # :260-283
    c = cuda.device_array((2, 3, 4))
    assert c.__cuda_array_interface__["strides"] is None
    assert c[:, 1, :].__cuda_array_interface__["strides"] is not None
    h = np.arange(10).reshape(2, 5)
    face = cuda.to_device(h).__cuda_array_interface__
    assert face["strides"] is None
    got = cuda.from_cuda_array_interface(face).copy_to_host()
    np.testing.assert_array_equal(got, h)
    assert got.flags["C_CONTIGUOUS"]
    face["strides"] = h.strides
    got = cuda.from_cuda_array_interface(face).copy_to_host()
    np.testing.assert_array_equal(got, h)
    assert got.flags["C_CONTIGUOUS"]


def streams_in_the_interface(cuda):
    # :285-336
    for make in (cuda.device_array, cuda.mapped_array, cuda.managed_array):
        assert make(10).__cuda_array_interface__["stream"] is None
        s = cuda.stream()
        assert make(10, stream=s).__cuda_array_interface__["stream"] == int(s.handle)
    assert cuda.as_cuda_array(ForeignArray(cuda.device_array(10))).stream == 0
    s = cuda.stream()
    imported = cuda.as_cuda_array(ForeignArray(cuda.device_array(10, stream=s)))
    assert imported.stream.external and int(imported.stream.handle) == int(s.handle)


def import_synchronises_the_producers_stream(cuda):
    # :338-378
    Stream = cuda.cudadrv.driver.Stream
    plain = ForeignArray(cuda.device_array(10))
    with patch.object(Stream, "synchronize", return_value=None) as sync:
        cuda.as_cuda_array(plain)
    sync.assert_not_called()
    s = cuda.stream()
    streamed = ForeignArray(cuda.device_array(10, stream=s))
    with patch.object(Stream, "synchronize", return_value=None) as sync:
        cuda.as_cuda_array(streamed)
    sync.assert_called_once_with()
    old = config.CUDA_ARRAY_INTERFACE_SYNC
    try:
        config.CUDA_ARRAY_INTERFACE_SYNC = False
        with patch.object(Stream, "synchronize", return_value=None) as sync:
            cuda.as_cuda_array(streamed)
        sync.assert_not_called()
    finally:
        config.CUDA_ARRAY_INTERFACE_SYNC = old


ALL = [import_and_ownership, views_of_an_imported_array, negative_strides_masks_and_empties,
       strides_in_the_interface, streams_in_the_interface, import_synchronises_the_producers_stream]
