"""Indexing, slicing and item assignment of device arrays as the reference's suite
pins them (numba_cuda/numba/cuda/tests/cudadrv/test_cuda_array_slicing.py), restated
with the lines each case follows.  Run on the fake library and on the GPU."""
from itertools import product
from unittest.mock import patch

import numpy as np
import pytest


def scalar_indexing(cuda):
    # :14-61
    for shape in ((10,), (3, 4), (3, 4, 5)):
        h = np.arange(int(np.prod(shape))).reshape(shape)
        d = cuda.to_device(h)
        for idx in product(*[range(-n, n) for n in shape]):
            assert h[idx] == d[idx]
        for axis, n in enumerate(shape):
            for bad in (-n - 1, n):
                idx = [0] * len(shape)
                idx[axis] = bad
                with pytest.raises(IndexError):
                    d[tuple(idx)]


def strided_slices(cuda):
    # :64-91
    for shape in ((10,), (6, 7), (6, 7, 8)):
        h = np.arange(int(np.prod(shape))).reshape(shape)
        d = cuda.to_device(h)
        for start in product(*[range(n) for n in shape]):
            key = tuple(slice(s, None, 2) for s in start)
            np.testing.assert_equal(h[key], d[key].copy_to_host())


def prefixes_and_selections(cuda):
    # :94-133
    h = np.arange(5)
    d = cuda.to_device(h)
    for i in range(5):
        assert np.all(h[i:] == d[i:].copy_to_host())
    h = np.arange(9).reshape(3, 3)
    d = cuda.to_device(h)
    for i, j in product(range(3), repeat=2):
        got = d[i:, j:]
        assert got.shape == h[i:, j:].shape and got.strides == h[i:, j:].strides
        assert np.all(h[i:, j:] == got.copy_to_host())
    h = np.arange(60).reshape(3, 4, 5)
    d = cuda.to_device(h)
    for key in [(i,) for i in range(3)] + list(product(range(3), range(4))):
        got = d[key]
        assert got.shape == h[key].shape and got.strides == h[key].strides
        assert np.all(h[key] == got.copy_to_host())
    # :135-176
    for order in "FC":
        h = np.arange(210).reshape(5, 6, 7, order=order)
        d = cuda.to_device(h)
        for i, j in product(range(5), range(6)):
            assert np.array_equal(d[i, j, :].copy_to_host(), h[i, j, :])
        for i, j in product(range(5), range(7)):
            assert np.array_equal(d[i, :, j].copy_to_host(), h[i, :, j])
        for i, j in product(range(6), range(7)):
            assert np.array_equal(d[:, i, j].copy_to_host(), h[:, i, j])
    h = np.arange(35).reshape(5, 7, order="F")
    assert np.all(cuda.to_device(h)[:1, 1].copy_to_host() == h[:1, 1])


def negative_and_empty_slices(cuda):
    # :178-191
    h = np.arange(10)
    d = cuda.to_device(h)
    for i, j in product(range(-10, 10), repeat=2):
        np.testing.assert_array_equal(h[i:j], d[i:j].copy_to_host())
    h = np.arange(12).reshape(3, 4)
    d = cuda.to_device(h)
    for x, y, w, s in product(range(-4, 4), repeat=4):
        np.testing.assert_array_equal(h[x:y, w:s], d[x:y, w:s].copy_to_host())
    # :193-217
    for h in (np.arange(5), np.arange(35).reshape(5, 7)):
        d = cuda.to_device(h)
        for i in range(h.shape[0]):
            np.testing.assert_array_equal(d[i:i].copy_to_host(), h[i:i])
        if h.ndim == 2:
            np.testing.assert_array_equal(d[3, :0].copy_to_host(), h[3, :0])
        assert not d[:0][:0].copy_to_host().size > 0
        np.testing.assert_array_equal(d[:0][:1].copy_to_host(), h[:0][:1])
        np.testing.assert_array_equal(d[:0][-1:].copy_to_host(), h[:0][-1:])


def item_assignment(cuda):
    # :226-298
    cases = [((5, 7), (2, 2), 500), ((5, 7), 2, 500), ((5, 7), (slice(None), 2), 500),
             ((5, 7), 2, np.full(7, 400)), ((5, 7), (slice(None), 2), np.full(5, 400)),
             ((5, 6, 7), 2, np.full((6, 7), 400)),
             ((5, 6, 7, 8), (slice(None), slice(None), 2), np.full((5, 6, 8), 400)),
             ((5, 7), slice(None), np.full((5, 7), 400))]
    for shape, key, value in cases:
        h = np.arange(int(np.prod(shape))).reshape(shape)
        d = cuda.to_device(h)
        h[key] = value
        d[key] = value
        np.testing.assert_array_equal(d.copy_to_host(), h)
    h = np.ones(20)
    d = cuda.to_device(h)
    h[::2] = 500
    d[::2] = 500
    np.testing.assert_array_equal(d.copy_to_host(), h)
    # :300-326
    with pytest.raises(ValueError) as e:
        cuda.to_device(np.arange(35))[:] = np.ones(shape=(1, 2, 3))
    assert str(e.value) == "Can't assign 3-D array to 1-D self"
    with pytest.raises(ValueError) as e:
        cuda.to_device(np.arange(5))[:] = [1, 3]
    assert str(e.value) == "Can't copy sequence with size 2 to array axis 0 with dimension 5"


def assignment_synchronises_only_without_a_stream(cuda):
    # :328-379
    Stream = cuda.cudadrv.driver.Stream
    d = cuda.to_device(np.arange(5))
    with patch.object(Stream, "synchronize", return_value=None) as sync:
        d[0] = 10
    sync.assert_called_once()
    streams = (cuda.stream(), cuda.default_stream(), cuda.legacy_default_stream(), cuda.per_thread_default_stream())
    for st in streams:
        d = cuda.to_device(np.arange(5), stream=st)
        with patch.object(Stream, "synchronize", return_value=None) as sync:
            d[0] = 10
        sync.assert_not_called()
    for st in streams:
        d = cuda.to_device(np.arange(5))
        with patch.object(Stream, "synchronize", return_value=None) as sync:
            d.setitem(0, 10, stream=st)
        sync.assert_not_called()


ALL = [scalar_indexing, strided_slices, prefixes_and_selections, negative_and_empty_slices, item_assignment,
       assignment_synchronises_only_without_a_stream]
