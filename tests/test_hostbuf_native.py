"""The native host-buffer extension (numba_cuda_amd/cext/hostbuf.c) against NumPy,
brute force and the oracle's extents (reference semantics: cext/mviewbuf.c:48-209)."""
import ctypes
import gc
import itertools
import weakref

import numpy as np
import pytest

from numba_cuda_amd import _hostbuf
from oracle import cref


def _touched(a):
    """Every byte address the items of `a` occupy, by enumeration."""
    base = a.__array_interface__["data"][0]
    out = set()
    for idx in np.ndindex(*a.shape):
        off = sum(i * s for i, s in zip(idx, a.strides))
        out.update(range(base + off, base + off + a.itemsize))
    return out


def test_extents_match_brute_force_for_every_sign_of_stride():
    big = np.arange(6 * 7 * 5, dtype=np.int32).reshape(6, 7, 5)
    for sl in itertools.product((slice(None), slice(None, None, -1), slice(1, None, 2), slice(4, 0, -3), slice(2, 2)),
                                repeat=3):
        v = big[sl]
        lo, hi = _hostbuf.extents(v)
        if v.size == 0:
            assert lo == hi
            continue
        touched = _touched(v)
        assert (lo, hi) == (min(touched), max(touched) + 1)
        rel = _hostbuf.extents_of(v.shape, v.strides, v.itemsize)
        assert rel == cref.extents(v.shape, v.strides, v.itemsize)
        base = v.__array_interface__["data"][0]
        assert (base + rel[0], base + rel[1]) == (lo, hi)


def test_extents_of_scalars_ctypes_and_zero_dimensions():
    s = np.asarray(np.uint32(7))
    assert _hostbuf.extents(s) == (s.ctypes.data, s.ctypes.data + 4)
    d = ctypes.c_double(1.5)
    assert _hostbuf.extents(d) == (ctypes.addressof(d), ctypes.addressof(d) + 8)
    assert _hostbuf.extents_of((), (), 16) == (0, 16)
    assert _hostbuf.extents_of((3, 0), (8, 8), 8) == (0, 0)
    with pytest.raises(ValueError):
        _hostbuf.extents_of((3,), (8,), 0)
    with pytest.raises(ValueError):
        _hostbuf.extents_of((3, 2), (8,), 8)


def test_address_honours_writability():
    a = np.arange(5)
    assert _hostbuf.address(a) == a.ctypes.data
    a.flags.writeable = False
    with pytest.raises((BufferError, ValueError)):
        _hostbuf.address(a)
    assert _hostbuf.address(a, False) == a.ctypes.data
    assert _hostbuf.address(b"abc", False) != 0
    with pytest.raises((BufferError, TypeError)):
        _hostbuf.address(b"abc")


def test_hostbuffer_subclass_exports_its_memory_and_is_kept_alive():
    backing = np.arange(16, dtype=np.uint8)

    class Mem(_hostbuf.HostBuffer):
        def __init__(self):
            self._bufptr_ = backing.ctypes.data
            self._buflen_ = backing.nbytes

    m = Mem()
    ref = weakref.ref(m)
    view = np.ndarray(4, dtype=np.uint32, buffer=m)
    assert view.tobytes() == backing.tobytes()
    view[0] = 0x01020304
    assert backing[:4].tolist() == [4, 3, 2, 1]
    mv = memoryview(m)
    assert mv.nbytes == 16 and not mv.readonly and mv.ndim == 1
    del m, mv
    gc.collect()
    assert ref() is not None          # the ndarray's buffer holds it
    del view
    gc.collect()
    assert ref() is None


def test_hostbuffer_with_nonsense_description_refuses():
    class Bad(_hostbuf.HostBuffer):
        _bufptr_ = 0
        _buflen_ = 8

    with pytest.raises(BufferError):
        memoryview(Bad())

    class Missing(_hostbuf.HostBuffer):
        pass

    with pytest.raises(AttributeError):
        memoryview(Missing())
