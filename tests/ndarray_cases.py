"""Behaviour of DeviceNDArray that the reference's own suite pins
(numba_cuda/numba/cuda/tests/cudadrv/test_cuda_ndarray.py), restated case by case
with the line each one follows.  Run against the host-RAM fake library on the CPU and
against the real library on the GPU.  Cases that need the kernel language or numba's
type system (:395-456, :533-560, :622-660) have no counterpart here."""
import itertools

import numpy as np
import pytest

from numba_cuda_amd.cudadrv import devicearray


def interface_and_shapes(cuda):
    # :16-27, :39-51
    for ary in (cuda.device_array(shape=100), cuda.to_device(np.empty(100)), cuda.to_device(np.asarray(1.234))):
        devicearray.verify_cuda_ndarray_interface(ary)
    assert cuda.to_device(np.asarray(1.234)).ndim == 0
    assert cuda.device_array(shape=(100,), dtype="f4").dtype == np.dtype("f4")
    cuda.to_device(np.arange(100, dtype=np.float32), copy=False)
    h = np.arange(24).reshape(2, 3, 4)
    d = cuda.to_device(h)
    assert d.shape == h.shape and d.shape[1:] == h.shape[1:]
    # :102-115
    for shape in ((3,), (3, 5), (3, 5, 7)):
        assert len(cuda.device_array(shape)) == len(np.empty(shape))


def readonly_source(cuda):
    # :29-37
    h = np.arange(100, dtype=np.float32)
    h.flags.writeable = False
    np.testing.assert_array_equal(cuda.to_device(h).copy_to_host(), h)


def shapes_must_be_integers(cuda):
    # :53-84
    for bad in (1.23, np.float64(1.23), np.array(1.23), np.array([1.1]), [1.1], (1.1,), np.array([1.1, 2.2]),
                [1.1, 2.2], (1.1, 2.2)):
        with pytest.raises(TypeError):
            cuda.device_array(shape=bad)
    assert cuda.device_array(shape=np.array([10, 10]), dtype=np.bool_).shape == (10, 10)
    assert cuda.device_array(shape=[10, 10], dtype=np.bool_).shape == (10, 10)


def copy_back_split_replace(cuda):
    # :86-141
    h = np.arange(100, dtype=np.int32)
    keep = h.copy()
    d = cuda.to_device(h)
    h[:] = 0
    d.copy_to_host(h)
    np.testing.assert_array_equal(h, keep)
    left, right = d.split(50)
    h[:] = 0
    right.copy_to_host(h[50:])
    left.copy_to_host(h[:50])
    np.testing.assert_array_equal(h, keep)
    cuda.to_device(keep * 2, to=d)
    d.copy_to_host(h)
    np.testing.assert_array_equal(h, keep * 2)
    st = cuda.stream()
    with st.auto_synchronize():
        arr = cuda.device_array((3, 3), dtype=np.float64, stream=st)
        assert arr.bind(st).stream == st and arr.stream == st


def transposition_through_numpy(cuda):
    # :143-189, :236-244
    with pytest.raises(NotImplementedError) as e:
        np.transpose(cuda.to_device(np.arange(12).reshape(3, 4, 1)))
    assert str(e.value) == "transposing a non-2D DeviceNDArray isn't supported"
    h3 = np.arange(24).reshape(3, 4, 2)
    assert np.all(np.transpose(cuda.to_device(h3), axes=(0, 1, 2)).copy_to_host() == h3)
    d = cuda.to_device(np.arange(12).reshape(3, 4))
    with pytest.raises(ValueError) as e:
        np.transpose(d, axes=(0, 0))
    assert str(e.value) == "invalid axes list (0, 0)"
    with pytest.raises(ValueError) as e:
        np.transpose(d, axes=(0, 2))
    assert str(e.value) == "invalid axes list (0, 2)"


def reinterpreting_views(cuda):
    # :191-234
    h = np.arange(12, dtype="i2").reshape(3, 4)
    d = cuda.to_device(h)
    for dtype in ("i4", "u4", "i8", "f8"):
        np.testing.assert_array_equal(d.view(dtype).copy_to_host(), h.view(dtype))
    h = np.arange(32, dtype="i2").reshape(4, 8)
    d = cuda.to_device(h)[:, ::2]
    np.testing.assert_array_equal(d.view("u2").copy_to_host(), h[:, ::2].view("u2"))
    with pytest.raises(ValueError) as e:
        d.view("i4")
    assert "To change to a dtype of a different size," in str(e.value)
    assert "the array must be C-contiguous" in str(e.value) or "the last axis must be contiguous" in str(e.value)
    with pytest.raises(ValueError) as e:
        cuda.to_device(np.arange(12, dtype="i2").reshape(4, 3)).view("i4")
    assert str(e.value) == ("When changing to a larger dtype, its size must be a divisor of the total size in bytes"
                            " of the last axis of the array.")


def copies_need_contiguous_targets(cuda):
    # :246-262, :348-362
    a = np.arange(25).reshape(5, 5, order="F")
    d = cuda.to_device(a)
    with pytest.raises(ValueError) as e:
        d[2].copy_to_device(np.full(fill_value=5, shape=(5,)))
    assert str(e.value) == devicearray.errmsg_contiguous_buffer
    d = cuda.to_device(np.arange(10))
    strided = np.arange(20)[::2]
    d.copy_to_device(strided)                       # a strided HOST source is fine
    np.testing.assert_array_equal(d.copy_to_host(), strided)
    d = cuda.to_device(np.arange(20))
    with pytest.raises(ValueError) as e:
        d.copy_to_device(cuda.to_device(np.arange(20))[::2])
    assert str(e.value) == devicearray.errmsg_contiguous_buffer


def copies_between_orders(cuda):
    # :264-325
    for a_c in (np.arange(125).reshape(5, 5, 5), np.arange(5)):
        a_f = np.array(a_c, order="F")
        for original, other in itertools.product((a_f, a_c), repeat=2):
            d = cuda.to_device(original)
            d.copy_to_device(other)
            assert np.all(d.copy_to_host() == a_c) and np.all(d.copy_to_host() == a_f)
    a_c = np.arange(125).reshape(5, 5, 5)
    a_f = np.array(a_c, order="F")
    for mine, theirs in ((a_c, a_f), (a_f, a_c)):
        d = cuda.to_device(mine)
        with pytest.raises(ValueError) as e:
            d.copy_to_device(cuda.to_device(theirs))
        assert str(e.value) == "incompatible strides: {} vs. {}".format(mine.strides, theirs.strides)
        d.copy_to_device(cuda.to_device(mine))
        assert np.all(d.copy_to_host() == mine)


def broadcast_sources(cuda):
    # :327-346
    core_c = np.arange(6).reshape((2, 3), order="C")
    core_f = np.arange(6).reshape((2, 3), order="F")
    for dim in range(2):
        index = (slice(None),) * dim + (np.newaxis,)
        shape = (2, 3)[:dim] + (4,) + (2, 3)[dim:]
        broad_c = np.broadcast_to(core_c[index], shape)
        broad_f = np.broadcast_to(core_f[index], shape)
        d_c, d_f = cuda.to_device(broad_c), cuda.to_device(broad_f)
        np.testing.assert_array_equal(d_c.copy_to_host(), broad_c)
        np.testing.assert_array_equal(d_f.copy_to_host(), broad_f)
        d_c.copy_to_device(broad_f)
        d_f.copy_to_device(broad_c)
        np.testing.assert_array_equal(d_c.copy_to_host(), broad_f)
        np.testing.assert_array_equal(d_f.copy_to_host(), broad_c)


def contiguity_flags(cuda):
    # :364-393
    relaxed = devicearray.DeviceNDArray((1, 10), (800, 8), np.float64)
    assert relaxed.flags["C_CONTIGUOUS"] and relaxed.flags["F_CONTIGUOUS"]
    for shape, order in itertools.product(((1, 4), (4, 1)), ("C", "F")):
        h = np.ndarray(shape, order=order)
        d = cuda.to_device(h)
        assert d.flags["C_CONTIGUOUS"] == h.flags["C_CONTIGUOUS"]
        assert d.flags["F_CONTIGUOUS"] == h.flags["F_CONTIGUOUS"]
    # :563-620
    views = [cuda.device_array(10, order="C"), cuda.device_array((10, 12), order="C"),
             cuda.device_array((10, 12, 14), order="C"),
             cuda.device_array(10, order="F"), cuda.device_array((10, 12), order="F"),
             cuda.device_array((10, 12, 14), order="F"),
             np.zeros(10)[::2], np.zeros(10, order="F")[::2], np.zeros((10, 12))[::2, ::2],
             np.zeros((10, 12), order="F")[::2, ::2]]
    from numba_cuda_amd.cudadrv import driver
    if type(driver.driver.lib).__name__ != "FakeLib":     # .T runs the transpose kernel
        views += [cuda.device_array((10, 12), order="C").T, cuda.device_array((10, 12), order="F").T]
    for v in views:
        assert devicearray.is_contiguous(v) == devicearray.array_core(v).flags["C_CONTIGUOUS"]


def empty_arrays_with_odd_strides(cuda):
    # :465-493
    d = devicearray.DeviceNDArray(shape=(0,), strides=(8,), dtype=np.int8)
    h = np.ndarray(shape=(0,), strides=(0,), dtype=np.int8)
    assert h.strides == (0,)
    d.copy_to_host(h)
    d.copy_to_device(h)
    from_host = cuda.to_device(h)
    assert from_host.shape == (0,) and from_host.strides == (0,)
    d.copy_to_device(from_host)
    from_host.copy_to_device(d)


def array_protocol(cuda):
    # :458-463, :504-531
    d16 = cuda.to_device(np.arange(10, dtype=np.int16))
    assert np.asarray(d16).dtype == d16.dtype
    d = cuda.to_device(np.asarray([1.0, 2.0, 3.0]))
    np.testing.assert_equal(d.copy_to_host(), np.array(d))
    np.testing.assert_equal(np.array(d, dtype=np.int32), d.copy_to_host().astype(np.int32))
    with pytest.raises(ValueError, match="`copy=False` is not"):
        np.array(d, copy=False)


ALL = [interface_and_shapes, readonly_source, shapes_must_be_integers, copy_back_split_replace,
       transposition_through_numpy, reinterpreting_views, copies_need_contiguous_targets, copies_between_orders,
       broadcast_sources, contiguity_flags, empty_arrays_with_odd_strides, array_protocol]
