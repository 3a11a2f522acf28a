"""Device-array plumbing checks shared by the CPU run (fake library, host RAM)
and the GPU run (libnbhip.so).  Each function takes the `cuda` namespace.

Expected behaviour is the reference's: numba_cuda/numba/cuda/tests/cudadrv/
test_cuda_ndarray.py, test_cuda_array_slicing.py, test_array_attr.py,
test_cuda_memory.py, test_deallocations.py (inputs and expected values, restated).
"""

import gc
import warnings

import numpy as np
import pytest

from numba_cuda_amd.cudadrv import devicearray, driver as drv


def roundtrip_and_attributes(cuda):
    a = np.arange(2 * 3 * 4, dtype=np.float32).reshape(2, 3, 4)
    d = cuda.to_device(a)
    assert isinstance(d, cuda.DeviceNDArray)
    assert (d.shape, d.strides, d.dtype, d.size, d.ndim) == (a.shape, a.strides, a.dtype, a.size, 3)
    assert d.nbytes == a.nbytes and d.alloc_size == a.nbytes and len(d) == 2
    assert d.flags == {"C_CONTIGUOUS": True, "F_CONTIGUOUS": False}
    assert d.is_c_contiguous() and not d.is_f_contiguous()
    np.testing.assert_array_equal(d.copy_to_host(), a)
    out = np.empty_like(a)
    assert d.copy_to_host(out) is out
    np.testing.assert_array_equal(out, a)
    np.testing.assert_array_equal(np.asarray(d), a)
    with pytest.raises(ValueError, match="copy=False"):
        d.__array__(copy=False)
    devicearray.verify_cuda_ndarray_interface(d)
    assert drv.is_device_memory(d) and devicearray.is_cuda_ndarray(d)
    assert d.device_ctypes_pointer.value == d.gpu_data.device_ctypes_pointer.value
    cai = d.__cuda_array_interface__
    assert cai["shape"] == a.shape and cai["strides"] is None and cai["typestr"] == a.dtype.str
    assert cai["version"] == 3 and cai["stream"] is None and cai["data"] == (d.device_ctypes_pointer.value, False)
    # Fortran order keeps its strides on the device
    f = np.asfortranarray(a)
    df = cuda.to_device(f)
    assert df.strides == f.strides and df.is_f_contiguous()
    np.testing.assert_array_equal(df.copy_to_host(), f)
    # to=, copy=False
    e = cuda.device_array_like(a)
    assert cuda.to_device(a * 2, to=e) is e
    np.testing.assert_array_equal(e.copy_to_host(), a * 2)
    # scalars and 0-d
    z = cuda.to_device(np.float64(3.5))
    assert z.shape == () and z.copy_to_host() == 3.5


def constructors(cuda):
    d = cuda.device_array(10)
    assert d.dtype == np.float64 and d.shape == (10,)
    d = cuda.device_array((3, 4), dtype=np.int16, order="F")
    assert d.strides == (2, 6)
    with pytest.raises(TypeError, match="shape must be an integer or tuple of integers"):
        cuda.device_array(3.0)
    with pytest.raises(ValueError, match="strides not match ndim"):
        cuda.DeviceNDArray((2, 3), (8,), np.float64)
    with pytest.raises(TypeError, match="shape elements must be integers"):
        cuda.DeviceNDArray((2, 3.0), (24, 8), np.float64)
    # like-constructors keep axis order but drop gaps
    a = np.zeros((4, 6, 8))[::2, :, ::2]
    like = cuda.device_array_like(a)
    assert like.shape == a.shape and like.strides == np.empty_like(a).strides
    at = np.zeros((4, 6)).T[::2]
    like = cuda.device_array_like(at)
    assert like.shape == at.shape and like.is_f_contiguous()
    # empty arrays own a NULL pointer
    e = cuda.device_array(0)
    assert e.size == 0 and e.alloc_size == 0 and (e.device_ctypes_pointer.value or 0) == 0
    assert e.copy_to_host().shape == (0,)
    e2 = cuda.to_device(np.zeros((3, 0, 2)))
    assert e2.copy_to_host().shape == (3, 0, 2)
    e.copy_to_device(np.zeros(0))            # nothing to do, no error


def slicing_views(cuda):
    a = np.arange(10 * 12, dtype=np.int64).reshape(10, 12)
    d = cuda.to_device(a)
    for idx in [slice(2, 5), (slice(None), slice(3, 9)), (slice(1, 9, 2), slice(None, None, 3)),
                (3,), (slice(None), 4), (slice(-4, None), slice(-5, -1)), (slice(5, 5),)]:
        v = d[idx]
        want = a[idx]
        assert v.shape == want.shape
        if want.size:
            assert v.strides == want.strides
            if v.is_c_contiguous() or v.is_f_contiguous():
                np.testing.assert_array_equal(v.copy_to_host(), want)
    # element access is a (blocking) one-item copy and gives a NumPy scalar
    x = d[3, 4]
    assert isinstance(x, np.int64) and x == a[3, 4]
    assert d[-1, -1] == a[-1, -1]
    with pytest.raises(IndexError):
        d[10, 0]
    with pytest.raises(IndexError):
        d[0, 0, 0]
    # views share ownership with the parent: the buffer outlives it
    col = d[2]
    del d
    gc.collect()
    np.testing.assert_array_equal(col.copy_to_host(), a[2])
    # non-contiguous views cannot be memcpy'd
    d = cuda.to_device(a)
    with pytest.raises(ValueError, match="non-contiguous buffer"):
        d[:, 2].copy_to_device(np.zeros(10, np.int64))
    # negative strides: view exists, host copy refused
    r = d[::-1]
    assert r.strides == (-96, 8)
    with pytest.raises(NotImplementedError, match="negative strides"):
        r.copy_to_host()
    # F-order rows are not contiguous (test_cuda_ndarray.py:246-260)
    f = cuda.to_device(np.arange(25).reshape(5, 5, order="F"))
    with pytest.raises(ValueError) as e:
        f[2].copy_to_device(np.full(5, 5))
    assert str(e.value) == devicearray.errmsg_contiguous_buffer


def copies_and_compatibility(cuda):
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    d = cuda.device_array_like(a)
    d.copy_to_device(a)
    d2 = cuda.device_array_like(a)
    d2.copy_to_device(d)                               # device to device
    np.testing.assert_array_equal(d2.copy_to_host(), a)
    with pytest.raises(TypeError, match="incompatible dtype: float32 vs. float64"):
        d.copy_to_device(a.astype(np.float64))
    with pytest.raises(ValueError, match="incompatible shape"):
        d.copy_to_device(np.zeros((4, 3), np.float32))
    with pytest.raises(ValueError, match="incompatible strides"):
        d.copy_to_host(np.zeros((4, 3), np.float32).T)
    # length-1 axes do not matter for compatibility
    d.copy_to_device(a.reshape(3, 1, 4).squeeze())
    e = cuda.device_array((3, 1, 4), np.float32)
    e.copy_to_device(a.reshape(3, 1, 4))
    # host arrays are re-laid-out to the device array's order when needed
    df = cuda.device_array((3, 4), np.float32, order="F")
    df.copy_to_device(np.asfortranarray(a))
    np.testing.assert_array_equal(df.copy_to_host(), a)
    # broadcast arrays: only the core travels
    b = np.broadcast_to(np.arange(4, dtype=np.float32), (3, 4))
    db = cuda.to_device(b)
    assert db.strides == b.strides and db.alloc_size == 16
    np.testing.assert_array_equal(db.copy_to_host(), b)
    # read-only host source is fine
    ro = np.arange(5.0)
    ro.setflags(write=False)
    np.testing.assert_array_equal(cuda.to_device(ro).copy_to_host(), ro)
    # structured scalars become DeviceRecords
    rec_t = np.dtype([("a", np.int32), ("b", np.float64)], align=True)
    rec = np.array([(7, 2.5)], dtype=rec_t)[0]
    dr = cuda.to_device(rec)
    assert isinstance(dr, cuda.DeviceRecord)
    assert dr["a"] == 7 and dr["b"] == 2.5
    dr["b"] = 4.25
    assert dr.copy_to_host()["b"] == 4.25
    arr = cuda.to_device(np.array([(1, 1.5), (2, 2.5)], dtype=rec_t))
    assert isinstance(arr[1], cuda.DeviceRecord) and arr[1]["a"] == 2


def reshape_view_ravel_split(cuda):
    a = np.arange(24, dtype=np.int16).reshape(4, 6)
    d = cuda.to_device(a)
    np.testing.assert_array_equal(d.reshape(6, 4).copy_to_host(), a.reshape(6, 4))
    np.testing.assert_array_equal(d.reshape((2, 12)).copy_to_host(), a.reshape(2, 12))
    np.testing.assert_array_equal(d.reshape(-1).copy_to_host(), a.reshape(-1))
    np.testing.assert_array_equal(d.reshape(4, 6).copy_to_host(), a)
    np.testing.assert_array_equal(d.ravel().copy_to_host(), a.ravel())
    with pytest.raises(NotImplementedError):
        d[:, ::2].ravel()
    with pytest.raises(NotImplementedError):
        d[:, :3].reshape(12)
    f = cuda.to_device(np.asfortranarray(a))
    np.testing.assert_array_equal(f.reshape(6, 4, order="F").copy_to_host(), a.reshape(6, 4, order="F"))
    np.testing.assert_array_equal(f.ravel(order="F").copy_to_host(), a.ravel(order="F"))
    # dtype views (test_cuda_ndarray.py:191-235)
    for dt in ("i4", "u4", "i8", "f8"):
        b = np.arange(12, dtype="i2").reshape(3, 4)
        np.testing.assert_array_equal(cuda.to_device(b).view(dt).copy_to_host(), b.view(dt))
    nc = cuda.to_device(np.arange(32, dtype="i2").reshape(4, 8))[:, ::2]
    assert nc.view("u2").shape == (4, 4)
    with pytest.raises(ValueError, match="To change to a dtype of a different size"):
        nc.view("i4")
    with pytest.raises(ValueError, match="its size must be a divisor of the total size in bytes"):
        cuda.to_device(np.arange(12, dtype="i2").reshape(4, 3)).view("i4")
    # squeeze
    s = cuda.to_device(np.zeros((1, 3, 1, 2)))
    assert s.squeeze().shape == (3, 2) and s.squeeze(axis=0).shape == (3, 1, 2)
    with pytest.raises(ValueError):
        s.squeeze(axis=1)
    # split
    v = cuda.to_device(np.arange(10))
    parts = [p.copy_to_host() for p in v.split(4)]
    assert [p.tolist() for p in parts] == [[0, 1, 2, 3], [4, 5, 6, 7], [8, 9]]
    with pytest.raises(ValueError, match="only support 1d array"):
        list(d.split(2))
    # bind
    st = cuda.stream()
    assert d.bind(st).stream is st and d.stream == 0


def streams_events_pinned(cuda):
    s = cuda.stream()
    assert int(s) != 0 and "HIP stream" in repr(s)
    a = cuda.pinned_array((64, 3), dtype=np.float32)
    assert isinstance(a, np.ndarray) and a.shape == (64, 3)
    a[:] = np.arange(192, dtype=np.float32).reshape(64, 3)
    d = cuda.to_device(a, stream=s)
    back = cuda.pinned_array_like(a)
    d.copy_to_host(back, stream=s)
    s.synchronize()
    np.testing.assert_array_equal(back, a)
    with s.auto_synchronize():
        d.copy_to_host(back, stream=s)
    e0, e1 = cuda.event(), cuda.event(timing=True)
    e0.record(s)
    d.copy_to_host(back, stream=s)
    e1.record(s)
    e1.synchronize()
    assert e1.query() is True
    e1.wait(s)
    assert cuda.event_elapsed_time(e0, e1) >= 0 and e0.elapsed_time(e1) >= 0
    assert cuda.default_stream() == 0
    assert cuda.external_stream(int(s)).external
    with pytest.raises(TypeError):
        cuda.external_stream("x")
    if type(drv.driver.lib).__name__ == "FakeLib":
        # page-locking memory that already exists (hipHostRegister) is refused on the
        # GPU machines these tests run on, so cuda.pinned() is only driven on the fake
        h = np.arange(100.0)
        with cuda.pinned(h):
            np.testing.assert_array_equal(cuda.to_device(h, stream=s).copy_to_host(stream=s), h)
    cuda.synchronize()
    free, total = cuda.current_context().get_memory_info()
    assert 0 < free <= total
    dev = cuda.get_current_device()
    assert dev.WARP_SIZE == 64 and dev.MAX_THREADS_PER_BLOCK == 1024 and dev.MULTIPROCESSOR_COUNT > 0
    with pytest.raises(AttributeError):
        dev.NO_SUCH_ATTRIBUTE
    assert cuda.select_device(0).id == 0 and len(cuda.gpus) >= 1 and cuda.gpus[0].id == 0
    with cuda.gpus[0]:
        assert cuda.get_current_device().id == 0


def deferred_deallocation(cuda):
    """Frees are queued, not executed, until thresholds are crossed
    (tests/cudadrv/test_deallocations.py:22-142)."""
    from numba_cuda_amd.core import config
    ctx = cuda.current_context()
    mm = ctx.memory_manager
    if type(mm) is not drv.NumbaCUDAMemoryManager:
        pytest.skip("the queue of waiting frees belongs to the default memory manager; "
                    "a pooling manager takes blocks back at once")
    mm.deallocations.clear()
    assert len(mm.deallocations) == 0
    for i in range(config.CUDA_DEALLOCS_COUNT):
        cuda.to_device(np.arange(1))
        gc.collect()
        assert len(mm.deallocations) == i + 1
    cuda.to_device(np.arange(1))
    gc.collect()
    assert len(mm.deallocations) == 0             # one more flushes the queue
    with cuda.defer_cleanup():
        with cuda.defer_cleanup():
            for i in range(config.CUDA_DEALLOCS_COUNT * 2):
                cuda.to_device(np.arange(1))
            gc.collect()
            assert len(mm.deallocations) == config.CUDA_DEALLOCS_COUNT * 2
        mm.deallocations.clear()
        assert len(mm.deallocations) == config.CUDA_DEALLOCS_COUNT * 2
    mm.deallocations.clear()
    assert len(mm.deallocations) == 0
    # a big free crosses the byte threshold at once
    old = mm.deallocations.memory_capacity
    try:
        mm.deallocations.memory_capacity = 1 << 20
        big = cuda.device_array(1 << 18, np.uint8)    # > 0.2 * 1 MiB
        del big
        gc.collect()
        assert len(mm.deallocations) == 0
    finally:
        mm.deallocations.memory_capacity = old


def implicit_copy_warning(cuda):
    from numba_cuda_amd.core.errors import NumbaPerformanceWarning
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        devicearray.auto_device(np.zeros(4))
        cuda.to_device(np.zeros(4))                   # explicit: no warning
    assert sum(issubclass(x.category, NumbaPerformanceWarning) for x in w) == 1


def managed_memory(cuda):
    """One buffer seen from both sides (tests/cudadrv/test_managed_alloc.py:75-124,
    tests/cudadrv/test_cuda_memory.py:49-51)."""
    ctx = cuda.current_context()
    mem = ctx.memallocmanaged(1024)
    assert drv.is_device_memory(mem) and mem.size == 1024
    for attach_global in (True, False):
        ary = cuda.managed_array(100, dtype=np.double, attach_global=attach_global)
        assert isinstance(ary, np.ndarray) and cuda.is_cuda_array(ary)
        ary.fill(123.456)
        assert all(ary == 123.456)
        # the device reads what the host wrote ...
        if type(drv.driver.lib).__name__ != "FakeLib":      # the fake library has no kernels
            assert cuda.reduce(lambda a, b: max(a, b))(ary, init=-1.0) == 123.456
        # ... and the host reads what the device wrote, after a synchronisation
        drv.device_memset(ary, 0, ary.nbytes)
        cuda.synchronize()
        assert all(ary == 0.0)
        ary[:] = np.arange(100.0)
        d = cuda.to_device(np.zeros(100))
        d.copy_to_device(ary)                         # device-to-device from managed memory
        np.testing.assert_array_equal(d.copy_to_host(), np.arange(100.0))
    m2 = cuda.managed_array((4, 6), dtype=np.int32, order="F")
    assert m2.flags["F_CONTIGUOUS"] and m2.strides == (4, 16)
    del mem, ary, m2
    gc.collect()


ALL = [managed_memory, roundtrip_and_attributes, constructors, slicing_views, copies_and_compatibility,
       reshape_view_ravel_split, streams_events_pinned, deferred_deallocation, implicit_copy_warning]
