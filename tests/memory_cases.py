"""Raw memory objects and copy functions as the reference's suite pins them
(numba_cuda/numba/cuda/tests/cudadrv/test_cuda_memory.py), restated with the lines
each case follows.  Run on the fake library and on the GPU."""
import ctypes
import gc

import numpy as np

from numba_cuda_amd.cudadrv import devices, driver


def _is_fake():
    return type(driver.driver.lib).__name__ == "FakeLib"


def memory_objects_are_device_memory(cuda):
    # :27-58
    ctx = devices.get_context()
    objs = [ctx.memalloc(1024), ctx.memalloc(1024).view(10), ctx.memhostalloc(1024, mapped=True),
            ctx.memallocmanaged(1024)]
    if _is_fake():      # page-locking existing memory is refused on the GPU machines used here
        ary = np.arange(10)
        objs.append(ctx.mempin(ary, ary.ctypes.data, ary.size * ary.dtype.itemsize, mapped=True))
    for obj in objs:
        assert driver.is_device_memory(obj)
        driver.require_device_memory(obj)
        assert isinstance(obj.device_ctypes_pointer, ctypes.c_size_t)


def derived_pointers_count_references(cuda):
    # :60-88
    ctx = devices.get_context()
    m = ctx.memalloc(1024)
    for offset in (0, 1):
        v1 = m.view(offset)
        assert int(v1.owner.handle) == int(m.handle) and m.refct == 2
        assert int(v1.handle) - offset == int(v1.owner.handle)
        v2 = v1.view(offset)
        assert int(v2.owner.handle) == int(m.handle)
        assert int(v2.handle) - 2 * offset == int(v2.owner.handle) and m.refct == 3
        del v2
        gc.collect()
        assert m.refct == 2
        del v1
        gc.collect()
        assert m.refct == 1


def user_pointers_run_their_finalizer(cuda):
    # :90-116
    ctx = devices.get_context()
    fake_ptr = ctypes.c_void_p(0xDEADBEEF)
    calls = [0]

    def dtor():
        calls[0] += 1

    ptr = driver.MemoryPointer(context=ctx, pointer=fake_ptr, size=40, finalizer=dtor)
    assert calls[0] == 0
    del ptr
    gc.collect()
    assert calls[0] == 1
    ptr = driver.MemoryPointer(context=ctx, pointer=fake_ptr, size=40, finalizer=dtor)
    owned = ptr.own()
    del owned
    gc.collect()
    assert calls[0] == 1
    del ptr
    gc.collect()
    assert calls[0] == 2


def copy_functions(cuda):
    # :128-162
    ctx = devices.get_context()
    h = np.arange(100, dtype=np.uint32)
    back = np.zeros_like(h)
    d = ctx.memalloc(h.nbytes)
    driver.host_to_device(d, h, h.nbytes)
    driver.device_to_host(back, d, h.nbytes)
    assert np.all(h == back)
    d = ctx.memalloc(40)
    driver.device_memset(d, 0xAB, 40)
    got = np.empty(10, np.uint32)
    driver.device_to_host(got, d, 40)
    assert np.all(got == np.uint32(0xABABABAB))
    d1, d2 = ctx.memalloc(h.nbytes), ctx.memalloc(h.nbytes)
    driver.host_to_device(d1, h, h.nbytes)
    driver.device_to_device(d2, d1, h.nbytes)
    back[:] = 0
    driver.device_to_host(back, d2, h.nbytes)
    assert np.all(h == back)


def host_extents(cuda):
    # :166-206
    for ary in (np.arange(100), np.asfortranarray(np.arange(100).reshape(2, 50)), np.asarray(np.uint32(1234))):
        start, _ = driver.host_memory_extents(ary)
        assert start == ary.ctypes.data
        assert driver.host_memory_size(ary) == ary.dtype.itemsize * ary.size

    class Pair(ctypes.Structure):
        _fields_ = [("x", ctypes.c_int), ("y", ctypes.c_int)]

    assert driver.host_memory_size(Pair(x=123, y=432)) == ctypes.sizeof(Pair)
    assert driver.host_memory_size(ctypes.c_double(1.234)) == ctypes.sizeof(ctypes.c_double)


ALL = [memory_objects_are_device_memory, derived_pointers_count_references, user_pointers_run_their_finalizer,
       copy_functions, host_extents]
