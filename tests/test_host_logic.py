"""Host-side logic that needs no GPU: functor recognition, deferred deallocation,
reference counting of memory pointers, argument normalisation, configuration,
and that the C-ABI library loads and exports what include/nbhip.h declares."""

import ctypes
import gc
import operator
import os
import re

import numpy as np
import pytest

import numba_cuda_amd as cuda
from numba_cuda_amd import _lib
from numba_cuda_amd.api_util import prepare_shape_strides_dtype
from numba_cuda_amd.core import config
from numba_cuda_amd.cudadrv import driver as drv
from numba_cuda_amd.kernels.reduction import classify_functor

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---------------------------------------------------------------- C ABI

def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "nbhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nbh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 40
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), name
    # the Python binding covers exactly the header
    assert sorted(_lib.SIGNATURES) == names


def test_library_loads_without_a_gpu_and_reports_errors_by_name():
    lib = _lib.load()
    assert lib.nbh_version() == 1
    assert lib.nbh_error_name(2) == b"hipErrorOutOfMemory"
    assert lib.nbh_reduce_scratch_bytes() >= 256
    n = ctypes.c_int(-1)
    assert lib.nbh_device_count(ctypes.byref(n)) == 0 and n.value >= 0
    # argument checking happens before any device work
    assert lib.nbh_reduce(0, 99, None, 1, 4, None, None, None, 0, None) != 0
    assert lib.nbh_transpose(None, None, -1, 1, 4, 4, 4, 4, 4, None) != 0
    assert lib.nbh_transpose(None, None, 0, 5, 4, 4, 4, 4, 4, None) == 0      # empty: nothing to do


def test_versions_of_driver_and_runtime(fake_gpu):
    """Driver.get_version / runtime.get_version / is_supported_version (reference
    cudadrv/driver.py:410-418, cudadrv/runtime.py:15-33, device_init.py:128-143)."""
    import numba_cuda_amd as cuda
    from numba_cuda_amd.cudadrv import driver, runtime
    assert driver.get_version() == (7, 2)
    assert runtime.get_version() == (7, 2) == cuda.runtime.get_version()
    assert cuda.is_supported_version() is True
    fake_gpu.nbh_hip_versions = lambda d, r: (fake_gpu._out(d, 50700000), fake_gpu._out(r, 50700000), 0)[2]
    driver.driver.__dict__.pop("nbh_hip_versions", None)      # the cached wrapper of the entry point
    assert runtime.get_version() == (5, 7)
    assert cuda.is_supported_version() is False


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libnbhip.so"))
    with pytest.raises(OSError, match="has not been built"):
        _lib.load()
    d = drv.driver
    saved = dict(d.__dict__)
    try:
        d.lib, d.is_initialized, d.initialization_error = None, False, None
        with pytest.raises(cuda.CudaSupportError, match="has not been built"):
            d.ensure_initialized()
        assert cuda.is_available() is False
    finally:
        d.__dict__.clear()
        d.__dict__.update(saved)


def test_simulator_request_is_refused(monkeypatch):
    monkeypatch.setenv("NUMBA_ENABLE_CUDASIM", "1")
    config.reload_config()
    d = drv.driver
    saved = dict(d.__dict__)
    try:
        d.lib, d.is_initialized, d.initialization_error = None, False, None
        with pytest.raises(cuda.CudaSupportError, match="simulator"):
            d.ensure_initialized()
    finally:
        d.__dict__.clear()
        d.__dict__.update(saved)
        monkeypatch.delenv("NUMBA_ENABLE_CUDASIM")
        config.reload_config()


# ---------------------------------------------------------------- functor recognition

@pytest.mark.parametrize("functor,want", [
    (lambda a, b: a + b, "add"), (lambda a, b: b + a, "add"), (operator.add, "add"), (np.add, "add"),
    (lambda a, b: a * b, "mul"), (operator.mul, "mul"),
    (lambda a, b: max(a, b), "max"), (max, "max"), (lambda a, b: a if a > b else b, "max"),
    (lambda a, b: b if b >= a else a, "max"), (lambda a, b: b if a < b else a, "max"),
    (lambda a, b: min(a, b), "min"), (min, "min"), (lambda a, b: a if a < b else b, "min"),
    (lambda a, b: b if a > b else a, "min"),
    (lambda a, b: a & b, "and"), (lambda a, b: b & a, "and"), (operator.and_, "and"), (np.bitwise_and, "and"),
    (lambda a, b: a | b, "or"), (operator.or_, "or"), (lambda a, b: a ^ b, "xor"), (np.bitwise_xor, "xor"),
])
def test_classify_functor(functor, want):
    assert classify_functor(functor) == want


@pytest.mark.parametrize("functor", [
    lambda a, b: a - b, lambda a, b: a + b + a, lambda a, b: a, lambda a, b: a + 1,
    lambda a, b: a / b, lambda a, b: 8, lambda a, b: a * a, lambda a, b: a if a else b,
    lambda a, b: a & 1, lambda a, b: (a ^ b) ^ a, lambda a, b: a << b,
])
def test_unrecognised_functors_raise(functor):
    with pytest.raises(NotImplementedError, match="a \\+ b, a \\* b, max"):
        classify_functor(functor)


def test_reduce_object_caches_its_operator():
    f = lambda a, b: a + b      # noqa: E731
    r1, r2 = cuda.Reduce(f), cuda.reduce(f)
    assert r1._op == r2._op == "add"
    assert cuda.Reduce._cache[f] == ("add", True)


@pytest.mark.parametrize("functor,kernel_form", [
    (lambda a, b: max(a, b), True), (max, True), (lambda a, b: b if b > a else a, True),
    (lambda a, b: b if a < b else a, True), (lambda a, b: min(a, b), True), (lambda a, b: b if b < a else a, True),
    (lambda a, b: b if a > b else a, True),
    # the same operators for integers; NaN or equal operands come out differently
    (lambda a, b: a if a > b else b, False), (lambda a, b: a if a >= b else b, False),
    (lambda a, b: b if b >= a else a, False), (lambda a, b: a if a < b else b, False),
    (lambda a, b: b if a >= b else a, False),
])
def test_comparison_spellings_that_differ_from_the_kernels_are_told_apart(functor, kernel_form):
    detail = {}
    assert classify_functor(functor, detail) in ("max", "min")
    assert detail.get("kernel_form", True) is kernel_form
    r = cuda.Reduce(functor)
    assert r._kernel_form is kernel_form and r._native_off is (not kernel_form)
    # what Python itself makes of NaN with this functor, against the kernels' rule
    nan = float("nan")
    op = classify_functor(functor)
    kernel = (lambda a, b: b if b > a else a) if op == "max" else (lambda a, b: b if b < a else a)
    same = all(repr(functor(a, b)) == repr(kernel(a, b)) for a, b in ((nan, 1.0), (1.0, nan), (0.0, -0.0), (-0.0, 0.0)))
    assert same is kernel_form


# ---------------------------------------------------------------- argument normalisation

def test_prepare_shape_strides_dtype():
    assert prepare_shape_strides_dtype(5, None, np.float32, "C") == ((5,), (4,), np.dtype(np.float32))
    assert prepare_shape_strides_dtype((2, 3), None, "f8", "C")[1] == (24, 8)
    assert prepare_shape_strides_dtype((2, 3), None, "f8", "F")[1] == (8, 16)
    assert prepare_shape_strides_dtype([2, 3], (100, 8), "f8", "C")[1] == (100, 8)
    assert prepare_shape_strides_dtype((), None, "f8", "C")[1] == ()
    assert prepare_shape_strides_dtype(np.array([2, 3]), None, "i2", "C")[0] == (2, 3)
    for bad in (2.0, np.float32(3), np.array([1.0, 2.0])):
        with pytest.raises(TypeError, match="shape must be an integer or tuple of integers"):
            prepare_shape_strides_dtype(bad, None, "f8", "C")
    with pytest.raises(ValueError, match="must be either C/F order"):
        prepare_shape_strides_dtype((2, 3), None, "f8", "K")


def test_memory_size_and_host_extents():
    assert drv.memory_size_from_info((3, 4), (32, 8), 8) == 2 * 32 + 3 * 8 + 8
    assert drv.memory_size_from_info((0, 4), (32, 8), 8) == 0
    assert drv.memory_size_from_info((), (), 16) == 16
    a = np.arange(24, dtype=np.int32).reshape(4, 6)
    base = a.ctypes.data
    assert drv.host_memory_extents(a) == (base, base + a.nbytes)
    v = a[::-1, ::2]
    lo, hi = drv.host_memory_extents(v)
    assert (lo, hi) == (base, base + 3 * 24 + 4 * 4 + 4)
    assert drv.host_memory_size(a[1:3]) == 2 * 24
    assert drv.host_pointer(a) == base
    assert drv.host_pointer(12345) == 12345
    ro = np.arange(4)
    ro.setflags(write=False)
    assert drv.host_pointer(ro, readonly=True) == ro.ctypes.data
    with pytest.raises(BufferError):
        drv.host_pointer(ro)
    assert drv.host_pointer(bytearray(b"abcd")) != 0
    d64 = np.zeros(3, "M8[s]")
    assert drv.host_pointer(d64) == d64.ctypes.data


# ---------------------------------------------------------------- pending deallocations

def test_pending_deallocs_flush_on_count(monkeypatch):
    # counts pinned by the reference's tests/cudadrv/test_deallocations.py:22-46
    monkeypatch.setattr(config, "CUDA_DEALLOCS_COUNT", 10)
    q = drv._PendingDeallocs(capacity=1 << 40)
    freed = []
    for i in range(10):
        q.add_item(freed.append, i, 4)
        assert len(q) == i + 1 and not freed
    q.add_item(freed.append, 10, 4)          # the 11th entry tips it over
    assert len(q) == 0 and freed == list(range(11))


def test_pending_deallocs_flush_on_bytes(monkeypatch):
    # test_deallocations.py:48-75: ratio 0.2 of the capacity
    monkeypatch.setattr(config, "CUDA_DEALLOCS_RATIO", 0.2)
    q = drv._PendingDeallocs(capacity=1000)
    freed = []
    q.add_item(freed.append, "a", 100)
    q.add_item(freed.append, "b", 100)
    assert len(q) == 2 and q.pending_bytes == 200 and q.byte_budget == 200      # not above 200 yet
    assert (q._size, q._max_pending_bytes) == (200, 200)    # names the reference's own tests read
    q.add_item(freed.append, "c", 1)
    assert len(q) == 0 and freed == ["a", "b", "c"] and q.pending_bytes == 0
    q.add_item(freed.append, "d")                  # unknown size counts as zero
    assert len(q) == 1 and q.pending_bytes == 0
    assert drv._PendingDeallocs().byte_budget == 0     # capacity not known yet


def test_pending_deallocs_survive_a_failing_release_and_reentry(monkeypatch):
    monkeypatch.setattr(config, "CUDA_DEALLOCS_COUNT", 100)
    q = drv._PendingDeallocs(capacity=1 << 40)
    freed = []

    def release(h):
        if h == "bad":
            raise ValueError("cannot release")
        if h == "again":
            q.add_item(freed.append, "late", 8)      # a release that parks another one
        freed.append(h)

    for h in ("a", "bad", "b", "again"):
        q.add_item(release, h, 10)
    with pytest.raises(ValueError):
        q.clear()
    assert freed == ["a"] and len(q) == 2 and q.pending_bytes == 20     # the rest is still waiting
    q.clear()
    assert freed == ["a", "b", "again"] and len(q) == 1
    q.clear()
    assert freed[-1] == "late" and len(q) == 0 and q.pending_bytes == 0


def test_pending_deallocs_from_many_threads(monkeypatch):
    import threading
    monkeypatch.setattr(config, "CUDA_DEALLOCS_COUNT", 7)
    q = drv._PendingDeallocs(capacity=1 << 40)
    freed = []

    def worker(base):
        for i in range(500):
            q.add_item(freed.append, base + i, 4)

    threads = [threading.Thread(target=worker, args=(k * 1000,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    q.clear()
    assert sorted(freed) == sorted(k * 1000 + i for k in range(8) for i in range(500))
    assert q.pending_bytes == 0


def test_pending_deallocs_disable_nests():
    # test_deallocations.py:78-142
    q = drv._PendingDeallocs(capacity=1 << 40)
    freed = []
    with q.disable():
        with q.disable():
            for i in range(30):
                q.add_item(freed.append, i)
            assert q.is_disabled and len(q) == 30 and not freed
        q.clear()
        assert len(q) == 30                     # still disabled by the outer block
    assert not q.is_disabled
    q.clear()
    assert len(q) == 0 and len(freed) == 30
    with pytest.raises(RuntimeError):
        with q.disable():
            raise RuntimeError("boom")
    assert not q.is_disabled                    # the counter unwinds on exceptions


# ---------------------------------------------------------------- memory pointers

def test_memory_pointer_refcounts_and_finalizers():
    # behaviour pinned by tests/cudadrv/test_cuda_memory.py:53-105
    dead = []
    m = drv.MemoryPointer(None, 0x1000, 256, finalizer=lambda: dead.append("m"))
    assert m.refct == 1 and m.is_managed and m.owner is m
    own = m.own()
    assert m.refct == 2
    v = m.view(16, 64)
    assert m.refct == 3
    assert v.device_ctypes_pointer.value == 0x1010 and v.size == 48
    assert m.view(200).size == 56
    assert m.refct == 3                            # the temporary view is gone again
    del own, v
    gc.collect()
    assert m.refct == 1 and not dead               # plain pointers live as long as the object
    m.free()
    assert dead == ["m"]
    with pytest.raises(RuntimeError, match="Freeing dead memory"):
        m.free()

    a = drv.AutoFreePointer(None, 0x2000, 64, finalizer=lambda: dead.append("a"))
    assert a.refct == 0
    o1, o2 = a.own(), a.own()
    assert a.refct == 2
    del o1
    gc.collect()
    assert a.refct == 1 and dead == ["m"]
    del o2
    gc.collect()
    assert dead == ["m", "a"]                      # last owned reference frees it

    with pytest.raises(RuntimeError, match="size cannot be negative"):
        m.view(10, 5)
    null = drv.MemoryPointer(None, 0, 0)
    assert null.view(0, 0).device_ctypes_pointer.value == 0 and null.view(0, 0).size == 0
    with pytest.raises(RuntimeError, match="non-empty slice into empty slice"):
        null.view(0, 4)

    class Foreign:
        pass

    f = Foreign()
    ext = drv.MemoryPointer(None, 0x3000, 32, owner=f)
    ev = ext.view(8)
    assert isinstance(ev, drv.MemoryPointer) and ev.owner is f     # carries the foreign owner along


def test_is_device_memory_duck_typing():
    class Mem:
        __cuda_memory__ = True
        device_ctypes_pointer = ctypes.c_size_t(42)

    assert drv.is_device_memory(Mem())
    assert not drv.is_device_memory(np.zeros(1))
    assert drv.device_pointer(Mem()) == 42
    assert drv.device_ctypes_pointer(None).value is None
    with pytest.raises(Exception, match="Not a CUDA memory object"):
        drv.require_device_memory(object())


def test_stream_handle_rules():
    assert drv._stream_handle(0) == 0
    assert drv._stream_handle(drv.Stream(77)) == 77
    with pytest.raises(TypeError, match="Expected a Stream object or 0"):
        drv._stream_handle("s")
    # a Stream object is always "a stream was given", the default stream too (the
    # reference's tests/cudadrv/test_cuda_array_slicing.py:341-379 depend on it)
    assert drv.Stream(0) and drv.Stream(5) and drv.Stream(0) == 0
    assert repr(drv.Stream(0)) == "<Default HIP stream>"
    assert int(drv.Stream(9)) == 9 and drv.Stream(9).__cuda_stream__() == (0, 9)


def test_config_reads_reference_variable_names(monkeypatch):
    monkeypatch.setenv("NUMBA_CUDA_MAX_PENDING_DEALLOCS_COUNT", "3")
    monkeypatch.setenv("NUMBA_CUDA_MAX_PENDING_DEALLOCS_RATIO", "0.5")
    monkeypatch.setenv("NUMBA_CUDA_WARN_ON_IMPLICIT_COPY", "0")
    config.reload_config()
    try:
        assert (config.CUDA_DEALLOCS_COUNT, config.CUDA_DEALLOCS_RATIO) == (3, 0.5)
        assert config.CUDA_WARN_ON_IMPLICIT_COPY == 0
    finally:
        for k in ("NUMBA_CUDA_MAX_PENDING_DEALLOCS_COUNT", "NUMBA_CUDA_MAX_PENDING_DEALLOCS_RATIO",
                  "NUMBA_CUDA_WARN_ON_IMPLICIT_COPY"):
            monkeypatch.delenv(k)
        config.reload_config()
    assert config.CUDA_DEALLOCS_COUNT == 10
