"""nbh_reduce_noalloc (the reduction whose scratch is part of the library image)
against nbh_reduce with a caller-owned scratch buffer, both through the C ABI.

Bar: identical bits (both run the same kernels on the same grid), for integers and
floating point alike, and the integer results equal the oracle's.  Each case makes
two calls in a row, the second on a smaller input, because the static array keeps
what the previous call left in it.
"""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd import _lib
from numba_cuda_amd.cudadrv import driver as drv
from oracle import cref

MAX_ITEMS = 1 << 36          # NBH_REDUCE_NOALLOC_MAX_ITEMS


def _say(*a):
    print(*a, flush=True)


def _both(op, a, init, stream=0):
    """(result of nbh_reduce, result of nbh_reduce_noalloc) for host array `a`."""
    cuda.current_context()
    lib = drv.driver.lib
    d = cuda.to_device(a)
    code = _lib.DTYPE_CODES[a.dtype.name]
    opc = _lib.OP_CODES[op]
    init_buf = np.array([init], dtype=a.dtype)
    out_a = cuda.to_device(np.full(1, 77, dtype=a.dtype))
    out_b = cuda.to_device(np.full(1, 99, dtype=a.dtype))
    hstream = drv._stream_handle(stream) or None
    scratch_bytes = lib.nbh_reduce_scratch_bytes()
    scratch = cuda.to_device(np.zeros(scratch_bytes, dtype=np.uint8))      # caller-owned, cleared once
    scratch_ptr = scratch.device_ctypes_pointer.value
    rc = lib.nbh_reduce(opc, code, d.device_ctypes_pointer.value, a.size, a.strides[0], init_buf.ctypes.data,
                        out_a.device_ctypes_pointer.value, scratch_ptr, scratch_bytes, hstream)
    assert rc == 0
    rc = lib.nbh_reduce_noalloc(opc, code, d.device_ctypes_pointer.value, a.size, a.strides[0],
                                init_buf.ctypes.data, out_b.device_ctypes_pointer.value, hstream)
    assert rc == 0
    if stream:
        stream.synchronize()
    else:
        cuda.synchronize()
    return out_a.copy_to_host()[0], out_b.copy_to_host()[0]


CASES = [
    ("add", np.int64, 1 << 22, 100003),
    ("add", np.float32, (1 << 24) + 5, 4097),
    ("max", np.float64, 3_000_001, 1),
    ("mul", np.uint32, 1 << 20, 129),
    ("add", np.complex128, 1 << 19, 33),
    ("xor", np.uint8, (1 << 23) + 3, 2049),
]


@pytest.mark.parametrize("op,dtype,n_big,n_small", CASES)
def test_noalloc_matches_reduce_twice_in_a_row(op, dtype, n_big, n_small):
    rng = np.random.default_rng(11)
    for n in (n_big, n_small):          # the second call finds the first one's partials
        _say("noalloc case", op, np.dtype(dtype).name, n)
        if np.dtype(dtype).kind == "c":
            a = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dtype)
        elif np.dtype(dtype).kind == "f":
            a = rng.standard_normal(n).astype(dtype)
        else:
            info = np.iinfo(dtype)
            a = rng.integers(info.min, info.max, n, dtype=dtype, endpoint=True)
        init = 3 if op != "xor" else 5
        want, got = _both(op, a, init)
        assert want.tobytes() == got.tobytes(), (want, got)
        if np.dtype(dtype).kind in "iu":
            assert got == cref.fold(op, a, init=init)


def test_noalloc_on_a_stream_and_back_to_back():
    s = cuda.stream()
    rng = np.random.default_rng(12)
    lib = drv.driver.lib
    a = rng.integers(-1000, 1000, 1 << 21).astype(np.int64)
    d = cuda.to_device(a, stream=s)
    outs = cuda.device_array(64, dtype=np.int64, stream=s)
    init_buf = np.zeros(1, dtype=np.int64)
    sizes = [a.size >> (k % 7) for k in range(64)]
    for k, n in enumerate(sizes):       # ordered on one stream: no overlap
        rc = lib.nbh_reduce_noalloc(0, _lib.DTYPE_CODES["int64"], d.device_ctypes_pointer.value, n, 8,
                                    init_buf.ctypes.data, outs.device_ctypes_pointer.value + 8 * k, s.handle)
        assert rc == 0
    s.synchronize()
    got = outs.copy_to_host()
    want = np.array([a[:n].sum() for n in sizes])
    assert (got == want).all()


def test_noalloc_rejects_sizes_beyond_its_limit_and_bad_arguments():
    lib = drv.driver.lib
    cuda.current_context()
    one = cuda.to_device(np.ones(4, dtype=np.float32))
    out = cuda.device_array(1, dtype=np.float32)
    init = np.zeros(1, dtype=np.float32)
    p, o = one.device_ctypes_pointer.value, out.device_ctypes_pointer.value
    f32 = _lib.DTYPE_CODES["float32"]
    # refused before anything is launched (the input is 16 bytes long)
    assert lib.nbh_reduce_noalloc(0, f32, p, MAX_ITEMS + 1, 4, init.ctypes.data, o, None) == 1   # hipErrorInvalidValue
    assert lib.nbh_reduce_noalloc(0, 99, p, 4, 4, init.ctypes.data, o, None) == 1
    assert lib.nbh_reduce_noalloc(0, f32, p, 0, 4, init.ctypes.data, o, None) == 1
    assert lib.nbh_reduce_noalloc(0, f32, p, 4, 4, init.ctypes.data, o, None) == 0
    cuda.synchronize()
    assert out.copy_to_host()[0] == 4.0


def test_calls_allocate_nothing():
    """Free device memory (and, with the pooling manager, what the pool holds) is the same
    after a loop of calls as after the first one: no hipMalloc behind this entry point."""
    import ctypes
    cuda.current_context()
    lib = drv.driver.lib
    a = np.random.default_rng(3).integers(-1000, 1000, 1 << 20, dtype=np.int64)
    d = cuda.to_device(a)
    out = cuda.device_array(1, np.int64)
    init = np.zeros(1, np.int64)
    code, op = _lib.DTYPE_CODES["int64"], _lib.OP_CODES["add"]

    def call(n):
        assert lib.nbh_reduce_noalloc(op, code, d.device_ctypes_pointer.value, n, 8, init.ctypes.data,
                                      out.device_ctypes_pointer.value, None) == 0

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert lib.nbh_mem_info(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    call(a.size)                      # first call on the device: looks the array up
    cuda.synchronize()
    before = free_bytes()
    for i in range(200):
        call(a.size - 17 * i)
    cuda.synchronize()
    assert free_bytes() == before
    assert out.copy_to_host()[0] == a[:a.size - 17 * 199].sum()


def test_overlap_on_another_stream_is_refused_not_raced():
    """A call on a second stream while the first stream's call is still running would share the
    ticket: hipErrorNotReady instead; after the first stream is done the same call goes through."""
    cuda.current_context()
    lib = drv.driver.lib
    big = cuda.to_device(np.ones(1 << 28, dtype=np.int32))
    small = cuda.to_device(np.arange(1000, dtype=np.int32))
    out_big, out_small = cuda.device_array(1, np.int32), cuda.device_array(1, np.int32)
    init = np.zeros(1, np.int32)
    code, op = _lib.DTYPE_CODES["int32"], _lib.OP_CODES["add"]
    s1, s2 = cuda.stream(), cuda.stream()
    cuda.synchronize()
    for _ in range(3):                # about half a millisecond of work on the first stream
        assert lib.nbh_reduce_noalloc(op, code, big.device_ctypes_pointer.value, big.size, 4, init.ctypes.data,
                                      out_big.device_ctypes_pointer.value, s1.handle) == 0
    rc = lib.nbh_reduce_noalloc(op, code, small.device_ctypes_pointer.value, small.size, 4, init.ctypes.data,
                                out_small.device_ctypes_pointer.value, s2.handle)
    HIP_ERROR_NOT_READY = 600
    assert rc == HIP_ERROR_NOT_READY
    s1.synchronize()
    assert out_big.copy_to_host()[0] == 1 << 28
    assert lib.nbh_reduce_noalloc(op, code, small.device_ctypes_pointer.value, small.size, 4, init.ctypes.data,
                                  out_small.device_ctypes_pointer.value, s2.handle) == 0
    s2.synchronize()
    assert out_small.copy_to_host()[0] == 499500
