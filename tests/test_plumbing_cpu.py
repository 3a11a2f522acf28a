"""Device-array plumbing on a machine without a GPU: the driver layer is bound to
a fake library that keeps device memory in host RAM (tests/fakelib.py)."""

import numpy as np
import pytest

import numba_cuda_amd as cuda
from tests import (attr_cases, cai_cases, dealloc_cases, device_cases, emm_cases, host_stream_cases,
                   memory_cases, ndarray_cases, plumbing_cases, pool_cases, record_cases, slicing_cases)

# plumbing_cases: this package's own; the others restate the reference's suites
CASES = (plumbing_cases.ALL + ndarray_cases.ALL + slicing_cases.ALL + memory_cases.ALL + host_stream_cases.ALL
         + record_cases.ALL + dealloc_cases.ALL + emm_cases.ALL + attr_cases.ALL + device_cases.ALL + cai_cases.ALL
         + pool_cases.ALL)


@pytest.mark.parametrize("case", CASES, ids=lambda f: f.__name__)
def test_plumbing(case, fake_gpu):
    case(cuda)


def test_out_of_memory_flushes_pending_frees_and_retries(fake_gpu):
    """driver.py:728-745 of the reference: one retry after flushing."""
    import gc
    with cuda.defer_cleanup():
        for _ in range(3):
            cuda.device_array(16)
        gc.collect()
    ctx = cuda.current_context()
    assert len(ctx.memory_manager.deallocations) == 3
    fake_gpu.fail_next_malloc = 1
    d = cuda.device_array(16)                     # first attempt fails, flush, retry succeeds
    assert d.size == 16 and len(ctx.memory_manager.deallocations) == 0
    fake_gpu.fail_next_malloc = 2
    with pytest.raises(cuda.CudaAPIError) as e:
        cuda.device_array(16)
    assert e.value.code == 2 and "hipErrorOutOfMemory" in str(e.value)
    assert "Call to nbh_malloc results in" in e.value.msg


def test_sync_vs_async_copy_selection(fake_gpu):
    """stream 0 -> synchronous entry point semantics (NULL stream); a Stream ->
    its handle is passed through (driver.py:2625-2670 of the reference)."""
    a = np.arange(8.0)
    d = cuda.to_device(a)
    s = cuda.stream()
    fake_gpu.calls.clear()
    d.copy_to_host()
    d.copy_to_host(stream=s)
    d.bind(s).copy_to_host()                      # bound stream is the default
    kinds = [(c[0], c[4]) for c in fake_gpu.calls if c[0] == "d2h"]
    assert kinds == [("d2h", 0), ("d2h", int(s)), ("d2h", int(s))]
    fake_gpu.calls.clear()
    d.copy_to_device(a)
    d.copy_to_device(a, stream=s)
    assert [(c[0], c[4]) for c in fake_gpu.calls if c[0] == "h2d"] == [("h2d", 0), ("h2d", int(s))]
    # element access copies exactly one item
    fake_gpu.calls.clear()
    assert d[3] == 3.0
    assert [c for c in fake_gpu.calls if c[0] == "d2h"][0][3] == 8


def test_compute_without_the_real_library_fails_loudly(fake_gpu):
    d = cuda.to_device(np.arange(8.0))
    with pytest.raises(AttributeError):
        cuda.reduce(lambda a, b: a + b)(d)
    with pytest.raises(AttributeError):
        cuda.to_device(np.zeros((2, 3))).T
    with pytest.raises(AttributeError):
        cuda.random.create_xoroshiro128p_states(4, seed=1)


def test_reduce_host_side_contract(fake_gpu):
    red = cuda.reduce(lambda a, b: a + b)
    with pytest.raises(TypeError, match="only support 1D array"):
        red(np.zeros((2, 2)))
    # empty input returns init converted to the dtype and never touches the device
    fake_gpu.calls.clear()
    got = red(np.zeros(0, np.float32), init=3)
    assert got == 3 and isinstance(got, np.float32)
    assert red(cuda.device_array(10, np.int16), size=0, init=2) == 2
    assert not [c for c in fake_gpu.calls if c[0] in ("h2d", "d2h")]
    with pytest.raises(NotImplementedError, match="dtype"):
        red(np.zeros(4, np.dtype("S4")))
    with pytest.raises(TypeError, match="not defined for complex64"):
        cuda.reduce(lambda a, b: max(a, b))(np.zeros(4, np.complex64))
    # booleans under + run as the uint8 `or` kernel, float16 has kernels of its own
    assert red._codes_for(np.dtype(np.bool_)) == (5, 4)
    assert cuda.reduce(lambda a, b: a * b)._codes_for(np.dtype(np.bool_)) == (4, 4)
    assert red._codes_for(np.dtype(np.float16)) == (0, 12)
    with pytest.raises(TypeError, match="bitwise xor is not defined for float32"):
        cuda.reduce(lambda a, b: a ^ b)(np.zeros(4, np.float32))


def test_random_host_scalar_functions_match_the_oracle():
    from numba_cuda_amd import random as nrandom
    from oracle import cref, xoroshiro_py as xp
    st = np.zeros(3, nrandom.xoroshiro128p_dtype)
    for i in range(3):
        nrandom.init_xoroshiro128p_state(st, i, 40 + i)
        assert (int(st[i]["s0"]), int(st[i]["s1"])) == xp.seed_state(40 + i)
    s = xp.seed_state(41)
    for _ in range(20):
        draw, a, b = xp.next_state(*s)
        s = (a, b)
        assert int(nrandom.xoroshiro128p_next(st, 1)) == draw
    nrandom.xoroshiro128p_jump(st, 2)
    assert (int(st[2]["s0"]), int(st[2]["s1"])) == xp.jump(*xp.seed_state(42))
    ref = cref.init_states(4, 9)
    mine = ref.copy()
    want32, _ = cref.fill(ref, 2, "uniform_f32")
    want64, _ = cref.fill(ref, 2, "uniform_f64")
    m2 = ref.copy()
    for t in range(4):
        for i in range(2):
            assert nrandom.xoroshiro128p_uniform_float32(mine, t) == want32[2 * t + i]
            assert nrandom.xoroshiro128p_uniform_float64(m2, t) == want64[2 * t + i]
    n32, _ = cref.fill(ref, 1, "normal_f32")
    n64, _ = cref.fill(ref, 1, "normal_f64")
    a, b = ref.copy(), ref.copy()
    for t in range(4):
        assert abs(nrandom.xoroshiro128p_normal_float32(a, t) - n32[t]) <= 2 * np.spacing(abs(n32[t]))
        assert abs(nrandom.xoroshiro128p_normal_float64(b, t) - n64[t]) <= 4 * np.spacing(abs(n64[t]))


def test_scalar_functions_on_device_states_go_through_the_one_generator_kernel(fake_gpu):
    """Host logic only (there is no kernel on the fake library): which record address,
    which kind and which output cell the per-generator functions pass on."""
    from numba_cuda_amd import random as nrandom
    d = cuda.device_array(4, dtype=nrandom.xoroshiro128p_dtype)
    base = d.device_ctypes_pointer.value
    calls = []

    def nbh_xoro_one(state, kind, out, stream):
        calls.append((state, kind, out))
        if out:
            ctypes.c_uint64.from_address(out).value = 0x3FF8000000000000       # 1.5 as a double
        return 0

    import ctypes
    fake_gpu.nbh_xoro_one = nbh_xoro_one
    got = nrandom.xoroshiro128p_uniform_float64(d, 2)
    assert isinstance(got, np.float64) and got == 1.5
    assert calls[-1][:2] == (base + 32, 3) and calls[-1][2]
    got = nrandom.xoroshiro128p_next(d, -1)
    assert isinstance(got, np.uint64) and calls[-1][:2] == (base + 48, 0)
    assert nrandom.xoroshiro128p_jump(d, 0) is None and calls[-1] == (base, 1, None)
    assert isinstance(nrandom.xoroshiro128p_normal_float32(d, 1), np.float32) and calls[-1][1] == 4
    with pytest.raises(IndexError):
        nrandom.xoroshiro128p_uniform_float32(d, 4)
    with pytest.raises(TypeError, match="device array"):
        nrandom.xoroshiro128p_fill(np.zeros(4, nrandom.xoroshiro128p_dtype), d)


def test_setitem_host_logic_and_synchronisation(fake_gpu):
    """`darr[key] = value`: broadcasting rules, error messages and when the call
    waits (reference: tests/cudadrv/test_cuda_array_slicing.py:220-379).  The fake
    library performs the strided assignment with NumPy."""
    a = np.arange(5 * 7, dtype=np.float64).reshape(5, 7)
    d = cuda.to_device(a)
    fake_gpu.calls.clear()
    d[2, 3] = 500                       # no stream anywhere: default stream + wait
    assert [c[0] for c in fake_gpu.calls if c[0] in ("assign", "stream_sync")][-2:] == ["assign", "stream_sync"]
    a[2, 3] = 500
    d[:, 2] = np.arange(5.0)
    a[:, 2] = np.arange(5.0)
    d[1:3] = np.array([[1.0], [2.0]])   # unit axis on the right repeats
    a[1:3] = np.array([[1.0], [2.0]])
    d[4] = 7
    a[4] = 7
    np.testing.assert_array_equal(d.copy_to_host(), a)
    s = cuda.stream()
    fake_gpu.calls.clear()
    d.setitem(0, 1.5, stream=s)         # explicit stream: asynchronous, no wait
    d.bind(s)[1] = 2.5                  # bound stream: asynchronous too
    kinds = [c[0] for c in fake_gpu.calls if c[0] in ("assign", "stream_sync")]
    assert kinds == ["assign", "assign"]
    assert all(c[4] == int(s) for c in fake_gpu.calls if c[0] == "assign")
    with pytest.raises(ValueError, match="Can't assign 3-D array to 2-D self"):
        d[:] = np.zeros((1, 5, 7))
    with pytest.raises(ValueError, match="Can't copy sequence with size 3 to array axis 1 with dimension 7"):
        d[:] = np.zeros((5, 3))
    with pytest.raises(TypeError, match="incompatible dtype"):
        d[:] = cuda.to_device(np.zeros((5, 7), np.float32))


def test_stream_callbacks(fake_gpu):
    import asyncio
    s = cuda.stream()
    seen = []
    s.add_callback(lambda stream, status, arg: seen.append((stream is s, status, arg)), "payload")
    assert seen == [(True, 0, "payload")]
    with pytest.warns(UserWarning, match="Exception in stream callback"):
        s.add_callback(lambda *a: 1 / 0)

    async def wait():
        return await s.async_done()

    assert asyncio.run(wait()) is s


class _RecordingManager(cuda.HostOnlyCUDAMemoryManager):
    """An External Memory Management plugin that only takes over device
    allocations (the shape of the reference's tests/cudadrv/test_emm_plugins.py
    :14-60 DeviceOnlyEMMPlugin)."""

    log = []

    def initialize(self):
        self.log.append("initialize")

    def memalloc(self, size):
        import ctypes
        from numba_cuda_amd.cudadrv import driver as drv
        buf = ctypes.create_string_buffer(size)
        self.log.append(("memalloc", size))
        key = ctypes.addressof(buf)

        def finalizer():
            self.log.append(("free", size))
            self.allocations.pop(key, None)

        mem = drv.AutoFreePointer(self.context, key, size, finalizer=finalizer)
        self.allocations[key] = (mem, buf)      # the manager keeps the pointer object alive
        return mem.own()

    def get_ipc_handle(self, memory):
        raise NotImplementedError

    def get_memory_info(self):
        self.log.append("get_memory_info")
        return cuda.MemoryInfo(free=32, total=64)

    @property
    def interface_version(self):
        return 1


def test_external_memory_manager_plugin(fake_gpu):
    import gc
    from numba_cuda_amd.cudadrv import driver as drv
    _RecordingManager.log.clear()
    cuda.set_memory_manager(_RecordingManager)
    try:
        ctx = cuda.current_context()
        assert isinstance(ctx.memory_manager, _RecordingManager)
        d = cuda.to_device(np.arange(10, dtype=np.int32))
        assert ("memalloc", 40) in _RecordingManager.log
        assert not any(c[0] == "malloc" for c in fake_gpu.calls)      # the default allocator is bypassed
        np.testing.assert_array_equal(d.copy_to_host(), np.arange(10))
        assert ctx.get_memory_info() == (32, 64)
        del d
        gc.collect()
        assert ("free", 40) in _RecordingManager.log

        class Wrong(_RecordingManager):
            @property
            def interface_version(self):
                return 2

        with pytest.raises(RuntimeError, match="EMM Plugin interface has version 2 - version 1 required"):
            cuda.set_memory_manager(Wrong)
    finally:
        drv._memory_manager = None
