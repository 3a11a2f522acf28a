"""Device-array plumbing on a machine without a GPU: the driver layer is bound to
a fake library that keeps device memory in host RAM (tests/fakelib.py)."""

import numpy as np
import pytest

import numba_cuda_amd as cuda
from tests import plumbing_cases


@pytest.mark.parametrize("case", plumbing_cases.ALL, ids=lambda f: f.__name__)
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
        red(np.zeros(4, np.complex64))


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


def test_device_states_are_refused_by_scalar_functions(fake_gpu):
    from numba_cuda_amd import random as nrandom
    d = cuda.device_array(4, dtype=nrandom.xoroshiro128p_dtype)
    with pytest.raises(TypeError, match="xoroshiro128p_fill"):
        nrandom.xoroshiro128p_uniform_float32(d, 0)
    with pytest.raises(TypeError, match="device array"):
        nrandom.xoroshiro128p_fill(np.zeros(4, nrandom.xoroshiro128p_dtype), d)
