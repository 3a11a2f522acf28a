"""Launching threads (kernels/reduction.py launch_threads, nbh_reduce_queued): the mode (on unless
NUMBA_CUDA_REDUCE_LAUNCH_THREADS=0) in which `Reduce(...)(arr, res=..., stream=s)` hands its kernel
launch to a thread that belongs to the stream, until the stream's handle is read by code outside
the package.  Results and ordering must be those of the default mode whatever else the
package does with the stream in between; integer data, so every comparison is exact."""
import ctypes
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd.cudadrv import driver as drv
from numba_cuda_amd.kernels import reduction

sum_reduce = cuda.Reduce(lambda a, b: a + b)


def _say(*a):
    print(*a, flush=True)


@pytest.fixture
def queued():
    reduction.launch_threads(True)
    yield


def test_switching_changes_the_entry_the_native_passage_calls():
    cuda.current_context()
    lib = drv.driver.lib
    direct = ctypes.cast(lib.nbh_reduce, ctypes.c_void_p).value
    through_queue = ctypes.cast(lib.nbh_reduce_queued, ctypes.c_void_p).value
    reduction.launch_threads(False)
    try:
        assert lib._reduce_entry == direct
    finally:
        reduction.launch_threads(True)
    assert lib._reduce_entry == through_queue


def test_rows_over_four_streams_match_numpy(queued):
    rng = np.random.default_rng(11)
    rows, cols = 3000, 4099
    host = rng.integers(-1000, 1000, (rows, cols), dtype=np.int32)
    dm = cuda.to_device(host)
    out = cuda.device_array(rows, np.int32)
    streams = [cuda.stream() for _ in range(4)]
    for rep in range(3):
        out[:] = 0
        for r in range(rows):
            sum_reduce(dm[r], res=out[r:r + 1], stream=streams[r & 3])
        # a copy on the default stream: waits for every queue, then for the device
        assert (out.copy_to_host() == host.sum(axis=1, dtype=np.int32)).all(), rep


def test_other_work_on_the_same_stream_keeps_its_place(queued):
    """fill, reduce, fill, reduce ... on one stream: a fill must not overtake the reduction
    queued before it, nor a reduction the fill before it."""
    s = cuda.stream()
    n, rounds = 50_000, 300
    work = cuda.device_array(n, np.int64, stream=s)
    out = cuda.device_array(rounds, np.int64)
    out[:] = -1
    for k in range(rounds):
        work.setitem(slice(None), k + 1, stream=s)
        sum_reduce(work, res=out[k:k + 1], stream=s)
    s.synchronize()
    assert (out.copy_to_host() == (np.arange(rounds, dtype=np.int64) + 1) * n).all()


def test_events_and_asynchronous_copies_follow_the_queue(queued):
    s = cuda.stream()
    host = np.arange(1, 200_001, dtype=np.int64)
    d = cuda.to_device(host, stream=s)
    res = cuda.device_array(1, np.int64)
    back = cuda.pinned_array(1, np.int64)
    back[0] = 0
    for _ in range(50):
        sum_reduce(d, res=res, stream=s)
    res.copy_to_host(back, stream=s)
    done = cuda.event()
    done.record(s)
    done.synchronize()
    assert back[0] == host.sum()


def test_inputs_released_right_after_the_call(queued):
    rng = np.random.default_rng(5)
    s = [cuda.stream() for _ in range(2)]
    out = cuda.device_array(400, np.int32)
    want = np.empty(400, np.int32)
    for k in range(400):
        h = rng.integers(-50, 50, 10_000 + k, dtype=np.int32)
        want[k] = h.sum(dtype=np.int32)
        d = cuda.to_device(h)
        sum_reduce(d, res=out[k:k + 1], stream=s[k & 1])
        del d                                   # its memory may go back before the launch is made
    assert (out.copy_to_host() == want).all()


def test_a_stream_destroyed_with_launches_still_queued(queued):
    host = np.arange(100_000, dtype=np.int64)
    d = cuda.to_device(host)
    out = cuda.device_array(64, np.int64)
    for rep in range(5):
        s = cuda.stream()
        for k in range(64):
            sum_reduce(d, res=out[k:k + 1], stream=s)
        del s
        cuda.synchronize()
        assert (out.copy_to_host() == host.sum()).all(), rep


def test_several_host_threads_on_one_stream_and_on_their_own(queued):
    rng = np.random.default_rng(9)
    shared = cuda.stream()
    host = rng.integers(-9, 9, (8, 500, 257), dtype=np.int64)
    dm = cuda.to_device(host)
    out = cuda.device_array((8, 500), np.int64)
    failures = []

    def worker(t):
        try:
            mine = shared if t < 4 else cuda.stream()
            for k in range(500):
                sum_reduce(dm[t, k], res=out[t, k:k + 1], stream=mine)
            mine.synchronize()
        except Exception as e:     # pragma: no cover - reported below
            failures.append(repr(e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures
    cuda.synchronize()
    assert (out.copy_to_host() == host.sum(axis=2)).all()


def test_a_launch_that_fails_is_reported_by_the_next_synchronize(queued):
    lib = drv.driver.lib
    ctx = cuda.current_context()
    s = cuda.stream()
    d = cuda.to_device(np.arange(64, dtype=np.int32))
    res = cuda.device_array(1, np.int32)
    scratch = ctx.reduce_scratch(s._h)              # `_h`: reading `handle` would take the stream out of the mode
    init = np.zeros(1, np.int32)
    # a stride that is no multiple of the item size: refused by the launch itself
    rc = lib.nbh_reduce_queued(0, 2, d.device_ctypes_pointer.value, 8, 6, init.ctypes.data,
                               res.device_ctypes_pointer.value, scratch[0], scratch[1], s._h)
    assert rc == 0                                              # queued, not yet looked at
    assert lib.nbh_stream_synchronize(s._h) == 1                # hipErrorInvalidValue, reported once
    assert lib.nbh_stream_synchronize(s._h) == 0
    sum_reduce(d, res=res, stream=s)                            # the stream is as good as before
    s.synchronize()
    assert res.copy_to_host()[0] == 64 * 63 // 2


def test_default_streams_are_never_queued(queued):
    d = cuda.to_device(np.arange(1000, dtype=np.int64))
    res = cuda.device_array(1, np.int64)
    sum_reduce(d, res=res)                       # stream 0: launched on this thread
    assert res.copy_to_host()[0] == 999 * 500
    assert sum_reduce(d) == 999 * 500            # and the value-returning form


def test_switching_back_and_forth_between_calls():
    rng = np.random.default_rng(21)
    host = rng.integers(-99, 99, (64, 3001), dtype=np.int64)
    dm = cuda.to_device(host)
    out = cuda.device_array(64, np.int64)
    streams = [cuda.stream() for _ in range(3)]
    try:
        for rep in range(20):
            reduction.launch_threads(rep % 2 == 0)
            for r in range(64):
                sum_reduce(dm[r], res=out[r:r + 1], stream=streams[r % 3])
            if rep % 5 == 4:
                streams[rep % 3] = cuda.stream()     # the old one goes with its thread
            assert (out.copy_to_host() == host.sum(axis=1)).all(), rep
    finally:
        reduction.launch_threads(True)


def test_exported_array_interface_waits_for_the_queues(queued):
    """A consumer of __cuda_array_interface__ is outside the package: reading the attribute
    puts the queued launches into their streams first (torch then synchronises on the device)."""
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    s = cuda.stream()
    host = np.arange(1, 100_001, dtype=np.int64)
    d = cuda.to_device(host)
    res = cuda.device_array(200, np.int64)
    for k in range(200):
        sum_reduce(d, res=res[k:k + 1], stream=s)
    t = torch.as_tensor(res, device="cuda")          # reads the interface
    torch.cuda.synchronize()
    assert bool((t == int(host.sum())).all())


def test_a_stream_that_leaves_the_package_is_launched_directly_from_then_on(queued):
    """Work queued before the handle is read is in the stream when the read returns; afterwards the
    stream's reductions are launched by the caller (a failing launch reports at the call, not at the
    next synchronize); a consumer of the array interface that carries the stream finds it in order."""
    lib = drv.driver.lib
    ctx = cuda.current_context()
    s = cuda.stream()
    host = np.arange(1, 200_001, dtype=np.int64)
    d = cuda.to_device(host, stream=s)
    res = cuda.device_array(300, np.int64, stream=s)
    for k in range(300):
        sum_reduce(d, res=res[k:k + 1], init=k, stream=s)
    raw = int(s)                                      # the handle leaves: everything queued is launched
    assert lib.nbh_stream_synchronize(raw) == 0
    assert (res.copy_to_host(stream=s) == host.sum() + np.arange(300)).all()
    # direct from now on: a launch the runtime refuses is reported by the call itself
    scratch = ctx.reduce_scratch(raw)
    init = np.zeros(1, np.int64)
    rc = lib.nbh_reduce_queued(0, 3, d.device_ctypes_pointer.value, 8, 6, init.ctypes.data,
                               res.device_ctypes_pointer.value, scratch[0], scratch[1], raw)
    assert rc != 0
    for k in range(300):
        sum_reduce(d, res=res[k:k + 1], init=-k, stream=s)
    s.synchronize()
    assert (res.copy_to_host() == host.sum() - np.arange(300)).all()
    # a stream seen first through the array interface of an array bound to it
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    s2 = cuda.stream()
    res2 = cuda.device_array(200, np.int64, stream=s2)
    for k in range(200):
        sum_reduce(d, res=res2[k:k + 1], init=7, stream=s2)
    desc = res2.__cuda_array_interface__
    assert desc["stream"] == s2._h and s2._exported
    t = torch.as_tensor(res2, device="cuda")
    torch.cuda.synchronize()
    assert bool((t == int(host.sum()) + 7).all())


def test_environment_variable_zero_switches_the_mode_off():
    import os
    import subprocess
    import sys
    code = (
        "import ctypes, numpy as np, numba_cuda_amd as cuda\n"
        "from numba_cuda_amd.cudadrv import driver as drv\n"
        "red = cuda.Reduce(lambda a, b: a + b)\n"
        "h = np.arange(1000, dtype=np.int64); d = cuda.to_device(h); out = cuda.device_array(1, np.int64)\n"
        "s = cuda.stream(); red(d, res=out, stream=s); s.synchronize()\n"
        "lib = drv.driver.lib\n"
        "assert lib._reduce_entry == ctypes.cast(lib.nbh_reduce, ctypes.c_void_p).value\n"
        "assert out.copy_to_host()[0] == h.sum()\n"
        "print('ok')\n")
    env = dict(os.environ, NUMBA_CUDA_REDUCE_LAUNCH_THREADS="0",
               PYTHONPATH=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    done = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert done.returncode == 0 and done.stdout.strip().endswith("ok"), done.stderr[-2000:]


def test_environment_variable_starts_the_mode():
    import os
    import subprocess
    import sys
    code = (
        "import ctypes, numpy as np, numba_cuda_amd as cuda\n"
        "from numba_cuda_amd.cudadrv import driver as drv\n"
        "red = cuda.Reduce(lambda a, b: a + b)\n"
        "h = np.arange(100000, dtype=np.int64); d = cuda.to_device(h); out = cuda.device_array(8, np.int64)\n"
        "ss = [cuda.stream() for _ in range(2)]\n"
        "for rep in range(3):\n"
        "    for k in range(8): red(d, res=out[k:k+1], stream=ss[k & 1])\n"
        "lib = drv.driver.lib\n"
        "assert lib._reduce_entry == ctypes.cast(lib.nbh_reduce_queued, ctypes.c_void_p).value\n"
        "assert (out.copy_to_host() == h.sum()).all()\n"
        "print('ok')\n")
    env = dict(os.environ, NUMBA_CUDA_REDUCE_LAUNCH_THREADS="1",
               PYTHONPATH=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    done = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=110)
    assert done.returncode == 0 and done.stdout.strip().endswith("ok"), done.stderr[-2000:]
