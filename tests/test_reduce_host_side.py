"""Host side of Reduce without a GPU: which scratch buffer and which result cell a
call uses, from several host threads and streams, and that nothing kept per stream
outlives the stream.  The kernel is replaced by a recording stand-in that adds the
input up with NumPy - the arithmetic is not what these tests are about."""

import ctypes
import gc
import threading
import time

import numpy as np
import pytest

import numba_cuda_amd as cuda
from numba_cuda_amd.cudadrv import driver as drv
from numba_cuda_amd.kernels import reduction


def _install_recording_reduce(lib, delay=0.0):
    """Give the fake library an nbh_reduce that records (thread, scratch, out) and
    writes sum(in) + init to `out` when the stream is synchronised - i.e. late, the
    way a kernel result arrives."""
    record = []
    pending = []
    lock = threading.Lock()

    def nbh_reduce(op, code, in_ptr, n, stride, init_ptr, out, scratch, scratch_bytes, stream):
        data = np.frombuffer((ctypes.c_ubyte * (8 * n)).from_address(in_ptr), dtype=np.int64)
        init = np.frombuffer((ctypes.c_ubyte * 8).from_address(init_ptr), dtype=np.int64)[0]
        with lock:
            record.append((threading.get_ident(), scratch, out, stream))
            pending.append((out, int(data.sum() + init)))
        return 0

    def nbh_stream_synchronize(stream):
        if delay:
            time.sleep(delay)          # lets other threads launch in between, as on a GPU
        with lock:
            done, pending[:] = list(pending), []
        for out, value in done:
            ctypes.c_int64.from_address(out).value = value
        return 0

    lib.nbh_reduce = nbh_reduce
    lib.nbh_stream_synchronize = nbh_stream_synchronize
    return record


def test_scratch_is_kept_per_stream_and_per_thread_for_the_per_thread_stream(fake_gpu):
    ctx = cuda.current_context()
    a0, size = ctx.reduce_scratch(0)
    assert size == fake_gpu.nbh_reduce_scratch_bytes()
    assert ctx.reduce_scratch(0) == (a0, size)                   # made once
    a7, _ = ctx.reduce_scratch(0x7000)
    assert a7 != a0                                              # streams may overlap: one each

    mine, _ = ctx.reduce_scratch(drv.HIP_STREAM_PER_THREAD)
    assert ctx.reduce_scratch(drv.HIP_STREAM_PER_THREAD)[0] == mine
    theirs = []
    t = threading.Thread(target=lambda: theirs.append(ctx.reduce_scratch(drv.HIP_STREAM_PER_THREAD)[0]))
    t.start()
    t.join()
    assert theirs[0] not in (mine, a0, a7)      # same handle, but another thread's stream


def test_scratch_of_a_dead_thread_is_released(fake_gpu):
    ctx = cuda.current_context()
    ctx.memory_manager.deallocations.clear()
    before = len(fake_gpu.buffers)

    def worker():
        ctx.reduce_scratch(drv.HIP_STREAM_PER_THREAD)

    for _ in range(20):
        t = threading.Thread(target=worker)
        t.start()
        t.join()
    gc.collect()
    ctx.memory_manager.deallocations.clear()
    assert len(fake_gpu.buffers) - before <= 1


def test_stream_cycles_do_not_accumulate_scratch(fake_gpu):
    ctx = cuda.current_context()
    _install_recording_reduce(fake_gpu)
    add = cuda.Reduce(lambda a, b: a + b)
    d = cuda.to_device(np.arange(10, dtype=np.int64))
    ctx.memory_manager.deallocations.clear()
    before = len(fake_gpu.buffers)
    for i in range(1000):
        s = cuda.stream()
        assert add(d, stream=s) == 45
        del s
    gc.collect()
    assert len(ctx._scratch) <= 1                       # nothing kept for destroyed streams
    ctx.deallocations.clear()
    ctx.memory_manager.deallocations.clear()
    assert len(fake_gpu.buffers) - before <= 2
    assert not fake_gpu.live_streams


def test_value_returning_reductions_from_many_threads_on_one_stream(fake_gpu):
    cuda.current_context()
    record = _install_recording_reduce(fake_gpu, delay=0.002)
    add = cuda.Reduce(lambda a, b: a + b)
    arrays = [cuda.to_device(np.full(16, k + 1, dtype=np.int64)) for k in range(8)]
    wrong = []

    def worker(k):
        for i in range(50):
            got = add(arrays[k], init=i)              # all on the default stream
            if got != 16 * (k + 1) + i:
                wrong.append((k, i, got))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not wrong, wrong[:5]
    assert len(record) == 400
    assert len({scratch for _, scratch, _, _ in record}) == 1       # one stream: one scratch buffer


def test_result_cells_are_reused_not_leaked(fake_gpu):
    ctx = cuda.current_context()
    _install_recording_reduce(fake_gpu)
    add = cuda.Reduce(lambda a, b: a + b)
    d = cuda.to_device(np.arange(5, dtype=np.int64))
    for _ in range(2000):
        assert add(d) == 10
    cells = ctx._result_cells
    assert len(cells._blocks) == 1 and len(cells._free) == cells.BLOCK // cells.CELL
    held = [ctx.take_result_cell() for _ in range(300)]            # more than one block holds
    assert len({c[0] for c in held}) == 300 and len(cells._blocks) == 2
    for c in held:
        ctx.give_back_result_cell(c)


def test_res_argument_bypasses_the_cells_and_returns_none(fake_gpu):
    ctx = cuda.current_context()
    record = _install_recording_reduce(fake_gpu)
    add = cuda.Reduce(lambda a, b: a + b)
    d = cuda.to_device(np.arange(5, dtype=np.int64))
    res = cuda.device_array(1, dtype=np.int64)
    assert add(d, res=res, init=5) is None
    assert record[-1][2] == res.device_ctypes_pointer.value
    assert not ctx._result_cells._blocks
    fake_gpu.nbh_stream_synchronize(None)
    assert res.copy_to_host()[0] == 15


def test_res_must_hold_one_item_in_its_first_slice(fake_gpu):
    """The reference writes the result with res[:1].copy_to_device(partials[:1])
    (kernels/reduction.py:259-262): an empty or wider `res` is an error there, not a write past its end."""
    record = _install_recording_reduce(fake_gpu)
    add = cuda.Reduce(lambda a, b: a + b)
    d = cuda.to_device(np.arange(10, dtype=np.int64))
    with pytest.raises(ValueError, match="incompatible shape"):
        add(d, res=cuda.device_array(0, np.int64))
    with pytest.raises(ValueError, match="incompatible shape"):
        add(d, res=cuda.device_array((2, 3), np.int64))
    with pytest.raises(IndexError):
        add(d, res=cuda.device_array((), np.int64))
    with pytest.raises(TypeError, match="dtype"):
        add(d, res=cuda.device_array(1, np.int32))
    assert record == []
    column = cuda.device_array((4, 1), np.int64)         # its first slice is one item: accepted
    add(d, res=column)
    fake_gpu.nbh_stream_synchronize(None)
    assert column.copy_to_host()[0, 0] == 45 and len(record) == 1


def test_init_values_are_told_apart_by_their_bits():
    f64 = np.dtype(np.float64)
    plus = reduction._init_buffer(f64, 0.0)
    minus = reduction._init_buffer(f64, -0.0)
    assert plus != minus
    assert reduction._init_buffer(f64, 0) == plus                      # converted first, then looked up
    assert ctypes.c_double.from_address(minus).value == 0.0
    assert np.signbit(ctypes.c_double.from_address(minus).value)
    nan1 = reduction._init_buffer(f64, float("nan"))
    assert reduction._init_buffer(f64, float("nan")) == nan1           # same bit pattern, found again


def test_stream_callback_thunks_outlive_their_own_call(fake_gpu):
    cuda.current_context()
    s = cuda.stream()
    seen = []
    for i in range(200):
        s.add_callback(lambda stream, status, arg: seen.append(arg), i)
    assert seen == list(range(200))
    assert not drv._pending_thunks                  # every callback has run ...
    assert 0 < len(drv._finished_thunks) <= 65      # ... and its thunk was parked, not dropped, while running


def test_launch_threads_switch_needs_a_library_that_has_them(monkeypatch):
    """kernels/reduction.py launch_threads on a library without nbh_launch_threads (an older
    build, a test double): says so instead of pretending."""
    from numba_cuda_amd.kernels import reduction
    from numba_cuda_amd.cudadrv import devices, driver as drv

    class Bare:
        pass

    monkeypatch.setattr(devices, "get_context", lambda *a: None)
    monkeypatch.setattr(drv.driver, "lib", Bare(), raising=False)
    with pytest.raises(NotImplementedError):
        reduction.launch_threads(True)


def test_launch_threads_flag_is_read_from_the_environment(monkeypatch):
    from numba_cuda_amd.core import config
    assert config.CUDA_REDUCE_LAUNCH_THREADS == 1          # on unless switched off
    monkeypatch.setenv("NUMBA_CUDA_REDUCE_LAUNCH_THREADS", "0")
    config.reload_config()
    try:
        assert config.CUDA_REDUCE_LAUNCH_THREADS == 0
    finally:
        monkeypatch.delenv("NUMBA_CUDA_REDUCE_LAUNCH_THREADS")
        config.reload_config()
    assert config.CUDA_REDUCE_LAUNCH_THREADS == 1


def test_reading_the_handle_hands_the_stream_out_of_the_package(fake_gpu):
    """`handle`, int() and __cuda_stream__ are how a stream leaves the package: the library is told
    once (nbh_stream_pin_direct), so that nothing stays queued for a stream foreign code may use.
    External streams are told at creation; the default streams never are; `_h` tells nobody."""
    pinned = []
    fake_gpu.nbh_stream_pin_direct = lambda s: pinned.append(s) or 0
    s = cuda.stream()
    assert s._h and not s._exported and pinned == []
    assert drv._stream_handle(s) == s._h and pinned == []          # the package's own way to the handle
    assert s.handle == s._h and pinned == [s._h]
    assert int(s) == s._h and s.__cuda_stream__() == (0, s._h) and pinned == [s._h]   # told once
    t = cuda.stream()
    assert int(t) == t._h and pinned[-1] == t._h
    u = cuda.stream()
    d = cuda.device_array(4, np.float32, stream=u)
    assert d.__cuda_array_interface__["stream"] == u._h and pinned[-1] == u._h
    ext = cuda.external_stream(0x7700)
    assert pinned[-1] == 0x7700 and ext.external
    before = list(pinned)
    assert cuda.default_stream().handle == 0 and cuda.per_thread_default_stream().handle == 2
    assert pinned == before
