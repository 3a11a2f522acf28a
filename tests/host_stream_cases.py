"""Host allocations, pinned copies, stream callbacks and events as the reference's
suite pins them (numba_cuda/numba/cuda/tests/cudadrv/test_host_alloc.py,
test_pinned.py, test_streams.py, test_events.py), restated with the lines each case
follows.  Run on the fake library and on the GPU."""
import asyncio
import threading

import numpy as np

from numba_cuda_amd.cudadrv import driver


def _is_fake():
    return type(driver.driver.lib).__name__ == "FakeLib"


def mapped_allocation_as_a_numpy_buffer(cuda):
    # test_host_alloc.py:14-28: the memory object itself is the buffer
    n = 32
    mem = cuda.current_context().memhostalloc(n, mapped=True)
    ary = np.ndarray(shape=n, dtype=np.uint8, buffer=mem)
    driver.device_memset(mem, 0xAB, n)
    cuda.synchronize()
    assert np.all(ary == 0xAB)
    ary.fill(n)
    recv = np.empty_like(ary)
    driver.device_to_host(recv, mem, ary.size)
    assert np.all(ary == recv) and np.all(recv == n)
    del mem                                  # the array keeps the allocation alive
    ary.fill(7)
    assert np.all(ary == 7)


def pinned_and_mapped_arrays(cuda):
    # test_host_alloc.py:30-64
    ary = cuda.pinned_array(10, dtype=np.uint32)
    ary.fill(123)
    assert all(ary == 123)
    dev = cuda.to_device(ary)
    driver.device_memset(dev, 0, driver.device_memory_size(dev))
    assert all(ary == 123)
    dev.copy_to_host(ary)
    assert all(ary == 0)
    ary = cuda.mapped_array(10, dtype=np.uint32)
    ary.fill(123)
    assert all(ary == 123)
    driver.device_memset(ary, 0, driver.device_memory_size(ary))
    cuda.synchronize()
    assert all(ary == 0) and sum(ary != 0) == 0
    for ary in (cuda.mapped_array(10, dtype=np.uint32), cuda.pinned_array(10, dtype=np.uint32)):
        ary[:] = range(10)
        assert sum(ary + 1) == 55 and sum((ary + 1) * 2 - 1) == 100
        assert sum(ary < 5) == 5 and sum(ary <= 5) == 6 and sum(ary > 6) == 3 and sum(ary >= 6) == 4
        assert sum(ary ** 2) == 285 and sum(ary // 2) == 20 and sum(ary / 2.0) == 22.5 and sum(ary % 2) == 5


def copies_on_a_stream(cuda):
    # test_pinned.py:11-37 (cuda.pinned() itself only on the fake library: page-locking
    # existing memory is refused on the GPU machines used here)
    def run(a):
        keep = np.copy(a)
        st = cuda.stream()
        d = cuda.to_device(a, copy=False, stream=st)
        d.copy_to_device(a, stream=st)
        d.copy_to_host(a, stream=st)
        st.synchronize()
        assert np.allclose(a, keep)

    run(np.arange(2 * 1024 * 1024))
    if _is_fake():
        a = np.arange(2097152)
        with cuda.pinned(a):
            run(a)
    p = cuda.pinned_array(1 << 20, dtype=np.int64)
    p[:] = np.arange(1 << 20)
    run(p)


def stream_callbacks(cuda):
    # test_streams.py:27-46
    def callback(stream, status, event):
        event.set()

    st = cuda.stream()
    fired = threading.Event()
    st.add_callback(callback, fired)
    assert fired.wait(1.0)
    seen = []
    fired2 = threading.Event()

    def callback2(stream, status, arg):
        seen.append(arg)
        fired2.set()

    st.add_callback(callback2)
    assert fired2.wait(1.0) and seen == [None]


def async_done(cuda):
    # test_streams.py:48-100
    async def one():
        st = cuda.stream()
        await st.async_done()

    async def parallel():
        async def task(value):
            st = cuda.stream()
            h_src, h_dst = cuda.pinned_array(8), cuda.pinned_array(8)
            h_src[:] = value
            d = cuda.to_device(h_src, stream=st)
            d.copy_to_host(h_dst, stream=st)
            assert await st.async_done() == st
            return h_dst.mean()

        values = [1, 2, 3, 4]
        out = await asyncio.gather(*[asyncio.create_task(task(v)) for v in values])
        assert np.allclose(values, out)

    async def many_on_one():
        st = cuda.stream()
        done = await asyncio.gather(*[st.async_done() for _ in range(4)])
        assert all(d == st for d in done)

    async def many_streams():
        streams = [cuda.stream() for _ in range(4)]
        done = await asyncio.gather(*[s.async_done() for s in streams])
        assert set(done) == set(streams)

    async def cancelled():
        st = cuda.stream()
        first, second = st.async_done(), st.async_done()
        first.cancel()
        await second
        assert first.cancelled() and second.done()

    for coro in (one, parallel, many_on_one, many_streams, cancelled):
        loop = asyncio.new_event_loop()
        try:
            loop.run_until_complete(coro())
        finally:
            loop.close()


def events(cuda):
    # test_events.py:12-46
    for st in (None, cuda.stream()):
        kw = {} if st is None else {"stream": st}
        d = cuda.device_array(32, dtype=np.double)
        start, end = cuda.event(), cuda.event()
        start.record(**kw)
        cuda.to_device(np.arange(32, dtype=np.double), to=d, **kw)
        end.record(**kw)
        end.wait(**kw)
        end.synchronize()
        assert start.elapsed_time(end) >= 0.0


ALL = [mapped_allocation_as_a_numpy_buffer, pinned_and_mapped_arrays, copies_on_a_stream, stream_callbacks, async_done,
       events]
