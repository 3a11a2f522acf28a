"""The pooling memory manager (numba_cuda_amd/pool.py over csrc/pool.hip): blocks are
reused, results stay right, statistics add up.  Run on the fake library and on the
GPU."""
import gc

import numpy as np

from numba_cuda_amd.cudadrv import driver
from numba_cuda_amd.pool import PoolMemoryManager


def _is_fake():
    return type(driver.driver.lib).__name__ == "FakeLib"


def pooled_arrays_reuse_blocks(cuda):
    ctx = cuda.current_context()
    ctx.reset()
    original = ctx.memory_manager
    ctx.memory_manager = PoolMemoryManager(context=ctx)
    try:
        mgr = cuda.current_context().memory_manager
        before = mgr.stats()
        a = cuda.to_device(np.arange(1000, dtype=np.float64))
        first = a.device_ctypes_pointer.value
        assert mgr.stats()["live_bytes"] - before["live_bytes"] == 8192      # 8000 B -> 512-byte classes
        hits_so_far = mgr.stats()["hits"]         # the pool outlives managers: `a` itself may have been a hit
        del a
        gc.collect()
        cuda.synchronize()
        st = mgr.stats()
        assert st["live_bytes"] == before["live_bytes"] and st["idle_bytes"] >= 8192
        b = cuda.to_device(np.arange(1000, dtype=np.float64) * 2)            # same class: the same block
        assert b.device_ctypes_pointer.value == first
        assert mgr.stats()["hits"] == hits_so_far + 1
        np.testing.assert_array_equal(b.copy_to_host(), np.arange(1000.0) * 2)
        # many short-lived arrays on several streams: values stay right, memory does not grow
        streams = [cuda.stream() for _ in range(3)]
        grown = mgr.stats()["idle_bytes"] + mgr.stats()["live_bytes"]
        for i in range(200):
            s = streams[i % 3]
            h = np.full(5000, i, dtype=np.int32)
            d = cuda.to_device(h, stream=s)
            e = cuda.device_array_like(d, stream=s)
            e.setitem(slice(None), d, stream=s)
            got = e.copy_to_host(stream=s)
            s.synchronize()
            assert (got == i).all()
        del d, e
        gc.collect()
        total = mgr.stats()["idle_bytes"] + mgr.stats()["live_bytes"]
        assert total <= grown + 16 * 20480       # a handful of 20 KiB blocks, not 400
        # big blocks: size classes above 1 MiB waste at most an eighth
        big = cuda.device_array(3 * (1 << 20) + 5, np.uint8)
        assert mgr.stats()["live_bytes"] >= big.nbytes
        del big, b
        gc.collect()
        mgr.trim()
        assert mgr.stats()["idle_bytes"] == 0
        info = ctx.get_memory_info()
        assert 0 < info.free <= info.total
    finally:
        gc.collect()
        ctx.reset()
        ctx.memory_manager = original
        cuda.current_context()


def a_block_in_use_on_another_stream_is_not_handed_out(cuda):
    """A released block that a queued kernel still reads must wait in the pool: release
    a 256 MiB array right after starting a reduction of it on stream A, then allocate and
    overwrite an array of the same size on stream B.  The reduction must see the old
    contents; only after A has finished may the block come back."""
    if _is_fake():
        return
    ctx = cuda.current_context()
    ctx.reset()
    original = ctx.memory_manager
    ctx.memory_manager = PoolMemoryManager(context=ctx)
    try:
        mgr = cuda.current_context().memory_manager
        n = 1 << 26
        sa, sb = cuda.stream(), cuda.stream()
        res = cuda.device_array(1, np.int32)
        add = cuda.Reduce(lambda x, y: x + y)
        ones = np.ones(n, dtype=np.int32)
        for trial in range(5):
            a = cuda.to_device(ones, stream=sa)
            sa.synchronize()
            add(a, res=res, stream=sa)                     # queued on A, reads `a`
            del a                                          # released while that kernel is queued / running
            gc.collect()
            b = cuda.device_array(n, np.int32, stream=sb)  # same size class
            b.gpu_data.memset(0xFF, stream=sb)             # would corrupt the sum if it were the same block early
            sb.synchronize()
            sa.synchronize()
            assert res.copy_to_host()[0] == n, trial
            del b
            gc.collect()
            # both streams are idle now: the next request of this class comes from the pool
            hits = mgr.stats()["hits"]
            c = cuda.device_array(n, np.int32)
            assert mgr.stats()["hits"] == hits + 1
            del c
            gc.collect()
        assert mgr.stats()["hits"] >= 4
    finally:
        gc.collect()
        ctx.reset()
        ctx.memory_manager = original
        cuda.current_context()


def pool_via_the_environment_hook(cuda):
    from numba_cuda_amd import pool
    assert pool._numba_memory_manager is PoolMemoryManager
    assert PoolMemoryManager(context=None).interface_version == 1


ALL = [pooled_arrays_reuse_blocks, a_block_in_use_on_another_stream_is_not_handed_out, pool_via_the_environment_hook]
