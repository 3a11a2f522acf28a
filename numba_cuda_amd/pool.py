"""A pooling memory manager for device arrays, behind the external-memory-manager
interface (reference: cudadrv/driver.py:592-703; the reference itself ships none and
its documentation points to RMM's pool).

    import numba_cuda_amd as cuda
    from numba_cuda_amd.pool import PoolMemoryManager
    cuda.set_memory_manager(PoolMemoryManager)      # before the first device array

or, without touching the program, ``NUMBA_CUDA_MEMORY_MANAGER=numba_cuda_amd.pool``.

Why: on an MI355X `hipMalloc` + `hipFree` cost 17 us for a kilobyte and 300 us for
64 MiB, and `hipFree` waits for the whole device; transposing those 64 MiB takes 25 us.
Code that allocates per call (`a.T`, `cuda.to_device` in a loop) is allocator-bound
under the default manager.  The pool (csrc/pool.hip) keeps released blocks and hands a
block out again once the work that this package had submitted to any stream before
the release has completed - tracked with events, without host-side waits.

The one rule a pool adds: work that OTHER libraries put on a stream is invisible to it.
An array whose memory such work still uses must be kept alive until that work is done.
"""

import ctypes
import weakref
from ctypes import byref, c_size_t, c_void_p

from numba_cuda_amd.cudadrv import driver as _drv


def _back_to_pool(ptr):
    _drv.driver.nbh_pool_free(ptr)


class PoolMemoryManager(_drv.NumbaCUDAMemoryManager):
    """Device allocations from the library's caching pool; everything else (host
    allocations, memory info, IPC handles) as in the default manager.
    `get_memory_info()` reports what the driver sees: blocks idling in the pool count
    as used (see `stats()`)."""

    def memalloc(self, size):
        def from_pool():
            out = c_void_p()
            _drv.driver.nbh_pool_malloc(byref(out), size)
            return out.value or 0

        address = self._attempt_allocation(from_pool)
        # straight back to the pool, not through the queue of waiting releases: giving a
        # block back neither frees memory nor waits for the device
        on_release = _drv._Release(_back_to_pool, address, table=self.allocations, key=address)
        mem = _drv.AutoFreePointer(weakref.proxy(self.context), address, size, finalizer=on_release)
        return self._track(mem, address)

    def reset(self):
        super().reset()
        _drv.driver.nbh_pool_trim()

    def trim(self):
        """Return every idle block to the driver."""
        _drv.driver.nbh_pool_trim()

    def stats(self):
        """dict(idle_bytes, live_bytes, hits, misses) of the current device's pool."""
        idle, live = c_size_t(), c_size_t()
        hits, misses = ctypes.c_uint64(), ctypes.c_uint64()
        _drv.driver.nbh_pool_stats(byref(idle), byref(live), byref(hits), byref(misses))
        return {"idle_bytes": idle.value, "live_bytes": live.value, "hits": hits.value, "misses": misses.value}


# the hook NUMBA_CUDA_MEMORY_MANAGER=<module> looks for (reference :2751-2764)
_numba_memory_manager = PoolMemoryManager
