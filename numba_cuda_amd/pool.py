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


class PoolMemoryManager(_drv.GetIpcHandleMixin, _drv.HostOnlyCUDAMemoryManager):
    """Device allocations from the library's caching pool; host allocations as in the
    default manager."""

    def initialize(self):
        if self.deallocations.memory_capacity == _drv._SizeNotSet:
            self.deallocations.memory_capacity = self.get_memory_info().total

    def memalloc(self, size):
        def allocator():
            p = c_void_p()
            _drv.driver.nbh_pool_malloc(byref(p), size)
            return p.value or 0

        ptr = self._attempt_allocation(allocator)
        allocations = self.allocations

        def finalizer():
            # straight back to the pool: releasing a block neither frees memory nor
            # waits for the device, so there is nothing to defer
            if allocations:
                allocations.pop(ptr, None)
            _drv.driver.nbh_pool_free(ptr)

        mem = _drv.AutoFreePointer(weakref.proxy(self.context), ptr, size, finalizer=finalizer)
        self.allocations[ptr] = mem
        return mem.own()

    def get_memory_info(self):
        """(free, total) as the driver sees them; blocks idling in the pool count as
        used (see `stats()`)."""
        free, total = c_size_t(), c_size_t()
        _drv.driver.nbh_mem_info(byref(free), byref(total))
        return _drv.MemoryInfo(free=free.value, total=total.value)

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

    @property
    def interface_version(self):
        return 1


# the hook NUMBA_CUDA_MEMORY_MANAGER=<module> looks for (reference :2751-2764)
_numba_memory_manager = PoolMemoryManager
