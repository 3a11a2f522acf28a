"""A stand-in for libnbhip.so that keeps "device" memory in host RAM.

Test double only: lets the device-array plumbing (views, copies, reference
counting, deferred deallocation) run on a machine without a GPU.  It implements
the memory / stream / event entry points and none of the compute kernels, so any
attempt to compute through it fails loudly.
"""

import ctypes

HIP_ERROR_OUT_OF_MEMORY = 2
HIP_ERROR_INVALID_VALUE = 1


def _addr(p):
    if p is None:
        return 0
    if hasattr(p, "value"):
        return p.value or 0
    return int(p)


class FakeLib:
    def __init__(self, total_memory=1 << 30):
        self.buffers = {}        # address -> ctypes buffer
        self.host_buffers = {}
        self.freed = []
        self.total_memory = total_memory
        self.calls = []
        self.fail_next_malloc = 0
        self._next_handle = 0x1000
        self.live_streams = set()
        self.live_events = set()
        self.sync_count = 0

    # -- helpers
    def _log(self, name, *args):
        self.calls.append((name,) + args)

    def _out(self, ptr_arg, value):
        # ptr_arg comes from ctypes.byref(c_xxx)
        ptr_arg._obj.value = value

    # -- library / device
    def nbh_version(self):
        return 1

    def nbh_hip_versions(self, driver_version, runtime_version):
        self._out(driver_version, 70226015)      # 7.2.26015
        self._out(runtime_version, 70226015)
        return 0

    def nbh_error_name(self, code):
        return {2: b"hipErrorOutOfMemory", 1: b"hipErrorInvalidValue", 600: b"hipErrorNotReady"}.get(
            code, b"hipErrorUnknown")

    def nbh_error_string(self, code):
        return self.nbh_error_name(code)

    def nbh_device_count(self, out):
        self._out(out, 1)
        return 0

    def nbh_set_device(self, dev):
        return 0 if dev == 0 else 101

    def nbh_get_device(self, out):
        self._out(out, 0)
        return 0

    def nbh_device_name(self, dev, buf, n):
        buf.value = b"Fake GPU"
        return 0

    def nbh_device_attr(self, dev, name, out):
        table = {b"MAX_THREADS_PER_BLOCK": 1024, b"MULTIPROCESSOR_COUNT": 256, b"WARP_SIZE": 64,
                 b"CAN_MAP_HOST_MEMORY": 1, b"COMPUTE_CAPABILITY_MAJOR": 9, b"COMPUTE_CAPABILITY_MINOR": 5,
                 b"PCI_BUS_ID": 1, b"PCI_DEVICE_ID": 2, b"PCI_DOMAIN_ID": 0}
        if name not in table:
            return HIP_ERROR_INVALID_VALUE
        self._out(out, table[name])
        return 0

    def nbh_mem_info(self, free, total):
        used = sum(len(b) for b in self.buffers.values())
        self._out(free, self.total_memory - used)
        self._out(total, self.total_memory)
        return 0

    def nbh_device_synchronize(self):
        self.sync_count += 1
        return 0

    # -- memory
    def nbh_malloc(self, out, nbytes):
        self._log("malloc", nbytes)
        if self.fail_next_malloc > 0:
            self.fail_next_malloc -= 1
            return HIP_ERROR_OUT_OF_MEMORY
        buf = ctypes.create_string_buffer(max(int(nbytes), 1) + 256)
        addr = (ctypes.addressof(buf) + 255) & ~255        # 256-byte aligned like hipMalloc
        self.buffers[addr] = buf
        self._out(out, addr)
        return 0

    def nbh_malloc_managed(self, out, nbytes, attach_global):
        self._log("malloc_managed", nbytes, attach_global)
        return self.nbh_malloc(out, nbytes)

    # the pool keeps blocks by exact size; nothing is ever pending on the fake
    def nbh_pool_malloc(self, out, nbytes):
        self._log("pool_malloc", nbytes)
        size = max((int(nbytes) + 511) & ~511, 512)
        idle = self.__dict__.setdefault("pool_idle", {})
        self.__dict__.setdefault("pool_hits", 0)
        if idle.get(size):
            addr = idle[size].pop()
            self.pool_hits += 1
            self._out(out, addr)
            return 0
        rc = self.nbh_malloc(out, size)
        if rc == 0:
            self.__dict__.setdefault("pool_sizes", {})[out._obj.value] = size
        return rc

    def nbh_pool_free(self, ptr):
        addr = _addr(ptr)
        self._log("pool_free", addr)
        size = self.__dict__.get("pool_sizes", {}).get(addr)
        if size is None:
            return HIP_ERROR_INVALID_VALUE
        self.__dict__.setdefault("pool_idle", {}).setdefault(size, []).append(addr)
        return 0

    def nbh_pool_trim(self):
        for size, addrs in self.__dict__.get("pool_idle", {}).items():
            for addr in addrs:
                self.buffers.pop(addr, None)
                self.pool_sizes.pop(addr, None)
        self.__dict__["pool_idle"] = {}
        return 0

    def nbh_pool_stats(self, idle, live, hits, misses):
        idle_map = self.__dict__.get("pool_idle", {})
        idle_bytes = sum(size * len(addrs) for size, addrs in idle_map.items())
        total = sum(self.__dict__.get("pool_sizes", {}).values())
        self._out(idle, idle_bytes)
        self._out(live, total - idle_bytes)
        self._out(hits, self.__dict__.get("pool_hits", 0))
        self._out(misses, 0)
        return 0

    def nbh_free(self, ptr):
        addr = _addr(ptr)
        self._log("free", addr)
        if addr not in self.buffers:
            return HIP_ERROR_INVALID_VALUE
        del self.buffers[addr]
        self.freed.append(addr)
        return 0

    def nbh_host_alloc(self, out, nbytes, flags):
        buf = ctypes.create_string_buffer(max(int(nbytes), 1))
        addr = ctypes.addressof(buf)
        self.host_buffers[addr] = buf
        self._out(out, addr)
        self._log("host_alloc", nbytes, flags)
        return 0

    def nbh_host_free(self, ptr):
        self._log("host_free", _addr(ptr))
        self.host_buffers.pop(_addr(ptr), None)
        return 0

    def nbh_host_register(self, ptr, nbytes, flags):
        self._log("host_register", _addr(ptr), nbytes, flags)
        return 0

    def nbh_host_unregister(self, ptr):
        self._log("host_unregister", _addr(ptr))
        return 0

    def nbh_host_get_device_pointer(self, out, hptr):
        self._out(out, _addr(hptr))
        return 0

    def nbh_mem_address_range(self, base, size, ptr):
        a = _addr(ptr)
        for addr, buf in self.buffers.items():
            if addr <= a < addr + len(buf):
                self._out(base, addr)
                self._out(size, len(buf) - (addr - ctypes.addressof(buf)))
                return 0
        for addr, buf in self.host_buffers.items():      # device-mapped host allocations
            if addr <= a < addr + len(buf):
                self._out(base, addr)
                self._out(size, len(buf))
                return 0
        return HIP_ERROR_INVALID_VALUE

    # "other processes" are this process: a handle is the address, spelled in 64 bytes
    def nbh_ipc_get_handle(self, handle, ptr):
        addr = _addr(ptr)
        if addr not in self.buffers:
            return HIP_ERROR_INVALID_VALUE
        raw = addr.to_bytes(8, "little") + b"fakelib!" + bytes(48)
        ctypes.memmove(handle, raw, 64)
        self._log("ipc_get_handle", addr)
        return 0

    def nbh_ipc_open(self, out, handle, nbytes):
        raw = handle if isinstance(handle, bytes) else ctypes.string_at(_addr(handle), 64)
        addr = int.from_bytes(raw[:8], "little")
        if raw[8:16] != b"fakelib!" or addr not in self.buffers:
            return HIP_ERROR_INVALID_VALUE
        self.__dict__.setdefault("ipc_open", []).append(addr)
        self._log("ipc_open", addr, int(nbytes))
        self._out(out, addr)
        return 0

    def nbh_ipc_close(self, ptr):
        addr = _addr(ptr)
        if addr not in self.__dict__.get("ipc_open", []):
            return HIP_ERROR_INVALID_VALUE
        self.ipc_open.remove(addr)
        self._log("ipc_close", addr)
        return 0

    def _copy(self, kind, dst, src, nbytes, stream):
        self._log(kind, _addr(dst), _addr(src), int(nbytes), _addr(stream))
        ctypes.memmove(_addr(dst), _addr(src), int(nbytes))
        return 0

    def nbh_memcpy_h2d(self, dst, src, nbytes, stream):
        return self._copy("h2d", dst, src, nbytes, stream)

    def nbh_memcpy_d2h(self, dst, src, nbytes, stream):
        return self._copy("d2h", dst, src, nbytes, stream)

    def nbh_memcpy_d2d(self, dst, src, nbytes, stream):
        return self._copy("d2d", dst, src, nbytes, stream)

    def nbh_memset8(self, dst, byte, nbytes, stream):
        self._log("memset", _addr(dst), byte, int(nbytes), _addr(stream))
        ctypes.memset(_addr(dst), byte, int(nbytes))
        return 0

    # -- streams / events
    def _handle(self):
        self._next_handle += 0x10
        return self._next_handle

    def nbh_stream_pin_direct(self, s):
        return 0

    def nbh_stream_create(self, out):
        h = self._handle()
        self.live_streams.add(h)
        self._out(out, h)
        return 0

    def nbh_stream_destroy(self, s):
        self.live_streams.discard(_addr(s))
        self._log("stream_destroy", _addr(s))
        return 0

    def nbh_stream_synchronize(self, s):
        self._log("stream_sync", _addr(s))
        return 0

    def nbh_stream_query(self, s):
        return 0

    def nbh_stream_add_callback(self, s, fn, user):
        fn(user)                       # nothing is ever pending on the fake
        return 0

    def nbh_fill(self, dst, ndim, shape, dst_strides, itemsize, value, stream):
        """dst[...] = one item, as a broadcast assignment from the host copy of the item."""
        keep = ctypes.create_string_buffer(ctypes.string_at(_addr(value), int(itemsize)), int(itemsize))
        zeros = (ctypes.c_int64 * max(ndim, 1))(*([0] * max(ndim, 1)))
        self._log("fill", _addr(dst), ndim, _addr(stream))
        rc = self.nbh_assign(dst, ctypes.addressof(keep), ndim, shape, dst_strides, zeros, itemsize, stream)
        self.calls.pop()          # the inner "assign" entry
        self.calls.append(("assign", _addr(dst), 0, ndim, _addr(stream)))
        return rc

    def nbh_assign(self, dst, src, ndim, shape, dst_strides, src_strides, itemsize, stream):
        """Strided broadcast assignment done with NumPy over raw host memory."""
        import numpy as np
        from numpy.lib.stride_tricks import as_strided
        self._log("assign", _addr(dst), _addr(src), ndim, _addr(stream))
        shp = tuple(shape[i] for i in range(ndim))
        ds = tuple(dst_strides[i] for i in range(ndim))
        ss = tuple(src_strides[i] for i in range(ndim))
        if any(n == 0 for n in shp):
            return 0
        item = np.dtype((np.void, int(itemsize)))

        def view(addr, strides):
            lo = sum(min(0, (n - 1) * st) for n, st in zip(shp, strides))
            hi = sum(max(0, (n - 1) * st) for n, st in zip(shp, strides)) + int(itemsize)
            raw = (ctypes.c_ubyte * (hi - lo)).from_address(addr + lo)
            base = np.frombuffer(raw, dtype=np.uint8)
            return as_strided(base[-lo:-lo + int(itemsize)].view(item), shape=shp, strides=strides)

        view(_addr(dst), ds)[...] = view(_addr(src), ss)
        return 0

    def nbh_event_create(self, out, timing):
        h = self._handle()
        self.live_events.add(h)
        self._out(out, h)
        return 0

    def nbh_event_destroy(self, e):
        self.live_events.discard(_addr(e))
        self._log("event_destroy", _addr(e))
        return 0

    def nbh_event_record(self, e, s):
        return 0

    def nbh_event_synchronize(self, e):
        return 0

    def nbh_event_query(self, e):
        return 0

    def nbh_stream_wait_event(self, s, e):
        return 0

    def nbh_event_elapsed_ms(self, out, a, b):
        self._out(out, 1.5)
        return 0

    def nbh_reduce_scratch_bytes(self):
        return 256 + 8 * 4096
