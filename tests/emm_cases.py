"""External memory-manager plugins as the reference's suite pins them
(numba_cuda/numba/cuda/tests/cudadrv/test_emm_plugins.py), restated with the lines
each case follows.  Run on the fake library and on the GPU (the plugin hands out fake
addresses, so nothing touches them)."""
import ctypes
import gc
import weakref

import numpy as np
import pytest


def _plugin_class(cuda):
    # :13-73
    class DeviceOnlyPlugin(cuda.HostOnlyCUDAMemoryManager):
        def __init__(self, *args, **kwargs):
            super().__init__(*args, **kwargs)
            self.allocations = {}
            self.count = 0
            self.initialized = self.memalloc_called = self.reset_called = False
            self.get_memory_info_called = self.get_ipc_handle_called = False

        def memalloc(self, size):
            if not self.initialized:
                raise RuntimeError("memalloc called before initialize")
            self.memalloc_called = True
            self.count += 1
            number = self.count
            self.allocations[number] = size
            book = self.allocations

            def finalizer():
                del book[number]

            return cuda.cudadrv.driver.AutoFreePointer(weakref.proxy(self.context), ctypes.c_void_p(number), size,
                                                       finalizer=finalizer)

        def initialize(self):
            self.initialized = True

        def reset(self):
            self.reset_called = True

        def get_memory_info(self):
            self.get_memory_info_called = True
            return cuda.MemoryInfo(free=32, total=64)

        def get_ipc_handle(self, memory):
            self.get_ipc_handle_called = True
            return "Dummy IPC handle for alloc %s" % memory.device_pointer_value

        @property
        def interface_version(self):
            return 1

    return DeviceOnlyPlugin


def plugin_is_called_as_documented(cuda):
    # :86-150
    ctx = cuda.current_context()
    ctx.reset()
    original = ctx.memory_manager
    ctx.memory_manager = _plugin_class(cuda)(context=ctx)
    try:
        mgr = cuda.current_context().memory_manager
        assert mgr.initialized
        a1 = np.arange(10)
        d1 = cuda.device_array_like(a1)
        assert mgr.memalloc_called and mgr.count == 1 and mgr.allocations[1] == a1.nbytes
        a2 = np.arange(5)
        d2 = cuda.device_array_like(a2)
        assert mgr.count == 2 and mgr.allocations[2] == a2.nbytes
        del d1
        gc.collect()
        assert 1 not in mgr.allocations and 2 in mgr.allocations
        handle = d2.get_ipc_handle()
        assert mgr.get_ipc_handle_called and "Dummy IPC handle for alloc 2" in handle._ipc_handle
        del d2
        gc.collect()
        assert 2 not in mgr.allocations
        info = ctx.get_memory_info()
        assert mgr.get_memory_info_called and (info.free, info.total) == (32, 64)
        ctx.reset()
        assert mgr.reset_called
    finally:
        ctx.reset()
        ctx.memory_manager = original
        cuda.current_context()


def wrong_interface_version_is_refused(cuda):
    # :153-168
    class BadVersion(_plugin_class(cuda)):
        @property
        def interface_version(self):
            return 2

    with pytest.raises(RuntimeError, match="version 1 required"):
        cuda.set_memory_manager(BadVersion)


ALL = [plugin_is_called_as_documented, wrong_interface_version_is_refused]
