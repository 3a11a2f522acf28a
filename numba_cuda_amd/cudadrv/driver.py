"""HIP driver layer: devices, contexts, memory objects, streams, events, copies.

Python owns every lifetime here, as in the reference
(numba_cuda/numba/cuda/cudadrv/driver.py): device memory is a `MemoryPointer`
whose finalizer does not free but *queues* the free in the context's
`_PendingDeallocs`, so that garbage collection never turns into a device-wide
synchronisation in the middle of asynchronous work.  Underneath there is no
driver binding, only the C entry points of libnbhip.so (include/nbhip.h).

HIP has one implicit primary context per device, so `Context` is a per-device
bookkeeping object (memory manager, pending frees, reduction scratch) rather
than a driver handle.
"""

import contextlib
import ctypes
import functools
import importlib
import logging
import os
import sys
import threading
import weakref
from abc import ABCMeta, abstractmethod
from collections import deque, namedtuple
from ctypes import c_int, c_size_t, c_void_p, byref

import numpy as np

from numba_cuda_amd import _lib

try:
    from numba_cuda_amd import _hostbuf
except ImportError:                      # not built yet: one gcc call, about a second
    from numba_cuda_amd import _build
    _build.build_hostbuf()
    from numba_cuda_amd import _hostbuf
from numba_cuda_amd.core import config
from numba_cuda_amd.core.errors import CudaDriverError, CudaSupportError  # noqa: F401


def make_logger():
    logger = logging.getLogger(__name__)
    lvl = str(config.CUDA_LOG_LEVEL).upper()
    lvl = getattr(logging, lvl, None)
    if not isinstance(lvl, int):
        logger.addHandler(logging.NullHandler())
    else:
        logger.setLevel(lvl)
        if not logger.handlers:
            handler = logging.StreamHandler(sys.stderr)
            handler.setFormatter(logging.Formatter("== HIP [%(relativeCreated)d] %(levelname)5s -- %(message)s"))
            logger.addHandler(handler)
    return logger


_logger = make_logger()


class CudaAPIError(CudaDriverError):
    """A libnbhip / HIP call returned a non-zero hipError_t (reference:
    driver.py:147-154; same name so that user except-clauses keep working)."""

    def __init__(self, code, msg):
        self.code = code
        self.msg = msg
        super().__init__(code, msg)

    def __str__(self):
        return "[%s] %s" % (self.code, self.msg)


HipAPIError = CudaAPIError


class Driver:
    """Checked access to libnbhip.so.  `driver.nbh_xxx(*args)` calls the entry
    point and raises CudaAPIError on a non-zero status (reference: Driver
    :245-419).  The library is loaded on first use; a load failure is kept in
    `initialization_error` and re-raised on every later use."""

    _singleton = None

    def __new__(cls):
        if cls._singleton is None:
            obj = object.__new__(cls)
            obj.lib = None
            obj.is_initialized = False
            obj.initialization_error = None
            obj.pid = None
            obj._lock = threading.Lock()
            cls._singleton = obj
        return cls._singleton

    def ensure_initialized(self):
        if self.is_initialized:
            if self.initialization_error is not None:
                raise CudaSupportError("Error at driver init: %s" % self.initialization_error)
            return
        with self._lock:
            if self.is_initialized:
                return
            self.is_initialized = True
            if config.DISABLE_CUDA:
                self.initialization_error = "GPU support disabled by NUMBA_DISABLE_CUDA=1"
            elif config.ENABLE_CUDASIM:
                self.initialization_error = ("NUMBA_ENABLE_CUDASIM=1 asks for the CPU simulator, "
                                             "which this GPU-only package does not provide")
            else:
                try:
                    self.lib = _lib.load()
                    self.pid = os.getpid()
                except OSError as e:
                    self.initialization_error = str(e)
        if self.initialization_error is not None:
            raise CudaSupportError("Error at driver init: %s" % self.initialization_error)

    @property
    def is_available(self):
        try:
            self.ensure_initialized()
        except CudaSupportError:
            return False
        return self.get_device_count() > 0

    def _error_name(self, code):
        name = self.lib.nbh_error_name(code)
        return name.decode() if name else "hipError_%d" % code

    def check(self, fname, code):
        if code != _lib.HIP_SUCCESS:
            if self.pid is not None and os.getpid() != self.pid:
                raise CudaDriverError("HIP initialized before forking")
            raise CudaAPIError(code, "Call to %s results in %s" % (fname, self._error_name(code)))

    def __getattr__(self, fname):
        if not fname.startswith("nbh_"):
            raise AttributeError(fname)
        self.ensure_initialized()
        cfn = getattr(self.lib, fname)

        def checked(*args):
            if config.CUDA_LOG_API_ARGS:
                _logger.debug("call driver api: %s%r", fname, args)
            else:
                _logger.debug("call driver api: %s", fname)
            self.check(fname, cfn(*args))

        setattr(self, fname, checked)
        return checked

    # --- devices
    def get_device_count(self):
        n = c_int(0)
        self.nbh_device_count(byref(n))
        return n.value

    @functools.lru_cache(maxsize=None)
    def get_device(self, devnum=0):
        if not 0 <= devnum < self.get_device_count():
            raise CudaAPIError(101, "Call to hipSetDevice results in hipErrorInvalidDevice")
        return Device(devnum)

    def list_devices(self):
        return [self.get_device(i) for i in range(self.get_device_count())]

    def get_version(self):
        return (self.lib.nbh_version(), 0)


driver = Driver()


class Device:
    """One GPU (reference: Device :470-587).  Attributes are looked up lazily by
    their CUDA names, e.g. MAX_THREADS_PER_BLOCK, MULTIPROCESSOR_COUNT, WARP_SIZE."""

    def __init__(self, devnum):
        self.id = devnum
        buf = ctypes.create_string_buffer(256)
        driver.nbh_device_name(devnum, buf, 256)
        self.name = buf.value.decode()
        self.primary_context = None
        self._ctx_lock = threading.Lock()

    def __getattr__(self, attr):
        if attr.startswith("_") or not attr.isupper():
            raise AttributeError(attr)
        value = c_int(0)
        try:
            driver.nbh_device_attr(self.id, attr.encode(), byref(value))
        except CudaAPIError:
            raise AttributeError("unknown device attribute %s" % attr) from None
        setattr(self, attr, value.value)
        return value.value

    @property
    def compute_capability(self):
        return (self.COMPUTE_CAPABILITY_MAJOR, self.COMPUTE_CAPABILITY_MINOR)

    def get_device_identity(self):
        return {"pci_domain_id": self.PCI_DOMAIN_ID, "pci_bus_id": self.PCI_BUS_ID,
                "pci_device_id": self.PCI_DEVICE_ID}

    @classmethod
    def from_identity(cls, identity):
        """The device with this PCI identity (reference :489-503)."""
        for dev in driver.list_devices():
            if dev.get_device_identity() == identity:
                return dev
        raise RuntimeError("No device of {} is found. Target device may not be visible in this process."
                           .format(identity))

    def get_primary_context(self):
        with self._ctx_lock:
            if self.primary_context is None:
                self.primary_context = Context(self)
            return self.primary_context

    def reset(self):
        if self.primary_context is not None:
            self.primary_context.reset()

    def __repr__(self):
        return "<HIP device %d '%s'>" % (self.id, self.name)

    def __hash__(self):
        return hash(self.id)

    def __eq__(self, other):
        return isinstance(other, Device) and self.id == other.id


# --------------------------------------------------------------------------------
# Pending deallocations
# --------------------------------------------------------------------------------

class _SizeNotSet(int):
    """Stand-in size of a resource whose footprint is unknown (counts as 0)."""

    def __new__(cls, *args, **kwargs):
        return super().__new__(cls, 0)

    def __str__(self):
        return "?"


_SizeNotSet = _SizeNotSet()


class _PendingDeallocs:
    """Queue of (destructor, handle, size) to run later (reference :975-1045).

    Flushed when more than CUDA_DEALLOCS_COUNT entries or more than
    CUDA_DEALLOCS_RATIO * capacity bytes are waiting, on out-of-memory, and on
    reset.  `disable()` is a nestable context manager that holds flushing off.
    """

    def __init__(self, capacity=_SizeNotSet):
        self._cons = deque()
        self._disable_count = 0
        self._size = 0
        self.memory_capacity = capacity

    @property
    def _max_pending_bytes(self):
        return int(self.memory_capacity * config.CUDA_DEALLOCS_RATIO)

    def add_item(self, dtor, handle, size=_SizeNotSet):
        _logger.info("add pending dealloc: %s %s bytes", getattr(dtor, "__name__", dtor), size)
        self._cons.append((dtor, handle, size))
        self._size += int(size)
        if len(self._cons) > config.CUDA_DEALLOCS_COUNT or self._size > self._max_pending_bytes:
            self.clear()

    def clear(self):
        if self.is_disabled:
            return
        while self._cons:
            dtor, handle, size = self._cons.popleft()
            _logger.info("dealloc: %s %s bytes", getattr(dtor, "__name__", dtor), size)
            dtor(handle)
        self._size = 0

    @contextlib.contextmanager
    def disable(self):
        self._disable_count += 1
        try:
            yield
        finally:
            self._disable_count -= 1
            assert self._disable_count >= 0

    @property
    def is_disabled(self):
        return self._disable_count > 0

    def __len__(self):
        return len(self._cons)


MemoryInfo = namedtuple("MemoryInfo", "free,total")


# --------------------------------------------------------------------------------
# Memory managers (the EMM plugin interface of the reference, :589-957)
# --------------------------------------------------------------------------------

class BaseCUDAMemoryManager(metaclass=ABCMeta):
    def __init__(self, *args, **kwargs):
        if "context" not in kwargs:
            raise RuntimeError("Memory manager requires a context")
        self.context = kwargs.pop("context")

    @abstractmethod
    def memalloc(self, size):
        """Allocate `size` bytes of device memory; returns a MemoryPointer."""

    @abstractmethod
    def memhostalloc(self, size, mapped, portable, wc):
        """Allocate page-locked host memory."""

    @abstractmethod
    def mempin(self, owner, pointer, size, mapped):
        """Page-lock host memory that already exists."""

    @abstractmethod
    def initialize(self):
        """Make the manager ready for use (may be called many times)."""

    @abstractmethod
    def get_ipc_handle(self, memory):
        """IPC handle of an allocation."""

    @abstractmethod
    def get_memory_info(self):
        """(free, total) bytes."""

    @abstractmethod
    def reset(self):
        """Drop everything allocated in this context."""

    @abstractmethod
    def defer_cleanup(self):
        """Context manager during which no deallocation happens."""

    @property
    @abstractmethod
    def interface_version(self):
        """Version of this interface the plugin implements (1)."""


class HostOnlyCUDAMemoryManager(BaseCUDAMemoryManager):
    """Host-side allocations plus the bookkeeping every manager needs; plugins
    that only care about device memory derive from this (reference :705-872)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.allocations = {}
        self.deallocations = _PendingDeallocs()

    def _attempt_allocation(self, allocator):
        """Run `allocator`; on out-of-memory flush pending frees and retry once."""
        try:
            return allocator()
        except CudaAPIError as e:
            if e.code != _lib.HIP_ERROR_OUT_OF_MEMORY:
                raise
            self.deallocations.clear()
            return allocator()

    def memhostalloc(self, size, mapped=False, portable=False, wc=False):
        flags = (1 if portable else 0) | (2 if mapped else 0) | (4 if wc else 0)

        def allocator():
            p = c_void_p()
            driver.nbh_host_alloc(byref(p), size, flags)
            return p.value or 0

        pointer = self._attempt_allocation(allocator) if mapped else allocator()
        finalizer = _hostalloc_finalizer(self, pointer, pointer, size, mapped)
        ctx = weakref.proxy(self.context)
        if mapped:
            mem = MappedMemory(ctx, pointer, size, finalizer=finalizer)
            self.allocations[pointer] = mem
            return mem.own()
        return PinnedMemory(ctx, pointer, size, finalizer=finalizer)

    def mempin(self, owner, pointer, size, mapped=False):
        flags = 2 if mapped else 0

        def allocator():
            driver.nbh_host_register(pointer, size, flags)

        if mapped:
            self._attempt_allocation(allocator)
        else:
            allocator()
        finalizer = _pin_finalizer(self, pointer, pointer, mapped)
        ctx = weakref.proxy(self.context)
        if mapped:
            mem = MappedMemory(ctx, pointer, size, owner=owner, finalizer=finalizer)
            self.allocations[pointer] = mem
            return mem.own()
        return PinnedMemory(ctx, pointer, size, owner=owner, finalizer=finalizer)

    def memallocmanaged(self, size, attach_global):
        def allocator():
            p = c_void_p()
            driver.nbh_malloc_managed(byref(p), size, 1 if attach_global else 0)
            return p.value or 0

        ptr = self._attempt_allocation(allocator)
        finalizer = _alloc_finalizer(self, ptr, ptr, size)
        mem = ManagedMemory(weakref.proxy(self.context), ptr, size, finalizer=finalizer)
        self.allocations[ptr] = mem
        return mem.own()

    def reset(self):
        self.allocations.clear()
        self.deallocations.clear()

    @contextlib.contextmanager
    def defer_cleanup(self):
        with self.deallocations.disable():
            yield


class GetIpcHandleMixin:
    """A default get_ipc_handle() for managers whose memory comes from hipMalloc
    (reference :861-878): the handle names the whole allocation, `offset` says where
    in it `memory` starts."""

    def get_ipc_handle(self, memory):
        base, end = device_extents(memory)
        if end - base >= IPC_ALLOCATION_LIMIT:
            raise ValueError("allocations of 2 GiB or more cannot be shared between processes "
                             "(this one has %d bytes)" % (end - base))
        raw = ctypes.create_string_buffer(_lib.IPC_HANDLE_BYTES)
        driver.nbh_ipc_get_handle(raw, base)
        offset = int(memory.handle) - base
        source_info = self.context.device.get_device_identity()
        return IpcHandle(memory, IpcMemHandle(raw.raw), memory.size, source_info, offset=offset)


class NumbaCUDAMemoryManager(GetIpcHandleMixin, HostOnlyCUDAMemoryManager):
    """Default manager: hipMalloc per allocation, deferred hipFree (reference
    :892-921)."""

    def initialize(self):
        if self.deallocations.memory_capacity == _SizeNotSet:
            self.deallocations.memory_capacity = self.get_memory_info().total

    def memalloc(self, size):
        def allocator():
            p = c_void_p()
            driver.nbh_malloc(byref(p), size)
            return p.value or 0

        ptr = self._attempt_allocation(allocator)
        finalizer = _alloc_finalizer(self, ptr, ptr, size)
        mem = AutoFreePointer(weakref.proxy(self.context), ptr, size, finalizer=finalizer)
        self.allocations[ptr] = mem
        return mem.own()

    def get_memory_info(self):
        free, total = c_size_t(), c_size_t()
        driver.nbh_mem_info(byref(free), byref(total))
        return MemoryInfo(free=free.value, total=total.value)

    @property
    def interface_version(self):
        return _SUPPORTED_EMM_INTERFACE_VERSION


_SUPPORTED_EMM_INTERFACE_VERSION = 1
_memory_manager = None


def _ensure_memory_manager():
    global _memory_manager
    if _memory_manager:
        return
    if config.CUDA_MEMORY_MANAGER == "default":
        _memory_manager = NumbaCUDAMemoryManager
        return
    try:
        mgr_module = importlib.import_module(config.CUDA_MEMORY_MANAGER)
        set_memory_manager(mgr_module._numba_memory_manager)
    except Exception:
        raise RuntimeError("Failed to use memory manager from %s" % config.CUDA_MEMORY_MANAGER)


def set_memory_manager(mm_plugin):
    """Use an External Memory Management plugin class for all later contexts."""
    global _memory_manager
    iv = mm_plugin(context=None).interface_version
    if iv != _SUPPORTED_EMM_INTERFACE_VERSION:
        raise RuntimeError("EMM Plugin interface has version %d - version %d required"
                           % (iv, _SUPPORTED_EMM_INTERFACE_VERSION))
    _memory_manager = mm_plugin


# --------------------------------------------------------------------------------
# Context
# --------------------------------------------------------------------------------

class Context:
    """Per-device state (reference: Context :1061-1301)."""

    def __init__(self, device):
        self.device = device
        self.handle = device.id
        self.deallocations = _PendingDeallocs()
        _ensure_memory_manager()
        self.memory_manager = _memory_manager(context=self)
        self.extras = {}
        self._scratch = {}   # stream handle -> device scratch for nbh_reduce
        self._result_slots = {}   # stream handle -> host-mapped slot for results that go back to the caller

    @property
    def memory_manager(self):
        return self._memory_manager

    @memory_manager.setter
    def memory_manager(self, manager):
        # a manager put in by hand is initialised the next time the context is fetched
        self._memory_manager = manager
        self.prepared = False

    def reset(self):
        _logger.info("reset context of device %s", self.device.id)
        self._scratch.clear()
        self._free_result_slots()
        self.memory_manager.reset()
        self.deallocations.clear()

    def prepare_for_use(self):
        self.memory_manager.initialize()
        self.prepared = True

    def get_ipc_handle(self, memory):
        """An IpcHandle for `memory`, to be sent to another process (reference :1190-1198)."""
        if not sys.platform.startswith("linux"):
            raise OSError("OS does not support CUDA IPC")
        return self.memory_manager.get_ipc_handle(memory)

    def open_ipc_handle(self, handle, size):
        """Map the allocation `handle` names into this process; `size` bytes of it
        will be used (reference :1200-1209).  IpcHandle.close() unmaps it."""
        dptr = c_void_p()
        driver.nbh_ipc_open(byref(dptr), bytes(handle.reserved), size)
        return MemoryPointer(context=weakref.proxy(self), pointer=dptr, size=size)

    def can_access_peer(self, peer_device):
        """One device per process here: only the device itself is reachable."""
        return int(peer_device) == self.device.id

    def get_memory_info(self):
        return self.memory_manager.get_memory_info()

    def memalloc(self, bytesize):
        return self.memory_manager.memalloc(bytesize)

    def memhostalloc(self, bytesize, mapped=False, portable=False, wc=False):
        return self.memory_manager.memhostalloc(bytesize, mapped, portable, wc)

    def memallocmanaged(self, bytesize, attach_global=True):
        return self.memory_manager.memallocmanaged(bytesize, attach_global)

    def mempin(self, owner, pointer, size, mapped=False):
        if mapped and not self.device.CAN_MAP_HOST_MEMORY:
            raise CudaDriverError("%s cannot map host memory" % self.device)
        return self.memory_manager.mempin(owner, pointer, size, mapped)

    def get_default_stream(self):
        return Stream(0)

    def get_legacy_default_stream(self):
        return Stream(0)

    def get_per_thread_default_stream(self):
        return Stream(HIP_STREAM_PER_THREAD)

    def create_stream(self):
        h = c_void_p()
        driver.nbh_stream_create(byref(h))
        handle = h.value or 0
        return Stream(handle, finalizer=_stream_finalizer(self.deallocations, handle))

    def create_external_stream(self, ptr):
        if not isinstance(ptr, int):
            raise TypeError("ptr for external stream must be an int")
        return Stream(ptr, external=True)

    def create_event(self, timing=True):
        h = c_void_p()
        driver.nbh_event_create(byref(h), 1 if timing else 0)
        handle = h.value or 0
        return Event(handle, finalizer=_event_finalizer(self.deallocations, handle))

    def synchronize(self):
        driver.nbh_device_synchronize()

    @contextlib.contextmanager
    def defer_cleanup(self):
        with self.memory_manager.defer_cleanup():
            with self.deallocations.disable():
                yield

    _RESULT_SLOT_BYTES = 256

    def reduce_scratch(self, stream_handle):
        """(scratch address, result slot address, scratch size) for nbh_reduce on
        the given stream, made and zeroed on first use.  Work on one stream is
        ordered, so consecutive reductions on it can share both; different streams
        get their own.  The slot sits behind the scratch area in the same
        allocation."""
        entry = self._scratch.get(stream_handle)
        if entry is None:
            nbytes = driver.lib.nbh_reduce_scratch_bytes()
            mem = self.memalloc(nbytes + self._RESULT_SLOT_BYTES)
            ptr = mem.device_ctypes_pointer.value
            driver.nbh_memset8(ptr, 0, nbytes + self._RESULT_SLOT_BYTES, None)
            entry = self._scratch[stream_handle] = (ptr, ptr + nbytes, nbytes, mem)
        return entry[0], entry[1], entry[2]

    def reduce_result_slot(self, stream_handle, dtype):
        """(device-visible address, one-item host array) of a result slot in page-locked,
        device-mapped host memory: a reduction that returns its value to the caller
        writes it there, and the host reads it after waiting for the stream - no
        device-to-host copy (which costs as much again as the launch).  One slot per
        stream, viewed through the dtype asked for."""
        entry = self._result_slots.get(stream_handle)
        if entry is None:
            host = c_void_p()
            driver.nbh_host_alloc(byref(host), self._RESULT_SLOT_BYTES, 2)       # 2: device-mapped
            dev = c_void_p()
            driver.nbh_host_get_device_pointer(byref(dev), host.value)
            raw = np.frombuffer((ctypes.c_ubyte * self._RESULT_SLOT_BYTES).from_address(host.value), dtype=np.uint8)
            entry = self._result_slots[stream_handle] = (dev.value, host.value, raw, {})
        view = entry[3].get(dtype)
        if view is None:
            view = entry[3][dtype] = entry[2][:dtype.itemsize].view(dtype)
        return entry[0], view

    def _free_result_slots(self):
        slots, self._result_slots = self._result_slots, {}
        for _, host, _, _ in slots.values():
            try:
                driver.nbh_host_free(host)
            except Exception:
                pass

    def __repr__(self):
        return "<HIP context of device %d>" % self.device.id

    def __eq__(self, other):
        return isinstance(other, Context) and self.handle == other.handle

    def __hash__(self):
        return hash(("ctx", self.handle))


HIP_STREAM_PER_THREAD = 2


def _alloc_finalizer(memory_manager, ptr, alloc_key, size):
    allocations = memory_manager.allocations
    deallocations = memory_manager.deallocations

    def core():
        if allocations:
            allocations.pop(alloc_key, None)
        deallocations.add_item(_free_device, ptr, size)

    return core


def _hostalloc_finalizer(memory_manager, ptr, alloc_key, size, mapped):
    allocations = memory_manager.allocations
    deallocations = memory_manager.deallocations
    if not mapped:
        size = _SizeNotSet

    def core():
        if mapped and allocations:
            allocations.pop(alloc_key, None)
        deallocations.add_item(_free_host, ptr, size)

    return core


def _pin_finalizer(memory_manager, ptr, alloc_key, mapped):
    # unregistering cannot wait: the same host buffer may be pinned again at once
    allocations = memory_manager.allocations

    def core():
        if mapped and allocations:
            allocations.pop(alloc_key, None)
        driver.nbh_host_unregister(ptr)

    return core


def _free_device(ptr):
    driver.nbh_free(ptr)


def _free_host(ptr):
    driver.nbh_host_free(ptr)


def _destroy_stream(handle):
    driver.nbh_stream_destroy(handle)


def _destroy_event(handle):
    driver.nbh_event_destroy(handle)


def _event_finalizer(deallocs, handle):
    def core():
        deallocs.add_item(_destroy_event, handle)

    return core


def _stream_finalizer(deallocs, handle):
    def core():
        deallocs.add_item(_destroy_stream, handle)

    return core


# --------------------------------------------------------------------------------
# Memory objects
# --------------------------------------------------------------------------------

IPC_ALLOCATION_LIMIT = 2 << 30   # opening larger allocations has been seen to hang


class IpcMemHandle:
    """The 64 opaque bytes of a hipIpcMemHandle_t; `reserved` is what travels."""

    def __init__(self, reserved=bytes(_lib.IPC_HANDLE_BYTES)):
        self.reserved = reserved

    @property
    def reserved(self):
        return self._reserved

    @reserved.setter
    def reserved(self, value):
        value = bytes(bytearray(value))          # bytes, or any sequence of small ints
        if len(value) != _lib.IPC_HANDLE_BYTES:
            raise ValueError("an IPC memory handle has %d bytes, got %d" % (_lib.IPC_HANDLE_BYTES, len(value)))
        self._reserved = value


class _DirectIpc:
    """An imported mapping of the exporter's allocation."""

    def __init__(self, parent):
        self.parent = parent
        self._opened = None

    def open(self, context):
        p = self.parent
        if p.base is not None:
            raise ValueError("opening IpcHandle from original process")
        if self._opened is not None:
            raise ValueError("IpcHandle is already opened")
        if p.offset + p.size >= IPC_ALLOCATION_LIMIT:
            raise ValueError("allocations of 2 GiB or more cannot be shared between processes")
        mem = context.open_ipc_handle(p.handle, p.offset + p.size)
        self._opened = mem            # this object owns the mapping until close()
        return mem.own().view(p.offset)

    def close(self):
        if self._opened is None:
            raise ValueError("IpcHandle not opened")
        driver.nbh_ipc_close(self._opened.handle)
        self._opened = None


class IpcHandle:
    """A picklable name for a device allocation that another process on the same
    machine can open (reference :1487-1603).

    base        the exporter's memory, kept alive by the handle (None once pickled)
    handle      IpcMemHandle
    size        bytes of the shared region
    source_info identity of the exporting device
    offset      where the region starts in the underlying allocation
    """

    def __init__(self, base, handle, size, source_info=None, offset=0):
        self.base = base
        self.handle = handle
        self.size = size
        self.source_info = source_info
        self.offset = offset
        self._impl = None

    def _sentry_source_info(self):
        if self.source_info is None:
            raise RuntimeError("IPC handle doesn't have source info")

    def can_access_peer(self, context):
        self._sentry_source_info()
        if self.source_info == context.device.get_device_identity():
            return True
        return context.can_access_peer(Device.from_identity(self.source_info).id)

    def open_staged(self, context):
        """Copy through the exporting device when the importer cannot reach it.  That
        needs a second device in the importing process, which this build never has."""
        self._sentry_source_info()
        if self._impl is not None:
            raise ValueError("IpcHandle is already opened")
        raise NotImplementedError("staged IPC between two devices is not part of this build")

    def open_direct(self, context):
        if self._impl is not None:
            raise ValueError("IpcHandle is already opened")
        self._impl = _DirectIpc(self)
        try:
            return self._impl.open(context)
        except Exception:
            self._impl = None
            raise

    def open(self, context):
        """Map the memory into `context`'s process -> device memory pointer."""
        if self.source_info is None or self.can_access_peer(context):
            return self.open_direct(context)
        return self.open_staged(context)

    def open_array(self, context, shape, dtype, strides=None):
        """open(), wrapped as a device array (1-d C-contiguous unless `strides` says otherwise)."""
        from numba_cuda_amd.cudadrv import devicearray
        if strides is None:
            strides = dtype.itemsize
        dptr = self.open(context)
        return devicearray.DeviceNDArray(shape=shape, strides=strides, dtype=dtype, gpu_data=dptr)

    def close(self):
        if self._impl is None:
            raise ValueError("IpcHandle not opened")
        self._impl.close()
        self._impl = None

    def __reduce__(self):
        return (_rebuild_ipc_handle, (self.__class__, self.handle.reserved, self.size, self.source_info, self.offset))

    @classmethod
    def _rebuild(cls, handle_bytes, size, source_info, offset):
        return cls(base=None, handle=IpcMemHandle(handle_bytes), size=size, source_info=source_info, offset=offset)


def _rebuild_ipc_handle(cls, *args):
    return cls._rebuild(*args)


class MemoryPointer:
    """A device buffer (reference :1606-1717).  `refct` counts the owned
    references handed out by own()/view(); for the base class the buffer lives as
    long as the instance, for AutoFreePointer as long as refct > 0."""

    __cuda_memory__ = True

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        if isinstance(pointer, (c_void_p, c_size_t)):
            pointer = pointer.value
        address = int(pointer or 0)
        self.context, self._owner = context, owner
        self.device_pointer = self.handle = address
        self.size = self._cuda_memsize_ = size
        self.refct = 1
        self.is_managed = finalizer is not None
        if self.is_managed:
            self._finalizer = weakref.finalize(self, finalizer)

    @property
    def owner(self):
        return self if self._owner is None else self._owner

    def own(self):
        return OwnedPointer(weakref.proxy(self))

    def free(self):
        """Send the buffer to the pending-deallocation queue now."""
        if self.is_managed:
            if not self._finalizer.alive:
                raise RuntimeError("Freeing dead memory")
            self._finalizer()
            assert not self._finalizer.alive

    def memset(self, byte, count=None, stream=0):
        count = self.size if count is None else count
        driver.nbh_memset8(self.device_pointer, byte, count, _stream_handle(stream) or None)

    def view(self, start, stop=None):
        size = (self.size - start) if stop is None else (stop - start)
        if not self.device_pointer_value:
            if size != 0:
                raise RuntimeError("non-empty slice into empty slice")
            view = self
        else:
            if size < 0:
                raise RuntimeError("size cannot be negative")
            view = MemoryPointer(self.context, self.device_pointer_value + start, size, owner=self.owner)
        if isinstance(self.owner, (MemoryPointer, OwnedPointer)):
            # the owner is memory we manage: the view holds a counted reference
            return OwnedPointer(weakref.proxy(self.owner), view)
        return view   # foreign owner: the view just carries it along

    @property
    def device_ctypes_pointer(self):
        return c_size_t(self.device_pointer)

    @property
    def device_pointer_value(self):
        return self.device_pointer or None


class AutoFreePointer(MemoryPointer):
    """Freed when the last owned reference goes away (reference :1719-1733)."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.refct -= 1


class _HostBufferMixin(_hostbuf.HostBuffer):
    """Host-visible memory objects export [_bufptr_, _bufptr_ + _buflen_) through the
    buffer protocol (`np.ndarray(shape, dtype, buffer=mem)`); the buffer keeps the
    allocation alive.  The base class is native (cext/hostbuf.c), as the reference's is
    (cext/mviewbuf.c:212-363)."""

    def as_buffer(self):
        return self


class MappedMemory(AutoFreePointer, _HostBufferMixin):
    """Page-locked host memory that is also addressable from the device."""

    __cuda_memory__ = True

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        self.owned = owner
        self.host_pointer = int(pointer)
        devptr = c_void_p()
        driver.nbh_host_get_device_pointer(byref(devptr), self.host_pointer)
        super().__init__(context, devptr.value or 0, size, finalizer=finalizer)
        self.handle = self.host_pointer
        self._bufptr_ = self.host_pointer
        self._buflen_ = self.size

    def own(self):
        return MappedOwnedPointer(weakref.proxy(self))


class ManagedMemory(AutoFreePointer, _HostBufferMixin):
    """Managed memory: one address, valid on the host and on the device
    (reference :1813-1845)."""

    __cuda_memory__ = True

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        self.owned = owner
        super().__init__(context, int(pointer), size, finalizer=finalizer)
        self.host_pointer = int(pointer)
        self._bufptr_ = self.host_pointer
        self._buflen_ = self.size

    def own(self):
        return ManagedOwnedPointer(weakref.proxy(self))


class PinnedMemory(_HostBufferMixin):
    """Page-locked host memory (reference :1770-1808)."""

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        self.context = context
        self.owned = owner
        self.size = size
        self.host_pointer = int(pointer)
        self.is_managed = finalizer is not None
        self.handle = self.host_pointer
        self._buflen_ = self.size
        self._bufptr_ = self.host_pointer
        if finalizer is not None:
            weakref.finalize(self, finalizer)

    def own(self):
        return self


class OwnedPointer:
    """A counted reference to a MemoryPointer, optionally looking at a sub-range
    of it (reference :1848-1880).  Creating one bumps the owner's `refct`; when it
    is collected the count drops again and the owner is freed at zero.  Attribute
    access falls through to the pointer it looks at."""

    def __init__(self, memptr, view=None):
        target = memptr if view is None else view
        if view is not None:
            assert not view.is_managed
        self._mem, self._view = memptr, target
        # used on every kernel argument: worth a real attribute
        self.device_ctypes_pointer = target.device_ctypes_pointer
        memptr.refct += 1
        weakref.finalize(self, _drop_reference, memptr)

    def __getattr__(self, fname):
        return getattr(self._view, fname)

    def view(self, start, stop=None):
        # a real method rather than a fall-through: in `ctx.memalloc(n).view(k)` the
        # temporary reference must outlive the call, or the memory is freed before the
        # derived pointer has taken its own reference
        return self._view.view(start, stop)


def _drop_reference(mem):
    try:
        mem.refct -= 1
        assert mem.refct >= 0
        if mem.refct == 0:
            mem.free()
    except ReferenceError:
        pass      # the owner went first; nothing left to release


class MappedOwnedPointer(OwnedPointer, _HostBufferMixin):
    pass


class ManagedOwnedPointer(OwnedPointer, _HostBufferMixin):
    pass


# --------------------------------------------------------------------------------
# Streams and events
# --------------------------------------------------------------------------------

class Stream:
    """A HIP stream; handle 0 is the legacy default stream (reference :1890-2017)."""

    def __init__(self, handle, finalizer=None, external=False):
        self.handle = int(handle or 0)
        self.external = external
        if finalizer is not None:
            weakref.finalize(self, finalizer)

    def __int__(self):
        return self.handle

    def __eq__(self, other):
        if isinstance(other, Stream):
            return self.handle == other.handle
        if isinstance(other, int):
            return self.handle == other
        return NotImplemented

    def __hash__(self):
        return hash(self.handle)

    def __cuda_stream__(self):
        return (0, self.handle)

    def __repr__(self):
        if self.handle == 0:
            return "<Default HIP stream>"
        if self.handle == HIP_STREAM_PER_THREAD:
            return "<Per-thread default HIP stream>"
        if self.external:
            return "<External HIP stream %d>" % self.handle
        return "<HIP stream %d>" % self.handle

    def synchronize(self):
        driver.nbh_stream_synchronize(self.handle or None)

    def query(self):
        return _query(driver.lib.nbh_stream_query(self.handle or None), "nbh_stream_query")

    @contextlib.contextmanager
    def auto_synchronize(self):
        yield self
        self.synchronize()

    def add_callback(self, callback, arg=None):
        """Call `callback(stream, status, arg)` from a runtime thread once everything
        queued on this stream so far has finished (status is 0).  The callback must
        not call back into the GPU API and should be short: later work on the stream
        waits for it."""
        token = object()

        def trampoline(_user):
            try:
                callback(self, 0, arg)
            except Exception as e:   # nothing can propagate out of a runtime thread
                import warnings
                warnings.warn("Exception in stream callback: %s" % (e,))
            finally:
                _live_callbacks.pop(token, None)

        cfn = _lib.HOST_FN(trampoline)
        _live_callbacks[token] = cfn          # keep the thunk alive until it has run
        try:
            driver.nbh_stream_add_callback(self.handle or None, cfn, None)
        except Exception:
            _live_callbacks.pop(token, None)
            raise

    def async_done(self):
        """Awaitable that resolves (to this stream) once all work queued so far is done."""
        import asyncio
        loop = asyncio.get_running_loop()
        future = loop.create_future()

        def resolver(fut, status):
            if fut.done():
                return
            if status == 0:
                fut.set_result(self)
            else:
                fut.set_exception(Exception("Stream error %s" % status))

        def callback(stream, status, fut):
            loop.call_soon_threadsafe(resolver, fut, status)

        self.add_callback(callback, future)
        return future


_live_callbacks = {}


def _query(code, fname):
    if code == _lib.HIP_ERROR_NOT_READY:
        return False
    driver.check(fname, code)
    return True


class Event:
    """A HIP event (reference :2037-2095)."""

    def __init__(self, handle, finalizer=None):
        self.handle = int(handle or 0)
        if finalizer is not None:
            weakref.finalize(self, finalizer)

    def query(self):
        driver.ensure_initialized()
        return _query(driver.lib.nbh_event_query(self.handle), "nbh_event_query")

    def record(self, stream=0):
        driver.nbh_event_record(self.handle, _stream_handle(stream) or None)

    def synchronize(self):
        driver.nbh_event_synchronize(self.handle)

    def wait(self, stream=0):
        driver.nbh_stream_wait_event(_stream_handle(stream) or None, self.handle)

    def elapsed_time(self, evtend):
        return event_elapsed_time(self, evtend)


def event_elapsed_time(evtstart, evtend):
    """Milliseconds between two recorded events."""
    ms = ctypes.c_float()
    driver.nbh_event_elapsed_ms(byref(ms), evtstart.handle, evtend.handle)
    return ms.value


def _stream_handle(stream):
    """0 or a Stream object -> raw handle (reference :2767-2789)."""
    if isinstance(stream, Stream):
        return stream.handle
    if isinstance(stream, int) and stream == 0:
        return 0
    if hasattr(stream, "__cuda_stream__"):
        ver, ptr = stream.__cuda_stream__()
        assert ver == 0
        return int(ptr)
    raise TypeError("Expected a Stream object or 0, got %s" % type(stream).__name__)


# --------------------------------------------------------------------------------
# Pointers, extents, copies
# --------------------------------------------------------------------------------

def _is_datetime_dtype(obj):
    dtype = getattr(obj, "dtype", None)
    return dtype is not None and dtype.char in "Mm"


def _workaround_for_datetime(obj):
    # datetime64 / timedelta64 do not export a buffer; their int64 view does
    return obj.view(np.int64) if _is_datetime_dtype(obj) else obj


def host_pointer(obj, readonly=False):
    """Address of a host buffer (reference :2537-2554 + cext/mviewbuf.c:48-70).
    Accepts an int, a NumPy array or scalar, or any buffer-protocol object."""
    if isinstance(obj, int):
        return obj
    obj = _workaround_for_datetime(obj)
    if isinstance(obj, np.ndarray):
        if not readonly and not obj.flags.writeable:
            raise BufferError("writable buffer requested from a read-only array")
        return obj.ctypes.data
    if isinstance(obj, np.generic):          # e.g. np.void records
        return obj.__array_interface__["data"][0]
    if isinstance(obj, ctypes.Array):
        return ctypes.addressof(obj)
    return _hostbuf.address(obj, not readonly)


def _extents(ptr, shape, strides, itemsize):
    """Half-open byte range an array touches (reference cext/mviewbuf.c:76-135)."""
    lo, hi = _hostbuf.extents_of(shape, strides, itemsize)
    return ptr + lo, ptr + hi


def host_memory_extents(obj):
    obj = _workaround_for_datetime(obj)
    if isinstance(obj, (np.ndarray, np.generic)):
        a = np.asarray(obj)
        return _extents(a.__array_interface__["data"][0], a.shape, a.strides, a.itemsize)
    return _hostbuf.extents(obj)


def host_memory_size(obj):
    s, e = host_memory_extents(obj)
    assert e >= s, "memory extend of negative size"
    return e - s


@functools.lru_cache(maxsize=4096)
def memory_size_from_info(shape, strides, itemsize):
    """Bytes spanned by an array with this shape and strides, gaps included."""
    assert len(shape) == len(strides), "# dim mismatch"
    s, e = _extents(0, shape, strides, itemsize)
    return e - s


def device_pointer(obj):
    return device_ctypes_pointer(obj).value


def device_ctypes_pointer(obj):
    if obj is None:
        return c_void_p(0)
    require_device_memory(obj)
    return obj.device_ctypes_pointer


def is_device_memory(obj):
    """Device memory is anything with a truthy __cuda_memory__ attribute."""
    try:
        return obj.__cuda_memory__
    except AttributeError:
        return False


def require_device_memory(obj):
    if not is_device_memory(obj):
        raise Exception("Not a CUDA memory object.")


def device_extents(devmem):
    """[begin, end) of the whole allocation that `devmem` points into."""
    base, size = c_void_p(), c_size_t()
    driver.nbh_mem_address_range(byref(base), byref(size), device_ctypes_pointer(devmem).value)
    b = base.value or 0
    return b, b + size.value


def device_memory_size(devmem):
    sz = getattr(devmem, "_cuda_memsize_", None)
    if sz is None:
        s, e = device_extents(devmem)
        sz = e - s
        devmem._cuda_memsize_ = sz
    assert sz >= 0, "{} length array".format(sz)
    return sz


def device_memory_depends(devmem, *objs):
    depset = getattr(devmem, "_depends_", [])
    depset.extend(objs)


def host_to_device(dst, src, size, stream=0):
    """Synchronous on stream 0, asynchronous on any other stream; the host buffer
    must stay untouched until an asynchronous copy has finished."""
    driver.nbh_memcpy_h2d(device_pointer(dst), host_pointer(src, readonly=True), size,
                          _stream_handle(stream) or None)


def device_to_host(dst, src, size, stream=0):
    driver.nbh_memcpy_d2h(host_pointer(dst), device_pointer(src), size, _stream_handle(stream) or None)


def device_to_device(dst, src, size, stream=0):
    driver.nbh_memcpy_d2d(device_pointer(dst), device_pointer(src), size, _stream_handle(stream) or None)


def device_memset(dst, val, size, stream=0):
    driver.nbh_memset8(device_pointer(dst), val, size, _stream_handle(stream) or None)


def profile_start():
    """Profiling is driven from outside the process with rocprofv3; nothing to arm."""


def profile_stop():
    pass


@contextlib.contextmanager
def profiling():
    profile_start()
    yield
    profile_stop()


def get_version():
    return driver.get_version()
