"""HIP driver layer: devices, contexts, memory objects, streams, events, copies.

The public names and their behaviour follow numba_cuda/numba/cuda/cudadrv/driver.py
of the reference (each class cites the lines it stands in for), so that code written
against `numba.cuda.cudadrv.driver` keeps working.  What is underneath is different:
there is no driver binding, only the C entry points of libnbhip.so (include/nbhip.h),
and HIP has one implicit primary context per device, so `Context` is a per-device
bookkeeping object (memory manager, releases that wait, reduction scratch) rather
than a driver handle.

Lifetimes are owned here, in Python.  Device memory is a `MemoryPointer`; when its
last owner goes away the raw free is not executed but parked in the context's queue
of waiting releases (`_PendingDeallocs`) and carried out in batches, so that garbage
collection never turns into a device-wide synchronisation in the middle of
asynchronous work.
"""

import ctypes
import importlib
import logging
import os
import sys
import threading
import weakref
from abc import ABCMeta, abstractmethod
from collections import namedtuple
from ctypes import byref, c_int, c_size_t, c_void_p

import numpy as np

from numba_cuda_amd import _lib

from numba_cuda_amd import _build

if _build.hostbuf_needs_building():      # not built yet, or older than its source: one gcc call, about a second
    try:
        _build.build_hostbuf()
    except Exception:
        import os as _os
        if not _os.path.exists(_build.HOSTBUF_PATH):
            raise
        # an older build is there and cannot be replaced (no compiler, read-only tree):
        # it lacks what was added since, and the callers of those parts check for them
from numba_cuda_amd import _hostbuf
from numba_cuda_amd.core import config
from numba_cuda_amd.core.errors import CudaDriverError, CudaSupportError  # noqa: F401


def make_logger():
    """Logger of this module.  NUMBA_CUDA_LOG_LEVEL names a level of the logging
    module; with anything else the logger stays silent."""
    log = logging.getLogger(__name__)
    level = getattr(logging, str(config.CUDA_LOG_LEVEL).upper(), None)
    if isinstance(level, int):
        log.setLevel(level)
        if not log.handlers:
            to_stderr = logging.StreamHandler(sys.stderr)
            to_stderr.setFormatter(logging.Formatter("== HIP [%(relativeCreated)d] %(levelname)5s -- %(message)s"))
            log.addHandler(to_stderr)
    else:
        log.addHandler(logging.NullHandler())
    return log


_logger = make_logger()


class CudaAPIError(CudaDriverError):
    """A libnbhip / HIP call returned a non-zero hipError_t (reference:
    driver.py:147-154; same name so that user except-clauses keep working).
    `code` is the hipError_t, `msg` names the call and the error."""

    def __init__(self, code, msg):
        super().__init__(code, msg)
        self.code, self.msg = code, msg

    def __str__(self):
        return "[{}] {}".format(self.code, self.msg)


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
            obj._devices = {}
            cls._singleton = obj
        return cls._singleton

    def _refuse_if_broken(self):
        if self.initialization_error is not None:
            raise CudaSupportError("Error at driver init: %s" % self.initialization_error)

    def ensure_initialized(self):
        if not self.is_initialized:
            with self._lock:
                if not self.is_initialized:
                    self._load()
                    self.is_initialized = True
        self._refuse_if_broken()

    def _load(self):
        if config.DISABLE_CUDA:
            self.initialization_error = "GPU support disabled by NUMBA_DISABLE_CUDA=1"
        elif config.ENABLE_CUDASIM:
            self.initialization_error = ("NUMBA_ENABLE_CUDASIM=1 selects the CPU mode (numba_cuda_amd.simulator): "
                                         "the GPU library is not loaded")
        else:
            try:
                self.lib = _lib.load()
                self.pid = os.getpid()
            except OSError as e:
                self.initialization_error = str(e)

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
        """Raise for a non-zero status of the call named `fname`."""
        if code == _lib.HIP_SUCCESS:
            return
        if self.pid is not None and os.getpid() != self.pid:
            # a forked child inherits a runtime it cannot use
            raise CudaDriverError("HIP initialized before forking")
        raise CudaAPIError(code, "Call to %s results in %s" % (fname, self._error_name(code)))

    def __getattr__(self, fname):
        # first use of an entry point: build its checked wrapper and keep it
        if not fname.startswith("nbh_"):
            raise AttributeError(fname)
        self.ensure_initialized()
        entry = getattr(self.lib, fname)
        check = self.check

        def checked(*args):
            if _logger.isEnabledFor(logging.DEBUG):
                if config.CUDA_LOG_API_ARGS:
                    _logger.debug("call driver api: %s%r", fname, args)
                else:
                    _logger.debug("call driver api: %s", fname)
            status = entry(*args)
            if status:
                check(fname, status)

        checked.__name__ = fname
        setattr(self, fname, checked)
        return checked

    # --- devices
    def get_device_count(self):
        n = c_int(0)
        self.nbh_device_count(byref(n))
        return n.value

    def get_device(self, devnum=0):
        dev = self._devices.get(devnum)
        if dev is None:
            if not 0 <= devnum < self.get_device_count():
                raise CudaAPIError(101, "Call to hipSetDevice results in hipErrorInvalidDevice")
            with self._lock:
                dev = self._devices.setdefault(devnum, Device(devnum))
        return dev

    def list_devices(self):
        return [self.get_device(i) for i in range(self.get_device_count())]

    def get_version(self):
        """The HIP driver's version as (major, minor); reference :410-418."""
        return self.hip_versions()[0]

    def hip_versions(self):
        """((major, minor) of the HIP driver, (major, minor) of the HIP runtime)."""
        drv, rt = c_int(0), c_int(0)
        self.nbh_hip_versions(byref(drv), byref(rt))
        return tuple((v // 10000000, v // 100000 % 100) for v in (drv.value, rt.value))

    # --- the calling thread's active context (reference :387-407; HIP has one implicit
    # context per device, so "pushed" contexts are a per-thread list kept here)
    def get_active_context(self):
        """Context manager describing what is active on the calling thread: `.devnum` and
        `.context_handle`, both None when the thread has not selected a device yet."""
        return _ActiveContext()

    def pop_active_context(self):
        """Take the calling thread's most recently pushed context off its stack and make the
        one below it (if any) current; returns the popped context's handle or None."""
        stack = _ActiveContext.pushed()
        if not stack:
            return None
        popped = stack.pop()
        if stack:
            self.nbh_set_device(stack[-1])
        return popped


class _ActiveContext:
    """What `Driver.get_active_context()` hands out (reference :420-470)."""

    _tls = threading.local()

    @classmethod
    def pushed(cls):
        try:
            return cls._tls.stack
        except AttributeError:
            stack = cls._tls.stack = []
            return stack

    def __enter__(self):
        from numba_cuda_amd.cudadrv import devices
        stack = self.pushed()
        self.devnum = stack[-1] if stack else devices._runtime.current_device
        self.context_handle = self.devnum
        return self

    def __exit__(self, *exc_info):
        return False

    def __bool__(self):
        return self.devnum is not None


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

    def release_primary_context(self):
        """Forget this device's context object after releasing what it holds (reference
        :559-565).  HIP keeps its own implicit context per device; the next use builds a
        fresh bookkeeping object."""
        with self._ctx_lock:
            ctx, self.primary_context = self.primary_context, None
        if ctx is not None:
            ctx.reset()

    # What the element types need from the hardware (reference :576-586 asks the compute
    # capability): every device this library runs on converts and computes in these.
    supports_float16 = True
    supports_bfloat16 = True
    supports_fp8 = True

    def __repr__(self):
        return "<HIP device %d '%s'>" % (self.id, self.name)

    def __eq__(self, other):
        return isinstance(other, Device) and other.id == self.id

    def __hash__(self):
        return hash(("hip-device", self.id))


# --------------------------------------------------------------------------------
# Releases that wait
# --------------------------------------------------------------------------------

class _Hold:
    """`with queue.disable():` - one more reason not to flush while inside."""

    __slots__ = ("_queue",)

    def __init__(self, queue):
        self._queue = queue

    def __enter__(self):
        with self._queue._lock:
            self._queue._holds += 1
        return self._queue

    def __exit__(self, exc_type, exc, tb):
        with self._queue._lock:
            self._queue._holds -= 1
        return False


class _PendingDeallocs:
    """Releases (`release(handle)` calls) parked until there are enough of them
    (reference :975-1045; the counts and thresholds are the ones its
    tests/cudadrv/test_deallocations.py pins).

    `add_item` parks one; the whole batch is carried out as soon as more than
    config.CUDA_DEALLOCS_COUNT entries, or more than config.CUDA_DEALLOCS_RATIO of
    `memory_capacity` bytes, are waiting - and by `clear()`, which the allocator
    calls when the device runs out of memory and the context calls on reset.
    Inside `with queue.disable():` (nestable) nothing is carried out at all.

    Finalizers run on whatever thread drops the last reference, so the queue is
    guarded by a lock; the batch is taken out of the queue before the first release
    runs, which makes a release that parks further entries harmless.

    `memory_capacity` is None until the memory manager has asked the device; the
    byte threshold is 0 until then."""

    def __init__(self, capacity=None):
        self.memory_capacity = capacity
        self._lock = threading.RLock()
        self._waiting = []          # (release, handle, bytes or None)
        self._waiting_bytes = 0
        self._holds = 0

    @property
    def byte_budget(self):
        """Bytes that may wait before a flush."""
        if self.memory_capacity is None:
            return 0
        return int(config.CUDA_DEALLOCS_RATIO * self.memory_capacity)

    @property
    def pending_bytes(self):
        """Bytes (of entries with a known size) waiting now."""
        return self._waiting_bytes

    # the reference's own test-suite reads these two private names
    _max_pending_bytes = byte_budget
    _size = pending_bytes

    def add_item(self, release, handle, size=None):
        """Park `release(handle)`; `size` is the footprint in bytes when known."""
        _logger.info("park release: %s, %s bytes", _name_of(release), "?" if size is None else size)
        with self._lock:
            self._waiting.append((release, handle, size))
            if size is not None:
                self._waiting_bytes += int(size)
            full = (len(self._waiting) > config.CUDA_DEALLOCS_COUNT
                    or self._waiting_bytes > self.byte_budget)
        if full:
            self.clear()

    def clear(self):
        """Carry out everything that waits - unless flushing is held off."""
        with self._lock:
            if self._holds:
                return
            batch, self._waiting = self._waiting, []
            self._waiting_bytes = 0
        done = 0
        try:
            for release, handle, size in batch:
                _logger.info("release: %s, %s bytes", _name_of(release), "?" if size is None else size)
                done += 1
                release(handle)
        finally:
            if done < len(batch):       # a release raised: the rest goes back to the front
                with self._lock:
                    rest = batch[done:]
                    self._waiting[:0] = rest
                    self._waiting_bytes += sum(int(s) for _, _, s in rest if s is not None)

    def disable(self):
        """Context manager: no flushing inside (the queue only grows)."""
        return _Hold(self)

    @property
    def is_disabled(self):
        return self._holds > 0

    def __len__(self):
        return len(self._waiting)


def _name_of(fn):
    return getattr(fn, "__name__", None) or repr(fn)


class _Release:
    """Finalizer of one tracked allocation: take it out of the manager's table of
    live allocations and hand the raw free to the queue of waiting releases - or,
    with no queue, carry it out on the spot (reference :1316-1371 has three
    closures for this).  Built from the tables themselves rather than the manager, so
    that the finalizer does not keep the manager (and its context) alive."""

    __slots__ = ("table", "key", "queue", "raw_free", "address", "nbytes")

    def __init__(self, raw_free, address, nbytes=None, table=None, key=None, queue=None):
        self.raw_free, self.address, self.nbytes = raw_free, address, nbytes
        self.table, self.key, self.queue = table, key, queue

    def __call__(self):
        if self.table is not None:
            self.table.pop(self.key, None)
        if self.queue is None:
            self.raw_free(self.address)
        else:
            self.queue.add_item(self.raw_free, self.address, self.nbytes)


def _free_device(ptr):
    driver.nbh_free(ptr)


def _free_host(ptr):
    driver.nbh_host_free(ptr)


def _unregister_host(ptr):
    driver.nbh_host_unregister(ptr)


def _destroy_stream(handle):
    driver.nbh_stream_destroy(handle)


def _destroy_event(handle):
    driver.nbh_event_destroy(handle)


MemoryInfo = namedtuple("MemoryInfo", "free,total")


# --------------------------------------------------------------------------------
# Memory managers (the EMM plugin interface of the reference, :589-957)
# --------------------------------------------------------------------------------

_SUPPORTED_EMM_INTERFACE_VERSION = 1


class BaseCUDAMemoryManager(metaclass=ABCMeta):
    """What an external memory manager has to provide.  One instance is made per
    context, with the context passed as a keyword."""

    def __init__(self, *args, **kwargs):
        try:
            self.context = kwargs.pop("context")
        except KeyError:
            raise RuntimeError("Memory manager requires a context") from None

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
    that only care about device memory derive from this (reference :705-872).

    `allocations` maps the address of every live tracked allocation to its memory
    object, `deallocations` is the queue of releases that wait."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.allocations = {}
        self.deallocations = _PendingDeallocs()

    def _attempt_allocation(self, allocator):
        """Result of `allocator()`.  If the device is out of memory, everything
        that waits to be released is released and the allocation tried once more."""
        for last_try in (False, True):
            try:
                return allocator()
            except CudaAPIError as e:
                if last_try or e.code != _lib.HIP_ERROR_OUT_OF_MEMORY:
                    raise
                self.deallocations.clear()

    def _track(self, mem, address):
        self.allocations[address] = mem
        return mem.own()

    def _context_proxy(self):
        return weakref.proxy(self.context)

    def memhostalloc(self, size, mapped=False, portable=False, wc=False):
        flags = (1 if portable else 0) | (2 if mapped else 0) | (4 if wc else 0)

        def allocate():
            out = c_void_p()
            driver.nbh_host_alloc(byref(out), size, flags)
            return out.value or 0

        if not mapped:
            # plain page-locked memory: not in the table, footprint on the device unknown
            address = allocate()
            return PinnedMemory(self._context_proxy(), address, size,
                                finalizer=_Release(_free_host, address, queue=self.deallocations))
        address = self._attempt_allocation(allocate)
        on_release = _Release(_free_host, address, size, self.allocations, address, self.deallocations)
        return self._track(MappedMemory(self._context_proxy(), address, size, finalizer=on_release), address)

    def mempin(self, owner, pointer, size, mapped=False):
        def register():
            driver.nbh_host_register(pointer, size, 2 if mapped else 0)

        # Page-locking is undone the moment the object dies, not queued: the same
        # host buffer may be pinned again right away (`with cuda.pinned(a): ...` twice).
        if not mapped:
            register()
            return PinnedMemory(self._context_proxy(), pointer, size, owner=owner,
                                finalizer=_Release(_unregister_host, pointer))
        self._attempt_allocation(register)
        on_release = _Release(_unregister_host, pointer, table=self.allocations, key=pointer)
        mem = MappedMemory(self._context_proxy(), pointer, size, owner=owner, finalizer=on_release)
        return self._track(mem, pointer)

    def memallocmanaged(self, size, attach_global):
        def allocate():
            out = c_void_p()
            driver.nbh_malloc_managed(byref(out), size, 1 if attach_global else 0)
            return out.value or 0

        address = self._attempt_allocation(allocate)
        on_release = _Release(_free_device, address, size, self.allocations, address, self.deallocations)
        return self._track(ManagedMemory(self._context_proxy(), address, size, finalizer=on_release), address)

    def reset(self):
        """Forget every tracked allocation (objects nobody else holds are finalized,
        which parks their frees), then carry out everything that waits."""
        tracked = self.allocations
        tracked.clear()
        self.deallocations.clear()

    def defer_cleanup(self):
        """Context manager: no waiting release is carried out inside."""
        return self.deallocations.disable()


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
    """The manager used unless another is plugged in: one hipMalloc per allocation,
    hipFree through the queue of waiting releases (reference :885-915)."""

    interface_version = _SUPPORTED_EMM_INTERFACE_VERSION

    def initialize(self):
        queue = self.deallocations
        if queue.memory_capacity is None:       # first use: now the device can be asked
            queue.memory_capacity = self.get_memory_info().total

    def memalloc(self, size):
        def allocate():
            out = c_void_p()
            driver.nbh_malloc(byref(out), size)
            return out.value or 0

        address = self._attempt_allocation(allocate)
        on_release = _Release(_free_device, address, size, self.allocations, address, self.deallocations)
        return self._track(AutoFreePointer(self._context_proxy(), address, size, finalizer=on_release), address)

    def get_memory_info(self):
        free, total = c_size_t(), c_size_t()
        driver.nbh_mem_info(byref(free), byref(total))
        return MemoryInfo(free=free.value, total=total.value)


# the class new contexts instantiate; None until the first context (or set_memory_manager)
_memory_manager = None


def set_memory_manager(mm_plugin):
    """Use an External Memory Management plugin class for all later contexts."""
    global _memory_manager
    found = mm_plugin(context=None).interface_version
    if found != _SUPPORTED_EMM_INTERFACE_VERSION:
        raise RuntimeError("EMM Plugin interface has version %d - version %d required"
                           % (found, _SUPPORTED_EMM_INTERFACE_VERSION))
    _memory_manager = mm_plugin


def _ensure_memory_manager():
    """Settle which manager class contexts use: one set by hand wins, then the
    module NUMBA_CUDA_MEMORY_MANAGER names (its `_numba_memory_manager`), then the
    built-in one."""
    global _memory_manager
    if _memory_manager is not None:
        return
    wanted = config.CUDA_MEMORY_MANAGER
    if wanted == "default":
        _memory_manager = NumbaCUDAMemoryManager
        return
    try:
        set_memory_manager(importlib.import_module(wanted)._numba_memory_manager)
    except Exception:
        raise RuntimeError("Failed to use memory manager from %s" % wanted)


# --------------------------------------------------------------------------------
# Context
# --------------------------------------------------------------------------------

HIP_STREAM_LEGACY = 1
HIP_STREAM_PER_THREAD = 2


class _ResultCells:
    """16-byte cells in page-locked, device-mapped host memory.  A reduction that
    returns its value to the caller has the kernel write it into a cell and reads it
    after waiting for the stream: no device-to-host copy, which would cost as much
    again as the launch.  Every call takes a cell of its own and gives it back after
    reading, so calls on any mix of host threads and streams never share one."""

    CELL = 16
    BLOCK = 4096

    def __init__(self):
        self._lock = threading.Lock()
        self._blocks = []       # (host address, uint8 array over the block)
        self._free = []         # (device address, uint8 view of the cell)

    def take(self):
        try:
            return self._free.pop()
        except IndexError:
            pass
        with self._lock:
            if not self._free:
                host, dev = c_void_p(), c_void_p()
                driver.nbh_host_alloc(byref(host), self.BLOCK, 2)       # 2: device-mapped
                driver.nbh_host_get_device_pointer(byref(dev), host.value)
                raw = np.frombuffer((ctypes.c_ubyte * self.BLOCK).from_address(host.value), dtype=np.uint8)
                self._blocks.append((host.value, raw))
                for off in range(0, self.BLOCK, self.CELL):
                    self._free.append((dev.value + off, raw[off:off + self.CELL]))
            return self._free.pop()

    def give_back(self, cell):
        self._free.append(cell)

    def release_all(self):
        with self._lock:
            blocks, self._blocks, self._free = self._blocks, [], []
        for host, _ in blocks:
            try:
                driver.nbh_host_free(host)
            except Exception:
                pass


class Context:
    """Per-device state (reference: Context :1061-1301)."""

    def __init__(self, device):
        self.device, self.handle = device, device.id
        self.extras = {}
        self.deallocations = _PendingDeallocs()      # streams and events; memory waits in the manager's queue
        _ensure_memory_manager()
        manager_class = _memory_manager
        self.memory_manager = manager_class(context=self)
        self._scratch_lock = threading.Lock()
        self._scratch = {}          # stream handle -> (address, bytes, memory) of nbh_reduce's scratch
        self._scratch_tls = threading.local()   # the same for each thread's per-thread default stream
        self._result_cells = _ResultCells()

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
        with self._scratch_lock:
            self._scratch.clear()
        self._scratch_tls = threading.local()
        self._result_cells.release_all()
        self._memory_manager.reset()
        self.deallocations.clear()

    def prepare_for_use(self):
        """Called whenever the context is fetched: lets the manager initialise (once)."""
        self._memory_manager.initialize()
        self.prepared = True

    def push(self):
        """Make this context's device current on the calling thread, remembering it on the
        thread's stack (reference :1161-1167)."""
        driver.nbh_set_device(self.device.id)
        _ActiveContext.pushed().append(self.device.id)
        self.prepare_for_use()

    def pop(self):
        """Undo the latest push; this context must be the one on top (reference :1169-1175)."""
        stack = _ActiveContext.pushed()
        assert stack and stack[-1] == self.device.id, "this context is not at the top of the thread's stack"
        driver.pop_active_context()

    # --- memory: all of it is the memory manager's business

    def get_memory_info(self):
        """(free, total) bytes of device memory."""
        return self._memory_manager.get_memory_info()

    def memalloc(self, bytesize):
        """Device memory -> owned MemoryPointer."""
        return self._memory_manager.memalloc(bytesize)

    def memallocmanaged(self, bytesize, attach_global=True):
        """Memory with one address valid on host and device."""
        return self._memory_manager.memallocmanaged(bytesize, attach_global)

    def memhostalloc(self, bytesize, mapped=False, portable=False, wc=False):
        """Page-locked host memory, optionally addressable from the device."""
        return self._memory_manager.memhostalloc(bytesize, mapped, portable, wc)

    def mempin(self, owner, pointer, size, mapped=False):
        """Page-lock `size` bytes of existing host memory at `pointer`."""
        if mapped and not self.device.CAN_MAP_HOST_MEMORY:
            raise CudaDriverError("%s cannot map host memory" % self.device)
        return self._memory_manager.mempin(owner, pointer, size, mapped)

    def defer_cleanup(self):
        """Context manager: neither the manager's nor the context's waiting
        releases are carried out inside."""
        return _Both(self._memory_manager.defer_cleanup(), self.deallocations.disable())

    # --- sharing memory with other processes

    def get_ipc_handle(self, memory):
        """An IpcHandle for `memory`, to be sent to another process (reference :1190-1198)."""
        if not sys.platform.startswith("linux"):
            raise OSError("OS does not support CUDA IPC")
        return self._memory_manager.get_ipc_handle(memory)

    def open_ipc_handle(self, handle, size):
        """Map the allocation `handle` names into this process; `size` bytes of it
        will be used (reference :1200-1209).  IpcHandle.close() unmaps it."""
        mapped_at = c_void_p()
        driver.nbh_ipc_open(byref(mapped_at), bytes(handle.reserved), size)
        return MemoryPointer(context=weakref.proxy(self), pointer=mapped_at, size=size)

    def can_access_peer(self, peer_device):
        """One device per process here: only the device itself is reachable."""
        return int(peer_device) == self.device.id

    # --- streams and events

    def get_default_stream(self):
        return Stream(0)

    def get_legacy_default_stream(self):
        return Stream(0)

    def get_per_thread_default_stream(self):
        return Stream(HIP_STREAM_PER_THREAD)

    def create_stream(self):
        out = c_void_p()
        driver.nbh_stream_create(byref(out))
        handle = out.value or 0
        return Stream(handle, finalizer=_StreamGone(self, handle))

    def create_external_stream(self, ptr):
        if isinstance(ptr, int):
            return Stream(ptr, external=True)
        raise TypeError("ptr for external stream must be an int")

    def create_event(self, timing=True):
        out = c_void_p()
        driver.nbh_event_create(byref(out), 1 if timing else 0)
        handle = out.value or 0
        return Event(handle, finalizer=_Release(_destroy_event, handle, queue=self.deallocations))

    def synchronize(self):
        driver.nbh_device_synchronize()

    # --- what nbh_reduce needs besides its input and output

    def reduce_scratch(self, stream_handle):
        """(address, size) of the scratch buffer (ticket + partials) for reductions
        on the given stream, allocated and zeroed on first use.

        Work on one stream runs in order, so every reduction on it can share one
        buffer, from any host thread; different streams may overlap and get their
        own.  The per-thread default stream is a different stream in every host
        thread under one handle: its buffer is kept per thread and goes away with
        the thread.  A buffer is released when its Stream object is destroyed."""
        if stream_handle == HIP_STREAM_PER_THREAD:
            entry = getattr(self._scratch_tls, "entry", None)
            if entry is None:
                entry = self._scratch_tls.entry = self._new_scratch()
            return entry[0], entry[1]
        entry = self._scratch.get(stream_handle)
        if entry is None:
            with self._scratch_lock:
                entry = self._scratch.get(stream_handle)
                if entry is None:
                    entry = self._scratch[stream_handle] = self._new_scratch()
        return entry[0], entry[1]

    def _new_scratch(self):
        nbytes = driver.lib.nbh_reduce_scratch_bytes()
        mem = self.memalloc(nbytes)
        address = mem.device_ctypes_pointer.value
        driver.nbh_memset8(address, 0, nbytes, None)
        return address, nbytes, mem

    def _forget_stream(self, stream_handle):
        """The stream is about to be destroyed: let go of what was kept for it."""
        with self._scratch_lock:
            self._scratch.pop(stream_handle, None)

    def take_result_cell(self):
        """(device address, 16 host bytes as a uint8 array) for one result; hand it
        back with give_back_result_cell() after reading."""
        return self._result_cells.take()

    def give_back_result_cell(self, cell):
        self._result_cells.give_back(cell)

    def __repr__(self):
        return "<HIP context of device %d>" % self.device.id

    def __eq__(self, other):
        return isinstance(other, Context) and other.handle == self.handle

    def __hash__(self):
        return hash(("hip-context", self.handle))


class _Both:
    """Two context managers entered together, left in reverse order."""

    def __init__(self, outer, inner):
        self._outer, self._inner = outer, inner

    def __enter__(self):
        self._outer.__enter__()
        try:
            self._inner.__enter__()
        except BaseException:
            self._outer.__exit__(*sys.exc_info())
            raise

    def __exit__(self, *exc):
        try:
            self._inner.__exit__(*exc)
        finally:
            self._outer.__exit__(*exc)
        return False


class _StreamGone:
    """Finalizer of a created stream: the context drops the scratch it kept for the
    stream (queued kernels may still use it - its free waits in the queue, and
    hipFree waits for the device), then the destroy call is parked too."""

    __slots__ = ("context", "handle")

    def __init__(self, context, handle):
        self.context = weakref.ref(context)
        self.handle = handle

    def __call__(self):
        ctx = self.context()
        if ctx is None:
            return
        ctx._forget_stream(self.handle)
        ctx.deallocations.add_item(_destroy_stream, self.handle)


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


class IpcHandle:
    """A picklable name for a device allocation that another process on the same
    machine can open (reference :1487-1603).

    base        the exporter's memory, kept alive by the handle (None once pickled)
    handle      IpcMemHandle
    size        bytes of the shared region
    source_info identity of the exporting device
    offset      where the region starts in the underlying allocation

    In the importing process open() maps the exporter's allocation and close()
    unmaps it; the handle owns the mapping in between."""

    def __init__(self, base, handle, size, source_info=None, offset=0):
        self.base, self.handle, self.size = base, handle, size
        self.source_info, self.offset = source_info, offset
        self._mapping = None        # MemoryPointer over the imported allocation while open
        self._staged = False        # open_staged() happened and close() has not yet

    def _refuse_if_open(self):
        if self._mapping is not None or self._staged:
            raise ValueError("IpcHandle is already opened")

    def _need_source_info(self):
        if self.source_info is None:
            raise RuntimeError("IPC handle doesn't have source info")

    def can_access_peer(self, context):
        self._need_source_info()
        here = context.device.get_device_identity()
        return self.source_info == here or context.can_access_peer(Device.from_identity(self.source_info).id)

    def open_staged(self, context):
        """For an importing device that cannot reach the exporting one: map the memory on
        the exporting device, copy it into a fresh allocation of `context` and unmap it
        again (reference :1445-1482).  The result is a COPY, owned by the caller; close()
        then has nothing left to undo.  The copy between two devices is the runtime's
        (direct if they are peers, through the host if not)."""
        from numba_cuda_amd.cudadrv import devices
        self._need_source_info()
        self._refuse_if_open()
        if self.base is not None:
            raise ValueError("opening IpcHandle from original process")
        wanted = self.offset + self.size
        if wanted >= IPC_ALLOCATION_LIMIT:
            raise ValueError("allocations of 2 GiB or more cannot be shared between processes")
        source = Device.from_identity(self.source_info)
        with devices.gpus[source.id]:
            mapping = devices.get_context().open_ipc_handle(self.handle, wanted)
        try:
            copy = context.memalloc(self.size)
            device_to_device(copy, mapping.view(self.offset), self.size)
        finally:
            with devices.gpus[source.id]:
                driver.nbh_ipc_close(mapping.handle)
        self._staged = True
        return copy

    def open_direct(self, context):
        self._refuse_if_open()
        if self.base is not None:
            raise ValueError("opening IpcHandle from original process")
        wanted = self.offset + self.size
        if wanted >= IPC_ALLOCATION_LIMIT:
            raise ValueError("allocations of 2 GiB or more cannot be shared between processes")
        self._mapping = context.open_ipc_handle(self.handle, wanted)
        return self._mapping.own().view(self.offset)

    def open(self, context):
        """Map the memory into `context`'s process -> device memory pointer."""
        if self.source_info is not None and not self.can_access_peer(context):
            return self.open_staged(context)
        return self.open_direct(context)

    def open_array(self, context, shape, dtype, strides=None):
        """open(), wrapped as a device array (1-d C-contiguous unless `strides` says otherwise)."""
        from numba_cuda_amd.cudadrv import devicearray
        memory = self.open(context)
        return devicearray.DeviceNDArray(shape=shape, strides=dtype.itemsize if strides is None else strides,
                                         dtype=dtype, gpu_data=memory)

    def close(self):
        if self._staged and self._mapping is None:     # a staged open left a copy, not a mapping
            self._staged = False
            return
        if self._mapping is None:
            raise ValueError("IpcHandle not opened")
        mapping, self._mapping = self._mapping, None
        driver.nbh_ipc_close(mapping.handle)

    def __reduce__(self):
        return (_rebuild_ipc_handle, (self.__class__, self.handle.reserved, self.size, self.source_info, self.offset))

    @classmethod
    def _rebuild(cls, handle_bytes, size, source_info, offset):
        return cls(base=None, handle=IpcMemHandle(handle_bytes), size=size, source_info=source_info, offset=offset)


def _rebuild_ipc_handle(cls, *args):
    return cls._rebuild(*args)


class MemoryPointer:
    """A range of device memory (reference :1606-1717).

    `refct` counts the references handed out by own() and view(), plus one for the
    object itself: a plain MemoryPointer therefore never drops to zero and its
    buffer lives exactly as long as the object (the finalizer, when one was given,
    runs when the object is collected or free() is called).  AutoFreePointer leaves
    the one for itself out, so there the last owned reference ends the buffer.

    `owner` is the object the buffer belongs to: the pointer itself, the pointer a
    view was cut from, or whatever foreign object was passed as `owner`."""

    __cuda_memory__ = True
    _counts_itself = 1

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        if isinstance(pointer, (c_void_p, c_size_t)):
            pointer = pointer.value
        self.context = context
        self.handle = self.device_pointer = int(pointer or 0)
        self.size = self._cuda_memsize_ = size
        self._owner = owner
        self.refct = self._counts_itself
        self.is_managed = finalizer is not None
        self._finalizer = weakref.finalize(self, finalizer) if self.is_managed else None

    @property
    def owner(self):
        return self._owner if self._owner is not None else self

    @property
    def device_pointer_value(self):
        """The address, or None for a null pointer."""
        return self.device_pointer or None

    @property
    def device_ctypes_pointer(self):
        return c_size_t(self.device_pointer)

    def own(self):
        """A counted reference to this memory."""
        return OwnedPointer(weakref.proxy(self))

    def _let_go(self):
        """One counted reference less; the last one ends the buffer."""
        self.refct -= 1
        if self.refct == 0:
            self.free()
        elif self.refct < 0:
            raise AssertionError("memory reference count below zero")

    def free(self):
        """Run the finalizer now (the raw free then waits in the queue)."""
        hook = self._finalizer
        if hook is None:
            return
        if not hook.alive:
            raise RuntimeError("Freeing dead memory")
        hook()

    def memset(self, byte, count=None, stream=0):
        nbytes = self.size if count is None else count
        driver.nbh_memset8(self.device_pointer, byte, nbytes, _stream_handle(stream) or None)

    def view(self, start, stop=None):
        """Pointer to bytes [start, stop) of this one (to the end without `stop`).
        When the buffer is memory managed here, the result holds a counted reference
        to the owner; with a foreign owner it simply carries that owner along."""
        nbytes = (self.size if stop is None else stop) - start
        if self.device_pointer_value is None:
            if nbytes:
                raise RuntimeError("non-empty slice into empty slice")
            piece = self                     # a view of nothing is the nothing itself
        elif nbytes < 0:
            raise RuntimeError("size cannot be negative")
        else:
            piece = MemoryPointer(self.context, self.device_pointer + start, nbytes, owner=self.owner)
        root = self.owner
        if isinstance(root, (MemoryPointer, OwnedPointer)):
            return OwnedPointer(weakref.proxy(root), piece)
        return piece


class AutoFreePointer(MemoryPointer):
    """Device memory that ends with its last owned reference (reference :1719-1733)."""

    _counts_itself = 0


class _HostBufferMixin(_hostbuf.HostBuffer):
    """Host-visible memory objects export [_bufptr_, _bufptr_ + _buflen_) through the
    buffer protocol (`np.ndarray(shape, dtype, buffer=mem)`); the buffer keeps the
    allocation alive.  The base class is native (cext/hostbuf.c), as the reference's is
    (cext/mviewbuf.c:212-363)."""

    def as_buffer(self):
        return self

    def _export(self, address, nbytes):
        self.host_pointer = self._bufptr_ = address
        self._buflen_ = nbytes


class MappedMemory(AutoFreePointer, _HostBufferMixin):
    """Page-locked host memory that is also addressable from the device
    (reference :1735-1768).  `handle` is the host address, `device_pointer` the
    address kernels use."""

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        host_address = int(pointer)
        seen_from_device = c_void_p()
        driver.nbh_host_get_device_pointer(byref(seen_from_device), host_address)
        super().__init__(context, seen_from_device.value or 0, size, finalizer=finalizer)
        self.owned = owner
        self.handle = host_address
        self._export(host_address, size)

    def own(self):
        return MappedOwnedPointer(weakref.proxy(self))


class ManagedMemory(AutoFreePointer, _HostBufferMixin):
    """Managed memory: one address, valid on the host and on the device
    (reference :1813-1845)."""

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        super().__init__(context, int(pointer), size, finalizer=finalizer)
        self.owned = owner
        self._export(self.device_pointer, size)

    def own(self):
        return ManagedOwnedPointer(weakref.proxy(self))


class PinnedMemory(_HostBufferMixin):
    """Page-locked host memory the device cannot address (reference :1770-1808).
    Not reference counted: own() is the object itself, and the finalizer runs when
    it is collected."""

    def __init__(self, context, pointer, size, owner=None, finalizer=None):
        self.context, self.owned, self.size = context, owner, size
        self._export(int(pointer), size)
        self.handle = self.host_pointer
        self.is_managed = bool(finalizer is not None)
        self._finalizer = weakref.finalize(self, finalizer) if self.is_managed else None

    def own(self):
        return self


def _let_go(memory):
    try:
        memory._let_go()
    except ReferenceError:
        pass      # the memory object went first; nothing left to release


class OwnedPointer:
    """A counted reference to a MemoryPointer, optionally looking at a sub-range
    of it (reference :1848-1880).  Creating one bumps the owner's `refct`; when it
    is collected the count drops again.  Every attribute not found here is the
    attribute of the pointer it looks at."""

    def __init__(self, memptr, view=None):
        if view is not None and view.is_managed:
            raise AssertionError("a view into owned memory cannot have a finalizer of its own")
        self._mem = memptr
        self._view = memptr if view is None else view
        # read for every kernel argument: worth real attributes
        self.device_ctypes_pointer = self._view.device_ctypes_pointer
        self.device_pointer = self._view.device_pointer
        memptr.refct += 1
        weakref.finalize(self, _let_go, memptr)

    def __getattr__(self, name):
        return getattr(self._view, name)

    def view(self, start, stop=None):
        # a real method rather than a fall-through: in `ctx.memalloc(n).view(k)` the
        # temporary reference must outlive the call, or the memory is freed before the
        # derived pointer has taken its own reference
        return self._view.view(start, stop)


class MappedOwnedPointer(OwnedPointer, _HostBufferMixin):
    pass


class ManagedOwnedPointer(OwnedPointer, _HostBufferMixin):
    pass


# --------------------------------------------------------------------------------
# Streams and events
# --------------------------------------------------------------------------------

class _SyncOnExit:
    """`with stream.auto_synchronize():` - wait for the stream when the block is
    left normally."""

    __slots__ = ("_stream",)

    def __init__(self, stream):
        self._stream = stream

    def __enter__(self):
        return self._stream

    def __exit__(self, exc_type, exc, tb):
        if exc_type is None:
            self._stream.synchronize()
        return False


class Stream:
    """A HIP stream; handle 0 is the legacy default stream (reference :1890-2017).

    The package keeps the raw handle in `_h`.  Whoever reads `handle`, converts the stream to
    an int or asks for `__cuda_stream__` is about to use the stream outside the package, where
    the launching threads' queues (kernels/reduction.py) are unknown: the stream's queue is
    launched first and its reductions are launched directly from then on."""

    def __init__(self, handle, finalizer=None, external=False):
        self._h = int(handle or 0)
        self.external = external
        self._exported = self._h in (0, HIP_STREAM_LEGACY, HIP_STREAM_PER_THREAD)   # default streams are never queued
        if external:
            self._export()
        if finalizer is not None:
            weakref.finalize(self, finalizer)

    def _export(self):
        self._exported = True
        if driver.is_initialized and driver.lib is not None:
            pin = getattr(driver.lib, "nbh_stream_pin_direct", None)
            if pin is not None:
                pin(self._h or None)

    @property
    def handle(self):
        if not self._exported:
            self._export()
        return self._h

    def __int__(self):
        return self.handle

    def __eq__(self, other):
        if isinstance(other, Stream):
            return self._h == other._h
        if isinstance(other, int):
            return self._h == other
        return NotImplemented

    def __hash__(self):
        return hash(self._h)

    def __cuda_stream__(self):
        return (0, self.handle)

    def __repr__(self):
        if self._h == 0:
            return "<Default HIP stream>"
        if self._h == HIP_STREAM_PER_THREAD:
            return "<Per-thread default HIP stream>"
        if self.external:
            return "<External HIP stream %d>" % self._h
        return "<HIP stream %d>" % self._h

    def synchronize(self):
        driver.nbh_stream_synchronize(self._h or None)

    def query(self):
        return _query(driver.lib.nbh_stream_query(self._h or None), "nbh_stream_query")

    def auto_synchronize(self):
        return _SyncOnExit(self)

    def add_callback(self, callback, arg=None):
        """Call `callback(stream, status, arg)` from a runtime thread once everything
        queued on this stream so far has finished (status is 0).  The callback must
        not call back into the GPU API and should be short: later work on the stream
        waits for it."""
        _drain_finished_thunks()
        slot = []

        def trampoline(_user):
            try:
                callback(self, 0, arg)
            except Exception as e:   # nothing can propagate out of a runtime thread
                import warnings
                warnings.warn("Exception in stream callback: %s" % (e,))
            finally:
                # The native thunk is still executing: it must not lose its last
                # reference here.  It moves to a list that later calls empty.
                _finished_thunks.append(_pending_thunks.pop(id(slot), None))

        thunk = _lib.HOST_FN(trampoline)
        slot.append(thunk)
        _pending_thunks[id(slot)] = (thunk, slot)
        try:
            driver.nbh_stream_add_callback(self._h or None, thunk, None)
        except Exception:
            _pending_thunks.pop(id(slot), None)
            raise

    def async_done(self):
        """Awaitable that resolves (to this stream) once all work queued so far is done."""
        import asyncio
        loop = asyncio.get_running_loop()
        future = loop.create_future()

        def settle(status):
            if future.done():
                return
            if status == 0:
                future.set_result(self)
            else:
                future.set_exception(Exception("Stream error %s" % status))

        self.add_callback(lambda _stream, status, _arg: loop.call_soon_threadsafe(settle, status))
        return future


_pending_thunks = {}     # id -> (thunk, holder) of callbacks that have not run yet
_finished_thunks = []    # thunks whose callback has run; dropped by a later call


def _drain_finished_thunks():
    # everything that was in the list when we got here returned from its thunk
    # at least one Python-level call ago
    n = len(_finished_thunks)
    if n > 64:
        del _finished_thunks[:n - 8]


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

    def record(self, stream=0):
        driver.nbh_event_record(self.handle, _stream_handle(stream) or None)

    def wait(self, stream=0):
        """Work queued on `stream` after this call starts after the event."""
        driver.nbh_stream_wait_event(_stream_handle(stream) or None, self.handle)

    def query(self):
        driver.ensure_initialized()
        return _query(driver.lib.nbh_event_query(self.handle), "nbh_event_query")

    def synchronize(self):
        driver.nbh_event_synchronize(self.handle)

    def elapsed_time(self, evtend):
        """Milliseconds from this event to `evtend`."""
        return event_elapsed_time(self, evtend)


def event_elapsed_time(evtstart, evtend):
    """Milliseconds between two recorded events."""
    ms = ctypes.c_float()
    driver.nbh_event_elapsed_ms(byref(ms), evtstart.handle, evtend.handle)
    return ms.value


def _stream_handle(stream):
    """0 or a Stream object (or anything with __cuda_stream__) -> raw handle
    (reference :2767-2789)."""
    if isinstance(stream, Stream):
        return stream._h
    if isinstance(stream, int) and stream == 0:
        return 0
    protocol = getattr(stream, "__cuda_stream__", None)
    if protocol is None:
        raise TypeError("Expected a Stream object or 0, got %s" % type(stream).__name__)
    version, address = protocol()
    if version != 0:
        raise TypeError("__cuda_stream__ protocol version %r is not supported" % (version,))
    return int(address)


# --------------------------------------------------------------------------------
# Pointers, extents, copies
# --------------------------------------------------------------------------------

def _plain_view(obj):
    # datetime64 / timedelta64 arrays do not export a buffer; their int64 view does
    dtype = getattr(obj, "dtype", None)
    if dtype is not None and dtype.char in "Mm":
        return obj.view(np.int64)
    return obj


def host_pointer(obj, readonly=False):
    """Address of a host buffer (reference :2537-2554 + cext/mviewbuf.c:48-70).
    Accepts an int, a NumPy array or scalar, or any buffer-protocol object."""
    if isinstance(obj, int):
        return obj
    obj = _plain_view(obj)
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
    """[begin, end) addresses a host object's data occupies."""
    obj = _plain_view(obj)
    if isinstance(obj, (np.ndarray, np.generic)):
        a = np.asarray(obj)
        return _extents(a.__array_interface__["data"][0], a.shape, a.strides, a.itemsize)
    return _hostbuf.extents(obj)


def host_memory_size(obj):
    begin, end = host_memory_extents(obj)
    if end < begin:
        raise AssertionError("memory extent of negative size")
    return end - begin


_SIZE_FROM_INFO = {}


def memory_size_from_info(shape, strides, itemsize):
    """Bytes spanned by an array with this shape and strides, gaps included."""
    key = (shape, strides, itemsize)
    try:
        return _SIZE_FROM_INFO[key]
    except KeyError:
        pass
    if len(shape) != len(strides):
        raise AssertionError("# dim mismatch")
    lo, hi = _extents(0, shape, strides, itemsize)
    if len(_SIZE_FROM_INFO) > 4096:
        _SIZE_FROM_INFO.clear()
    _SIZE_FROM_INFO[key] = hi - lo
    return hi - lo


def is_device_memory(obj):
    """Device memory is anything with a truthy __cuda_memory__ attribute."""
    return getattr(obj, "__cuda_memory__", False)


def require_device_memory(obj):
    """Raise unless `obj` is device memory."""
    if is_device_memory(obj):
        return
    raise Exception("Not a CUDA memory object.")


def device_ctypes_pointer(obj):
    """ctypes pointer of a device memory object (a null c_void_p for None)."""
    if obj is not None:
        require_device_memory(obj)
        return obj.device_ctypes_pointer
    return c_void_p(0)


def device_pointer(obj):
    """Address of a device memory object as an int."""
    return device_ctypes_pointer(obj).value


def device_extents(devmem):
    """[begin, end) of the whole allocation that `devmem` points into."""
    base, size = c_void_p(), c_size_t()
    driver.nbh_mem_address_range(byref(base), byref(size), device_ctypes_pointer(devmem).value)
    begin = base.value or 0
    return begin, begin + size.value


def device_memory_size(devmem):
    """Size of the allocation behind `devmem`; looked up once and kept on the object."""
    try:
        known = devmem._cuda_memsize_
    except AttributeError:
        known = None
    if known is None:
        begin, end = device_extents(devmem)
        known = devmem._cuda_memsize_ = end - begin
    if known < 0:
        raise AssertionError("%d length array" % known)
    return known


def device_memory_depends(devmem, *objs):
    """Keep `objs` alive as long as `devmem` lives."""
    kept = getattr(devmem, "_depends_", None)
    if kept is None:
        kept = devmem._depends_ = []
    kept.extend(objs)


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
    """See profile_start()."""


class profiling:
    """`with profiling():` - kept for source compatibility; see profile_start()."""

    def __enter__(self):
        profile_start()

    def __exit__(self, *exc):
        profile_stop()
        return False


def get_version():
    return driver.get_version()
