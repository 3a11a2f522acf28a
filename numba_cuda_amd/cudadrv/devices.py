"""Current-device management (reference: numba_cuda/numba/cuda/cudadrv/devices.py
:24-247).

The reference keeps a thread-local stack of CUDA primary contexts.  HIP's runtime
API already has one implicit context per device and a per-thread current device,
so this collapses to: remember which device each host thread selected, call
hipSetDevice when it changes, and hand out the per-device `Context` bookkeeping
object.
"""

import functools
import threading
from collections.abc import Sequence

from .driver import driver


class _DeviceList(Sequence):
    """`cuda.gpus`: the devices as a read-only sequence (index, iterate, `len()`); each
    entry is also a context manager that makes its device current inside `with`.  The
    devices are asked for on first use, not at import."""

    _entries = None

    @property
    def lst(self):
        entries = self._entries
        if entries is None:
            count = driver.get_device_count()
            entries = self._entries = [_DeviceContextManager(driver.get_device(i)) for i in range(count)]
        return entries

    def __getitem__(self, devnum):
        return self.lst[devnum]

    def __len__(self):
        return len(self.lst)

    def __str__(self):
        return ", ".join(map(str, self.lst))

    @property
    def current(self):
        """The device of the calling thread's active context, or None."""
        devnum = _runtime.current_device
        return None if devnum is None else self.lst[devnum]


class _DeviceContextManager:
    """A device that can be entered: `with cuda.gpus[i]:` selects it for the calling
    thread and goes back to the thread's earlier device on the way out.  Everything
    else is the device's own attribute."""

    def __init__(self, device):
        self._device = device
        self._came_from = threading.local()   # per host thread: the devices to go back to

    def __getattr__(self, name):
        return getattr(self._device, name)

    def __enter__(self):
        self._came_from.__dict__.setdefault("stack", []).append(_runtime.current_device)
        _runtime.get_or_create_context(self._device.id)

    def __exit__(self, *exc_info):
        earlier = self._came_from.stack.pop()
        if earlier is not None:
            _runtime.get_or_create_context(earlier)

    def __str__(self):
        return "<Managed Device %d>" % self._device.id


class _Runtime:
    """Which device each host thread uses."""

    def __init__(self):
        self.gpus = _DeviceList()
        self._tls = threading.local()
        self._lock = threading.RLock()

    @property
    def current_device(self):
        return getattr(self._tls, "devnum", None)

    def get_or_create_context(self, devnum):
        """Context of device `devnum` (None: the thread's current device, or
        device 0 when the thread has not chosen yet), made current."""
        if devnum is None:
            ctx = getattr(self._tls, "ctx", None)
            if ctx is not None and ctx.prepared:   # the common case: this thread already has a device
                return ctx
            devnum = self.current_device
            if devnum is None:
                devnum = 0
        if self.current_device != devnum:
            device = driver.get_device(devnum)   # validates devnum
            driver.nbh_set_device(devnum)
            self._tls.devnum = devnum
            self._tls.ctx = None
        else:
            device = driver.get_device(devnum)
        with self._lock:
            ctx = device.get_primary_context()
        ctx.prepare_for_use()
        self._tls.ctx = ctx
        return ctx

    def reset(self):
        """Drop every context's resources and forget the thread's device."""
        for dev in driver.list_devices() if driver.is_initialized and driver.lib else []:
            dev.reset()
        self._tls.devnum = None
        self._tls.ctx = None


_runtime = _Runtime()
gpus = _runtime.gpus


def get_context(devnum=None):
    """The context of the given device, or of the calling thread's current one."""
    return _runtime.get_or_create_context(devnum)


def require_context(fn):
    """Decorator: make sure a device is selected before `fn` runs."""

    @functools.wraps(fn)
    def _require_cuda_context(*args, **kws):
        _runtime.get_or_create_context(None)
        return fn(*args, **kws)

    return _require_cuda_context


def reset():
    _runtime.reset()
