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

from .driver import driver


class _DeviceList:
    """`cuda.gpus`: indexable, iterable, `len()`-able list of devices; each entry
    is also a context manager that makes the device current inside `with`."""

    def __getattr__(self, attr):
        if attr == "lst":
            lst = [_DeviceContextManager(driver.get_device(i)) for i in range(driver.get_device_count())]
            self.lst = lst
            return lst
        raise AttributeError(attr)

    def __getitem__(self, devnum):
        return self.lst[devnum]

    def __str__(self):
        return ", ".join(str(d) for d in self.lst)

    def __iter__(self):
        return iter(self.lst)

    def __len__(self):
        return len(self.lst)

    @property
    def current(self):
        """The device of the calling thread's active context, or None."""
        devnum = _runtime.current_device
        return None if devnum is None else self.lst[devnum]


class _DeviceContextManager:
    def __init__(self, device):
        self._device = device

    def __getattr__(self, item):
        return getattr(self._device, item)

    def __enter__(self):
        self._previous = _runtime.current_device
        _runtime.get_or_create_context(self._device.id)

    def __exit__(self, exc_type, exc_val, exc_tb):
        if self._previous is not None:
            _runtime.get_or_create_context(self._previous)

    def __str__(self):
        return "<Managed Device {self.id}>".format(self=self)


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
