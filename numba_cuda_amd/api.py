"""The host API exported as `numba_cuda_amd.*`.

Same names, arguments and behaviour as numba_cuda/numba/cuda/api.py:24-591
(arrays :24-168, :211-259, :290-374; streams and events :378-481; devices
:484-567; defer_cleanup :570-586).  Every function that touches the GPU first makes
sure the calling thread has a device selected.
"""

import contextlib

import numpy as np

from numba_cuda_amd.api_util import prepare_shape_strides_dtype
from numba_cuda_amd.core import config
from numba_cuda_amd.cudadrv import devicearray, devices, driver

require_context = devices.require_context
current_context = devices.get_context
gpus = devices.gpus


def _ctx():
    return devices.get_context()


# ---- device arrays ---------------------------------------------------------------------

def device_array(shape, dtype=np.float64, strides=None, order="C", stream=0):
    """Uninitialised device array, like numpy.empty."""
    _ctx()
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    return devicearray.DeviceNDArray(shape=shape, strides=strides, dtype=dtype, stream=stream)


def to_device(obj, stream=0, copy=True, to=None):
    """Allocate a device array like `obj` and copy `obj` into it; with `to=` copy
    into that existing device array instead.  Asynchronous iff `stream` is non-zero.

        d_ary = cuda.to_device(ary)               # host -> device
        hary = d_ary.copy_to_host()               # and back
        d_ary.copy_to_host(ary, stream=stream)    # into an existing array, on a stream
    """
    _ctx()
    if to is not None:
        if copy:
            to.copy_to_device(obj, stream=stream)
        return to
    return devicearray.auto_device(obj, stream=stream, copy=copy, user_explicit=True)[0]


def _auto_device(ary, stream=0, copy=True):
    """(device array, was a copy made): what kernel launchers use for their arguments."""
    return devicearray.auto_device(ary, stream=stream, copy=copy)


def _layout_like(ary):
    """(strides, order) that give a compact array with `ary`'s shape and axis
    ordering; strides is None when plain C / F order already does."""
    order = "F" if ary.flags["F_CONTIGUOUS"] and not ary.flags["C_CONTIGUOUS"] else "C"
    return _contiguous_strides_like_array(ary), order


def _contiguous_strides_like_array(ary):
    if ary.ndim <= 1 or ary.flags["C_CONTIGUOUS"] or ary.flags["F_CONTIGUOUS"]:
        return None
    # rank the axes by stride (stable), then lay them out in that order, innermost first
    strides = [0] * ary.ndim
    step = ary.dtype.itemsize
    for axis in sorted(range(ary.ndim), key=lambda k: ary.strides[k]):
        strides[axis] = step
        step *= ary.shape[axis]
    return tuple(strides)


def _order_like_array(ary):
    return _layout_like(ary)[1]


def device_array_like(ary, stream=0):
    strides, order = _layout_like(ary)
    return device_array(shape=ary.shape, dtype=ary.dtype, strides=strides, order=order, stream=stream)


def _pinned_ndarray(shape, dtype, strides, order, **alloc_flags):
    """(ndarray over fresh page-locked host memory, the memory object)"""
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    nbytes = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    mem = _ctx().memhostalloc(nbytes, **alloc_flags)
    ary = np.ndarray(shape=shape, strides=strides, dtype=dtype, order=order, buffer=mem)
    return ary, mem


def pinned_array(shape, dtype=np.float64, strides=None, order="C"):
    """Host ndarray in page-locked memory, like numpy.empty; copies to and from it
    can be truly asynchronous."""
    return _pinned_ndarray(shape, dtype, strides, order)[0]


def pinned_array_like(ary):
    strides, order = _layout_like(ary)
    return pinned_array(shape=ary.shape, dtype=ary.dtype, strides=strides, order=order)


def mapped_array(shape, dtype=np.float64, strides=None, order="C", stream=0, portable=False, wc=False):
    """Host ndarray in page-locked memory that is also mapped into the device's
    address space; usable wherever a device array is.  `portable`: usable from
    every device; `wc`: write-combined (fast to write from the host, slow to read)."""
    ary, mem = _pinned_ndarray(shape, dtype, strides, order, mapped=True, portable=portable, wc=wc)
    out = np.ndarray.view(ary, type=devicearray.MappedNDArray)
    out.device_setup(mem, stream=stream)
    return out


def mapped_array_like(ary, stream=0, portable=False, wc=False):
    strides, order = _layout_like(ary)
    return mapped_array(shape=ary.shape, dtype=ary.dtype, strides=strides, order=order, stream=stream,
                        portable=portable, wc=wc)


def managed_array(shape, dtype=np.float64, strides=None, order="C", stream=0, attach_global=True):
    """Host ndarray in managed memory: the same address is valid on the host and on
    the device, and the array can be passed wherever a device array is.
    `attach_global=False` attaches the memory to the host only."""
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    nbytes = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    mem = _ctx().memallocmanaged(nbytes, attach_global=attach_global)
    ary = np.ndarray(shape=shape, strides=strides, dtype=dtype, order=order, buffer=mem)
    out = np.ndarray.view(ary, type=devicearray.ManagedNDArray)
    out.device_setup(mem, stream=stream)
    return out


def from_cuda_array_interface(desc, owner=None, sync=True):
    """Wrap the memory described by a __cuda_array_interface__ dict in a
    DeviceNDArray without copying; `owner` is kept alive by the result.  If the
    description carries a stream and `sync` is true, that stream is synchronised
    first (switch off globally with NUMBA_CUDA_ARRAY_INTERFACE_SYNC=0)."""
    ctx = _ctx()
    if desc.get("version") >= 1 and desc.get("mask") is not None:
        raise NotImplementedError("Masked arrays are not supported")
    shape, strides, dtype = prepare_shape_strides_dtype(desc["shape"], desc.get("strides"),
                                                        desc["typestr"], order="C")
    nbytes = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    mem = driver.MemoryPointer(ctx, desc["data"][0], size=nbytes, owner=owner)
    stream = 0
    foreign = desc.get("stream", None)
    if foreign is not None:
        stream = external_stream(foreign)
        if sync and config.CUDA_ARRAY_INTERFACE_SYNC:
            stream.synchronize()
    return devicearray.DeviceNDArray(shape=shape, strides=strides, dtype=dtype, gpu_data=mem, stream=stream)


def as_cuda_array(obj, sync=True):
    """View any object exporting __cuda_array_interface__ as a DeviceNDArray."""
    if not is_cuda_array(obj):
        raise TypeError("*obj* doesn't implement the cuda array interface.")
    return from_cuda_array_interface(obj.__cuda_array_interface__, owner=obj, sync=sync)


def is_cuda_array(obj):
    """True if `obj` exports __cuda_array_interface__ (its validity is not checked)."""
    return hasattr(obj, "__cuda_array_interface__")


@contextlib.contextmanager
def open_ipc_array(handle, shape, dtype, strides=None, offset=0):
    """Open an IPC memory handle given as its raw bytes (bytes, or a sequence of
    ints) and yield it as a device array of `shape`, `dtype` and `strides` (1-d
    C-contiguous when omitted); the mapping is closed when the block is left
    (reference api.py:263-287)."""
    dtype = np.dtype(dtype)
    size = int(np.prod(shape)) * dtype.itemsize
    ipchandle = driver.IpcHandle(None, driver.IpcMemHandle(handle), size, offset=offset)
    yield ipchandle.open_array(_ctx(), shape=shape, strides=strides, dtype=dtype)
    ipchandle.close()


@contextlib.contextmanager
def pinned(*arylist):
    "Temporarily page-lock the host arrays in `arylist`."
    ctx = _ctx()
    locks = [ctx.mempin(a, driver.host_pointer(a), driver.host_memory_size(a), mapped=False) for a in arylist]
    yield
    del locks


@contextlib.contextmanager
def mapped(*arylist, **kws):
    "Temporarily page-lock and device-map the host arrays; yields device arrays."
    assert not kws or "stream" in kws, "Only accept 'stream' as keyword."
    ctx = _ctx()
    stream = kws.get("stream", 0)
    locks = [ctx.mempin(a, driver.host_pointer(a), driver.host_memory_size(a), mapped=True) for a in arylist]
    views = [devicearray.from_array_like(a, gpu_data=lock, stream=stream) for a, lock in zip(arylist, locks)]
    try:
        yield views[0] if len(views) == 1 else views
    finally:
        # the caller's name for the yielded array outlives the with-block, so
        # unmapping cannot wait for reference counts
        for lock in locks:
            lock.free()


# ---- streams, events, synchronisation ------------------------------------------------------

def synchronize():
    "Wait for all work on the current device."
    return _ctx().synchronize()


def stream():
    "A new stream (it synchronises with the default stream, as CUDA's default flags do)."
    return _ctx().create_stream()


def default_stream():
    "The default stream; in this API that is always the legacy (synchronising) one."
    return _ctx().get_default_stream()


def legacy_default_stream():
    return _ctx().get_legacy_default_stream()


def per_thread_default_stream():
    return _ctx().get_per_thread_default_stream()


def external_stream(ptr):
    "Wrap a hipStream_t created elsewhere, given as an int."
    return _ctx().create_external_stream(ptr)


def event(timing=True):
    "A new event; `timing=False` makes it cheaper but unusable with elapsed_time."
    return _ctx().create_event(timing=timing)


event_elapsed_time = driver.event_elapsed_time


@contextlib.contextmanager
def defer_cleanup():
    """Hold every deallocation off until the (outermost) block exits, so that no free
    interrupts asynchronous work issued inside it."""
    with _ctx().defer_cleanup():
        yield


def profile_start():
    _ctx()
    driver.profile_start()


def profile_stop():
    _ctx()
    driver.profile_stop()


@contextlib.contextmanager
def profiling():
    profile_start()
    yield
    profile_stop()


# ---- devices ----------------------------------------------------------------------------------

def select_device(device_id):
    "Make `device_id` the calling thread's device; returns the Device."
    return devices.get_context(device_id).device


def get_current_device():
    return _ctx().device


def list_devices():
    return devices.gpus


def close():
    "Release every resource this package holds on every device."
    devices.reset()


def detect():
    "Print a summary of the GPUs found; returns True if any is supported."
    found = list_devices()
    print("Found %d HIP devices" % len(found))
    usable = 0
    for dev in found:
        ok = dev.WARP_SIZE == 64
        usable += ok
        print("id %d    %20s %40s" % (dev.id, dev.name, "[SUPPORTED]" if ok else "[NOT SUPPORTED: needs wave64]"))
        facts = {"Compute units": dev.MULTIPROCESSOR_COUNT, "PCI Device ID": dev.PCI_DEVICE_ID,
                 "PCI Bus ID": dev.PCI_BUS_ID, "Wavefront size": dev.WARP_SIZE}
        for key, val in facts.items():
            print("%40s: %s" % (key, val))
    print("Summary:")
    print("\t%d/%d devices are supported" % (usable, len(found)))
    return usable > 0


def is_available():
    "True if the HIP library loads and sees at least one GPU."
    return driver.driver.is_available


def cuda_error():
    "Why initialisation failed, or None."
    return driver.driver.initialization_error


def is_supported_version():
    """True if the HIP runtime is a version this package is tested with (reference:
    device_init.py:128-143; other versions may still work)."""
    from numba_cuda_amd.cudadrv.runtime import runtime
    return runtime.is_supported_version()


def is_float16_supported():
    return True


def is_bfloat16_supported():
    return True


def is_fp8_supported():
    "gfx950 has 8-bit floating-point conversions and matrix instructions (reference: api.py:108-113)."
    return True
