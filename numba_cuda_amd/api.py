"""The host API exported as `numba_cuda_amd.*` (reference:
numba_cuda/numba/cuda/api.py:24-591)."""

import contextlib

import numpy as np

from numba_cuda_amd.api_util import prepare_shape_strides_dtype
from numba_cuda_amd.core import config
from numba_cuda_amd.cudadrv import devicearray, devices, driver

require_context = devices.require_context
current_context = devices.get_context
gpus = devices.gpus


# ---- arrays ------------------------------------------------------------------------

@require_context
def from_cuda_array_interface(desc, owner=None, sync=True):
    """Wrap the memory described by a __cuda_array_interface__ dict in a
    DeviceNDArray without copying; `owner` is kept alive by the result.  If the
    description carries a stream and `sync` is true, that stream is synchronised
    first (switch off globally with NUMBA_CUDA_ARRAY_INTERFACE_SYNC=0)."""
    version = desc.get("version")
    if 1 <= version and desc.get("mask") is not None:
        raise NotImplementedError("Masked arrays are not supported")
    shape, strides, dtype = prepare_shape_strides_dtype(
        desc["shape"], desc.get("strides"), desc["typestr"], order="C")
    size = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    data = driver.MemoryPointer(current_context(), desc["data"][0], size=size, owner=owner)
    stream_ptr = desc.get("stream", None)
    if stream_ptr is not None:
        stream = external_stream(stream_ptr)
        if sync and config.CUDA_ARRAY_INTERFACE_SYNC:
            stream.synchronize()
    else:
        stream = 0
    return devicearray.DeviceNDArray(shape=shape, strides=strides, dtype=dtype, gpu_data=data,
                                     stream=stream)


def as_cuda_array(obj, sync=True):
    """View any object exporting __cuda_array_interface__ as a DeviceNDArray."""
    interface = getattr(obj, "__cuda_array_interface__", None)
    if interface is None:
        raise TypeError("*obj* doesn't implement the cuda array interface.")
    return from_cuda_array_interface(interface, owner=obj, sync=sync)


def is_cuda_array(obj):
    return hasattr(obj, "__cuda_array_interface__")


@require_context
def to_device(obj, stream=0, copy=True, to=None):
    """Allocate a device array like `obj` and copy `obj` into it; with `to=` copy
    into an existing device array instead.  Asynchronous iff `stream` is non-zero."""
    if to is None:
        to, _ = devicearray.auto_device(obj, stream=stream, copy=copy, user_explicit=True)
        return to
    if copy:
        to.copy_to_device(obj, stream=stream)
    return to


@require_context
def device_array(shape, dtype=np.float64, strides=None, order="C", stream=0):
    """Uninitialised device array, like numpy.empty."""
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    return devicearray.DeviceNDArray(shape=shape, strides=strides, dtype=dtype, stream=stream)


@require_context
def pinned_array(shape, dtype=np.float64, strides=None, order="C"):
    """Host ndarray in page-locked memory, like numpy.empty."""
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    bytesize = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    mem = current_context().memhostalloc(bytesize)
    return np.ndarray(shape=shape, strides=strides, dtype=dtype, order=order, buffer=mem.as_buffer())


@require_context
def mapped_array(shape, dtype=np.float64, strides=None, order="C", stream=0, portable=False, wc=False):
    """Host ndarray in page-locked memory that is also mapped into the device's
    address space; usable wherever a device array is."""
    shape, strides, dtype = prepare_shape_strides_dtype(shape, strides, dtype, order)
    bytesize = driver.memory_size_from_info(shape, strides, dtype.itemsize)
    mem = current_context().memhostalloc(bytesize, mapped=True, portable=portable, wc=wc)
    npary = np.ndarray(shape=shape, strides=strides, dtype=dtype, order=order, buffer=mem.as_buffer())
    mappedview = np.ndarray.view(npary, type=devicearray.MappedNDArray)
    mappedview.device_setup(mem, stream=stream)
    return mappedview


def synchronize():
    "Wait for all work on the current device."
    return current_context().synchronize()


def _contiguous_strides_like_array(ary):
    """Strides of a compact array with `ary`'s shape and axis ordering, or None if
    plain C / F strides already do."""
    if ary.flags["C_CONTIGUOUS"] or ary.flags["F_CONTIGUOUS"] or ary.ndim <= 1:
        return None
    # rank axes by stride (stable), then lay them out in that order, innermost first
    ranked = sorted(range(ary.ndim), key=lambda k: ary.strides[k])
    strides = [0] * ary.ndim
    step = ary.dtype.itemsize
    for k in ranked:
        strides[k] = step
        step *= ary.shape[k]
    return tuple(strides)


def _order_like_array(ary):
    return "F" if ary.flags["F_CONTIGUOUS"] and not ary.flags["C_CONTIGUOUS"] else "C"


def device_array_like(ary, stream=0):
    return device_array(shape=ary.shape, dtype=ary.dtype, strides=_contiguous_strides_like_array(ary),
                        order=_order_like_array(ary), stream=stream)


def mapped_array_like(ary, stream=0, portable=False, wc=False):
    return mapped_array(shape=ary.shape, dtype=ary.dtype, strides=_contiguous_strides_like_array(ary),
                        order=_order_like_array(ary), stream=stream, portable=portable, wc=wc)


def pinned_array_like(ary):
    return pinned_array(shape=ary.shape, dtype=ary.dtype, strides=_contiguous_strides_like_array(ary),
                        order=_order_like_array(ary))


# ---- streams and events --------------------------------------------------------------

@require_context
def stream():
    "A new stream (it synchronises with the default stream, as CUDA's default flags do)."
    return current_context().create_stream()


@require_context
def default_stream():
    return current_context().get_default_stream()


@require_context
def legacy_default_stream():
    return current_context().get_legacy_default_stream()


@require_context
def per_thread_default_stream():
    return current_context().get_per_thread_default_stream()


@require_context
def external_stream(ptr):
    "Wrap a hipStream_t created elsewhere, given as an int."
    return current_context().create_external_stream(ptr)


@require_context
@contextlib.contextmanager
def pinned(*arylist):
    "Temporarily page-lock the host arrays in `arylist`."
    pmlist = []
    for ary in arylist:
        pmlist.append(current_context().mempin(ary, driver.host_pointer(ary),
                                               driver.host_memory_size(ary), mapped=False))
    yield
    del pmlist


@require_context
@contextlib.contextmanager
def mapped(*arylist, **kws):
    "Temporarily page-lock and device-map the host arrays; yields device arrays."
    assert not kws or "stream" in kws, "Only accept 'stream' as keyword."
    stream = kws.get("stream", 0)
    pmlist, devarylist = [], []
    for ary in arylist:
        pm = current_context().mempin(ary, driver.host_pointer(ary), driver.host_memory_size(ary),
                                      mapped=True)
        pmlist.append(pm)
        devarylist.append(devicearray.from_array_like(ary, gpu_data=pm, stream=stream))
    try:
        yield devarylist[0] if len(devarylist) == 1 else devarylist
    finally:
        # the caller's name for the yielded array outlives the with-block, so
        # unmapping cannot wait for reference counts
        for pm in pmlist:
            pm.free()


def event(timing=True):
    "A new event; `timing=False` makes it cheaper but unusable with elapsed_time."
    return current_context().create_event(timing=timing)


event_elapsed_time = driver.event_elapsed_time


# ---- devices ------------------------------------------------------------------------

def select_device(device_id):
    "Make `device_id` the calling thread's device; returns the Device."
    return devices.get_context(device_id).device


def get_current_device():
    return current_context().device


def list_devices():
    return devices.gpus


def close():
    "Release every resource this package holds on every device."
    devices.reset()


def detect():
    "Print a summary of the GPUs found; returns True if any is supported."
    devlist = list_devices()
    print("Found %d HIP devices" % len(devlist))
    supported = 0
    for dev in devlist:
        ok = dev.WARP_SIZE == 64
        supported += ok
        print("id %d    %20s %40s" % (dev.id, dev.name, "[SUPPORTED]" if ok else "[NOT SUPPORTED: needs wave64]"))
        for key, val in (("Compute units", dev.MULTIPROCESSOR_COUNT), ("PCI Device ID", dev.PCI_DEVICE_ID),
                         ("PCI Bus ID", dev.PCI_BUS_ID), ("Wavefront size", dev.WARP_SIZE)):
            print("%40s: %s" % (key, val))
    print("Summary:")
    print("\t%d/%d devices are supported" % (supported, len(devlist)))
    return supported > 0


@contextlib.contextmanager
def defer_cleanup():
    "Hold every deallocation off until the (outermost) block exits."
    with current_context().defer_cleanup():
        yield


profiling = require_context(driver.profiling)
profile_start = require_context(driver.profile_start)
profile_stop = require_context(driver.profile_stop)


def is_available():
    "True if the HIP library loads and sees at least one GPU."
    return driver.driver.is_available


def cuda_error():
    "Why initialisation failed, or None."
    return driver.driver.initialization_error


def is_float16_supported():
    return True


def is_bfloat16_supported():
    return True
