"""Device arrays: n-d views over device memory with NumPy-like shape algebra and
host <-> device copies.

Public names, signatures and error texts are those of
numba_cuda/numba/cuda/cudadrv/devicearray.py (DeviceNDArrayBase :60-429,
DeviceRecord :432-531, DeviceNDArray :578-790, helpers :858-961,
check_array_compatibility :1104-1119), so that code written against the reference
keeps working.  An object is device memory if it has a truthy `__cuda_memory__`;
it is a device array if it also has `__cuda_ndarray__`, `shape`, `strides`,
`dtype` and `size`.

How it is put together here: a device array is a `dummyarray.Array` (where the
items are) plus a counted reference to a `MemoryPointer` (what keeps them alive)
plus a default stream.  Every view-producing operation asks the layout object for
the new layout and re-wraps the same memory; nothing but `copy_to_*`, element
access and `__setitem__` ever touches the device.
"""

import copy
import ctypes
import functools
import math
from ctypes import c_void_p
from warnings import warn

import numpy as np

from numba_cuda_amd.core import config
from numba_cuda_amd.core.errors import NumbaPerformanceWarning
from numba_cuda_amd.api_util import prepare_shape_strides_dtype
from . import devices, dummyarray
from . import driver as _driver

_MAX_ASSIGN_NDIM = 8     # NBH_ASSIGN_MAX_NDIM of the C ABI

errmsg_contiguous_buffer = ("Array contains non-contiguous buffer and cannot "
                            "be transferred as a single memory region. Please "
                            "ensure contiguous buffer with numpy "
                            ".ascontiguousarray()")


# ---- small predicates ----------------------------------------------------------------

def is_cuda_ndarray(obj):
    "True for objects that declare themselves device ndarrays"
    return getattr(obj, "__cuda_ndarray__", False)


def require_cuda_ndarray(obj):
    "ValueError unless `obj` is a device ndarray"
    if not is_cuda_ndarray(obj):
        raise ValueError("require an cuda ndarray object")


def verify_cuda_ndarray_interface(obj):
    "Check that `obj` carries the attributes a device ndarray must have"
    require_cuda_ndarray(obj)
    wanted = {"shape": tuple, "strides": tuple, "dtype": np.dtype, "size": int}
    for attr, typ in wanted.items():
        if not hasattr(obj, attr):
            raise AttributeError(attr)
        if not isinstance(getattr(obj, attr), typ):
            raise AttributeError("%s must be of type %s" % (attr, typ))


def is_contiguous(ary):
    """C-contiguity of `ary` when broadcast (stride 0) and length-1 axes are left
    out of the picture."""
    expect = ary.dtype.itemsize
    for n, stride in zip(ary.shape[::-1], ary.strides[::-1]):
        if n > 1 and stride != 0:
            if stride != expect:
                return False
            expect *= n
    return True


def array_core(ary):
    """The part of a broadcast array that really exists in memory: index 0 along
    every zero-stride axis.  Contiguity and copies are decided on this core."""
    if not ary.strides or not ary.size or 0 not in ary.strides:
        return ary          # nothing is repeated: the array is its own core
    picks = [slice(None) if stride else 0 for stride in ary.strides]
    return ary[tuple(picks)]


def sentry_contiguous(ary):
    flags = array_core(ary).flags
    if not (flags["C_CONTIGUOUS"] or flags["F_CONTIGUOUS"]):
        raise ValueError(errmsg_contiguous_buffer)


def check_array_compatibility(ary1, ary2):
    """Raise unless a raw byte copy between the two arrays is meaningful: same
    dtype, and same shape and strides once length-1 axes are dropped."""
    if ary1.dtype != ary2.dtype:
        raise TypeError("incompatible dtype: %s vs. %s" % (ary1.dtype, ary2.dtype))
    if ary1.shape == ary2.shape and (ary1.strides == ary2.strides or not ary1.size):
        return              # the common case needs no squeezed views
    sq1, sq2 = ary1.squeeze(), ary2.squeeze()
    if sq1.shape != sq2.shape:
        raise ValueError("incompatible shape: %s vs. %s" % (ary1.shape, ary2.shape))
    # strides of an empty copy are irrelevant (and may legitimately differ)
    if ary1.size and sq1.strides != sq2.strides:
        raise ValueError("incompatible strides: %s vs. %s" % (ary1.strides, ary2.strides))


def _normalise_shape(shape):
    if isinstance(shape, int):
        return (shape,)
    out = []
    for s in shape:
        if not isinstance(s, (int, np.integer)):
            raise TypeError("shape elements must be integers, got %s" % type(s).__name__)
        out.append(int(s))
    return tuple(out)


# ---- the array types -------------------------------------------------------------------

_FILL_ITEMSIZES = (1, 2, 4, 8, 16)   # what nbh_fill takes by value


@functools.lru_cache(maxsize=1024)
def _layout_of(shape, strides, itemsize):
    """The stride calculus object for an array that starts at offset 0.  Layout objects
    are never modified, so arrays of the same shape and strides share one."""
    return dummyarray.Array.from_desc(0, shape, strides, itemsize)


class DeviceNDArrayBase:
    """An n-d array in device memory."""

    __cuda_memory__ = True
    __cuda_ndarray__ = True   # promises a gpu_data attribute

    def __init__(self, shape, strides, dtype, stream=0, gpu_data=None):
        """
        shape, strides : ints or sequences of ints (strides in bytes)
        dtype          : anything np.dtype accepts
        stream         : default stream for operations on this array
        gpu_data       : existing device memory to wrap; allocated when None
        """
        shape = _normalise_shape(shape)
        if isinstance(strides, int):
            strides = (strides,)
        elif strides:
            strides = tuple(strides)
        self.dtype = np.dtype(dtype)
        self.ndim = len(shape)
        if len(strides) != self.ndim:
            raise ValueError("strides not match ndim")
        layout = _layout_of(shape, strides, self.dtype.itemsize)
        self._dummy = layout
        self.shape, self.strides, self.size = layout.shape, layout.strides, layout.size
        if self.size == 0:
            # nothing to hold: a NULL pointer of size 0, whatever was passed in
            self.alloc_size = 0
            gpu_data = _driver.MemoryPointer(context=devices.get_context(), pointer=0, size=0)
        else:
            self.alloc_size = _driver.memory_size_from_info(self.shape, self.strides, self.dtype.itemsize)
            if gpu_data is None:
                gpu_data = devices.get_context().memalloc(self.alloc_size)
        self.gpu_data = gpu_data
        self.stream = stream

    # -- identity ---------------------------------------------------------------------
    @property
    def device_ctypes_pointer(self):
        """ctypes integer holding the device address of item [0, ..., 0]"""
        data = self.gpu_data
        return data.device_ctypes_pointer if hasattr(data, "device_ctypes_pointer") else c_void_p(0)

    @property
    def __cuda_array_interface__(self):
        # whoever reads this is about to use the memory outside this package: launches still
        # waiting in a launching thread's queue (kernels/reduction.py launch_threads) go first
        lib = _driver.driver.lib if _driver.driver.is_initialized else None
        if getattr(lib, "_launch_threads", False):
            lib.nbh_launch_threads_wait(None)
        return {
            "shape": self.shape,
            "strides": None if is_contiguous(self) else tuple(self.strides),
            "data": (self.device_ctypes_pointer.value or 0, False),
            "typestr": self.dtype.str,
            "stream": int(self.stream) if self.stream != 0 else None,
            "version": 3,
        }

    @property
    def nbytes(self):
        # bytes of the items, not of the (possibly gappy) allocation
        return self.size * self.dtype.itemsize

    def as_cuda_arg(self):
        return self.gpu_data

    def get_ipc_handle(self):
        """An IpcArrayHandle - the memory manager's IPC handle for this allocation plus
        the array's layout - that another process can open as a device array
        (reference :331-340)."""
        handle = devices.get_context().get_ipc_handle(self.gpu_data)
        return IpcArrayHandle(ipc_handle=handle, array_desc=dict(shape=self.shape, strides=self.strides,
                                                                 dtype=self.dtype))

    def _default_stream(self, stream):
        return stream if stream else self.stream

    def _rewrap(self, layout, stream=None, data=None):
        """The same memory (or `data`) seen through another layout."""
        return DeviceNDArray(shape=layout.shape, strides=layout.strides, dtype=self.dtype,
                             stream=self.stream if stream is None else stream,
                             gpu_data=self.gpu_data if data is None else data)

    def bind(self, stream=0):
        """A shallow copy of this array whose default stream is `stream`."""
        twin = copy.copy(self)
        twin.stream = stream
        return twin

    # -- transposition ------------------------------------------------------------------
    @property
    def T(self):
        return self.transpose()

    def transpose(self, axes=None):
        if axes and tuple(axes) == tuple(range(self.ndim)):
            return self
        if self.ndim != 2:
            raise NotImplementedError("transposing a non-2D DeviceNDArray isn't supported")
        if axes is not None and set(axes) != set(range(self.ndim)):
            raise ValueError("invalid axes list %r" % (axes,))
        from numba_cuda_amd.kernels.transpose import transpose as device_transpose
        return device_transpose(self)

    # -- copies -------------------------------------------------------------------------
    def copy_to_device(self, ary, stream=0):
        """Copy `ary` into this array: device-to-device if `ary` is device memory,
        host-to-device otherwise.  Asynchronous iff a non-zero stream is in play."""
        if ary.size == 0:
            return
        devices.get_context()
        sentry_contiguous(self)
        stream = self._default_stream(stream)
        mine, theirs = array_core(self), array_core(ary)
        if _driver.is_device_memory(ary):
            sentry_contiguous(ary)
            check_array_compatibility(mine, theirs)
            _driver.device_to_device(self, ary, self.alloc_size, stream=stream)
            return
        # lay the host data out like this array; NumPy copies only if it has to
        order = "C" if mine.flags["C_CONTIGUOUS"] else "F"
        theirs = np.array(theirs, order=order, subok=True, copy=None)
        check_array_compatibility(mine, theirs)
        _driver.host_to_device(self, theirs, self.alloc_size, stream=stream)

    def copy_to_host(self, ary=None, stream=0):
        """Copy this array into `ary` (or a new ndarray) and return the host array.
        Synchronous unless a non-zero stream is given or bound."""
        if min(self.strides, default=0) < 0:
            raise NotImplementedError(
                "D->H copy not implemented for negative strides: {}".format(self.strides))
        assert self.alloc_size >= 0, "Negative memory size"
        devices.get_context()
        stream = self._default_stream(stream)
        if ary is not None:
            check_array_compatibility(self, ary)
            if self.alloc_size:
                _driver.device_to_host(ary, self, self.alloc_size, stream=stream)
            return ary
        # fetch the raw extent, then look at it with this array's shape and strides
        raw = np.empty(self.alloc_size, dtype=np.byte)
        if self.alloc_size:
            _driver.device_to_host(raw, self, self.alloc_size, stream=stream)
        if self.size == 0:
            return np.ndarray(shape=self.shape, dtype=self.dtype, buffer=raw)
        return np.ndarray(shape=self.shape, dtype=self.dtype, strides=self.strides, buffer=raw)

    # -- views ----------------------------------------------------------------------------
    def split(self, section, stream=0):
        """Yield consecutive 1-d views of `section` items (the last may be shorter)."""
        stream = self._default_stream(stream)
        if self.ndim != 1:
            raise ValueError("only support 1d array")
        itemsize = self.dtype.itemsize
        if self.strides[0] != itemsize:
            raise ValueError("only support unit stride")
        for k in range(int(math.ceil(float(self.size) / section))):
            lo, hi = k * section, min((k + 1) * section, self.size)
            yield DeviceNDArray((hi - lo,), self.strides, dtype=self.dtype, stream=stream,
                                gpu_data=self.gpu_data.view(lo * itemsize, hi * itemsize))

    def squeeze(self, axis=None, stream=0):
        """View without the length-1 axes (all of them, or those in `axis`)."""
        layout, _ = self._dummy.squeeze(axis=axis)
        return self._rewrap(layout, stream=self._default_stream(stream))

    def view(self, dtype):
        """Reinterpret the bytes as another dtype without copying."""
        dtype = np.dtype(dtype)
        shape, strides = list(self.shape), list(self.strides)
        old, new = self.dtype.itemsize, dtype.itemsize
        if old != new:
            if not self.is_c_contiguous():
                raise ValueError("To change to a dtype of a different size,"
                                 " the array must be C-contiguous")
            shape[-1], leftover = divmod(shape[-1] * old, new)
            if leftover:
                raise ValueError("When changing to a larger dtype,"
                                 " its size must be a divisor of the total size in bytes"
                                 " of the last axis of the array.")
            strides[-1] = new
        return DeviceNDArray(shape=shape, strides=strides, dtype=dtype, stream=self.stream,
                             gpu_data=self.gpu_data)


class DeviceRecord(DeviceNDArrayBase):
    """One structured item in device memory."""

    def __init__(self, dtype, stream=0, gpu_data=None):
        super().__init__((), (), dtype, stream, gpu_data)

    @property
    def flags(self):
        return dict(self._dummy.flags)

    def getitem(self, item, stream=0):
        """`self[item]` on a given stream: a field as NumPy scalar, nested record or
        sub-array view."""
        devices.get_context()
        stream = self._default_stream(stream)
        field_type, offset = self.dtype.fields[item]
        field_mem = self.gpu_data.view(offset)
        if field_type.shape:
            shape, strides, base = prepare_shape_strides_dtype(field_type.shape, None,
                                                               field_type.subdtype[0], "C")
            return DeviceNDArray(shape=shape, strides=strides, dtype=base, gpu_data=field_mem, stream=stream)
        if field_type.names is not None:
            return DeviceRecord(dtype=field_type, stream=stream, gpu_data=field_mem)
        host = np.empty(1, dtype=field_type)
        _driver.device_to_host(dst=host, src=field_mem, size=field_type.itemsize, stream=stream)
        return host[0]

    def __getitem__(self, item):
        return self.getitem(item)

    _do_getitem = getitem

    def setitem(self, key, value, stream=0):
        """`self[key] = value` on a given stream (waits unless a stream is in play)."""
        devices.get_context()
        stream = self._default_stream(stream)
        wait = not stream
        if wait:
            stream = devices.get_context().get_default_stream()
        field_type, offset = self.dtype.fields[key]
        target = type(self)(dtype=field_type, stream=stream, gpu_data=self.gpu_data.view(offset))
        if target.dtype.itemsize in _FILL_ITEMSIZES and not target.dtype.fields and not target.dtype.shape:
            item = np.asarray(value).astype(target.dtype).reshape(1)
            none = (ctypes.c_int64 * 1)(0)
            _driver.driver.nbh_fill(target.device_ctypes_pointer.value, 0, none, none, target.dtype.itemsize,
                                    item.ctypes.data, _driver._stream_handle(stream) or None)
        else:
            source, _ = auto_device(target.dtype.type(value), stream=stream)
            _driver.device_to_device(target, source, source.dtype.itemsize, stream)
        if wait:
            stream.synchronize()

    def __setitem__(self, key, value):
        self.setitem(key, value)

    _do_setitem = setitem


class DeviceNDArray(DeviceNDArrayBase):
    """An array in device memory."""

    # -- layout queries -------------------------------------------------------------------
    @property
    def flags(self):
        # a plain dict: NumPy's flags object cannot be built without an ndarray
        return dict(self._dummy.flags)

    def is_c_contiguous(self):
        return self._dummy.is_c_contig

    def is_f_contiguous(self):
        return self._dummy.is_f_contig

    def __len__(self):
        return self.shape[0]

    def __array__(self, dtype=None, copy=None):
        """Copies to the host; `copy=False` cannot be honoured."""
        if copy is False:
            raise ValueError("`copy=False` is not supported. A copy is always created.")
        host = self.copy_to_host()
        return host.__array__(dtype) if dtype else host.__array__()

    # -- shape changes --------------------------------------------------------------------
    def _same_memory_or_refuse(self, layout, extents, stream=0):
        if extents != [self._dummy.extent]:
            raise NotImplementedError("operation requires copying")
        return type(self)(shape=layout.shape, strides=layout.strides, dtype=self.dtype,
                          gpu_data=self.gpu_data, stream=stream)

    def reshape(self, *newshape, **kws):
        """Reshape without moving data, like numpy.ndarray.reshape; raises
        NotImplementedError when that is impossible."""
        if len(newshape) == 1 and isinstance(newshape[0], (tuple, list)):
            newshape = newshape[0]
        if newshape == self.shape:
            return type(self)(shape=self.shape, strides=self.strides, dtype=self.dtype,
                              gpu_data=self.gpu_data)
        layout, extents = self._dummy.reshape(*newshape, **kws)
        return self._same_memory_or_refuse(layout, extents)

    def ravel(self, order="C", stream=0):
        """Flatten a contiguous array without moving data."""
        layout, extents = self._dummy.ravel(order=order)
        return self._same_memory_or_refuse(layout, extents, stream=self._default_stream(stream))

    # -- indexing ---------------------------------------------------------------------------
    def getitem(self, item, stream=0):
        """`self[item]` on a given stream: a view for slices, a NumPy scalar (one
        blocking copy) or a DeviceRecord for a fully indexed item."""
        devices.get_context()
        stream = self._default_stream(stream)
        picked = self._dummy[item]
        # the view starts at the selection's first item and spans to its last;
        # shape and strides say what lies in between
        mem = self.gpu_data.view(*picked.extent)
        if picked.is_array:
            return type(self)(shape=picked.shape, strides=picked.strides, dtype=self.dtype,
                              gpu_data=mem, stream=stream)
        if self.dtype.names is not None:
            return DeviceRecord(dtype=self.dtype, stream=stream, gpu_data=mem)
        host = np.empty(1, dtype=self.dtype)
        _driver.device_to_host(dst=host, src=mem, size=self.dtype.itemsize, stream=stream)
        return host[0]

    def __getitem__(self, item):
        return self.getitem(item)

    _do_getitem = getitem

    def setitem(self, key, value, stream=0):
        """`self[key] = value` on a given stream.  `value` may be a scalar, a host
        array or a device array and is broadcast NumPy-style (missing leading axes,
        unit axes).  Waits for completion unless a stream is given or bound."""
        devices.get_context()
        stream = self._default_stream(stream)
        wait = not stream
        if wait:
            stream = devices.get_context().get_default_stream()

        # left-hand side: a view of the selected items (0-d for a single item)
        picked = self._dummy[key]
        mem = self.gpu_data.view(*picked.extent)
        shape, strides = (picked.shape, picked.strides) if picked.is_array else ((), ())
        lhs = type(self)(shape=shape, strides=strides, dtype=self.dtype, gpu_data=mem, stream=stream)

        # right-hand side: on the device, padded with leading unit axes
        if not _driver.is_device_memory(value) and not hasattr(value, "__cuda_array_interface__"):
            # host values take the dtype of the target, as a NumPy assignment would
            value = np.asarray(value).astype(self.dtype, copy=False)
            if value.size == 1 and value.ndim <= lhs.ndim and self.dtype.itemsize in _FILL_ITEMSIZES:
                # one item: it travels as a kernel argument, no device-side source needed
                if lhs.ndim > _MAX_ASSIGN_NDIM:
                    raise NotImplementedError("assignment supports at most %d axes" % _MAX_ASSIGN_NDIM)
                item = np.ascontiguousarray(value).reshape(1)
                vec = ctypes.c_int64 * max(lhs.ndim, 1)
                _driver.driver.nbh_fill(lhs.device_ctypes_pointer.value, lhs.ndim, vec(*lhs.shape),
                                        vec(*lhs.strides), self.dtype.itemsize, item.ctypes.data,
                                        _driver._stream_handle(stream) or None)
                if wait:
                    stream.synchronize()
                return
        rhs, _ = auto_device(value, stream=stream, user_explicit=True)
        if rhs.ndim > lhs.ndim:
            raise ValueError("Can't assign %s-D array to %s-D self" % (rhs.ndim, lhs.ndim))
        if rhs.dtype != lhs.dtype:
            raise TypeError("incompatible dtype: %s vs. %s" % (lhs.dtype, rhs.dtype))
        pad = lhs.ndim - rhs.ndim
        rhs_shape = (1,) * pad + tuple(rhs.shape)
        rhs_strides = (0,) * pad + tuple(rhs.strides)
        for axis, (want, have) in enumerate(zip(lhs.shape, rhs_shape)):
            if have != 1 and have != want:
                raise ValueError("Can't copy sequence with size %d to array "
                                 "axis %d with dimension %d" % (have, axis, want))
        # a unit axis on the right repeats along the matching axis on the left
        src_strides = tuple(0 if n == 1 else s for n, s in zip(rhs_shape, rhs_strides))

        if lhs.ndim > _MAX_ASSIGN_NDIM:
            raise NotImplementedError("assignment supports at most %d axes" % _MAX_ASSIGN_NDIM)
        vec = ctypes.c_int64 * max(lhs.ndim, 1)
        _driver.driver.nbh_assign(lhs.device_ctypes_pointer.value, rhs.device_ctypes_pointer.value,
                                  lhs.ndim, vec(*lhs.shape), vec(*lhs.strides), vec(*src_strides),
                                  self.dtype.itemsize, _driver._stream_handle(stream) or None)
        if wait:
            stream.synchronize()

    def __setitem__(self, key, value):
        self.setitem(key, value)

    _do_setitem = setitem


class IpcArrayHandle:
    """What get_ipc_handle() returns: the memory manager's handle plus the array
    layout; open() in another process yields a DeviceNDArray over the shared memory
    (reference :793-835)."""

    def __init__(self, ipc_handle, array_desc):
        self._array_desc = array_desc
        self._ipc_handle = ipc_handle

    def open(self):
        shared = self._ipc_handle.open(devices.get_context())
        return DeviceNDArray(gpu_data=shared, **self._array_desc)

    def close(self):
        self._ipc_handle.close()

    def __enter__(self):
        return self.open()

    def __exit__(self, exc_type, exc, tb):
        self.close()


class _HostVisibleArray(DeviceNDArrayBase, np.ndarray):
    """An ndarray whose buffer the device can address too.  It is created as a view of
    a plain ndarray (so DeviceNDArrayBase.__init__ never runs) and told its memory
    with device_setup(); NumPy views of it (slices, reshapes) find their own device
    range from the parent's."""

    gpu_data = None
    stream = 0

    def device_setup(self, gpu_data, stream=0):
        self.gpu_data = gpu_data
        self.stream = stream

    def __array_finalize__(self, parent):
        data = getattr(parent, "gpu_data", None)
        if data is None or not isinstance(parent, _HostVisibleArray):
            return
        start = self.__array_interface__["data"][0] - parent.__array_interface__["data"][0]
        if 0 <= start <= data.size:
            self.gpu_data = data.view(start) if start else data
            self.stream = parent.stream

    @property
    def _dummy(self):
        return _layout_of(tuple(self.shape), tuple(self.strides), self.dtype.itemsize)

    @property
    def alloc_size(self):
        return _driver.memory_size_from_info(self.shape, self.strides, self.dtype.itemsize)


class MappedNDArray(_HostVisibleArray):
    """A host array in pinned memory that the device can address."""


class ManagedNDArray(_HostVisibleArray):
    """A host array in managed memory (reference :848-855)."""


# ---- constructors from host objects ------------------------------------------------------

def from_array_like(ary, stream=0, gpu_data=None):
    "A DeviceNDArray with the shape, strides and dtype of `ary`."
    return DeviceNDArray(ary.shape, ary.strides, ary.dtype, stream=stream, gpu_data=gpu_data)


def from_record_like(rec, stream=0, gpu_data=None):
    "A DeviceRecord with the dtype of `rec`."
    return DeviceRecord(rec.dtype, stream=stream, gpu_data=gpu_data)


def auto_device(obj, stream=0, copy=True, user_explicit=False):
    """Return (device object, created?) for `obj`: device memory passes through,
    objects exporting __cuda_array_interface__ are wrapped without copying,
    anything else is turned into an ndarray and (optionally) copied over."""
    if _driver.is_device_memory(obj):
        return obj, False
    if hasattr(obj, "__cuda_array_interface__"):
        from numba_cuda_amd.api import from_cuda_array_interface
        return from_cuda_array_interface(obj.__cuda_array_interface__, owner=obj), False
    if isinstance(obj, np.void):
        target = from_record_like(obj, stream=stream)
    else:
        obj = np.array(obj, copy=None, subok=True)
        sentry_contiguous(obj)
        target = from_array_like(obj, stream=stream)
    if copy:
        implicit = not user_explicit and isinstance(obj, np.ndarray)
        if implicit and config.CUDA_WARN_ON_IMPLICIT_COPY and not config.DISABLE_PERFORMANCE_WARNINGS:
            warn(NumbaPerformanceWarning("Host array used in CUDA kernel will incur "
                                         "copy overhead to/from device."))
        target.copy_to_device(obj, stream=stream)
    return target, True
