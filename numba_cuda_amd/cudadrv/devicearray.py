"""Device arrays: n-d views over device memory with NumPy-like shape algebra and
host <-> device copies.

API and error behaviour follow numba_cuda/numba/cuda/cudadrv/devicearray.py
(DeviceNDArrayBase :60-429, DeviceRecord :432-531, DeviceNDArray :578-790,
helpers :858-961, check_array_compatibility :1104-1119).  An object is device
memory if it has a truthy `__cuda_memory__`; it is a device array if it also has
`__cuda_ndarray__`, `shape`, `strides`, `dtype` and `size`.
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


def is_cuda_ndarray(obj):
    "Check if an object is a device ndarray"
    return getattr(obj, "__cuda_ndarray__", False)


def verify_cuda_ndarray_interface(obj):
    "Verify the device ndarray interface for an obj"
    require_cuda_ndarray(obj)
    for attr, typ in (("shape", tuple), ("strides", tuple), ("dtype", np.dtype), ("size", int)):
        if not hasattr(obj, attr):
            raise AttributeError(attr)
        if not isinstance(getattr(obj, attr), typ):
            raise AttributeError("%s must be of type %s" % (attr, typ))


def require_cuda_ndarray(obj):
    "Raises ValueError if is_cuda_ndarray(obj) evaluates False"
    if not is_cuda_ndarray(obj):
        raise ValueError("require an cuda ndarray object")


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
        if isinstance(shape, int):
            shape = (shape,)
        else:
            for s in shape:
                if not isinstance(s, (int, np.integer)):
                    raise TypeError("shape elements must be integers, got %s" % type(s).__name__)
            shape = tuple(int(s) for s in shape)
        if isinstance(strides, int):
            strides = (strides,)
        elif strides:
            strides = tuple(strides)
        dtype = np.dtype(dtype)
        self.ndim = len(shape)
        if len(strides) != self.ndim:
            raise ValueError("strides not match ndim")
        self._dummy = dummy = dummyarray.Array.from_desc(0, shape, strides, dtype.itemsize)
        self.shape = dummy.shape
        self.strides = dummy.strides
        self.dtype = dtype
        self.size = dummy.size
        if self.size:
            self.alloc_size = _driver.memory_size_from_info(self.shape, self.strides, dtype.itemsize)
            if gpu_data is None:
                gpu_data = devices.get_context().memalloc(self.alloc_size)
        else:
            # empty arrays own a NULL pointer of size 0
            gpu_data = _driver.MemoryPointer(context=devices.get_context(), pointer=0, size=0)
            self.alloc_size = 0
        self.gpu_data = gpu_data
        self.stream = stream

    @property
    def __cuda_array_interface__(self):
        stream = self.stream
        return {
            "shape": self.shape,
            "strides": None if is_contiguous(self) else tuple(self.strides),
            "data": (self.device_ctypes_pointer.value or 0, False),
            "typestr": self.dtype.str,
            "stream": int(stream) if stream != 0 else None,
            "version": 3,
        }

    def bind(self, stream=0):
        """A shallow copy of this array whose default stream is `stream`."""
        clone = copy.copy(self)
        clone.stream = stream
        return clone

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
        from numba_cuda_amd.kernels.transpose import transpose
        return transpose(self)

    def _default_stream(self, stream):
        return self.stream if not stream else stream

    @property
    def device_ctypes_pointer(self):
        """ctypes integer holding the device address of item [0, ..., 0]"""
        try:
            return self.gpu_data.device_ctypes_pointer
        except AttributeError:
            return c_void_p(0)

    @devices.require_context
    def copy_to_device(self, ary, stream=0):
        """Copy `ary` into this array: device-to-device if `ary` is device memory,
        host-to-device otherwise.  Asynchronous iff a non-zero stream is in play."""
        if ary.size == 0:
            return
        sentry_contiguous(self)
        stream = self._default_stream(stream)
        self_core, ary_core = array_core(self), array_core(ary)
        if _driver.is_device_memory(ary):
            sentry_contiguous(ary)
            check_array_compatibility(self_core, ary_core)
            _driver.device_to_device(self, ary, self.alloc_size, stream=stream)
        else:
            # lay the host data out like self; copies only if it has to
            ary_core = np.array(ary_core, order="C" if self_core.flags["C_CONTIGUOUS"] else "F",
                                subok=True, copy=None)
            check_array_compatibility(self_core, ary_core)
            _driver.host_to_device(self, ary_core, self.alloc_size, stream=stream)

    @devices.require_context
    def copy_to_host(self, ary=None, stream=0):
        """Copy this array into `ary` (or a new ndarray) and return the host array.
        Synchronous unless a non-zero stream is given or bound."""
        if any(s < 0 for s in self.strides):
            raise NotImplementedError(
                "D->H copy not implemented for negative strides: {}".format(self.strides))
        assert self.alloc_size >= 0, "Negative memory size"
        stream = self._default_stream(stream)
        if ary is None:
            hostary = np.empty(shape=self.alloc_size, dtype=np.byte)
        else:
            check_array_compatibility(self, ary)
            hostary = ary
        if self.alloc_size != 0:
            _driver.device_to_host(hostary, self, self.alloc_size, stream=stream)
        if ary is None:
            if self.size == 0:
                hostary = np.ndarray(shape=self.shape, dtype=self.dtype, buffer=hostary)
            else:
                hostary = np.ndarray(shape=self.shape, dtype=self.dtype, strides=self.strides,
                                     buffer=hostary)
        return hostary

    def split(self, section, stream=0):
        """Yield consecutive 1-d views of `section` items (the last may be shorter)."""
        stream = self._default_stream(stream)
        if self.ndim != 1:
            raise ValueError("only support 1d array")
        if self.strides[0] != self.dtype.itemsize:
            raise ValueError("only support unit stride")
        itemsize = self.dtype.itemsize
        for i in range(int(math.ceil(float(self.size) / section))):
            begin = i * section
            end = min(begin + section, self.size)
            yield DeviceNDArray((end - begin,), self.strides, dtype=self.dtype, stream=stream,
                                gpu_data=self.gpu_data.view(begin * itemsize, end * itemsize))

    def as_cuda_arg(self):
        return self.gpu_data

    def get_ipc_handle(self):
        raise NotImplementedError("IPC handles are not part of this build")

    def squeeze(self, axis=None, stream=0):
        """View without the length-1 axes (all of them, or those in `axis`)."""
        new_dummy, _ = self._dummy.squeeze(axis=axis)
        return DeviceNDArray(shape=new_dummy.shape, strides=new_dummy.strides, dtype=self.dtype,
                             stream=self._default_stream(stream), gpu_data=self.gpu_data)

    def view(self, dtype):
        """Reinterpret the bytes as another dtype without copying."""
        dtype = np.dtype(dtype)
        shape = list(self.shape)
        strides = list(self.strides)
        if self.dtype.itemsize != dtype.itemsize:
            if not self.is_c_contiguous():
                raise ValueError("To change to a dtype of a different size,"
                                 " the array must be C-contiguous")
            shape[-1], rem = divmod(shape[-1] * self.dtype.itemsize, dtype.itemsize)
            if rem != 0:
                raise ValueError("When changing to a larger dtype,"
                                 " its size must be a divisor of the total size in bytes"
                                 " of the last axis of the array.")
            strides[-1] = dtype.itemsize
        return DeviceNDArray(shape=shape, strides=strides, dtype=dtype, stream=self.stream,
                             gpu_data=self.gpu_data)

    @property
    def nbytes(self):
        # bytes of the items, not of the (possibly gappy) allocation
        return self.dtype.itemsize * self.size


class DeviceRecord(DeviceNDArrayBase):
    """One structured item in device memory."""

    def __init__(self, dtype, stream=0, gpu_data=None):
        super().__init__((), (), dtype, stream, gpu_data)

    @property
    def flags(self):
        return dict(self._dummy.flags)

    @devices.require_context
    def __getitem__(self, item):
        return self._do_getitem(item)

    @devices.require_context
    def getitem(self, item, stream=0):
        """`self[item]` on a given stream"""
        return self._do_getitem(item, stream)

    def _do_getitem(self, item, stream=0):
        stream = self._default_stream(stream)
        typ, offset = self.dtype.fields[item]
        newdata = self.gpu_data.view(offset)
        if typ.shape == ():
            if typ.names is not None:
                return DeviceRecord(dtype=typ, stream=stream, gpu_data=newdata)
            hostary = np.empty(1, dtype=typ)
            _driver.device_to_host(dst=hostary, src=newdata, size=typ.itemsize, stream=stream)
            return hostary[0]
        shape, strides, dtype = prepare_shape_strides_dtype(typ.shape, None, typ.subdtype[0], "C")
        return DeviceNDArray(shape=shape, strides=strides, dtype=dtype, gpu_data=newdata, stream=stream)

    @devices.require_context
    def __setitem__(self, key, value):
        return self._do_setitem(key, value)

    @devices.require_context
    def setitem(self, key, value, stream=0):
        """`self[key] = value` on a given stream"""
        return self._do_setitem(key, value, stream=stream)

    def _do_setitem(self, key, value, stream=0):
        stream = self._default_stream(stream)
        synchronous = not stream
        if synchronous:
            stream = devices.get_context().get_default_stream()
        typ, offset = self.dtype.fields[key]
        lhs = type(self)(dtype=typ, stream=stream, gpu_data=self.gpu_data.view(offset))
        rhs, _ = auto_device(lhs.dtype.type(value), stream=stream)
        _driver.device_to_device(lhs, rhs, rhs.dtype.itemsize, stream)
        if synchronous:
            stream.synchronize()


class DeviceNDArray(DeviceNDArrayBase):
    """An array in device memory."""

    def is_f_contiguous(self):
        return self._dummy.is_f_contig

    def is_c_contiguous(self):
        return self._dummy.is_c_contig

    @property
    def flags(self):
        # a plain dict: NumPy's flags object cannot be built without an ndarray
        return dict(self._dummy.flags)

    def __array__(self, dtype=None, copy=None):
        """Copies to the host; `copy=False` cannot be honoured."""
        if copy is False:
            raise ValueError("`copy=False` is not supported. A copy is always created.")
        host = self.copy_to_host()
        return host.__array__(dtype) if dtype else host.__array__()

    def __len__(self):
        return self.shape[0]

    def reshape(self, *newshape, **kws):
        """Reshape without moving data, like numpy.ndarray.reshape; raises
        NotImplementedError when that is impossible."""
        if len(newshape) == 1 and isinstance(newshape[0], (tuple, list)):
            newshape = newshape[0]
        cls = type(self)
        if newshape == self.shape:
            return cls(shape=self.shape, strides=self.strides, dtype=self.dtype, gpu_data=self.gpu_data)
        newarr, extents = self._dummy.reshape(*newshape, **kws)
        if extents == [self._dummy.extent]:
            return cls(shape=newarr.shape, strides=newarr.strides, dtype=self.dtype,
                       gpu_data=self.gpu_data)
        raise NotImplementedError("operation requires copying")

    def ravel(self, order="C", stream=0):
        """Flatten a contiguous array without moving data."""
        stream = self._default_stream(stream)
        newarr, extents = self._dummy.ravel(order=order)
        if extents == [self._dummy.extent]:
            return type(self)(shape=newarr.shape, strides=newarr.strides, dtype=self.dtype,
                              gpu_data=self.gpu_data, stream=stream)
        raise NotImplementedError("operation requires copying")

    @devices.require_context
    def __getitem__(self, item):
        return self._do_getitem(item)

    @devices.require_context
    def getitem(self, item, stream=0):
        """`self[item]` on a given stream"""
        return self._do_getitem(item, stream)

    def _do_getitem(self, item, stream=0):
        stream = self._default_stream(stream)
        arr = self._dummy.__getitem__(item)
        cls = type(self)
        if not arr.is_array:
            newdata = self.gpu_data.view(*arr.extent)
            if self.dtype.names is not None:
                return DeviceRecord(dtype=self.dtype, stream=stream, gpu_data=newdata)
            # a single item: fetch it (blocking when no stream is involved)
            hostary = np.empty(1, dtype=self.dtype)
            _driver.device_to_host(dst=hostary, src=newdata, size=self._dummy.itemsize, stream=stream)
            return hostary[0]
        # contiguous or not, the view starts at the selection's first item and
        # spans to its last; shape and strides say what lies in between
        newdata = self.gpu_data.view(*arr.extent)
        return cls(shape=arr.shape, strides=arr.strides, dtype=self.dtype, gpu_data=newdata, stream=stream)

    @devices.require_context
    def __setitem__(self, key, value):
        return self._do_setitem(key, value)

    @devices.require_context
    def setitem(self, key, value, stream=0):
        """`self[key] = value` on a given stream"""
        return self._do_setitem(key, value, stream=stream)

    def _do_setitem(self, key, value, stream=0):
        stream = self._default_stream(stream)
        # no stream bound and none given: work on the default stream and wait for it
        synchronous = not stream
        if synchronous:
            stream = devices.get_context().get_default_stream()

        # left-hand side: a view of the selected items (0-d for a single item)
        arr = self._dummy.__getitem__(key)
        newdata = self.gpu_data.view(*arr.extent)
        if isinstance(arr, dummyarray.Element):
            shape, strides = (), ()
        else:
            shape, strides = arr.shape, arr.strides
        lhs = type(self)(shape=shape, strides=strides, dtype=self.dtype, gpu_data=newdata, stream=stream)

        # right-hand side: on the device, padded with leading unit axes, broadcastable
        if not _driver.is_device_memory(value) and not hasattr(value, "__cuda_array_interface__"):
            # host values take the dtype of the target, as a NumPy assignment would
            value = np.asarray(value).astype(self.dtype, copy=False)
        rhs, _ = auto_device(value, stream=stream, user_explicit=True)
        if rhs.ndim > lhs.ndim:
            raise ValueError("Can't assign %s-D array to %s-D self" % (rhs.ndim, lhs.ndim))
        if rhs.dtype != lhs.dtype:
            raise TypeError("incompatible dtype: %s vs. %s" % (lhs.dtype, rhs.dtype))
        pad = lhs.ndim - rhs.ndim
        rhs_shape = (1,) * pad + tuple(rhs.shape)
        rhs_strides = (0,) * pad + tuple(rhs.strides)
        for i, (l, r) in enumerate(zip(lhs.shape, rhs_shape)):
            if r != 1 and l != r:
                raise ValueError("Can't copy sequence with size %d to array "
                                 "axis %d with dimension %d" % (r, i, l))
        # a unit axis on the right repeats along the matching axis on the left
        src_strides = tuple(0 if r == 1 else s for r, s in zip(rhs_shape, rhs_strides))

        nd = lhs.ndim
        if nd > _MAX_ASSIGN_NDIM:
            raise NotImplementedError("assignment supports at most %d axes" % _MAX_ASSIGN_NDIM)
        vec = ctypes.c_int64 * max(nd, 1)
        _driver.driver.nbh_assign(lhs.device_ctypes_pointer.value, rhs.device_ctypes_pointer.value, nd,
                                  vec(*lhs.shape), vec(*lhs.strides), vec(*src_strides),
                                  self.dtype.itemsize, _driver._stream_handle(stream) or None)
        if synchronous:
            stream.synchronize()


_MAX_ASSIGN_NDIM = 8


class MappedNDArray(DeviceNDArrayBase, np.ndarray):
    """A host array in pinned memory that the device can address."""

    def device_setup(self, gpu_data, stream=0):
        self.gpu_data = gpu_data
        self.stream = stream


def from_array_like(ary, stream=0, gpu_data=None):
    "A DeviceNDArray with the shape, strides and dtype of `ary`."
    return DeviceNDArray(ary.shape, ary.strides, ary.dtype, stream=stream, gpu_data=gpu_data)


def from_record_like(rec, stream=0, gpu_data=None):
    "A DeviceRecord with the dtype of `rec`."
    return DeviceRecord(rec.dtype, stream=stream, gpu_data=gpu_data)


def array_core(ary):
    """The part of a broadcast array that really exists in memory: index 0 along
    every zero-stride axis.  Contiguity and copies are decided on this core."""
    if not ary.strides or not ary.size:
        return ary
    return ary[tuple(0 if stride == 0 else slice(None) for stride in ary.strides)]


def is_contiguous(ary):
    """True iff `ary` is C-contiguous once broadcast and length-1 axes are ignored."""
    size = ary.dtype.itemsize
    for shape, stride in zip(reversed(ary.shape), reversed(ary.strides)):
        if shape > 1 and stride != 0:
            if size != stride:
                return False
            size *= shape
    return True


errmsg_contiguous_buffer = ("Array contains non-contiguous buffer and cannot "
                            "be transferred as a single memory region. Please "
                            "ensure contiguous buffer with numpy "
                            ".ascontiguousarray()")


def sentry_contiguous(ary):
    core = array_core(ary)
    if not core.flags["C_CONTIGUOUS"] and not core.flags["F_CONTIGUOUS"]:
        raise ValueError(errmsg_contiguous_buffer)


def auto_device(obj, stream=0, copy=True, user_explicit=False):
    """Return (device object, created?) for `obj`: device memory passes through,
    objects exporting __cuda_array_interface__ are wrapped without copying,
    anything else is turned into an ndarray and (optionally) copied over."""
    if _driver.is_device_memory(obj):
        return obj, False
    interface = getattr(obj, "__cuda_array_interface__", None)
    if interface is not None:
        from numba_cuda_amd.api import from_cuda_array_interface
        return from_cuda_array_interface(interface, owner=obj), False
    if isinstance(obj, np.void):
        devobj = from_record_like(obj, stream=stream)
    else:
        obj = np.array(obj, copy=None, subok=True)
        sentry_contiguous(obj)
        devobj = from_array_like(obj, stream=stream)
    if copy:
        if (config.CUDA_WARN_ON_IMPLICIT_COPY and not config.DISABLE_PERFORMANCE_WARNINGS
                and not user_explicit and isinstance(obj, np.ndarray)):
            warn(NumbaPerformanceWarning("Host array used in CUDA kernel will incur "
                                         "copy overhead to/from device."))
        devobj.copy_to_device(obj, stream=stream)
    return devobj, True


def check_array_compatibility(ary1, ary2):
    ary1sq, ary2sq = ary1.squeeze(), ary2.squeeze()
    if ary1.dtype != ary2.dtype:
        raise TypeError("incompatible dtype: %s vs. %s" % (ary1.dtype, ary2.dtype))
    if ary1sq.shape != ary2sq.shape:
        raise ValueError("incompatible shape: %s vs. %s" % (ary1.shape, ary2.shape))
    # strides of an empty copy are irrelevant (and may legitimately differ)
    if ary1.size and ary1sq.strides != ary2sq.strides:
        raise ValueError("incompatible strides: %s vs. %s" % (ary1.strides, ary2.strides))
