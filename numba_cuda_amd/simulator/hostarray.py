"""NumPy-backed stand-in for the device array, for the CPU mode (NUMBA_ENABLE_CUDASIM=1).

Mirrors what the reference's simulator offers in place of DeviceNDArray
(numba_cuda/numba/cuda/simulator/cudadrv/devicearray.py:102-272 the array,
:320-462 the constructors and checks): the "device" memory is an ordinary NumPy
array owned by the wrapper, copies are NumPy copies, `.T` is a view.
"""

from contextlib import contextmanager

import numpy as np

NON_CONTIGUOUS = ("Array contains non-contiguous buffer and cannot be transferred as a single memory region. "
                  "Please ensure contiguous buffer with numpy .ascontiguousarray()")


class _Shape(tuple):
    """A shape whose items cannot be asked for from the end, as inside device code."""

    def __getitem__(self, k):
        if isinstance(k, int) and k < 0:
            raise IndexError("tuple index out of range")
        return super().__getitem__(k)


def _binary(name):
    def op(self, other):
        return HostBackedArray(getattr(self._ary, name)(getattr(other, "_ary", other)))
    op.__name__ = name
    return op


class HostBackedArray:
    """What to_device / device_array return in the CPU mode."""

    __cuda_ndarray__ = True

    def __init__(self, ary, stream=0):
        self._ary = ary
        self.stream = stream

    # anything not defined here is the wrapped array's (dtype, strides, ndim, size, ...)
    def __getattr__(self, name):
        if name == "_ary":
            raise AttributeError(name)
        try:
            return getattr(self._ary, name)
        except AttributeError as e:
            raise AttributeError("Wrapped array has no attribute '%s'" % name) from e

    @property
    def shape(self):
        return _Shape(self._ary.shape)

    @property
    def nbytes(self):
        return self._ary.nbytes

    @property
    def alloc_size(self):
        return self._ary.nbytes

    @property
    def T(self):
        return self.transpose()

    def bind(self, stream=0):
        return HostBackedArray(self._ary, stream)

    def transpose(self, axes=None):
        return HostBackedArray(np.transpose(self._ary, axes=axes))

    def ravel(self, *args, **kwargs):
        return HostBackedArray(self._ary.ravel(*args, **kwargs))

    def reshape(self, *args, **kwargs):
        return HostBackedArray(self._ary.reshape(*args, **kwargs))

    def view(self, *args, **kwargs):
        return HostBackedArray(self._ary.view(*args, **kwargs))

    def split(self, section, stream=0):
        return [HostBackedArray(part) for part in np.split(self._ary, range(section, len(self), section))]

    def is_c_contiguous(self):
        return self._ary.flags.c_contiguous

    def is_f_contiguous(self):
        return self._ary.flags.f_contiguous

    def __getitem__(self, idx):
        got = self._ary[idx]
        if type(got) in (np.ndarray, np.void):
            return HostBackedArray(got, stream=self.stream)
        return got

    def __setitem__(self, idx, value):
        self._ary[idx] = getattr(value, "_ary", value)

    def __len__(self):
        return len(self._ary)

    def __str__(self):
        return str(self._ary)

    def __repr__(self):
        return repr(self._ary)

    def __array__(self, dtype=None, copy=None):
        return np.asarray(self._ary, dtype=dtype)

    def copy_to_host(self, ary=None, stream=0):
        if ary is None:
            ary = np.empty_like(self._ary)
        else:
            check_array_compatibility(self, ary)
        np.copyto(ary, self._ary)
        return ary

    def copy_to_device(self, ary, stream=0):
        """Copy `ary` (host or HostBackedArray) into this array; the two must match in
        dtype, squeezed shape and strides."""
        sentry_contiguous(self)
        mine, theirs = array_core(self), array_core(ary)
        if isinstance(ary, HostBackedArray):
            sentry_contiguous(ary)
        else:
            theirs = np.array(theirs, order="C" if mine.flags["C_CONTIGUOUS"] else "F", subok=True, copy=None)
        check_array_compatibility(mine, theirs)
        np.copyto(mine._ary, getattr(theirs, "_ary", theirs))

    __eq__ = _binary("__eq__")
    __ne__ = _binary("__ne__")
    __lt__ = _binary("__lt__")
    __le__ = _binary("__le__")
    __gt__ = _binary("__gt__")
    __ge__ = _binary("__ge__")
    __add__ = _binary("__add__")
    __sub__ = _binary("__sub__")
    __mul__ = _binary("__mul__")
    __floordiv__ = _binary("__floordiv__")
    __truediv__ = _binary("__truediv__")
    __mod__ = _binary("__mod__")
    __pow__ = _binary("__pow__")
    __hash__ = None


def array_core(ary):
    """The array without its repeated (zero-stride) axes."""
    if not ary.strides or not ary.size:
        return ary
    return ary[tuple(0 if stride == 0 else slice(None) for stride in ary.strides)]


def is_contiguous(ary):
    """C-contiguous, leaving aside broadcast and one-item axes."""
    expect = ary.dtype.itemsize
    for extent, stride in zip(reversed(ary.shape), reversed(ary.strides)):
        if extent > 1 and stride != 0:
            if stride != expect:
                return False
            expect *= extent
    return True


def sentry_contiguous(ary):
    core = array_core(ary)
    if not core.flags["C_CONTIGUOUS"] and not core.flags["F_CONTIGUOUS"]:
        raise ValueError(NON_CONTIGUOUS)


def check_array_compatibility(a, b):
    a_sq, b_sq = a.squeeze(), b.squeeze()
    if a.dtype != b.dtype:
        raise TypeError("incompatible dtype: %s vs. %s" % (a.dtype, b.dtype))
    if a_sq.shape != b_sq.shape:
        raise ValueError("incompatible shape: %s vs. %s" % (a.shape, b.shape))
    if a_sq.strides != b_sq.strides:
        raise ValueError("incompatible strides: %s vs. %s" % (a.strides, b.strides))


def to_device(ary, stream=0, copy=True, to=None):
    ary = np.array(ary, copy=None, subok=True)
    sentry_contiguous(ary)
    if to is not None:
        to.copy_to_device(ary, stream=stream)
        return None
    # a private copy of the bytes, seen through the caller's shape and strides
    raw = np.int64 if ary.dtype.char in "Mm" else ary.dtype
    owned = np.ndarray(buffer=np.copy(array_core(ary)).view(raw), dtype=ary.dtype, shape=ary.shape,
                       strides=ary.strides).view(type=type(ary))
    return HostBackedArray(owned)


def device_array(*args, **kwargs):
    stream = kwargs.pop("stream", 0)
    return HostBackedArray(np.ndarray(*args, **kwargs), stream=stream)


def _contiguous_strides_like_array(ary):
    if ary.flags["C_CONTIGUOUS"] or ary.flags["F_CONTIGUOUS"] or ary.ndim <= 1:
        return None
    # keep the order of the axes by stride, make them dense
    strides = [0] * ary.ndim
    step = ary.dtype.itemsize
    for axis, _ in sorted(enumerate(ary.strides), key=lambda pair: pair[1]):
        strides[axis] = step
        step *= ary.shape[axis]
    return tuple(strides)


def _order_like_array(ary):
    return "F" if ary.flags["F_CONTIGUOUS"] and not ary.flags["C_CONTIGUOUS"] else "C"


def device_array_like(ary, stream=0):
    return device_array(shape=ary.shape, dtype=ary.dtype, strides=_contiguous_strides_like_array(ary),
                        order=_order_like_array(ary))


def pinned_array(shape, dtype=np.float64, strides=None, order="C"):
    return np.ndarray(shape=shape, strides=strides, dtype=dtype, order=order)


managed_array = pinned_array


def pinned_array_like(ary):
    return pinned_array(shape=ary.shape, dtype=ary.dtype, strides=_contiguous_strides_like_array(ary),
                        order=_order_like_array(ary))


def mapped_array(*args, **kwargs):
    kwargs.pop("portable", None)
    kwargs.pop("wc", None)
    return device_array(*args, **kwargs)


mapped_array_like = device_array_like


@contextmanager
def pinned(*arylist):
    yield


@contextmanager
def mapped(*arylist, **kws):
    made = [HostBackedArray(np.asarray(a)) for a in arylist]
    yield made[0] if len(made) == 1 else made


def auto_device(ary, stream=0, copy=True):
    if isinstance(ary, HostBackedArray):
        return ary, False
    if not isinstance(ary, np.void):
        ary = np.array(ary, copy=None, subok=True)
    return to_device(ary, stream, copy), True


def is_cuda_ndarray(obj):
    return getattr(obj, "__cuda_ndarray__", False)


def require_cuda_ndarray(obj):
    if not is_cuda_ndarray(obj):
        raise ValueError("require an cuda ndarray object")


def verify_cuda_ndarray_interface(obj):
    require_cuda_ndarray(obj)
    for attr, kind in (("shape", tuple), ("strides", tuple), ("dtype", np.dtype), ("size", int)):
        if not hasattr(obj, attr):
            raise AttributeError(attr)
        if not isinstance(getattr(obj, attr), kind):
            raise AttributeError("%s must be of type %s" % (attr, kind))


DeviceNDArray = HostBackedArray
DeviceRecord = None
from_record_like = None
