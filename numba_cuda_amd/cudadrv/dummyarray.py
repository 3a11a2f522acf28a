"""Stride calculus for arrays without data.

`Array` describes where the items of an n-d array live relative to a base pointer:
a byte offset of item [0, ..., 0], a shape, byte strides and an item size.  It
answers the questions device arrays ask - what does this index expression select,
can this be reshaped without copying, which byte range is touched, is it
contiguous - with NumPy's rules, and never touches memory.

Interface follows numba_cuda/numba/cuda/cudadrv/dummyarray.py (Array :221-515,
Element :212-219, Extent :11, iter_strides_c/f_contig :518-542); the
implementation is independent of it: an Array is an immutable (offset, shape,
strides) triple and every operation is a function of those three tuples.
"""

import functools
import itertools
import operator
from collections import namedtuple

import numpy as np

Extent = namedtuple("Extent", ["begin", "end"])


def _as_int(x, what):
    if isinstance(x, (int, np.integer)) and not isinstance(x, bool):
        return int(x)
    raise TypeError("all elements of %s must be ints" % what)


def _prod(seq):
    return functools.reduce(operator.mul, seq, 1)


def c_strides(shape, itemsize):
    """Byte strides of a C-ordered array of `shape`."""
    out, acc = [], itemsize
    for n in reversed(shape):
        out.append(acc)
        acc *= n
    return tuple(reversed(out))


def f_strides(shape, itemsize):
    """Byte strides of a Fortran-ordered array of `shape`."""
    out, acc = [], itemsize
    for n in shape:
        out.append(acc)
        acc *= n
    return tuple(out)


def iter_strides_c_contig(arr, shape=None):
    return iter(c_strides(arr.shape if shape is None else shape, arr.itemsize))


def iter_strides_f_contig(arr, shape=None):
    return iter(f_strides(arr.shape if shape is None else shape, arr.itemsize))


def layout_flags(shape, strides, itemsize):
    """C/F contiguity with NumPy's relaxed rules: axes of length 1 carry no
    constraint, empty arrays are both, a zero stride on a longer axis is neither."""
    if 0 in shape:
        return {"C_CONTIGUOUS": True, "F_CONTIGUOUS": True}
    live = [(n, s) for n, s in zip(shape, strides) if n != 1]
    if any(s == 0 for _, s in live):
        return {"C_CONTIGUOUS": False, "F_CONTIGUOUS": False}
    dims = [n for n, _ in live]
    got = tuple(s for _, s in live)
    return {"C_CONTIGUOUS": got == c_strides(dims, itemsize),
            "F_CONTIGUOUS": got == f_strides(dims, itemsize)}


def _merge_groups(old_shape, old_strides, new_shape, itemsize, fortran):
    """Strides that present `old` as `new_shape` without moving data, or None.

    Walk both shapes (old one without its length-1 axes) in lock step, cutting
    them into the shortest runs with equal products.  A run of old axes can stand
    for one flat axis only if each axis continues where its neighbour ends; the
    run of new axes then subdivides that flat axis.
    """
    olds = [(n, s) for n, s in zip(old_shape, old_strides) if n != 1]
    new_strides = [None] * len(new_shape)
    oi = ni = 0
    while oi < len(olds) and ni < len(new_shape):
        oj, nj = oi + 1, ni + 1
        op, np_ = olds[oi][0], new_shape[ni]
        while op != np_:
            if np_ < op:
                np_ *= new_shape[nj]
                nj += 1
            else:
                op *= olds[oj][0]
                oj += 1
        run = olds[oi:oj]
        for a, b in zip(run, run[1:]):
            # C order: outer stride == inner extent * inner stride; F order mirrored
            if fortran:
                if b[1] != a[0] * a[1]:
                    return None
            elif a[1] != b[0] * b[1]:
                return None
        if fortran:
            acc = run[0][1]
            for k in range(ni, nj):
                new_strides[k] = acc
                acc *= new_shape[k]
        else:
            acc = run[-1][1]
            for k in range(nj - 1, ni - 1, -1):
                new_strides[k] = acc
                acc *= new_shape[k]
        oi, ni = oj, nj
    # whatever is left of the new shape is length-1 axes
    if ni >= 1:
        filler = new_strides[ni - 1] * (new_shape[ni - 1] if fortran else 1)
    else:
        filler = itemsize
    for k in range(ni, len(new_shape)):
        new_strides[k] = filler
    return tuple(new_strides)


def attempt_nocopy_reshape(nd, dims, strides, newnd, newdims, newstrides, itemsize, is_f_order):
    """Fill `newstrides` and return 1 if dims/strides can be viewed as newdims
    without a copy, else return 0 (calling convention of dummyarray.py:14-120)."""
    dims, newdims = tuple(dims[:nd]), tuple(newdims[:newnd])
    if _prod(dims) != _prod(newdims):
        return 0
    if _prod(newdims) == 0:
        for i in range(newnd):
            newstrides[i] = itemsize
        return 1
    got = _merge_groups(dims, tuple(strides[:nd]), newdims, itemsize, bool(is_f_order))
    if got is None:
        return 0
    for i, s in enumerate(got):
        newstrides[i] = s
    return 1


class Element:
    """What indexing returns when every axis got an integer."""

    is_array = False

    def __init__(self, extent):
        self.extent = extent

    def iter_contiguous_extent(self):
        yield self.extent


class Array:
    """Data-less n-d array: ndim, shape, strides, itemsize, size, extent, flags."""

    is_array = True

    def __init__(self, offset, shape, strides, itemsize):
        self.offset = offset
        self.shape = tuple(shape)
        self.strides = tuple(strides)
        self.ndim = len(self.shape)
        self.itemsize = itemsize
        self.size = _prod(self.shape)
        self.flags = layout_flags(self.shape, self.strides, itemsize)
        # from item [0,...,0] to one past item [-1,...,-1]; never negative
        last = offset + sum((n - 1) * s for n, s in zip(self.shape, self.strides)) + itemsize
        self.extent = Extent(offset, max(last, offset))

    @classmethod
    def from_desc(cls, offset, shape, strides, itemsize):
        shape = tuple(_as_int(n, "shape") for n in shape)
        strides = tuple(_as_int(s, "strides") for s in strides)
        return cls(_as_int(offset, "offset"), shape, strides, itemsize)

    def __repr__(self):
        return "<Array offset=%d shape=%s strides=%s itemsize=%d>" % (
            self.offset, self.shape, self.strides, self.itemsize)

    @property
    def is_c_contig(self):
        return self.flags["C_CONTIGUOUS"]

    @property
    def is_f_contig(self):
        return self.flags["F_CONTIGUOUS"]

    # ---- indexing -------------------------------------------------------------
    def __getitem__(self, item):
        items = list(item) if isinstance(item, tuple) else [item]
        if len(items) > self.ndim:
            raise IndexError("%d extra indices given" % (len(items) - self.ndim,))
        items += [slice(None)] * (self.ndim - len(items))
        offset = self.offset
        shape, strides = [], []
        for it, n, s in zip(items, self.shape, self.strides):
            if isinstance(it, slice):
                start, stop, step = it.indices(n)
                count = len(range(start, stop, step))
                offset += start * s
                shape.append(count)
                strides.append(s * step)
            else:
                idx = operator.index(it)
                if idx < 0:
                    idx += n
                if not 0 <= idx < n:
                    raise IndexError("index %d is out of bounds for axis with size %d" % (it, n))
                offset += idx * s
        if not shape and self.ndim:
            return Element(Extent(offset, offset + self.itemsize))
        return Array(offset, shape, strides, self.itemsize)

    # ---- contiguous pieces ------------------------------------------------------
    def iter_contiguous_extent(self):
        """Byte ranges, in no particular order, that together hold every item."""
        if self.is_c_contig or self.is_f_contig:
            yield self.extent
            return
        if self.size == 0:
            return
        # treat the axis with the smallest stride as the candidate run
        inner = min(range(self.ndim), key=lambda k: abs(self.strides[k]) if self.shape[k] > 1 else float("inf"))
        outer = [k for k in range(self.ndim) if k != inner]
        if self.strides[inner] == self.itemsize:
            run = self.shape[inner] * self.itemsize
            for idx in itertools.product(*(range(self.shape[k]) for k in outer)):
                base = self.offset + sum(i * self.strides[k] for i, k in zip(idx, outer))
                yield base, base + run
        else:
            for idx in itertools.product(*(range(n) for n in self.shape)):
                base = self.offset + sum(i * s for i, s in zip(idx, self.strides))
                yield base, base + self.itemsize

    # ---- shape changes ----------------------------------------------------------
    def reshape(self, *newdims, **kws):
        """Returns (Array, extents) or raises NotImplementedError when the new
        shape cannot be a view."""
        if newdims == self.shape:
            return self, None
        order = kws.pop("order", "C")
        if kws:
            raise TypeError("unknown keyword arguments %s" % kws.keys())
        if order not in "CFA":
            raise ValueError("order not C|F|A")
        newdims = tuple(operator.index(d) for d in newdims)
        unknown = [i for i, d in enumerate(newdims) if d < 0]
        if len(unknown) > 1:
            raise ValueError("can only specify one unknown dimension")
        if unknown:
            known = _prod(d for d in newdims if d >= 0)
            if known == 0 or self.size % known:
                raise ValueError("cannot infer valid shape for unknown dimension")
            i = unknown[0]
            newdims = newdims[:i] + (self.size // known,) + newdims[i + 1:]
        if _prod(newdims) != self.size:
            raise ValueError("reshape changes the size of the array")
        if order == "A":
            order = "F" if self.is_f_contig else "C"
        if order == "C" and self.is_c_contig:
            newstrides = c_strides(newdims, self.itemsize)
        elif order == "F" and self.is_f_contig:
            newstrides = f_strides(newdims, self.itemsize)
        elif self.size == 0:
            newstrides = (self.itemsize,) * len(newdims)
        else:
            newstrides = _merge_groups(self.shape, self.strides, newdims, self.itemsize, order == "F")
            if newstrides is None:
                raise NotImplementedError("reshape would require copy")
        out = Array(self.extent.begin, newdims, newstrides, self.itemsize)
        return out, list(self.iter_contiguous_extent())

    def squeeze(self, axis=None):
        if axis is None:
            drop = {k for k, n in enumerate(self.shape) if n == 1}
        else:
            axes = axis if isinstance(axis, tuple) else (axis,)
            drop = {a % self.ndim if self.ndim else a for a in axes}
            for a in drop:
                if self.shape[a] != 1:
                    raise ValueError("cannot select an axis to squeeze out which has size "
                                     "not equal to one")
        keep = [k for k in range(self.ndim) if k not in drop]
        out = Array(self.extent.begin, [self.shape[k] for k in keep],
                    [self.strides[k] for k in keep], self.itemsize)
        return out, list(self.iter_contiguous_extent())

    def ravel(self, order="C"):
        if order not in "CFA":
            raise ValueError("order not C|F|A")
        if (order in "CA" and self.is_c_contig) or (order in "FA" and self.is_f_contig):
            out = Array(self.extent.begin, (self.size,), (self.itemsize,), self.itemsize)
            return out, list(self.iter_contiguous_extent())
        raise NotImplementedError("ravel on non-contiguous array")


def is_element_indexing(item, ndim):
    if isinstance(item, slice):
        return False
    if isinstance(item, tuple):
        return len(item) == ndim and not any(isinstance(it, slice) for it in item)
    return True
