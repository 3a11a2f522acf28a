"""Stride calculus against NumPy itself (the approach of the reference's
numba_cuda/numba/cuda/tests/nocuda/test_dummyarray.py): whatever NumPy says about
shape, strides, offset, contiguity and no-copy reshapes of a view, the data-less
Array must say too."""

import itertools

import numpy as np
import pytest

from numba_cuda_amd.cudadrv.dummyarray import Array, Element, attempt_nocopy_reshape


def _desc(a, base):
    off = a.__array_interface__["data"][0] - base.__array_interface__["data"][0]
    return off, a.shape, a.strides


def _same(dummy, view, base):
    off, shape, strides = _desc(view, base)
    assert dummy.shape == shape
    if view.size:                       # strides/offset of empty views are immaterial
        assert dummy.strides == strides
        assert dummy.extent.begin == off
    assert dummy.is_c_contig == view.flags["C_CONTIGUOUS"]
    assert dummy.is_f_contig == view.flags["F_CONTIGUOUS"]
    assert dummy.size == view.size


SLICES_1D = [slice(None), slice(1, None), slice(None, -1), slice(2, 7, 2), slice(None, None, -1),
             slice(8, 1, -3), slice(5, 5), slice(-3, None), slice(100, 200), slice(None, None, 4)]


@pytest.mark.parametrize("sl", SLICES_1D)
def test_slicing_1d(sl):
    base = np.arange(10, dtype=np.int32)
    d = Array.from_desc(0, base.shape, base.strides, base.itemsize)
    _same(d[sl], base[sl], base)
    for sl2 in SLICES_1D[:6]:           # slice of a slice, also of reversed views
        _same(d[sl][sl2], base[sl][sl2], base)


def test_slicing_2d_and_3d_products():
    base = np.arange(5 * 6 * 7, dtype=np.float64).reshape(5, 6, 7)
    d = Array.from_desc(0, base.shape, base.strides, base.itemsize)
    choices = [slice(None), slice(1, 4), slice(None, None, 2), slice(None, None, -1), 2, -1]
    for idx in itertools.product(choices, repeat=3):
        want = base[idx]
        got = d[idx]
        if isinstance(want, np.ndarray):
            _same(got, want, base)
        else:
            assert isinstance(got, Element)
            off = sum(int(i % n) * s for i, n, s in zip(idx, base.shape, base.strides))
            assert got.extent == (off, off + 8)
    for idx in (1, (2,), (slice(None), 3), (4, slice(1, 3))):   # fewer indices than axes
        _same(d[idx], base[idx], base)


def test_index_errors():
    d = Array.from_desc(0, (3, 4), (32, 8), 8)
    with pytest.raises(IndexError):
        d[3]
    with pytest.raises(IndexError):
        d[0, -5]
    with pytest.raises(IndexError):
        d[0, 0, 0]


def test_element_extent_and_offsets():
    d = Array.from_desc(16, (3, 4), (32, 8), 8)
    assert d.extent == (16, 16 + 3 * 32)
    e = d[1, 2]
    assert not e.is_array and e.extent == (16 + 32 + 16, 16 + 32 + 24)
    assert list(e.iter_contiguous_extent()) == [e.extent]


@pytest.mark.parametrize("order", ["C", "F"])
def test_contiguity_flags_follow_numpy(order):
    for shape in [(), (1,), (5,), (1, 1), (1, 5), (5, 1), (3, 4), (2, 1, 3), (0, 3), (3, 0, 2), (1, 1, 1)]:
        a = np.zeros(shape, order=order)
        d = Array.from_desc(0, a.shape, a.strides, a.itemsize)
        assert d.flags == {"C_CONTIGUOUS": a.flags["C_CONTIGUOUS"], "F_CONTIGUOUS": a.flags["F_CONTIGUOUS"]}
    b = np.broadcast_to(np.zeros((3, 1)), (3, 4))
    d = Array.from_desc(0, b.shape, b.strides, b.itemsize)
    assert d.flags == {"C_CONTIGUOUS": False, "F_CONTIGUOUS": False}


def _all_reshapes(size):
    out = set()
    for a in range(1, size + 1):
        if size % a == 0:
            out.add((a, size // a))
            for b in range(1, size // a + 1):
                if (size // a) % b == 0:
                    out.add((a, b, size // a // b))
    out.add((size,))
    out.add((1, size, 1))
    return sorted(out)


@pytest.mark.parametrize("order", ["C", "F"])
def test_reshape_of_views_matches_numpy(order):
    base = np.arange(4 * 6 * 2, dtype=np.int16).reshape(4, 6, 2)
    views = [base, base.T, base[::2], base[:, ::3], base[:, :, 0], base[1:3, 2:4], base[:, :, ::-1][:, :, :1],
             np.asfortranarray(base), base[:, 1:2, :], base.transpose(1, 0, 2), base[::3, ::5, :]]
    for v in views:
        root = v
        while root.base is not None:
            root = root.base
        d = Array.from_desc(*_desc(v, root), v.itemsize)
        for newshape in _all_reshapes(v.size):
            # NumPy tells us whether a view is possible: try reshaping in place
            probe = v.view()
            try:
                if order == "C":
                    probe.shape = newshape
                    want = probe
                else:
                    t = v.T.view()
                    t.shape = newshape[::-1]
                    want = t.T
                possible = True
            except AttributeError:
                possible = False
            if not possible:
                with pytest.raises(NotImplementedError):
                    d.reshape(*newshape, order=order)
                continue
            got, _ = d.reshape(*newshape, order=order)
            assert got.shape == want.shape
            # the same items must be addressed: compare the byte offset of every item
            assert _offsets(got.extent.begin, got.shape, got.strides) == \
                _offsets(*_desc(want, root)), (v.shape, v.strides, newshape, order)


def _offsets(begin, shape, strides):
    idx = np.indices(shape).reshape(len(shape), -1).T
    return (begin + (idx * np.asarray(strides, dtype=np.int64)).sum(axis=1)).tolist()


def test_reshape_minus_one_and_errors():
    d = Array.from_desc(0, (4, 6), (48, 8), 8)
    assert d.reshape(-1, 3)[0].shape == (8, 3)
    assert d.reshape(2, -1, 2)[0].shape == (2, 6, 2)
    assert d.reshape(4, 6)[0] is d
    with pytest.raises(ValueError, match="one unknown dimension"):
        d.reshape(-1, -1)
    with pytest.raises(ValueError, match="cannot infer"):
        d.reshape(-1, 5)
    with pytest.raises(ValueError, match="changes the size"):
        d.reshape(5, 5)
    with pytest.raises(ValueError):
        d.reshape(24, order="K")
    z = Array.from_desc(0, (0, 3), (24, 8), 8)
    assert z.reshape(0)[0].shape == (0,)


def test_attempt_nocopy_reshape_calling_convention():
    a = np.zeros((4, 6))[:, ::2]            # (4, 3), strides (48, 16): rows chain up
    new = [0, 0]
    assert attempt_nocopy_reshape(2, a.shape, a.strides, 2, (2, 6), new, 8, False) == 1
    assert new == [96, 16]
    new = [0]
    assert attempt_nocopy_reshape(2, a.shape, a.strides, 1, (12,), new, 8, False) == 1
    assert new == [16]
    b = np.zeros((4, 6))[:, :3]             # (4, 3), strides (48, 8): gap after each row
    assert attempt_nocopy_reshape(2, b.shape, b.strides, 1, (12,), [0], 8, False) == 0
    assert attempt_nocopy_reshape(2, (2, 3), (24, 8), 1, (7,), [0], 8, False) == 0


def test_squeeze_and_ravel():
    base = np.zeros((1, 3, 1, 4))
    d = Array.from_desc(0, base.shape, base.strides, 8)
    s, _ = d.squeeze()
    assert (s.shape, s.strides) == (base.squeeze().shape, base.squeeze().strides)
    s, _ = d.squeeze(axis=0)
    assert s.shape == (3, 1, 4)
    s, _ = d.squeeze(axis=(0, 2))
    assert s.shape == (3, 4)
    with pytest.raises(ValueError, match="cannot select an axis"):
        d.squeeze(axis=1)
    r, ext = d.ravel()
    assert r.shape == (12,) and r.strides == (8,) and ext == [d.extent]
    f = np.asfortranarray(np.zeros((3, 4)))
    df = Array.from_desc(0, f.shape, f.strides, 8)
    assert df.ravel(order="F")[0].shape == (12,)
    assert df.ravel(order="A")[0].shape == (12,)
    with pytest.raises(NotImplementedError):
        df.ravel(order="C")
    with pytest.raises(NotImplementedError):
        Array.from_desc(0, (3, 2), (32, 8), 8).ravel()


def test_iter_contiguous_extent_covers_exactly_the_items():
    base = np.arange(6 * 8, dtype=np.int32).reshape(6, 8)
    for v in (base, base[:, 2:5], base[::2, ::2], base.T[1:3]):
        d = Array.from_desc(*_desc(v, base), 4)
        covered = set()
        for lo, hi in d.iter_contiguous_extent():
            assert (hi - lo) % 4 == 0
            covered.update(range(lo, hi, 4))
        assert covered == set(_offsets(*_desc(v, base)))


def test_shape_must_be_ints():
    with pytest.raises(TypeError):
        Array.from_desc(0, (2.0, 3), (24, 8), 8)
