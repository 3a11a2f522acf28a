"""Pins the reduction, transpose and extent parts of the oracle.

Known answers held by the reference's own tests
(numba_cuda/numba/cuda/tests/cudapy/test_reduction.py:15-90,
 test_transpose.py:16-86) plus what the mathematics fixes.
"""

import math
import operator

import numpy as np
import pytest

from oracle import cref, reduce_simt, sim

# test_reduction.py:29-45
REFERENCE_SIZES = [1, 15, 16, 17, 127, 128, 129, 1023, 1024, 1025, 1536,
                   1048576, 1049600, 1049728, 34567]


@pytest.mark.parametrize("n", REFERENCE_SIZES)
def test_sum_of_1_to_n_is_exact(n):
    a = np.arange(n, dtype=np.float64) + 1
    want = n * (n + 1) // 2          # closed form, exact below 2^53
    assert cref.tree("add", a) == want
    assert cref.fold("add", a) == want


def test_empty_returns_init():
    a = np.arange(0, dtype=np.float64)
    assert cref.tree("add", a) == 0
    assert cref.tree("add", a, 7) == 7
    assert cref.fold("mul", a, 3) == 3


def test_prod_1_to_64():
    # test_reduction.py:63-68
    a = np.arange(64, dtype=np.float64) + 1
    np.testing.assert_allclose(cref.tree("mul", a, 1), float(math.factorial(64)), rtol=1e-12)
    np.testing.assert_allclose(cref.fold("mul", a, 1), float(math.factorial(64)), rtol=1e-12)


def test_max_1_to_3717_and_init_3():
    a = np.arange(3717, dtype=np.float64) + 1
    assert cref.tree("max", a, 0) == 3717
    assert cref.tree("min", a, 5000) == 1
    b = np.arange(10, dtype=np.float64) + 1
    assert cref.tree("add", b, 3) == 58


SIMT_SIZES = [1, 2, 31, 32, 33, 63, 64, 65, 95, 96, 97, 127, 128, 129, 160, 161, 255, 256,
              257, 1000, 4095, 4096, 4097, 8191, 8192, 8193, 8320, 8321, 16384, 16385 + 128,
              20000, 34567, 65536, 100003]


@pytest.mark.parametrize("n", SIMT_SIZES)
def test_tree_order_matches_literal_simt_emulation_f32(n):
    """float32 sums expose the association order: the closed-form C loops and
    the statement-by-statement kernel emulation must agree to the bit."""
    rng = np.random.default_rng(n)
    a = (rng.standard_normal(n) * 1000).astype(np.float32)
    init = np.float32(0.37)
    for op in ("add", "max", "min"):
        got = cref.tree(op, a, init)
        want = reduce_simt.reduce(op, a, init)
        assert got.tobytes() == want.tobytes(), (op, n)
    # products: keep magnitudes near 1 so nothing over/underflows
    b = (1.0 + rng.standard_normal(n) * 1e-3).astype(np.float32)
    assert cref.tree("mul", b, 1).tobytes() == reduce_simt.reduce("mul", b, 1).tobytes()


def test_tree_order_is_not_the_left_fold():
    """Guards the previous test against vacuity: on float32 data the two
    association orders give different bits."""
    rng = np.random.default_rng(0)
    a = (rng.standard_normal(50000) * 1000).astype(np.float32)
    assert cref.tree("add", a) != cref.fold("add", a)


def test_tree_small_cases_by_hand():
    # n = 3 (tail launch only, one partially filled warp): ((a0+a1)+a2)+init
    a = np.array([1e8, 1.0, -1e8], np.float32)
    want = np.float32(np.float32(np.float32(a[0] + a[1]) + a[2]) + np.float32(0.5))
    assert cref.tree("add", a, 0.5) == want
    # n = 33: warp 0 is full (tree), warp 1 holds one value; result (tree + a32) + init
    rng = np.random.default_rng(5)
    a = (rng.standard_normal(33) * 100).astype(np.float32)
    v = a[:32].copy()
    for width in (16, 8, 4, 2, 1):
        v[:width] = v[:width] + v[width:2 * width]
    want = np.float32(np.float32(v[0] + a[32]) + np.float32(2.0))
    assert cref.tree("add", a, 2.0) == want
    # n = 32: the only warp is exactly full but still folded sequentially
    # (strict '<' at reduction.py:119)
    a = (rng.standard_normal(32) * 100).astype(np.float32)
    acc = a[0]
    for x in a[1:]:
        acc = np.float32(acc + x)
    assert cref.tree("add", a, 0) == np.float32(acc + np.float32(0))


@pytest.mark.parametrize("sfx", list(cref.SUFFIX))
@pytest.mark.parametrize("op", cref.OPS)
def test_all_ops_all_dtypes_brute_force(op, sfx):
    dt = np.dtype(cref.SUFFIX[sfx])
    rng = np.random.default_rng(hash((op, sfx)) % 2**32)
    pyop = {"add": operator.add, "mul": operator.mul, "max": max, "min": min}[op]
    for n in (1, 5, 130, 1000, 9000):
        if dt.kind == "f":
            a = (1.0 + rng.standard_normal(n) * 1e-2).astype(dt)
            init = dt.type(1)
            want = math.fsum(a.tolist()) + 1 if op == "add" else None
            got_t, got_f = cref.tree(op, a, init), cref.fold(op, a, init)
            if op == "add":
                tol = 2 * n * np.finfo(dt).eps * np.abs(a).sum()
                assert abs(float(got_t) - want) <= tol and abs(float(got_f) - want) <= tol
            elif op == "mul":
                want = np.prod(a.astype(np.longdouble)) * 1
                assert abs(got_t / want - 1) < n * np.finfo(dt).eps * 4
                assert abs(got_f / want - 1) < n * np.finfo(dt).eps * 4
            else:
                assert got_t == got_f == pyop(float(pyop(a.tolist())), 1.0)
        else:
            info = np.iinfo(dt)
            a = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
            init = 3
            acc = 3
            for x in a.tolist():
                acc = pyop(acc, x)
            bits = dt.itemsize * 8
            acc &= (1 << bits) - 1              # python big-int, then wrap
            if dt.kind == "i" and acc >= 1 << (bits - 1):
                acc -= 1 << bits
            assert int(cref.tree(op, a, init)) == acc
            assert int(cref.fold(op, a, init)) == acc


@pytest.mark.parametrize("sfx", list(cref.INT_SUFFIX))
@pytest.mark.parametrize("op", cref.BITWISE_OPS)
def test_bitwise_ops_against_numpy(op, sfx):
    """and / or / xor are associative and commutative: both orders of the oracle must give
    NumPy's left-to-right result, bit for bit, for every integer type."""
    dt = np.dtype(cref.SUFFIX[sfx])
    info = np.iinfo(dt)
    ufunc = {"and": np.bitwise_and, "or": np.bitwise_or, "xor": np.bitwise_xor}[op]
    rng = np.random.default_rng(abs(hash((op, sfx))) % 2**32)
    for n in (1, 2, 31, 32, 33, 127, 128, 129, 4097, 70001):
        a = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        if op == "and":
            a |= rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        for init in (0, 5, info.max, info.min):
            want = ufunc(ufunc.reduce(a), dt.type(init))
            assert cref.fold(op, a, init) == want
            assert cref.tree(op, a, init) == want


def test_minmax_follow_python_semantics_for_nan_and_signed_zero():
    # cpython/builtins.py:224-269: max(a, b) = b if b > a else a
    a = np.array([np.nan, 1.0, 2.0], np.float64)
    assert np.isnan(sim.Reduce(lambda x, y: max(x, y))(a, init=np.float64(np.nan)))
    assert np.isnan(cref.fold("max", a, np.nan))
    # NaN first in the data but a number as init: every comparison with the
    # NaN is False so the accumulator survives until a bigger number comes
    assert cref.fold("max", a, 0.0) == 2.0
    z = np.array([0.0, -0.0], np.float64)
    assert math.copysign(1, cref.fold("max", z, -0.0)) == -1.0   # ties keep the earlier operand
    assert math.copysign(1, cref.fold("min", z, 0.0)) == 1.0


def test_complex_reductions_of_the_oracle():
    """Pins: componentwise sums equal the real-valued oracle on each component (same
    association); products of Gaussian integers are exact and equal NumPy's; a
    conjugated input gives the conjugated product (sign symmetry of the formula)."""
    rng = np.random.default_rng(4)
    for dt, real in ((np.complex64, np.float32), (np.complex128, np.float64)):
        for n in (1, 31, 32, 33, 127, 128, 129, 8192, 8321, 20000):
            a = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dt)
            for fam in (cref.fold, cref.tree):
                got = fam("add", a, 0.5 - 0.25j)
                re = fam("add", np.ascontiguousarray(a.real), real(0.5))
                im = fam("add", np.ascontiguousarray(a.imag), real(-0.25))
                assert (got.real, got.imag) == (re, im)
        g = (rng.integers(-3, 4, 12) + 1j * rng.integers(-3, 4, 12)).astype(dt)
        want = np.prod(g.astype(np.complex128))
        assert cref.fold("mul", g, 1) == want == cref.tree("mul", g, 1)
        u = np.exp(1j * rng.uniform(0, 6, 300)).astype(dt)
        assert cref.tree("mul", np.conj(u), 1) == np.conj(cref.tree("mul", u, 1))
        assert abs(abs(cref.tree("mul", u, 1)) - 1) < 300 * 4 * np.finfo(real).eps


def test_fold_matches_simulator_path():
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, 65536).astype(np.float32)       # the 65536-element simulator case
    got = sim.Reduce(lambda x, y: x + y)(a[:4096], init=0)
    assert isinstance(got, np.float32)
    assert got == cref.fold("add", a[:4096], 0)


def test_sum_exact_yardstick():
    a = np.array([1e30, 1.0, -1e30, 1e-3], np.float64)
    s, sa = cref.sum_exact(a)
    assert s == math.fsum(a.tolist())
    assert sa == math.fsum(np.abs(a).tolist())
    b = np.arange(1, 100001, dtype=np.float32)
    assert cref.sum_exact(b)[0] == 100000 * 100001 / 2


# ---------------------------------------------------------------- transpose

recordwith2darray = np.dtype([("i", np.int32), ("j", np.float32, (3, 2))])


@pytest.mark.parametrize("rows,cols,dtype", [(5, 6, np.float64), (128, 128, np.complex128),
                                             (1025, 512, np.float64), (3, 1, np.int8)])
def test_transpose_reference_variants(rows, cols, dtype):
    # test_transpose.py:17-32
    x = np.arange(rows * cols, dtype=dtype).reshape(cols, rows)
    y = cref.transpose(x)
    assert y.flags["C_CONTIGUOUS"] and y.shape == (rows, cols)
    np.testing.assert_array_equal(x.transpose(), y)


@pytest.mark.parametrize("rows,cols", [(2, 3), (16, 16), (16, 17), (17, 16), (14, 15), (15, 14), (14, 14)])
def test_transpose_record_and_bool(rows, cols):
    # test_transpose.py:33-71; 28-byte items
    assert recordwith2darray.itemsize == 28
    arr = np.zeros((rows, cols), dtype=recordwith2darray)
    for x in range(rows):
        for y in range(cols):
            arr[x, y]["i"] = x ** 2 + y
            arr[x, y]["j"] = np.arange(6, dtype=np.float32).reshape(3, 2) * x + y
    np.testing.assert_array_equal(arr.T, cref.transpose(arr))
    b = np.random.default_rng(rows * cols).integers(0, 2, (rows, cols)).astype(np.bool_)
    np.testing.assert_array_equal(b.T, cref.transpose(b))


def test_transpose_strided_views():
    # test_transpose.py:73-86
    a = np.arange(120, dtype=np.int64).reshape((10, 12))
    v = a[::2, ::2]
    t = cref.transpose(v)
    assert t.shape == (6, 5) and t.strides == (40, 8)
    np.testing.assert_array_equal(v.T, t)
    np.testing.assert_array_equal(a[::-1, ::3].T, cref.transpose(a[::-1, ::3]))
    f = np.asfortranarray(a)
    np.testing.assert_array_equal(f.T, cref.transpose(f))
    assert np.array_equal(cref.transpose(cref.transpose(v)), v)     # involution


# ------------------------------------------------------------------ extents

@pytest.mark.parametrize("shape,strides,itemsize", [
    ((10,), (8,), 8), ((10, 12), (96, 8), 8), ((5, 6), (192, 16), 8), ((4, 3), (-24, 8), 8),
    ((4, 3), (24, -8), 8), ((0, 3), (24, 8), 8), ((), (), 4), ((3, 4), (0, 4), 4), ((1, 1), (100, 100), 2),
])
def test_extents_against_numpy(shape, strides, itemsize):
    lo, hi = cref.extents(shape, strides, itemsize)
    if 0 in shape:
        assert (lo, hi) == (0, 0)
        return
    # brute force over every element's byte range
    idx = np.indices(shape).reshape(len(shape), -1).T if shape else np.zeros((1, 0), int)
    offs = (idx * np.asarray(strides, int)).sum(axis=1) if shape else np.array([0])
    assert lo == offs.min() and hi == offs.max() + itemsize


# ---------------------------------------------------------------- float16 and boolean elements

def test_software_float16_matches_numpy_on_every_bit_pattern():
    bits = np.arange(65536, dtype=np.uint16)
    as_double = bits.view(np.float16).astype(np.float64)
    for b, want in zip(bits.tolist(), as_double.tolist()):
        got = cref.f16_to_double(b)
        assert got == want or (got != got and want != want), b
        if want == want:
            assert cref.f16_from_double(want) == b, b
    # rounding: random doubles, the overflow boundary, the subnormal range, ties
    rng = np.random.default_rng(5)
    x = np.concatenate([rng.standard_normal(30000) * 10.0 ** rng.integers(-9, 6, 30000),
                        [65519.999, 65520.0, 65504.0, 1e-8, 2.9802322387695312e-08, 2.98e-8, 8.9406967163085938e-08,
                         1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -14 - 2.0 ** -25, -0.0]])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([cref.f16_from_double(v) for v in x], dtype=np.uint16)
    assert (want == got).all()


@pytest.mark.parametrize("n", [1, 2, 31, 33, 127, 128, 129, 1000, 4097, 8192, 8321, 20000])
def test_float16_folds_and_trees_round_once_per_operation(n):
    """Left fold against functools.reduce over NumPy float16 scalars (NumPy computes
    each operation in float32 and rounds to float16: one effective rounding), tree
    against the statement-by-statement kernel emulation run on float16 arrays."""
    import functools
    rng = np.random.default_rng(n)
    a = (rng.standard_normal(n) * 4).astype(np.float16)
    init = np.float16(0.37)
    with np.errstate(over="ignore"):
        for op, fn in (("add", lambda x, y: x + y), ("max", lambda x, y: y if y > x else x),
                       ("min", lambda x, y: y if y < x else x)):
            assert cref.fold(op, a, init).tobytes() == functools.reduce(fn, a, init).tobytes(), (op, n)
            assert cref.tree(op, a, init).tobytes() == reduce_simt.reduce(op, a, init).tobytes(), (op, n)
        b = (1.0 + rng.standard_normal(n) * 1e-2).astype(np.float16)
        assert cref.fold("mul", b, 1).tobytes() == functools.reduce(lambda x, y: x * y, b, np.float16(1)).tobytes()
        assert cref.tree("mul", b, 1).tobytes() == reduce_simt.reduce("mul", b, 1).tobytes()
    assert cref.fold("add", a, init).dtype == np.float16


def test_float16_sum_shows_its_own_rounding():
    # 2048 + 1 is not a float16: a half accumulator sticks at 2048, a wider one would not
    a = np.ones(4000, np.float16)
    assert cref.fold("add", a, 0) == 2048
    assert cref.tree("add", a, 0) == 4000        # 8192 lanes hold one element each; the tree adds equal powers of two


@pytest.mark.parametrize("n", [1, 2, 33, 127, 129, 5000, 8321])
def test_boolean_sums_and_products_are_any_and_all(n):
    rng = np.random.default_rng(n)
    for p in (0.0, 1.0, 0.5, 1.0 / n):
        a = rng.random(n) < p
        for init in (False, True, 0, 1, 2):
            for fam in (cref.fold, cref.tree):
                got = fam("add", a, init)
                assert got.dtype == np.bool_ and got == (a.any() or bool(init)), (n, p, init)
                got = fam("mul", a, init)
                assert got.dtype == np.bool_ and got == (a.all() and bool(init)), (n, p, init)
