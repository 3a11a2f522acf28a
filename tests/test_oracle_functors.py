"""Pins the oracle's Python restatements for general functors (oracle/cref.py
functor_fold / functor_tree / typed_functor) against what is already pinned: the C
restatements orc_fold_* / orc_tree_* for the four standard operators (bit for bit, with
float32 sums, which move when the association order moves), and closed forms on wrapped
integers for the typing."""

import numpy as np
import pytest

from oracle import cref

STANDARD = [("add", lambda a, b: a + b), ("mul", lambda a, b: a * b), ("max", lambda a, b: max(a, b)),
            ("min", lambda a, b: a if a < b else b)]


@pytest.mark.parametrize("n", [1, 2, 31, 32, 33, 127, 128, 129, 255, 1000, 8192, 8192 + 77, 8192 + 128, 20000])
def test_tree_and_fold_orders_match_the_c_restatement(n):
    rng = np.random.default_rng(n)
    f32 = rng.standard_normal(n).astype(np.float32)
    i32 = rng.integers(-2**31, 2**31, n).astype(np.int32)
    u8 = rng.integers(0, 256, n).astype(np.uint8)
    for name, functor in STANDARD:
        for data, init in ((f32, 0.5), (i32, 3), (u8, 1)):
            if name == "mul" and data.dtype.kind == "f":
                data = (1 + data / 64).astype(np.float32)
            assert cref.functor_tree(functor, data, init).tobytes() == cref.tree(name, data, init).tobytes()
            assert cref.functor_fold(functor, data, init).tobytes() == cref.fold(name, data, init).tobytes()


def test_typing_on_wrapped_integers_closed_forms():
    rng = np.random.default_rng(5)
    for dtype in (np.int8, np.uint8, np.int32, np.uint32, np.int64, np.uint64):
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, 3000, dtype=dtype, endpoint=True)
        exact = [int(x) for x in a]
        bits = 8 * np.dtype(dtype).itemsize

        def wrap(v):
            v &= (1 << bits) - 1
            return v - (1 << bits) if info.min < 0 and v >= 1 << (bits - 1) else v
        # a + b + 1 over n elements and init: sum + init + n
        assert int(cref.functor_tree(lambda x, y: x + y + 1, a, 7)) == wrap(sum(exact) + 7 + len(exact))
        # a * b + a + b = (a + 1)(b + 1) - 1
        prod = 1
        for x in exact + [2]:
            prod = prod * (x + 1) % (1 << 64)
        assert int(cref.functor_tree(lambda x, y: x * y + x + y, a, 2)) == wrap(prod - 1)
        assert int(cref.functor_fold(lambda x, y: x * y + x + y, a, 2)) == wrap(prod - 1)


def test_typing_of_booleans_and_float_results():
    f = cref.typed_functor(lambda a, b: a + b, np.bool_)
    assert f(True, True) is np.True_ and f(False, False) is np.False_
    g = cref.typed_functor(lambda a, b: a / 2 + b / 2, np.int32)
    assert g(np.int32(-3), np.int32(0)) == -1 and isinstance(g(1, 1), np.int32)       # towards zero
    h = cref.typed_functor(lambda a, b: a * b, np.float32)
    assert h(np.float32(1.1), np.float32(1.1)) == np.float32(1.1) * np.float32(1.1)


@pytest.mark.parametrize("n", [1, 2, 33, 127, 129, 1000, 8192 + 77, 20000])
def test_complex_elements_match_the_c_restatement(n):
    """complex128 runs on Python complex numbers, complex64 on NumPy scalars: sums and products
    must come out as the C restatement's (part by part; (ac - bd) + (ad + bc)i), in tree and
    fold order."""
    rng = np.random.default_rng(n)
    for dtype in (np.complex64, np.complex128):
        z = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dtype)
        near_one = (1 + z / 64).astype(dtype)
        for name, functor, data in (("add", lambda a, b: a + b, z), ("mul", lambda a, b: a * b, near_one)):
            assert cref.functor_tree(functor, data, 0.5 - 2j).tobytes() == cref.tree(name, data, 0.5 - 2j).tobytes()
            assert cref.functor_fold(functor, data, 0.5 - 2j).tobytes() == cref.fold(name, data, 0.5 - 2j).tobytes()


def test_complex128_quotient_is_the_algorithm_the_jit_lowers():
    """typed_functor divides complex128 with Python's own `/`.  The reference lowers the quotient
    as written at numba/cuda/cpython/numbers.py:1150-1177 (scale by the larger part of the
    divisor): Python's must be that algorithm to the bit, also where the two parts of the
    divisor are equal in size, of opposite sign, or one of them zero."""
    def lowered(a, b):
        if abs(b.real) >= abs(b.imag):
            ratio = b.imag / b.real
            denom = b.real + b.imag * ratio
            return complex((a.real + a.imag * ratio) / denom, (a.imag - a.real * ratio) / denom)
        ratio = b.real / b.imag
        denom = b.real * ratio + b.imag
        return complex((a.real * ratio + a.imag) / denom, (a.imag * ratio - a.real) / denom)

    rng = np.random.default_rng(11)
    a = rng.standard_normal(20000) + 1j * rng.standard_normal(20000)
    b = rng.standard_normal(20000) * 10.0 ** rng.integers(-3, 4, 20000) + 1j * rng.standard_normal(20000)
    b[:4] = [1 + 1j, 2 - 2j, 3 + 0j, 0 - 5j]
    f = cref.typed_functor(lambda x, y: x / y, np.complex128)
    for x, y in zip(a, b):
        want = lowered(complex(x), complex(y))
        assert f(x, y).tobytes() == np.complex128(want).tobytes(), (x, y)
