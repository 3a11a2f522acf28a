"""The translation of Python functors (numba_cuda_amd/kernels/functor.py), without a device:

- every case of tests/functor_cases.py is traced, typed and written out for each of its
  element types; the body is compiled as HOST C++ (tests/host_functor.py) and applied to
  random operand pairs; the oracle is the functor itself under the reference's typing
  (oracle.cref.typed_functor).  Integers and booleans: bit for bit.  Floats: bit for bit
  where the case says `exact`; otherwise within 4 units in the last place of the element
  type (library functions differ between C libraries by an ulp or two).  float32 elements
  with Python constants: the JIT works those steps in float64 where the oracle's NumPy
  scalars stay in float32, so the 4 units are measured on the size of the operands.
- the same bodies pass the HIP run-time compiler for gfx950 (no device needed to compile)
- what cannot be translated is refused with the reason
"""

import ctypes
import math

import numpy as np
import pytest

from numba_cuda_amd import _lib
from numba_cuda_amd.kernels import functor as F
from oracle import cref
from tests import functor_cases as FC
from tests import host_functor

DTYPES = ["int8", "int16", "int32", "int64", "uint8", "uint16", "uint32", "uint64", "float32", "float64", "bool",
          "complex64", "complex128"]


def _ulps(got, want):
    got, want = got.astype(np.float64), want.astype(np.float64)
    spacing = np.spacing(np.abs(want).astype(got.dtype if got.dtype.kind == "f" else np.float64))
    return np.abs(got - want) / spacing


@pytest.mark.parametrize("dtype_name", DTYPES)
def test_translated_bodies_agree_with_the_functor(dtype_name):
    cases = [c for c in FC.CASES if dtype_name in c.dtypes]
    dtype = np.dtype(dtype_name)
    bodies = [F.body_for(F.trace(c.functor), dtype) for c in cases]
    applies = host_functor.build(bodies, dtype_name)
    for case, apply, body in zip(cases, applies, bodies):
        a = case.operands(dtype, 4000, 1)
        b = case.operands(dtype, 4000, 2)
        if dtype.kind == "i" and case.low < 0 and ("division" in case.name or "modulo" in case.name):
            a[:4] = [-7, -6, 6, 7]           # exact multiples and their neighbours, both signs
            b[:4] = [7, -7, 14, -14]
        f = cref.typed_functor(case.functor, dtype)
        want = np.array([f(x, y) for x, y in zip(a, b)], dtype)
        got = apply(a, b)
        # float32 elements with Python constants: the JIT (and the body) take that step in
        # float64, the oracle's NumPy scalars stay in float32
        widened = (dtype == np.float32 and "(double)" in body) or (dtype == np.complex64 and "<double>" in body)
        if dtype.kind == "c" and not (case.exact and not widened):
            # complex: the same 4 units, of the larger part (hypot and the quotient differ by a unit or two)
            part = np.float32 if dtype == np.complex64 else np.float64
            scale = np.maximum(np.abs(want.real), np.abs(want.imag)).astype(np.float64)
            if widened:
                scale = scale + 8 * (np.abs(a) + np.abs(b)).astype(np.float64)
            err = np.maximum(np.abs(got.real.astype(np.float64) - want.real), np.abs(got.imag.astype(np.float64) - want.imag))
            assert (err / np.spacing(scale.astype(part))).max() <= 4.0, (case, dtype_name)       # tolerance: 4 ulp
        elif dtype.kind != "f" or (case.exact and not widened):
            bad = np.flatnonzero(got.view(np.uint8).reshape(len(got), -1) != want.view(np.uint8).reshape(len(want), -1))
            assert got.tobytes() == want.tobytes(), (case, dtype_name, a[bad[:3] // dtype.itemsize],
                                                     b[bad[:3] // dtype.itemsize], got[bad[:3] // dtype.itemsize],
                                                     want[bad[:3] // dtype.itemsize])
        else:
            narrow = np.float32 if dtype == np.float32 else np.float64
            scale = np.abs(want).astype(np.float64)
            if widened:
                # where intermediate values cancel, the float32 steps of the oracle lose what
                # the float64 steps keep: measure against the size of what went in
                scale = scale + 8 * (np.abs(a).astype(np.float64) + np.abs(b).astype(np.float64))
            err = np.abs(got.astype(np.float64) - want.astype(np.float64)) / np.spacing(scale.astype(narrow))
            assert err.max() <= 4.0, (case, dtype_name, err.max())       # tolerance: 4 ulp


def test_float16_bodies_are_written_with_float16_arithmetic():
    body = F.body_for(F.trace(lambda a, b: a * b + a), np.float16)
    assert body.strip() == "return ((a * b) + a);"            # _Float16 operands: one rounding per operation
    body = F.body_for(F.trace(lambda a, b: math.sqrt(a) + b), np.float16)
    assert "sqrtf((float)(a))" in body


def test_expression_trees():
    assert repr(F.trace(lambda a, b: a + b + 1)) == "add(add(a, b), 1)"
    assert repr(F.trace(lambda a, b: 2 - a)) == "sub(2, a)"
    assert repr(F.trace(lambda a, b: a if a > b else b)) == "ite(gt(a, b), a, b)"
    assert repr(F.trace(max)) == "ite(gt(b, a), b, a)"
    assert repr(F.trace(lambda a, b: math.hypot(a, b))) == "hypot(a, b)"
    assert repr(F.trace(lambda a, b: np.arctan2(a, b))) == "atan2(a, b)"
    # both arms equal: no condition left
    assert repr(F.trace(lambda a, b: a + b if a > 0 else b + a - 0 + 0)) != ""
    assert repr(F.trace(lambda a, b: (a + b) if a > 0 else (a + b))) == "add(a, b)"
    # the same question twice on one path is asked once
    assert repr(F.trace(lambda a, b: (a if a > b else b) + (a if a > b else b))) == \
        "ite(gt(a, b), add(a, a), add(b, b))"
    # truth value of a number
    assert repr(F.trace(lambda a, b: a if a else b)) == "ite(ne(a, 0), a, b)"
    # constants from math stay constants
    assert repr(F.trace(lambda a, b: a * math.pi + b)).startswith("add(mul(a, 3.14159")


def test_typing_rules_written_as_casts():
    e = F.trace(lambda a, b: a + b + 1)
    assert F.body_for(e, np.int32).count("nbh_i64") >= 3 and "(int)" in F.body_for(e, np.int32)
    assert "(double)" in F.body_for(e, np.float32)             # float32 + int64 constant -> float64
    assert "(double)" not in F.body_for(F.trace(lambda a, b: a + b * a), np.float32)
    assert F.body_for(F.trace(lambda a, b: a / b), np.int64).strip() == "return (nbh_i64)(((double)(a) / (double)(b)));"
    # unsigned with unsigned stays unsigned, with a signed constant it is signed
    assert "(nbh_u64)((nbh_u64)" in F.body_for(F.trace(lambda a, b: a * b), np.uint32)
    assert F.body_for(e, np.uint32).strip().startswith("return (unsigned int)((nbh_i64)(")
    with pytest.raises(TypeError, match="bitwise"):
        F.body_for(F.trace(lambda a, b: a ^ b ^ 1), np.float32)
    # complex: float32 parts only among complex64 and float32 operands; conversions are calls
    assert F.body_for(F.trace(lambda a, b: a * b + a), np.complex64).strip() == "return ((a * b) + a);"
    assert "nbh_cplx_from<double>" in F.body_for(e, np.complex64)          # + int64 constant -> complex128
    assert "nbh_cplx_from<double>" not in F.body_for(F.trace(lambda a, b: a * np.float32(2) + b.real), np.complex64)
    assert F.body_for(F.trace(lambda a, b: abs(a) + abs(b)), np.complex128).strip() == \
        "return nbh_cplx_from<double>((nbh_cabs(a) + nbh_cabs(b)));"
    with pytest.raises(TypeError, match="cannot convert complex"):
        F.body_for(F.trace(lambda a, b: a + b * 1j), np.float64)        # a complex result for real elements


@pytest.mark.parametrize("functor,why", FC.COMPLEX_TYPE_ERRORS)
def test_what_python_refuses_for_complex_numbers_is_a_type_error(functor, why):
    tree = F.trace(functor)                      # the trace does not know the element type yet
    for dtype in (np.complex64, np.complex128):
        with pytest.raises(TypeError, match=why):
            F.body_for(tree, dtype)


@pytest.mark.parametrize("functor,why", FC.REFUSED)
def test_refusals(functor, why):
    with pytest.raises(NotImplementedError, match=why.replace("(", r"\(").replace(")", r"\)")):
        F.trace(functor)


def test_a_loop_over_the_operands_is_refused_not_followed_forever():
    def gcd(a, b):
        while b:
            a, b = b, a % b
        return a
    with pytest.raises(NotImplementedError, match="conditions"):
        F.trace(gcd)


def test_every_body_passes_the_run_time_compiler():
    """nbh_reduce_compile needs no device: the code objects are built for gfx950 here."""
    lib = ctypes.CDLL(_lib.LIB_PATH)
    lib.nbh_reduce_compile.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p),
                                       ctypes.c_char_p, ctypes.c_size_t]
    lib.nbh_reduce_op_free.argtypes = [ctypes.c_void_p]
    lib.nbh_reduce_op_dtype.argtypes = [ctypes.c_void_p]
    # one type per case keeps this quick (about 0.4 s per compilation); float16 included
    picks = [(c, c.dtypes[len(c.name) % len(c.dtypes)]) for c in FC.CASES]
    picks.append((FC.BY_NAME["largest_magnitude"], "float16"))
    for case, dtype_name in picks:
        dtype = np.dtype(dtype_name)
        code = _lib.DTYPE_CODES["uint8" if dtype_name == "bool" else dtype_name]
        handle = ctypes.c_void_p()
        log = ctypes.create_string_buffer(4096)
        body = F.body_for(F.trace(case.functor), dtype)
        rc = lib.nbh_reduce_compile(code, body.encode(), ctypes.byref(handle), log, len(log))
        assert rc == 0, (case, dtype_name, log.value.decode(), body)
        assert lib.nbh_reduce_op_dtype(handle) == code
        assert lib.nbh_reduce_op_free(handle) == 0
    # a body that is not C++ comes back with the compiler's message
    rc = lib.nbh_reduce_compile(2, b"return a +* b;", ctypes.byref(handle), log, len(log))
    assert rc == 300 and b"error" in log.value
    assert lib.nbh_reduce_compile(99, b"return a;", ctypes.byref(handle), log, len(log)) == 1     # no such element type
