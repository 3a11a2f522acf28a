"""Functors for the translated-Reduce tests: what they compute, on which element types,
and from which operands the comparison is meaningful.

`fold` marks the functors that are associative and commutative on the operands drawn for
them, so that a reduction has ONE right answer whatever the order of association
(integers: bit for bit; floats: see the tolerance each test states)."""

import math
from math import sqrt as imported_sqrt

import numpy as np

SIGNED = ("int8", "int16", "int32", "int64")
UNSIGNED = ("uint8", "uint16", "uint32", "uint64")
INTS = SIGNED + UNSIGNED
FLOATS = ("float32", "float64")
COMPLEX = ("complex64", "complex128")

_weight = 3          # read from the module's globals by a functor below


def _closure_case():
    scale = 5
    return lambda a, b: a * scale + b - _weight


def abs_difference(a, b):
    if a > b:
        return a - b
    else:
        return b - a


def clipped_sum(a, b):
    s = a + b
    if s > 1000:
        s = 1000
    return s


class Case:
    def __init__(self, name, functor, dtypes, low, high, fold=False, exact=True, init=0, selects=False):
        self.name, self.functor, self.dtypes = name, functor, dtypes
        self.low, self.high, self.fold, self.exact, self.init = low, high, fold, exact, init
        self.selects = selects          # the result is one of the operands: no rounding, any order

    def operands(self, dtype, n, seed):
        dtype = np.dtype(dtype)
        rng = np.random.default_rng(seed)
        if dtype.kind == "b":
            return rng.integers(0, 2, n).astype(np.bool_)
        if dtype.kind in "iu":
            info = np.iinfo(dtype)
            lo = max(info.min, self.low)
            hi = min(info.max, self.high)
            return rng.integers(lo, hi, n, dtype=np.int64 if dtype.kind == "i" else np.uint64,
                                endpoint=True).astype(dtype)
        low, high = self.low, self.high
        if dtype == np.float16:
            low, high = max(low, -60000), min(high, 60000)
        if dtype.kind == "c":
            return ((rng.random(n) * (high - low) + low) + 1j * (rng.random(n) * (high - low) + low)).astype(dtype)
        return (rng.random(n) * (high - low) + low).astype(dtype)

    def __repr__(self):
        return self.name


FULL = (-2**63, 2**64 - 1)        # clipped to the element type

CASES = [
    Case("sum_plus_one", lambda a, b: a + b + 1, INTS + FLOATS + ("bool",), *FULL, fold=True, init=7),
    Case("one_plus_products", lambda a, b: a * b + a + b, INTS, *FULL, fold=True, init=2),
    Case("xor_and_flip", lambda a, b: a ^ b ^ 1, INTS, *FULL, fold=True, init=5),
    # (ties between x and -x go to the positive one: a total order, so any association agrees)
    Case("largest_magnitude", lambda a, b: a if abs(a) > abs(b) or (abs(a) == abs(b) and a > b) else b, SIGNED + FLOATS + ("float16",), -10**6, 10**6,
         fold=True, selects=True),
    Case("sum_modulo_prime", lambda a, b: (a + b) % 1000003, ("int32", "int64", "uint32", "uint64"), 0, 1000002,
         fold=True, init=11),
    Case("saturating_sum", lambda a, b: min(a + b, 1000), ("int16", "int32", "int64", "uint16", "uint32"), 0, 40,
         fold=True, init=3),
    Case("clipped_sum_statement", clipped_sum, ("int32", "uint64"), 0, 40, fold=True),
    Case("hypot_math", lambda a, b: math.sqrt(a * a + b * b), FLOATS, -100, 100, fold=True, exact=False, init=0),
    Case("hypot_numpy", lambda a, b: np.sqrt(a * a + b * b), FLOATS, -100, 100, fold=True, exact=False),
    Case("hypot_imported", lambda a, b: imported_sqrt(a * a + b * b), ("float64",), -100, 100, fold=True, exact=False),
    Case("log_sum_exp", lambda a, b: math.log(math.exp(a) + math.exp(b)), FLOATS, 1, 5, fold=True, exact=False),
    Case("different", lambda a, b: a != b, ("bool",), 0, 1, fold=True, init=False),
    Case("both_or_neither", lambda a, b: (a and b) or (not a and not b), ("bool",), 0, 1, fold=True, init=True),
    # one application at a time only: not associative
    Case("difference", lambda a, b: a - b, INTS + FLOATS, *FULL),
    Case("abs_difference_statement", abs_difference, INTS + FLOATS, -10**9, 10**9),
    Case("spread", lambda a, b: max(a, b) - min(a, b), INTS + FLOATS, -10**9, 10**9),
    Case("floor_division", lambda a, b: a // 3 + b // -7, SIGNED + FLOATS, -10**6, 10**6, exact=True),
    Case("floor_division_unsigned", lambda a, b: a // 3 + b % 5, UNSIGNED, 0, 10**6),
    Case("python_modulo", lambda a, b: a % 7 + b % -5, SIGNED, -10**6, 10**6),
    Case("shifts", lambda a, b: (a << 2) ^ (b >> 1), INTS, *FULL),
    Case("invert_negate", lambda a, b: ~a + -b, INTS, *FULL),
    Case("halves", lambda a, b: a / 2 + b / 4, INTS + FLOATS, -10**6, 10**6),
    Case("squares", lambda a, b: a ** 2 + b ** 3, ("int32", "int64", "uint32", "float64"), -1000, 1000, exact=False),
    Case("globals_and_closure", _closure_case(), INTS + FLOATS, -10**5, 10**5),
    Case("unsigned_against_negative", lambda a, b: a if a > -1 else b, UNSIGNED, *FULL),
    Case("nested_conditions", lambda a, b: a if (a > b and a > 0) or b < -5 else b, SIGNED + FLOATS, -20, 20),
    Case("floor_and_ceil", lambda a, b: math.floor(a / 3) + math.ceil(b / 3), ("int32", "float64"), -10**4, 10**4),
    Case("numpy_maximum", lambda a, b: np.maximum(a, b) - np.float32(2) * np.minimum(a, b), FLOATS, -50, 50),
    Case("float_constant", lambda a, b: 0.5 * a + b, FLOATS + ("int32",), -10**4, 10**4, exact=False),
    Case("nan_aware", lambda a, b: b if math.isnan(a) else a, FLOATS, -1, 1),
    Case("tangent", lambda a, b: math.atan2(a, b) + math.tanh(a), FLOATS, -3, 3, exact=False),
    # complex elements (complex64 only where nothing divides: see oracle.cref.typed_functor)
    Case("complex_sum_plus_i", lambda a, b: a + b + 1j, COMPLEX, -100, 100, fold=True, init=2 - 1j),
    Case("complex_product_mix", lambda a, b: a * b + a - b, COMPLEX, -2, 2),
    Case("complex_quotient", lambda a, b: a / (b + 2) - b / a, ("complex128",), -1.5, 1.5),
    Case("complex_quotient_narrow", lambda a, b: a / (b + 2), ("complex64",), -1.5, 1.5, exact=False),
    Case("conjugate_and_parts", lambda a, b: a.conjugate() * b + (a.real - b.imag), COMPLEX, -2, 2),
    Case("parts_of_real_numbers", lambda a, b: a.real + b.conjugate() - a.imag, ("int32", "float64"), -1000, 1000),
    Case("square_and_compare", lambda a, b: a ** 2 if a != b else -b, ("complex128",), -2, 2),
    Case("modulus", lambda a, b: abs(a) + abs(b) * 1j, COMPLEX, -3, 3, exact=False),
    Case("truth_of_complex", lambda a, b: a if a and not b == 0 else b + (1 + 2j), COMPLEX, -1, 1),
    Case("numpy_complex_constant", lambda a, b: np.complex64(0.5 + 0.25j) * np.conjugate(b) + a, COMPLEX, -8, 8),
]

BY_NAME = {c.name: c for c in CASES}

# what cannot be translated, with a fragment of the reason
REFUSED = [
    (lambda a, b: int(a) + b, "int()"),
    (lambda a, b: float(a) + b, "float()"),
    (lambda a, b: sum(x for x in range(a)), "index"),
    (lambda a, b: math.factorial(a) + b, "math.factorial"),
    (lambda a, b: "text", "not a number"),
    (lambda a, b: a[0] + b, "indexing"),
    (lambda a, b: a + "x", "TypeError"),
    (lambda a, b: np.cumsum(a), "not a number"),
    (lambda a, b: complex(a) + b, "complex()"),
    (lambda a, b: a.bit_length() + b, "AttributeError"),
]

# refused for complex elements with Python's own TypeError, when the element type is known
COMPLEX_TYPE_ERRORS = [
    (lambda a, b: a if a > b else b, "not supported"),
    (lambda a, b: max(a, b), "not supported"),
    (lambda a, b: a // b, "floor"),
    (lambda a, b: a % b, "floor or mod"),
    (lambda a, b: a ^ b, "bitwise"),
    (lambda a, b: math.sqrt(a) + b, "complex to float"),
    (lambda a, b: ~a + b, "unary"),
]
