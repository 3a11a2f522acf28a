"""ctypes access to oracle/liboracle.so (the C restatement in oracle.c).

Test infrastructure: see the package docstring.
"""

import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

_c_i64 = ctypes.c_int64
_c_u64 = ctypes.c_uint64
_vp = ctypes.c_void_p

# dtype name used in the C symbol names -> numpy dtype
SUFFIX = {
    "i8": np.int8, "i16": np.int16, "i32": np.int32, "i64": np.int64,
    "u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64,
    "f32": np.float32, "f64": np.float64,
}
# float16 (carried as its 16 bits in C) takes the four arithmetic operators; booleans
# take add and mul here (their and / or / xor / max / min run as uint8)
HALF_SUFFIX = {"f16": np.float16}
BOOL_SUFFIX = {"b1": np.bool_}
BOOL_OPS = ("add", "mul")
# complex elements reduce with add and mul only
COMPLEX_SUFFIX = {"c64": np.complex64, "c128": np.complex128}
COMPLEX_OPS = ("add", "mul")
_SUFFIX_OF = {np.dtype(v): k for k, v in list(SUFFIX.items()) + list(COMPLEX_SUFFIX.items())
              + list(HALF_SUFFIX.items()) + list(BOOL_SUFFIX.items())}
OPS = ("add", "mul", "max", "min")
# bitwise functors exist for the integer element types only
BITWISE_OPS = ("and", "or", "xor")
INT_SUFFIX = {k: v for k, v in SUFFIX.items() if np.dtype(v).kind in "iu"}

STATE_DTYPE = np.dtype([("s0", np.uint64), ("s1", np.uint64)], align=True)


def build(force=False):
    """Compile oracle.c with the Makefile beside it."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-s"] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_xoro_seed_state.argtypes = [_c_u64, _vp]
        L.orc_xoro_next.argtypes = [_vp]
        L.orc_xoro_next.restype = _c_u64
        L.orc_xoro_jump.argtypes = [_vp]
        L.orc_xoro_init_states.argtypes = [_vp, _c_i64, _c_u64, _c_u64]
        L.orc_u64_to_unit_f64.argtypes = [_c_u64]
        L.orc_u64_to_unit_f64.restype = ctypes.c_double
        L.orc_u64_to_unit_f32.argtypes = [_c_u64]
        L.orc_u64_to_unit_f32.restype = ctypes.c_float
        for kind in ("uniform_f32", "uniform_f64", "normal_f32", "normal_f64"):
            getattr(L, "orc_xoro_fill_" + kind).argtypes = [_vp, _c_i64, _vp, _c_i64]
        for op in OPS:
            for sfx in SUFFIX:
                for fam in ("fold", "tree"):
                    getattr(L, f"orc_{fam}_{op}_{sfx}").argtypes = [_vp, _c_i64, _vp, _vp]
        for op in BITWISE_OPS:
            for sfx in INT_SUFFIX:
                for fam in ("fold", "tree"):
                    getattr(L, f"orc_{fam}_{op}_{sfx}").argtypes = [_vp, _c_i64, _vp, _vp]
        for op in COMPLEX_OPS:
            for sfx in COMPLEX_SUFFIX:
                for fam in ("fold", "tree"):
                    getattr(L, f"orc_{fam}_{op}_{sfx}").argtypes = [_vp, _c_i64, _vp, _vp]
        for fam in ("fold", "tree"):
            for op in OPS:
                getattr(L, f"orc_{fam}_{op}_f16").argtypes = [_vp, _c_i64, _vp, _vp]
            for op in BOOL_OPS:
                getattr(L, f"orc_{fam}_{op}_b1").argtypes = [_vp, _c_i64, _vp, _vp]
        L.orc_f16_to_double.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_double.restype = ctypes.c_double
        L.orc_f16_from_double.argtypes = [ctypes.c_double]
        L.orc_f16_from_double.restype = ctypes.c_uint16
        L.orc_sum_exact_f32.argtypes = [_vp, _c_i64, _vp, _vp]
        L.orc_sum_exact_f64.argtypes = [_vp, _c_i64, _vp, _vp]
        L.orc_transpose.argtypes = [_vp, _vp] + [_c_i64] * 7
        L.orc_extents.argtypes = [_vp, _vp, ctypes.c_int, _c_i64, _vp, _vp]
        _lib = L
    return _lib


def _ptr(a):
    return a.ctypes.data


# ----------------------------------------------------------------------------
# RNG
# ----------------------------------------------------------------------------

def seed_state(seed):
    s = np.zeros(2, np.uint64)
    lib().orc_xoro_seed_state(int(seed) & (2**64 - 1), _ptr(s))
    return int(s[0]), int(s[1])


def next_u64(state):
    """state: uint64[2] array, advanced in place; returns the draw."""
    return int(lib().orc_xoro_next(_ptr(state)))


def jump(state):
    lib().orc_xoro_jump(_ptr(state))


def init_states(n, seed, subsequence_start=0):
    states = np.zeros(n, STATE_DTYPE)
    lib().orc_xoro_init_states(_ptr(states), n, int(seed) & (2**64 - 1),
                               int(subsequence_start) & (2**64 - 1))
    return states


def u64_to_unit_f64(x):
    return float(lib().orc_u64_to_unit_f64(int(x)))


def u64_to_unit_f32(x):
    return np.float32(lib().orc_u64_to_unit_f32(int(x)))


def fill(states, count, kind):
    """kind in uniform_f32/uniform_f64/normal_f32/normal_f64.  Advances a copy
    of `states`; returns (out[n*count] thread-major, new_states)."""
    st = np.ascontiguousarray(states).copy()
    n = st.shape[0]
    out = np.empty(n * count, np.float32 if kind.endswith("f32") else np.float64)
    getattr(lib(), "orc_xoro_fill_" + kind)(_ptr(st), n, _ptr(out), count)
    return out, st


# ----------------------------------------------------------------------------
# Reduction
# ----------------------------------------------------------------------------

def f16_to_double(bits):
    return float(lib().orc_f16_to_double(int(bits)))


def f16_from_double(x):
    """Bit pattern of the float16 nearest to x (ties to even)."""
    return int(lib().orc_f16_from_double(float(x)))


def _reduce(fam, op, a, init):
    a = np.ascontiguousarray(a)
    sfx = _SUFFIX_OF[a.dtype]
    ini = np.array([a.dtype.type(init)], dtype=a.dtype)     # arr.dtype.type(init), kernels/reduction.py:224
    out = np.zeros(1, a.dtype)
    getattr(lib(), f"orc_{fam}_{op}_{sfx}")(_ptr(a), a.size, _ptr(ini), _ptr(out))
    return out[0]


def fold(op, a, init=0):
    """Strict left fold (the simulator's order)."""
    return _reduce("fold", op, a, init)


def tree(op, a, init=0):
    """The association order of the reference's CUDA kernels."""
    return _reduce("tree", op, a, init)


# ---- general functors --------------------------------------------------------------
# Pure Python: for small inputs only.  Pinned by tests/test_oracle_functors.py: with
# a + b, a * b, max and min these give, bit for bit, what the C restatements orc_fold_* /
# orc_tree_* above give (float32 sums included, which are sensitive to the order), and the
# typing is checked against closed forms on wrapped integers.

def typed_functor(functor, dtype):
    """functor(a, b) on elements of `dtype`, converted back to `dtype`, the way the
    reference's JIT types it (kernels/reduction.py:15-20 compiles the functor for the
    element type; the kernels store every intermediate result in arrays of that type,
    :32-37, :96):
      integers  operands enter as exact integers (the JIT computes in 64 bits: equal
                after the final wrap for + - * & | ^ and for everything else as long as
                no intermediate value leaves 64 bits), the result wraps to the type
      booleans  operands are bools, the result is `!= 0`
      float64   Python floats are float64
      complex128  Python complex numbers: their product is (ac - bd) + (ad + bc)i and their
                quotient CPython's algorithm, which is what the JIT lowers
                (numba/cuda/cpython/numbers.py:1123-1179)
      complex64  NumPy scalars: sums, differences and products part by part in float32
                like the JIT's; NumPy's QUOTIENT is another algorithm (it multiplies by a
                reciprocal), so complex64 functors that divide agree to rounding only
      float32 / float16  NumPy scalars of that type.  A Python float constant in the
                functor makes the JIT compute that step in float64, NumPy keeps it in
                the narrow type: such functors agree to the narrow type's rounding."""
    dtype = np.dtype(dtype)
    if dtype.kind in "iu":
        bits = 8 * dtype.itemsize
        mask, top = (1 << bits) - 1, 1 << (bits - 1)

        def on_integers(a, b):
            r = functor(int(a), int(b))
            if isinstance(r, (float, np.floating)):
                r = int(r)                   # conversion of a float result: towards zero
            r = int(r) & mask
            if dtype.kind == "i" and r >= top:
                r -= 1 << bits
            return dtype.type(r)
        return on_integers
    if dtype.kind == "b":
        return lambda a, b: np.bool_(bool(functor(bool(a), bool(b))))
    if dtype == np.dtype(np.float64):
        return lambda a, b: np.float64(functor(float(a), float(b)))
    if dtype == np.dtype(np.complex128):
        return lambda a, b: np.complex128(functor(complex(a), complex(b)))
    scalar = dtype.type
    narrow = _with_narrow_math(functor, scalar)

    def on_narrow_floats(a, b):
        with np.errstate(all="ignore"):
            return scalar(narrow(scalar(a), scalar(b)))
    return on_narrow_floats


class _NarrowMath:
    """`math` whose functions return the narrow float type when they are given one: the
    JIT types math.exp(float32) as float32 (the float32 routine), while Python's math
    module works in float64 - one rounding of the float64 value stands in for it."""

    def __init__(self, scalar):
        self._scalar = scalar

    def wrap(self, fn):
        scalar = self._scalar

        def narrow(*args):
            out = fn(*[float(x) if isinstance(x, np.floating) else x for x in args])
            if isinstance(out, float) and any(isinstance(x, scalar) for x in args):
                return scalar(out)
            return out
        return narrow

    def __getattr__(self, name):
        value = getattr(math, name)
        return self.wrap(value) if callable(value) else value


def _with_narrow_math(functor, scalar):
    import types
    if not isinstance(functor, types.FunctionType):
        return functor
    proxy = _NarrowMath(scalar)

    def swap(value):
        if value is math:
            return proxy
        if isinstance(value, types.BuiltinFunctionType) and getattr(math, value.__name__, None) is value:
            return proxy.wrap(value)
        return value
    new_globals = dict(functor.__globals__)
    for name in functor.__code__.co_names:
        if name in new_globals:
            new_globals[name] = swap(new_globals[name])
    closure = functor.__closure__
    if closure:
        closure = tuple(types.CellType(swap(c.cell_contents)) for c in closure)
    clone = types.FunctionType(functor.__code__, new_globals, functor.__name__, functor.__defaults__, closure)
    clone.__kwdefaults__ = functor.__kwdefaults__
    return clone


def functor_fold(functor, a, init=0):
    """simulator/reduction.py:7-19: functools.reduce(functor, a, init), typed."""
    a = np.asarray(a)
    f = typed_functor(functor, a.dtype)
    acc = a.dtype.type(init)
    for x in a:
        acc = f(acc, x)
    return acc


_WARP, _NWARPS, _MAXGRID = 32, 4, 64


def functor_tree(functor, a, init=0):
    """kernels/reduction.py:194-265 with the device functions at :22-166, in the
    association order a CUDA run uses - the same walk as orc_tree_* in oracle.c, with a
    Python functor in place of the operator."""
    a = np.asarray(a)
    f = typed_functor(functor, a.dtype)
    init = a.dtype.type(init)
    n = a.size
    if n < 1:
        return init
    block = _WARP * _NWARPS

    def warp_tree(v):                        # :22-41, one full warp
        v = list(v)
        width = _WARP // 2
        while width:
            for lane in range(width):
                v[lane] = f(v[lane], v[lane + width])
            width //= 2
        return v[0]

    def one_block(items):                    # :99-141, fewer than 128 lanes
        m = len(items)
        results = []
        for w in range((m + _WARP - 1) // _WARP):
            if (w + 1) * _WARP < m:
                results.append(warp_tree(items[w * _WARP:(w + 1) * _WARP]))
            else:
                acc = items[w * _WARP]
                for x in items[w * _WARP + 1:m]:
                    acc = f(acc, x)
                results.append(acc)
        r = results[0]
        for x in results[1:]:
            r = f(r, x)
        return r

    size_full = (n // block) * block
    grid = min(size_full // block, _MAXGRID)
    stride = block * grid
    partials = []
    for blk in range(grid):                  # :43-97, :233-248
        per_warp = []
        for w in range(_NWARPS):
            lanes = []
            for lane in range(_WARP):
                g = blk * block + w * _WARP + lane
                acc = a[g]
                for i in range(g + stride, size_full, stride):
                    acc = f(acc, a[i])
                lanes.append(acc)
            per_warp.append(warp_tree(lanes))
        partials.append(f(f(per_warp[0], per_warp[2]), f(per_warp[1], per_warp[3])))
    if grid:
        partials[0] = f(partials[0], init)   # :163-164
    if n - size_full:                        # :250-254
        partials.append(one_block(list(a[size_full:])))
        if not grid:
            partials[0] = f(partials[0], init)
    if len(partials) > 1:                    # :256-258
        partials[0] = one_block(partials)
    return partials[0]


def sum_exact(a):
    """(sum, sum of magnitudes) in compensated long double."""
    a = np.ascontiguousarray(a)
    s = np.zeros(1, np.float64)
    sa = np.zeros(1, np.float64)
    fn = {np.dtype(np.float32): lib().orc_sum_exact_f32,
          np.dtype(np.float64): lib().orc_sum_exact_f64}[a.dtype]
    fn(_ptr(a), a.size, _ptr(s), _ptr(sa))
    return float(s[0]), float(sa[0])


# ----------------------------------------------------------------------------
# Transpose / extents
# ----------------------------------------------------------------------------

def transpose(a):
    """C-contiguous transpose of a 2-D array of any dtype and strides."""
    assert a.ndim == 2
    rows, cols = a.shape
    out = np.empty((cols, rows), a.dtype)
    if a.size:
        # the base address of a possibly negative-strided view is a.ctypes.data
        lib().orc_transpose(_ptr(a), _ptr(out), rows, cols, a.strides[0], a.strides[1],
                            out.strides[0], out.strides[1], a.dtype.itemsize)
    return out


def extents(shape, strides, itemsize):
    nd = len(shape)
    sh = np.asarray(shape, np.int64).reshape(nd)
    st = np.asarray(strides, np.int64).reshape(nd)
    lo = np.zeros(1, np.int64)
    hi = np.zeros(1, np.int64)
    lib().orc_extents(_ptr(sh), _ptr(st), nd, itemsize, _ptr(lo), _ptr(hi))
    return int(lo[0]), int(hi[0])
