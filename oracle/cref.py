"""ctypes access to oracle/liboracle.so (the C restatement in oracle.c).

Test infrastructure: see the package docstring.
"""

import ctypes
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
