"""Compile translated functor bodies as HOST C++ and apply them to arrays.

The device source in csrc/reduce_custom.hip keeps everything up to `nbh_op` valid as host
C++; this takes that part (the helpers with Python's division rules), appends one function
per body, and builds a shared object with g++.  Test infrastructure only."""

import ctypes
import os
import re
import subprocess
import tempfile

import numpy as np

_SRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "numba_cuda_amd", "csrc", "reduce_custom.hip")

CTYPE = {"int8": "signed char", "int16": "short", "int32": "int", "int64": "long long",
         "uint8": "unsigned char", "uint16": "unsigned short", "uint32": "unsigned int",
         "uint64": "unsigned long long", "float32": "float", "float64": "double", "bool": "unsigned char",
         "complex64": "nbh_c64", "complex128": "nbh_c128"}


def helpers(ctype):
    """The device source up to nbh_op, with the element type put in where the library puts it."""
    text = open(_SRC).read()
    start = text.index('R"NBHSRC(') + len('R"NBHSRC(')
    stop = text.index("__device__ __forceinline__ T nbh_op(T a, T b)")
    part = text[start:stop]
    assert part.count("@T@") == 1
    return re.sub(r"typedef unsigned int nbh_u32x4[^\n]*\n", "", part).replace("@T@", ctype)


def build(bodies, dtype_name):
    """-> list of callables f(a, b) -> array, one per body, for arrays of the dtype."""
    src = ["#include <cmath>", "#include <cstdint>", "using namespace std;", "#define __device__",
           "#define __forceinline__ inline", helpers(CTYPE[dtype_name])]
    for k, body in enumerate(bodies):
        src.append("static inline T op_%d(T a, T b)\n{\n%s\n}" % (k, body))
        src.append('extern "C" void apply_%d(const T *a, const T *b, T *out, long n)\n'
                   "{ for (long i = 0; i < n; ++i) out[i] = op_%d(a[i], b[i]); }" % (k, k))
    tmp = tempfile.mkdtemp(prefix="nbh_functor_")
    cpp, so = os.path.join(tmp, "ops.cpp"), os.path.join(tmp, "ops.so")
    with open(cpp, "w") as f:
        f.write("\n".join(src))
    proc = subprocess.run(["g++", "-O1", "-std=c++17", "-ffp-contract=off", "-fwrapv", "-shared", "-fPIC", cpp,
                           "-o", so], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode:
        raise RuntimeError("host build failed:\n%s\n%s" % (proc.stdout, "\n".join(src)))
    lib = ctypes.CDLL(so)
    dtype = np.dtype(dtype_name)

    def bind(k):
        fn = getattr(lib, "apply_%d" % k)
        fn.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_long]
        fn.restype = None

        def apply(a, b):
            a, b = np.ascontiguousarray(a, dtype), np.ascontiguousarray(b, dtype)
            out = np.empty_like(a)
            fn(a.ctypes.data, b.ctypes.data, out.ctypes.data, a.size)
            return out
        apply._keep = lib
        return apply
    return [bind(k) for k in range(len(bodies))]
