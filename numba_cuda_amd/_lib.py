"""ctypes binding of libnbhip.so, the only native code this package calls.

Every signature here mirrors a declaration in include/nbhip.h.  If the library is
missing the import fails with instructions; there is no other implementation to
fall back to.
"""

import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libnbhip.so")
IPC_HANDLE_BYTES = 64      # NBH_IPC_HANDLE_BYTES

c_int = ctypes.c_int
c_i64 = ctypes.c_int64
c_u64 = ctypes.c_uint64
c_size = ctypes.c_size_t
c_vp = ctypes.c_void_p
c_char_p = ctypes.c_char_p
P = ctypes.POINTER

# name -> (restype, argtypes); must list every symbol include/nbhip.h declares
SIGNATURES = {
    "nbh_version": (c_int, []),
    "nbh_hip_versions": (c_int, [P(c_int), P(c_int)]),
    "nbh_error_name": (c_char_p, [c_int]),
    "nbh_error_string": (c_char_p, [c_int]),
    "nbh_device_count": (c_int, [P(c_int)]),
    "nbh_set_device": (c_int, [c_int]),
    "nbh_get_device": (c_int, [P(c_int)]),
    "nbh_device_name": (c_int, [c_int, c_char_p, c_int]),
    "nbh_device_attr": (c_int, [c_int, c_char_p, P(c_int)]),
    "nbh_mem_info": (c_int, [P(c_size), P(c_size)]),
    "nbh_device_synchronize": (c_int, []),
    "nbh_malloc": (c_int, [P(c_vp), c_size]),
    "nbh_free": (c_int, [c_vp]),
    "nbh_malloc_managed": (c_int, [P(c_vp), c_size, c_int]),
    "nbh_pool_malloc": (c_int, [P(c_vp), c_size]),
    "nbh_pool_free": (c_int, [c_vp]),
    "nbh_pool_trim": (c_int, []),
    "nbh_pool_stats": (c_int, [P(c_size), P(c_size), P(ctypes.c_uint64), P(ctypes.c_uint64)]),
    "nbh_host_alloc": (c_int, [P(c_vp), c_size, ctypes.c_uint]),
    "nbh_host_free": (c_int, [c_vp]),
    "nbh_host_register": (c_int, [c_vp, c_size, ctypes.c_uint]),
    "nbh_host_unregister": (c_int, [c_vp]),
    "nbh_host_get_device_pointer": (c_int, [P(c_vp), c_vp]),
    "nbh_mem_address_range": (c_int, [P(c_vp), P(c_size), c_vp]),
    "nbh_ipc_get_handle": (c_int, [c_vp, c_vp]),
    "nbh_ipc_open": (c_int, [P(c_vp), c_vp, c_size]),
    "nbh_ipc_close": (c_int, [c_vp]),
    "nbh_memcpy_h2d": (c_int, [c_vp, c_vp, c_size, c_vp]),
    "nbh_memcpy_d2h": (c_int, [c_vp, c_vp, c_size, c_vp]),
    "nbh_memcpy_d2d": (c_int, [c_vp, c_vp, c_size, c_vp]),
    "nbh_memset8": (c_int, [c_vp, c_int, c_size, c_vp]),
    "nbh_stream_create": (c_int, [P(c_vp)]),
    "nbh_stream_destroy": (c_int, [c_vp]),
    "nbh_stream_synchronize": (c_int, [c_vp]),
    "nbh_stream_query": (c_int, [c_vp]),
    "nbh_stream_add_callback": (c_int, [c_vp, ctypes.CFUNCTYPE(None, c_vp), c_vp]),
    "nbh_event_create": (c_int, [P(c_vp), c_int]),
    "nbh_event_destroy": (c_int, [c_vp]),
    "nbh_event_record": (c_int, [c_vp, c_vp]),
    "nbh_event_synchronize": (c_int, [c_vp]),
    "nbh_event_query": (c_int, [c_vp]),
    "nbh_stream_wait_event": (c_int, [c_vp, c_vp]),
    "nbh_event_elapsed_ms": (c_int, [P(ctypes.c_float), c_vp, c_vp]),
    "nbh_reduce_scratch_bytes": (c_size, []),
    "nbh_reduce": (c_int, [c_int, c_int, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_size, c_vp]),
    "nbh_reduce_ordered": (c_int, [c_int, c_int, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_size, c_vp]),
    "nbh_reduce_queued": (c_int, [c_int, c_int, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_size, c_vp]),
    "nbh_launch_threads": (c_int, [c_int]),
    "nbh_launch_threads_wait": (c_int, [c_vp]),
    "nbh_stream_pin_direct": (c_int, [c_vp]),
    "nbh_reduce_noalloc": (c_int, [c_int, c_int, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp]),
    "nbh_reduce_compile": (c_int, [c_int, ctypes.c_char_p, ctypes.POINTER(c_vp), ctypes.c_char_p, c_size]),
    "nbh_reduce_op_dtype": (c_int, [c_vp]),
    "nbh_reduce_op_free": (c_int, [c_vp]),
    "nbh_reduce_custom": (c_int, [c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_size, c_vp]),
    "nbh_reduce_custom_ordered": (c_int, [c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_size, c_vp]),
    "nbh_transpose": (c_int, [c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "nbh_assign": (c_int, [c_vp, c_vp, c_int, P(c_i64), P(c_i64), P(c_i64), c_i64, c_vp]),
    "nbh_fill": (c_int, [c_vp, c_int, P(c_i64), P(c_i64), c_i64, c_vp, c_vp]),
    "nbh_xoro_init_states": (c_int, [c_vp, c_i64, c_u64, c_u64, c_vp]),
    "nbh_xoro_uniform_f32": (c_int, [c_vp, c_i64, c_vp, c_i64, c_vp]),
    "nbh_xoro_uniform_f64": (c_int, [c_vp, c_i64, c_vp, c_i64, c_vp]),
    "nbh_xoro_normal_f32": (c_int, [c_vp, c_i64, c_vp, c_i64, c_vp]),
    "nbh_xoro_normal_f64": (c_int, [c_vp, c_i64, c_vp, c_i64, c_vp]),
    "nbh_xoro_one": (c_int, [c_vp, c_int, c_vp, c_vp]),
}

# enum nbh_dtype / enum nbh_op
DTYPE_CODES = {"int8": 0, "int16": 1, "int32": 2, "int64": 3,
               "uint8": 4, "uint16": 5, "uint32": 6, "uint64": 7,
               "float32": 8, "float64": 9, "complex64": 10, "complex128": 11,
               "float16": 12}
OP_CODES = {"add": 0, "mul": 1, "max": 2, "min": 3, "and": 4, "or": 5, "xor": 6}

# hipError_t values the Python layer branches on
HIP_SUCCESS = 0
HIP_ERROR_OUT_OF_MEMORY = 2
HIP_ERROR_NOT_READY = 600

HOST_FN = ctypes.CFUNCTYPE(None, c_vp)

_lib = None


class LibraryNotBuiltError(OSError):
    pass


def load():
    """Return the loaded library, loading it on first use."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryNotBuiltError(
                "%s is missing: the HIP back end has not been built. Run "
                "`python -m numba_cuda_amd._build` (needs hipcc); there is no "
                "CPU implementation to fall back to." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)   # AttributeError if the library is stale
            fn.restype = restype
            fn.argtypes = argtypes
        if lib.nbh_version() != 1:
            raise LibraryNotBuiltError("libnbhip.so has ABI version %d, expected 1; rebuild it"
                                       % lib.nbh_version())
        _lib = lib
    return _lib
