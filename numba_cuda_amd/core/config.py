"""Environment-variable configuration.

Honours the subset of the reference's NUMBA_* variables that touch the array
library (numba_cuda/numba/cuda/core/config.py:197-212 _readenv, :252, :440-480,
:586, :635-639 reload_config; docs/source/reference/envvars.rst:29-101).  Values
are module globals, re-read by reload_config().
"""

import os
import warnings


def _readenv(name, ctor, default):
    value = os.environ.get(name)
    if value is None:
        return default() if callable(default) else default
    try:
        return ctor(value)
    except Exception:
        warnings.warn("environ %s defined but failed to parse '%s'" % (name, value), RuntimeWarning)
        return default() if callable(default) else default


def reload_config():
    g = globals()
    # the reference swaps in a CPU simulator here; this package has no CPU path
    g["ENABLE_CUDASIM"] = _readenv("NUMBA_ENABLE_CUDASIM", int, 0)
    g["DISABLE_CUDA"] = _readenv("NUMBA_DISABLE_CUDA", int, 0)
    g["CUDA_LOG_LEVEL"] = _readenv("NUMBA_CUDA_LOG_LEVEL", str, "")
    g["CUDA_LOG_API_ARGS"] = _readenv("NUMBA_CUDA_LOG_API_ARGS", int, 0)
    g["CUDA_DEALLOCS_COUNT"] = _readenv("NUMBA_CUDA_MAX_PENDING_DEALLOCS_COUNT", int, 10)
    g["CUDA_DEALLOCS_RATIO"] = _readenv("NUMBA_CUDA_MAX_PENDING_DEALLOCS_RATIO", float, 0.2)
    g["CUDA_WARN_ON_IMPLICIT_COPY"] = _readenv("NUMBA_CUDA_WARN_ON_IMPLICIT_COPY", int, 1)
    g["DISABLE_PERFORMANCE_WARNINGS"] = _readenv("NUMBA_DISABLE_PERFORMANCE_WARNINGS", int, 0)
    g["CUDA_LOW_OCCUPANCY_WARNINGS"] = _readenv("NUMBA_CUDA_LOW_OCCUPANCY_WARNINGS", int, 1)
    g["CUDA_ARRAY_INTERFACE_SYNC"] = _readenv("NUMBA_CUDA_ARRAY_INTERFACE_SYNC", int, 1)
    g["CUDA_MEMORY_MANAGER"] = _readenv("NUMBA_CUDA_MEMORY_MANAGER", str, "default")
    # not in the reference: 1 makes Reduce apply its operator in the association order of the
    # reference's kernels, so that floating-point results have the reference's bits
    g["CUDA_REDUCE_REFERENCE_ORDER"] = _readenv("NUMBA_CUDA_REDUCE_REFERENCE_ORDER", int, 0)
    # not in the reference: 1 (the default) hands the kernel launches of Reduce(...)(arr, res=..., stream=s)
    # on streams made by cuda.stream() to a launching thread per stream, until the stream's handle is
    # read by code outside the package (kernels/reduction.py launch_threads); 0 launches on the caller's thread
    g["CUDA_REDUCE_LAUNCH_THREADS"] = _readenv("NUMBA_CUDA_REDUCE_LAUNCH_THREADS", int, 1)


reload_config()
