"""Exception and warning types (names follow numba_cuda/numba/cuda/core/errors.py
and cudadrv/error.py so that user `except` clauses keep working)."""


class NumbaWarning(Warning):
    pass


class NumbaPerformanceWarning(NumbaWarning):
    """Host arrays passed where device arrays are expected, and similar."""


class CudaDriverError(Exception):
    pass


class CudaRuntimeError(Exception):
    pass


class CudaSupportError(ImportError):
    pass
