"""MI355X-native data-parallel array library with the numba.cuda API.

    import numba_cuda_amd as cuda

    d = cuda.to_device(host_array)
    total = cuda.reduce(lambda a, b: a + b)(d)
    dt = d2.T                                  # tiled transpose
    states = cuda.random.create_xoroshiro128p_states(n, seed=1)

Host code is Python; everything that touches the GPU goes through libnbhip.so
(hand-written HIP for gfx950, built by `python -m numba_cuda_amd._build`).
There is no JIT compiler.  With NUMBA_ENABLE_CUDASIM=1 in the environment the same names are
backed by NumPy on the host instead (numba_cuda_amd/simulator): for machines without a GPU.
"""

import sys as _sys

from numba_cuda_amd.core import config

if config.ENABLE_CUDASIM:
    # the CPU mode: NumPy-backed arrays, inert streams, Reduce as a left fold; no GPU library
    from numba_cuda_amd import simulator as _simulator
    from numba_cuda_amd.simulator import *  # noqa: F401,F403
    from numba_cuda_amd.simulator import (_auto_device, _contiguous_strides_like_array,  # noqa: F401
                                          _order_like_array, devicearray, random, reduction)
    # modules a user may import by name get the CPU mode's versions
    for _name, _module in (("random", "simulator.random"), ("api", "simulator"), ("args", "simulator.args"),
                           ("kernels.reduction", "simulator.reduction"), ("kernels.transpose", "simulator.transpose"),
                           ("cudadrv.devicearray", "simulator.hostarray")):
        _sys.modules[__name__ + "." + _name] = _sys.modules[__name__ + "." + _module]
    reduce = Reduce  # noqa: F405
else:
    from numba_cuda_amd.core.errors import (CudaDriverError, CudaSupportError,  # noqa: F401
                                            NumbaPerformanceWarning)
    from numba_cuda_amd import cudadrv  # noqa: F401
    from numba_cuda_amd.cudadrv import devicearray, devices, driver  # noqa: F401
    from numba_cuda_amd.cudadrv.driver import (BaseCUDAMemoryManager, CudaAPIError,  # noqa: F401
                                               GetIpcHandleMixin, HostOnlyCUDAMemoryManager, IpcHandle,
                                               ManagedMemory, MemoryPointer, MappedMemory,
                                               PinnedMemory, MemoryInfo, set_memory_manager)
    from numba_cuda_amd.cudadrv.devicearray import DeviceNDArray, DeviceRecord  # noqa: F401
    from numba_cuda_amd.cudadrv.runtime import runtime  # noqa: F401
    from numba_cuda_amd.api import *  # noqa: F401,F403
    from numba_cuda_amd.api import (_auto_device, _contiguous_strides_like_array, _order_like_array,  # noqa: F401
                                    current_context, gpus, require_context)
    from numba_cuda_amd.args import In, InOut, Out  # noqa: F401
    from numba_cuda_amd import kernels  # noqa: F401
    from numba_cuda_amd.kernels import reduction  # noqa: F401  (the reference exposes the module as cuda.reduction)
    from numba_cuda_amd.kernels import transpose as _transpose  # noqa: F401
    from numba_cuda_amd.kernels.reduction import Reduce
    from numba_cuda_amd import random  # noqa: F401

    reduce = Reduce

__version__ = "0.1.0"
