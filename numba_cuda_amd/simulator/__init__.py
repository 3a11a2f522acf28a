"""The CPU mode of the package: what `import numba_cuda_amd as cuda` gives when
NUMBA_ENABLE_CUDASIM=1 (the reference swaps its whole API for a NumPy implementation
under that variable, numba_cuda/numba/cuda/__init__.py:32-36, simulator/__init__.py:38-66).

Everything runs at once on the calling thread over NumPy arrays: `Reduce` is the
strict left fold, device arrays are NumPy-backed, streams and events are inert,
the RNG runs on host state arrays.  No GPU library is loaded in this mode.
"""

from numba_cuda_amd.core.errors import CudaDriverError, CudaSupportError, NumbaPerformanceWarning  # noqa: F401
from numba_cuda_amd.simulator.args import In, InOut, Out  # noqa: F401
from numba_cuda_amd.simulator import hostarray as devicearray  # noqa: F401
from numba_cuda_amd.simulator import random, reduction  # noqa: F401
from numba_cuda_amd.simulator.hostarray import (HostBackedArray, DeviceNDArray, DeviceRecord,  # noqa: F401
                                                _contiguous_strides_like_array, _order_like_array, auto_device,
                                                device_array, device_array_like, is_cuda_ndarray, managed_array,
                                                mapped, mapped_array, mapped_array_like, pinned, pinned_array,
                                                pinned_array_like, require_cuda_ndarray, to_device,
                                                verify_cuda_ndarray_interface)
from numba_cuda_amd.simulator.reduction import Reduce
from numba_cuda_amd.simulator.runtime import (Event, Stream, close, cuda_error, current_context,  # noqa: F401
                                              default_stream, defer_cleanup, detect, event, event_elapsed_time,
                                              external_stream, get_context, get_current_device, gpus,
                                              is_available, is_bfloat16_supported, is_float16_supported,
                                              is_supported_version, legacy_default_stream, list_devices,
                                              per_thread_default_stream, profile_start, profile_stop, profiling,
                                              require_context, reset, select_device, stream, synchronize)
from numba_cuda_amd.simulator.transpose import transpose  # noqa: F401

reduce = Reduce
_auto_device = auto_device
