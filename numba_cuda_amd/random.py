"""xoroshiro128+ random numbers (drop-in for numba_cuda/numba/cuda/random.py).

Differences in mechanism, not in results:
  * init_xoroshiro128p_states builds the states ON THE DEVICE (GF(2) jump
    matrices) instead of as a sequential CPU chain followed by an upload; the
    states are bit-identical to the reference's (random.py:241-282)
  * the reference offers per-thread device functions for use inside JIT kernels;
    there is no kernel language here, so draws are bulk operations:
    `xoroshiro128p_fill(states, out, count, distribution)` produces, for every
    generator t, `count` values into out[t*count + i] - the layout of the
    reference's own test kernels (tests/cudapy/test_random.py:29-52)
  * the scalar functions `xoroshiro128p_next(states, index)` etc. keep their
    reference meaning when called from host code, on host state arrays and on the
    device array create_xoroshiro128p_states returned alike (the reference's
    simulator allows both): on a device array the one generator is stepped by a
    one-lane kernel running the same routines as the bulk draws, and the value
    comes back through a cell of device-mapped host memory.
"""

import numpy as np

from numba_cuda_amd.cudadrv import devices
from numba_cuda_amd.cudadrv import driver as _driver
from numba_cuda_amd import api as _api
from numba_cuda_amd import _xoroshiro_host as _host

xoroshiro128p_dtype = _host.xoroshiro128p_dtype

UNIFORM = 1
NORMAL = 2

_M64 = (1 << 64) - 1


# ---- bulk device operations -----------------------------------------------------------

def _check_states(states):
    if states.ndim != 1 or states.dtype.itemsize != 16:
        raise TypeError("states must be a 1D array of xoroshiro128p_dtype")
    if not _driver.is_device_memory(states):
        raise TypeError("states must be a device array (see create_xoroshiro128p_states)")
    if states.size and states.strides[0] != 16:
        raise ValueError("states must have unit stride")


@devices.require_context
def init_xoroshiro128p_states(states, seed, subsequence_start=0, stream=0):
    """Initialise `states` so that states[i] is the generator seeded with `seed`
    advanced by (subsequence_start + i) * 2**64 steps: independent subsequences
    as long as no generator draws more than 2**64 numbers.

    states : 1D DeviceNDArray of xoroshiro128p_dtype
    seed, subsequence_start : reduced modulo 2**64
    """
    _check_states(states)
    _driver.driver.nbh_xoro_init_states(states.device_ctypes_pointer.value, states.size,
                                        int(seed) & _M64, int(subsequence_start) & _M64,
                                        _driver._stream_handle(stream) or None)


@devices.require_context
def create_xoroshiro128p_states(n, seed, subsequence_start=0, stream=0):
    """New device array of `n` initialised generator states."""
    states = _api.device_array(n, dtype=xoroshiro128p_dtype, stream=stream)
    init_xoroshiro128p_states(states, seed, subsequence_start, stream)
    return states


_FILL = {
    (UNIFORM, "float32"): "nbh_xoro_uniform_f32",
    (UNIFORM, "float64"): "nbh_xoro_uniform_f64",
    (NORMAL, "float32"): "nbh_xoro_normal_f32",
    (NORMAL, "float64"): "nbh_xoro_normal_f64",
}


@devices.require_context
def xoroshiro128p_fill(states, out, count=None, distribution=UNIFORM, stream=0):
    """Every generator t draws `count` values of out.dtype into
    out[t*count + i], i = 0..count-1, and its state advances in place (by `count`
    steps for UNIFORM, 2*count for NORMAL - Box-Muller uses two draws per value).

    out          : 1D device array of float32 or float64 with at least
                   len(states)*count items; `count` defaults to out.size // len(states)
    distribution : UNIFORM -> [0, 1)  (float32 values may round up to exactly 1.0,
                   as in the reference), NORMAL -> mean 0, sigma 1
    """
    _check_states(states)
    if not _driver.is_device_memory(out):
        raise TypeError("out must be a device array")
    if out.ndim != 1 or (out.size and out.strides[0] != out.dtype.itemsize):
        raise ValueError("out must be a 1D unit-stride array")
    n = states.size
    if count is None:
        count = out.size // n if n else 0
    count = int(count)
    if count < 0 or n * count > out.size:
        raise ValueError("out has %d items, need %d generators x %d draws" % (out.size, n, count))
    fn = _FILL.get((distribution, out.dtype.name))
    if fn is None:
        raise TypeError("unsupported distribution/dtype: %r / %s" % (distribution, out.dtype))
    getattr(_driver.driver, fn)(states.device_ctypes_pointer.value, n, out.device_ctypes_pointer.value,
                                count, _driver._stream_handle(stream) or None)
    return out


def xoroshiro128p_fill_uniform(states, out, count=None, stream=0):
    return xoroshiro128p_fill(states, out, count, UNIFORM, stream)


def xoroshiro128p_fill_normal(states, out, count=None, stream=0):
    return xoroshiro128p_fill(states, out, count, NORMAL, stream)


# ---- scalar functions (reference semantics, random.py:62-238) --------------------------

_ONE_NEXT, _ONE_JUMP, _ONE_UNIFORM_F32, _ONE_UNIFORM_F64, _ONE_NORMAL_F32, _ONE_NORMAL_F64 = range(6)   # nbh_xoro_kind
_ONE_RESULT = {_ONE_NEXT: np.dtype(np.uint64), _ONE_UNIFORM_F32: np.dtype(np.float32),
               _ONE_UNIFORM_F64: np.dtype(np.float64), _ONE_NORMAL_F32: np.dtype(np.float32),
               _ONE_NORMAL_F64: np.dtype(np.float64)}


def _record_address(states, index):
    """Device address of generator `index` of a device-resident state array."""
    if states.ndim != 1 or states.dtype.itemsize != 16:
        raise TypeError("states must be a 1D array of xoroshiro128p_dtype")
    index = int(index)
    n = states.size
    if not -n <= index < n:
        raise IndexError("index %d is out of bounds for %d generator states" % (index, n))
    return states.device_ctypes_pointer.value + (index % n) * states.strides[0]


def _on_device(states, index, kind):
    """Run one per-generator function on generator `index` of a device array and
    return its value (None for the jump)."""
    ctx = devices.get_context()
    address = _record_address(states, index)
    drv = _driver.driver
    if kind == _ONE_JUMP:
        drv.nbh_xoro_one(address, kind, None, None)
        return None
    cell = ctx.take_result_cell()
    try:
        drv.nbh_xoro_one(address, kind, cell[0], None)
        drv.nbh_stream_synchronize(None)
        dtype = _ONE_RESULT[kind]
        return cell[1][:dtype.itemsize].view(dtype)[0]
    finally:
        ctx.give_back_result_cell(cell)


def init_xoroshiro128p_state(states, index, seed):
    """SplitMix64 step of `seed`; the same word goes into both halves."""
    if _driver.is_device_memory(states):
        devices.get_context()
        _driver.driver.nbh_xoro_init_states(_record_address(states, index), 1, int(seed) & _M64, 0, None)
        return
    _host.init_state(states, index, seed)


rotl = _host.rotl
uint64_to_unit_float64 = _host.uint64_to_unit_float64
uint64_to_unit_float32 = _host.uint64_to_unit_float32
TWO_PI_FLOAT32 = _host.TWO_PI_FLOAT32
TWO_PI_FLOAT64 = _host.TWO_PI_FLOAT64


def xoroshiro128p_next(states, index):
    """Next uint64 of generator `index`; advances it."""
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_NEXT)
    return _host.next_u64(states, index)


def xoroshiro128p_jump(states, index):
    """Advance generator `index` by 2**64 steps."""
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_JUMP)
    _host.jump(states, index)


def xoroshiro128p_uniform_float32(states, index):
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_UNIFORM_F32)
    return _host.uniform_float32(states, index)


def xoroshiro128p_uniform_float64(states, index):
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_UNIFORM_F64)
    return _host.uniform_float64(states, index)


def xoroshiro128p_normal_float32(states, index):
    """Box-Muller (cosine branch) in float32; uses two draws."""
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_NORMAL_F32)
    return _host.normal_float32(states, index)


def xoroshiro128p_normal_float64(states, index):
    """Box-Muller (cosine branch); float32 uniforms and logarithm, float64 rest."""
    if _driver.is_device_memory(states):
        return _on_device(states, index, _ONE_NORMAL_F64)
    return _host.normal_float64(states, index)


def init_xoroshiro128p_states_cpu(states, seed, subsequence_start):
    """Fill a HOST array of states exactly as init_xoroshiro128p_states fills a device
    array (the reference's helper of this name, random.py:241-257, builds them as a
    sequential chain; here the chain is unrolled by doubling with GF(2) jump matrices)."""
    if states.ndim != 1 or states.dtype.itemsize != 16:
        raise TypeError("states must be a 1D array of xoroshiro128p_dtype")
    _host.init_states_cpu(states, seed, subsequence_start)
