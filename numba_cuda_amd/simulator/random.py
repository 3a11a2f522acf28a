"""xoroshiro128+ in the CPU mode: the functions of numba_cuda/numba/cuda/random.py on
NumPy-backed state arrays.  The states, the uint64 draws and the uniform values are
the GPU path's bit for bit; the normals are computed as the reference's simulator
computes them (its expressions evaluated by the interpreter: double-precision
logarithm, cosine and square root on float32 uniforms), which differs from the
GPU's float32 arithmetic in the last bits."""

import numpy as np

from numba_cuda_amd import _xoroshiro_host as _host
from numba_cuda_amd.simulator.hostarray import HostBackedArray, device_array

xoroshiro128p_dtype = _host.xoroshiro128p_dtype
UNIFORM = 1
NORMAL = 2
TWO_PI_FLOAT32 = _host.TWO_PI_FLOAT32
TWO_PI_FLOAT64 = _host.TWO_PI_FLOAT64
rotl = _host.rotl
uint64_to_unit_float32 = _host.uint64_to_unit_float32
uint64_to_unit_float64 = _host.uint64_to_unit_float64


def _host_view(states):
    states = getattr(states, "_ary", states)
    if states.ndim != 1 or states.dtype.itemsize != 16:
        raise TypeError("states must be a 1D array of xoroshiro128p_dtype")
    return states


def init_xoroshiro128p_state(states, index, seed):
    _host.init_state(_host_view(states), index, seed)


def xoroshiro128p_next(states, index):
    return _host.next_u64(_host_view(states), index)


def xoroshiro128p_jump(states, index):
    _host.jump(_host_view(states), index)


def xoroshiro128p_uniform_float32(states, index):
    return _host.uniform_float32(_host_view(states), index)


def xoroshiro128p_uniform_float64(states, index):
    return _host.uniform_float64(_host_view(states), index)


def xoroshiro128p_normal_float32(states, index):
    return _host.normal_float32_object_mode(_host_view(states), index)


def xoroshiro128p_normal_float64(states, index):
    return _host.normal_float64_object_mode(_host_view(states), index)


def init_xoroshiro128p_states_cpu(states, seed, subsequence_start):
    _host.init_states_cpu(_host_view(states), seed, subsequence_start)


def init_xoroshiro128p_states(states, seed, subsequence_start=0, stream=0):
    _host.init_states_cpu(_host_view(states), seed, subsequence_start)


def create_xoroshiro128p_states(n, seed, subsequence_start=0, stream=0):
    states = device_array(n, dtype=xoroshiro128p_dtype, stream=stream)
    init_xoroshiro128p_states(states, seed, subsequence_start, stream)
    return states


def xoroshiro128p_fill(states, out, count=None, distribution=UNIFORM, stream=0):
    """Every generator t draws `count` values of out.dtype into out[t*count + i]."""
    st = _host_view(states)
    dest = getattr(out, "_ary", out)
    if dest.ndim != 1 or (dest.size and dest.strides[0] != dest.dtype.itemsize):
        raise ValueError("out must be a 1D unit-stride array")
    if dest.dtype not in (np.dtype(np.float32), np.dtype(np.float64)) or distribution not in (UNIFORM, NORMAL):
        raise TypeError("unsupported distribution/dtype: %r / %s" % (distribution, dest.dtype))
    n = st.size
    if count is None:
        count = dest.size // n if n else 0
    count = int(count)
    if count < 0 or n * count > dest.size:
        raise ValueError("out has %d items, need %d generators x %d draws" % (dest.size, n, count))
    _host.fill(st, dest, count, distribution == NORMAL)
    return out


def xoroshiro128p_fill_uniform(states, out, count=None, stream=0):
    return xoroshiro128p_fill(states, out, count, UNIFORM, stream)


def xoroshiro128p_fill_normal(states, out, count=None, stream=0):
    return xoroshiro128p_fill(states, out, count, NORMAL, stream)
