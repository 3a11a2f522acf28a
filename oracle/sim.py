"""The reference's CPU path (its CUDA simulator, NUMBA_ENABLE_CUDASIM=1), restated.

Test infrastructure: the single-core baseline that the benchmark times beside
the GPU numbers.  The simulator is plain Python over NumPy scalars; it is
single-threaded by construction (one interpreter, blocks run one after another,
numba_cuda/numba/cuda/simulator/kernel.py:125-128).
"""

from functools import reduce as _pyreduce

import numpy as np

_U = np.uint64


def Reduce(func):
    """simulator/reduction.py:7-19: a strict left fold through the Python
    callable, one call per element; `init` is used as given (not cast)."""

    def reduce_wrapper(seq, res=None, init=0):
        r = _pyreduce(func, seq, init)
        if res is not None:
            res[0] = r
            return None
        return r

    return reduce_wrapper


def transpose(a):
    """simulator/cudadrv/devicearray.py:151-156: a NumPy view, no data moves."""
    return np.transpose(a)


# --- RNG in the simulator's flavour: the functions of random.py run in object
# mode on NumPy records, every intermediate an np.uint64 scalar (random.py:39-45
# explains the casts).

def init_state(states, index, seed):
    """random.py:62-85"""
    with np.errstate(over="ignore"):
        z = _U(seed) + _U(0x9E3779B97F4A7C15)
        z = (z ^ (z >> _U(30))) * _U(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> _U(27))) * _U(0x94D049BB133111EB)
        z = z ^ (z >> _U(31))
    states[index]["s0"] = z
    states[index]["s1"] = z


def rotl(x, k):
    """random.py:88-93"""
    return (_U(x) << _U(k)) | (_U(x) >> _U(64 - k))


def next_u64(states, index):
    """random.py:96-115"""
    s0 = states[index]["s0"]
    s1 = states[index]["s1"]
    with np.errstate(over="ignore"):
        result = s0 + s1
    s1 ^= s0
    states[index]["s0"] = rotl(s0, 55) ^ s1 ^ (s1 << _U(14))
    states[index]["s1"] = rotl(s1, 36)
    return result


def jump(states, index):
    """random.py:118-142"""
    words = (_U(0xBEAC0467EBA5FACB), _U(0xD86B048B86AA9922))
    s0 = _U(0)
    s1 = _U(0)
    for i in range(2):
        for b in range(64):
            if words[i] & (_U(1) << _U(b)):
                s0 ^= states[index]["s0"]
                s1 ^= states[index]["s1"]
            next_u64(states, index)
    states[index]["s0"] = s0
    states[index]["s1"] = s1


def init_states(states, seed, subsequence_start=0):
    """random.py:241-257"""
    n = states.shape[0]
    if n >= 1:
        init_state(states, 0, seed)
        for _ in range(int(subsequence_start)):
            jump(states, 0)
        for i in range(1, n):
            states[i] = states[i - 1]
            jump(states, i)


def uniform_float64(states, index):
    """random.py:145-149, :171-184"""
    x = next_u64(states, index)
    return (x >> _U(11)) * (np.float64(1) / np.float64(_U(1) << _U(53)))


def uniform_float32(states, index):
    """random.py:152-169"""
    return np.float32(uniform_float64(states, index))


_TWO_PI_F32 = np.float32(2 * np.pi)
_TWO_PI_F64 = np.float64(2 * np.pi)


def normal_float32(states, index):
    """random.py:191-213 in object mode: `math.log` / `math.cos` / `math.sqrt` of a
    NumPy float32 go through Python floats (float64 precision), so only the products
    round to float32.  Parity unpinned: derivable from the source, not confirmable
    without running the reference."""
    import math
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    return math.sqrt(-np.float32(2.0) * math.log(u1)) * math.cos(_TWO_PI_F32 * u2)


def normal_float64(states, index):
    """random.py:216-238 in object mode (float32 uniforms, float64 arithmetic)."""
    import math
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    return math.sqrt(-np.float64(2.0) * math.log(u1)) * math.cos(_TWO_PI_F64 * u2)
