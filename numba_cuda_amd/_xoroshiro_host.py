"""xoroshiro128+ on host arrays: the per-generator functions of the reference's
random module (numba_cuda/numba/cuda/random.py:62-238) as plain Python over NumPy
records, and `init_xoroshiro128p_states_cpu` (random.py:241-257) without its
sequential chain.

The reference fills states[i] = jump(states[i-1]) one generator after the other
(about a millisecond each in its object-mode simulator).  The jump is a linear
map over GF(2) on the 128 state bits, so states[k:2k] = J^k applied to
states[0:k]: the array is filled by doubling, each doubling one batched
matrix-vector product done with byte-indexed look-up tables in NumPy.  The
states are the reference's, bit for bit.

Nothing here touches a GPU; the GPU module and the CPU mode both use it.
"""

import math

import numpy as np

xoroshiro128p_dtype = np.dtype([("s0", np.uint64), ("s1", np.uint64)], align=True)

_M64 = (1 << 64) - 1
_JUMP_WORDS = (0xBEAC0467EBA5FACB, 0xD86B048B86AA9922)


# ---- one generator at a time (Python integers; any indexable record array) -------------

def seed_word(seed):
    """SplitMix64 step of the seed (random.py:62-85): the word both halves start from."""
    z = (int(seed) + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def init_state(states, index, seed):
    z = seed_word(seed)
    states[int(index)]["s0"] = z
    states[int(index)]["s1"] = z


def rotl(x, k):
    x = int(x) & _M64
    return ((x << k) & _M64) | (x >> (64 - k))


def _step(s0, s1):
    """-> (draw, s0', s1') on Python integers (random.py:96-115)"""
    draw = (s0 + s1) & _M64
    s1 ^= s0
    return draw, rotl(s0, 55) ^ s1 ^ ((s1 << 14) & _M64), rotl(s1, 36)


def next_u64(states, index):
    index = int(index)
    draw, a, b = _step(int(states[index]["s0"]), int(states[index]["s1"]))
    states[index]["s0"] = a
    states[index]["s1"] = b
    return np.uint64(draw)


def _jump_pair(s0, s1):
    """2**64 steps on Python integers (random.py:118-142)"""
    a = b = 0
    for word in _JUMP_WORDS:
        for bit in range(64):
            if (word >> bit) & 1:
                a ^= s0
                b ^= s1
            _, s0, s1 = _step(s0, s1)
    return a, b


def jump(states, index):
    index = int(index)
    a, b = _jump_pair(int(states[index]["s0"]), int(states[index]["s1"]))
    states[index]["s0"] = a
    states[index]["s1"] = b


def uint64_to_unit_float64(x):
    return np.float64((int(x) >> 11) * (1.0 / (1 << 53)))


def uint64_to_unit_float32(x):
    return np.float32(uint64_to_unit_float64(x))


def uniform_float32(states, index):
    return uint64_to_unit_float32(next_u64(states, index))


def uniform_float64(states, index):
    return uint64_to_unit_float64(next_u64(states, index))


TWO_PI_FLOAT32 = np.float32(2 * math.pi)
TWO_PI_FLOAT64 = np.float64(2 * math.pi)


def normal_float32(states, index):
    """Box-Muller, cosine branch, all in float32 (random.py:191-213); two draws."""
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    with np.errstate(divide="ignore"):
        r = np.sqrt(-np.float32(2.0) * np.log(u1))
    return np.float32(r * np.cos(TWO_PI_FLOAT32 * u2))


def normal_float64(states, index):
    """Box-Muller with float32 uniforms and logarithm, float64 elsewhere (random.py:216-238)."""
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    with np.errstate(divide="ignore"):
        r = np.sqrt(-np.float64(2.0) * np.float64(np.log(u1)))
    return np.float64(r * np.cos(TWO_PI_FLOAT64 * np.float64(u2)))


def normal_float32_object_mode(states, index):
    """The same draw as the reference's simulator computes it: its source expression
    (random.py:191-213) evaluated by the Python interpreter, where `math.log`, `math.cos`
    and `math.sqrt` work in double precision on the float32 uniforms and only the
    products with float32 constants round to float32.  Returns a Python float."""
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    if u1 == 0:
        return math.inf * math.cos(TWO_PI_FLOAT32 * u2)   # math.log(0) raises; the GPU gives sqrt(-2 * -inf)
    return math.sqrt(-np.float32(2.0) * math.log(u1)) * math.cos(TWO_PI_FLOAT32 * u2)


def normal_float64_object_mode(states, index):
    """random.py:216-238 evaluated by the Python interpreter: float32 uniforms, double elsewhere."""
    u1 = uniform_float32(states, index)
    u2 = uniform_float32(states, index)
    if u1 == 0:
        return math.inf * math.cos(TWO_PI_FLOAT64 * u2)
    return math.sqrt(-np.float64(2.0) * math.log(u1)) * math.cos(TWO_PI_FLOAT64 * u2)


# ---- GF(2) matrices on the 128 state bits, applied to many states at once ---------------
#
# A linear map M is kept as its 128 images of the unit vectors, `cols`, a (128, 2)
# uint64 array (bit b of s0 is unit vector b, bit b of s1 unit vector 64 + b).
# Applying it to a batch: for each of the 16 bytes of a state, a 256-entry table of
# the XOR of the columns that byte selects; a state's image is the XOR of 16 entries.

def _tables(cols):
    """(16, 256, 2) uint64: tables[p, v] = XOR of cols[8p + b] over the bits b set in v."""
    t = np.zeros((16, 256, 2), np.uint64)
    c = cols.reshape(16, 8, 2)
    for b in range(8):
        step = 1 << b
        # entries [step, 2 step) are entries [0, step) with column b added
        t[:, step:2 * step] = t[:, :step] ^ c[:, b][:, None, :]
    return t


def _apply(tables, states):
    """states: (n, 2) uint64 -> their images, (n, 2) uint64"""
    as_bytes = np.ascontiguousarray(states).view(np.uint8).reshape(-1, 16)   # little-endian bytes of s0 then s1
    out = tables[0][as_bytes[:, 0]]
    for p in range(1, 16):
        out ^= tables[p][as_bytes[:, p]]
    return out


def _jump_matrix():
    """Columns of J, the 2**64-step jump: the images of the 128 unit vectors."""
    cols = np.zeros((128, 2), np.uint64)
    for b in range(128):
        a, c = _jump_pair(1 << b if b < 64 else 0, 1 << (b - 64) if b >= 64 else 0)
        cols[b] = (a, c)
    return cols


_J = None


def _jump_columns():
    global _J
    if _J is None:
        _J = _jump_matrix()
    return _J


def _square(cols):
    return _apply(_tables(cols), cols)


def init_states_cpu(states, seed, subsequence_start=0):
    """states[i] = the generator seeded with `seed`, advanced (subsequence_start + i) * 2**64
    steps: the result of the reference's sequential chain (random.py:241-257), by doubling."""
    n = states.shape[0]
    if n < 1:
        return
    z = seed_word(seed)
    first = np.array([[z, z]], np.uint64)
    # J ** subsequence_start by squaring, applied to the seed state
    power = _jump_columns()
    e = int(subsequence_start) & _M64
    while e:
        if e & 1:
            first = _apply(_tables(power), first)
        e >>= 1
        if e:
            power = _square(power)
    flat = np.empty((n, 2), np.uint64)
    flat[0] = first[0]
    have = 1
    power = _jump_columns()     # J ** have
    while have < n:
        take = min(have, n - have)
        flat[have:have + take] = _apply(_tables(power), flat[:take])
        have += take
        if have < n:
            power = _square(power)
    states["s0"] = flat[:, 0]
    states["s1"] = flat[:, 1]


# ---- all generators of an array at once (the bulk draws of the CPU mode) ----------------

def _next_all(s0, s1):
    """One step of every generator: returns the draws, updates s0 / s1 (uint64 arrays) in place."""
    with np.errstate(over="ignore"):
        draw = s0 + s1
    s1 ^= s0
    a = ((s0 << np.uint64(55)) | (s0 >> np.uint64(9))) ^ s1 ^ (s1 << np.uint64(14))
    b = (s1 << np.uint64(36)) | (s1 >> np.uint64(28))
    s0[...] = a
    s1[...] = b
    return draw


def _unit_float64_all(x):
    return (x >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def fill(states, out, count, normal):
    """Every generator t draws `count` values of out.dtype into out[t * count + i]; normals in
    the precision mix of the *_object_mode functions above."""
    s0 = states["s0"].copy()
    s1 = states["s1"].copy()
    n = s0.shape[0]
    view = out[:n * count].reshape(n, count)
    wide = out.dtype == np.float64
    for i in range(count):
        if not normal:
            u = _unit_float64_all(_next_all(s0, s1))
            view[:, i] = u if wide else u.astype(np.float32)
            continue
        u1 = _unit_float64_all(_next_all(s0, s1)).astype(np.float32)
        u2 = _unit_float64_all(_next_all(s0, s1)).astype(np.float32)
        with np.errstate(divide="ignore"):
            lg = np.log(u1.astype(np.float64))
        if wide:
            view[:, i] = np.sqrt(np.float64(-2.0) * lg) * np.cos(TWO_PI_FLOAT64 * u2.astype(np.float64))
        else:
            scaled = np.float32(-2.0) * lg.astype(np.float32)      # float32 constant times a Python float: float32
            view[:, i] = np.sqrt(scaled.astype(np.float64)) * np.cos((TWO_PI_FLOAT32 * u2).astype(np.float64))
    states["s0"] = s0
    states["s1"] = s1
