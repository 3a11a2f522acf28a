"""Big-int restatement of the reference RNG (numba_cuda/numba/cuda/random.py).

Test infrastructure.  Python integers are unbounded, so every operation is
followed by an explicit reduction mod 2^64; this is deliberately a different
style of arithmetic from the uint64_t code in oracle.c, so that the two can be
checked against each other.  Also holds the GF(2) machinery that pins `jump`
to the mathematics: jump must equal 2^64 applications of `next`.
"""

import numpy as np

M64 = (1 << 64) - 1


def seed_state(seed):
    """random.py:62-85: one SplitMix64 step, stored in both words."""
    z = (seed + 0x9E3779B97F4A7C15) & M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    z = z ^ (z >> 31)
    return z, z


def rotl(x, k):
    """random.py:88-93"""
    return ((x << k) & M64) | (x >> (64 - k))


def next_state(s0, s1):
    """random.py:96-115: returns (draw, new_s0, new_s1)."""
    draw = (s0 + s1) & M64
    s1 ^= s0
    return draw, rotl(s0, 55) ^ s1 ^ ((s1 << 14) & M64), rotl(s1, 36)


JUMP_WORDS = (0xBEAC0467EBA5FACB, 0xD86B048B86AA9922)


def jump(s0, s1):
    """random.py:118-142"""
    a0 = a1 = 0
    for word in JUMP_WORDS:
        for b in range(64):
            if (word >> b) & 1:
                a0 ^= s0
                a1 ^= s1
            _, s0, s1 = next_state(s0, s1)
    return a0, a1


def init_states(n, seed, subsequence_start=0):
    """random.py:241-257: list of (s0, s1)."""
    out = []
    if n >= 1:
        s = seed_state(seed & M64)
        for _ in range(subsequence_start & M64):
            s = jump(*s)
        out.append(s)
        for _ in range(1, n):
            s = jump(*s)
            out.append(s)
    return out


def unit_float64(x):
    """random.py:145-149.  (x >> 11) < 2^53 is exact in a double and the
    multiplication by 2^-53 only changes the exponent."""
    return (x >> 11) * (1.0 / (1 << 53))


def unit_float32(x):
    """random.py:152-156"""
    return np.float32(unit_float64(x))


def unit_float32_by_integer_rounding(x):
    """The same value derived without any floating-point conversion: round the
    53-bit integer m = x >> 11 to 24 significant bits, ties to even, then scale
    by 2^-53.  Pins the double->float step of unit_float32."""
    m = x >> 11
    if m == 0:
        return np.float32(0.0)
    nbits = m.bit_length()
    if nbits > 24:
        shift = nbits - 24
        q, r = m >> shift, m & ((1 << shift) - 1)
        half = 1 << (shift - 1)
        if r > half or (r == half and (q & 1)):
            q += 1
        m = q << shift
    # m now has at most 24 significant bits -> exactly representable
    return np.float32(np.ldexp(np.float64(m), -53))


# ----------------------------------------------------------------------------
# GF(2) linear algebra on the 128-bit state (bit i of s0 = coordinate i, bit i
# of s1 = coordinate 64 + i).  `next` is linear over GF(2), so it is a 128x128
# bit matrix and 2^64 steps are 64 squarings of it.
# ----------------------------------------------------------------------------

def _to_vec(s0, s1):
    v = np.zeros(128, np.uint8)
    for i in range(64):
        v[i] = (s0 >> i) & 1
        v[64 + i] = (s1 >> i) & 1
    return v


def _from_vec(v):
    s0 = sum(int(v[i]) << i for i in range(64))
    s1 = sum(int(v[64 + i]) << i for i in range(64))
    return s0, s1


def matrix_of(step):
    """Matrix (columns = images of the basis states) of a linear map
    step(s0, s1) -> (s0, s1)."""
    m = np.zeros((128, 128), np.uint8)
    for j in range(128):
        s0, s1 = (1 << j, 0) if j < 64 else (0, 1 << (j - 64))
        m[:, j] = _to_vec(*step(s0, s1))
    return m


def mat_mul(a, b):
    return (a.astype(np.uint32) @ b.astype(np.uint32) & 1).astype(np.uint8)


def mat_apply(m, s0, s1):
    return _from_vec((m.astype(np.uint32) @ _to_vec(s0, s1).astype(np.uint32)) & 1)


def next_matrix():
    return matrix_of(lambda a, b: next_state(a, b)[1:])


def next_pow2_matrix(log2_steps):
    m = next_matrix()
    for _ in range(log2_steps):
        m = mat_mul(m, m)
    return m
