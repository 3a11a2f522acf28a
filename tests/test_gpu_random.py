"""Parity of the xoroshiro128+ device path with the oracle: states and uniform
bits exact; Box-Muller normals within 2 ulp of the correctly rounded restatement
(their bit-level parity with the reference's libdevice is unpinned: no file of
the reference records those bits)."""

import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd import random as nrandom
from oracle import cref


def _say(*a):
    print(*a, flush=True)


def test_create_distinct_states():
    # numba_cuda/numba/cuda/tests/cudapy/test_random.py:57-60
    s = cuda.random.create_xoroshiro128p_states(10, seed=1).copy_to_host()
    assert s.dtype == nrandom.xoroshiro128p_dtype
    assert len(np.unique(s)) == 10


def test_create_subsequence_start():
    # test_random.py:62-72
    s1 = cuda.random.create_xoroshiro128p_states(10, seed=1).copy_to_host()
    s2 = cuda.random.create_xoroshiro128p_states(10, seed=1, subsequence_start=3).copy_to_host()
    np.testing.assert_array_equal(s1[3:], s2[:-3])


def test_create_stream():
    stream = cuda.stream()
    s = cuda.random.create_xoroshiro128p_states(10, seed=1, stream=stream)
    stream.synchronize()
    assert len(np.unique(s.copy_to_host())) == 10


@pytest.mark.parametrize("n,seed,start", [(1, 0, 0), (10, 1, 0), (63, 1, 1), (64, 42, 0), (65, 42, 5),
                                          (4095, 7, 2), (4097, 2**64 - 1, 0), (16385, -3, 9),
                                          (70001, 42, 0), (262143, 3, 1), (262144, 5, 2),
                                          (300000, 12345678901234567890, 17), (1048576 + 4097, 8, 3),
                                          (3 * 2**20 + 100, 11, 4), (2**23 - 5, 6, 1)])
def test_states_bit_exact_against_sequential_chain(n, seed, start):
    _say("states", n, seed, start)
    got = cuda.random.create_xoroshiro128p_states(n, seed=seed, subsequence_start=start).copy_to_host()
    np.testing.assert_array_equal(got, cref.init_states(n, seed, start))


def test_states_of_random_sizes_seeds_and_starts():
    """Sizes on both sides of every choice the launch makes (one step per wavefront up to 2^18
    states, more above; whole and ragged last runs), random seeds and subsequence starts."""
    rng = np.random.default_rng(77)
    sizes = [int(rng.integers(1, 5000)) for _ in range(4)] + [int(rng.integers(5000, 300000)) for _ in range(4)] + \
            [int(rng.integers(300000, 3000000)) for _ in range(4)] + [262145, 524288, 524289, 4096 * 64 * 3]
    for n in sizes:
        seed = int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2))
        start = int(rng.integers(0, 2**20))
        _say("states, random", n, seed, start)
        got = cuda.random.create_xoroshiro128p_states(n, seed=seed, subsequence_start=start).copy_to_host()
        np.testing.assert_array_equal(got, cref.init_states(n, seed, start))


def test_huge_subsequence_start_is_consistent():
    """2^40+3 and 2^64-1 jumps cannot be walked sequentially; the chain property
    states[i+1] == jump(states[i]) and the shift property still pin them."""
    for start in (2**40 + 3, 2**64 - 1):
        got = cuda.random.create_xoroshiro128p_states(300, seed=9, subsequence_start=start).copy_to_host()
        st = np.array([got[0]["s0"], got[0]["s1"]], np.uint64)
        for i in range(1, 300):
            cref.jump(st)
            assert (got[i]["s0"], got[i]["s1"]) == (st[0], st[1])
    a = cuda.random.create_xoroshiro128p_states(5, seed=9, subsequence_start=2**40).copy_to_host()
    b = cuda.random.create_xoroshiro128p_states(5, seed=9, subsequence_start=2**40 + 2).copy_to_host()
    np.testing.assert_array_equal(a[2:], b[:-2])


def _ulps(got, want):
    fin = np.isfinite(want)
    assert np.array_equal(got[~fin], want[~fin], equal_nan=True)
    return np.abs(got[fin].astype(np.float64) - want[fin].astype(np.float64)) / \
        np.spacing(np.abs(want[fin])).astype(np.float64)


@pytest.mark.parametrize("n", [1, 64, 257, 5000, 70001])
@pytest.mark.parametrize("kind,count", [("uniform_f32", 64), ("uniform_f32", 1), ("uniform_f32", 33),
                                        ("uniform_f32", 128), ("uniform_f32", 192), ("uniform_f32", 96),
                                        ("uniform_f64", 7), ("uniform_f64", 40), ("uniform_f64", 32), ("uniform_f64", 96),
                                        ("normal_f32", 33), ("normal_f64", 16)])
def test_fill_against_oracle(n, kind, count):
    _say("fill", kind, n, count)
    host_states = cref.init_states(n, 42, 5)
    states = cuda.to_device(host_states)
    dtype = np.float32 if kind.endswith("f32") else np.float64
    out = cuda.device_array(n * count, dtype=dtype)
    dist = nrandom.UNIFORM if kind.startswith("uniform") else nrandom.NORMAL
    nrandom.xoroshiro128p_fill(states, out, count, dist)
    want, want_states = cref.fill(host_states, count, kind)
    got = out.copy_to_host()
    np.testing.assert_array_equal(states.copy_to_host(), want_states)
    if dist == nrandom.UNIFORM:
        assert got.tobytes() == want.tobytes()
    else:
        assert _ulps(got, want).max() <= 2.0      # tolerance: 2 ulp


@pytest.mark.parametrize("kind", ["uniform_f32", "uniform_f64", "normal_f32", "normal_f64"])
def test_fill_for_every_kind_of_round(kind):
    """Runs of every shape: whole rounds (128 bytes per generator), short rounds of whole
    16-byte packets, ragged rounds, runs longer than a line that start anywhere in it,
    with the output starting on and off a 128-byte line and generator counts that leave
    the last wavefront partly empty."""
    dtype = np.float32 if kind.endswith("f32") else np.float64
    dist = nrandom.UNIFORM if kind.startswith("uniform") else nrandom.NORMAL
    for n in (300, 65, 1):
        host_states = cref.init_states(n, 7, 1)
        # the last row: runs of whole lines, in rounds of one, two or four lines with every tail
        for count in (1, 2, 3, 4, 8, 12, 15, 16, 17, 24, 25, 31, 32, 33, 36, 47, 48, 49, 50, 63, 64, 65, 97, 100, 127,
                      129, 250,
                      80, 96, 128, 160, 512, 528, 544, 560, 1024, 1056, 1088, 1120):
            if n != 300 and count not in (3, 25, 50, 64, 97, 250, 96, 560, 1120):
                continue
            if count > 250 and dist != nrandom.UNIFORM and count not in (512, 560):
                continue
            for lead in (0, 1, 5):
                _say("fill rounds", kind, n, count, lead)
                states = cuda.to_device(host_states)
                # values before and after the runs must stay as they are
                buf = cuda.to_device(np.full(n * count + lead + 40, -7, dtype=dtype))
                out = buf[lead:lead + n * count]
                nrandom.xoroshiro128p_fill(states, out, count, dist)
                want, want_states = cref.fill(host_states, count, kind)
                whole = buf.copy_to_host()
                got = whole[lead:lead + n * count]
                assert (whole[:lead] == -7).all() and (whole[lead + n * count:] == -7).all(), (n, count, lead)
                np.testing.assert_array_equal(states.copy_to_host(), want_states)
                if dist == nrandom.UNIFORM:
                    assert got.tobytes() == want.tobytes(), (n, count, lead)
                else:
                    assert _ulps(got, want).max() <= 2.0, (n, count, lead)      # tolerance: 2 ulp


def test_reference_statistics():
    # test_random.py:82-113
    for dtype in (np.float32, np.float64):
        states = cuda.random.create_xoroshiro128p_states(64, seed=1)
        out = cuda.device_array(64 * 32, dtype=dtype)
        u = nrandom.xoroshiro128p_fill(states, out, 32, nrandom.UNIFORM).copy_to_host()
        assert abs(u.min()) < 1e-3 and abs(u.max() - 1.0) < 1e-3
        assert abs(u.mean() - 0.5) < 1.5e-2
        assert abs(u.std() - 1.0 / (2 * math.sqrt(3))) < 6e-3
        states = cuda.random.create_xoroshiro128p_states(64, seed=1)
        g = nrandom.xoroshiro128p_fill(states, out, 32, nrandom.NORMAL).copy_to_host()
        assert abs(g.mean()) < 4e-3
        assert abs(g.std() - 1.0) < 2e-3


def test_float32_uniform_can_be_exactly_one_and_log_of_zero_is_unguarded():
    # states chosen so that the first draw s0 + s1 is all ones / zero
    st = np.zeros(2, nrandom.xoroshiro128p_dtype)
    st[0] = (2**64 - 1, 0)       # draw = 2^64-1 -> 1.0f
    st[1] = (0, 0)               # draw = 0      -> 0.0f -> log = -inf -> inf * cos
    d = cuda.to_device(st)
    out = cuda.device_array(2, np.float32)
    nrandom.xoroshiro128p_fill(d, out, 1, nrandom.UNIFORM)
    got = out.copy_to_host()
    assert got[0] == np.float32(1.0) and got[1] == 0.0
    d = cuda.to_device(st)
    nrandom.xoroshiro128p_fill(d, out, 1, nrandom.NORMAL)
    want, _ = cref.fill(st, 1, "normal_f32")
    np.testing.assert_array_equal(out.copy_to_host(), want)


def test_montecarlo_integration_end_to_end():
    """docs example (tests/doc_examples/test_montecarlo.py:109-115): integral of
    1/x over [1,2] and [2,3] with RNG + reduce, seed 42."""
    n = 1_000_000
    states = cuda.random.create_xoroshiro128p_states(n, seed=42)
    u = cuda.device_array(n, np.float32)
    nrandom.xoroshiro128p_fill(states, u, 1, nrandom.UNIFORM)
    uh = u.copy_to_host().astype(np.float64)
    for lo, hi, want in ((1, 2, 0.69315), (2, 3, 0.4055)):
        y = (1.0 / (lo + uh * (hi - lo))).astype(np.float32)
        est = cuda.reduce(lambda a, b: a + b)(cuda.to_device(y)) * (hi - lo) / n
        assert abs(est - want) < 1e-3


# ---- full-size case: 2^24 generators -----------------------------------------------------

@pytest.mark.parametrize("start", [0, 5])
def test_fullsize_states_2_pow_24(start):
    n = 2**24
    states = cuda.random.create_xoroshiro128p_states(n, seed=42, subsequence_start=start)
    got = states.copy_to_host()
    _say("oracle chain for", n)
    want = cref.init_states(n, 42, start)
    assert got.tobytes() == want.tobytes()


def test_fullsize_uniform_float32_2_pow_30_and_normal_float64():
    n, count = 2**24, 64
    host_states = cref.init_states(n, 42, 0)
    states = cuda.to_device(host_states)
    out = cuda.device_array(n * count, np.float32)
    nrandom.xoroshiro128p_fill(states, out, count, nrandom.UNIFORM)
    after = states.copy_to_host()
    chunk = 2**20
    for lo in range(0, n, chunk):
        want, want_states = cref.fill(host_states[lo:lo + chunk], count, "uniform_f32")
        got = out[lo * count:(lo + chunk) * count].copy_to_host()
        assert got.tobytes() == want.tobytes(), lo
        assert after[lo:lo + chunk].tobytes() == want_states.tobytes(), lo
    del out
    # separately, fresh states: 16 normal float64 per generator
    states = cuda.to_device(host_states)
    out = cuda.device_array(n * 16, np.float64)
    nrandom.xoroshiro128p_fill(states, out, 16, nrandom.NORMAL)
    after = states.copy_to_host()
    worst = 0.0
    for lo in range(0, n, chunk):
        want, want_states = cref.fill(host_states[lo:lo + chunk], 16, "normal_f64")
        got = out[lo * 16:(lo + chunk) * 16].copy_to_host()
        worst = max(worst, _ulps(got, want).max())
        assert after[lo:lo + chunk].tobytes() == want_states.tobytes(), lo
    _say("normal_f64 worst ulp", worst)
    assert worst <= 2.0


def test_normals_over_every_float32_mantissa_of_u1():
    """The logarithm is the sensitive step of Box-Muller: a one-ulp float32
    difference in log(u1) moves a float64 normal by ~2^28 ulp.  Sweep u1 over every
    24-bit mantissa of two binades (crafted states whose first draw is chosen) and
    require the usual 2 ulp against the oracle for both variants."""
    n = 1 << 23
    mant = np.arange(n, dtype=np.uint64)
    rng = np.random.default_rng(11)
    for top in (np.uint64(1) << np.uint64(63), np.uint64(1) << np.uint64(62)):
        # first draw = s0 + s1; u1 = float32((draw >> 11) * 2^-53): put the mantissa
        # just below the leading bit, random low bits
        draw = top | (mant << np.uint64(40 if top >> np.uint64(63) else 39)) | \
            rng.integers(0, 1 << 30, n, dtype=np.uint64)
        st = np.zeros(n, nrandom.xoroshiro128p_dtype)
        st["s1"] = rng.integers(0, 2**63, n, dtype=np.uint64)
        st["s0"] = draw - st["s1"]
        for kind, dtype in (("normal_f32", np.float32), ("normal_f64", np.float64)):
            d = cuda.to_device(st)
            out = cuda.device_array(n, dtype)
            nrandom.xoroshiro128p_fill(d, out, 1, nrandom.NORMAL)
            want, want_states = cref.fill(st, 1, kind)
            got = out.copy_to_host()
            u = _ulps(got, want)
            _say(kind, "binade", int(top).bit_length(), "worst ulp", u.max(), "mismatching", int((u > 0).sum()))
            assert u.max() <= 2.0
            np.testing.assert_array_equal(d.copy_to_host(), want_states)


@pytest.mark.parametrize("binades", [range(1, 7), range(7, 13), range(13, 19), range(19, 25), range(25, 31),
                                     range(31, 54)])
def test_normals_for_every_value_the_first_uniform_can_take(binades):
    """u1 = float32((draw >> 11) * 2^-53) is zero or one of 30 * 2^23 + 2^23 - 1 values: all 2^23
    mantissas of the binades [2^-k, 2^-k+1) for k = 1 .. 30, and below that the multiples of
    2^-53.  Every one of them goes through the device's logarithm and square root here (states
    made so that the first draw is the chosen one; the second uniform is whatever the state
    then yields): float32 normals must have the oracle's bits, float64 normals stay within
    2 ulp."""
    rng = np.random.default_rng(binades[0])
    for k in binades:
        if k <= 30:
            mant = np.arange(1 << 23, dtype=np.uint64)
            m53 = ((np.uint64(1) << np.uint64(23)) | mant) << np.uint64(30 - k)
        else:
            m53 = np.arange(1 << (53 - k), 1 << (54 - k), dtype=np.uint64)
        n = m53.size
        draw = m53 << np.uint64(11)
        st = np.zeros(n, nrandom.xoroshiro128p_dtype)
        st["s1"] = rng.integers(0, 2**63, n, dtype=np.uint64)
        st["s0"] = draw - st["s1"]
        for kind, dtype in (("normal_f32", np.float32), ("normal_f64", np.float64)):
            d = cuda.to_device(st)
            out = cuda.device_array(n, dtype)
            nrandom.xoroshiro128p_fill(d, out, 1, nrandom.NORMAL)
            want, _ = cref.fill(st, 1, kind)
            got = out.copy_to_host()
            if dtype is np.float32:
                assert got.tobytes() == want.tobytes(), (k, kind, int((got != want).sum()))
            else:
                u = _ulps(got, want)
                assert u.max() <= 2.0, (k, kind, float(u.max()))
        _say("binade 2^-%d: %d values of u1" % (k, n))


def _states_whose_second_draw_is(draw2, rng):
    """States (s0, s1) whose SECOND 64-bit draw is `draw2`: pick the state after the first
    step freely (s0' + s1' = draw2) and run the step backwards (random.py:62-93:
    s1' = rotl(t, 36), s0' = rotl(s0, 55) ^ t ^ (t << 14) with t = s0 ^ s1)."""
    u64 = np.uint64
    def rotr(x, k):
        return (x >> u64(k)) | (x << u64(64 - k))
    s1n = rng.integers(0, 2**63, draw2.size, dtype=np.uint64)
    s0n = draw2 - s1n
    t = rotr(s1n, 36)
    s0 = rotr(s0n ^ t ^ (t << u64(14)), 55)
    st = np.zeros(draw2.size, nrandom.xoroshiro128p_dtype)
    st["s0"] = s0
    st["s1"] = t ^ s0
    return st


@pytest.mark.parametrize("binades", [range(1, 7), range(7, 13), range(13, 19), range(19, 25), range(25, 31),
                                     range(31, 54)])
def test_normals_for_every_value_the_second_uniform_can_take(binades):
    """The same for u2, the argument of the cosine: states whose second draw is the chosen one
    (the step run backwards), the first uniform whatever it then is."""
    rng = np.random.default_rng(100 + binades[0])
    for k in binades:
        if k <= 30:
            mant = np.arange(1 << 23, dtype=np.uint64)
            m53 = ((np.uint64(1) << np.uint64(23)) | mant) << np.uint64(30 - k)
        else:
            m53 = np.arange(1 << (53 - k), 1 << (54 - k), dtype=np.uint64)
        st = _states_whose_second_draw_is(m53 << np.uint64(11), rng)
        if k == 1:   # the construction itself: the oracle's second uniform is the chosen one
            u, _ = cref.fill(st[:1000], 2, "uniform_f64")
            assert (u.reshape(-1, 2)[:, 1] == m53[:1000].astype(np.float64) * 2.0**-53).all()
        n = st.size
        for kind, dtype in (("normal_f32", np.float32), ("normal_f64", np.float64)):
            d = cuda.to_device(st)
            out = cuda.device_array(n, dtype)
            nrandom.xoroshiro128p_fill(d, out, 1, nrandom.NORMAL)
            want, _ = cref.fill(st, 1, kind)
            got = out.copy_to_host()
            if dtype is np.float32:
                assert got.tobytes() == want.tobytes(), (k, kind, int((got != want).sum()))
            else:
                u = _ulps(got, want)
                assert u.max() <= 2.0, (k, kind, float(u.max()))
        _say("binade 2^-%d: %d values of u2" % (k, n))


def test_scalar_functions_on_device_resident_states():
    """numba_cuda/numba/cuda/random.py:96-238 called from host code on the array
    create_xoroshiro128p_states returned: state and integer / uniform bits exact against
    the oracle, normals within 2 ulp of it and bit-equal to the bulk fill."""
    n = 6
    states = cuda.random.create_xoroshiro128p_states(n, seed=1)
    host = cref.init_states(n, 1)
    np.testing.assert_array_equal(states.copy_to_host(), host)

    # next: the raw 64-bit draws of generators 4 and -1, interleaved
    twin = {4: np.array([host[4]["s0"], host[4]["s1"]], np.uint64),
            5: np.array([host[5]["s0"], host[5]["s1"]], np.uint64)}
    for i in range(20):
        for idx, key in ((4, 4), (-1, 5)):
            got = nrandom.xoroshiro128p_next(states, idx)
            assert isinstance(got, np.uint64) and int(got) == cref.next_u64(twin[key]), (i, idx)
    after = states.copy_to_host()
    assert (after[4]["s0"], after[4]["s1"]) == tuple(twin[4])
    assert (after[5]["s0"], after[5]["s1"]) == tuple(twin[5])
    np.testing.assert_array_equal(after[:4], host[:4])            # the others did not move

    # uniform draws: bit patterns of generator 0 (float32) and 1 (float64)
    want32, st32 = cref.fill(host[0:1], 9, "uniform_f32")
    got32 = np.array([nrandom.xoroshiro128p_uniform_float32(states, 0) for _ in range(9)])
    assert got32.dtype == np.float32 and got32.tobytes() == want32.tobytes()
    want64, st64 = cref.fill(host[1:2], 9, "uniform_f64")
    got64 = np.array([nrandom.xoroshiro128p_uniform_float64(states, 1) for _ in range(9)])
    assert got64.dtype == np.float64 and got64.tobytes() == want64.tobytes()
    after = states.copy_to_host()
    np.testing.assert_array_equal(after[0:1], st32)
    np.testing.assert_array_equal(after[1:2], st64)

    # normal draws of generators 2 and 3: two steps per value
    for idx, kind, fn, dtype in ((2, "normal_f32", nrandom.xoroshiro128p_normal_float32, np.float32),
                                 (3, "normal_f64", nrandom.xoroshiro128p_normal_float64, np.float64)):
        want, st = cref.fill(host[idx:idx + 1], 11, kind)
        bulk_states = cuda.to_device(host[idx:idx + 1])
        bulk = cuda.device_array(11, dtype=dtype)
        nrandom.xoroshiro128p_fill(bulk_states, bulk, 11, nrandom.NORMAL)
        got = np.array([fn(states, idx) for _ in range(11)])
        assert got.dtype == dtype
        assert got.tobytes() == bulk.copy_to_host().tobytes()
        assert _ulps(got, want).max() <= 2.0                       # tolerance: 2 ulp
        np.testing.assert_array_equal(states.copy_to_host()[idx:idx + 1], st)

    # jump: one step along the chain of subsequences
    fresh = cuda.random.create_xoroshiro128p_states(4, seed=9)
    chain = cref.init_states(5, 9)
    for idx in range(4):
        assert nrandom.xoroshiro128p_jump(fresh, idx) is None
    np.testing.assert_array_equal(fresh.copy_to_host(), chain[1:])

    # seeding one generator in place
    nrandom.init_xoroshiro128p_state(fresh, 2, 12345)
    s0, s1 = cref.seed_state(12345)
    got = fresh.copy_to_host()
    assert (int(got[2]["s0"]), int(got[2]["s1"])) == (s0, s1)
    np.testing.assert_array_equal(got[[0, 1, 3]], chain[[1, 2, 4]])

    with pytest.raises(IndexError):
        nrandom.xoroshiro128p_next(states, n)
