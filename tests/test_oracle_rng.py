"""Pins the RNG part of the oracle without importing the reference.

Known answers:
 * SplitMix64 published first outputs (seed 0 and seed 1234567)
 * jump == next applied 2^64 times, by GF(2) matrix power (64 squarings)
 * algebra: next is GF(2)-linear; jump commutes with next
 * reference-held invariants: numba_cuda/numba/cuda/tests/cudapy/test_random.py
   :57-60 (10 states from seed 1 are distinct) and :62-72
   (states(seed 1, subsequence_start=3)[:-3] == states(seed 1)[3:])
 * closed form of the uint64 -> unit float conversions on edge inputs
 * C restatement == big-int restatement on long runs
"""

import numpy as np
import pytest

from oracle import cref, sim, xoroshiro_py as xp


def test_splitmix64_published_vectors():
    # first outputs of the published SplitMix64 generator
    assert xp.seed_state(0)[0] == 0xE220A8397B1DCDAF
    assert xp.seed_state(1234567)[0] == 6457827717110365317
    assert cref.seed_state(0) == (0xE220A8397B1DCDAF, 0xE220A8397B1DCDAF)
    assert cref.seed_state(1234567)[0] == 6457827717110365317
    # both words hold the same value (random.py:84-85)
    for seed in (1, 42, 2**63, 2**64 - 1):
        assert cref.seed_state(seed) == xp.seed_state(seed)
        assert cref.seed_state(seed)[0] == cref.seed_state(seed)[1]


def test_seed_is_reduced_mod_2_64():
    assert cref.seed_state(2**64 + 5) == cref.seed_state(5)
    assert cref.seed_state(-1) == xp.seed_state(2**64 - 1)


def test_next_hand_computed():
    # s0 = 1, s1 = 0: draw = 1; s1' = 1; new s0 = rotl(1,55) ^ 1 ^ (1<<14);
    # new s1 = rotl(1,36)
    d, a, b = xp.next_state(1, 0)
    assert d == 1
    assert a == (1 << 55) | 1 | (1 << 14)
    assert b == 1 << 36
    st = np.array([1, 0], np.uint64)
    assert cref.next_u64(st) == 1
    assert (int(st[0]), int(st[1])) == (a, b)
    # wrap-around of the sum and of the rotation
    d, a, b = xp.next_state(2**64 - 1, 2)
    assert d == 1
    st = np.array([2**64 - 1, 2], np.uint64)
    assert cref.next_u64(st) == 1
    assert (int(st[0]), int(st[1])) == (a, b)


def test_c_and_bigint_agree_on_a_long_run():
    s = xp.seed_state(42)
    st = np.array(s, np.uint64)
    for _ in range(200_000):
        d, a, b = xp.next_state(*s)
        s = (a, b)
        assert cref.next_u64(st) == d
    assert (int(st[0]), int(st[1])) == s


def test_next_is_gf2_linear():
    rng = np.random.default_rng(7)
    for _ in range(50):
        a = tuple(int(x) for x in rng.integers(0, 2**64, 2, dtype=np.uint64))
        b = tuple(int(x) for x in rng.integers(0, 2**64, 2, dtype=np.uint64))
        na = xp.next_state(*a)[1:]
        nb = xp.next_state(*b)[1:]
        nab = xp.next_state(a[0] ^ b[0], a[1] ^ b[1])[1:]
        assert nab == (na[0] ^ nb[0], na[1] ^ nb[1])


def test_jump_equals_2_pow_64_steps_of_next():
    """The jump polynomial is fixed by the mathematics: jumping must be the
    128x128 GF(2) matrix of `next` raised to the power 2^64."""
    big = xp.next_pow2_matrix(64)
    rng = np.random.default_rng(11)
    for _ in range(20):
        s = tuple(int(x) for x in rng.integers(0, 2**64, 2, dtype=np.uint64))
        want = xp.mat_apply(big, *s)
        assert xp.jump(*s) == want
        st = np.array(s, np.uint64)
        cref.jump(st)
        assert (int(st[0]), int(st[1])) == want
    # and a wrong power must NOT match (the check can fail)
    wrong = xp.next_pow2_matrix(63)
    assert xp.mat_apply(wrong, 1, 2) != xp.jump(1, 2)


def test_jump_commutes_with_next():
    s = xp.seed_state(99)
    a = xp.jump(*xp.next_state(*s)[1:])
    b = xp.next_state(*xp.jump(*s))[1:]
    assert a == b


def test_states_chain_c_vs_bigint_vs_sim():
    want = xp.init_states(40, 1, 2)
    got = cref.init_states(40, 1, 2)
    assert [(int(r["s0"]), int(r["s1"])) for r in got] == want
    st = np.zeros(6, cref.STATE_DTYPE)
    sim.init_states(st, 1, 2)
    assert [(int(r["s0"]), int(r["s1"])) for r in st] == want[:6]


def test_reference_invariant_distinct_states():
    s = cref.init_states(10, 1)
    assert len(np.unique(s)) == 10


def test_reference_invariant_subsequence_start():
    s1 = cref.init_states(10, 1)
    s2 = cref.init_states(10, 1, subsequence_start=3)
    np.testing.assert_array_equal(s1[3:], s2[:-3])


def test_state_record_layout():
    # random.py:47-50: aligned record {s0: u64 @0, s1: u64 @8}, 16 bytes
    assert cref.STATE_DTYPE.itemsize == 16
    assert cref.STATE_DTYPE.fields["s0"][1] == 0
    assert cref.STATE_DTYPE.fields["s1"][1] == 8


EDGE_M = [0, 1, 2**24 - 1, 2**24, 2**24 + 1, 2**53 - 2**28 - 1, 2**53 - 2**28,
          2**53 - 1, 2**29 + 1, (2**24 + 1) << 5, ((2**24 + 1) << 5) + 1,
          ((2**25 + 1) << 4), ((2**25 + 3) << 4)]


@pytest.mark.parametrize("m", EDGE_M)
def test_unit_float_closed_form(m):
    x = (m << 11) | 0x5A5  # low 11 bits are discarded
    # float64: exactly m / 2^53
    assert cref.u64_to_unit_f64(x) == m / 2.0**53
    assert xp.unit_float64(x) == m / 2.0**53
    # float32: one round-to-nearest-even of that value
    want = xp.unit_float32_by_integer_rounding(x)
    assert cref.u64_to_unit_f32(x) == want
    assert xp.unit_float32(x) == want


def test_unit_float32_can_round_up_to_one():
    # random.py:152-156 casts [0,1) double to float32: values within 2^-25 of 1
    # round to exactly 1.0f
    assert cref.u64_to_unit_f32(2**64 - 1) == np.float32(1.0)
    assert cref.u64_to_unit_f32((2**53 - 2**28) << 11) == np.float32(1.0)
    assert cref.u64_to_unit_f32((2**53 - 2**28 - 1) << 11) < np.float32(1.0)
    assert cref.u64_to_unit_f64(2**64 - 1) < 1.0


def test_unit_float32_random_inputs_vs_integer_rounding():
    rng = np.random.default_rng(3)
    for x in rng.integers(0, 2**64, 3000, dtype=np.uint64):
        x = int(x) >> int(rng.integers(0, 60))   # exercise small magnitudes too
        assert cref.u64_to_unit_f32(x) == xp.unit_float32_by_integer_rounding(x)


def test_fill_layout_and_state_advance():
    st = cref.init_states(5, 7)
    out, st2 = cref.fill(st, 3, "uniform_f64")
    for t in range(5):
        s = (int(st[t]["s0"]), int(st[t]["s1"]))
        for i in range(3):
            d, a, b = xp.next_state(*s)
            s = (a, b)
            assert out[t * 3 + i] == xp.unit_float64(d)
        assert (int(st2[t]["s0"]), int(st2[t]["s1"])) == s
    # normals consume two draws each (random.py:206-207, :231-232)
    _, st3 = cref.fill(st, 3, "normal_f32")
    _, st6 = cref.fill(st, 6, "uniform_f32")
    np.testing.assert_array_equal(st3, st6)


def test_reference_statistics_of_uniform_and_normal():
    # tests/cudapy/test_random.py:82-113 (64 states from seed 1, 32 draws each)
    st = cref.init_states(64, 1)
    for kind in ("uniform_f32", "uniform_f64"):
        out, _ = cref.fill(st, 32, kind)
        assert abs(out.min() - 0.0) < 1e-3
        assert abs(out.max() - 1.0) < 1e-3
        assert abs(out.mean() - 0.5) < 1.5e-2
        assert abs(out.std() - 1.0 / (2 * np.sqrt(3))) < 6e-3
    for kind in ("normal_f32", "normal_f64"):
        out, _ = cref.fill(st, 32, kind)
        assert abs(out.mean()) < 4e-3
        assert abs(out.std() - 1.0) < 2e-3


def test_normal_precision_mix():
    """random.py:191-238 restated with numpy scalars of the stated widths."""
    st = cref.init_states(8, 5)
    u, _ = cref.fill(st, 2, "uniform_f32")
    n32, _ = cref.fill(st, 1, "normal_f32")
    n64, _ = cref.fill(st, 1, "normal_f64")
    for t in range(8):
        u1, u2 = np.float32(u[2 * t]), np.float32(u[2 * t + 1])
        lg = np.float32(np.log(np.float64(u1)))
        z32 = np.float32(np.sqrt(np.float64(np.float32(-2.0) * lg))) * np.float32(
            np.cos(np.float64(np.float32(2 * np.pi) * u2)))
        assert abs(np.float32(z32) - n32[t]) <= 2 * np.spacing(np.abs(n32[t]))
        z64 = np.sqrt(-2.0 * np.float64(lg)) * np.cos(np.float64(2 * np.pi) * np.float64(u2))
        assert abs(z64 - n64[t]) <= 4 * np.spacing(np.abs(n64[t]))


def test_simulator_flavour_normals_track_the_compiled_flavour():
    """The simulator evaluates log/cos through Python floats (random.py:191-238 in
    object mode); the compiled flavour takes a float32 logarithm.  Same uniforms, same
    states afterwards, values equal to within a float32 rounding of log(u1)."""
    st = cref.init_states(16, 7)
    for kind, draw, tol in (("normal_f32", sim.normal_float32, 2e-6), ("normal_f64", sim.normal_float64, 2e-6)):
        want, after = cref.fill(st, 3, kind)
        mine = st.copy()
        got = np.array([[draw(mine, t) for _ in range(3)] for t in range(16)]).reshape(-1)
        np.testing.assert_array_equal(mine, after)          # two generator steps per normal
        np.testing.assert_allclose(got, want, rtol=tol, atol=1e-7)
