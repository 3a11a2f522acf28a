"""The committed fixtures (tests/golden/*.json, written by tests/golden/make_golden.py
from the big-int and lock-step restatements) against the C oracle: a second, frozen
opinion on what the oracle computes."""
import json
import os

import numpy as np
import pytest

from oracle import cref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with open(os.path.join(GOLDEN, name)) as fh:
        return json.load(fh)


def reduce_inputs(case):
    """The seeded inputs of one reduce_order_vectors.json case."""
    rng = np.random.default_rng(case["seed"])
    f = rng.standard_normal(case["n"]).astype(np.float32)
    i = rng.integers(-2**20, 2**20, case["n"], dtype=np.int64, endpoint=True)
    near_one = (1 + 1e-3 * np.random.default_rng(case["seed"] + 100).standard_normal(case["n"])).astype(np.float32)
    return f, i, near_one


def test_published_splitmix64_outputs():
    for vec in load("xoroshiro128p_vectors.json")["splitmix64_published"]:
        s = cref.seed_state(vec["seed"])
        assert int(s[0]) == int(s[1]) == vec["first_output"]


def test_state_chains():
    for chain in load("xoroshiro128p_vectors.json")["chains"]:
        want = chain["states"]
        got = cref.init_states(len(want), chain["seed"], chain["subsequence_start"]) \
            if chain["subsequence_start"] <= 64 else None
        if got is None:
            continue          # 2^20 jumps: only the matrix route and the GPU get there
        assert [[int(r["s0"]), int(r["s1"])] for r in got] == want


def test_draws_and_unit_conversions():
    for vec in load("xoroshiro128p_vectors.json")["draws"]:
        st = np.zeros(1, cref.STATE_DTYPE)
        s = cref.seed_state(vec["seed"])
        st[0]["s0"], st[0]["s1"] = s[0], s[1]
        u64, after = cref.fill(st, 12, "uniform_f64")
        assert u64.view(np.uint64).tolist() == vec["uniform_f64_bits"]
        u32, after32 = cref.fill(st, 12, "uniform_f32")
        assert u32.view(np.uint32).tolist() == vec["uniform_f32_bits"]
        assert [int(after[0]["s0"]), int(after[0]["s1"])] == vec["state_after"]
        assert after32.tobytes() == after.tobytes()
        raw = np.array(vec["next_u64"], dtype=np.uint64)
        assert [cref.u64_to_unit_f64(int(x)) for x in raw] == u64.tolist()


@pytest.mark.parametrize("case", load("reduce_order_vectors.json")["cases"], ids=lambda c: "n%d" % c["n"])
def test_reduction_in_reference_order(case):
    f, i, near_one = reduce_inputs(case)
    for op, bits in case["float32_standard_normal"].items():
        got = cref.tree(op, f, np.float32(0.5))
        assert int(np.float32(got).view(np.uint32)) == bits, op
    assert int(np.float32(cref.tree("mul", near_one, 1)).view(np.uint32)) == case["float32_near_one_product"]
    for op, want in case["int64_uniform_pm_2_20"].items():
        assert int(cref.tree(op, i, 3)) == want == int(cref.fold(op, i, 3))


def test_closed_forms():
    forms = load("closed_forms.json")
    for row in forms["sum_of_1_to_n"]:
        a = np.arange(row["n"], dtype=np.float64) + 1
        assert cref.tree("add", a, 0) == row["sum"] == cref.fold("add", a, 0)
    assert int(cref.tree("mul", np.arange(1, 21, dtype=np.int64), 1)) == forms["factorial_20_int64"]
    assert cref.transpose(np.arange(12).reshape(3, 4)).tolist() == forms["transpose_of_arange_3x4"]
