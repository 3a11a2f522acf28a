"""The committed fixtures (tests/golden/*.json) against the GPU, through the public API
and hence the C ABI: RNG states and uniform bits exactly, integer reductions exactly,
float32 reductions within 2 n eps sum|x| of the fixture's value (the fixture follows
the reference's association, the GPU its own), closed forms exactly."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd import random as nrandom
from oracle import cref
from tests.test_golden import load, reduce_inputs


def test_state_chains_on_the_device():
    for chain in load("xoroshiro128p_vectors.json")["chains"]:
        want = chain["states"]
        states = nrandom.create_xoroshiro128p_states(len(want), chain["seed"], chain["subsequence_start"])
        got = states.copy_to_host()
        assert [[int(r["s0"]), int(r["s1"])] for r in got] == want, (chain["seed"], chain["subsequence_start"])
    # a long array passes through the table kernel: its first states must be the same ones
    chain = load("xoroshiro128p_vectors.json")["chains"][2]
    got = nrandom.create_xoroshiro128p_states(1 << 19, chain["seed"], chain["subsequence_start"]).copy_to_host()
    assert [[int(r["s0"]), int(r["s1"])] for r in got[:len(chain["states"])]] == chain["states"]


def test_uniform_draw_bits_on_the_device():
    for vec in load("xoroshiro128p_vectors.json")["draws"]:
        for kind, key, dtype, bits in (("f32", "uniform_f32_bits", np.float32, np.uint32),
                                       ("f64", "uniform_f64_bits", np.float64, np.uint64)):
            host = np.zeros(1, nrandom.xoroshiro128p_dtype)
            nrandom.init_xoroshiro128p_state(host, 0, vec["seed"])
            states = cuda.to_device(host)
            out = cuda.device_array(12, dtype)
            nrandom.xoroshiro128p_fill(states, out, 12, nrandom.UNIFORM)
            assert out.copy_to_host().view(bits).tolist() == vec[key], (vec["seed"], kind)
            after = states.copy_to_host()[0]
            assert [int(after["s0"]), int(after["s1"])] == vec["state_after"]


@pytest.mark.parametrize("case", load("reduce_order_vectors.json")["cases"], ids=lambda c: "n%d" % c["n"])
def test_reductions_against_reference_order_values(case):
    f, i, near_one = reduce_inputs(case)
    n = case["n"]
    eps = np.finfo(np.float32).eps
    ops = {"add": lambda a, b: a + b, "max": lambda a, b: max(a, b), "min": lambda a, b: min(a, b)}
    for op, bits in case["float32_standard_normal"].items():
        want = np.array([bits], np.uint32).view(np.float32)[0]
        got = cuda.Reduce(ops[op])(f, init=0.5)
        if op == "add":
            _, sum_abs = cref.sum_exact(f)
            assert abs(float(got) - float(want)) <= 2 * (2 * n * eps * (sum_abs + 0.5))   # tolerance: 2 x (2 n eps sum|x|)
        else:
            assert got == want
    want = np.array([case["float32_near_one_product"]], np.uint32).view(np.float32)[0]
    got = cuda.Reduce(lambda a, b: a * b)(near_one, init=1)
    assert abs(float(got) / float(want) - 1) <= 4 * n * eps                               # tolerance: 4 n eps, relative
    for op, value in case["int64_uniform_pm_2_20"].items():
        assert int(cuda.Reduce(ops[op])(i, init=3)) == value
    # in the reference's association order the device reproduces the recorded bits
    for op, bits in case["float32_standard_normal"].items():
        got = cuda.Reduce(ops[op], reference_order=True)(f, init=0.5)
        assert int(np.asarray(got).view(np.uint32)) == bits, (n, op)
    got = cuda.Reduce(lambda a, b: a * b, reference_order=True)(near_one, init=1)
    assert int(np.asarray(got).view(np.uint32)) == case["float32_near_one_product"], n


def test_closed_forms_on_the_device():
    forms = load("closed_forms.json")
    add = cuda.Reduce(lambda a, b: a + b)
    for row in forms["sum_of_1_to_n"]:
        assert add(np.arange(row["n"], dtype=np.float64) + 1) == row["sum"]
    assert int(cuda.Reduce(lambda a, b: a * b)(np.arange(1, 21, dtype=np.int64), init=1)) == forms["factorial_20_int64"]
    t = cuda.to_device(np.arange(12).reshape(3, 4)).T.copy_to_host()
    assert t.tolist() == forms["transpose_of_arange_3x4"]
