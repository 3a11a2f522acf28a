"""Writes the fixtures in this directory.

    python tests/golden/make_golden.py

The reference (numba-cuda) cannot be imported where this repository is built (no
numba / llvmlite / CUDA), and it ships no golden-vector files for this path, so the
vectors are produced by the two INDEPENDENT restatements that the oracle itself is
pinned against - never by the C oracle or the GPU code they are later compared with:

  * xoroshiro128p_vectors.json   oracle/xoroshiro_py.py (Python big-int arithmetic,
        reference: numba_cuda/numba/cuda/random.py:62-184, :241-257) plus the two
        published SplitMix64 outputs (seed 0 and seed 1234567)
  * reduce_order_vectors.json    oracle/reduce_simt.py (a literal lock-step emulation
        of numba_cuda/numba/cuda/kernels/reduction.py:22-166 and of the launches at
        :194-265) on seeded inputs; float results as bit patterns
  * closed_forms.json            answers fixed by arithmetic: n(n+1)/2 for the sizes the
        reference tests use (tests/cudapy/test_reduction.py:15-47), 20!, a transposed
        index pattern

Inputs are regenerated in the tests from the recorded seeds with numpy's default_rng.
"""
import json
import os
import struct
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import reduce_simt, xoroshiro_py as xp  # noqa: E402


def f32_bits(x):
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def f64_bits(x):
    return struct.unpack("<Q", struct.pack("<d", float(x)))[0]


def rng_vectors():
    out = {"splitmix64_published": [{"seed": 0, "first_output": 0xE220A8397B1DCDAF},
                                    {"seed": 1234567, "first_output": 6457827717110365317}],
           "chains": [], "draws": []}
    for seed, start, n in ((0, 0, 6), (1, 0, 6), (42, 0, 6), (42, 5, 6), (2**64 - 1, 3, 4), (12345, 2**20, 3)):
        if start <= 64:
            states = xp.init_states(n, seed, start)
        else:
            # advance by `start` jumps with the matrix powers (2^20 jumps are out of reach step by step)
            s = xp.seed_state(seed)
            for k in range(start.bit_length()):
                if (start >> k) & 1:
                    s = xp.mat_apply(xp.next_pow2_matrix(64 + k), *s)
            states = [s]
            for _ in range(n - 1):
                states.append(xp.jump(*states[-1]))
        out["chains"].append({"seed": seed, "subsequence_start": start,
                              "states": [[int(a), int(b)] for a, b in states]})
    for seed in (0, 7, 42):
        s = xp.seed_state(seed)
        raw, u32, u64 = [], [], []
        for _ in range(12):
            x, a, b = xp.next_state(*s)
            s = (a, b)
            raw.append(int(x))
            u32.append(f32_bits(xp.unit_float32(x)))
            u64.append(f64_bits(xp.unit_float64(x)))
        out["draws"].append({"seed": seed, "next_u64": raw, "uniform_f32_bits": u32, "uniform_f64_bits": u64,
                             "state_after": [int(s[0]), int(s[1])]})
    return out


def reduce_vectors():
    cases = []
    for seed, n in ((1, 1), (2, 31), (3, 33), (4, 127), (5, 128), (6, 129), (7, 1000), (8, 8192), (9, 8321),
                    (10, 20000)):
        rng = np.random.default_rng(seed)
        f = rng.standard_normal(n).astype(np.float32)
        i = rng.integers(-2**20, 2**20, n, dtype=np.int64, endpoint=True)
        near_one = (1 + 1e-3 * np.random.default_rng(seed + 100).standard_normal(n)).astype(np.float32)
        cases.append({
            "seed": seed, "n": n,
            "float32_standard_normal": {op: f32_bits(reduce_simt.reduce(op, f, init=np.float32(0.5) if op != "mul" else 1))
                                        for op in ("add", "max", "min")},
            "float32_near_one_product": f32_bits(reduce_simt.reduce("mul", near_one, init=1)),
            "int64_uniform_pm_2_20": {op: int(reduce_simt.reduce(op, i, init=3)) for op in ("add", "max", "min")},
        })
    return {"note": "float32 init is 0.5 for add/max/min and 1 for the product; int64 init is 3", "cases": cases}


def closed_forms():
    sizes = [1, 15, 16, 17, 31, 32, 33, 127, 128, 129, 1023, 1024, 1025, 1536, 1048576, 1049600, 1049600 + 1, 1053696,
             1053696 + 1, 1053696 + 15]
    fact = 1
    for k in range(1, 21):
        fact *= k
    return {"sum_of_1_to_n": [{"n": n, "sum": n * (n + 1) // 2} for n in sizes],
            "factorial_20_int64": fact,
            "transpose_of_arange_3x4": [[0, 4, 8], [1, 5, 9], [2, 6, 10], [3, 7, 11]]}


def main():
    for name, data in (("xoroshiro128p_vectors.json", rng_vectors()), ("reduce_order_vectors.json", reduce_vectors()),
                       ("closed_forms.json", closed_forms())):
        with open(os.path.join(HERE, name), "w") as fh:
            json.dump(data, fh, indent=1)
            fh.write("\n")
        print("wrote", name)


if __name__ == "__main__":
    main()
