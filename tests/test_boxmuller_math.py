"""Host-side sweep of the Box-Muller logarithm and cosine (numba_cuda_amd/csrc/
boxmuller_math.h) against long double: the same source the GPU kernels compile, built
here with g++.  What is checked is independent of the oracle: x87 `logl` / `cosl`
carry 64 bits, eleven more than the routines under test produce."""
import os
import re
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "numba_cuda_amd", "csrc")


@pytest.fixture(scope="module")
def sweep(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("bm") / "check")
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-pthread", "-I", CSRC,
                    os.path.join(HERE, "boxmuller_math_check.cpp"), "-o", exe], check=True)
    # every 7th mantissa: 1.2 M logarithms per binade and 2.4 M cosines per variant in ~1.5 s;
    # "all": also the float32 rounding of the logarithm and of the float32 variant's cosine for
    # every possible argument (~40 core-seconds, 5 s on 8 cores)
    out = subprocess.run([exe, "7", "all"], check=True, capture_output=True, text=True).stdout
    return out


def test_logarithm_is_within_one_ulp_and_rounds_to_the_right_float32(sweep):
    rows = re.findall(r"log binade 2\^-(\d+): n=(\d+) worst_ulp=([\d.]+) float_flips=(\d+)", sweep)
    assert [int(r[0]) for r in rows] == [1, 2, 3, 24, 53]
    for _, n, worst, flips in rows:
        assert int(n) > 1_000_000
        assert float(worst) <= 5.0           # tolerance: 5 ulp of the double result (4.5 where u is just below 1)
        assert int(flips) == 0
    assert "log edge: log(1)=0 signbit=0 log(0)=-inf" in sweep
    assert "log edge, rounded: log(1)=0 signbit=0 log(0)=-inf" in sweep


def test_logarithm_rounds_to_the_right_float32_for_every_possible_argument(sweep):
    """A generator's uniform is 0 or a float32 in [2^-53, 1]: 53 binades of 2^23 values and
    1.0 (checked above).  Both normal variants round the logarithm to float32; that rounding
    must be that of the exact logarithm rounded to double (long double carries 11 more bits
    than the double under test) for every one of them."""
    m = re.search(r"log every float32 of \[2\^-53, 1\): n=(\d+) float_flips=(\d+)", sweep)
    assert int(m.group(1)) == 53 << 23 and int(m.group(2)) == 0


def test_float32_cosine_rounds_to_the_right_float32_for_every_possible_argument(sweep):
    """The float32 normal takes the cosine of RN32(RN32(2 pi) * u) in double and rounds it to
    float32: the same yardstick, every u in [2^-53, 1).  Together with the logarithm above
    (and a correctly rounded float32 square root and product) this makes the float32 normals
    the bits of the CPU restatement for every pair of uniforms, not only for the sampled ones."""
    m = re.search(r"cos f32 every float32 of \[2\^-53, 1\): n=(\d+) float_flips=(\d+)", sweep)
    assert int(m.group(1)) == 53 << 23 and int(m.group(2)) == 0


def test_cosine_is_within_one_ulp(sweep):
    rows = re.findall(r"cos variant (f\d+): n=(\d+) worst_ulp=([\d.]+) float_flips=(\d+)", sweep)
    assert [r[0] for r in rows] == ["f64", "f32"]
    for _, n, worst, flips in rows:
        assert int(n) > 2_000_000
        assert float(worst) <= 0.80          # tolerance: 0.8 ulp of the double result
        assert int(flips) == 0
    tiny = re.search(r"cos tiny arguments: worst_ulp=([\d.]+)", sweep)
    assert float(tiny.group(1)) <= 0.5
