"""The launching threads' queue (numba_cuda_amd/csrc/launchq.hip) on the host, under the thread
sanitizer: tests/launchq_check.cpp drives the real source with a stand-in for nbh_reduce."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "numba_cuda_amd", "csrc")


@pytest.fixture(scope="module")
def check(tmp_path_factory):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    exe = str(tmp_path_factory.mktemp("launchq") / "check")
    subprocess.run([hipcc, "-x", "hip", "--offload-arch=gfx950", "-O1", "-g", "-std=c++17", "-w",
                    "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-Xarch_host", "-fsanitize=thread",
                    os.path.join(HERE, "launchq_check.cpp"), os.path.join(CSRC, "launchq.hip"),
                    "-o", exe, "-pthread"], check=True)
    return exe


@pytest.mark.parametrize("bursts", [False, True])
def test_order_counts_and_no_data_race(check, bursts):
    env = dict(os.environ)
    if bursts:
        env["BURSTS"] = "1"
    done = subprocess.run([check], env=env, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stdout[-2000:] + done.stderr[-4000:]
    assert done.stdout.strip().endswith("launches") and "ok" in done.stdout
    assert "ThreadSanitizer" not in done.stderr
