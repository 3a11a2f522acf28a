"""The pool's stream bookkeeping (numba_cuda_amd/csrc/pool_core.h) on the host, against
a scripted device: the same header the library compiles, built here with g++."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "numba_cuda_amd", "csrc")


def test_pool_bookkeeping_against_a_scripted_device(tmp_path):
    exe = str(tmp_path / "pool_core_check")
    subprocess.run(["g++", "-O1", "-std=c++17", "-Wall", "-I", CSRC, os.path.join(HERE, "pool_core_check.cpp"),
                    "-o", exe], check=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and "pool core ok" in out.stdout, out.stdout + out.stderr
