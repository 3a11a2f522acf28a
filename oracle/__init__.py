"""CPU checker for the HIP kernels.  TEST INFRASTRUCTURE ONLY.

Only the test-suite, the smoke check and the benchmark's CPU-baseline leg may
import this package.  The shipped package never does: it fails loudly when its
HIP library is missing instead of falling back to anything in here.

Contents
--------
oracle.c / cref.py   C restatement of the reference algorithms + ctypes access
xoroshiro_py.py      independent big-int restatement of the RNG (second twin)
reduce_simt.py       literal lock-step SIMT emulation of the reference's
                     reduction kernels (pins the association order of oracle.c)
sim.py               the reference's CPU path (its CUDA simulator) restated:
                     the single-core baseline that the benchmark times
"""

from . import cref  # noqa: F401
