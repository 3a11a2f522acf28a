"""_hostbuf.call_reduce: the integer-only passage from Reduce.__call__ to nbh_reduce.
Checked against a small native function compiled here that records its arguments."""

import ctypes
import os
import shutil
import subprocess

import pytest

from numba_cuda_amd import _hostbuf

SOURCE = r"""
#include <stdint.h>
#include <stddef.h>
static long long seen[10];
int fake_reduce(int op, int dtype, const void *in, int64_t n, int64_t stride, const void *init, void *out,
                void *scratch, size_t scratch_bytes, void *stream)
{
    seen[0] = op; seen[1] = dtype; seen[2] = (long long)(intptr_t)in; seen[3] = n; seen[4] = stride;
    seen[5] = (long long)(intptr_t)init; seen[6] = (long long)(intptr_t)out; seen[7] = (long long)(intptr_t)scratch;
    seen[8] = (long long)scratch_bytes; seen[9] = (long long)(intptr_t)stream;
    return op == 99 ? 719 : 0;
}
long long *fake_seen(void) { return seen; }
"""


@pytest.fixture(scope="module")
def fake(tmp_path_factory):
    cc = shutil.which("gcc") or shutil.which("cc")
    if not cc:
        pytest.skip("no C compiler")
    d = tmp_path_factory.mktemp("fake_reduce")
    src = d / "fake.c"
    src.write_text(SOURCE)
    so = d / "libfake.so"
    subprocess.check_call([cc, "-O1", "-shared", "-fPIC", str(src), "-o", str(so)])
    lib = ctypes.CDLL(str(so))
    lib.fake_seen.restype = ctypes.POINTER(ctypes.c_longlong * 10)
    return lib


def test_arguments_arrive_unchanged(fake):
    entry = ctypes.cast(fake.fake_reduce, ctypes.c_void_p).value
    rc = _hostbuf.call_reduce(entry, 3, 8, 0x7F0000001000, 65536, -4, 0x1234, 0x7F0000002000, 0x7F0000003000, 33024,
                              0xABCDEF)
    assert rc == 0
    assert list(fake.fake_seen().contents) == [3, 8, 0x7F0000001000, 65536, -4, 0x1234, 0x7F0000002000,
                                               0x7F0000003000, 33024, 0xABCDEF]
    # None stands for a null pointer (the default stream); a status comes back as is
    assert _hostbuf.call_reduce(entry, 99, 0, 16, 1, 4, 32, 48, 64, 1, None) == 719
    assert list(fake.fake_seen().contents)[9] == 0


def test_bad_calls_raise(fake):
    entry = ctypes.cast(fake.fake_reduce, ctypes.c_void_p).value
    with pytest.raises(TypeError):
        _hostbuf.call_reduce(entry, 0, 0)
    with pytest.raises(ValueError):
        _hostbuf.call_reduce(0, 0, 0, 1, 1, 4, 1, 1, 1, 1, 0)
    with pytest.raises(TypeError):
        _hostbuf.call_reduce(entry, 0, 0, "x", 1, 4, 1, 1, 1, 1, 0)
    with pytest.raises(OverflowError):
        _hostbuf.call_reduce(entry, 0, 0, -5, 1, 4, 1, 1, 1, 1, 0)
