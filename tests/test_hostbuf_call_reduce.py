"""_hostbuf.call_reduce: the integer-only passage from Reduce.__call__ to nbh_reduce.
Checked against a small native function compiled here that records its arguments."""

import ctypes
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


# ---- reduce_into: from the array objects to the launch -------------------------------------

class _Arr:
    def __init__(self, rk=None):
        if rk is not None:
            self._rk = rk


class _Stream:
    def __init__(self, handle):
        self._h = handle


class _Ctx:
    def __init__(self, scratch, prepared=True):
        self._scratch, self.prepared = scratch, prepared


class _Tls:
    pass


class _Lib:
    pass


def _setup(fake):
    import numpy as np
    f32 = np.dtype(np.float32)
    lib = _Lib()
    lib._reduce_entry = ctypes.cast(fake.fake_reduce, ctypes.c_void_p).value
    tls = _Tls()
    tls.ctx = _Ctx({0x5151: (0x7F0000003000, 33024, object())})
    codes = {f32: (1, 8)}
    init_cache = {(f32, 0): 0x1234, (f32, 3): 0x5678}
    arr = _Arr((0x7F0000001000, 65536, 4, f32))
    res = _Arr((0x7F0000002000, 1, 4, f32))
    return dict(codes=codes, arr=arr, res=res, stream=_Stream(0x5151), tls=tls, cache=init_cache, lib=lib, f32=f32)


def _go(s, **over):
    a = dict(s, **over)
    return _hostbuf.reduce_into(a["codes"], a["arr"], a["res"], a.get("init", 0), a["stream"], a["tls"], _Stream,
                                a["cache"], a["lib"])


def test_reduce_into_launches_the_plain_case(fake):
    s = _setup(fake)
    assert _go(s) is None
    assert list(fake.fake_seen().contents) == [1, 8, 0x7F0000001000, 65536, 4, 0x1234, 0x7F0000002000,
                                               0x7F0000003000, 33024, 0x5151]
    assert _go(s, init=3) is None
    assert list(fake.fake_seen().contents)[5] == 0x5678
    # a failing launch hands its status back
    s["codes"][s["f32"]] = (99, 8)
    assert _go(s) == 719


def test_reduce_into_declines_everything_else(fake):
    import numpy as np
    s = _setup(fake)
    fake.fake_seen().contents[0] = -1
    declined = [
        dict(arr=_Arr()),                                            # not seen before
        dict(res=_Arr()),
        dict(res=_Arr((0x7F0000002000, 1, 8, np.dtype(np.float64)))),   # another dtype
        dict(arr=_Arr((0x7F0000001000, 0, 4, s["f32"]))),             # empty
        dict(init=0.5), dict(init=7), dict(init=True),               # not a cached int
        dict(stream=0), dict(stream=_Stream(2)), dict(stream=_Stream(0x9999)),   # default, per-thread, no scratch yet
        dict(codes={}),                                              # dtype not paired with the operator yet
    ]
    for over in declined:
        assert _go(s, **over) is NotImplemented, over
    tls = _Tls()
    assert _go(s, tls=tls) is NotImplemented                         # this thread has no context yet
    tls.ctx = _Ctx(s["tls"].ctx._scratch, prepared=False)
    assert _go(s, tls=tls) is NotImplemented
    lib = _Lib()
    assert _go(s, lib=lib) is NotImplemented                         # entry point not looked up yet
    lib._reduce_entry = 0
    assert _go(s, lib=lib) is NotImplemented
    assert fake.fake_seen().contents[0] == -1                        # nothing was launched
    with pytest.raises(TypeError):
        _hostbuf.reduce_into(1, 2, 3)
