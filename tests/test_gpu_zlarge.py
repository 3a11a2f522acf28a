"""Sizes beyond 2^31 items / 2^32 bytes: every index in the kernels must be 64-bit.
(The module name sorts last: these cases move tens of GiB and come after the rest.)"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd.kernels.transpose import transpose


def _say(*a):
    print(*a, flush=True)


def _pattern(n):
    """uint8 pattern with period 251 (prime, so no power-of-two stride aliases it)."""
    reps = -(-n // 251)
    return np.tile(np.arange(251, dtype=np.uint8), reps)[:n]


def test_reduce_over_more_than_2_pow_31_items():
    n = (1 << 31) + 12345
    _say("reduce uint8", n)
    h = _pattern(n)
    d = cuda.to_device(h)
    assert cuda.reduce(lambda a, b: a + b)(d) == h.sum(dtype=np.uint8)
    assert cuda.reduce(lambda a, b: max(a, b))(d, init=0) == 250
    # the very last item decides: only 64-bit indexing reaches it
    h[-1] = 255
    d[n - 1:n] = np.array([255], dtype=np.uint8)
    assert cuda.reduce(lambda a, b: max(a, b))(d, init=0) == 255
    assert cuda.reduce(lambda a, b: a + b)(d) == h.sum(dtype=np.uint8)
    # and a strided view whose byte offsets pass 2^32
    v = d[::3]
    assert cuda.reduce(lambda a, b: a + b)(v) == h[::3].sum(dtype=np.uint8)


def test_flat_and_block_copies_beyond_4_gib():
    n = 70000 * 65536 + 7                          # 4.59e9 > 2^32
    _say("copy uint8", n)
    h = _pattern(n)
    src = cuda.to_device(h)
    dst = cuda.device_array(n, np.uint8)
    dst[:] = src                                   # flat copy kernel
    tail = dst[n - 4096:].copy_to_host()
    assert tail.tobytes() == h[n - 4096:].tobytes()
    assert cuda.reduce(lambda a, b: a + b)(dst) == h.sum(dtype=np.uint8)
    dst2 = cuda.device_array(n, np.uint8)
    dst2.copy_to_device(src)                       # device-to-device path
    assert dst2[n - 4096:].copy_to_host().tobytes() == h[n - 4096:].tobytes()
    assert cuda.reduce(lambda a, b: a + b)(dst2) == h.sum(dtype=np.uint8)
    # pitched block: 70000 rows of 61000 bytes out of 65536-byte rows (4.3 GiB spanned)
    rows, pitch, width = 70000, 65536, 61000
    big_src = src[:rows * pitch].reshape(rows, pitch)
    big_dst = cuda.device_array((rows, pitch), np.uint8)
    big_dst[:, 100:100 + width] = big_src[:, 300:300 + width]
    hv = h[:rows * pitch].reshape(rows, pitch)
    for r in (0, 1, 32767, 32768, 65535, 65536, rows - 1):
        got = big_dst[r, 100:100 + width].copy_to_host()
        assert got.tobytes() == hv[r, 300:300 + width].tobytes(), r


def test_transpose_of_more_than_2_pow_32_bytes():
    rows, cols = 70001, 61003                      # 4.27e9 one-byte items, nothing aligned
    _say("transpose uint8", rows, cols)
    h = _pattern(rows * cols).reshape(rows, cols)
    d = cuda.to_device(h)
    t = transpose(d)
    assert t.shape == (cols, rows)
    for c in (0, 1, 4095, 32768, cols - 2, cols - 1):
        got = t[c].copy_to_host()
        assert got.tobytes() == h[:, c].tobytes(), c
    del t
    # two-byte items through the line-aligned kernel (output rows are off the line grid)
    rows2, cols2 = 46001, 46507                    # 4.28e9 bytes
    h2 = _pattern(rows2 * cols2 * 2).view(np.uint16).reshape(rows2, cols2)
    t2 = transpose(cuda.to_device(h2))
    for c in (0, 1, 777, cols2 - 1):
        assert t2[c].copy_to_host().tobytes() == h2[:, c].tobytes(), c
