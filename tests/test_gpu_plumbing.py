"""Device-array plumbing on the real library and GPU."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from tests import (attr_cases, cai_cases, dealloc_cases, device_cases, emm_cases, host_stream_cases,
                   memory_cases, ndarray_cases, plumbing_cases, pool_cases, record_cases, slicing_cases)

# plumbing_cases: this package's own; the others restate the reference's suites
CASES = (plumbing_cases.ALL + ndarray_cases.ALL + slicing_cases.ALL + memory_cases.ALL + host_stream_cases.ALL
         + record_cases.ALL + dealloc_cases.ALL + emm_cases.ALL + attr_cases.ALL + device_cases.ALL + cai_cases.ALL
         + pool_cases.ALL)


@pytest.mark.parametrize("case", CASES, ids=lambda f: f.__name__)
def test_plumbing(case):
    print(case.__name__, flush=True)
    case(cuda)


def test_memset_and_views_of_raw_memory():
    d = cuda.device_array(64, np.uint8)
    d.gpu_data.memset(0xAB)
    assert (d.copy_to_host() == 0xAB).all()
    cuda.cudadrv.driver.device_memset(d, 1, 16)
    assert d.copy_to_host().tolist() == [1] * 16 + [0xAB] * 48
    lo, hi = cuda.cudadrv.driver.device_extents(d)
    assert lo <= d.device_ctypes_pointer.value < hi
    assert cuda.cudadrv.driver.device_memory_size(d.gpu_data) == 64


def test_mapped_array_is_device_addressable():
    m = cuda.mapped_array(1000, dtype=np.float32)
    m[:] = np.arange(1000, dtype=np.float32)
    got = cuda.reduce(lambda a, b: a + b)(m)
    assert got == np.arange(1000, dtype=np.float32).sum()


def test_numpy_views_of_managed_and_mapped_arrays_are_device_arguments():
    for make in (cuda.managed_array, cuda.mapped_array):
        m = make((8, 1000), dtype=np.float64)
        m[:] = np.arange(8000.0).reshape(8, 1000)
        row = m[3]                                   # NumPy view: same class, own device range
        assert type(row) is type(m)
        assert row.device_ctypes_pointer.value == m.device_ctypes_pointer.value + 3 * 8000
        assert cuda.reduce(lambda a, b: a + b)(row) == np.arange(3000.0, 4000.0).sum()
        t = cuda.kernels.transpose.transpose(m[:, :500])
        np.testing.assert_array_equal(t.copy_to_host(), np.asarray(m)[:, :500].T)
        cuda.synchronize()


def test_cuda_array_interface_with_torch_tensors():
    """Zero-copy import of a PyTorch-ROCm tensor, checked against torch itself."""
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("torch sees no GPU")
    t = torch.arange(1 << 20, dtype=torch.float32, device="cuda").reshape(1024, 1024)
    torch.cuda.synchronize()
    assert cuda.is_cuda_array(t)
    d = cuda.as_cuda_array(t)
    assert d.shape == (1024, 1024) and d.device_ctypes_pointer.value == t.data_ptr()
    got = cuda.reduce(lambda a, b: a + b)(d.reshape(-1))
    assert got == float(t.sum().item())
    tt = d.T
    back = torch.as_tensor(tt, device="cuda")
    assert torch.equal(back, t.t().contiguous())
    with pytest.raises(TypeError):
        cuda.as_cuda_array(np.zeros(3))


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.complex128])
def test_flat_assignment_at_every_alignment(dtype):
    """dst[a:a+n] = src[b:b+n]: the copy kernel starts its 16-byte packets at the
    destination's first 128-byte line; what lies in front and behind goes item by item."""
    rng = np.random.default_rng(11)
    size = 140000
    src_host = rng.integers(0, 255, size * np.dtype(dtype).itemsize, dtype=np.uint8).view(dtype)
    src = cuda.to_device(src_host)
    for n in (1, 7, 31, 32, 33, 127, 128, 129, 1000, 4099, 100003):
        for d_off, s_off in ((0, 0), (1, 0), (0, 3), (5, 9), (37, 64)):
            want = np.zeros(size, dtype)
            dst = cuda.to_device(want)
            dst[d_off:d_off + n] = src[s_off:s_off + n]
            want[d_off:d_off + n] = src_host[s_off:s_off + n]
            got = dst.copy_to_host()
            assert got.tobytes() == want.tobytes(), (n, d_off, s_off)


@pytest.mark.parametrize("dtype", [np.uint8, np.int16, np.float32, np.float64, np.complex128, np.bool_])
def test_scalar_assignment_at_every_alignment_and_layout(dtype):
    """`d[key] = scalar` passes the item by value: flat ranges from any offset (the
    16-byte pattern must be in phase with the item), strided columns, blocks, 0-d."""
    dt = np.dtype(dtype)
    value = {"b": True, "c": 2.5 - 1.5j}.get(dt.kind, 77)
    rng = np.random.default_rng(15)
    base = rng.integers(0, 2, 5000 * dt.itemsize, dtype=np.uint8).view(dt) if dt.kind != "b" else np.zeros(5000, dt)
    for lo, n in ((0, 5000), (1, 4999), (3, 17), (5, 1), (129, 3000), (7, 4093), (31, 33)):
        want = base.copy()
        d = cuda.to_device(want)
        d[lo:lo + n] = value
        want[lo:lo + n] = value
        assert d.copy_to_host().tobytes() == want.tobytes(), (lo, n)
    m = base[:4800].reshape(60, 80).copy()
    d = cuda.to_device(m)
    for key in ((slice(None), 3), (7, slice(None)), (slice(2, 50, 3), slice(1, 70, 7)), (slice(5, 55), slice(10, 20)),
                (4, 9), slice(None)):
        d[key] = value
        m[key] = value
        assert d.copy_to_host().tobytes() == m.tobytes(), key
    z = cuda.to_device(np.zeros((), dt))
    z[()] = value
    assert z.copy_to_host()[()] == dt.type(value)
    st = cuda.stream()
    d.setitem(slice(None), 0, stream=st)
    st.synchronize()
    assert not d.copy_to_host().any()


def test_large_pageable_copies_go_through_the_staging_ring():
    """Host copies from a few MiB on are pipelined through page-locked buffers by several
    threads, in chunks of a quarter of the copy (1 to 16 MiB): sizes around every threshold
    and chunk size, ragged sizes, odd offsets, fresh destination pages, Python threads at
    once, and the ordering hipMemcpy gives after work on a stream."""
    import threading
    rng = np.random.default_rng(14)
    big = rng.integers(0, 255, (80 << 20) + 12345, dtype=np.uint8)
    for lo, n in ((0, big.size), (1, (32 << 20)), (4097, (48 << 20) + 1), (3, (32 << 20) - 1),
                  (0, (2 << 20) - 1), (5, 2 << 20), (0, (2 << 20) + 1), (7, (4 << 20) + 3), (1, (8 << 20) - 1),
                  (2, 8 << 20), (0, (9 << 20) + 17), (3, (16 << 20) + 1), (0, (64 << 20) + 1), (9, 1 << 20)):
        src = big[lo:lo + n]
        d = cuda.to_device(src)                                  # pageable -> device
        back = d.copy_to_host()                                  # device -> fresh pageable memory
        assert back.tobytes() == src.tobytes(), (lo, n)
        into = np.zeros(n + 10, np.uint8)
        d.copy_to_host(into[5:5 + n])                            # into the middle of an existing array
        assert into[5:5 + n].tobytes() == src.tobytes() and not into[:5].any() and not into[-5:].any()
    # ordering: a kernel on a (blocking) stream, then a synchronous copy without any wait in between
    st = cuda.stream()
    a = cuda.to_device(big[: 64 << 20])
    b = cuda.device_array(64 << 20, np.uint8)
    b.setitem(slice(None), a, stream=st)
    assert b.copy_to_host().tobytes() == big[: 64 << 20].tobytes()
    # on a stream: the legs run on that stream, the call still returns a finished copy
    d = cuda.to_device(big[: 50 << 20], stream=st)
    got = np.empty(50 << 20, np.uint8)
    d.copy_to_host(got, stream=st)
    assert got.tobytes() == big[: 50 << 20].tobytes()
    # two threads copying at the same time
    results = {}

    def worker(key, lo):
        dd = cuda.to_device(big[lo:lo + (40 << 20)])
        results[key] = dd.copy_to_host().tobytes() == big[lo:lo + (40 << 20)].tobytes()

    threads = [threading.Thread(target=worker, args=(k, k * 1000 + 7)) for k in range(3)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert results == {0: True, 1: True, 2: True}


def test_large_device_to_device_copies():
    """copy_to_device between device arrays of a MiB and more runs on the library's own
    copy kernel (smaller ones on hipMemcpy): with and without a stream, at odd offsets."""
    rng = np.random.default_rng(13)
    host = rng.integers(0, 255, (1 << 22) + 77, dtype=np.uint8)
    src = cuda.to_device(host)
    st = cuda.stream()
    for lo, n in ((0, 1 << 22), (3, (1 << 21) + 5), (129, (1 << 20)), (1, (1 << 20) - 1), (0, 100)):
        dst = cuda.device_array(n + 64, np.uint8)
        dst.gpu_data.memset(0)
        dst[16:16 + n].copy_to_device(src[lo:lo + n])
        got = dst.copy_to_host()
        assert got[16:16 + n].tobytes() == host[lo:lo + n].tobytes() and not got[:16].any() and not got[16 + n:].any()
        dst2 = cuda.device_array(n, np.uint8)
        dst2.copy_to_device(src[lo:lo + n], stream=st)
        st.synchronize()
        assert dst2.copy_to_host().tobytes() == host[lo:lo + n].tobytes()
    m = cuda.mapped_array(1 << 21, np.uint8)          # not plain device memory: hipMemcpy's business
    m[:] = host[:1 << 21]
    d = cuda.device_array(1 << 21, np.uint8)
    d.copy_to_device(m)
    assert d.copy_to_host().tobytes() == host[:1 << 21].tobytes()


@pytest.mark.parametrize("dtype", [np.uint8, np.float32, np.complex128])
def test_block_assignment_in_pitched_arrays(dtype):
    """dst[r0:r1, c0:c1] = src[...]: rows are runs of bytes at whatever alignment the
    slice gives them; also rows shorter than a packet, a broadcast row, and 3-D blocks."""
    rng = np.random.default_rng(12)
    item = np.dtype(dtype).itemsize

    def rand(shape):
        return rng.integers(0, 255, int(np.prod(shape)) * item, dtype=np.uint8).view(dtype).reshape(shape)

    src_host = rand((300, 700))
    src = cuda.to_device(src_host)
    for (r0, r1, c0, c1, sr, sc) in ((0, 300, 0, 700, 0, 0), (3, 290, 5, 650, 1, 7), (10, 11, 1, 2, 0, 0),
                                     (0, 300, 699, 700, 0, 3), (7, 207, 33, 36, 50, 100), (1, 256, 16, 528, 2, 32)):
        want = np.zeros((300, 700), dtype)
        dst = cuda.to_device(want)
        h, w = r1 - r0, c1 - c0
        dst[r0:r1, c0:c1] = src[sr:sr + h, sc:sc + w]
        want[r0:r1, c0:c1] = src_host[sr:sr + h, sc:sc + w]
        assert dst.copy_to_host().tobytes() == want.tobytes(), (r0, r1, c0, c1, sr, sc)
    # one row broadcast down a block
    want = np.zeros((300, 700), dtype)
    dst = cuda.to_device(want)
    dst[5:205, 9:409] = src[17, 3:403]
    want[5:205, 9:409] = src_host[17, 3:403]
    assert dst.copy_to_host().tobytes() == want.tobytes()
    # three axes that do not fuse
    cube_host = rand((20, 30, 40))
    cube = cuda.to_device(cube_host)
    want = np.zeros((20, 30, 40), dtype)
    dst = cuda.to_device(want)
    dst[1:19, 2:29, 3:39] = cube[0:18, 1:28, 4:40]
    want[1:19, 2:29, 3:39] = cube_host[0:18, 1:28, 4:40]
    assert dst.copy_to_host().tobytes() == want.tobytes()
    dst[2:4, :, 8:24] = cube[5:7, :, 16:32]
    want[2:4, :, 8:24] = cube_host[5:7, :, 16:32]
    assert dst.copy_to_host().tobytes() == want.tobytes()


def test_setitem_scalars_rows_columns_broadcast():
    """`darr[key] = value` (reference: tests/cudadrv/test_cuda_array_slicing.py:220-379)."""
    a = np.arange(5 * 7, dtype=np.float64).reshape(5, 7)
    d = cuda.to_device(a)
    d[2, 3] = 500
    a[2, 3] = 500
    d[1] = np.arange(7) * 10.0
    a[1] = np.arange(7) * 10.0
    d[:, 2] = 3.5                                   # scalar broadcast over a strided column
    a[:, 2] = 3.5
    d[:, 4] = np.arange(5.0)                        # 1-d into a column
    a[:, 4] = np.arange(5.0)
    d[3:, 5:] = cuda.to_device(np.full((2, 2), -1.0))   # device source
    a[3:, 5:] = -1.0
    d[::2, ::3] = np.array([[9.0], [8.0], [7.0]])   # broadcast along the inner axis
    a[::2, ::3] = np.array([[9.0], [8.0], [7.0]])
    d[4] = 7                                        # int value into a float array
    a[4] = 7
    np.testing.assert_array_equal(d.copy_to_host(), a)
    d[:] = 0.25
    assert (d.copy_to_host() == 0.25).all()
    with pytest.raises(ValueError, match="Can't assign 3-D array to 2-D self"):
        d[:] = np.zeros((1, 5, 7))
    with pytest.raises(ValueError, match="Can't copy sequence with size 3 to array axis 1 with dimension 7"):
        d[:] = np.zeros((5, 3))
    with pytest.raises(IndexError):
        d[5, 0] = 1.0
    # on a stream: asynchronous, same result
    s = cuda.stream()
    d.setitem((slice(None), 0), np.arange(5.0) + 100, stream=s)
    s.synchronize()
    np.testing.assert_array_equal(d.copy_to_host()[:, 0], np.arange(5.0) + 100)
    # other item sizes, many axes, big flat copy
    for dt in (np.int8, np.int16, np.complex128, np.dtype([("i", np.int32), ("j", np.float32, (3, 2))])):
        rng = np.random.default_rng(0)
        dt = np.dtype(dt)
        h = rng.integers(0, 255, 4 * 3 * 5 * 6 * dt.itemsize, dtype=np.uint8).view(dt).reshape(4, 3, 5, 6)
        z = cuda.to_device(np.zeros_like(h))
        z[1:, :, ::2, 1:5] = np.ascontiguousarray(h[1:, :, ::2, 1:5])   # host sources must be contiguous
        with pytest.raises(ValueError, match="non-contiguous buffer"):
            z[1:, :, ::2, 1:5] = h[1:, :, ::2, 1:5]
        want = np.zeros_like(h)
        want[1:, :, ::2, 1:5] = h[1:, :, ::2, 1:5]
        assert z.copy_to_host().tobytes() == want.tobytes()
    big = np.random.default_rng(1).integers(0, 2**31, 3_000_001, dtype=np.int32)
    t = cuda.device_array_like(big)
    t[:] = cuda.to_device(big)
    np.testing.assert_array_equal(t.copy_to_host(), big)
    t[1:] = cuda.to_device(big)[:-1]                 # misaligned flat copy
    np.testing.assert_array_equal(t.copy_to_host()[1:], big[:-1])


def test_stream_callback_and_async_done():
    import asyncio
    import threading
    s = cuda.stream()
    a = cuda.to_device(np.arange(1 << 20, dtype=np.float32), stream=s)
    done = threading.Event()
    seen = []

    def cb(stream, status, arg):
        seen.append((stream is s, status, arg))
        done.set()

    out = cuda.device_array(1, np.float32)
    cuda.reduce(lambda x, y: x + y)(a, res=out, stream=s)
    s.add_callback(cb, "tag")
    assert done.wait(10)
    assert seen == [(True, 0, "tag")]

    async def wait():
        return await s.async_done()

    assert asyncio.run(wait()) is s
    assert abs(float(out[0]) - float(np.arange(1 << 20, dtype=np.float64).sum())) <= 2 * (1 << 20) * 6e-8 * 5.5e11
