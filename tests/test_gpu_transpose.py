"""Parity of transpose (HIP path) with the oracle / numpy: bit-exact."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd.kernels.transpose import transpose
from oracle import cref

recordwith2darray = np.dtype([("i", np.int32), ("j", np.float32, (3, 2))])


def _say(*a):
    print(*a, flush=True)


def _same_bytes(a, b):
    return a.shape == b.shape and np.ascontiguousarray(a).tobytes() == np.ascontiguousarray(b).tobytes()


@pytest.mark.parametrize("rows,cols,dtype", [(5, 6, np.float64), (128, 128, np.complex128),
                                             (1025, 512, np.float64)])
def test_transpose_reference_variants(rows, cols, dtype):
    # numba_cuda/numba/cuda/tests/cudapy/test_transpose.py:17-32
    x = np.arange(rows * cols, dtype=dtype).reshape(cols, rows)
    y = np.zeros(rows * cols, dtype=dtype).reshape(rows, cols)
    dx = cuda.to_device(x)
    dy = cuda.cudadrv.devicearray.from_array_like(y)
    assert transpose(dx, dy) is dy
    dy.copy_to_host(y)
    np.testing.assert_array_equal(x.transpose(), y)
    np.testing.assert_array_equal(cref.transpose(x), y)


SMALL = [(2, 3), (16, 16), (16, 17), (17, 16), (14, 15), (15, 14), (14, 14)]


@pytest.mark.parametrize("rows,cols", SMALL)
def test_transpose_record_and_bool(rows, cols):
    arr = np.zeros((rows, cols), dtype=recordwith2darray)
    for x in range(rows):
        for y in range(cols):
            arr[x, y]["i"] = x ** 2 + y
            arr[x, y]["j"] = np.arange(6, dtype=np.float32).reshape(3, 2) * x + y
    d_t = cuda.device_array_like(arr.T)
    transpose(cuda.to_device(arr), d_t)
    np.testing.assert_array_equal(arr.T, d_t.copy_to_host())
    b = np.random.default_rng(rows * 31 + cols).integers(0, 2, (rows, cols)).astype(np.bool_)
    d_b = cuda.device_array_like(b.T)
    transpose(cuda.to_device(b), d_b)
    np.testing.assert_array_equal(b.T, d_b.copy_to_host())


def test_transpose_view():
    # test_transpose.py:73-86
    a = np.arange(120, dtype=np.int64).reshape((10, 12))
    d_a = cuda.to_device(a)
    d_t = d_a[::2, ::2].T
    assert d_t.shape == (6, 5)
    assert d_t.strides == (40, 8)
    np.testing.assert_array_equal(a[::2, ::2].T, d_t.copy_to_host())
    # negative and mixed strides, F order
    np.testing.assert_array_equal(a[::-1, ::3].T, d_a[::-1, ::3].T.copy_to_host())
    np.testing.assert_array_equal(a[1:, 2:].T, d_a[1:, 2:].T.copy_to_host())
    f = np.asfortranarray(a)
    np.testing.assert_array_equal(f.T, cuda.to_device(f).T.copy_to_host())


def test_T_and_transpose_api():
    a = np.arange(12, dtype=np.float32).reshape(3, 4)
    d = cuda.to_device(a)
    assert d.transpose((0, 1)) is d
    with pytest.raises(ValueError, match="invalid axes list"):
        d.transpose((0, 2))
    with pytest.raises(NotImplementedError, match="non-2D"):
        cuda.to_device(np.zeros(4)).T
    np.testing.assert_array_equal(d.transpose((1, 0)).copy_to_host(), a.T)
    # host arrays are accepted on both sides
    out = np.zeros((4, 3), np.float32)
    with pytest.warns(cuda.NumbaPerformanceWarning):
        assert transpose(a, out) is out
    np.testing.assert_array_equal(out, a.T)
    with pytest.raises(ValueError, match="incompatible shape"):
        transpose(d, cuda.device_array((3, 4), np.float32))
    # empty
    e = cuda.to_device(np.zeros((0, 5), np.float32)).T
    assert e.shape == (5, 0)


@pytest.mark.parametrize("dtype", [np.int8, np.uint16, np.float32, np.int64, np.complex128,
                                   np.dtype("S3"), np.dtype("S12"), recordwith2darray])
@pytest.mark.parametrize("shape", [(1, 1), (1, 300), (300, 1), (64, 64), (65, 63), (127, 129),
                                   (257, 515), (1000, 777), (2049, 33), (7001, 131)])
def test_every_item_size_and_ragged_shapes(shape, dtype):
    dtype = np.dtype(dtype)
    _say("transpose", shape, dtype)
    rng = np.random.default_rng(shape[0] * 7919 + shape[1])
    a = rng.integers(0, 256, shape[0] * shape[1] * dtype.itemsize, dtype=np.uint8).view(dtype).reshape(shape)
    got = cuda.to_device(a).T.copy_to_host()
    assert _same_bytes(got, a.T)
    assert _same_bytes(got, cref.transpose(a))


@pytest.mark.parametrize("itemsize", [3, 5, 6, 12, 20, 24, 28, 33, 100, 128, 200, 512, 520])
def test_record_items_of_any_size(itemsize):
    """Tile edge, chunk width and fallback all depend on the item size: below 33 bytes,
    below 129, below 513, above."""
    dtype = np.dtype("V%d" % itemsize)
    for shape in ((70, 45), (1, 130), (257, 3)):
        _say("transpose records", itemsize, shape)
        raw = np.random.default_rng(itemsize).integers(0, 256, shape[0] * shape[1] * itemsize, dtype=np.uint8)
        a = raw.view(dtype).reshape(shape)
        got = cuda.to_device(a).T.copy_to_host()
        assert got.shape == (shape[1], shape[0])
        assert _same_bytes(got, np.ascontiguousarray(a.T))


def test_sixteen_byte_items_that_are_only_eight_byte_aligned():
    a = (np.arange(90 * 64) + 1j * np.arange(90 * 64)[::-1]).reshape(90, 64)
    flat = cuda.to_device(np.zeros(90 * 64 * 2 + 1))
    src = flat[1:].view(np.complex128).reshape(90, 64)       # base address = 8 mod 16
    src.copy_to_device(a)
    assert src.device_ctypes_pointer.value % 16 == 8
    np.testing.assert_array_equal(transpose(src).copy_to_host(), a.T)


def test_row_padded_inputs_and_outputs():
    """Rows longer than the logical width on both sides (pitched allocations)."""
    rng = np.random.default_rng(9)
    big = rng.integers(0, 2**31, (300, 520), dtype=np.int32)
    d_big = cuda.to_device(big)
    src = d_big[:, 3:500]                       # row stride 520*4, misaligned start
    dst_full = cuda.to_device(np.zeros((497, 333), np.int32))
    dst = dst_full[:, 7:307]
    transpose(src, dst)
    want = np.zeros((497, 333), np.int32)
    want[:, 7:307] = big[:, 3:500].T
    np.testing.assert_array_equal(dst_full.copy_to_host(), want)


@pytest.mark.parametrize("dtype", [np.int16, np.uint32, np.float64, np.complex128])
@pytest.mark.parametrize("shape", [(1237, 1093), (3001, 2777)])
def test_ragged_views_with_interior_and_edge_tiles(shape, dtype):
    """Both sides off the 128-byte grid (pitched rows, item-aligned bases): large enough that
    the ring kernel runs tiles wholly inside the matrix as well as every kind of edge tile."""
    dtype = np.dtype(dtype)
    rows, cols = shape
    _say("transpose ragged views", shape, dtype)
    rng = np.random.default_rng(rows + cols + dtype.itemsize)
    big = rng.integers(0, 256, (rows, (cols + 3) * dtype.itemsize), dtype=np.uint8).view(dtype)
    src = cuda.to_device(big)[:, 1:1 + cols]
    dst_full = cuda.to_device(np.full((cols, rows + 5), 0, dtype=np.uint8).astype(dtype))
    dst = dst_full[:, 2:2 + rows]
    transpose(src, dst)
    want = np.zeros((cols, rows + 5), dtype)
    want[:, 2:2 + rows] = big[:, 1:1 + cols].T
    assert _same_bytes(dst_full.copy_to_host(), want)


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_pitches_and_offsets(seed):
    """Shapes, row pitches and base offsets drawn at random, every packet size: tiles inside
    the matrix, on every edge, and the empty workgroups of a padded grid all occur."""
    rng = np.random.default_rng(1000 + seed)
    for case in range(14):
        itemsize = int(rng.choice([1, 2, 4, 8, 16]))
        dtype = np.dtype({1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64, 16: np.complex128}[itemsize])
        rows = int(rng.integers(1, 2600))
        cols = int(rng.integers(1, 2600))
        pad_in, pad_out = int(rng.integers(0, 40)), int(rng.integers(0, 40))
        off_in, off_out = int(rng.integers(0, pad_in + 1)), int(rng.integers(0, pad_out + 1))
        _say("transpose random", seed, case, dtype, (rows, cols), (pad_in, off_in), (pad_out, off_out))
        big = rng.integers(0, 256, (rows, (cols + pad_in) * itemsize), dtype=np.uint8).view(dtype)
        src = cuda.to_device(big)[:, off_in:off_in + cols]
        dst_full = cuda.to_device(np.zeros((cols, rows + pad_out), dtype))
        dst = dst_full[:, off_out:off_out + rows]
        transpose(src, dst)
        want = np.zeros((cols, rows + pad_out), dtype)
        want[:, off_out:off_out + rows] = big[:, off_in:off_in + cols].T
        assert _same_bytes(dst_full.copy_to_host(), want), (dtype, rows, cols, pad_in, off_in, pad_out, off_out)


@pytest.mark.parametrize("dtype,rows,cols", [(np.int16, 16384, 256), (np.int16, 16384, 1100), (np.uint16, 16384, 4096),
                                             (np.float32, 8192, 128), (np.float32, 8192, 2048), (np.uint32, 8192, 8192),
                                             (np.float64, 4096, 64), (np.float64, 4096, 1000), (np.int64, 4096, 4096)])
def test_output_rows_32_kib_apart(dtype, rows, cols):
    """Output rows exactly 32 KiB apart: with input rows a power of two of at most that the
    workgroups take the tiles in diagonal order (several column bands, one band, bands whose
    number does not divide the rows' tiles), otherwise in the plain one."""
    dtype = np.dtype(dtype)
    _say("transpose 32 KiB output pitch", dtype, rows, cols)
    rng = np.random.default_rng(rows + cols)
    a = rng.integers(0, 256, (rows, cols * dtype.itemsize), dtype=np.uint8).view(dtype)
    got = transpose(cuda.to_device(a)).copy_to_host()
    assert _same_bytes(got, a.T)


# ---- full-size matrices, seed 2 --------- ------------------------------------------------

def test_fullsize_float32_16384_square():
    a = np.random.default_rng(2).random((16384, 16384), dtype=np.float32)
    d = cuda.to_device(a)
    t = d.T
    got = t.copy_to_host()
    assert _same_bytes(got, a.T)
    back = t.T.copy_to_host()           # involution on the device
    assert _same_bytes(back, a)


def test_fullsize_int16_16384_square_in_diagonal_order():
    """Both pitches 32 KiB: the workgroups take the tiles in diagonal order."""
    a = np.random.default_rng(3).integers(-32768, 32767, (16384, 16384), dtype=np.int16, endpoint=True)
    got = cuda.to_device(a).T.copy_to_host()
    assert _same_bytes(got, a.T)


def test_fullsize_float64_ragged_12345_by_6789():
    a = np.random.default_rng(2).random((12345, 6789))
    got = cuda.to_device(a).T.copy_to_host()
    assert got.shape == (6789, 12345)
    assert _same_bytes(got, a.T)


def test_fullsize_int16_8192_by_32768():
    a = np.random.default_rng(2).integers(-32768, 32767, (8192, 32768), dtype=np.int16, endpoint=True)
    got = cuda.to_device(a).T.copy_to_host()
    assert _same_bytes(got, a.T)
