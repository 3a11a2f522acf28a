"""Reduce(functor, reference_order=True) / NUMBA_CUDA_REDUCE_REFERENCE_ORDER=1: the HIP path
through nbh_reduce_ordered against the oracle's restatement of the reference's association
order (oracle.cref.tree: kernels/reduction.py:22-166, :194-265 operation for operation, itself
pinned by a literal lock-step emulation of the kernels).  Floating-point results must have the
oracle's BITS: float16 / float32 / float64 / complex sums and products, and the results of
max / min over NaN and signed zeros."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd.core import config
from oracle import cref

FUNCTORS = {"add": lambda a, b: a + b, "mul": lambda a, b: a * b, "max": lambda a, b: max(a, b),
            "min": lambda a, b: min(a, b)}
SIZES = [1, 2, 31, 32, 33, 127, 128, 129, 255, 256, 257, 1000, 4096, 8191, 8192, 8193, 8192 + 128, 20000, 65536,
         100003, 1 << 20, (1 << 22) + 77]


def _say(*what):
    print("reference order:", *what, flush=True)


def _bits(x):
    return np.asarray(x).tobytes()


def _data(rng, dtype, n, op):
    dtype = np.dtype(dtype)
    if dtype.kind == "c":
        a = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dtype)
    else:
        a = rng.standard_normal(n).astype(dtype)
    if op == "mul":                       # keep products in range: factors close to one
        a = (1 + a / 64).astype(dtype)
    return a


@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.float64, np.complex64, np.complex128])
def test_bits_equal_the_reference_order(dtype):
    rng = np.random.default_rng(np.dtype(dtype).itemsize)
    reducers = {op: cuda.Reduce(f, reference_order=True) for op, f in FUNCTORS.items()}
    for n in SIZES:
        for op, red in reducers.items():
            if np.dtype(dtype).kind == "c" and op in ("max", "min"):
                continue
            a = _data(rng, dtype, n, op)
            init = np.dtype(dtype).type(0.5 if op != "mul" else 1.25)
            _say(np.dtype(dtype).name, n, op)
            got = red(cuda.to_device(a), init=init)
            assert got.dtype == a.dtype
            assert _bits(got) == _bits(cref.tree(op, a, init)), (np.dtype(dtype).name, n, op)


def test_own_order_differs_in_bits_but_not_beyond_the_bound():
    """The two orders are different orders: on float32 sums they part in the last bits."""
    a = np.random.default_rng(3).standard_normal(1 << 22).astype(np.float32)
    d = cuda.to_device(a)
    exact = float(np.sum(a.astype(np.float64)))
    ours = cuda.Reduce(FUNCTORS["add"])(d)
    theirs = cuda.Reduce(FUNCTORS["add"], reference_order=True)(d)
    assert _bits(theirs) == _bits(cref.tree("add", a, np.float32(0)))
    bound = 2 * a.size * np.finfo(np.float32).eps * float(np.sum(np.abs(a.astype(np.float64))))
    assert abs(float(ours) - exact) <= bound and abs(float(theirs) - exact) <= bound
    assert abs(float(ours) - float(theirs)) <= bound


def test_nan_and_signed_zeros_as_the_reference_treats_them():
    rng = np.random.default_rng(4)
    for dtype in (np.float32, np.float64):
        for n in (200, 5000, 70001):
            a = rng.standard_normal(n).astype(dtype)
            a[rng.integers(0, n, n // 7)] = 0.0
            a[rng.integers(0, n, n // 7)] = -0.0
            zeros = np.where(a == 0, a, 0).astype(dtype)            # only zeros of both signs
            with_nan = a.copy()
            with_nan[rng.integers(0, n, 3)] = np.nan
            for data in (zeros, with_nan, -np.abs(zeros)):
                for op in ("max", "min", "add"):
                    for init in (dtype(0.0), dtype(-0.0)):
                        _say("special values", np.dtype(dtype).name, n, op, init)
                        got = cuda.Reduce(FUNCTORS[op], reference_order=True)(cuda.to_device(data), init=init)
                        assert _bits(got) == _bits(cref.tree(op, data, init)), (np.dtype(dtype).name, n, op, init)


def test_views_size_res_and_streams():
    a = np.random.default_rng(5).standard_normal(50001).astype(np.float32)
    d = cuda.to_device(a)
    red = cuda.Reduce(FUNCTORS["add"], reference_order=True)
    for name, view in (("a[1:]", lambda x: x[1:]), ("a[3:-5]", lambda x: x[3:-5]), ("a[::3]", lambda x: x[::3]),
                       ("a[::-1]", lambda x: x[::-1]), ("a[7::-2]", lambda x: x[7::-2])):
        _say("view", name)
        want = cref.tree("add", np.ascontiguousarray(view(a)), np.float32(0))
        assert _bits(red(view(d))) == _bits(want), name
    assert _bits(red(d, size=12345, init=2)) == _bits(cref.tree("add", a[:12345], np.float32(2)))
    stream = cuda.stream()
    res = cuda.device_array(3, np.float32)
    assert red(d, res=res[1:], init=7, stream=stream) is None
    stream.synchronize()
    assert _bits(res.copy_to_host()[1]) == _bits(cref.tree("add", a, np.float32(7)))
    assert red(a) == red(d)                                       # a host array is copied in
    assert red(d[:0], init=3) == np.float32(3)                    # empty: `init`


def test_integers_and_booleans_are_the_same_either_way():
    rng = np.random.default_rng(6)
    for dtype in (np.int8, np.uint16, np.int32, np.int64, np.uint64):
        info = np.iinfo(dtype)
        a = rng.integers(info.min, info.max, 100003, dtype=dtype, endpoint=True)
        d = cuda.to_device(a)
        for op in ("add", "mul", "max", "min"):
            assert _bits(cuda.Reduce(FUNCTORS[op], reference_order=True)(d, init=3)) == \
                _bits(cuda.Reduce(FUNCTORS[op])(d, init=3)) == _bits(cref.tree(op, a, dtype(3)))
    b = rng.integers(0, 2, 5000).astype(np.bool_)
    assert cuda.Reduce(lambda x, y: x | y, reference_order=True)(cuda.to_device(b)) == b.any()


def test_environment_switch():
    a = np.random.default_rng(7).standard_normal(300001).astype(np.float32)
    d = cuda.to_device(a)
    want = cref.tree("add", a, np.float32(0))
    before = config.CUDA_REDUCE_REFERENCE_ORDER
    try:
        config.CUDA_REDUCE_REFERENCE_ORDER = 1
        assert _bits(cuda.Reduce(FUNCTORS["add"])(d)) == _bits(want)
        assert _bits(cuda.reduce(FUNCTORS["add"])(d)) == _bits(want)
        config.CUDA_REDUCE_REFERENCE_ORDER = 0
        assert cuda.Reduce(FUNCTORS["add"])._ordered is False
        assert cuda.Reduce(FUNCTORS["add"], reference_order=True)._ordered is True
    finally:
        config.CUDA_REDUCE_REFERENCE_ORDER = before


def test_back_to_back_on_several_streams_share_no_state():
    """Ticket and partial slots are those of the unordered kernel: alternate the two on one
    stream and run others beside them."""
    rng = np.random.default_rng(8)
    rows = [rng.standard_normal(n).astype(np.float32) for n in (8192 * 3 + 5, 70001, 999, 8192 * 40)]
    wants = [cref.tree("add", r, np.float32(1)) for r in rows]
    devs = [cuda.to_device(r) for r in rows]
    streams = [cuda.stream() for _ in range(3)]
    ordered, plain = cuda.Reduce(FUNCTORS["add"], reference_order=True), cuda.Reduce(FUNCTORS["add"])
    out = cuda.device_array(400, np.float32)
    k = 0
    for rep in range(25):
        for i, d in enumerate(devs):
            s = streams[(rep + i) % 3]
            ordered(d, res=out[k:k + 1], init=1, stream=s)
            plain(d, res=out[k + 1:k + 2], init=1, stream=s)
            k += 2
    for s in streams:
        s.synchronize()
    got = out.copy_to_host()[:k]
    for j in range(0, k, 2):
        assert _bits(got[j]) == _bits(wants[(j // 2) % 4]), j


def test_fullsize_float32_and_float64_sums():
    """BASELINE configs[1] inputs: the sums come out with the reference order's bits."""
    rng = np.random.default_rng(1)
    a = rng.standard_normal(2**28, dtype=np.float32)
    _say("2^28 float32")
    got = cuda.Reduce(FUNCTORS["add"], reference_order=True)(cuda.to_device(a))
    assert _bits(got) == _bits(cref.tree("add", a, np.float32(0)))
    del a
    b = rng.standard_normal(2**27)
    _say("2^27 float64")
    got = cuda.Reduce(FUNCTORS["add"], reference_order=True)(cuda.to_device(b))
    assert _bits(got) == _bits(cref.tree("add", b, np.float64(0)))
