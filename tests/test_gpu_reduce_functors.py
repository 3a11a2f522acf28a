"""Reduce with functors that are translated and compiled at run time (HIP path through
nbh_reduce_compile / nbh_reduce_custom), against the oracle.

Oracle: oracle.cref.functor_tree - the functor itself, typed as the reference's JIT types
it, applied in the association order of the reference's kernels - for sizes it finishes
in seconds; closed forms at 2^24 elements.  Every functor here is associative and
commutative on its operands, so the order of association cannot change an integer or
boolean result: those are compared bit for bit.  Floats: `largest_magnitude` selects an
element (bit for bit); sums and the hypot and log-sum-exp folds accumulate a rounding (and
a library call) per application in an order that differs from the oracle's: tolerance
4 n eps, relative to the sum of magnitudes for sums and to the result otherwise (written
at the assertion).
"""

import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from numba_cuda_amd.kernels import reduction
from oracle import cref
from tests import functor_cases as FC

FOLDS = [c for c in FC.CASES if c.fold]
SIZES = [1, 2, 63, 64, 65, 255, 256, 257, 1023, 4099, 70001]


def _say(*a):
    print(*a, flush=True)


def _check(case, dtype, got, want, n, data):
    dtype = np.dtype(dtype)
    assert isinstance(got, dtype.type), (case, dtype, type(got))
    if dtype.kind not in "fc" or case.selects:
        assert got.tobytes() == want.tobytes(), (case, dtype, n, got, want)
    else:
        # sums: against the sum of magnitudes; the other folds: against the result
        eps = np.finfo(dtype).eps
        wide = np.complex128 if dtype.kind == "c" else np.float64
        sums = case.name in ("sum_plus_one", "complex_sum_plus_i")
        scale = float(np.abs(data.astype(wide)).sum()) + n if sums else abs(wide(want))
        assert abs(wide(got) - wide(want)) <= 4 * max(n, 8) * eps * scale, (case, dtype, n, got, want)


@pytest.mark.parametrize("case", FOLDS, ids=repr)
def test_folds_against_the_reference_order(case):
    red = cuda.Reduce(case.functor)
    for dtype in case.dtypes:
        for n in SIZES:
            _say(case, dtype, n)
            data = case.operands(dtype, n, n)
            want = cref.functor_tree(case.functor, data, case.init)
            _check(case, dtype, red(data, init=case.init), want, n, data)


def _wrap(value, dtype):
    info = np.iinfo(dtype)
    bits = 8 * np.dtype(dtype).itemsize
    value &= (1 << bits) - 1
    if info.min < 0 and value >= 1 << (bits - 1):
        value -= 1 << bits
    return np.dtype(dtype).type(value)


def test_closed_forms_at_2p24():
    n = 1 << 24
    rng = np.random.default_rng(24)
    for dtype in (np.int32, np.uint16, np.int64, np.uint64):
        info = np.iinfo(dtype)
        data = rng.integers(info.min, info.max, n, dtype=dtype, endpoint=True)
        d = cuda.to_device(data)
        _say("sum_plus_one", np.dtype(dtype))
        got = cuda.Reduce(FC.BY_NAME["sum_plus_one"].functor)(d, init=7)
        total = int(np.sum(data.astype(np.uint64), dtype=np.uint64))       # modulo 2^64
        assert got == _wrap(total + 7 + n, dtype)
        _say("xor_and_flip", np.dtype(dtype))
        got = cuda.Reduce(FC.BY_NAME["xor_and_flip"].functor)(d, init=5)
        assert got == _wrap(int(np.bitwise_xor.reduce(data)) ^ 5 ^ (n & 1), dtype)
        _say("one_plus_products", np.dtype(dtype))
        got = cuda.Reduce(FC.BY_NAME["one_plus_products"].functor)(d, init=2)
        prod = int(np.multiply.reduce(data.astype(np.uint64) + np.uint64(1), dtype=np.uint64))       # wraps modulo 2^64
        assert got == _wrap(prod * 3 - 1, dtype)
    # saturation and the modulus
    small = rng.integers(0, 40, n, dtype=np.int32)
    assert cuda.Reduce(FC.BY_NAME["saturating_sum"].functor)(small, init=3) == 1000
    assert cuda.Reduce(FC.BY_NAME["saturating_sum"].functor)(small[:20], init=3) == min(1000, int(small[:20].sum()) + 3)
    residues = rng.integers(0, 1000003, n, dtype=np.int64)
    assert cuda.Reduce(FC.BY_NAME["sum_modulo_prime"].functor)(residues, init=11) == (int(residues.sum()) + 11) % 1000003
    # floats
    for dtype, tol in ((np.float32, 1e-4), (np.float64, 1e-11)):
        x = (rng.standard_normal(n) * 100).astype(dtype)
        d = cuda.to_device(x)
        got = cuda.Reduce(FC.BY_NAME["largest_magnitude"].functor)(d, init=0)
        assert abs(got) == np.abs(x).max() and got in x and isinstance(got, dtype)
        got = cuda.Reduce(FC.BY_NAME["hypot_math"].functor)(d, init=0)
        want = np.sqrt(np.sum(x.astype(np.float64) ** 2))
        assert abs(got - want) <= tol * want, (dtype, got, want)      # tolerance: 1e-4 / 1e-11 relative at 2^24
    flags = rng.integers(0, 2, n).astype(np.bool_)
    got = cuda.Reduce(FC.BY_NAME["different"].functor)(flags, init=False)
    assert got == bool(flags.sum() & 1) and isinstance(got, np.bool_)


@pytest.mark.parametrize("dtype,items,skip", [(np.int32, 40_000_001, 3), (np.uint16, 80_000_003, 1),
                                              (np.int64, 20_000_003, 1), (np.uint8, 150_000_011, 5)])
def test_closed_forms_on_large_inputs_of_awkward_length_and_start(dtype, items, skip):
    """From 128 MiB on the translated kernel reads 16 KiB pieces dealt out to the workgroups:
    lengths that leave part of a piece and of a packet over, starts off a 16-byte boundary."""
    rng = np.random.default_rng(items)
    info = np.iinfo(dtype)
    data = rng.integers(info.min, info.max, items, dtype=dtype, endpoint=True)
    d = cuda.to_device(data)[skip:]
    ref = data[skip:]
    assert d.nbytes >= 128 << 20
    _say("large sum_plus_one", np.dtype(dtype), items, skip)
    got = cuda.Reduce(FC.BY_NAME["sum_plus_one"].functor)(d, init=7)
    total = int(np.sum(ref.astype(np.uint64), dtype=np.uint64))       # modulo 2^64
    assert got == _wrap(total + 7 + ref.size, dtype)
    got = cuda.Reduce(FC.BY_NAME["xor_and_flip"].functor)(d, init=5)
    assert got == _wrap(int(np.bitwise_xor.reduce(ref)) ^ 5 ^ (ref.size & 1), dtype)


def test_float16_and_booleans():
    rng = np.random.default_rng(16)
    x = (rng.standard_normal(5000) * 100).astype(np.float16)
    x[1234] = np.float16(-60000)
    got = cuda.Reduce(FC.BY_NAME["largest_magnitude"].functor)(x)
    assert got == np.float16(-60000) and isinstance(got, np.float16)
    for name in ("different", "both_or_neither", "sum_plus_one"):
        case = FC.BY_NAME[name]
        for n in (1, 7, 1000, 4097):
            flags = case.operands("bool", n, n)
            want = cref.functor_tree(case.functor, flags, case.init)
            got = cuda.Reduce(case.functor)(flags, init=case.init)
            assert got == want and isinstance(got, np.bool_), (name, n)


def test_views_res_streams_and_size():
    case = FC.BY_NAME["sum_plus_one"]
    red = cuda.Reduce(case.functor)
    rng = np.random.default_rng(3)
    base = rng.integers(-1000, 1000, 100003).astype(np.int32)
    d = cuda.to_device(base)

    def expect(view, init=0):
        return np.int32(int(view.astype(np.int64).sum()) + init + view.size)
    assert red(d) == expect(base)
    assert red(d, size=1000, init=5) == expect(base[:1000], 5)
    for view_of in (lambda a: a[1:], lambda a: a[3:-5], lambda a: a[::3], lambda a: a[::-1], lambda a: a[7::-2],
                    lambda a: a[4:4 + 4096]):
        _say("view", view_of(base).shape, view_of(base).strides)
        assert red(view_of(d)) == expect(view_of(base))
    # result into device memory, on a stream, nothing comes back until asked
    stream = cuda.stream()
    res = cuda.device_array(3, np.int32)
    res.copy_to_device(np.array([-1, -2, -3], np.int32))
    assert red(d, res=res[1:], init=2, stream=stream) is None
    stream.synchronize()
    assert list(res.copy_to_host()) == [-1, expect(base, 2), -3]
    with pytest.raises(TypeError, match="dtype"):
        red(d, res=cuda.device_array(1, np.int64))
    with pytest.raises(TypeError, match="1D"):
        red(np.zeros((2, 2), np.int32))
    # empty input: init, converted, the device is not asked
    assert red(np.zeros(0, np.int16), init=9) == 9
    # init takes part exactly once
    assert red(np.array([5], np.int32), init=100) == 106
    assert red(np.array([5, 6], np.int32), init=100) == 113


def test_compiled_once_per_functor_and_type():
    def functor(a, b):
        return a + b + 2
    before = len(reduction._COMPILED)
    red = cuda.Reduce(functor)
    assert red(np.arange(10, dtype=np.int32)) == 45 + 20
    assert len(reduction._COMPILED) == before + 1
    assert cuda.Reduce(functor)(np.arange(10, dtype=np.int32), init=1) == 45 + 21       # same functor: cached
    assert len(reduction._COMPILED) == before + 1
    assert red(np.arange(10, dtype=np.float64)) == 65.0                                  # another type: another build
    assert len(reduction._COMPILED) == before + 2
    # an equal body from another functor object shares the build
    assert cuda.Reduce(lambda x, y: x + y + 2)(np.arange(4, dtype=np.int32)) == 6 + 8
    assert len(reduction._COMPILED) == before + 2
    # the decorator form of the reference
    @cuda.reduce
    def plus_three(a, b):
        return a + b + 3
    assert plus_three(np.arange(4, dtype=np.int64)) == 6 + 12


def test_interleaved_with_the_kernels_of_the_standard_operators():
    """Both kinds of calls share one scratch buffer per stream; the translated kernels
    must leave the ticket of the single-launch kernels alone."""
    rng = np.random.default_rng(8)
    data = rng.integers(-100, 100, 1 << 20).astype(np.int64)
    d = cuda.to_device(data)
    plain = cuda.Reduce(lambda a, b: a + b)
    custom = cuda.Reduce(lambda a, b: a + b + 1)
    total = int(data.sum())
    for _ in range(5):
        assert plain(d) == total
        assert custom(d) == total + data.size
        assert plain(d, init=3) == total + 3


def test_threads_on_their_own_streams():
    case = FC.BY_NAME["xor_and_flip"]
    red = cuda.Reduce(case.functor)
    rng = np.random.default_rng(12)
    arrays = [rng.integers(0, 2**31, 200000 + 1000 * k).astype(np.int32) for k in range(4)]
    wants = [np.int32(int(np.bitwise_xor.reduce(a)) ^ (a.size & 1)) for a in arrays]
    errors = []

    def work(k):
        try:
            cuda.select_device(0)
            d = cuda.to_device(arrays[k])
            s = cuda.stream()
            for _ in range(20):
                got = red(d, stream=s)
                if got != wants[k]:
                    errors.append((k, got, wants[k]))
        except Exception as e:      # pragma: no cover
            errors.append((k, repr(e)))
    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    [t.start() for t in threads]
    [t.join() for t in threads]
    assert not errors, errors[:3]


def test_untranslatable_functor_is_refused_when_the_object_is_made():
    with pytest.raises(NotImplementedError, match="could not translate"):
        cuda.Reduce(lambda a, b: int(a) + b)
    with pytest.raises(TypeError, match="bitwise"):
        cuda.Reduce(FC.BY_NAME["xor_and_flip"].functor)(np.zeros(4, np.float32))
    with pytest.raises(TypeError, match="not supported"):          # complex numbers are not ordered
        cuda.Reduce(FC.BY_NAME["saturating_sum"].functor)(np.zeros(4, np.complex64))
    with pytest.raises(TypeError, match="cannot convert complex"):  # a complex result for real elements
        cuda.Reduce(lambda a, b: a + b * 1j)(np.zeros(4, np.float64))


def test_max_min_spelled_with_other_comparisons_keep_their_own_nan_rule():
    """`a if a >= b else b` and its relatives are max / min for integers (native kernels) but drop
    or keep NaN differently from `max(a, b)`: on floating point they run as translated functors,
    whose comparison is the functor's own.  With NaN among the operands these functors are not
    associative, so only inputs of one or two items have an answer that does not depend on the
    order of association: those are compared with the functor applied as the reference applies
    it (oracle.cref.functor_tree), NaN for NaN; NaN-free inputs of every size bit for bit."""
    spellings = [lambda a, b: a if a >= b else b, lambda a, b: a if a > b else b,
                 lambda a, b: b if b >= a else a, lambda a, b: a if a < b else b, lambda a, b: a if a <= b else b]
    rng = np.random.default_rng(77)
    nan = np.float32(np.nan)
    for k, functor in enumerate(spellings):
        red = cuda.Reduce(functor)
        assert not red._kernel_form
        for data in ([nan], [1.0], [nan, 2.0], [2.0, nan], [nan, nan], [0.0, -0.0], [-0.0, 0.0]):
            for init in (0.25, nan, -0.0):
                data32 = np.array(data, np.float32)
                _say("spelling", k, data, init)
                want = cref.functor_tree(functor, data32, init)
                got = red(data32, init=init)
                assert got.tobytes() == want.tobytes() or (np.isnan(got) and np.isnan(want)), (k, data, init, got, want)
        for n in (65, 1000, 70001):
            clean = rng.standard_normal(n).astype(np.float32)
            assert red(clean, init=0.25).tobytes() == cref.functor_tree(functor, clean, 0.25).tobytes()
        # integers: the native kernels, exact
        ints = rng.integers(-1000, 1000, 5000).astype(np.int32)
        assert red(ints, init=0) == cref.functor_tree(functor, ints, 0)


# ---- translated functors in the reference's order of association ---------------------------
# With reference_order=True every application is made on the same pair of values as in a run
# of the reference's kernels, so the comparison with oracle.cref.functor_tree is bit for bit
# also for functors that are NOT associative (a - b, a / 2 + b / 4 ...) and for floating-point
# roundings that depend on the order.  float32 only with functors whose constants (if any) do
# not change the precision of a step: a Python number in the functor makes the JIT compute
# that step in float64 where NumPy scalars, which the oracle runs on, stay in float32
# (`a + b + 1` is safe: rounding the exact float64 sum once more to float32 gives the float32 sum).
FLOAT32_SAFE = ("sum_plus_one", "difference", "abs_difference_statement", "spread", "nested_conditions",
                "largest_magnitude", "nan_aware")
ORDER_SIZES = [1, 2, 31, 32, 33, 127, 128, 129, 255, 256, 1000, 4099, 8191, 8192, 8192 * 2 + 128 * 5 + 3, 30011]


def _ordered_cases():
    for case in FC.CASES:
        if not case.exact:
            continue
        ints = [d for d in case.dtypes if np.dtype(d).kind in "iu"]
        chosen = ints[:1] + ints[-1:] if len(ints) > 1 else ints
        if "float64" in case.dtypes:
            chosen.append("float64")
        if "float32" in case.dtypes and case.name in FLOAT32_SAFE:
            chosen.append("float32")
        if "bool" in case.dtypes:
            chosen.append("bool")
        chosen += [d for d in case.dtypes if d.startswith("complex")]
        for dtype in chosen:
            yield pytest.param(case, dtype, id="%s-%s" % (case.name, dtype))


def _same_bits(got, want):
    return got.tobytes() == want.tobytes() or (got != got and want != want)


@pytest.mark.parametrize("case,dtype", list(_ordered_cases()))
def test_translated_functors_in_the_reference_order(case, dtype):
    red = cuda.Reduce(case.functor, reference_order=True)
    for n in ORDER_SIZES:
        _say("ordered", case, dtype, n)
        data = case.operands(dtype, n, n + 1)
        want = cref.functor_tree(case.functor, data, case.init)
        got = red(data, init=case.init)
        assert isinstance(got, np.dtype(dtype).type)
        assert _same_bits(got, want), (case, dtype, n, got, want)


@pytest.mark.parametrize("name,dtype,n", [("difference", "float32", 8192 * 300 + 12345),
                                          ("difference", "int16", 8192 * 261 + 77),
                                          ("sum_plus_one", "float64", 8192 * 150 + 128 * 37),
                                          ("halves", "float64", 128 * 40 * 70 + 5)])
def test_reference_order_over_many_batches_of_rows(name, dtype, n):
    """Chains longer than the rows a workgroup parks at a time (128 rows of 1 - 4 byte items, 64
    of 8-byte ones), grids below the reference's 64 blocks, views and `res=`."""
    case = FC.BY_NAME[name]
    _say("ordered, long", name, dtype, n)
    data = case.operands(dtype, n, 5)
    want = cref.functor_tree(case.functor, data, 3)
    red = cuda.Reduce(case.functor, reference_order=True)
    d = cuda.to_device(data)
    assert _same_bits(red(d, init=3), want)
    res = cuda.device_array(2, dtype)
    s = cuda.stream()
    assert red(d, res=res[1:], init=3, stream=s) is None
    s.synchronize()
    assert _same_bits(res.copy_to_host()[1], want)
    every_third = data[::3]
    assert _same_bits(red(d[::3], init=3), cref.functor_tree(case.functor, every_third, 3))
    backwards = data[100000:50:-1]
    assert _same_bits(red(d[100000:50:-1], init=3), cref.functor_tree(case.functor, backwards, 3))


def test_reference_order_interleaves_with_the_other_kernels_on_one_scratch_buffer():
    rng = np.random.default_rng(9)
    data = rng.standard_normal(200003).astype(np.float32)
    d = cuda.to_device(data)
    minus = lambda a, b: a - b
    ordered = cuda.Reduce(minus, reference_order=True)
    plain = cuda.Reduce(lambda a, b: a + b + 1)
    native = cuda.Reduce(lambda a, b: a + b, reference_order=True)
    want_minus = cref.functor_tree(minus, data, 0.5)
    want_native = cref.tree("add", data, 0.5)
    ints = cuda.to_device(np.arange(100000, dtype=np.int64))
    for _ in range(4):
        assert _same_bits(ordered(d, init=0.5), want_minus)
        assert plain(ints) == 99999 * 100000 // 2 + 100000
        assert _same_bits(native(d, init=0.5), np.float32(want_native))


@pytest.mark.parametrize("name", ["modulus", "complex_quotient_narrow"])
def test_complex_functors_that_call_the_library_or_divide_in_float32(name):
    """abs() is hypot from the device library, and NumPy, which the oracle runs complex64 on,
    divides by another algorithm than the JIT: a unit or two in the last place per
    application.  Reference order, compared part by part within 16 n eps of the larger part."""
    case = FC.BY_NAME[name]
    red = cuda.Reduce(case.functor, reference_order=True)
    for dtype in case.dtypes:
        eps = np.finfo(dtype).eps
        for n in (1, 2, 33, 128, 1000, 4099):
            _say(name, dtype, n)
            data = case.operands(dtype, n, n)
            want = cref.functor_tree(case.functor, data, 0.25 + 0.5j)
            got = red(data, init=0.25 + 0.5j)
            assert isinstance(got, np.dtype(dtype).type)
            assert abs(np.complex128(got) - np.complex128(want)) <= 16 * max(n, 8) * eps * abs(np.complex128(want))
