"""Parity of Reduce (HIP path, through the C ABI) with the oracle.

Bar: bit-exact for integers and for min/max; floating-point sums within
|err| <= 2 n eps sum|x| of the exact sum AND of the value the reference's
association order produces (oracle `tree`); products within 4 n eps relative.
"""

import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import numba_cuda_amd as cuda
from oracle import cref

sum_reduce = cuda.Reduce(lambda a, b: a + b)

# numba_cuda/numba/cuda/tests/cudapy/test_reduction.py:29-45
REFERENCE_SIZES = [1, 15, 16, 17, 127, 128, 129, 1023, 1024, 1025, 1536,
                   1048576, 1049600, 1049728, 34567]


def _say(*a):
    print(*a, flush=True)


@pytest.mark.parametrize("n", REFERENCE_SIZES)
def test_sum_reduce_reference_sizes(n):
    A = np.arange(n, dtype=np.float64) + 1
    got = sum_reduce(A)
    assert got == A.sum() == n * (n + 1) / 2
    assert isinstance(got, np.float64)


def test_empty_array_host_and_device():
    A = np.arange(0, dtype=np.float64) + 1
    assert sum_reduce(A) == 0
    assert sum_reduce(cuda.to_device(A)) == 0
    res = cuda.to_device(np.array([123.0]))
    assert sum_reduce(A, res=res, init=7) == 7     # returns init, leaves res untouched
    assert res[0] == 123.0


def test_prod_max_min_init_res():
    prod_reduce = cuda.reduce(lambda a, b: a * b)
    A = np.arange(64, dtype=np.float64) + 1
    np.testing.assert_allclose(prod_reduce(A, init=1), float(math.factorial(64)))
    max_reduce = cuda.Reduce(lambda a, b: max(a, b))
    B = np.arange(3717, dtype=np.float64) + 1
    assert max_reduce(B, init=0) == 3717
    assert cuda.Reduce(lambda a, b: min(a, b))(B, init=5000) == 1
    C = np.arange(10, dtype=np.float64) + 1
    assert sum_reduce(C, init=3) == C.sum() + 3
    got = cuda.to_device(np.zeros(1, dtype=np.float64))
    assert sum_reduce(C, res=got) is None
    assert got[0] == C.sum()


def test_only_1d_and_unknown_functor():
    with pytest.raises(TypeError, match="only support 1D array"):
        sum_reduce(np.zeros((2, 2)))
    with pytest.raises(NotImplementedError):
        cuda.Reduce(lambda a, b: int(a) - b)


def test_size_argument_and_offset_views():
    rng = np.random.default_rng(1)
    a = rng.integers(-1000, 1000, 5000).astype(np.int64)
    d = cuda.to_device(a)
    assert sum_reduce(d, size=1234) == a[:1234].sum()
    assert sum_reduce(d, size=10**9) == a.sum()         # clamped like a slice
    for lo in (1, 2, 3, 5, 127):
        assert sum_reduce(d[lo:]) == a[lo:].sum()
        assert sum_reduce(d[lo:4000 - lo]) == a[lo:4000 - lo].sum()
    b = rng.integers(-100, 100, 3001).astype(np.int8)
    db = cuda.to_device(b)
    for lo in (0, 1, 7, 15, 16, 17):
        assert sum_reduce(db[lo:]) == cref.fold("add", b[lo:])


@pytest.mark.parametrize("sfx", list(cref.SUFFIX))
@pytest.mark.parametrize("op", cref.OPS)
def test_every_operator_and_dtype_against_oracle(op, sfx):
    dt = np.dtype(cref.SUFFIX[sfx])
    functor = {"add": lambda a, b: a + b, "mul": lambda a, b: a * b,
               "max": lambda a, b: max(a, b), "min": lambda a, b: min(a, b)}[op]
    red = cuda.Reduce(functor)
    rng = np.random.default_rng(abs(hash((op, sfx))) % 2**32)
    # the last size is past 16 MiB for every element type: every workgroup loops over its slice
    for n in (1, 7, 64, 65, 255, 256, 257, 4096, 65536, 300001, 2**21 + 3, 2**24 + 5):
        _say("reduce", op, sfx, n)
        if dt.kind == "f":
            a = rng.standard_normal(n).astype(dt) if op != "mul" else (1 + rng.standard_normal(n) * 1e-3).astype(dt)
            init = 1.5
        else:
            info = np.iinfo(dt)
            a = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
            init = 3
        got = red(a, init=init)
        assert got.dtype == dt
        if dt.kind == "f" and op == "add":
            exact, sum_abs = cref.sum_exact(a)
            tol = 2 * n * np.finfo(dt).eps * (sum_abs + 1.5)
            assert abs(float(got) - (exact + 1.5)) <= tol
            assert abs(float(got) - float(cref.tree(op, a, init))) <= 2 * tol
        elif dt.kind == "f" and op == "mul":
            assert abs(float(got) / float(cref.tree(op, a, init)) - 1) <= 4 * n * np.finfo(dt).eps
        else:
            assert got == cref.fold(op, a, init)
            assert got == cref.tree(op, a, init)


@pytest.mark.parametrize("sfx", list(cref.INT_SUFFIX))
@pytest.mark.parametrize("op", cref.BITWISE_OPS)
def test_bitwise_operators_on_every_integer_type(op, sfx):
    """`a & b`, `a | b`, `a ^ b`: bit-exact against the oracle in both association orders
    (they are associative and commutative, so every order gives the same bits)."""
    dt = np.dtype(cref.SUFFIX[sfx])
    functor = {"and": lambda a, b: a & b, "or": lambda a, b: a | b, "xor": lambda a, b: a ^ b}[op]
    red = cuda.Reduce(functor)
    rng = np.random.default_rng(abs(hash((op, sfx))) % 2**32)
    info = np.iinfo(dt)
    for n in (1, 7, 64, 65, 257, 4096, 300001, 2**21 + 3, 2**24 + 5):
        _say("reduce", op, sfx, n)
        a = rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        if op == "and":                     # keep some bits alive: most elements have most bits set
            a |= rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
            a |= rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
        elif op == "or":
            a &= rng.integers(info.min, info.max, n, dtype=dt, endpoint=True)
            a &= rng.integers(info.min, info.max, n, dtype=dt, endpoint=True) if n > 64 else a
        init = {"and": -1 if dt.kind == "i" else info.max, "or": 0, "xor": 5}[op]
        got = red(a, init=init)
        assert got.dtype == dt
        want = {"and": np.bitwise_and, "or": np.bitwise_or, "xor": np.bitwise_xor}[op].reduce(a)
        if op == "xor":
            want = want ^ dt.type(5)
        assert got == want == cref.fold(op, a, init) == cref.tree(op, a, init), (n, got, want)
    # strided view and a device result slot
    d = cuda.to_device(a)
    res = cuda.device_array(1, dt)
    red(d[::3], res=res, init=init)
    assert res.copy_to_host()[0] == cref.fold(op, np.ascontiguousarray(a[::3]), init)


def test_boolean_arrays_any_all_parity():
    """`a | b`, `a & b`, `a ^ b`, max and min of booleans: any, all, parity, as booleans."""
    rng = np.random.default_rng(8)
    any_, all_, par = (cuda.Reduce(lambda a, b: a | b), cuda.Reduce(lambda a, b: a & b),
                       cuda.Reduce(lambda a, b: a ^ b))
    mx, mn = cuda.Reduce(lambda a, b: max(a, b)), cuda.Reduce(lambda a, b: min(a, b))
    for n in (1, 2, 63, 64, 65, 5000, 300001, 2**24 + 5):
        for p in (0.0, 1.0, 0.5, 1.0 / n, 1.0 - 1.0 / n):
            a = rng.random(n) < p
            _say("bool reduce", n, p)
            got = [any_(a, init=False), all_(a, init=True), par(a, init=False), mx(a, init=False), mn(a, init=True)]
            assert all(g.dtype == np.bool_ for g in got)
            assert got == [a.any(), a.all(), bool(a.sum() & 1), a.any(), a.all()], (n, p, got)
    d = cuda.to_device(a)
    res = cuda.device_array(1, np.bool_)
    any_(d[::2], res=res)
    assert res.copy_to_host()[0] == a[::2].any()


def test_boolean_sums_and_products():
    """`a + b` / `a * b` on booleans: int64 in the reference's JIT, converted back with
    `!= 0` at every store into its boolean arrays - any / all, as np.bool_."""
    rng = np.random.default_rng(9)
    add, mul = cuda.Reduce(lambda a, b: a + b), cuda.Reduce(lambda a, b: a * b)
    for n in (1, 2, 63, 65, 5000, 300001, 2**24 + 5):
        for p in (0.0, 1.0, 0.5, 1.0 / n, 1.0 - 1.0 / n):
            a = rng.random(n) < p
            _say("bool add/mul", n, p)
            d = cuda.to_device(a)
            for init in (0, 1, 2, False, True):
                got_add, got_mul = add(d, init=init), mul(d, init=init)
                assert got_add.dtype == np.bool_ and got_mul.dtype == np.bool_
                assert got_add == cref.tree("add", a, init) == cref.fold("add", a, init) == (a.any() or bool(init))
                assert got_mul == cref.tree("mul", a, init) == cref.fold("mul", a, init) == (a.all() and bool(init))
    res = cuda.device_array(1, np.bool_)
    add(d[::2], res=res)
    assert res.copy_to_host()[0] == a[::2].any()


def test_float16_reductions():
    """float16 is accumulated in float16 (one rounding per operation), like the reference's
    JIT does.  Bar: max / min bit-exact; sums bit-exact where every partial sum is a
    float16 in any association; other sums within 2 n eps sum|x| (eps = 2^-11) of the exact
    sum and of the reference-order value; products within 4 n eps relative."""
    rng = np.random.default_rng(10)
    add, mul = cuda.Reduce(lambda a, b: a + b), cuda.Reduce(lambda a, b: a * b)
    mx, mn = cuda.Reduce(lambda a, b: max(a, b)), cuda.Reduce(lambda a, b: min(a, b))
    eps = 2.0 ** -11
    for n in (1, 2, 7, 8, 9, 63, 64, 65, 511, 512, 513, 4097, 100003, 2**22 + 3):
        _say("float16 reduce", n)
        a = (rng.standard_normal(n) * 8).astype(np.float16)
        d = cuda.to_device(a)
        got = [mx(d, init=-np.inf), mn(d, init=np.inf)]
        assert all(g.dtype == np.float16 for g in got)
        assert got[0].tobytes() == cref.tree("max", a, -np.inf).tobytes() == a.max().tobytes()
        assert got[1].tobytes() == cref.tree("min", a, np.inf).tobytes() == a.min().tobytes()
        # small integers whose running totals stay below 2048 in magnitude: exact in every order
        k = rng.integers(-3, 4, n).astype(np.float16)
        if np.abs(k.astype(np.float64)).sum() < 2048:
            got = add(k, init=5)
            assert got.dtype == np.float16
            assert got.tobytes() == cref.tree("add", k, 5).tobytes() == cref.fold("add", k, 5).tobytes()
            assert float(got) == k.astype(np.float64).sum() + 5
        if n <= 4097:
            got = float(add(d, init=0))
            exact = a.astype(np.float64).sum()
            bound = 2 * n * eps * np.abs(a.astype(np.float64)).sum() + eps * abs(exact)    # tolerance
            assert abs(got - exact) <= bound, (n, got, exact)
            assert abs(got - float(cref.tree("add", a, 0))) <= 2 * bound
            b = (1.0 + rng.standard_normal(n) * 2e-3).astype(np.float16)
            got = float(mul(b, init=1))
            exact = float(np.prod(b.astype(np.float64)))
            assert abs(got - exact) <= (4 * n + 1) * eps * abs(exact), (n, got, exact)     # tolerance
    # the accumulator is a half: 2^20 ones overflow it (65504 is the largest float16),
    # in the reference's association as in this one
    ones = np.ones(2**20, np.float16)
    assert float(add(ones)) == float(cref.tree("add", ones, 0)) == np.inf
    # strided view, device result slot, offset views
    d = cuda.to_device(a)
    res = cuda.device_array(1, np.float16)
    mx(d[::3], res=res, init=-np.inf)
    assert res.copy_to_host()[0] == a[::3].max()
    for lo in (1, 2, 3, 7, 9):
        assert mn(d[lo:], init=np.inf) == a[lo:].min()


@pytest.mark.parametrize("dtype", [np.complex64, np.complex128])
def test_complex_sums_and_products(dtype):
    """Complex elements: sums within 2 n eps sum|x| per component of the exact sums;
    products of near-unit factors within 8 n eps (relative) of the oracle's value in
    the reference's association order; integers-valued inputs exactly."""
    dt = np.dtype(dtype)
    real = np.float32 if dt == np.complex64 else np.float64
    eps = np.finfo(real).eps
    rng = np.random.default_rng(21)
    add, mul = cuda.Reduce(lambda a, b: a + b), cuda.Reduce(lambda a, b: a * b)
    for n in (1, 2, 3, 63, 64, 65, 1000, 4097, 300001, 2**21 + 5):
        _say("complex reduce", dt, n)
        a = (rng.standard_normal(n) + 1j * rng.standard_normal(n)).astype(dt)
        got = add(a, init=1 - 2j)
        assert got.dtype == dt
        for part, off in (("real", 1.0), ("imag", -2.0)):
            exact, sum_abs = cref.sum_exact(np.ascontiguousarray(getattr(a, part)))
            tol = 2 * n * eps * (sum_abs + 2.0)                       # tolerance: 2 n eps sum|x|
            assert abs(float(getattr(got, part)) - (exact + off)) <= tol
        # exactly representable partial sums: every association gives the same bits
        k = (rng.integers(-1000, 1000, n) + 1j * rng.integers(-1000, 1000, n)).astype(dt)
        assert add(k, init=3 + 4j) == cref.tree("add", k, 3 + 4j) == cref.fold("add", k, 3 + 4j)
        m = min(n, 5000)
        u = (np.exp(1j * rng.uniform(0, 2 * np.pi, m)) * (1 + 1e-3 * rng.standard_normal(m))).astype(dt)
        got = mul(u, init=1)
        want = cref.tree("mul", u, 1)
        assert abs(got - want) <= 8 * m * eps * abs(want)             # tolerance: 8 n eps, relative
    # Gaussian integers: products are exact while they fit the mantissa
    g = np.array([1 + 1j, 2 - 1j, -1 + 3j, 2 + 2j, 1 - 4j, 3 + 1j], dtype=dt)
    assert mul(g, init=1j) == np.prod(g.astype(np.complex128)) * 1j == cref.tree("mul", g, 1j)
    d = cuda.to_device((rng.standard_normal(1001) + 1j * rng.standard_normal(1001)).astype(dt))
    np.testing.assert_allclose(add(d[::-2]), d.copy_to_host()[::-2].sum(), rtol=1e-4 if dt == np.complex64 else 1e-12)
    res = cuda.device_array(1, dt)
    assert add(d, res=res) is None and res.copy_to_host()[0] == add(d)
    for op in (lambda a, b: max(a, b), lambda a, b: min(a, b)):
        with pytest.raises(TypeError, match="not defined for complex"):
            cuda.Reduce(op)(d)


def test_simulator_case_65536_uniform_seed_0():
    """The CPU-runnable configuration of the reference (its simulator: a strict left
    fold of 65 536 float32 drawn uniform [-1, 1) from seed 0, init 0) beside the GPU:
    both within 2 n eps sum|x| of the exact sum, hence within twice that of each other."""
    from oracle import sim
    a = np.random.default_rng(0).uniform(-1, 1, 65536).astype(np.float32)
    want = sim.Reduce(lambda x, y: x + y)(a, init=0)
    assert isinstance(want, np.float32) and want == cref.fold("add", a, 0)
    got = sum_reduce(cuda.to_device(a), init=0)
    assert got.dtype == np.float32
    exact, sum_abs = cref.sum_exact(a)
    tol = 2 * a.size * np.finfo(np.float32).eps * sum_abs          # tolerance: 2 n eps sum|x|
    assert abs(float(got) - exact) <= tol and abs(float(want) - exact) <= tol
    assert abs(float(got) - float(want)) <= 2 * tol
    res = cuda.device_array(1, np.float32)
    assert sum_reduce(a, res=res, init=0) is None and res.copy_to_host()[0] == got


def test_runs_are_bitwise_reproducible():
    rng = np.random.default_rng(5)
    a = cuda.to_device(rng.standard_normal(3_000_017).astype(np.float32))
    first = sum_reduce(a)
    for _ in range(10):
        assert sum_reduce(a).tobytes() == first.tobytes()
    # past 16 MiB, where the workgroups loop
    b = cuda.to_device(rng.standard_normal(20_000_003).astype(np.float32))
    first = sum_reduce(b)
    for _ in range(20):
        assert sum_reduce(b).tobytes() == first.tobytes()


def test_stream_and_result_slot_round_robin():
    """The batched-reduction case in small: independent row sums issued over 4 streams into
    slots of one device vector."""
    rng = np.random.default_rng(3)
    rows, cols = 64, 65536
    m = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    dm = cuda.to_device(m)
    out = cuda.device_array(rows, dtype=np.float32)
    streams = [cuda.stream() for _ in range(4)]
    for i in range(rows):
        assert sum_reduce(dm[i], res=out[i:i + 1], stream=streams[i % 4]) is None
    for s in streams:
        s.synchronize()
    got = out.copy_to_host()
    for i in range(rows):
        exact, sum_abs = cref.sum_exact(m[i])
        assert abs(float(got[i]) - exact) <= 2 * cols * np.finfo(np.float32).eps * sum_abs
    # the same call returns the value when no `res` is given, also on a stream
    v = sum_reduce(dm[5], stream=streams[1])
    assert v.tobytes() == got[5].tobytes()


def test_batched_row_sums_full_shape_4096_rows_over_four_streams():
    """The batched configuration at its real shape: 4096 independent float32 sums over the
    65 536-item rows of a uniform [-1, 1) matrix (seed 3), each issued with its own call into a
    slot of one device vector, round-robin over 4 streams.  Every row against the exact sum
    (tolerance 2 n eps sum|x|) and, bit for bit, against the same reduction issued alone."""
    rng = np.random.default_rng(3)
    rows, cols = 4096, 65536
    m = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    dm = cuda.to_device(m)
    out = cuda.device_array(rows, dtype=np.float32)
    streams = [cuda.stream() for _ in range(4)]
    views = [dm[i] for i in range(rows)]
    slots = [out[i:i + 1] for i in range(rows)]
    _say("batched: issuing", rows, "reductions")
    for i in range(rows):
        sum_reduce(views[i], res=slots[i], stream=streams[i & 3])
    for s in streams:
        s.synchronize()
    got = out.copy_to_host()
    eps = np.finfo(np.float32).eps
    for i in range(rows):
        exact, sum_abs = cref.sum_exact(m[i])
        assert abs(float(got[i]) - exact) <= 2 * cols * eps * sum_abs, i      # tolerance
    for i in (0, 1, 2, 3, 1000, 4095):
        assert sum_reduce(views[i]).tobytes() == got[i].tobytes()


# ---- full HBM-scale inputs, seed 1 ---------------- --------------------------------

def test_fullsize_float32_sum_and_max_2_pow_28():
    n = 2**28
    _say("generating f32", n)
    a = np.random.default_rng(1).standard_normal(n, dtype=np.float32)
    d = cuda.to_device(a)
    got = sum_reduce(d)
    exact, sum_abs = cref.sum_exact(a)
    tol = 2 * n * np.finfo(np.float32).eps * sum_abs
    assert abs(float(got) - exact) <= tol
    assert abs(float(got) - float(cref.tree("add", a))) <= 2 * tol
    # in practice the tree order is far tighter than the bound; keep a tripwire
    assert abs(float(got) - exact) <= 1e-3 * tol
    mx = cuda.Reduce(lambda x, y: max(x, y))(d, init=-np.inf)
    assert mx == a.max() == cref.tree("max", a, -np.inf)


def test_fullsize_float64_sum_2_pow_27():
    n = 2**27
    a = np.random.default_rng(1).standard_normal(n)
    got = sum_reduce(cuda.to_device(a))
    exact, sum_abs = cref.sum_exact(a)
    tol = 2 * n * np.finfo(np.float64).eps * sum_abs
    assert abs(float(got) - exact) <= tol
    assert abs(float(got) - float(cref.tree("add", a))) <= 2 * tol


def test_fullsize_int64_sum_2_pow_28_bit_exact():
    n = 2**28
    a = np.random.default_rng(1).integers(-2**20, 2**20, n, dtype=np.int64, endpoint=True)
    got = sum_reduce(cuda.to_device(a))
    assert got == cref.tree("add", a) == a.sum()


@pytest.mark.parametrize("dtype,items,skip", [
    (np.int8, 150_000_011, 3), (np.uint16, 80_000_003, 1), (np.int32, 40_000_001, 3),
    (np.int64, 20_000_003, 1), (np.float64, 25_000_007, 1), (np.complex128, 10_000_019, 0),
    (np.float32, 35_000_017, 2), (np.int32, 33_554_432 + 1024 * 4 * 5, 0)])
def test_large_inputs_of_awkward_length_and_start(dtype, items, skip):
    """From 128 MiB on the input is read in 16 KiB pieces dealt out to the workgroups: lengths
    that leave part of a piece and part of a 16-byte packet over, views that start off a
    16-byte boundary, every item size.  Integers wrap, so every association gives the same
    bits; the floating-point data are small integers whose sums are exact in any order."""
    rng = np.random.default_rng(items)
    dt = np.dtype(dtype)
    _say("large", dt.name, items, skip)
    if dt.kind in "iu":
        info = np.iinfo(dt)
        host = rng.integers(info.min, info.max, items, dtype=dt, endpoint=True)
    elif dt.kind == "c":
        host = (rng.integers(-8, 8, items) + 1j * rng.integers(-8, 8, items)).astype(dt)
    else:
        host = rng.integers(-8, 8, items).astype(dt)
    whole = cuda.to_device(host)
    dev, ref = whole[skip:], host[skip:]
    assert dev.nbytes >= 128 << 20
    got = sum_reduce(dev)
    if dt.kind in "iu":
        assert got == ref.sum(dtype=dt)
    elif dt == np.float32:   # partial sums stay far below 2^24 in practice but nothing bounds them
        assert abs(float(got) - float(ref.sum(dtype=np.float64))) <= 2 * ref.size * np.finfo(dt).eps * float(np.abs(ref).sum(dtype=np.float64))
    else:
        assert got == ref.sum()
    if dt.kind != "c":
        # a maximum in the last item and a minimum in the first: the edges of the range count
        host[-1], host[skip] = host.max(), host.min()
        whole[items - 1:items] = host[-1:]
        whole[skip:skip + 1] = host[skip:skip + 1]
        lo, hi = (np.iinfo(dt).min, np.iinfo(dt).max) if dt.kind in "iu" else (-np.inf, np.inf)
        assert cuda.Reduce(lambda x, y: max(x, y))(dev, init=lo) == ref.max()
        assert cuda.Reduce(lambda x, y: min(x, y))(dev, init=hi) == ref.min()
        marked = host.copy()
        spot = items - 1 - (items - skip) % 4096 // 2   # inside what is left over behind the last piece
        marked[spot] = hi if dt.kind in "iu" else 1000
        whole[spot:spot + 1] = marked[spot:spot + 1]
        assert cuda.Reduce(lambda x, y: max(x, y))(dev, init=lo) == marked[skip:].max()


@pytest.mark.parametrize("n_min,n_max,calls", [(5000, 3_000_000, 3000), (2_200_000, 9_000_000, 1500)])
def test_back_to_back_reductions_never_see_stale_partials(n_min, n_max, calls):
    """Thousands of launches reuse one scratch buffer per stream with different
    data each time; a partial read from a stale cache line would change an integer
    sum.  Sizes span 2 to 512 workgroups; in the second case every launch has all 512
    and they finish close together."""
    rng = np.random.default_rng(77)
    base = rng.integers(-2**40, 2**40, n_max + 4096, dtype=np.int64)
    d = cuda.to_device(base)
    offs = rng.integers(0, 4096, calls)
    sizes = rng.integers(n_min, n_max, calls)
    sizes[::7] = rng.integers(max(n_min, 2_500_000), n_max, len(sizes[::7]))
    out = cuda.device_array(calls, np.int64)
    streams = [cuda.stream() for _ in range(3)]
    for i in range(calls):
        sum_reduce(d[offs[i]:offs[i] + sizes[i]], res=out[i:i + 1], init=i, stream=streams[i % 3])
    for s in streams:
        s.synchronize()
    got = out.copy_to_host()
    csum = np.concatenate([[0], np.cumsum(base)])
    want = csum[offs + sizes] - csum[offs] + np.arange(calls)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (bad[:10], got[bad[:10]], want[bad[:10]])


def test_strided_and_reversed_views():
    """The reference indexes `arr[i]`, so any 1-D view reduces; here non-unit strides
    take the item-by-item path of the same kernel."""
    rng = np.random.default_rng(21)
    a = rng.integers(-10**6, 10**6, 200_003).astype(np.int64)
    d = cuda.to_device(a)
    mx = cuda.Reduce(lambda x, y: max(x, y))
    for view, want in ((d[::2], a[::2]), (d[1::3], a[1::3]), (d[::-1], a[::-1]), (d[5000:100:-7], a[5000:100:-7]),
                       (d[::1000], a[::1000]), (d[7:8:5], a[7:8:5])):
        assert sum_reduce(view, init=3) == want.sum() + 3
        assert mx(view, init=-10**9) == want.max()
    m = rng.standard_normal((300, 257)).astype(np.float32)
    dm = cuda.to_device(m)
    col = dm[:, 5]                                   # a column: stride = one row
    exact, sum_abs = cref.sum_exact(np.ascontiguousarray(m[:, 5]))
    assert abs(float(sum_reduce(col)) - exact) <= 2 * 300 * np.finfo(np.float32).eps * sum_abs
    b = rng.integers(-128, 127, 70_001).astype(np.int8)
    assert sum_reduce(cuda.to_device(b)[::3]) == cref.fold("add", np.ascontiguousarray(b[::3]))


def test_value_returning_reductions_from_four_threads_on_one_stream():
    """Each call has its own result cell: threads that share a stream (here the default
    one, then a created one) must each get their own value back, bit-exact."""
    import threading
    rng = np.random.default_rng(21)
    hosts = [rng.integers(-10**6, 10**6, 40_000 + 1000 * k).astype(np.int64) for k in range(4)]
    devs = [cuda.to_device(h) for h in hosts]
    wants = [int(h.sum()) for h in hosts]
    for stream in (0, cuda.stream()):
        _say("threads on stream", stream)
        wrong = []

        def worker(k):
            for i in range(2000):
                got = sum_reduce(devs[k], init=i, stream=stream)
                if int(got) != wants[k] + i:
                    wrong.append((k, i, int(got)))
                    return

        threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not wrong, wrong


def test_per_thread_default_stream_keeps_scratch_per_thread():
    """cuda.per_thread_default_stream() is one handle but a different stream in every
    host thread: reductions on it may overlap, so every thread needs scratch of its own."""
    import threading
    rng = np.random.default_rng(22)
    hosts = [rng.integers(-10**6, 10**6, 3_000_000 + 4096 * k).astype(np.int64) for k in range(4)]
    devs = [cuda.to_device(h) for h in hosts]
    wants = [int(h.sum()) for h in hosts]
    wrong = []

    def worker(k):
        s = cuda.per_thread_default_stream()
        for i in range(300):
            got = sum_reduce(devs[k], init=i, stream=s)
            if int(got) != wants[k] + i:
                wrong.append((k, i, int(got)))
                return

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not wrong, wrong


def test_by_the_book_publication_build_gives_the_same_bits():
    """libnbhip_release_publish.so is the same library with the reduction kernels publishing
    their partials through ordinary stores and a release at agent scope
    (-DNBH_REDUCE_RELEASE_PUBLISH=1) instead of the written-through atomic stores the shipped
    build relies on.  Loaded beside the shipped library and driven through the C ABI on the same
    device memory: integer sums from 1200 back-to-back launches of changing sizes must equal the
    exact prefix-sum differences and the shipped build's results, bit for bit."""
    import ctypes
    import os
    from numba_cuda_amd import _build, _lib
    from numba_cuda_amd.cudadrv import driver as drv
    if not os.path.exists(_build.RELEASE_PUBLISH_LIB):
        pytest.fail("%s is missing: __graft_entry__.build() makes it" % _build.RELEASE_PUBLISH_LIB)
    other = ctypes.CDLL(_build.RELEASE_PUBLISH_LIB)
    for name in ("nbh_reduce", "nbh_reduce_scratch_bytes", "nbh_stream_synchronize"):
        getattr(other, name).restype, getattr(other, name).argtypes = _lib.SIGNATURES[name]
    cuda.current_context()
    shipped = drv.driver.lib
    rng = np.random.default_rng(123)
    calls, n_max = 1200, 6_000_000
    base = rng.integers(-2**40, 2**40, n_max + 4096, dtype=np.int64)
    d = cuda.to_device(base)
    offs = rng.integers(0, 4096, calls)
    sizes = rng.integers(3000, n_max, calls)
    out_a, out_b = cuda.device_array(calls, np.int64), cuda.device_array(calls, np.int64)
    nbytes = other.nbh_reduce_scratch_bytes()
    assert nbytes == shipped.nbh_reduce_scratch_bytes()
    scratch_a = cuda.to_device(np.zeros(nbytes, np.uint8))
    scratch_b = cuda.to_device(np.zeros(nbytes, np.uint8))
    stream = cuda.stream()
    code, op = _lib.DTYPE_CODES["int64"], _lib.OP_CODES["add"]
    inits = np.arange(calls, dtype=np.int64)
    for i in range(calls):
        src = d.device_ctypes_pointer.value + 8 * int(offs[i])
        for lib, out, scratch in ((shipped, out_a, scratch_a), (other, out_b, scratch_b)):
            rc = lib.nbh_reduce(op, code, src, int(sizes[i]), 8, inits[i:i + 1].ctypes.data,
                                out.device_ctypes_pointer.value + 8 * i, scratch.device_ctypes_pointer.value, nbytes,
                                stream.handle)
            assert rc == 0
    stream.synchronize()
    csum = np.concatenate([[0], np.cumsum(base)])
    want = csum[offs + sizes] - csum[offs] + np.arange(calls)
    got_a, got_b = out_a.copy_to_host(), out_b.copy_to_host()
    assert (got_b == want).all() and (got_a == got_b).all()
    # floating point: the same kernels and grid, so the same bits
    f = cuda.to_device(rng.standard_normal(3_000_001).astype(np.float32))
    fa, fb = cuda.device_array(1, np.float32), cuda.device_array(1, np.float32)
    zero = np.zeros(1, np.float32)
    for lib, out, scratch in ((shipped, fa, scratch_a), (other, fb, scratch_b)):
        assert lib.nbh_reduce(op, _lib.DTYPE_CODES["float32"], f.device_ctypes_pointer.value, f.size, 4, zero.ctypes.data,
                              out.device_ctypes_pointer.value, scratch.device_ctypes_pointer.value, nbytes, stream.handle) == 0
    stream.synchronize()
    assert fa.copy_to_host().tobytes() == fb.copy_to_host().tobytes()
