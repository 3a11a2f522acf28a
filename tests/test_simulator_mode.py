"""The package's CPU mode (NUMBA_ENABLE_CUDASIM=1, numba_cuda_amd/simulator) against the
restated reference simulator (oracle/sim.py), the C oracle and the golden fixtures.  The
mode itself never imports the oracle; these tests do, as the checker."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from numba_cuda_amd import _xoroshiro_host as host_rng
from numba_cuda_amd import simulator as simcuda
from numba_cuda_amd.simulator import hostarray
from oracle import cref, sim

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def load(name):
    with open(os.path.join(GOLDEN, name)) as fh:
        return json.load(fh)


# ---- Reduce: the strict left fold --------------------------------------------------------

@pytest.mark.parametrize("n", [0, 1, 2, 31, 1000, 65536])
def test_reduce_is_the_left_fold_of_the_restated_simulator(n):
    a = np.random.default_rng(0).uniform(-1, 1, n).astype(np.float32)
    ours = simcuda.reduce(lambda x, y: x + y)
    theirs = sim.Reduce(lambda x, y: x + y)
    got, want = ours(simcuda.to_device(a), init=0), theirs(a, init=0)
    assert type(got) is type(want) and got == want
    # `init` is used as given, not cast to the array's dtype: with no elements it comes back untouched
    assert ours(simcuda.to_device(a[:0]), init=7) == 7


def test_reduce_into_a_result_array_and_other_operators():
    a = np.arange(1, 21, dtype=np.int64)
    res = simcuda.device_array(1, np.int64)
    assert simcuda.Reduce(lambda x, y: x * y)(simcuda.to_device(a), res=res, init=1) is None
    assert res.copy_to_host()[0] == load("closed_forms.json")["factorial_20_int64"]
    for vec in load("closed_forms.json")["sum_of_1_to_n"]:
        assert simcuda.reduce(lambda x, y: x + y)(np.arange(1, vec["n"] + 1)) == vec["sum"]
    assert simcuda.reduce(lambda x, y: max(x, y))(simcuda.to_device(np.array([3., -1., 9., 2.])), init=-np.inf) == 9.0


def test_reduce_takes_the_gpu_mode_constructor_arguments():
    """Code written for the GPU mode (`Reduce(functor, reference_order=True)`) runs unchanged:
    the left fold has one order, the argument chooses nothing."""
    minus = lambda x, y: x - y
    a = np.arange(10, dtype=np.float32)
    assert simcuda.Reduce(minus, reference_order=True)(a, init=1) == sim.Reduce(minus)(a, init=1)
    assert simcuda.Reduce(minus, reference_order=False)(a, init=1) == simcuda.reduce(minus)(a, init=1)


# ---- arrays -------------------------------------------------------------------------------

def test_to_device_owns_its_bytes_and_round_trips():
    a = np.arange(24, dtype=np.float64).reshape(4, 6)
    d = simcuda.to_device(a)
    a[0, 0] = -1
    assert d.copy_to_host()[0, 0] == 0
    assert d.shape == (4, 6) and d.dtype == np.float64 and d.strides == (48, 8) and d.size == 24 and d.ndim == 2
    assert d.nbytes == d.alloc_size == 192
    with pytest.raises(IndexError):
        d.shape[-1]
    f = simcuda.to_device(np.asfortranarray(a))
    assert f.is_f_contiguous() and not f.is_c_contiguous()
    with pytest.raises(ValueError, match="non-contiguous"):
        simcuda.to_device(a[:, ::2])


def test_views_slices_and_assignment():
    d = simcuda.to_device(np.arange(12, dtype=np.int32).reshape(3, 4))
    assert d[1, 2] == 6 and isinstance(d[1], hostarray.HostBackedArray)
    assert d[1].copy_to_host().tolist() == [4, 5, 6, 7]
    assert d.T.shape == (4, 3) and d.transpose().copy_to_host().tolist() == np.arange(12).reshape(3, 4).T.tolist()
    d[0] = 9
    d[2, 1:3] = simcuda.to_device(np.array([70, 80], np.int32))
    assert d.copy_to_host().tolist() == [[9, 9, 9, 9], [4, 5, 6, 7], [8, 70, 80, 11]]
    assert d.reshape(4, 3).shape == (4, 3) and d.ravel().shape == (12,)
    assert [p.copy_to_host().tolist() for p in simcuda.to_device(np.arange(5)).split(2)] == [[0, 1], [2, 3], [4]]
    assert (d + 1).copy_to_host()[1, 0] == 5 and bool((d == d).copy_to_host().all())


def test_copies_check_dtype_shape_and_strides():
    d = simcuda.device_array((2, 3), np.float32)
    d.copy_to_device(np.ones((2, 3), np.float32))
    assert d.copy_to_host().sum() == 6
    with pytest.raises(TypeError, match="incompatible dtype"):
        d.copy_to_device(np.ones((2, 3), np.float64))
    with pytest.raises(ValueError, match="incompatible shape"):
        d.copy_to_device(np.ones((3, 2), np.float32))
    with pytest.raises(ValueError, match="incompatible shape"):
        d.copy_to_host(np.empty((6,), np.float32))
    simcuda.to_device(np.full((2, 3), 5, np.float32), to=d)
    assert d.copy_to_host()[1, 2] == 5


def test_like_constructors_pinned_mapped_and_auto_device():
    a = np.zeros((3, 5, 7))[:, ::2, :]
    like = simcuda.device_array_like(a)
    assert like.shape == a.shape and like.is_c_contiguous()
    f = simcuda.device_array_like(np.asfortranarray(np.zeros((3, 4))))
    assert f.is_f_contiguous()
    assert type(simcuda.pinned_array((2, 2))) is np.ndarray and type(simcuda.managed_array(3)) is np.ndarray
    assert isinstance(simcuda.mapped_array(4, np.int8, portable=True, wc=True), hostarray.HostBackedArray)
    with simcuda.pinned(np.zeros(3)):
        pass
    d, fresh = simcuda._auto_device(np.arange(3))
    assert fresh and simcuda._auto_device(d) == (d, False)
    assert simcuda.is_cuda_ndarray(d) and not simcuda.is_cuda_ndarray(np.arange(3))
    with pytest.raises(ValueError):
        simcuda.require_cuda_ndarray(np.arange(3))
    simcuda.verify_cuda_ndarray_interface(d)


def test_streams_events_and_devices_are_inert():
    s = simcuda.stream()
    with s.auto_synchronize():
        s.synchronize()
    e0, e1 = simcuda.event(), simcuda.event(timing=False)
    e0.record(s)
    e1.record()
    e1.wait(s)
    e1.synchronize()
    assert e0.elapsed_time(e1) == -1.0
    with pytest.raises(RuntimeError, match="External streams"):
        simcuda.external_stream(1234)
    assert len(simcuda.gpus) == 1 and simcuda.get_current_device().name == "SIMULATOR"
    assert simcuda.select_device(0) is simcuda.gpus[0].device
    with pytest.raises(AssertionError):
        simcuda.select_device(1)
    with simcuda.defer_cleanup():
        simcuda.synchronize()
    assert simcuda.is_available() and simcuda.current_context().get_memory_info().total > 0


def test_in_out_inout():
    from numba_cuda_amd.simulator.args import In, InOut, Out
    host = np.arange(4.0)
    for hint, back in ((In, False), (Out, True), (InOut, True)):
        after = []
        dev = hint(host).to_device(after)
        assert isinstance(dev, hostarray.HostBackedArray) and bool(after) == back
    dev[0] = 42
    after[0]()
    assert host[0] == 42


def test_transpose_function():
    a = np.random.default_rng(2).integers(-9, 9, (5, 7)).astype(np.int16)
    out = simcuda.transpose(simcuda.to_device(a))
    assert out.shape == (7, 5) and (out.copy_to_host() == sim.transpose(a)).all()
    into = simcuda.device_array((7, 5), np.int16)
    assert simcuda.transpose(simcuda.to_device(a), into) is into and (into.copy_to_host() == a.T).all()
    assert simcuda.transpose(simcuda.to_device(np.arange(12).reshape(3, 4))).copy_to_host().tolist() == \
        load("closed_forms.json")["transpose_of_arange_3x4"]


# ---- RNG ----------------------------------------------------------------------------------

def test_state_chains_match_the_fixtures_and_the_oracle():
    for chain in load("xoroshiro128p_vectors.json")["chains"]:
        want = chain["states"]
        st = simcuda.random.create_xoroshiro128p_states(len(want), chain["seed"], chain["subsequence_start"])
        got = st.copy_to_host()
        assert [[int(r["s0"]), int(r["s1"])] for r in got] == want
    for n, seed, start in ((1, 1, 0), (2, 5, 1), (1000, 42, 3), (4097, 2**64 - 1, 17)):
        got = np.zeros(n, host_rng.xoroshiro128p_dtype)
        host_rng.init_states_cpu(got, seed, start)
        assert got.tobytes() == cref.init_states(n, seed, start).tobytes()


def test_the_chain_by_doubling_is_the_sequential_chain():
    # the reference's own construction (random.py:241-257) through the restated simulator, 40 generators
    want = np.zeros(40, cref.STATE_DTYPE)
    sim.init_states(want, 7, 2)
    got = np.zeros(40, host_rng.xoroshiro128p_dtype)
    host_rng.init_states_cpu(got, 7, 2)
    assert got.tobytes() == want.tobytes()
    # a start far beyond any chain: J^(a + b) = J^a J^b
    x = np.zeros(4, host_rng.xoroshiro128p_dtype)
    y = np.zeros(4, host_rng.xoroshiro128p_dtype)
    host_rng.init_states_cpu(x, 9, 2**40 + 3)
    host_rng.init_states_cpu(y, 9, 2**40)
    assert x[0] == y[3]


def test_scalar_draws_match_the_restated_simulator():
    ours = simcuda.random.create_xoroshiro128p_states(3, 11)
    theirs = np.zeros(3, cref.STATE_DTYPE)
    sim.init_states(theirs, 11)
    r = simcuda.random
    pairs = ((r.xoroshiro128p_next, sim.next_u64), (r.xoroshiro128p_uniform_float32, sim.uniform_float32),
             (r.xoroshiro128p_uniform_float64, sim.uniform_float64), (r.xoroshiro128p_normal_float32, sim.normal_float32),
             (r.xoroshiro128p_normal_float64, sim.normal_float64))
    for _ in range(20):
        for mine, ref in pairs:
            for t in range(3):
                a, b = mine(ours, t), ref(theirs, t)
                assert type(a) is type(b) and a == b
    r.xoroshiro128p_jump(ours, 1)
    sim.jump(theirs, 1)
    assert ours.copy_to_host().tobytes() == theirs.tobytes()


@pytest.mark.parametrize("kind,dtype,distribution", [("uniform_f32", np.float32, 1), ("uniform_f64", np.float64, 1),
                                                    ("normal_f32", np.float32, 2), ("normal_f64", np.float64, 2)])
def test_bulk_draws_against_the_c_oracle(kind, dtype, distribution):
    n, count = 37, 9
    st = simcuda.random.create_xoroshiro128p_states(n, 42, 1)
    want, want_states = cref.fill(st.copy_to_host(), count, kind)
    out = simcuda.device_array(n * count, dtype)
    simcuda.random.xoroshiro128p_fill(st, out, count, distribution)
    got = out.copy_to_host()
    if distribution == 1:
        assert got.tobytes() == want.tobytes()          # uniform values: bit for bit
    else:
        # normals: the simulator's flavour (double-precision functions), one generator at a time
        theirs = cref.init_states(n, 42, 1)
        draw = sim.normal_float32 if dtype is np.float32 else sim.normal_float64
        ref = np.array([[draw(theirs, t) for _ in range(count)] for t in range(n)]).astype(dtype).reshape(-1)
        assert np.all(np.abs(got - ref) <= np.spacing(np.abs(ref)))     # NumPy's log / cos against libm's
        # and within float32 rounding of the GPU flavour the C oracle holds
        assert np.allclose(got, want, rtol=0, atol=4e-6)
    assert st.copy_to_host().tobytes() == want_states.tobytes()


def test_fixture_draws():
    for vec in load("xoroshiro128p_vectors.json")["draws"]:
        st = simcuda.random.create_xoroshiro128p_states(1, vec["seed"])
        raw = [int(simcuda.random.xoroshiro128p_next(st, 0)) for _ in range(12)]
        assert raw == vec["next_u64"]


# ---- the switch ---------------------------------------------------------------------------

def test_environment_variable_switches_the_whole_package():
    """BASELINE's CPU configuration, through `import numba_cuda_amd as cuda` on a machine
    without a GPU: float32 sum of 65 536 values uniform in [-1, 1), seed 0, init = 0."""
    code = r'''
import sys, numpy as np
import numba_cuda_amd as cuda
from numba_cuda_amd.kernels.reduction import Reduce
from numba_cuda_amd.kernels.transpose import transpose
from numba_cuda_amd import random as rnd
a = np.random.default_rng(0).uniform(-1, 1, 65536).astype(np.float32)
d = cuda.to_device(a)
total = cuda.reduce(lambda x, y: x + y)(d, init=0)
res = cuda.device_array(1, np.float32)
Reduce(lambda x, y: x + y)(d, res=res, init=0)
assert res.copy_to_host()[0] == total
assert (transpose(cuda.to_device(np.arange(6).reshape(2, 3))).copy_to_host() == np.arange(6).reshape(2, 3).T).all()
st = rnd.create_xoroshiro128p_states(4, 42)
u = rnd.xoroshiro128p_uniform_float32(st, 0)
loaded = [m for m in sys.modules if m.startswith("numba_cuda_amd.cudadrv.driver") or m == "oracle" or m.startswith("oracle.")]
maps = open("/proc/self/maps").read()
print(repr(float(total)), repr(float(u)), loaded, "libnbhip" in maps, "liboracle" in maps)
'''
    env = dict(os.environ, NUMBA_ENABLE_CUDASIM="1", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    total, u, loaded, hip, orc = out.stdout.strip().rsplit(" ", 4)[0], None, None, None, None
    fields = out.stdout.strip().split(" ", 2)
    a = np.random.default_rng(0).uniform(-1, 1, 65536).astype(np.float32)
    assert float(fields[0]) == float(sim.Reduce(lambda x, y: x + y)(a, init=0))
    theirs = np.zeros(4, cref.STATE_DTYPE)
    sim.init_states(theirs, 42)
    assert float(fields[1]) == float(sim.uniform_float32(theirs, 0))
    assert fields[2] == "[] False False"
