#!/usr/bin/env python
"""Benchmark of the hot path on one MI355X.

Default workload (the configuration the headline metric is quoted
on): cuda.reduce float32 sum over 2^28 elements N(0,1), seed 1.  A "step" is one
full reduction, issued through the public API into a device result slot; inputs
are resident in HBM before the clock starts.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-others]
                    [--view-cols N] [--elements N]

Without --workload the same line carries an `others` array with every other
benchmark configuration measured in the same process: reduce_f32_max,
reduce_f64_sum, reduce_i64_sum, reduce_f32_functor (a translated functor),
reduce_f32_sum_reference_order (the reference's association order), transpose_f32,
transpose_f64, transpose_i16, rng_init, rng_uniform_f32, rng_normal_f64, batched_reduce, and ends with
`others_summary`, the same figures in short.  --workload NAME measures just one of them (or copy_f32, the counter
calibration kernel) as the headline; --view-cols N (transposes: the first N columns only, pitches unchanged) and
--elements N (copy_f32) give the time-against-size tables of profiles/.
"""

import argparse
import json
import math
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E published peak

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
# (see profiles/); filled in per workload once measured, else None
MEASURED_TRAFFIC = {
    # fetched + written bytes per launch; each figure is derived in the profiles/ file TRAFFIC_SOURCE names
    "reduce_f32_sum": 1073804215,
    "copy_f32": 2147483648,                      # the calibration kernel itself
    "transpose_f32": 2147948643,
    "transpose_f64": 1349570873,
    "transpose_i16": 1073941648,
    "reduce_f32_max": 1073819617,
    "reduce_f64_sum": 1073818517,
    "reduce_i64_sum": 2147532373,
    "reduce_f32_sum_reference_order": 1073951990,
    "reduce_f32_functor": 1073931926,
    "rng_uniform_f32": 4831199483,
    "rng_normal_f64": 2683917445,
    "rng_init": 298423381,
}


def _event_timed_launches(cuda, stream, launch, reps):
    """Average duration (ms) of one launch: one HIP event pair, recorded on the
    stream the kernels run on, around `reps` back-to-back launches.  Launches on one
    stream run one after another, so elapsed / reps is the per-launch duration
    including the (sub-microsecond) hand-over between consecutive kernels."""
    start, stop = cuda.event(timing=True), cuda.event(timing=True)
    start.record(stream)
    for i in range(reps):
        launch(i)
    stop.record(stream)
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def _cpu_baseline_reduce(a_host, target_seconds=12.0, functor=lambda x, y: x + y):
    """The reference's CPU path for reduce (its simulator: a left fold through the
    Python functor, one call per element, single core by construction), timed on a
    bounded prefix of the same input."""
    from oracle import sim
    red = sim.Reduce(functor)
    probe = a_host[:1 << 18]
    t0 = time.perf_counter()
    red(probe, init=0)
    per_elem = (time.perf_counter() - t0) / probe.size
    n = int(min(a_host.size, max(1 << 18, target_seconds / per_elem)))
    n = 1 << (n.bit_length() - 1)
    sample = a_host[:n]
    t0 = time.perf_counter()
    red(sample, init=0)
    dt = time.perf_counter() - t0
    return {"value": round(sample.nbytes / dt / 1e9, 6), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "left fold over the first 2^%d %s elements, %.1f s" % (n.bit_length() - 1, a_host.dtype.name, dt),
            "elements_per_s": round(n / dt, 1), "host_cores_available": os.cpu_count()}


def _cpu_baseline_transpose(shape, dtype):
    """The simulator's transpose is a NumPy view (no data moves); what a user then
    pays is the materialising copy.  Timed on the 256 x 256 case the configuration
    names, repeated for about a second."""
    from oracle import sim
    a = np.random.default_rng(2).random((256, 256)).astype(dtype)
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 1.0:
        np.ascontiguousarray(sim.transpose(a))
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    return {"value": round(2 * a.nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "256 x 256 %s view + copy, %d repetitions" % (np.dtype(dtype).name, reps),
            "host_cores_available": os.cpu_count()}


def _cpu_baseline_rng(name, nthreads=4096):
    """The simulator's RNG: sequential jump chain, then per-thread draws, all in
    Python over NumPy uint64 scalars, one core.  4096 generators are what the
    configuration names (about 5 s for the chain, 3 s for the draws); the bounded
    baselines of the `others` array use 1024."""
    from oracle import sim
    from oracle.cref import STATE_DTYPE
    states = np.zeros(nthreads, dtype=STATE_DTYPE)
    t0 = time.perf_counter()
    sim.init_states(states, 42)
    t_init = time.perf_counter() - t0
    if name == "rng_init":
        return {"value": round(16 * nthreads / t_init / 1e9, 9), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "%d states, sequential jump chain, %.1f s" % (nthreads, t_init),
                "states_per_s": round(nthreads / t_init, 1), "host_cores_available": os.cpu_count()}
    draw, count, size = ((sim.uniform_float32, 64, 4) if name == "rng_uniform_f32" else (sim.normal_float64, 16, 8))
    t0 = time.perf_counter()
    for t in range(nthreads):
        for _ in range(count):
            draw(states, t)
    dt = time.perf_counter() - t0
    return {"value": round(size * nthreads * count / dt / 1e9, 9), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "%d generators x %d draws, %.1f s (+ %.1f s state init)" % (nthreads, count, dt, t_init),
            "outputs_per_s": round(nthreads * count / dt, 1), "host_cores_available": os.cpu_count()}


def _hypot(a, b):
    return math.sqrt(a * a + b * b)


def _workload(name, cuda, options):
    """-> dict(desc, dtype, algo_bytes, units, step(i), stream, host_input, kernel).  `options`:
    view_cols (transposes: only the first N columns of the matrix, a view with the full
    matrix's row pitches on both sides) and elements (copy_f32: another size)."""
    from numba_cuda_amd import random as nrandom
    from numba_cuda_amd.kernels.transpose import transpose
    stream = cuda.stream()
    add = cuda.Reduce(lambda a, b: a + b)
    mx = cuda.Reduce(lambda a, b: max(a, b))
    rng = np.random.default_rng(1)
    if name.startswith("reduce_"):
        if name == "reduce_f32_functor":
            # a functor without a kernel of its own: translated and compiled at run time
            host = rng.standard_normal(2**28, dtype=np.float32)
            desc = "cuda.reduce fp32 with lambda a, b: sqrt(a*a + b*b) (translated functor), 2^28 elements N(0,1), seed 1"
        elif name == "reduce_f32_sum_reference_order":
            # the same sum with the association order of the reference's kernels: its bits
            host = rng.standard_normal(2**28, dtype=np.float32)
            desc = "cuda.reduce fp32 sum in the reference's association order (bit-identical result), 2^28 elements N(0,1), seed 1"
        elif name == "reduce_f32_sum" or name == "reduce_f32_max":
            host = rng.standard_normal(2**28, dtype=np.float32)
            desc = "cuda.reduce fp32 %s, 2^28 elements N(0,1), seed 1" % ("sum" if name.endswith("sum") else "max")
        elif name == "reduce_f64_sum":
            host = rng.standard_normal(2**27)
            desc = "cuda.reduce fp64 sum, 2^27 elements N(0,1), seed 1"
        elif name == "reduce_i64_sum":
            host = rng.integers(-2**20, 2**20, 2**28, dtype=np.int64, endpoint=True)
            desc = "cuda.reduce int64 sum, 2^28 elements in [-2^20, 2^20], seed 1"
        else:
            raise SystemExit("unknown workload %s" % name)
        # two resident copies, alternated, so no launch can be served from the
        # 256 MB Infinity Cache by its predecessor
        bufs = [cuda.to_device(host), cuda.to_device(host)]
        res = cuda.device_array(1, dtype=host.dtype)
        red = mx if name.endswith("max") else add
        init = -np.inf if name.endswith("max") else 0
        ctype = {"float32": "float", "float64": "double", "int64": "long"}[host.dtype.name]
        kernel = "reduce_kernel<%s, (anonymous namespace)::%s, false>" % (ctype, "OpMax" if name.endswith("max") else "OpAdd")
        if name.endswith("functor"):
            red = cuda.Reduce(_hypot)
            kernel = "nbh_custom_reduce"
        if name.endswith("reference_order"):
            red = cuda.Reduce(lambda a, b: a + b, reference_order=True)
            kernel = "reduce_ordered_kernel<float, (anonymous namespace)::OpAdd, true>"

        def step(i):
            red(bufs[i & 1], res=res, init=init, stream=stream)

        return dict(desc=desc, dtype={"float32": "f32", "float64": "f64", "int64": "int64"}[host.dtype.name],
                    algo_bytes=host.nbytes, units=host.size, step=step, stream=stream, host=host,
                    kernel=kernel, keep=(bufs, res))
    if name.startswith("transpose_"):
        rng = np.random.default_rng(2)
        if name == "transpose_f32":
            host = rng.random((16384, 16384), dtype=np.float32)
        elif name == "transpose_f64":
            host = rng.random((12345, 6789))
        elif name == "transpose_i16":
            host = rng.integers(-32768, 32767, (8192, 32768), dtype=np.int16, endpoint=True)
        else:
            raise SystemExit("unknown workload %s" % name)
        src = cuda.to_device(host).bind(stream)
        dst = cuda.device_array((host.shape[1], host.shape[0]), dtype=host.dtype, stream=stream)
        desc = "transpose %s %dx%d, seed 2" % (host.dtype.name, host.shape[0], host.shape[1])
        moved, items = 2 * host.nbytes, host.size
        view_cols = options.get("view_cols")
        if view_cols:
            # the first columns only, both arrays keeping their pitches: how the time grows with
            # the size of the matrix while everything else stays what it is
            view_cols = min(int(view_cols), host.shape[1])
            src, dst = src[:, :view_cols], dst[:view_cols, :]
            desc += ", columns 0..%d only (row pitches unchanged)" % view_cols
            items = host.shape[0] * view_cols
            moved = 2 * items * host.dtype.itemsize

        def step(i):
            transpose(src, dst)

        return dict(desc=desc,
                    dtype=host.dtype.name, algo_bytes=moved, units=items, step=step,
                    stream=stream, host=None, keep=(src, dst),
                    kernel={"transpose_f32": "transpose_packets<4, true, (anonymous namespace)::ShapeOf<4> >",
                            "transpose_f64": "transpose_sheared<(anonymous namespace)::RingCfg<8, 128, 32, 4, 256, 1, 128> >",
                            "transpose_i16": "transpose_packets<2, true, (anonymous namespace)::ShapeOf<2> >"}[name])
    if name.startswith("rng_"):
        n = 2**24
        states = cuda.device_array(n, dtype=nrandom.xoroshiro128p_dtype)
        nrandom.init_xoroshiro128p_states(states, 42)
        if name == "rng_init":
            def step(i):
                nrandom.init_xoroshiro128p_states(states, 42, 0, stream)
            return dict(desc="create_xoroshiro128p_states 2^24 states, seed 42", dtype="u64",
                        algo_bytes=16 * n, units=n, step=step, stream=stream, host=None,
                        kernel="init_states_tables_kernel", keep=(states,))
        if name == "rng_uniform_f32":
            out = cuda.device_array(n * 64, np.float32)

            def step(i):
                nrandom.xoroshiro128p_fill(states, out, 64, nrandom.UNIFORM, stream)
            return dict(desc="xoroshiro128p 2^24 generators x 64 uniform float32", dtype="u64",
                        algo_bytes=4 * n * 64 + 32 * n, units=n * 64, step=step, stream=stream, host=None,
                        kernel="fill_regs_kernel<(anonymous namespace)::UniformF32>", keep=(states, out))
        if name == "rng_normal_f64":
            out = cuda.device_array(n * 16, np.float64)

            def step(i):
                nrandom.xoroshiro128p_fill(states, out, 16, nrandom.NORMAL, stream)
            return dict(desc="xoroshiro128p 2^24 generators x 16 normal float64", dtype="f64",
                        algo_bytes=8 * n * 16 + 32 * n, units=n * 16, step=step, stream=stream, host=None,
                        kernel="fill_kernel<(anonymous namespace)::NormalF64, true, 1>", keep=(states, out))
    if name == "copy_f32":
        # flat device-to-device assignment: the plain copy kernel of known size that
        # the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are calibrated against
        host = np.random.default_rng(4).random(int(options.get("elements") or 2**28), dtype=np.float32)
        src = cuda.to_device(host)
        dst = cuda.device_array_like(host)
        everything = slice(None)

        def step(i):
            dst.setitem(everything, src, stream=stream)

        return dict(desc="flat copy dst[:] = src, %d float32 (counter calibration)" % host.size, dtype="u8",
                    algo_bytes=2 * host.nbytes, units=host.size, step=step, stream=stream, host=None,
                    kernel="copy_flat<4>", keep=(src, dst))
    if name == "batched_reduce":
        rows, cols = 4096, 65536
        host = np.random.default_rng(3).uniform(-1, 1, (rows, cols)).astype(np.float32)
        dm = cuda.to_device(host)
        out = cuda.device_array(rows, np.float32)
        streams = [cuda.stream() for _ in range(4)]
        views = [dm[i] for i in range(rows)]
        slots = [out[i:i + 1] for i in range(rows)]

        def step(i):
            for r in range(rows):
                add(views[r], res=slots[r], stream=streams[r & 3])
            for s in streams[1:]:
                s.synchronize()

        def extras():
            """Where a call's time goes: the issuing loop alone (no waiting), the same
            4096 launches of this kernel issued through the bare native call with precomputed
            integer arguments on the calling thread - what the runtime's launch path costs per
            call, the floor under any per-call interface on one host thread - and the whole step
            again with the launching threads switched off (every launch made by the caller)."""
            from numba_cuda_amd.cudadrv import driver as drv
            from numba_cuda_amd.kernels import reduction
            cuda.synchronize()
            t0 = time.perf_counter()
            for r in range(rows):
                add(views[r], res=slots[r], stream=streams[r & 3])
            issue = time.perf_counter() - t0
            cuda.synchronize()
            reduction.launch_threads(False)
            try:
                lib, ctx = drv.driver.lib, cuda.current_context()
                entry = lib._reduce_entry
                handles = [s._h for s in streams]      # `_h`: the streams stay inside the package
                scratch = [ctx.reduce_scratch(h) for h in handles]
                init_ptr = reduction._init_buffer(np.dtype(np.float32), 0)
                a, o = dm.gpu_data.device_pointer, out.gpu_data.device_pointer
                args = [(entry, 0, 8, a + r * cols * 4, cols, 4, init_ptr, o + 4 * r, scratch[r & 3][0], scratch[r & 3][1],
                         handles[r & 3]) for r in range(rows)]
                call = drv._hostbuf.call_reduce
                t0 = time.perf_counter()
                for t in args:
                    call(*t)
                floor = time.perf_counter() - t0
                cuda.synchronize()
                step(0)
                cuda.synchronize()
                t0 = time.perf_counter()
                for k in range(3):
                    step(k)
                cuda.synchronize()
                direct = (time.perf_counter() - t0) / (3 * rows)
            finally:
                reduction.launch_threads(True)
            return {"issue_us_per_call": round(issue / rows * 1e6, 3),
                    "native_launch_us_per_call": round(floor / rows * 1e6, 3),
                    "caller_thread_launches_us_per_call": round(direct * 1e6, 3)}

        return dict(desc="4096 x (65536 fp32) row sums round-robin over 4 streams, seed 3", dtype="f32",
                    algo_bytes=host.nbytes, units=rows, step=step, stream=streams[0], host=host,
                    kernel="reduce_kernel<float, (anonymous namespace)::OpAdd, false>", keep=(dm, out, streams, views, slots),
                    calls_per_step=rows,
                    extras=extras)
    raise SystemExit("unknown workload %s" % name)


TRAFFIC_SOURCE = {
    "reduce_f32_sum": "profiles/reduce_kernel_f32_sum_2p28.txt",
    "copy_f32": "profiles/copy_flat_f32_2p28.txt",
    "transpose_f32": "profiles/transpose_packets_f32_16384sq.txt",
    "transpose_i16": "profiles/transpose_packets_f32_16384sq.txt",
    "transpose_f64": "profiles/transpose_sheared_f64_12345x6789.txt",
    "reduce_f32_max": "profiles/reduce_kernel_other_dtypes_and_batched.txt",
    "reduce_f64_sum": "profiles/reduce_kernel_other_dtypes_and_batched.txt",
    "reduce_i64_sum": "profiles/reduce_kernel_other_dtypes_and_batched.txt",
    "reduce_f32_functor": "profiles/reduce_kernel_other_dtypes_and_batched.txt",
    "reduce_f32_sum_reference_order": "profiles/reduce_ordered_kernel_f32_sum_2p28.txt",
    "rng_init": "profiles/xoroshiro_fill_and_init_2p24.txt",
    "rng_uniform_f32": "profiles/xoroshiro_fill_and_init_2p24.txt",
    "rng_normal_f64": "profiles/xoroshiro_fill_and_init_2p24.txt",
}

OTHER_WORKLOADS = ["reduce_f32_max", "reduce_f64_sum", "reduce_i64_sum", "reduce_f32_functor", "reduce_f32_sum_reference_order",
                   "transpose_f32", "transpose_f64",
                   "transpose_i16", "rng_init", "rng_uniform_f32", "rng_normal_f64", "batched_reduce"]


def _cpu_baseline(name, w, seconds):
    if name.startswith("reduce_"):
        is_max = name.endswith("max")
        functor = _hypot if name.endswith("functor") else (lambda x, y: max(x, y)) if is_max else (lambda x, y: x + y)
        return _cpu_baseline_reduce(w["host"], target_seconds=seconds, functor=functor)
    if name == "batched_reduce":
        return _cpu_baseline_reduce(w["host"].reshape(-1), target_seconds=seconds)
    if name.startswith("transpose_"):
        return _cpu_baseline_transpose(None, w["dtype"])
    if name.startswith("rng_"):
        # the sequential jump chain costs about 1.2 ms per generator
        return _cpu_baseline_rng(name, nthreads=4096 if seconds >= 8 else 1024)
    return None


# Workloads whose kernels run long enough and hot enough for the device's power management to
# show: the first launches after an idle spell run fast, the next ones are throttled (up to
# 40 % on the arithmetic-heavy generators) and it takes some fifty launches to settle.  For
# these the line carries both figures: `first10_us_avg`, the ten launches that follow the
# driver's own --warmup, and the settled one (after SETTLE_LAUNCHES more untimed launches),
# which `value` and `roofline` are.
POWER_MANAGED = ("rng_uniform_f32", "rng_normal_f64", "reduce_f32_functor", "reduce_f32_sum_reference_order")
SETTLE_LAUNCHES = 50


def measure(cuda, name, steps, warmup, cpu_seconds, options=None):
    """One workload: `warmup` untimed steps, `steps` timed ones between device-wide
    synchronisations (wall clock -> value), the same number again between a HIP
    event pair on the launch stream (-> roofline), and the CPU baseline beside it
    (cpu_seconds = 0: none)."""
    w = _workload(name, cuda, options or {})
    stream, step = w["stream"], w["step"]
    for i in range(warmup):
        step(i)
    stream.synchronize()
    cuda.synchronize()
    first10 = None
    if name in POWER_MANAGED:
        first10 = _event_timed_launches(cuda, stream, step, 10) * 1e3
        for i in range(SETTLE_LAUNCHES):
            step(i)
        stream.synchronize()
        cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i)
    stream.synchronize()
    cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / steps * 1e3
    gbs = w["algo_bytes"] / (ms_per_step * 1e-3) / 1e9

    roofline = None
    if "calls_per_step" not in w:
        launch_ms = _event_timed_launches(cuda, stream, step, steps)
        achieved = w["algo_bytes"] / (launch_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC.get(name),
                    # `traffic` was not measured in this run: it is the rocprofv3 counter
                    # figure recorded in the named file for this workload
                    "traffic_source": TRAFFIC_SOURCE.get(name),
                    "kernel": w["kernel"], "algorithmic_bytes_per_launch": w["algo_bytes"],
                    "launch_us_avg": round(launch_ms * 1e3, 2), "launches_timed": steps}
        if first10 is not None:
            roofline["first10_us_avg"] = round(first10, 2)
            roofline["settle_launches"] = SETTLE_LAUNCHES
        if options:
            roofline["traffic"] = None          # a view or another size than the counters were taken on
    cpu = _cpu_baseline(name, w, cpu_seconds) if cpu_seconds > 0 else None
    out = {"name": name, "workload": w["desc"], "dtype": w["dtype"], "value": round(gbs, 1), "unit": "GB/s",
           "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 5),
           "pct_of_hbm_peak": round(100 * gbs / HBM_PEAK_GBS, 2),
           "units_per_s": round(w["units"] / (ms_per_step * 1e-3), 1),
           "roofline": roofline, "cpu_baseline": cpu}
    if "calls_per_step" in w:
        out["us_per_call"] = round(ms_per_step * 1e3 / w["calls_per_step"], 3)
    if "extras" in w:
        out.update(w["extras"]())
    return out


def _release_device_memory(cuda):
    import gc
    gc.collect()
    ctx = cuda.current_context()
    ctx.memory_manager.deallocations.clear()
    ctx.deallocations.clear()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default=None,
                    help="measure only this workload (default: the headline workload, then every other "
                         "configuration in an `others` array)")
    ap.add_argument("--view-cols", type=int, default=None,
                    help="transpose workloads: only the first N columns of the matrix (a view; pitches unchanged)")
    ap.add_argument("--elements", type=int, default=None, help="copy_f32: number of float32 items")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-others", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path "
                         "(run with --gpus 1)")

    import numba_cuda_amd as cuda
    if not cuda.is_available():
        raise SystemExit("no GPU / HIP library: %s" % cuda.cuda_error())

    name = args.workload or "reduce_f32_sum"
    options = {k: v for k, v in (("view_cols", args.view_cols), ("elements", args.elements)) if v}
    head = measure(cuda, name, args.steps, args.warmup, 0 if args.no_cpu_baseline else 12.0, options)
    line = {
        "metric": "achieved HBM GB/s (% of 8 TB/s) for cuda.reduce fp32 sum at 2^28 elems"
        if name == "reduce_f32_sum" else "achieved HBM GB/s for " + name,
        "value": head["value"], "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": head["workload"], "name": name},
        "pct_of_hbm_peak": head["pct_of_hbm_peak"], "units_per_s": head["units_per_s"],
        "roofline": head["roofline"], "cpu_baseline": head["cpu_baseline"],
    }
    for key in head:
        if key.endswith("us_per_call"):
            line[key] = head[key]

    if args.workload is None and not args.no_others:
        # every other benchmark configuration, in this same process: fewer steps, and a CPU
        # baseline bounded to about two seconds each
        others = []
        for other in OTHER_WORKLOADS:
            _release_device_memory(cuda)
            steps, warmup = (10, 2) if other == "batched_reduce" else (min(args.steps, 50), min(args.warmup, 5))
            print("bench: %s ..." % other, file=sys.stderr, flush=True)
            others.append(measure(cuda, other, steps, warmup, 0 if args.no_cpu_baseline else 2.0))
        line["others"] = others
        # the same figures once more, compact and LAST on the line, so that a reader who keeps
        # only the end of the line still has every workload: name -> [GB/s, fraction of the HBM
        # peak by the event-timed launches (None: per-call workload), ms per step]
        line["others_summary"] = {o["name"]: [o["value"], (o["roofline"] or {}).get("frac"), o["ms_per_step"]]
                                  for o in [dict(head, name=name)] + others}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
