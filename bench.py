"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms 150] [--workload stencil] [--no-others] [--no-cpu]

Prints ONE JSON line.  The headline workload is the 3-D diffusion/advection stencil,
Float64 512x512x256 with 3-cell halos, 10 timesteps traced into one module.  A "step" is one execution of that module (10 timesteps)
with all inputs resident in HBM; `value` is achieved HBM GB/s counting only the
algorithmic bytes (per timestep: read c,u,v,w + write c over the interior
= 5*512*512*256*8 B).  The kernels advance several timesteps per launch and move those bytes once, so `value` and
`roofline.frac` can exceed the HBM peak; `roofline.frac_physical` is the counter-measured traffic over the peak.  `roofline` describes the dominant kernel (the stencil kernel
that advances two timesteps per launch: its algorithmic bytes are those of both), timed with HIP events on the stream it runs on, inside the timed
region.  `cpu_baseline` times the oracle's C/OpenMP restatement of the stencil on the
host cores (a bounded number of repetitions of the same module, same inputs).  `others` carries the remaining four configs
(sinsum_add, f32 GEMM, bf16 MLP, FP8 linear), each with its own roofline entry, its own `check` against the oracle and
its own `cpu_baseline` (full size, all host cores, at least three repetitions); their step time is the median over five runs of the K plain executions, and the pass with an event pair
on every launch is reported beside it.  Every workload's result is verified after its timed region (`check`):
the stencil bit for bit against the C restatement, the others on sampled rows against float64 / the numpy oracle.
`roofline.traffic` is read from profiles/bench_all_configs_hbm_traffic.txt (rocprofv3 counters) and is null when the
kernel name or launch size there does not match this run's launch list.
Before the W warm-up steps of a workload come untimed executions of it until the device has been under that load for
`--settle-ms` milliseconds (`load_before_warmup_ms` in the line): after an idle period -- compilation, a host-side check, a
CPU baseline -- the first 20 ms or so of a load run up to 20 % slower on this part, whatever the kernel.
`--workload conv|cumsum|maxpool|colsum|transpose` run one of the windowed / layout ops instead, `--workload polybench` /
`polybench_linalg` the reference's polybench stencil and linear-algebra suites (never part of `others`).
"""
import argparse
import importlib
import importlib.util
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# HBM bytes per launch of each kernel as rocprofv3 counted them (FETCH_SIZE / WRITE_SIZE scaled by the readings of a
# plain 1 GiB copy kernel): counters cannot be read from inside this process, so the tracked summary of that profile is
# the one source of the figures.  A row is used only if its kernel name and its launch size (work-items) are the ones
# of this run's launch list; otherwise `traffic` is null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "bench_all_configs_hbm_traffic.txt")
_FULL_SIZE = [True]   # cleared by --small
OPTS = {"check": True, "cpu": True, "settle_ms": 150.0}


def _traffic_table():
    table = {}
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                t = line.split()
                if len(t) == 5 and t[0].startswith("rx_") and t[1].isdigit():
                    table[(t[0], int(t[1]))] = float(t[4]) * 1e6
    except OSError:
        pass
    return table


def _launch_sizes(exe):
    """kernel name -> work-items per launch, from the plan report ("[i] name kind=... grid=AxBxC block=N")."""
    import re
    out = {}
    for m in re.finditer(r"\] (\S+) kind=\S+ grid=(\d+)x(\d+)x(\d+) block=(\d+)", exe.report()):
        out[m.group(1)] = int(m.group(2)) * int(m.group(3)) * int(m.group(4)) * int(m.group(5))
    return out


def _traffic(exe, kernel):
    if not _FULL_SIZE[0]:
        return None
    return _traffic_table().get((kernel, _launch_sizes(exe).get(kernel, -1)))


def _hbm_roofline(exe, kernel, kms, algo_bytes, **extra):
    tr = _traffic(exe, kernel)
    return {"bound": "hbm", "kernel": kernel, **extra, "kernel_ms": kms,
            "achieved": algo_bytes / (kms * 1e-3) / 1e9 if kms else None, "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": algo_bytes / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS if kms else None,
            "traffic": tr,
            # what the memory system actually moved, as a fraction of the HBM peak (counter bytes / kernel time): the
            # physical figure.  `frac` counts algorithmic bytes, which a kernel that advances several timesteps per launch
            # moves only once, so it can exceed 1; it is then flagged
            "frac_physical": tr / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS if (tr and kms) else None,
            "traffic_frac": tr / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS if (tr and kms) else None,
            "frac_above_one": bool(kms and algo_bytes / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS > 1.0)}


PEAK_HBM_GBS = 8000.0
PEAK_TFLOPS = {"f32": 157.3, "bf16": 2500.0, "f8": 5000.0}


def _pkg():
    d = os.path.join(ROOT, "reactant.jl_amd")
    if "reactant_jl_amd" in sys.modules:
        return sys.modules["reactant_jl_amd"]
    spec = importlib.util.spec_from_file_location("reactant_jl_amd", os.path.join(d, "__init__.py"),
                                                  submodule_search_locations=[d])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["reactant_jl_amd"] = mod
    spec.loader.exec_module(mod)
    return mod


def _upload(rx, client, arr, dt):
    return rx.Buffer.from_host(client, arr, dt)


def _time_steps(rx, client, exe, make_args, steps, warmup, carry=None):
    """Run warmup + steps executions.  `make_args(prev_results)` returns (buffers, donated).
    The timed steps are queued without waiting in between; every kernel launch sits between two
    HIP events recorded on the library's stream, read after the final synchronization.
    Returns (seconds for the timed steps, per-launch mean ms over the timed steps, last results)."""
    dev = client.default_device()
    res = None
    # untimed executions until the device has been under this workload for OPTS["settle_ms"] (see _settle), then the W warm-up steps
    t_load = time.perf_counter()
    while OPTS["settle_ms"] > 0 and (time.perf_counter() - t_load) * 1e3 < OPTS["settle_ms"]:
        for _ in range(10):
            bufs, don = make_args(res)
            res = exe.execute_profiled(bufs, don)
        dev.synchronize()
    for _ in range(warmup):
        bufs, don = make_args(res)
        res = exe.execute_profiled(bufs, don)
    dev.synchronize()
    exe.take_timings()
    t0 = time.perf_counter()
    for _ in range(steps):
        bufs, don = make_args(res)
        res = exe.execute_profiled(bufs, don)
    dev.synchronize()
    t1 = time.perf_counter()
    runs, mean_ms = exe.take_timings()
    assert runs == steps
    return t1 - t0, np.asarray(mean_ms), res


def _settle(dev, run_one):
    """Untimed executions until the device has been under the workload for OPTS["settle_ms"] milliseconds.  After an idle
    period (compilation, a host-side check, the CPU baseline of the previous workload) the first 20 ms or so of a load run
    up to 20 % slower on this part, whatever the kernel (a bf16 8192 x 4096 x 4096 product: 246 us per launch 5 ms after the
    start, 201 us from 22 ms on); five warm-up steps of 0.3 ms end inside that window."""
    t0 = time.perf_counter()
    while OPTS["settle_ms"] > 0 and (time.perf_counter() - t0) * 1e3 < OPTS["settle_ms"]:
        for _ in range(10):
            run_one()
        dev.synchronize()


def _time_plain(client, exe, bufs, steps, warmup):
    """K steps as a caller runs them: queued without waiting, no event pair on the launches (a pair
    costs a few microseconds of stream time, which shows on steps of less than 0.1 ms).  The K steps are run five
    times, each run queued whole and timed by the host clock around a synchronization (whose wake-up, some tens of
    microseconds, is spread over the K steps of a run); returns the median of the runs' seconds per step."""
    dev = client.default_device()
    _settle(dev, lambda: exe.execute_sharded(bufs))
    for _ in range(warmup):
        exe.execute_sharded(bufs)
    dev.synchronize()
    times = []
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(steps):
            exe.execute_sharded(bufs)
        dev.synchronize()
        times.append((time.perf_counter() - t0) / steps)
    return float(np.median(times))


def _cpu_threads():
    """Threads numpy's BLAS uses on this host (the GEMM-shaped CPU baselines run on it)."""
    try:
        import threadpoolctl
        n = [i.get("num_threads", 1) for i in threadpoolctl.threadpool_info() if i.get("user_api") == "blas"]
        return int(max(n)) if n else 1
    except Exception:
        return 1


def _timed_reps(fn, budget_s, max_reps):
    """Run fn() until `budget_s` seconds or `max_reps` repetitions; (seconds per repetition, repetitions, last result)."""
    t0, reps, res = time.perf_counter(), 0, None
    while True:
        res = fn()
        reps += 1
        if time.perf_counter() - t0 > budget_s or reps >= max_reps:
            break
    return (time.perf_counter() - t0) / reps, reps, res


def _dominant(launches, mean_ms, kinds):
    """Aggregate the launches whose kind is in `kinds`: (count, mean ms per launch, bytes/launch, flops/launch)."""
    idx = [i for i, l in enumerate(launches) if l["kind"] in kinds]
    if not idx:
        return 0, 0.0, 0.0, 0.0
    ms = float(np.mean([mean_ms[i] for i in idx]))
    b = float(np.mean([launches[i]["algorithmic_bytes"] for i in idx]))
    f = float(np.mean([launches[i]["flops"] for i in idx]))
    return len(idx), ms, b, f


# ----------------------------------------------------------------------------
# workloads
# ----------------------------------------------------------------------------
def _oracle_c():
    try:
        from oracle import build_c
        return build_c, build_c.load()
    except (ImportError, OSError):
        return None, None


def bench_stencil(rx, client, P, steps, warmup, nx=512, ny=512, nz=256, nsteps=10):
    H = 3
    full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
    c = np.zeros(full)
    c[H:-H, H:-H, H:-H] = np.random.default_rng(0).uniform(0, 1, (nz, ny, nx))
    text = P.stencil(nx, ny, nz, steps=nsteps)
    exe = rx.xla_compile(client, text)
    cb = _upload(rx, client, c, "f64")
    host_vel = [np.random.default_rng(s).uniform(-1, 1, full) for s in (1, 2, 3)]
    vel = [_upload(rx, client, a, "f64") for a in host_vel]

    def make_args(prev):
        cur = prev[0] if prev else cb
        return [cur] + vel, [1, 0, 0, 0]   # the tracer field is donated, as `tf.aliasing_output` says

    secs, mean_ms, _ = _time_steps(rx, client, exe, make_args, steps, warmup)
    launches = exe.launches()
    cells = nx * ny * nz
    algo_step = 5.0 * cells * 8 * nsteps
    # the dominant kernel: two timesteps per launch when the steps pair up, else one
    nk, kms, _b, _f = _dominant(launches, mean_ms, ("map_stencil_lds2",))
    per_launch = 2
    if nk == 0:
        nk, kms, _b, _f = _dominant(launches, mean_ms, ("map_stencil_lds", "map_stencil", "map"))
        per_launch = 1
    algo_launch = 5.0 * cells * 8 * per_launch
    res = {
        "workload": "stencil f64 %dx%dx%d halo 3, %d timesteps per module" % (nx, ny, nz, nsteps),
        "ms_per_step": 1e3 * secs / steps,
        "value": algo_step / (secs / steps) / 1e9, "unit": "GB/s", "dtype": "f64",
        "roofline": _hbm_roofline(exe, launches[0]["kernel"], kms, algo_launch, launches_per_step=nk, timesteps_per_launch=per_launch),
        "plan": exe.report(),
    }
    # after the timed region: one module call from the initial field, bit for bit against the C restatement of the
    # same ten timesteps on the same inputs; that CPU run is also the first repetition of the CPU baseline
    build_c, lib = _oracle_c() if (OPTS["check"] or OPTS["cpu"]) else (None, None)
    if lib is not None:
        t0 = time.perf_counter()
        want = build_c.stencil_steps(lib, c, *host_vel, nx, ny, nz, nsteps)
        first = time.perf_counter() - t0
        if OPTS["check"]:
            out = exe.execute_sharded([_upload(rx, client, c, "f64")] + vel)
            got = rx.decode(out[0].synced_buffer().to_host(), "f64").reshape(full)
            res["check"] = {"against": "oracle/stencil_cpu.c, same inputs, %d timesteps" % nsteps, "cells": int(got.size),
                            "bit_exact": bool(np.array_equal(got, want)), "mismatches": int(np.count_nonzero(got != want))}
            del got, out
        if OPTS["cpu"]:
            per, reps, _ = _timed_reps(lambda: build_c.stencil_steps(lib, c, *host_vel, nx, ny, nz, nsteps), 10.0, 9)
            per = (per * reps + first) / (reps + 1)
            res["cpu_baseline"] = {"value": algo_step / per / 1e9, "unit": "GB/s", "cores": int(lib.rx_oracle_threads()), "kind": "port",
                                   "sample": "C restatement of the stencil (oracle/stencil_cpu.c, OpenMP), the GPU run's inputs, full %dx%dx%d grid, "
                                             "%d timesteps per repetition, %d repetitions (%.2f s each)" % (nx, ny, nz, nsteps, reps + 1, per)}
    elif OPTS["check"] or OPTS["cpu"]:
        res["check"] = {"skipped": "oracle/_build/liboracle_c.so is not built"}
        if OPTS["cpu"]:
            res["cpu_baseline"] = cpu_baseline_stencil_numpy(P)
    return res


def bench_sinsum(rx, client, P, steps, warmup, n=1 << 26):
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
    exe = rx.xla_compile(client, P.sinsum_add(n))
    bx, by = _upload(rx, client, x, "f32"), _upload(rx, client, y, "f32")
    secs, mean_ms, res = _time_steps(rx, client, exe, lambda prev: ([bx, by], [0, 0]), steps, warmup)
    launches = exe.launches()
    _, kms, _, _ = _dominant(launches, mean_ms, ("reduce",))
    algo = 8.0 * n
    plain = _time_plain(client, exe, [bx, by], steps, warmup)
    # the step time is that of the plain executions; the pass with an event pair on every launch gives the kernel times
    out = {"workload": "sinsum_add f32[2^26] x2 -> scalar", "ms_per_step": 1e3 * plain,
           "value": algo / plain / 1e9, "unit": "GB/s", "dtype": "f32",
           "with_launch_events": {"ms_per_step": 1e3 * secs / steps, "value": algo / (secs / steps) / 1e9},
           "roofline": _hbm_roofline(exe, launches[0]["kernel"], kms, algo)}
    if OPTS["check"]:
        got = float(rx.decode(res[0].to_host(), "f32"))
        terms = np.sin(x.astype(np.float64)) + y.astype(np.float64)
        exact, mag = float(np.sum(terms)), float(np.sum(np.abs(terms)))
        # f32 accumulation over n terms: within 1e-6 of the sum of magnitudes (far inside the 1e-5 sqrt(n) allowance)
        out["check"] = {"against": "float64 numpy", "got": got, "f64_reference": exact, "err_over_sum_of_magnitudes": abs(got - exact) / mag,
                        "pass": bool(abs(got - exact) <= 1e-6 * mag)}
    if OPTS["cpu"]:
        build_c, lib = _oracle_c()
        if lib is not None:
            per, reps, _ = _timed_reps(lambda: build_c.sinsum_add(lib, x, y), 3.0, 20)
            out["cpu_baseline"] = {"value": algo / per / 1e9, "unit": "GB/s", "cores": int(lib.rx_oracle_threads()), "kind": "port",
                                   "sample": "C restatement (oracle/reduce_cpu.c, OpenMP), full 2^%d vectors, %d repetitions (%.3f s each)"
                                             % (int(np.log2(n)), reps, per)}
        else:
            per, reps, _ = _timed_reps(lambda: float(np.sum(np.sin(x) + y, dtype=np.float64)), 3.0, 5)
            out["cpu_baseline"] = {"value": algo / per / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": "numpy, full vectors, %d repetitions (%.3f s each)" % (reps, per)}
    return out


def _dot_entry(name, exe, secs, steps, mean_ms, dtype_key, dtype, plain=None):
    launches = exe.launches()
    dots = [i for i, l in enumerate(launches) if l["flops"] > 0]
    flops = sum(launches[i]["flops"] for i in dots)
    dms = sum(mean_ms[i] for i in dots)
    big = max(dots, key=lambda i: launches[i]["flops"])
    ach = launches[big]["flops"] / (mean_ms[big] * 1e-3) / 1e12
    # the step time is that of the plain executions; the pass with an event pair on every launch gives the kernel times
    step = plain if plain is not None else secs / steps
    # kernel times come from the pass with an event pair on every launch: compare them with that pass's step time
    extra = {} if plain is None else {"with_launch_events": {"ms_per_step": 1e3 * secs / steps, "value": flops / (secs / steps) / 1e12,
                                                             "kernel_ms_sum": float(np.sum(mean_ms))}}
    return {"workload": name, "ms_per_step": 1e3 * step, "value": flops / step / 1e12,
            "unit": "TFLOP/s", "dtype": dtype, **extra,
            "kernels": [{"kernel": l["kernel"], "kind": l["kind"], "ms": float(m)} for l, m in zip(launches, mean_ms)],
            "dot_tflops_kernel_time_only": flops / (dms * 1e-3) / 1e12,
            # the whole step against the same peak: what a caller gets, epilogues and the launches around the products included
            "whole_step_frac": flops / step / 1e12 / PEAK_TFLOPS[dtype_key],
            "roofline": {"bound": "mfma", "kernel": launches[big]["kernel"], "kernel_ms": float(mean_ms[big]), "timed_in": "with_launch_events",
                         "achieved": ach, "peak": PEAK_TFLOPS[dtype_key], "unit": "TFLOP/s",
                         "frac": ach / PEAK_TFLOPS[dtype_key], "traffic": _traffic(exe, launches[big]["kernel"])}}


def _mfma_ceiling(rx, client, entry, kind):
    """What the MFMA pipe sustains on this device with operands in registers and nothing else running (about 10 ms per
    launch, clock settled under the power limit), beside the published peak: with pseudo-random operands, as a GEMM on
    N(0,1) data toggles the multipliers, and with all-zero operands."""
    try:
        dev = client.default_device()
        tf_r, mhz_r = rx.mfma_ceiling(dev, kind, False)
        tf_z, mhz_z = rx.mfma_ceiling(dev, kind, True)
    except Exception as e:  # report, never hide
        entry["sustained_mfma"] = {"error": str(e)[:200]}
        return
    entry["sustained_mfma"] = {"random_operands": {"TFLOP/s": tf_r, "clock_MHz": mhz_r}, "zero_operands": {"TFLOP/s": tf_z, "clock_MHz": mhz_z},
                               "kernel_frac_of_random": entry["roofline"]["achieved"] / tf_r if tf_r else None}
    # the config's large GEMM kernel with a probe inside (plain scaling epilogue, pseudo-random operands, 150 ms under load
    # before the timed launches): the ratio of the shader-cycle counter to the real-time counter over a sleep of known
    # length in the middle of the K loop (the compute unit of the sleeping wavefront soon idles at a barrier: the chip's
    # clock) and over the workgroups' lifetimes; for bf16 also the ping-pong body that the compiled program runs on, with
    # the same ratio over its compute phases (MFMAs issued back to back: the clock of a compute unit whose pipes are full)
    try:
        entry["gemm_clock_probe"] = rx.gemm_clock_probe(dev, kind)
        if kind == "bf16":
            entry["gemm_clock_probe"]["pingpong_body"] = rx.gemm_clock_probe(dev, "bf16_pingpong")
    except Exception as e:
        entry["gemm_clock_probe"] = {"error": str(e)[:200]}


def _cw_err(got, ref, bound):
    return float(np.max(np.abs(np.asarray(got, np.float64) - np.asarray(ref, np.float64)) / np.maximum(np.asarray(bound, np.float64), 1e-300)))


def bench_gemm(rx, client, P, steps, warmup, n=4096):
    A, B, C = [np.random.default_rng(s).normal(size=(n, n)).astype(np.float32) for s in (0, 1, 2)]
    exe = rx.xla_compile(client, P.gemm(n, n, n))
    bufs = [_upload(rx, client, a, "f32") for a in (A, B, C)]
    secs, mean_ms, res = _time_steps(rx, client, exe, lambda prev: (bufs, [0, 0, 0]), steps, warmup)
    out = _dot_entry("gemm f32 %d^3, alpha=1.5 beta=1.2" % n, exe, secs, steps, mean_ms, "f32", "f32",
                     plain=_time_plain(client, exe, bufs, steps, warmup))
    if OPTS["check"]:
        # buffers are the Julia arrays with dims reversed: C_raw = 1.5 B_raw A_raw + 1.2 C_raw; a sample of rows in float64,
        # every entry against 1e-6 (1.5 |B||A| + 1.2 |C|)
        got = rx.decode(res[0].to_host(), "f32").reshape(n, n)
        pick = np.unique(np.concatenate([np.arange(4), np.linspace(0, n - 1, 56).astype(int), np.arange(n - 4, n)]))
        Bs, A64 = B[pick].astype(np.float64), A.astype(np.float64)
        want = 1.5 * (Bs @ A64) + 1.2 * C[pick].astype(np.float64)
        err = _cw_err(got[pick], want, 1.5 * (np.abs(Bs) @ np.abs(A64)) + 1.2 * np.abs(C[pick]).astype(np.float64))
        out["check"] = {"against": "float64 numpy, %d rows" % len(pick), "componentwise_err": err, "tolerance": 1e-6, "pass": bool(err <= 1e-6)}
    if OPTS["cpu"]:
        per, reps, _ = _timed_reps(lambda: np.float32(1.5) * (B @ A) + np.float32(1.2) * C, 4.0, 10)
        out["cpu_baseline"] = {"value": (2.0 * n ** 3 + 3.0 * n * n) / per / 1e12, "unit": "TFLOP/s", "cores": _cpu_threads(), "kind": "port",
                               "sample": "numpy float32 restatement (OpenBLAS sgemm + axpby), full %d^3, %d repetitions (%.3f s each)" % (n, reps, per)}
    return out


def _rows_args(I, raw, pick, dts):
    """Oracle tensors of the sampled rows of the first operand and of the other operands whole."""
    args = [I.Tensor.from_bytes(np.ascontiguousarray(raw[0][pick]).tobytes(), dts[0], (len(pick),) + raw[0].shape[1:])]
    for a, dt in zip(raw[1:], dts[1:]):
        args.append(I.Tensor.from_bytes(np.ascontiguousarray(a).tobytes(), dt, a.shape))
    return args


def bench_mlp(rx, client, P, steps, warmup, batch=8192, widths=(1024, 4096, 4096, 1024)):
    exe = rx.xla_compile(client, P.mlp(batch, widths))
    raw = [rx.encode(np.random.default_rng(0).normal(size=(batch, widths[0])).astype(np.float32), "bf16")]
    for l in range(len(widths) - 1):
        lim = np.sqrt(6.0 / (widths[l] + widths[l + 1]))
        w = np.random.default_rng(1 + l).uniform(-lim, lim, size=(widths[l], widths[l + 1])).astype(np.float32)
        b = (np.random.default_rng(4 + l).normal(size=(widths[l + 1],)) * 0.01).astype(np.float32)
        raw += [rx.encode(w, "bf16"), rx.encode(b, "bf16")]
    bufs = [_upload(rx, client, a, "bf16") for a in raw]
    secs, mean_ms, res = _time_steps(rx, client, exe, lambda prev: (bufs, [0] * len(bufs)), steps, warmup)
    out = _dot_entry("mlp bf16 batch %d widths %s, bias+gelu, softmax" % (batch, "->".join(map(str, widths))), exe, secs,
                     steps, mean_ms, "bf16", "bf16", plain=_time_plain(client, exe, bufs, steps, warmup))
    _mfma_ceiling(rx, client, out, "bf16")
    if OPTS["check"]:
        # rows are independent: the numpy oracle recomputes a sample of them (float64 accumulation, bf16 rounding where the
        # module stores) for the whole network; then every layer on its own at full size (its GEMM shape with the bias + gelu
        # epilogue, fed the previous layer's output as the GPU computed it): |got - ref|_ij <= 1e-2 (|x| |W| + |b|)_ij on
        # sampled rows, the bound the specification states for a bf16 product
        from oracle import stablehlo_interp as I
        rows = min(256, batch)
        pick = np.linspace(0, batch - 1, rows).astype(int)
        ref = I.run_text(P.mlp(rows, widths), _rows_args(I, raw, pick, ["bf16"] * len(raw)), hifi=True, excess=True)[0].a.astype(np.float64)
        got = rx.decode(res[0].to_host(), "bf16").astype(np.float64).reshape(batch, widths[-1])
        err = float(np.max(np.abs(got[pick] - ref)) / np.max(np.abs(ref)))
        rowsum = float(np.max(np.abs(got.sum(axis=1) - 1.0)))
        lrows = min(64, batch)
        lpick = np.linspace(0, batch - 1, lrows).astype(int)
        layer_err, h_buf, h_raw = [], bufs[0], raw[0]
        for l in range(len(widths) - 1):
            k, n = widths[l], widths[l + 1]
            lexe = rx.xla_compile(client, P.mlp(batch, (k, n), softmax=False))
            lout = lexe.execute_sharded([h_buf, bufs[1 + 2 * l], bufs[2 + 2 * l]])[0].synced_buffer()
            lgot = lout.to_host().reshape(batch, n)
            largs = _rows_args(I, [h_raw, raw[1 + 2 * l], raw[2 + 2 * l]], lpick, ["bf16"] * 3)
            lref = I.run_text(P.mlp(lrows, (k, n), softmax=False), largs, hifi=True, excess=True)[0].a.astype(np.float64)
            xf, wf, bf = [t.a.astype(np.float64) for t in largs]
            layer_err.append(_cw_err(rx.decode(lgot[lpick], "bf16"), lref, np.abs(xf) @ np.abs(wf) + np.abs(bf)[None, :]))
            h_buf, h_raw = lout, lgot
        out["check"] = {"against": "numpy oracle: every layer at full size on %d sampled rows, componentwise against 1e-2 (|x||W| + |b|); the whole network on %d "
                                   "sampled rows; softmax row sums on every row" % (lrows, rows),
                        "layer_componentwise_err": layer_err, "tolerance": 1e-2, "network_max_err_over_max_entry": err, "max_row_sum_deviation": rowsum,
                        "pass": bool(max(layer_err) <= 1e-2 and err <= 2e-2 and rowsum <= 2e-2)}
    if OPTS["cpu"]:
        # single precision on all host cores, full size: operands decoded to float32 before the timed calls; three sgemm
        # (OpenBLAS) + bias + gelu + softmax (oracle/dense_cpu.c, OpenMP)
        build_c, lib = _oracle_c()
        if lib is not None:
            f32 = [rx.decode(a, "bf16").astype(np.float32) for a in raw]
            per, reps, _ = _timed_reps(lambda: build_c.mlp_f32(lib, f32[0], f32[1::2], f32[2::2]), 3.0, 10)
            if reps < 3:
                per, reps, _ = _timed_reps(lambda: build_c.mlp_f32(lib, f32[0], f32[1::2], f32[2::2]), 1e9, 3)
            flops = sum(l["flops"] for l in exe.launches())
            out["cpu_baseline"] = {"value": flops / per / 1e12, "unit": "TFLOP/s", "cores": max(_cpu_threads(), int(lib.rx_oracle_threads())), "kind": "port",
                                   "sample": "float32 restatement at full size (numpy sgemm on OpenBLAS x3, bias + gelu + softmax in oracle/dense_cpu.c with OpenMP; "
                                             "operands decoded to float32 before the timed calls), %d repetitions (%.3f s each)" % (reps, per)}
        else:
            out["cpu_baseline"] = {"skipped": "oracle/_build/liboracle_c.so is not built"}
    return out


def bench_fp8(rx, client, P, steps, warmup, n=8192):
    exe = rx.xla_compile(client, P.fp8_linear(n, n, n))
    act = np.random.default_rng(0).normal(size=(n, n)).astype(np.float32)
    act[0, 0] = 9.0   # the per-tensor absmax sits in a row that the check samples
    a = rx.encode(act, "bf16")
    w = np.random.default_rng(1).normal(size=(n, n)).astype(np.float32)
    sw = np.float32(np.abs(w).max() / 448.0)
    wq = rx.encode(w / sw, "f8E4M3FN")
    del act, w
    bufs = [_upload(rx, client, a, "bf16"), _upload(rx, client, wq, "f8E4M3FN"), _upload(rx, client, np.asarray(sw), "f32")]
    secs, mean_ms, res = _time_steps(rx, client, exe, lambda prev: (bufs, [0, 0, 0]), steps, warmup)
    out = _dot_entry("fp8 linear %d^3 e4m3 per-tensor scales, bf16 out + RMSNorm" % n, exe, secs, steps, mean_ms, "f8",
                     "f8E4M3FN", plain=_time_plain(client, exe, bufs, steps, warmup))
    _mfma_ceiling(rx, client, out, "f8")
    if OPTS["check"]:
        from oracle import stablehlo_interp as I
        rows = min(128, n)
        args = [I.Tensor.from_bytes(np.ascontiguousarray(a[:rows]).tobytes(), "bf16", (rows, n)),
                I.Tensor.from_bytes(np.ascontiguousarray(wq).tobytes(), "f8E4M3FN", (n, n)), I.Tensor(sw, "f32")]
        ref = I.run_text(P.fp8_linear(rows, n, n), args, hifi=True, excess=True)[0].a.astype(np.float64)
        got = rx.decode(res[0].to_host(), "bf16").astype(np.float64).reshape(n, n)
        err = float(np.max(np.max(np.abs(got[:rows] - ref), axis=1) / np.max(np.abs(ref), axis=1)))
        ms = float(np.max(np.abs((got ** 2).mean(axis=1) - 1.0)))
        out["check"] = {"against": "numpy oracle, first %d rows (the absmax is in row 0); RMSNorm mean square on every row" % rows,
                        "max_err_over_row_max": err, "tolerance": 1e-2, "max_mean_square_deviation": ms, "pass": bool(err <= 1e-2 and ms <= 2e-2)}
        del got
    if OPTS["cpu"]:
        # single precision on all host cores, full size: the activations quantized and both operands decoded to float32
        # before the timed calls (e4m3 values and their products are exact in float32); timed: sgemm (OpenBLAS), the
        # dequantizing scale and the row-wise RMSNorm (oracle/dense_cpu.c, OpenMP)
        build_c, lib = _oracle_c()
        if lib is not None:
            a32 = rx.decode(a, "bf16").astype(np.float32)
            sa = np.float32(np.abs(a32).max()) / np.float32(448.0)
            np.divide(a32, sa, out=a32)
            np.clip(a32, -448.0, 448.0, out=a32)
            q = rx.decode(rx.encode(a32, "f8E4M3FN"), "f8E4M3FN").astype(np.float32)
            del a32
            w32 = rx.decode(wq, "f8E4M3FN").astype(np.float32)
            per, reps, _ = _timed_reps(lambda: build_c.fp8_linear_f32(lib, q, w32, sa * sw), 3.0, 5)
            if reps < 3:
                per, reps, _ = _timed_reps(lambda: build_c.fp8_linear_f32(lib, q, w32, sa * sw), 1e9, 3)
            flops = sum(l["flops"] for l in exe.launches())
            out["cpu_baseline"] = {"value": flops / per / 1e12, "unit": "TFLOP/s", "cores": max(_cpu_threads(), int(lib.rx_oracle_threads())), "kind": "port",
                                   "sample": "float32 restatement at full size (numpy sgemm on OpenBLAS, dequantizing scale + RMSNorm in oracle/dense_cpu.c with OpenMP; "
                                             "activations quantized and operands decoded to float32 before the timed calls), %d repetitions (%.3f s each)" % (reps, per)}
        else:
            out["cpu_baseline"] = {"skipped": "oracle/_build/liboracle_c.so is not built"}
    return out


# ----------------------------------------------------------------------------
# windowed ops next to the hot path (not part of the default run: --workload conv|cumsum|maxpool)
# ----------------------------------------------------------------------------
def _window_entry(name, exe, secs, steps, mean_ms, algo_bytes, flops, dtype, bound_kind):
    launches = exe.launches()
    big = int(np.argmax(mean_ms))
    entry = {"workload": name, "ms_per_step": 1e3 * secs / steps, "dtype": dtype,
             "kernels": [{"kernel": l["kernel"], "kind": l["kind"], "ms": float(m)} for l, m in zip(launches, mean_ms)]}
    if flops:
        ach = flops / (secs / steps) / 1e12
        entry.update(value=ach, unit="TFLOP/s")
        dot = [i for i, l in enumerate(launches) if l["flops"] > 0]
        dot.sort(key=lambda i: -float(mean_ms[i]))      # the longest of the launches that multiply
        kms = float(mean_ms[dot[0]]) if dot else float(mean_ms[big])
        kach = (launches[dot[0]]["flops"] if dot else flops) / (kms * 1e-3) / 1e12   # that launch's own flops (a chain has several)
        entry["roofline"] = {"bound": "mfma", "kernel": launches[dot[0] if dot else big]["kernel"], "kernel_ms": kms, "achieved": kach,
                             "peak": PEAK_TFLOPS[bound_kind], "unit": "TFLOP/s", "frac": kach / PEAK_TFLOPS[bound_kind], "traffic": None}
    else:
        entry.update(value=algo_bytes / (secs / steps) / 1e9, unit="GB/s")
        # every launch of these programs is a pass over the data: the roofline is quoted on their sum
        kms = float(np.sum(mean_ms))
        entry["roofline"] = {"bound": "hbm", "kernel": launches[big]["kernel"], "kernel_ms": kms, "achieved": algo_bytes / (kms * 1e-3) / 1e9,
                             "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": algo_bytes / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": None}
    return entry


def bench_conv(rx, client, P, steps, warmup, batch=32, cin=64, cout=64, hw=56):
    """3x3 convolution, padding 1, bias + relu (a VGG/ResNet body layer) in f32."""
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    text, out_shape = NN.convolution([batch, cin, hw, hw], [cout, cin, 3, 3], "f32", padding=[[1, 1], [1, 1]], epilogue="bias_relu")
    exe = rx.xla_compile(client, text)
    rng = np.random.default_rng(0)
    bufs = [_upload(rx, client, rng.normal(size=s).astype(np.float32), "f32") for s in ([batch, cin, hw, hw], [cout, cin, 3, 3], [cout])]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0, 0, 0]), steps, warmup)
    flops = 2.0 * batch * cout * hw * hw * cin * 9
    return _window_entry("conv 3x3 pad 1 f32 %dx%dx%dx%d -> %d features, bias + relu" % (batch, cin, hw, hw, cout), exe, secs, steps, mean_ms,
                         0.0, flops, "f32", "f32")


def bench_conv16(rx, client, P, steps, warmup, batch=32, channels=256, hw=56, layers=3):
    """Three 3x3 convolutions of 256 -> 256 features with bias + relu in bf16 (the body of a VGG block): the products with
    row shifts, the maps between them and the layout maps at both ends."""
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    text, shapes = NN.conv_chain(batch, channels, hw, layers, "bf16")
    exe = rx.xla_compile(client, text)
    rng = np.random.default_rng(0)
    bufs = [_upload(rx, client, rx.encode((rng.normal(size=s) * (0.02 if len(s) == 4 and k > 0 else 1.0)).astype(np.float32), "bf16"), "bf16") for k, s in enumerate(shapes)]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0] * len(bufs)), steps, warmup)
    flops = layers * 2.0 * batch * channels * hw * hw * channels * 9
    return _window_entry("%d x (conv 3x3 pad 1 bf16 %dx%dx%dx%d -> %d features, bias + relu)" % (layers, batch, channels, hw, hw, channels), exe, secs, steps, mean_ms,
                         0.0, flops, "bf16", "bf16")


def bench_vgg11(rx, client, P, steps, warmup, batch=4, dt="f32", hw=224, layers=None, dense=4096):
    """Forward pass of VGG-11 with batch norm in test mode on `batch` images of 224 x 224 (the model and input of
    benchmark/nn/vision.jl:24-34, there in f32 on 4 images): eight 3x3 convolutions + batch norm + relu, five max pools,
    three dense layers; `value` counts the convolutions' and dense layers' flops."""
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    text, shapes, flops = NN.vgg11(batch=batch, hw=hw, dt=dt, layers=layers or NN.VGG11_LAYERS, dense=dense)
    exe = rx.xla_compile(client, text)
    rng = np.random.default_rng(0)
    nconv = sum(1 for l in (layers or NN.VGG11_LAYERS) if l != "M")

    def values(k, s):
        if len(s) == 1 and 0 < k <= 5 * nconv and (k - 1) % 5 == 4:
            return rng.uniform(0.5, 2.0, size=s)                       # running variances
        if len(s) == 4 and k > 0:
            return rng.normal(size=s) * np.sqrt(2.0 / np.prod(s[1:]))
        if len(s) == 2:
            return rng.normal(size=s) * np.sqrt(2.0 / s[0])
        return rng.normal(size=s)
    bufs = [_upload(rx, client, rx.encode(values(k, s).astype(np.float32), dt) if dt != "f32" else values(k, s).astype(np.float32), dt) for k, s in enumerate(shapes)]
    # a step of 24 to 35 launches: timed as a caller runs it; the per-launch times come from a second pass with an event pair on every launch
    plain = _time_plain(client, exe, bufs, steps, warmup)
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0] * len(bufs)), steps, warmup)
    entry = _window_entry("VGG-11 (batch norm, test mode) forward, %s, %d x 3 x %d x %d" % (dt, batch, hw, hw), exe, plain * steps, steps, mean_ms, 0.0, flops, dt, dt)
    entry["with_launch_events"] = {"ms_per_step": 1e3 * secs / steps, "kernel_ms_sum": float(np.sum(mean_ms))}
    entry["roofline"]["timed_in"] = "with_launch_events"
    return entry


def bench_vgg11_bf16(rx, client, P, steps, warmup, batch=32, **kw):
    return bench_vgg11(rx, client, P, steps, warmup, batch=batch, dt="bf16", **kw)


def bench_cumsum(rx, client, P, steps, warmup, n=1 << 26):
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    exe = rx.xla_compile(client, NN.cumulative([n], "f32", 0))
    bufs = [_upload(rx, client, np.random.default_rng(0).normal(size=n).astype(np.float32), "f32")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0]), steps, warmup)
    return _window_entry("cumsum f32[2^%d]" % int(np.log2(n)), exe, secs, steps, mean_ms, 8.0 * n, 0.0, "f32", None)


def bench_maxpool(rx, client, P, steps, warmup, batch=64, c=64, hw=112):
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    text, out_shape = NN.reduce_window([batch, c, hw, hw], "f32", "maximum", [1, 1, 2, 2], strides=[1, 1, 2, 2])
    exe = rx.xla_compile(client, text)
    bufs = [_upload(rx, client, np.random.default_rng(0).normal(size=(batch, c, hw, hw)).astype(np.float32), "f32")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0]), steps, warmup)
    return _window_entry("maxpool 2x2 stride 2 f32 %dx%dx%dx%d" % (batch, c, hw, hw), exe, secs, steps, mean_ms,
                         4.0 * batch * c * hw * hw * 1.25, 0.0, "f32", None)


def bench_colsum(rx, client, P, steps, warmup, n=8192):
    """Column sums of an n x n f32 matrix (a reduction that keeps the minor dimension)."""
    t, o = "tensor<%dx%dxf32>" % (n, n), "tensor<%dxf32>" % n
    text = ("module { func.func @main(%%a: %s) -> %s { %%c = stablehlo.constant dense<0.0> : tensor<f32>\n"
            " %%0 = stablehlo.reduce(%%a init: %%c) applies stablehlo.add across dimensions = [0] : (%s, tensor<f32>) -> %s\n return %%0 : %s } }" % (t, o, t, o, o))
    exe = rx.xla_compile(client, text)
    bufs = [_upload(rx, client, np.random.default_rng(0).normal(size=(n, n)).astype(np.float32), "f32")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0]), steps, warmup)
    return _window_entry("column sums f32 %dx%d" % (n, n), exe, secs, steps, mean_ms, 4.0 * n * n, 0.0, "f32", None)


def bench_transpose(rx, client, P, steps, warmup, n=8192):
    """Transpose of an n x n f32 matrix (a map that reads its input with the two minor roles swapped)."""
    t = "tensor<%dx%dxf32>" % (n, n)
    text = "module { func.func @main(%%a: %s) -> %s { %%0 = stablehlo.transpose %%a, dims = [1, 0] : (%s) -> %s\n return %%0 : %s } }" % (t, t, t, t, t)
    exe = rx.xla_compile(client, text)
    bufs = [_upload(rx, client, np.random.default_rng(0).normal(size=(n, n)).astype(np.float32), "f32")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0]), steps, warmup)
    return _window_entry("transpose f32 %dx%d" % (n, n), exe, secs, steps, mean_ms, 8.0 * n * n, 0.0, "f32", None)


def bench_polybench(rx, client, P, steps, warmup, scale=1):
    """The reference's polybench stencil suite at its own sizes (benchmark/polybench/stencil.jl:71,170,
    229,301; f32, vectorized forms as traced loops): seconds per whole program (all its time steps),
    and the same programs with one launch per update step for comparison.  `value` is array cells
    updated per second over the four programs."""
    PB = importlib.import_module("reactant_jl_amd.polybench_programs")
    rng = np.random.default_rng(0)
    progs, total_cells, total_s = [], 0.0, 0.0
    for name in ("heat_3d", "jacobi_1d", "jacobi_2d", "fdtd_2d"):
        sz = dict(PB.POLYBENCH_SIZES[name])
        for key in ("tsteps", "tmax"):
            if key in sz:
                sz[key] = max(2, sz[key] // scale)
        shapes = {"heat_3d": [(sz.get("n"),) * 3] * 2, "jacobi_1d": [(sz.get("n"),)] * 2, "jacobi_2d": [(sz.get("n"),) * 2] * 2,
                  "fdtd_2d": [(sz.get("ny"), sz.get("nx"))] * 3 + [(sz.get("tmax"),)]}[name]
        trips = sz.get("tsteps", sz.get("tmax"))
        updates = {"heat_3d": 2, "jacobi_1d": 2, "jacobi_2d": 2, "fdtd_2d": 3}[name]
        cells = float(np.prod(shapes[0])) * trips * updates
        text = PB.build(name, **sz)
        bufs = [_upload(rx, client, rng.random(s, dtype=np.float32), "f32") for s in shapes]
        exe = rx.xla_compile(client, text)
        secs = _time_plain(client, exe, bufs, steps, warmup)
        os.environ["RX_CHAIN_STEPS"] = "1"
        try:
            exe1 = rx.xla_compile(client, text)
        finally:
            del os.environ["RX_CHAIN_STEPS"]
        secs1 = _time_plain(client, exe1, bufs, max(2, steps // 2), 1)
        kinds = [l["kind"] for l in exe.launches()]
        progs.append({"program": name, "sizes": sz, "ms": 1e3 * secs, "launches": len(kinds), "chain_kernels": kinds.count("map_chain"),
                      "ms_one_launch_per_step": 1e3 * secs1, "launches_one_per_step": len(exe1.launches()),
                      "Gcells_per_s": cells / secs / 1e9})
        total_cells += cells
        total_s += secs
    return {"workload": "polybench stencils f32 (heat_3d 128^3 x256, jacobi_1d 2048 x1024, jacobi_2d 512^2 x1024, fdtd_2d 1024x2048 x256)",
            "ms_per_step": 1e3 * total_s, "value": total_cells / total_s / 1e9, "unit": "Gcell/s", "dtype": "f32", "programs": progs,
            "roofline": None}


def bench_polybench_linalg(rx, client, P, steps, warmup, scale=1):
    """The BLAS / linear-algebra / data-mining programs of the reference's polybench suite at its sizes
    (benchmark/polybench/blas.jl, linalg_kernels.jl, data_mining.jl; f32, vectorized forms): seconds per
    program.  Matrix-product programs report TFLOP/s of their products, matrix-vector programs GB/s of
    the matrix bytes they must read.  `value` is the suite's total time in ms (lower is better)."""
    PB = importlib.import_module("reactant_jl_amd.polybench_programs")
    rng = np.random.default_rng(0)
    # flops of the products / matrix bytes read once, per program
    def work(name, kw):
        n = kw.get("n", 0)
        if name == "gemm": return 2.0 * n * n * kw["m"], 0
        if name in ("syr2k",): return 4.0 * n ** 3, 0
        if name in ("syrk", "correlation", "covariance"): return 2.0 * n ** 3, 0
        if name == "2mm": return 4.0 * n ** 3, 0
        if name == "3mm": return 2.0 * (kw["p"] * kw["q"] * kw["r"] + kw["r"] * kw["s"] * kw["p"] + kw["p"] * kw["r"] * kw["p"]), 0
        if name == "doitgen": return 2.0 * kw["r"] * kw["q"] * kw["p"] * kw["p"], 0
        if name == "gemver": return 0, 4.0 * n * n * 4        # read A, write Â, read Â twice
        if name == "gesummv": return 0, 2.0 * n * n * 4
        if name == "atax": return 0, 2.0 * n * n * 4
        if name == "bicg": return 0, 2.0 * n * kw["m"] * 4
        if name == "mvt": return 0, 2.0 * n * n * 4
        return 0, 0
    progs, total = [], 0.0
    for name in PB.LINALG_SIZES:
        kw = {k: max(8, v // scale) for k, v in PB.LINALG_SIZES[name].items()}
        text, shapes = PB.linalg(name, **kw)
        bufs = [_upload(rx, client, np.asarray(rng.random(tuple(reversed(s)), dtype=np.float32)), "f32") for s in shapes]
        exe = rx.xla_compile(client, text)
        secs = _time_plain(client, exe, bufs, steps, warmup)
        flops, nbytes = work(name, kw)
        e = {"program": name, "sizes": kw, "ms": 1e3 * secs, "launches": [l["kind"] for l in exe.launches()]}
        if flops:
            e["TFLOP_per_s"] = flops / secs / 1e12
        if nbytes:
            e["GB_per_s"] = nbytes / secs / 1e9
        progs.append(e)
        total += secs
    return {"workload": "polybench BLAS / linear-algebra / data-mining programs f32 at the reference's sizes", "ms_per_step": 1e3 * total,
            "value": 1e3 * total, "unit": "ms", "dtype": "f32", "programs": progs, "roofline": None, "higher_is_better": False}


def cpu_baseline_stencil_numpy(P):
    """Fallback when the C restatement is not built: the numpy interpreter on a smaller grid, one timestep."""
    from oracle import stablehlo_interp as I
    H, nx, ny, nz, nsteps = 3, 256, 256, 128, 1
    full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
    c = np.zeros(full)
    c[H:-H, H:-H, H:-H] = np.random.default_rng(0).uniform(0, 1, (nz, ny, nx))
    args = [I.Tensor(c, "f64")] + [I.Tensor(np.random.default_rng(s).uniform(-1, 1, full), "f64") for s in (1, 2, 3)]
    interp = I.Interpreter(I.parse_module(P.stencil(nx, ny, nz, steps=nsteps)))
    secs, reps, _ = _timed_reps(lambda: interp.run(args), 10.0, 20)
    return {"value": 5.0 * nx * ny * nz * 8 * nsteps / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "numpy oracle, %dx%dx%d interior, %d timestep, %d repetitions (%.2f s each)" % (nx, ny, nz, nsteps, reps, secs)}


def reference_probe():
    """Is the reference itself (Julia + Reactant with its XLA-CPU backend) installed on this host?  If it is, its CPU
    backend could be timed beside these figures; this records what was found."""
    import shutil
    import subprocess
    julia = shutil.which("julia")
    if julia is None:
        return {"julia": None, "reactant": False, "note": "no julia on PATH: the CPU baselines are restatements (kind \"port\"), not Reactant's XLA-CPU backend"}
    try:
        r = subprocess.run([julia, "-e", "using Reactant; print(\"ok\")"], capture_output=True, text=True, timeout=180)
        ok = r.returncode == 0 and "ok" in r.stdout
    except Exception:
        ok = False
    return {"julia": julia, "reactant": ok, "note": "Reactant %s" % ("loads: its CPU backend can be timed with the same programs" if ok else "is not installed")}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="stencil", choices=["stencil", "sinsum", "gemm", "mlp", "fp8", "conv", "conv16", "vgg11", "vgg11_bf16", "cumsum", "maxpool", "colsum", "transpose", "polybench", "polybench_linalg"])
    ap.add_argument("--settle-ms", type=float, default=150.0, help="untimed executions of a workload before its warm-up steps until the device has been under that load this long (0: none)")
    ap.add_argument("--no-others", action="store_true", help="skip the other four configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-check", action="store_true", help="skip the verification of the results after the timed regions (profiling runs)")
    ap.add_argument("--small", action="store_true", help="reduced sizes (debugging only; not a valid result)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend runs on one GPU; --gpus %d is not supported (no collectives, no sharding)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)
    rx = _pkg()
    P = importlib.import_module("reactant_jl_amd.programs")
    client = rx.set_default_backend("gpu")
    table = {"stencil": bench_stencil, "sinsum": bench_sinsum, "gemm": bench_gemm, "mlp": bench_mlp, "fp8": bench_fp8,
             "conv": bench_conv, "conv16": bench_conv16, "vgg11": bench_vgg11, "vgg11_bf16": bench_vgg11_bf16, "cumsum": bench_cumsum, "maxpool": bench_maxpool, "colsum": bench_colsum, "transpose": bench_transpose, "polybench": bench_polybench, "polybench_linalg": bench_polybench_linalg}
    small = {"stencil": dict(nx=128, ny=128, nz=64), "sinsum": dict(n=1 << 22), "gemm": dict(n=1024),
             "mlp": dict(batch=1024, widths=(256, 512, 512, 256)), "fp8": dict(n=1024), "conv": dict(batch=2, hw=28), "conv16": dict(batch=2, channels=64, hw=28), "vgg11": dict(batch=2, hw=32, dense=64), "vgg11_bf16": dict(batch=2, hw=32, dense=64),
             "cumsum": dict(n=1 << 20), "maxpool": dict(batch=4), "colsum": dict(n=1024), "transpose": dict(n=1024), "polybench": dict(scale=16), "polybench_linalg": dict(scale=8)}
    _FULL_SIZE[0] = not args.small
    OPTS["check"], OPTS["cpu"], OPTS["settle_ms"] = not args.no_check, not args.no_cpu, args.settle_ms
    kw = small[args.workload] if args.small else {}
    main_res = table[args.workload](rx, client, P, args.steps, args.warmup, **kw)
    copy_ms = rx._call("RxCalibrationCopy", client.default_device().handle, 1 << 30, 10)
    out = {
        "metric": "achieved HBM GB/s (map/reduce/stencil) + dot_general TFLOP/s, % of peak, 1 GPU",
        "value": main_res["value"], "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "load_before_warmup_ms": args.settle_ms,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": main_res.get("higher_is_better", True), "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic", "config": {"workload": main_res["workload"]},
        "roofline": main_res["roofline"],
        "copy_kernel_GBs": 2.0 * (1 << 30) / (copy_ms * 1e-3) / 1e9 if copy_ms > 0 else None,
    }
    for key in ("check", "cpu_baseline", "whole_step_frac", "sustained_mfma", "gemm_clock_probe", "with_launch_events"):
        if key in main_res:
            out[key] = main_res[key]
    if "kernels" in main_res:
        out["kernels"] = main_res["kernels"]
    if "programs" in main_res:
        out["programs"] = main_res["programs"]
    if not args.no_cpu:
        out.setdefault("cpu_baseline", None)
        out["reference_probe"] = reference_probe()
    if not args.no_others:
        others = []
        for name in ("sinsum", "gemm", "mlp", "fp8", "stencil"):
            if name == args.workload:
                continue
            try:
                r = table[name](rx, client, P, args.steps, args.warmup, **(small[name] if args.small else {}))
                r.pop("plan", None)
                others.append(r)
            except Exception as e:  # report, never hide
                others.append({"workload": name, "error": str(e)[:400]})
        out["others"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
