"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload stencil] [--no-others] [--no-cpu]

Prints ONE JSON line.  The headline workload is the 3-D diffusion/advection stencil,
Float64 512x512x256 with 3-cell halos, 10 timesteps traced into one module.  A "step" is one execution of that module (10 timesteps)
with all inputs resident in HBM; `value` is achieved HBM GB/s counting only the
algorithmic bytes (per timestep: read c,u,v,w + write c over the interior
= 5*512*512*256*8 B).  `roofline` describes the dominant kernel (the stencil kernel
that advances two timesteps per launch: its algorithmic bytes are those of both), timed with HIP events on the stream it runs on, inside the timed
region.  `cpu_baseline` times the oracle's C/OpenMP restatement of the stencil on the
host cores (a bounded number of repetitions of the same module).  `others` carries the remaining four configs
(sinsum_add, f32 GEMM, bf16 MLP, FP8 linear), each with its own roofline entry; their step time is that
of plain executions, and the pass with an event pair on every launch is reported beside it.
`--workload conv|cumsum|maxpool` run one of the windowed ops instead, `--workload polybench` /
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

# HBM bytes per launch of each dominant kernel, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and
# scaled by the readings of a plain 1 GiB copy kernel (profiles/bench_all_configs_hbm_traffic.txt).
# Counters cannot be read from inside this process, so the figures of that profile are quoted here;
# they are reported only for the kernel and shape they were measured on.
MEASURED_TRAFFIC_BYTES = {
    "rx_stencil_k0_stencil2m": 3549.6e6,
    "rx_sinsum_add_k0_reduce": 537.1e6,
    "rx_gemm_k0_gemm": 547.5e6,
    "rx_mlp_k1_gemm": 470.1e6,
    "rx_fp8_linear_k2_gemm": 965.7e6,
}
_FULL_SIZE = [True]   # cleared by --small: the table only holds the full-size shapes


def _traffic(kernel):
    return MEASURED_TRAFFIC_BYTES.get(kernel) if _FULL_SIZE[0] else None


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


def _time_plain(client, exe, bufs, steps, warmup):
    """K steps as a caller runs them: queued without waiting, no event pair on the launches (a pair
    costs a few microseconds of stream time, which shows on steps of less than 0.1 ms).  Seconds per step."""
    dev = client.default_device()
    for _ in range(warmup):
        exe.execute_sharded(bufs)
    dev.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        exe.execute_sharded(bufs)
    dev.synchronize()
    return (time.perf_counter() - t0) / steps


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
def bench_stencil(rx, client, P, steps, warmup, nx=512, ny=512, nz=256, nsteps=10):
    H = 3
    full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
    c = np.zeros(full)
    c[H:-H, H:-H, H:-H] = np.random.default_rng(0).uniform(0, 1, (nz, ny, nx))
    text = P.stencil(nx, ny, nz, steps=nsteps)
    exe = rx.xla_compile(client, text)
    cb = _upload(rx, client, c, "f64")
    vel = [_upload(rx, client, np.random.default_rng(s).uniform(-1, 1, full), "f64") for s in (1, 2, 3)]
    del c

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
    return {
        "workload": "stencil f64 %dx%dx%d halo 3, %d timesteps per module" % (nx, ny, nz, nsteps),
        "ms_per_step": 1e3 * secs / steps,
        "value": algo_step / (secs / steps) / 1e9, "unit": "GB/s", "dtype": "f64",
        "roofline": {"bound": "hbm", "kernel": launches[0]["kernel"] if launches else None, "launches_per_step": nk,
                     "timesteps_per_launch": per_launch,
                     "kernel_ms": kms, "achieved": algo_launch / (kms * 1e-3) / 1e9 if kms else None,
                     "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": algo_launch / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS if kms else None,
                     "traffic": _traffic(launches[0]["kernel"]) if launches else None},
        "plan": exe.report(),
    }


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
    got = float(rx.decode(res[0].to_host(), "f32"))
    exact = float(np.sum(np.sin(x.astype(np.float64)) + y.astype(np.float64)))
    # the step time is that of the plain executions; the pass with an event pair on every launch gives the kernel times
    return {"workload": "sinsum_add f32[2^26] x2 -> scalar", "ms_per_step": 1e3 * plain,
            "value": algo / plain / 1e9, "unit": "GB/s", "dtype": "f32",
            "with_launch_events": {"ms_per_step": 1e3 * secs / steps, "value": algo / (secs / steps) / 1e9},
            "check": {"got": got, "f64_reference": exact},
            "roofline": {"bound": "hbm", "kernel": launches[0]["kernel"], "kernel_ms": kms,
                         "achieved": algo / (kms * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                         "frac": algo / (kms * 1e-3) / 1e9 / PEAK_HBM_GBS, "traffic": _traffic(launches[0]["kernel"])}}


def _dot_entry(name, exe, secs, steps, mean_ms, dtype_key, dtype, plain=None):
    launches = exe.launches()
    dots = [i for i, l in enumerate(launches) if l["flops"] > 0]
    flops = sum(launches[i]["flops"] for i in dots)
    dms = sum(mean_ms[i] for i in dots)
    big = max(dots, key=lambda i: launches[i]["flops"])
    ach = launches[big]["flops"] / (mean_ms[big] * 1e-3) / 1e12
    # the step time is that of the plain executions; the pass with an event pair on every launch gives the kernel times
    step = plain if plain is not None else secs / steps
    extra = {} if plain is None else {"with_launch_events": {"ms_per_step": 1e3 * secs / steps, "value": flops / (secs / steps) / 1e12}}
    return {"workload": name, "ms_per_step": 1e3 * step, "value": flops / step / 1e12,
            "unit": "TFLOP/s", "dtype": dtype, **extra,
            "kernels": [{"kernel": l["kernel"], "kind": l["kind"], "ms": float(m)} for l, m in zip(launches, mean_ms)],
            "dot_tflops_kernel_time_only": flops / (dms * 1e-3) / 1e12,
            "roofline": {"bound": "mfma", "kernel": launches[big]["kernel"], "kernel_ms": float(mean_ms[big]),
                         "achieved": ach, "peak": PEAK_TFLOPS[dtype_key], "unit": "TFLOP/s",
                         "frac": ach / PEAK_TFLOPS[dtype_key], "traffic": _traffic(launches[big]["kernel"])}}


def bench_gemm(rx, client, P, steps, warmup, n=4096):
    A, B, C = [np.random.default_rng(s).normal(size=(n, n)).astype(np.float32) for s in (0, 1, 2)]
    exe = rx.xla_compile(client, P.gemm(n, n, n))
    bufs = [_upload(rx, client, a, "f32") for a in (A, B, C)]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0, 0, 0]), steps, warmup)
    return _dot_entry("gemm f32 %d^3, alpha=1.5 beta=1.2" % n, exe, secs, steps, mean_ms, "f32", "f32",
                      plain=_time_plain(client, exe, bufs, steps, warmup))


def bench_mlp(rx, client, P, steps, warmup, batch=8192, widths=(1024, 4096, 4096, 1024)):
    exe = rx.xla_compile(client, P.mlp(batch, widths))
    bufs = [_upload(rx, client, rx.encode(np.random.default_rng(0).normal(size=(batch, widths[0])).astype(np.float32), "bf16"), "bf16")]
    for l in range(len(widths) - 1):
        lim = np.sqrt(6.0 / (widths[l] + widths[l + 1]))
        w = np.random.default_rng(1 + l).uniform(-lim, lim, size=(widths[l], widths[l + 1])).astype(np.float32)
        b = (np.random.default_rng(4 + l).normal(size=(widths[l + 1],)) * 0.01).astype(np.float32)
        bufs += [_upload(rx, client, rx.encode(w, "bf16"), "bf16"), _upload(rx, client, rx.encode(b, "bf16"), "bf16")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0] * len(bufs)), steps, warmup)
    return _dot_entry("mlp bf16 batch %d widths %s, bias+gelu, softmax" % (batch, "->".join(map(str, widths))), exe, secs,
                      steps, mean_ms, "bf16", "bf16", plain=_time_plain(client, exe, bufs, steps, warmup))


def bench_fp8(rx, client, P, steps, warmup, n=8192):
    exe = rx.xla_compile(client, P.fp8_linear(n, n, n))
    a = rx.encode(np.random.default_rng(0).normal(size=(n, n)).astype(np.float32), "bf16")
    w = np.random.default_rng(1).normal(size=(n, n)).astype(np.float32)
    sw = np.float32(np.abs(w).max() / 448.0)
    wq = rx.encode(w / sw, "f8E4M3FN")
    bufs = [_upload(rx, client, a, "bf16"), _upload(rx, client, wq, "f8E4M3FN"), _upload(rx, client, np.asarray(sw), "f32")]
    secs, mean_ms, _ = _time_steps(rx, client, exe, lambda prev: (bufs, [0, 0, 0]), steps, warmup)
    return _dot_entry("fp8 linear %d^3 e4m3 per-tensor scales, bf16 out + RMSNorm" % n, exe, secs, steps, mean_ms, "f8",
                      "f8E4M3FN", plain=_time_plain(client, exe, bufs, steps, warmup))


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
        kms = float(mean_ms[dot[0]]) if dot else float(mean_ms[big])
        kach = flops / (kms * 1e-3) / 1e12
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


def cpu_baseline_stencil(P, nx=512, ny=512, nz=256, nsteps=10):
    """The oracle's C restatement of the stencil (oracle/stencil_cpu.c, OpenMP on all host cores,
    same bits as the GPU result) on the full grid, a bounded number of repetitions of the
    10-timestep module.  If that library was not built, the numpy interpreter on a smaller grid."""
    H = 3
    try:
        from oracle import build_c
        lib = build_c.load()
    except (ImportError, OSError):
        lib = None
    if lib is None:
        from oracle import stablehlo_interp as I
        nx, ny, nz, nsteps = 256, 256, 128, 1
        full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
        c = np.zeros(full)
        c[H:-H, H:-H, H:-H] = np.random.default_rng(0).uniform(0, 1, (nz, ny, nx))
        args = [I.Tensor(c, "f64")] + [I.Tensor(np.random.default_rng(s).uniform(-1, 1, full), "f64") for s in (1, 2, 3)]
        interp = I.Interpreter(I.parse_module(P.stencil(nx, ny, nz, steps=nsteps)))
        t0, reps = time.perf_counter(), 0
        while True:
            interp.run(args)
            reps += 1
            if time.perf_counter() - t0 > 10.0 or reps >= 20:
                break
        secs = (time.perf_counter() - t0) / reps
        return {"value": 5.0 * nx * ny * nz * 8 * nsteps / secs / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "numpy oracle, %dx%dx%d interior, %d timestep, %d repetitions (%.2f s each)" % (nx, ny, nz, nsteps, reps, secs)}
    full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
    c = np.zeros(full)
    c[H:-H, H:-H, H:-H] = np.random.default_rng(0).random((nz, ny, nx))
    u = 2.0 * np.random.default_rng(1).random(full) - 1.0
    v, w = -u, u[::-1].copy()          # timing does not depend on the values; two generators' worth of time saved
    build_c.stencil_steps(lib, c, u, v, w, nx, ny, nz, 1)      # touch every page once
    t0, reps = time.perf_counter(), 0
    while True:
        build_c.stencil_steps(lib, c, u, v, w, nx, ny, nz, nsteps)
        reps += 1
        if time.perf_counter() - t0 > 12.0 or reps >= 10:
            break
    secs = (time.perf_counter() - t0) / reps
    return {"value": 5.0 * nx * ny * nz * 8 * nsteps / secs / 1e9, "unit": "GB/s", "cores": int(lib.rx_oracle_threads()), "kind": "port",
            "sample": "C restatement of the stencil (OpenMP), full %dx%dx%d grid, %d timesteps per repetition, %d repetitions (%.2f s each)"
                      % (nx, ny, nz, nsteps, reps, secs)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="stencil", choices=["stencil", "sinsum", "gemm", "mlp", "fp8", "conv", "cumsum", "maxpool", "polybench", "polybench_linalg"])
    ap.add_argument("--no-others", action="store_true", help="skip the other four configs")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
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
             "conv": bench_conv, "cumsum": bench_cumsum, "maxpool": bench_maxpool, "polybench": bench_polybench, "polybench_linalg": bench_polybench_linalg}
    small = {"stencil": dict(nx=128, ny=128, nz=64), "sinsum": dict(n=1 << 22), "gemm": dict(n=1024),
             "mlp": dict(batch=1024, widths=(256, 512, 512, 256)), "fp8": dict(n=1024), "conv": dict(batch=2, hw=28),
             "cumsum": dict(n=1 << 20), "maxpool": dict(batch=4), "polybench": dict(scale=16), "polybench_linalg": dict(scale=8)}
    _FULL_SIZE[0] = not args.small
    kw = small[args.workload] if args.small else {}
    main_res = table[args.workload](rx, client, P, args.steps, args.warmup, **kw)
    copy_ms = rx._call("RxCalibrationCopy", client.default_device().handle, 1 << 30, 10)
    out = {
        "metric": "achieved HBM GB/s (map/reduce/stencil) + dot_general TFLOP/s, % of peak, 1 GPU",
        "value": main_res["value"], "unit": main_res["unit"], "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"], "higher_is_better": main_res.get("higher_is_better", True), "scaling": "weak", "vs_baseline": None,
        "dtype": main_res["dtype"], "data": "synthetic", "config": {"workload": main_res["workload"]},
        "roofline": main_res["roofline"],
        "copy_kernel_GBs": 2.0 * (1 << 30) / (copy_ms * 1e-3) / 1e9 if copy_ms > 0 else None,
    }
    if "check" in main_res:
        out["check"] = main_res["check"]
    if "kernels" in main_res:
        out["kernels"] = main_res["kernels"]
    if "programs" in main_res:
        out["programs"] = main_res["programs"]
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_stencil(P) if args.workload == "stencil" else None
    if not args.no_others:
        others = []
        for name in ("sinsum", "gemm", "mlp", "fp8", "stencil"):
            if name == args.workload:
                continue
            try:
                r = table[name](rx, client, P, max(3, min(args.steps, 5)), 2, **(small[name] if args.small else {}))
                r.pop("plan", None)
                others.append(r)
            except Exception as e:  # report, never hide
                others.append({"workload": name, "error": str(e)[:400]})
        out["others"] = others
    print(json.dumps(out))


if __name__ == "__main__":
    main()
