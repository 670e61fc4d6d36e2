"""TEST INFRASTRUCTURE (oracle).  Builds the C restatements in this directory (stencil_cpu.c, reduce_cpu.c, dense_cpu.c) with gcc
(-O3 -fopenmp -ffp-contract=off, baseline x86-64 so the library runs on any host) into oracle/_build/liboracle_c.so and loads it with ctypes."""
import ctypes
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "_build", "liboracle_c.so")


def build(force=False):
    srcs = [os.path.join(HERE, f) for f in ("stencil_cpu.c", "reduce_cpu.c", "dense_cpu.c")]
    if not force and os.path.exists(SO) and all(os.path.getmtime(SO) >= os.path.getmtime(s) for s in srcs):
        return SO
    os.makedirs(os.path.dirname(SO), exist_ok=True)
    subprocess.check_call(["gcc", "-O3", "-fopenmp", "-ffp-contract=off", "-fPIC", "-shared", "-o", SO] + srcs + ["-lm"])
    return SO


def load():
    """The library, built beforehand (build() is called by __graft_entry__.build())."""
    if not os.path.exists(SO):
        raise ImportError("oracle/_build/liboracle_c.so is not built (run `python -c 'import oracle.build_c as b; b.build()'`)")
    lib = ctypes.CDLL(SO)
    dp = ctypes.POINTER(ctypes.c_double)
    lib.rx_oracle_stencil_step.restype = None
    lib.rx_oracle_stencil_step.argtypes = [dp, dp, dp, dp, dp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                           ctypes.c_double, ctypes.c_double, ctypes.c_double, ctypes.c_int]
    lib.rx_oracle_threads.restype = ctypes.c_int
    fp = ctypes.POINTER(ctypes.c_float)
    lib.rx_oracle_sinsum_add.restype = ctypes.c_double
    lib.rx_oracle_sinsum_add.argtypes = [fp, fp, ctypes.c_longlong]
    ll = ctypes.c_longlong
    lib.rx_oracle_bias_gelu_bf16.restype = None
    lib.rx_oracle_bias_gelu_bf16.argtypes = [fp, fp, ll, ll]
    lib.rx_oracle_softmax_rows_bf16.restype = None
    lib.rx_oracle_softmax_rows_bf16.argtypes = [fp, ll, ll]
    lib.rx_oracle_scale_rmsnorm_bf16.restype = None
    lib.rx_oracle_scale_rmsnorm_bf16.argtypes = [fp, ctypes.c_float, ctypes.c_float, ll, ll]
    return lib


def mlp_f32(lib, x, weights, biases, softmax=True):
    """The dense network of programs.mlp in single precision: x [batch][w0], weights[l] [w_l][w_{l+1}], biases[l] [w_{l+1}],
    all float32 arrays holding bf16 values.  Each layer is numpy's sgemm, then bias + gelu rounded to bf16 (C, OpenMP);
    softmax over the last layer's rows.  Returns float32 [batch][w_last]."""
    import numpy as np
    fp = ctypes.POINTER(ctypes.c_float)
    h = np.ascontiguousarray(x, dtype=np.float32)
    for w, b in zip(weights, biases):
        h = np.ascontiguousarray(h @ w)
        b = np.ascontiguousarray(b, dtype=np.float32)
        lib.rx_oracle_bias_gelu_bf16(h.ctypes.data_as(fp), b.ctypes.data_as(fp), h.shape[0], h.shape[1])
    if softmax:
        lib.rx_oracle_softmax_rows_bf16(h.ctypes.data_as(fp), h.shape[0], h.shape[1])
    return h


def fp8_linear_f32(lib, q, w, scale, eps=1e-6):
    """The product and what follows it in programs.fp8_linear, in single precision: q [batch][k] and w [n][k] are float32
    arrays holding e4m3 values (products of two such values and their sums over k <= 2^16 terms are formed by sgemm in
    float32), scale = scale_a * scale_w.  Returns bf16(rmsnorm(bf16(scale * q w^T))) as float32 [batch][n]."""
    import numpy as np
    fp = ctypes.POINTER(ctypes.c_float)
    h = np.ascontiguousarray(q @ w.T)
    lib.rx_oracle_scale_rmsnorm_bf16(h.ctypes.data_as(fp), ctypes.c_float(float(scale)), ctypes.c_float(float(eps)), h.shape[0], h.shape[1])
    return h


def sinsum_add(lib, x, y):
    """sum(sin.(x) .+ y) over float32 vectors: terms in single precision, summed in double."""
    import numpy as np
    fp = ctypes.POINTER(ctypes.c_float)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.ascontiguousarray(y, dtype=np.float32)
    assert x.shape == y.shape and x.ndim == 1
    return float(lib.rx_oracle_sinsum_add(x.ctypes.data_as(fp), y.ctypes.data_as(fp), x.size))


def stencil_steps(lib, c, u, v, w, nx, ny, nz, steps, halo=3, dt=0.05, dx=1.0, kappa=1.0, embed="pad"):
    """`steps` timesteps on float64 arrays of shape (nz+2H, ny+2H, nx+2H); returns the new field."""
    import numpy as np
    dp = ctypes.POINTER(ctypes.c_double)
    cur = np.ascontiguousarray(c, dtype=np.float64).copy()
    nxt = np.empty_like(cur)
    u, v, w = [np.ascontiguousarray(a, dtype=np.float64) for a in (u, v, w)]
    for _ in range(steps):
        lib.rx_oracle_stencil_step(cur.ctypes.data_as(dp), u.ctypes.data_as(dp), v.ctypes.data_as(dp), w.ctypes.data_as(dp),
                                   nxt.ctypes.data_as(dp), nz, ny, nx, halo, dt, 1.0 / dx, kappa / (dx * dx), 1 if embed == "dus" else 0)
        cur, nxt = nxt, cur
    return cur
