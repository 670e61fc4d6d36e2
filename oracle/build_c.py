"""TEST INFRASTRUCTURE (oracle).  Builds the C restatements in this directory (stencil_cpu.c, reduce_cpu.c) with gcc
(-O3 -fopenmp -ffp-contract=off, baseline x86-64 so the library runs on any host) into oracle/_build/liboracle_c.so and loads it with ctypes."""
import ctypes
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
SO = os.path.join(HERE, "_build", "liboracle_c.so")


def build(force=False):
    srcs = [os.path.join(HERE, f) for f in ("stencil_cpu.c", "reduce_cpu.c")]
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
    return lib


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
