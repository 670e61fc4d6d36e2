"""Loop-nest restatements of the reference's polybench stencils as written in Julia
(benchmark/polybench/stencil.jl: the scalar-loop functions fdtd_2d :8-39, heat_3d :89-124,
jacobi_1d :192-203, jacobi_2d :245-268), on numpy arrays indexed like the Julia arrays, and random
programs made of in-place update steps."""
import importlib

import numpy as np

from _loader import load_pkg

load_pkg()
P = importlib.import_module("reactant_jl_amd.polybench_programs")


def jacobi_1d(tsteps, A, B):
    A, B = A.copy(), B.copy()
    T = A.dtype.type
    for _ in range(tsteps):
        B[1:-1] = T(1 / 3) * ((A[:-2] + A[1:-1]) + A[2:])
        A[1:-1] = T(1 / 3) * ((B[:-2] + B[1:-1]) + B[2:])
    return A, B


def jacobi_2d(tsteps, A, B):
    """A, B indexed [i, j] like the Julia matrices."""
    A, B = A.copy(), B.copy()
    T = A.dtype.type

    def half(X):
        return T(0.2) * ((((X[1:-1, 1:-1] + X[1:-1, :-2]) + X[1:-1, 2:]) + X[2:, 1:-1]) + X[:-2, 1:-1])
    for _ in range(tsteps):
        B[1:-1, 1:-1] = half(A)
        A[1:-1, 1:-1] = half(B)
    return A, B


def heat_3d(tsteps, A, B):
    A, B = A.copy(), B.copy()
    T = A.dtype.type

    def half(X):
        c = X[1:-1, 1:-1, 1:-1]
        return ((T(0.125) * ((X[2:, 1:-1, 1:-1] - T(2) * c) + X[:-2, 1:-1, 1:-1])
                 + T(0.125) * ((X[1:-1, 2:, 1:-1] - T(2) * c) + X[1:-1, :-2, 1:-1]))
                + T(0.125) * ((X[1:-1, 1:-1, 2:] - T(2) * c) + X[1:-1, 1:-1, :-2])) + c
    for _ in range(tsteps):
        B[1:-1, 1:-1, 1:-1] = half(A)
        A[1:-1, 1:-1, 1:-1] = half(B)
    return A, B


def fdtd_2d(EX, EY, HZ, fict):
    EX, EY, HZ = EX.copy(), EY.copy(), HZ.copy()
    T = EX.dtype.type
    for t in range(len(fict)):
        EY[0, :] = fict[t]
        EY[1:, :] = EY[1:, :] - T(0.5) * (HZ[1:, :] - HZ[:-1, :])
        EX[:, 1:] = EX[:, 1:] - T(0.5) * (HZ[:, 1:] - HZ[:, :-1])
        HZ[:-1, :-1] = HZ[:-1, :-1] - T(0.7) * (((EX[:-1, 1:] - EX[:-1, :-1]) + EY[1:, :-1]) - EY[:-1, :-1])
    return HZ


def random_update_program(rng, shape, nfields, nsteps, dt="f32", results=None, self_offsets=False):
    """`nsteps` steps over `nfields` arrays of one shape; each step overwrites a random box of one
    field with a combination of shifted views of the fields (its own only at the same position,
    unless `self_offsets`).  Returns the module text; all fields are arguments, `results` (default:
    all) are returned in their last version."""
    b = P._Loop()
    r = len(shape)
    t = P._tt(shape, dt)
    names = ["%%arg%d" % i for i in range(nfields)]
    for a in names:
        b.types[a] = t
    cur = list(names)
    for _ in range(nsteps):
        fw = int(rng.integers(nfields))
        reach = [int(rng.integers(0, 3)) for _ in range(r)]
        lo = [int(rng.integers(reach[d], max(reach[d] + 1, shape[d] // 3))) for d in range(r)]
        hi = [int(rng.integers(reach[d], max(reach[d] + 1, shape[d] // 3))) for d in range(r)]
        size = [shape[d] - lo[d] - hi[d] for d in range(r)]
        acc = b.view(cur[fw], lo, size)
        for _ in range(int(rng.integers(1, 4))):
            f = int(rng.integers(nfields))
            if f == fw and not self_offsets:
                off = [0] * r
            else:
                off = [int(rng.integers(-reach[d], reach[d] + 1)) for d in range(r)]
            v = b.view(cur[f], [lo[d] + off[d] for d in range(r)], size)
            if dt[0] == "f":
                v = b.bin("multiply", b.const(float(np.float32(rng.uniform(-0.5, 0.5))), size, dt), v)
            acc = b.bin(["add", "subtract"][int(rng.integers(2))], acc, v)
        cur[fw] = b.update(cur[fw], acc, lo)
    results = list(range(nfields)) if results is None else results
    rt = ", ".join([t] * len(results))
    sig = ", ".join("%s: %s" % (a, t) for a in names)
    return (P._HDR.format(name="update_steps") + "  func.func @main(%s) -> %s {\n" % (sig, "(%s)" % rt if len(results) > 1 else rt)
            + b.text() + "    return %s : %s\n  }\n}\n" % (", ".join(cur[i] for i in results), rt))
