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


# The BLAS / linear-algebra / data-mining programs of the suite (benchmark/polybench/blas.jl,
# linalg_kernels.jl, data_mining.jl) as numpy formulas on arrays indexed like the Julia ones,
# evaluated in float64; arguments in the order of the Julia functions (numbers first where they are).
def _f64(xs):
    return [np.asarray(x, dtype=np.float64) for x in xs]


LINALG_REFERENCE = {
    "gemm": lambda al, be, A, B, C: [al * (A @ B) + be * C],
    "gemver": lambda al, be, u1, u2, v1, v2, A, y, z: (lambda Ah: (lambda x: [Ah, x, al * (Ah @ x)])(be * (Ah.T @ y) + z))(A + np.outer(u1, v1) + np.outer(u2, v2)),
    "gesummv": lambda al, be, A, B, x: [(al * A + be * B) @ x],
    "syr2k": lambda al, be, A, B, C: [al * (A @ B.T) + al * (B @ A.T) + be * C],
    "syrk": lambda al, be, A, C: [al * (A @ A.T) + be * C],
    "2mm": lambda al, be, A, B, C, D: [al * (A @ B @ C) + be * D],
    "3mm": lambda A, B, C, D: [(A @ B) @ (C @ D)],
    "atax": lambda A, x: [A.T @ (A @ x)],
    "bicg": lambda A, p, r: [A.T @ r, A @ p],
    "doitgen": lambda A, x: [np.einsum("rqs,sp->rqp", A, x)],
    "mvt": lambda x1, x2, y1, y2, A: [x1 + A @ y1, x2 + A.T @ y2],
    "covariance": lambda D: (lambda X: [X.T @ X / (D.shape[0] - 1)])(D - D.mean(axis=0, keepdims=True)),
}


def _correlation(D):
    n = D.shape[0]
    X = D - D.mean(axis=0, keepdims=True)
    sig = np.sqrt((X * X).sum(axis=0, keepdims=True))
    sig = np.where(sig <= 0.1, 1.0, sig)
    Xn = X / (sig / np.sqrt(n - 1))
    return [Xn.T @ Xn / (n - 1)]


LINALG_REFERENCE["correlation"] = _correlation

LINALG_SMALL = {
    "gemm": dict(n=96, m=160), "gemver": dict(n=200), "gesummv": dict(n=300), "syr2k": dict(n=128), "syrk": dict(n=130),
    "2mm": dict(n=144), "3mm": dict(p=40, q=72, r=136, s=264), "atax": dict(n=257), "bicg": dict(n=120, m=333),
    "doitgen": dict(r=6, q=10, p=36), "mvt": dict(n=310), "correlation": dict(n=150), "covariance": dict(n=150),
}


def linalg_args(shapes, seed=0):
    """Arguments as Julia arrays (numbers for the 0-d ones), rand(Float32) like the reference's drivers."""
    rng = np.random.default_rng(seed)
    return [np.float32(rng.random()) if s == () else rng.random(s, dtype=np.float32) for s in shapes]


def to_tensor(I, a):
    """Julia array -> the dim-reversed tensor the module takes"""
    a = np.asarray(a, dtype=np.float32)
    return I.tensor(np.ascontiguousarray(a.T) if a.ndim else a, "f32")


def from_tensor(t):
    return np.asarray(t.a).T
