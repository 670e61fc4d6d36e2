"""StableHLO text of the reference's polybench stencil suite in its vectorized form
(benchmark/polybench/stencil.jl:41-68 fdtd_2d, :126-167 heat_3d, :205-226 jacobi_1d, :270-298
jacobi_2d): one `stablehlo.while` per program (`@trace track_numbers = false for`, src/Ops.jl:2349-2460)
whose body reads shifted views with `stablehlo.slice` (range `getindex`, src/Indexing.jl:552-626) and
writes the updated interior back with `stablehlo.dynamic_update_slice` at constant starts (range
`setindex!`, src/Indexing.jl:438-443).  Tensors carry the Julia arrays' dims reversed.  No Julia is
available to print the modules, so the text is written from the traced operations; the reference's
sizes are in `POLYBENCH_SIZES`."""
import numpy as np

from .programs import _B, _HDR, _tt

POLYBENCH_SIZES = {
    "heat_3d": dict(n=128, tsteps=256),            # benchmark/polybench/stencil.jl:170
    "jacobi_1d": dict(n=2048, tsteps=1024),        # :229
    "jacobi_2d": dict(n=512, tsteps=1024),         # :301
    "fdtd_2d": dict(nx=1024, ny=2048, tmax=256),   # :71
}


class _Loop(_B):
    """A counted `stablehlo.while` over some carried tensors; `body(b, carried names)` returns the new ones."""

    def loop(self, trips, carried, body):
        ti64 = _tt([], "i64")
        c0, c1, cn = self.const(0, [], "i64"), self.const(1, [], "i64"), self.const(trips, [], "i64")
        res = self.new("")
        names = ["%iterArg"] + ["%%iterArg_%d" % i for i in range(len(carried))]
        tys = [ti64] + [self.types[c] for c in carried]
        self.lines.append("    %s:%d = stablehlo.while(%s) : %s" % (
            res, len(names), ", ".join("%s = %s" % (n, v) for n, v in zip(names, [c0] + list(carried))), ", ".join(tys)))
        self.lines.append("     cond {")
        p = self.new(_tt([], "i1"))
        self.lines.append("      %s = stablehlo.compare  LT, %%iterArg, %s,  SIGNED : (%s, %s) -> tensor<i1>" % (p, cn, ti64, ti64))
        self.lines.append("      stablehlo.return %s : tensor<i1>" % p)
        self.lines.append("    } do {")
        for n, t in zip(names, tys):
            self.types[n] = t
        new = body(self, names[0], names[1:])
        inc = self.bin("add", "%iterArg", c1)
        self.lines.append("      stablehlo.return %s : %s" % (", ".join([inc] + list(new)), ", ".join(tys)))
        self.lines.append("    }")
        return ["%s#%d" % (res, i + 1) for i in range(len(carried))]

    def view(self, x, starts, sizes):
        shape = [int(s) for s in self.types[x][len("tensor<"):-1].split("x")[:-1]]
        dt = self.types[x][len("tensor<"):-1].split("x")[-1]
        return self.slice(x, shape, dt, starts, [s + n for s, n in zip(starts, sizes)])

    def update(self, x, upd, starts):
        idx = [self.const(s, [], "i64") for s in starts]
        r = self.new(self.types[x])
        self.lines.append("    %s = stablehlo.dynamic_update_slice %s, %s, %s : (%s, %s, %s) -> %s" % (
            r, x, upd, ", ".join(idx), self.types[x], self.types[upd], ", ".join(["tensor<i64>"] * len(idx)), self.types[x]))
        return r


def _module(name, b, args, results, aliased=True):
    sig = ", ".join("%s: %s%s" % (a, b.types[a], " {tf.aliasing_output = %d : i32}" % results.index_of[a] if aliased and a in results.index_of else "")
                    for a in args)
    rt = ", ".join(b.types[r.split("#")[0]] if "#" not in r else results.types[r] for r in results.names)
    return (_HDR.format(name=name) + "  func.func @main(%s) -> %s {\n" % (sig, "(%s)" % rt if len(results.names) > 1 else rt)
            + b.text() + "    return %s : %s\n  }\n}\n" % (", ".join(results.names), rt))


class _Results:
    def __init__(self, names, types, index_of):
        self.names, self.types, self.index_of = names, types, index_of


def _star(b, x, inner, center, arms, scale, dt):
    """scale * (sum of the views of `x` at `center` + each offset in `arms`)"""
    acc = None
    for off in arms:
        v = b.view(x, [c + o for c, o in zip(center, off)], inner)
        acc = v if acc is None else b.bin("add", acc, v)
    return b.bin("multiply", b.const(scale, inner, dt), acc)


def jacobi_1d(n, tsteps, dt="f32"):
    """B[2:N-1] = (A[1:N-2] + A[2:N-1] + A[3:N]) / 3, then the same from B into A; returns (A, B)."""
    b = _Loop()
    t = _tt([n], dt)
    b.types["%arg0"] = b.types["%arg1"] = t

    third = 1.0 / 3.0 if dt == "f64" else float(np.float32(1.0 / 3.0))      # T(1 / 3)

    def body(b, _, c):
        A, B = c
        B = b.update(B, _star(b, A, [n - 2], [1], [[-1], [0], [1]], third, dt), [1])
        A = b.update(A, _star(b, B, [n - 2], [1], [[-1], [0], [1]], third, dt), [1])
        return [A, B]

    out = b.loop(tsteps, ["%arg0", "%arg1"], body)
    return _module("jacobi_1d_vectorized", b, ["%arg0", "%arg1"], _Results(out, {out[0]: t, out[1]: t}, {"%arg0": 0, "%arg1": 1}))


def jacobi_2d(n, tsteps, dt="f32"):
    """B interior = 0.2 * (A center + left + right + bottom + top), then the same from B into A."""
    b = _Loop()
    t = _tt([n, n], dt)
    b.types["%arg0"] = b.types["%arg1"] = t
    # Julia A[i, j] is raw [j-1][i-1]; offsets in the order the reference adds them (raw dims)
    arms = [[0, 0], [-1, 0], [1, 0], [0, 1], [0, -1]]

    def body(b, _, c):
        A, B = c
        B = b.update(B, _star(b, A, [n - 2, n - 2], [1, 1], arms, 0.2, dt), [1, 1])
        A = b.update(A, _star(b, B, [n - 2, n - 2], [1, 1], arms, 0.2, dt), [1, 1])
        return [A, B]

    out = b.loop(tsteps, ["%arg0", "%arg1"], body)
    return _module("jacobi_2d_vectorized", b, ["%arg0", "%arg1"], _Results(out, {out[0]: t, out[1]: t}, {"%arg0": 0, "%arg1": 1}))


def heat_3d(n, tsteps, dt="f32"):
    """B interior = sum over the three axes of 0.125 * (A[+1] - 2 A + A[-1]) + A, then the same from B into A."""
    b = _Loop()
    t = _tt([n, n, n], dt)
    b.types["%arg0"] = b.types["%arg1"] = t
    inner = [n - 2] * 3

    def half(b, X):
        ctr = lambda: b.view(X, [1, 1, 1], inner)
        acc = None
        for axis in (2, 1, 0):                               # Julia dims 1, 2, 3 are raw dims 2, 1, 0
            hi, lo = [1, 1, 1], [1, 1, 1]
            hi[axis], lo[axis] = 2, 0
            d = b.bin("subtract", b.view(X, hi, inner), b.bin("multiply", b.const(2.0, inner, dt), ctr()))
            d = b.bin("add", d, b.view(X, lo, inner))
            term = b.bin("multiply", b.const(0.125, inner, dt), d)
            acc = term if acc is None else b.bin("add", acc, term)
        return b.bin("add", acc, ctr())

    def body(b, _, c):
        A, B = c
        B = b.update(B, half(b, A), [1, 1, 1])
        A = b.update(A, half(b, B), [1, 1, 1])
        return [A, B]

    out = b.loop(tsteps, ["%arg0", "%arg1"], body)
    return _module("heat_3d_vectorized", b, ["%arg0", "%arg1"], _Results(out, {out[0]: t, out[1]: t}, {"%arg0": 0, "%arg1": 1}))


def fdtd_2d(nx, ny, tmax, dt="f32"):
    """Per step t: EY[1, :] = fict[t]; EY[2:NX, :] -= 0.5 (HZ[2:NX, :] - HZ[1:NX-1, :]);
    EX[:, 2:NY] -= 0.5 (HZ[:, 2:NY] - HZ[:, 1:NY-1]);
    HZ[1:NX-1, 1:NY-1] -= 0.7 (EX[1:NX-1, 2:NY] - EX[1:NX-1, 1:NY-1] + EY[2:NX, 1:NY-1] - EY[1:NX-1, 1:NY-1]).
    Arguments EX, EY, HZ (raw [NY][NX]) and fict [TMAX]; returns HZ.  `fict[t]` is a dynamic_slice at the
    loop counter (scalar `getindex` inside a traced loop)."""
    b = _Loop()
    t = _tt([ny, nx], dt)
    for a in ("%arg0", "%arg1", "%arg2"):
        b.types[a] = t
    b.types["%arg3"] = _tt([tmax], dt)

    def body(b, i, c):
        EX, EY, HZ = c
        f1 = b.new(_tt([1], dt))
        b.lines.append("    %s = stablehlo.dynamic_slice %%arg3, %s, sizes = [1] : (%s, tensor<i64>) -> %s" % (f1, i, b.types["%arg3"], b.types[f1]))
        col = b.new(_tt([ny, 1], dt))
        b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [1] : (%s) -> %s" % (col, f1, b.types[f1], b.types[col]))
        EY = b.update(EY, col, [0, 0])
        half = lambda shape: b.const(0.5, shape, dt)
        # EY[2:NX, 1:NY]  (raw [:, 1:NX])
        s = [ny, nx - 1]
        d = b.bin("subtract", b.view(HZ, [0, 1], s), b.view(HZ, [0, 0], s))
        EY = b.update(EY, b.bin("subtract", b.view(EY, [0, 1], s), b.bin("multiply", half(s), d)), [0, 1])
        # EX[1:NX, 2:NY]  (raw [1:NY, :])
        s = [ny - 1, nx]
        d = b.bin("subtract", b.view(HZ, [1, 0], s), b.view(HZ, [0, 0], s))
        EX = b.update(EX, b.bin("subtract", b.view(EX, [1, 0], s), b.bin("multiply", half(s), d)), [1, 0])
        # HZ[1:NX-1, 1:NY-1]
        s = [ny - 1, nx - 1]
        d = b.bin("subtract", b.view(EX, [1, 0], s), b.view(EX, [0, 0], s))
        d = b.bin("add", d, b.view(EY, [0, 1], s))
        d = b.bin("subtract", d, b.view(EY, [0, 0], s))
        HZ = b.update(HZ, b.bin("subtract", b.view(HZ, [0, 0], s), b.bin("multiply", b.const(0.7, s, dt), d)), [0, 0])
        return [EX, EY, HZ]

    out = b.loop(tmax, ["%arg0", "%arg1", "%arg2"], body)
    return _module("fdtd_2d_vectorized", b, ["%arg0", "%arg1", "%arg2", "%arg3"], _Results([out[2]], {out[2]: t}, {"%arg2": 0}))


def build(name, dt="f32", **sizes):
    """Module text of one of the four programs, by default at the reference's sizes."""
    kw = dict(POLYBENCH_SIZES[name])
    kw.update(sizes)
    return {"heat_3d": heat_3d, "jacobi_1d": jacobi_1d, "jacobi_2d": jacobi_2d, "fdtd_2d": fdtd_2d}[name](dt=dt, **kw)
