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


# ----------------------------------------------------------------------------
# The BLAS, linear-algebra and data-mining programs of the suite in their vectorized forms
# (benchmark/polybench/blas.jl, linalg_kernels.jl, data_mining.jl): matrix products, matrix-vector
# products and broadcasts.  `_J` values are Julia arrays; the tensor behind one has the dims reversed.
# ----------------------------------------------------------------------------
class _J:
    def __init__(self, b, name, shape, dt):
        self.b, self.name, self.shape, self.dt = b, name, tuple(shape), dt

    @property
    def raw(self):
        return list(reversed(self.shape))

    @property
    def ty(self):
        return _tt(self.raw, self.dt)


class _Trace(_B):
    """Writes what the traced array operations of the programs below lower to (src/Ops.jl: dot_general
    :1075-1200, broadcast_in_dim :1320-1357, reduce :3491-3622, transpose, reshape)."""

    def __init__(self, dt):
        super().__init__()
        self.dt = dt
        self.args = []

    def arg(self, shape):
        j = _J(self, "%%arg%d" % len(self.args), shape, self.dt)
        self.types[j.name] = j.ty
        self.args.append(j)
        return j

    def _val(self, shape, line_fmt):
        j = _J(self, None, shape, self.dt)
        j.name = self.new(j.ty)
        self.lines.append("    " + line_fmt.replace("@R@", j.name).replace("@T@", j.ty))
        return j

    def adj(self, a):
        return self._val((a.shape[1], a.shape[0]), "@R@ = stablehlo.transpose %s, dims = [1, 0] : (%s) -> @T@" % (a.name, a.ty))

    def mm(self, a, x):
        """a * x for a matrix a and a matrix or vector x"""
        assert a.shape[1] == x.shape[0]
        if len(x.shape) == 1:
            return self._val((a.shape[0],), "@R@ = stablehlo.dot_general %s, %s, contracting_dims = [0] x [0] : (%s, %s) -> @T@" % (a.name, x.name, a.ty, x.ty))
        return self._val((a.shape[0], x.shape[1]),
                         "@R@ = stablehlo.dot_general %s, %s, contracting_dims = [1] x [0] : (%s, %s) -> @T@" % (x.name, a.name, x.ty, a.ty))

    def _expand(self, a, shape):
        if isinstance(a, (int, float)):
            c = self.const(float(a) if self.dt[0] == "f" else a, list(reversed(shape)), self.dt)
            return _J(self, c, shape, self.dt)
        if a.shape == tuple(shape):
            return a
        rr, ro = len(shape), len(a.shape)
        dims = ", ".join(str(rr - ro + j) for j in range(ro))
        return self._val(shape, "@R@ = stablehlo.broadcast_in_dim %s, dims = [%s] : (%s) -> @T@" % (a.name, dims, a.ty))

    def bc(self, op, x, y):
        """x .op y with Julia's broadcasting (dims aligned from the first one; numbers are splat constants)"""
        sx = () if isinstance(x, (int, float)) else x.shape
        sy = () if isinstance(y, (int, float)) else y.shape
        n = max(len(sx), len(sy))
        px, py = sx + (1,) * (n - len(sx)), sy + (1,) * (n - len(sy))
        shape = tuple(max(p, q) for p, q in zip(px, py))
        xe, ye = self._expand(x, shape), self._expand(y, shape)
        return self._val(shape, "@R@ = stablehlo.%s %s, %s : @T@" % (op, xe.name, ye.name))

    def un(self, op, x):
        return self._val(x.shape, "@R@ = stablehlo.%s %s : @T@" % (op, x.name))

    def sum_dim1(self, x):
        """sum(x; dims=1) of a matrix: 1 x m"""
        zero = self.const(0.0, [], self.dt)
        red = self._val((x.shape[1],), "@R@ = stablehlo.reduce(%s init: %s) applies stablehlo.add across dimensions = [1] : (%s, %s) -> @T@"
                        % (x.name, zero, x.ty, _tt([], self.dt)))
        return self.reshape(red, (1, x.shape[1]))

    def reshape(self, x, shape):
        return self._val(shape, "@R@ = stablehlo.reshape %s : (%s) -> @T@" % (x.name, x.ty))

    def select_le(self, x, bound, then, other):
        """ifelse.(x .<= bound, then, other)"""
        b_ = self._expand(bound, x.shape)
        t_ = self._expand(then, x.shape)
        p = self.new(_tt(x.raw, "i1"))
        self.lines.append("    %s = stablehlo.compare  LE, %s, %s,  FLOAT : (%s, %s) -> %s" % (p, x.name, b_.name, x.ty, x.ty, _tt(x.raw, "i1")))
        return self._val(x.shape, "@R@ = stablehlo.select %s, %s, %s : %s, @T@" % (p, t_.name, other.name, _tt(x.raw, "i1")))

    def scalar_arg(self):
        j = _J(self, "%%arg%d" % len(self.args), (), self.dt)
        self.types[j.name] = j.ty
        self.args.append(j)
        return j

    def module(self, name, results):
        sig = ", ".join("%s: %s" % (a.name, a.ty) for a in self.args)
        rt = ", ".join(r.ty for r in results)
        return (_HDR.format(name=name) + "  func.func @main(%s) -> %s {\n" % (sig, "(%s)" % rt if len(results) > 1 else rt) + self.text()
                + "    return %s : %s\n  }\n}\n" % (", ".join(r.name for r in results), rt))


LINALG_SIZES = {   # benchmark/polybench/blas.jl:27,103,151,195,236; linalg_kernels.jl:46,107,145,184,227,267; data_mining.jl:104
    "gemm": dict(n=2048, m=4096), "gemver": dict(n=2048), "gesummv": dict(n=4096), "syr2k": dict(n=2048), "syrk": dict(n=2048),
    "2mm": dict(n=2048), "3mm": dict(p=256, q=1024, r=2048, s=4096), "atax": dict(n=2048), "bicg": dict(n=2048, m=4096),
    "doitgen": dict(r=256, q=1024, p=512), "mvt": dict(n=4096), "correlation": dict(n=2048), "covariance": dict(n=2048),
}


def linalg(name, dt="f32", **sizes):
    """(module text, Julia shapes of the arguments; () is a number passed as a 0-d tensor) of one program
    of the suite; the argument order is the Julia function's."""
    kw = dict(LINALG_SIZES[name])
    kw.update(sizes)
    t = _Trace(dt)
    g = lambda k: kw[k]
    if name == "gemm":            # α .* A * B .+ β .* C
        al, be = t.scalar_arg(), t.scalar_arg()
        A, B, C = t.arg((g("n"), g("m"))), t.arg((g("m"), g("n"))), t.arg((g("n"), g("n")))
        res = [t.bc("add", t.mm(t.bc("multiply", al, A), B), t.bc("multiply", be, C))]
    elif name == "gemver":        # Â = A .+ u1 .* v1' .+ u2 .* v2'; x = β .* Â' * y .+ z; w = α .* Â * x
        al, be = t.scalar_arg(), t.scalar_arg()
        n = g("n")
        u1, u2, v1, v2 = t.arg((n,)), t.arg((n,)), t.arg((n,)), t.arg((n,))
        A, y, z = t.arg((n, n)), t.arg((n,)), t.arg((n,))
        row = lambda v: t.reshape(v, (1, n))                      # v' of a real vector
        Ah = t.bc("add", t.bc("add", A, t.bc("multiply", u1, row(v1))), t.bc("multiply", u2, row(v2)))
        x = t.bc("add", t.mm(t.bc("multiply", be, t.adj(Ah)), y), z)
        w = t.mm(t.bc("multiply", al, Ah), x)
        res = [Ah, x, w]
    elif name == "gesummv":       # (α .* A .+ β .* B) * x
        al, be = t.scalar_arg(), t.scalar_arg()
        n = g("n")
        A, B, x = t.arg((n, n)), t.arg((n, n)), t.arg((n,))
        res = [t.mm(t.bc("add", t.bc("multiply", al, A), t.bc("multiply", be, B)), x)]
    elif name == "syr2k":         # α .* A * B' + α .* B * A' + β .* C
        al, be = t.scalar_arg(), t.scalar_arg()
        n = g("n")
        A, B, C = t.arg((n, n)), t.arg((n, n)), t.arg((n, n))
        res = [t.bc("add", t.bc("add", t.mm(t.bc("multiply", al, A), t.adj(B)), t.mm(t.bc("multiply", al, B), t.adj(A))), t.bc("multiply", be, C))]
    elif name == "syrk":          # (α .* A * A') + (β .* C)
        al, be = t.scalar_arg(), t.scalar_arg()
        n = g("n")
        A, C = t.arg((n, n)), t.arg((n, n))
        res = [t.bc("add", t.mm(t.bc("multiply", al, A), t.adj(A)), t.bc("multiply", be, C))]
    elif name == "2mm":           # (α .* A * B * C) .+ (β .* D)
        al, be = t.scalar_arg(), t.scalar_arg()
        n = g("n")
        A, B, C, D = (t.arg((n, n)) for _ in range(4))
        res = [t.bc("add", t.mm(t.mm(t.bc("multiply", al, A), B), C), t.bc("multiply", be, D))]
    elif name == "3mm":           # (A * B) * (C * D)
        A, B, C, D = t.arg((g("p"), g("q"))), t.arg((g("q"), g("r"))), t.arg((g("r"), g("s"))), t.arg((g("s"), g("p")))
        res = [t.mm(t.mm(A, B), t.mm(C, D))]
    elif name == "atax":          # A' * (A * x)
        A, x = t.arg((g("n"), g("n"))), t.arg((g("n"),))
        res = [t.mm(t.adj(A), t.mm(A, x))]
    elif name == "bicg":          # (A' * r, A * p)
        A, p, r = t.arg((g("n"), g("m"))), t.arg((g("m"),)), t.arg((g("n"),))
        res = [t.mm(t.adj(A), r), t.mm(A, p)]
    elif name == "doitgen":       # reshape(reshape(A, R * Q, S) * x, R, Q, S)
        A, x = t.arg((g("r"), g("q"), g("p"))), t.arg((g("p"), g("p")))
        res = [t.reshape(t.mm(t.reshape(A, (g("r") * g("q"), g("p"))), x), (g("r"), g("q"), g("p")))]
    elif name == "mvt":           # (x1 .+ A * y1, x2 .+ A' * y2)
        n = g("n")
        x1, x2, y1, y2, A = t.arg((n,)), t.arg((n,)), t.arg((n,)), t.arg((n,)), t.arg((n, n))
        res = [t.bc("add", x1, t.mm(A, y1)), t.bc("add", x2, t.mm(t.adj(A), y2))]
    elif name in ("correlation", "covariance"):
        n = g("n")
        D = t.arg((n, n))
        mu = t.bc("divide", t.sum_dim1(D), float(n))
        X = t.bc("subtract", D, mu)
        if name == "correlation":
            sig = t.un("sqrt", t.sum_dim1(t.bc("multiply", X, X)))
            sig = t.select_le(sig, 0.1, 1.0, sig)
            X = t.bc("divide", X, t.bc("divide", sig, float(np.sqrt(np.float32(n - 1)))))
        res = [t.bc("divide", t.mm(t.adj(X), X), float(n - 1))]
    else:
        raise KeyError(name)
    return t.module(name, res), [a.shape for a in t.args]
