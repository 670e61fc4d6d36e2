"""StableHLO modules for the five benchmark programs, as text.

On a machine with Julia these modules come out of Reactant itself
(`@code_hlo` / `string(mod)` at the reference's src/compiler/Compiler.jl:1318-1321,
or the `*_pre_xla_compile.mlir` dump of src/mlir/IR/Pass.jl:85-173).  This file
writes the same programs by hand so that the backend can be driven without the
Julia front end.  Conventions followed (reference citations):

* every tensor type carries the Julia dims REVERSED (src/TracedUtils.jl:235-248,
  text sample test/core/buffer_donation.jl:64-72);
* `sum(f.(x))` -> elementwise ops + `stablehlo.reduce ... applies stablehlo.add`
  with init `reduce_empty(+, T) = 0` (src/TracedRArray.jl:128-230, src/Ops.jl:3593-3622);
* range `getindex` -> `stablehlo.slice`, re-embedding -> `stablehlo.pad` or
  `stablehlo.dynamic_update_slice` (src/Indexing.jl:350-445,552-626; src/Ops.jl:739-792);
* `ifelse.(u .> 0, a, b)` -> `compare GT` + `select` (src/Ops.jl:1865-1930);
* `mul!(C, A, B, alpha, beta)` -> dot_general, multiply by splat alpha, multiply C by
  splat beta, add (src/stdlibs/LinearAlgebra.jl:274-332);
* NNlib `gelu_tanh` -> `enzymexla.math.gelu` TANH, lowered to a tanh chain
  (ext/ReactantNNlibExt/Implementations.jl:11-26), softmax -> max/sub/exp/sum/div
  (src/Ops.jl:4537-4546);
* scalars passed with `track_numbers` arrive as 0-d tensors; mutated arguments are
  marked `tf.aliasing_output` (src/compiler/Compiler.jl:1084-1127).
"""
import math

_HDR = ("module @reactant_{name} attributes {{mhlo.num_partitions = 1 : i64, "
        "mhlo.num_replicas = 1 : i64}} {{\n")


def _f(v):
    """Decimal literal that round-trips a float64 (MLIR prints %.6e when exact)."""
    s = "%.6e" % v
    if float(s) == v:
        return s
    return repr(float(v))


def _tt(shape, dt):
    return "tensor<" + "x".join([str(int(s)) for s in shape] + [dt]) + ">"


class _B:
    """Tiny SSA text builder."""

    def __init__(self):
        self.lines = []
        self.k = 0
        self.ck = 0
        self.types = {}

    def new(self, ty, prefix="%"):
        name = "%%%d" % self.k
        self.k += 1
        self.types[name] = ty
        return name

    def const(self, v, shape, dt):
        name = "%%cst_%d" % self.ck if self.ck else "%cst"
        self.ck += 1
        ty = _tt(shape, dt)
        if isinstance(v, str):
            lit = v
        elif dt.startswith("f") or dt == "bf16":
            lit = _f(v)
        else:
            lit = str(int(v))
        self.lines.append("    %s = stablehlo.constant dense<%s> : %s" % (name, lit, ty))
        self.types[name] = ty
        return name

    def un(self, op, x):
        ty = self.types[x]
        r = self.new(ty)
        self.lines.append("    %s = stablehlo.%s %s : %s" % (r, op, x, ty))
        return r

    def bin(self, op, x, y):
        ty = self.types[x]
        r = self.new(ty)
        self.lines.append("    %s = stablehlo.%s %s, %s : %s" % (r, op, x, y, ty))
        return r

    def slice(self, x, shape_in, dt, starts, limits):
        out = [l - s for s, l in zip(starts, limits)]
        ty = _tt(out, dt)
        r = self.new(ty)
        rng = ", ".join("%d:%d" % (s, l) for s, l in zip(starts, limits))
        self.lines.append("    %s = stablehlo.slice %s [%s] : (%s) -> %s"
                          % (r, x, rng, self.types[x], ty))
        return r

    def raw(self, line, name, ty):
        self.lines.append("    " + line)
        self.types[name] = ty

    def text(self):
        return "\n".join(self.lines) + "\n"


# ----------------------------------------------------------------------------
# 1. sinsum_add:  sum(sin.(x) .+ y)
# ----------------------------------------------------------------------------
def sinsum_add(n, dt="f32"):
    t = _tt([n], dt)
    s = _tt([], dt)
    return _HDR.format(name="sinsum_add") + (
            "  func.func @main(%arg0: {t}, %arg1: {t}) -> {s} {{\n"
            "    %cst = stablehlo.constant dense<0.000000e+00> : {s}\n"
            "    %0 = stablehlo.sine %arg0 : {t}\n"
            "    %1 = stablehlo.add %0, %arg1 : {t}\n"
            "    %2 = stablehlo.reduce(%1 init: %cst) applies stablehlo.add across dimensions = [0] : "
            "({t}, {s}) -> {s}\n"
            "    return %2 : {s}\n"
            "  }}\n}}\n").format(t=t, s=s)


# ----------------------------------------------------------------------------
# 2. 3-D diffusion + first-order upwind advection, halo H, `steps` unrolled
# ----------------------------------------------------------------------------
STENCIL_DEFAULTS = dict(dt=0.05, dx=1.0, kappa=1.0)


def stencil(nx, ny, nz, steps=10, halo=3, dt=0.05, dx=1.0, kappa=1.0, embed="pad", elt="f64", loop="unrolled"):
    """c,u,v,w are Julia arrays (nx+2H, ny+2H, nz+2H): raw dims (nz+2H, ny+2H, nx+2H).

    Per step, on the interior:
        lap   = (c[i-1]+c[i+1]+c[j-1]+c[j+1]+c[k-1]+c[k+1] - 6c) * kappa/dx^2
        adv_a = ifelse(a > 0, a*(c - c[-1]), a*(c[+1] - c)) / dx      for a in (u,v,w)
        c_new = c + dt*(lap - (adv_x + adv_y + adv_z))
    and the interior is re-embedded with zero halos (`embed="pad"`) or written over
    the previous field (`embed="dus"`).  `loop="unrolled"` is a plain Julia `for` (the steps are
    traced one after another); `loop="while"` is what `@trace for` gives: one `stablehlo.while`
    carrying a counter and the field (src/Ops.jl:2349-2460).
    """
    H = halo
    full = [nz + 2 * H, ny + 2 * H, nx + 2 * H]
    inner = [nz, ny, nx]
    tf, ti = _tt(full, elt), _tt(inner, elt)
    b = _B()
    for a in ("%arg0", "%arg1", "%arg2", "%arg3"):
        b.types[a] = tf
    zero = b.const(0.0, [], elt)
    six = b.const(6.0, inner, elt)
    kdx2 = b.const(kappa / (dx * dx), inner, elt)
    zi = b.const(0.0, inner, elt)
    rdx = b.const(1.0 / dx, inner, elt)
    dtc = b.const(dt, inner, elt)
    if embed == "dus":
        hidx = b.const(H, [], "i64")

    def sh(x, dz, dy, dx_):
        st = [H + dz, H + dy, H + dx_]
        return b.slice(x, full, elt, st, [s + n for s, n in zip(st, inner)])

    ui, vi, wi = sh("%arg1", 0, 0, 0), sh("%arg2", 0, 0, 0), sh("%arg3", 0, 0, 0)
    def step(c):
        ci = sh(c, 0, 0, 0)
        cxm, cxp = sh(c, 0, 0, -1), sh(c, 0, 0, 1)
        cym, cyp = sh(c, 0, -1, 0), sh(c, 0, 1, 0)
        czm, czp = sh(c, -1, 0, 0), sh(c, 1, 0, 0)
        s = b.bin("add", cxm, cxp)
        s = b.bin("add", s, cym)
        s = b.bin("add", s, cyp)
        s = b.bin("add", s, czm)
        s = b.bin("add", s, czp)
        lap = b.bin("multiply", b.bin("subtract", s, b.bin("multiply", six, ci)), kdx2)
        adv = None
        for vel, cm, cp in ((ui, cxm, cxp), (vi, cym, cyp), (wi, czm, czp)):
            pos = b.new(_tt(inner, "i1"))
            b.lines.append("    %s = stablehlo.compare  GT, %s, %s,  FLOAT : (%s, %s) -> %s"
                           % (pos, vel, zi, ti, ti, _tt(inner, "i1")))
            back = b.bin("multiply", vel, b.bin("subtract", ci, cm))
            fwd = b.bin("multiply", vel, b.bin("subtract", cp, ci))
            sel = b.new(ti)
            b.lines.append("    %s = stablehlo.select %s, %s, %s : %s, %s"
                           % (sel, pos, back, fwd, _tt(inner, "i1"), ti))
            a = b.bin("multiply", sel, rdx)
            adv = a if adv is None else b.bin("add", adv, a)
        cn = b.bin("add", ci, b.bin("multiply", dtc, b.bin("subtract", lap, adv)))
        nc = b.new(tf)
        if embed == "pad":
            b.lines.append("    %s = stablehlo.pad %s, %s, low = [%d, %d, %d], high = [%d, %d, %d], "
                           "interior = [0, 0, 0] : (%s, %s) -> %s"
                           % (nc, cn, zero, H, H, H, H, H, H, ti, _tt([], elt), tf))
        else:
            b.lines.append("    %s = stablehlo.dynamic_update_slice %s, %s, %s, %s, %s : "
                           "(%s, %s, tensor<i64>, tensor<i64>, tensor<i64>) -> %s"
                           % (nc, c, cn, hidx, hidx, hidx, tf, ti, tf))
        return nc

    c = "%arg0"
    if loop == "while":
        ti64 = _tt([], "i64")
        c0, c1, cn_ = b.const(0, [], "i64"), b.const(1, [], "i64"), b.const(steps, [], "i64")
        res = b.new(tf)
        b.lines.append("    %s:2 = stablehlo.while(%%iterArg = %s, %%iterArg_0 = %s) : %s, %s" % (res, c0, c, ti64, tf))
        b.lines.append("     cond {")
        p = b.new(_tt([], "i1"))
        b.lines.append("      %s = stablehlo.compare  LT, %%iterArg, %s,  SIGNED : (%s, %s) -> tensor<i1>" % (p, cn_, ti64, ti64))
        b.lines.append("      stablehlo.return %s : tensor<i1>" % p)
        b.lines.append("    } do {")
        b.types["%iterArg"] = ti64
        b.types["%iterArg_0"] = tf
        inc = b.bin("add", "%iterArg", c1)
        nc = step("%iterArg_0")
        b.lines.append("      stablehlo.return %s, %s : %s, %s" % (inc, nc, ti64, tf))
        b.lines.append("    }")
        c = res + "#1"
    else:
        for _ in range(steps):
            c = step(c)
    return (_HDR.format(name="stencil") +
            "  func.func @main(%%arg0: %s {tf.aliasing_output = 0 : i32}, %%arg1: %s, %%arg2: %s, "
            "%%arg3: %s) -> %s {\n" % (tf, tf, tf, tf, tf) + b.text() +
            "    return %s : %s\n  }\n}\n" % (c, tf))


# ----------------------------------------------------------------------------
# 3. GEMM  C = alpha*A*B + beta*C   (Julia A[m,k], B[k,n], C[m,n])
# ----------------------------------------------------------------------------
def gemm(m, n, k, alpha=1.5, beta=1.2, dt="f32", form="propagated"):
    """Raw buffers: A -> [k][m], B -> [n][k], C -> [n][m]  (dims reversed).

    form="propagated": boundary transposes cancelled by the optimizer, the module
        contracts raw B with raw A:  C_raw[n][m] = B_raw[n][k] . A_raw[k][m].
    form="transposed": `dot_general %A, %B, contracting_dims = [0] x [1]` in Julia
        index order followed by the exit `transpose dims = [1, 0]`.
    """
    ta, tb, tc = _tt([k, m], dt), _tt([n, k], dt), _tt([n, m], dt)
    body = ""
    if form == "propagated":
        body += ("    %0 = stablehlo.dot_general %arg1, %arg0, contracting_dims = [1] x [0], "
                 "precision = [DEFAULT, DEFAULT] : ({tb}, {ta}) -> {tc}\n")
        acc = "%0"
        nxt = 1
    else:
        tj = _tt([m, n], dt)
        body += ("    %0 = stablehlo.dot_general %arg0, %arg1, contracting_dims = [0] x [1], "
                 "precision = [DEFAULT, DEFAULT] : ({ta}, {tb}) -> " + tj + "\n"
                 "    %1 = stablehlo.transpose %0, dims = [1, 0] : (" + tj + ") -> {tc}\n")
        acc = "%1"
        nxt = 2
    body += ("    %{a} = stablehlo.multiply " + acc + ", %cst : {tc}\n"
             "    %{b} = stablehlo.multiply %arg2, %cst_0 : {tc}\n"
             "    %{c} = stablehlo.add %{a}, %{b} : {tc}\n"
             "    return %{c} : {tc}\n").replace("{a}", str(nxt)).replace("{b}", str(nxt + 1)) \
        .replace("{c}", str(nxt + 2))
    head = ("  func.func @main(%arg0: {ta}, %arg1: {tb}, %arg2: {tc} {{tf.aliasing_output = 0 : i32}}) "
            "-> {tc} {{\n"
            "    %cst = stablehlo.constant dense<" + _f(alpha) + "> : {tc}\n"
            "    %cst_0 = stablehlo.constant dense<" + _f(beta) + "> : {tc}\n")
    txt = _HDR.format(name="gemm") + head.format(ta=ta, tb=tb, tc=tc) + \
        body.replace("{ta}", ta).replace("{tb}", tb).replace("{tc}", tc) + "  }\n}\n"
    return txt


# ----------------------------------------------------------------------------
# 4. MLP: dense -> bias -> gelu (x3), softmax over features
# ----------------------------------------------------------------------------
def _gelu_tanh(b, x, shape, dt):
    half = b.const(0.5, shape, dt)
    one = b.const(1.0, shape, dt)
    c0 = b.const(math.sqrt(2.0 / math.pi), shape, dt)
    c1 = b.const(0.044715, shape, dt)
    x3 = b.bin("multiply", b.bin("multiply", x, x), x)
    inner = b.bin("multiply", c0, b.bin("add", x, b.bin("multiply", c1, x3)))
    t = b.un("tanh", inner)
    return b.bin("multiply", b.bin("multiply", half, x), b.bin("add", one, t))


def mlp(batch, widths=(1024, 4096, 4096, 1024), dt="bf16", gelu="chain", softmax=True):
    """x raw [batch][w0]; W_l raw [w_l][w_{l+1}] (Julia W(out,in)); b_l raw [w_{l+1}]."""
    b = _B()
    args = ["%arg0: " + _tt([batch, widths[0]], dt)]
    b.types["%arg0"] = _tt([batch, widths[0]], dt)
    nl = len(widths) - 1
    for l in range(nl):
        tw = _tt([widths[l], widths[l + 1]], dt)
        tb = _tt([widths[l + 1]], dt)
        args.append("%%arg%d: %s" % (1 + 2 * l, tw))
        args.append("%%arg%d: %s" % (2 + 2 * l, tb))
        b.types["%%arg%d" % (1 + 2 * l)] = tw
        b.types["%%arg%d" % (2 + 2 * l)] = tb
    h = "%arg0"
    for l in range(nl):
        shape = [batch, widths[l + 1]]
        ty = _tt(shape, dt)
        d = b.new(ty)
        w, bias = "%%arg%d" % (1 + 2 * l), "%%arg%d" % (2 + 2 * l)
        b.lines.append("    %s = stablehlo.dot_general %s, %s, contracting_dims = [1] x [0], "
                       "precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s"
                       % (d, h, w, b.types[h], b.types[w], ty))
        bb = b.new(ty)
        b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [1] : (%s) -> %s"
                       % (bb, bias, b.types[bias], ty))
        s = b.bin("add", d, bb)
        if gelu == "chain":
            h = _gelu_tanh(b, s, shape, dt)
        else:
            h = b.new(ty)
            b.lines.append('    %s = "enzymexla.math.gelu"(%s) <{gelu_approximation = '
                           '#enzymexla<gelu_approximation TANH>}> : (%s) -> %s' % (h, s, ty, ty))
    shape = [batch, widths[-1]]
    ty = _tt(shape, dt)
    if softmax:
        tr = _tt([batch], dt)
        ninf = b.const("0xFF80" if dt == "bf16" else "0xFF800000", [], dt)
        zero = b.const(0.0, [], dt)
        m = b.new(tr)
        b.lines.append("    %s = stablehlo.reduce(%s init: %s) applies stablehlo.maximum across "
                       "dimensions = [1] : (%s, %s) -> %s" % (m, h, ninf, ty, _tt([], dt), tr))
        mb = b.new(ty)
        b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [0] : (%s) -> %s" % (mb, m, tr, ty))
        e = b.un("exponential", b.bin("subtract", h, mb))
        sm = b.new(tr)
        b.lines.append("    %s = stablehlo.reduce(%s init: %s) applies stablehlo.add across "
                       "dimensions = [1] : (%s, %s) -> %s" % (sm, e, zero, ty, _tt([], dt), tr))
        sb = b.new(ty)
        b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [0] : (%s) -> %s" % (sb, sm, tr, ty))
        h = b.bin("divide", e, sb)
    return (_HDR.format(name="mlp") + "  func.func @main(" + ", ".join(args) + ") -> " + ty + " {\n" +
            b.text() + "    return %s : %s\n  }\n}\n" % (h, ty))


# ----------------------------------------------------------------------------
# 5. FP8 quantized linear + RMSNorm
# ----------------------------------------------------------------------------
def fp8_linear(batch, k, n, eps=1e-6, weight_layout="nk", dot_form="convert"):
    """act raw [batch][k] bf16;  W8 raw [n][k] ("nk": Julia W(k,n), y = W' * x) or
    [k][n] ("kn": Julia W(n,k), y = W * x);  scale_w: tensor<f32>.

    absmax -> scale_a = amax/448 -> q = f8(clamp(x/scale_a, -448, 448)) ->
    acc(f32) = q . W8 -> y = bf16(acc * (scale_a*scale_w)) -> y * rsqrt(mean(y^2) + eps).

    dot_form="convert": both f8 operands are converted to f32 and contracted in f32
        (what `Ops.dot_general` allows, src/Ops.jl:1120,1192: result eltype is the
        promoted operand eltype); "direct": the hlo_call form with f8 operands and an
        f32 result.
    """
    b = _B()
    ta = _tt([batch, k], "bf16")
    tw = _tt([n, k] if weight_layout == "nk" else [k, n], "f8E4M3FN")
    b.types.update({"%arg0": ta, "%arg1": tw, "%arg2": "tensor<f32>"})
    taf = _tt([batch, k], "f32")
    ninf = b.const("0xFF80", [], "bf16")
    ab = b.un("abs", "%arg0")
    amax = b.new("tensor<bf16>")
    b.lines.append("    %s = stablehlo.reduce(%s init: %s) applies stablehlo.maximum across "
                   "dimensions = [0, 1] : (%s, tensor<bf16>) -> tensor<bf16>" % (amax, ab, ninf, ta))
    amf = b.new("tensor<f32>")
    b.lines.append("    %s = stablehlo.convert %s : (tensor<bf16>) -> tensor<f32>" % (amf, amax))
    c448 = b.const(448.0, [], "f32")
    sa = b.bin("divide", amf, c448)
    xf = b.new(taf)
    b.lines.append("    %s = stablehlo.convert %%arg0 : (%s) -> %s" % (xf, ta, taf))
    sab = b.new(taf)
    b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [] : (tensor<f32>) -> %s" % (sab, sa, taf))
    xs = b.bin("divide", xf, sab)
    lo = b.const(-448.0, [], "f32")
    hi = b.const(448.0, [], "f32")
    cl = b.new(taf)
    b.lines.append("    %s = stablehlo.clamp %s, %s, %s : (tensor<f32>, %s, tensor<f32>) -> %s"
                   % (cl, lo, xs, hi, taf, taf))
    ta8 = _tt([batch, k], "f8E4M3FN")
    q = b.new(ta8)
    b.lines.append("    %s = stablehlo.convert %s : (%s) -> %s" % (q, cl, taf, ta8))
    to = _tt([batch, n], "f32")
    rc = "[1] x [1]" if weight_layout == "nk" else "[1] x [0]"
    acc = b.new(to)
    if dot_form == "convert":
        qf = b.new(taf)
        b.lines.append("    %s = stablehlo.convert %s : (%s) -> %s" % (qf, q, ta8, taf))
        twf = tw.replace("f8E4M3FN", "f32")
        wf = b.new(twf)
        b.lines.append("    %s = stablehlo.convert %%arg1 : (%s) -> %s" % (wf, tw, twf))
        b.lines.append("    %s = stablehlo.dot_general %s, %s, contracting_dims = %s, "
                       "precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s" % (acc, qf, wf, rc, taf, twf, to))
    else:
        b.lines.append("    %s = stablehlo.dot_general %s, %%arg1, contracting_dims = %s, "
                       "precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s" % (acc, q, rc, ta8, tw, to))
    sc = b.bin("multiply", sa, "%arg2")
    scb = b.new(to)
    b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [] : (tensor<f32>) -> %s" % (scb, sc, to))
    yf = b.bin("multiply", acc, scb)
    tob = _tt([batch, n], "bf16")
    y = b.new(tob)
    b.lines.append("    %s = stablehlo.convert %s : (%s) -> %s" % (y, yf, to, tob))
    # RMSNorm over features (raw minor dim), math in f32 as Julia's Float32 promotion gives
    y32 = b.new(to)
    b.lines.append("    %s = stablehlo.convert %s : (%s) -> %s" % (y32, y, tob, to))
    sq = b.bin("multiply", y32, y32)
    zero = b.const(0.0, [], "f32")
    tr = _tt([batch], "f32")
    ss = b.new(tr)
    b.lines.append("    %s = stablehlo.reduce(%s init: %s) applies stablehlo.add across "
                   "dimensions = [1] : (%s, tensor<f32>) -> %s" % (ss, sq, zero, to, tr))
    invn = b.const(1.0 / n, [batch], "f32")
    epsc = b.const(eps, [batch], "f32")
    r = b.un("rsqrt", b.bin("add", b.bin("multiply", ss, invn), epsc))
    rb = b.new(to)
    b.lines.append("    %s = stablehlo.broadcast_in_dim %s, dims = [0] : (%s) -> %s" % (rb, r, tr, to))
    o32 = b.bin("multiply", y32, rb)
    o = b.new(tob)
    b.lines.append("    %s = stablehlo.convert %s : (%s) -> %s" % (o, o32, to, tob))
    return (_HDR.format(name="fp8_linear") +
            "  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: tensor<f32>) -> %s {\n" % (ta, tw, tob) +
            b.text() + "    return %s : %s\n  }\n}\n" % (o, tob))
