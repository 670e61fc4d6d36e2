"""GPU parity of the five benchmark programs at sizes the oracle finishes in
seconds.  Tolerances are the ones the project states: integers bit-exact, fp32
maps 1e-6 relative, fp32 reductions 1e-5*sqrt(n) relative, bf16/fp8 contractions
1e-2 relative to an f32/f64-accumulated reference."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run, max_rel_to_scale, contraction_err, abs_args
from _loader import load_programs
from oracle import stablehlo_interp as I

pytestmark = pytest.mark.gpu
P = load_programs()


@pytest.mark.parametrize("n", [1, 7, 64, 1000, 4096, 1 << 20])
def test_sinsum_add(rx, client, n):
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
    args = [I.Tensor(x, "f32"), I.Tensor(y, "f32")]
    text = P.sinsum_add(n)
    got, _ = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True)
    exact = np.sum(np.sin(x.astype(np.float64)) + y.astype(np.float64))
    scale = np.sum(np.abs(np.sin(x.astype(np.float64)) + y.astype(np.float64)))
    # fp32 reduction: 1e-5*sqrt(n) relative (to the magnitude of the summands)
    tol = 1e-5 * np.sqrt(n)
    assert abs(float(got[0].a) - exact) <= tol * max(scale / max(n, 1), abs(exact), 1e-6) + 1e-6 * scale / np.sqrt(n)
    assert abs(float(ref[0].a) - exact) <= tol * max(abs(exact), 1e-6) + 1e-6 * scale


def test_sinsum_add_single_launch_reduction(rx, client, monkeypatch):
    """The one-launch form of the full reduction (last workgroup combines) gives the same bits as
    the two-launch form: partials are combined in the same order."""
    n = 1 << 20
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
    args = [I.Tensor(x, "f32"), I.Tensor(y, "f32")]
    two, exe2 = gpu_run(rx, client, P.sinsum_add(n), args)
    monkeypatch.setenv("RX_SINGLE_PASS_REDUCE", "1")
    one, exe1 = gpu_run(rx, client, P.sinsum_add(n), args)
    assert len(exe1.launches()) == 1 and len(exe2.launches()) == 2
    for _ in range(3):      # the slots are back at zero after every run
        again, _ = gpu_run(rx, client, P.sinsum_add(n), args, exe=exe1)
        assert again[0].a.tobytes() == one[0].a.tobytes()
    assert one[0].a.tobytes() == two[0].a.tobytes()


@pytest.mark.parametrize("dt,op,init", [("f64", "add", "0.000000e+00"), ("i32", "maximum", "-2147483648"), ("i64", "add", "0"),
                                        ("bf16", "minimum", "0x7F80")])
def test_single_launch_reduction_of_other_types(rx, client, monkeypatch, dt, op, init):
    """Partials of 8 bytes travel as two flagged words, narrower ones as one: same bits as the two-launch form, run after run."""
    shape = (1500, 700)      # not a whole number of workgroup tiles
    text = ("module {\n  func.func @main(%%arg0: tensor<1500x700x%s>) -> tensor<%s> {\n"
            "    %%c = stablehlo.constant dense<%s> : tensor<%s>\n"
            "    %%0 = stablehlo.reduce(%%arg0 init: %%c) applies stablehlo.%s across dimensions = [0, 1] : (tensor<1500x700x%s>, tensor<%s>) -> tensor<%s>\n"
            "    return %%0 : tensor<%s>\n  }\n}\n" % (dt, dt, init, dt, op, dt, dt, dt, dt))
    rng = np.random.default_rng(4)
    a = I.tensor(rng.integers(-1000, 1000, shape) if dt.startswith("i") else rng.normal(size=shape), dt)
    two, exe2 = gpu_run(rx, client, text, [a])
    monkeypatch.setenv("RX_SINGLE_PASS_REDUCE", "1")
    one, exe1 = gpu_run(rx, client, text, [a])
    assert len(exe1.launches()) == 1 and len(exe2.launches()) == 2
    assert one[0].a.tobytes() == two[0].a.tobytes()
    for _ in range(2):
        again, _ = gpu_run(rx, client, text, [a], exe=exe1)
        assert again[0].a.tobytes() == one[0].a.tobytes()
    ref = oracle_run(text, [a])
    if dt.startswith("i") or op != "add":
        assert one[0].a.tobytes() == ref[0].a.tobytes()
    else:
        assert abs(float(one[0].a) - float(ref[0].a)) <= 1e-9 * np.sum(np.abs(np.asarray(a.a, dtype=np.float64)))


@pytest.mark.parametrize("shape,embed", [((6, 5, 4), "pad"), ((6, 5, 4), "dus"), ((32, 16, 8), "pad"),
                                         ((64, 64, 32), "pad")])
def test_stencil(rx, client, shape, embed):
    nx, ny, nz = shape
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(0)
    c = np.zeros(full)
    c[3:-3, 3:-3, 3:-3] = rng.uniform(0, 1, (nz, ny, nx))
    u, v, w = [np.random.default_rng(s).uniform(-1, 1, full) for s in (1, 2, 3)]
    args = [I.Tensor(a, "f64") for a in (c, u, v, w)]
    text = P.stencil(nx, ny, nz, steps=3, embed=embed)
    got, _ = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args)
    # add/mul chains evaluated in the module's order with contraction off: bit-exact
    assert np.array_equal(got[0].a, ref[0].a)


def _stencil_case(rx, client, shape, embed, steps, elt="f64"):
    nx, ny, nz = shape
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(0)
    c = np.zeros(full)
    c[3:-3, 3:-3, 3:-3] = rng.uniform(0, 1, (nz, ny, nx))
    u, v, w = [np.random.default_rng(s).uniform(-1, 1, full) for s in (1, 2, 3)]
    if elt == "f32":
        c, u, v, w = [a.astype(np.float32) for a in (c, u, v, w)]
    args = [I.Tensor(a, elt) for a in (c, u, v, w)]
    text = P.stencil(nx, ny, nz, steps=steps, embed=embed, elt=elt)
    got, exe = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args)
    return got[0].a, ref[0].a, exe


@pytest.mark.parametrize("shape,embed,steps", [((70, 21, 9), "pad", 2), ((70, 21, 9), "dus", 2), ((64, 40, 20), "pad", 4),
                                               ((130, 17, 6), "pad", 3), ((58, 26, 5), "dus", 5), ((250, 10, 2), "pad", 2), ((20, 130, 4), "pad", 2),
                                               ((20, 150, 4), "dus", 3)])
@pytest.mark.parametrize("march", ["1", "0"])
def test_stencil_two_steps_per_kernel(rx, client, monkeypatch, shape, embed, steps, march):
    """Pairs of steps share one kernel (the first step's field lives only in LDS): the values are
    the same bits as the oracle's, for tiles cut by every array edge and an odd step left over.
    Both traversals: marching along the slowest dimension with plane rings, and 3-D tiles."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    monkeypatch.setenv("RX_STENCIL_MARCH2", march)
    got, ref, exe = _stencil_case(rx, client, shape, embed, steps)
    launches = exe.launches()
    kinds = [l["kind"] for l in launches]
    assert kinds.count("map_stencil_lds2") == steps // 2 and len(kinds) == steps // 2 + steps % 2
    assert launches[0]["kernel"].endswith("_stencil2m" if march == "1" else "_stencil2")
    assert np.array_equal(got, ref)


def _lopsided_stencil(nx, ny, nz, steps, offsets, H=3):
    """steps of c <- pad(sum of c at `offsets` (dz, dy, dx) + u) with one-sided neighbourhoods."""
    full, inner = [nz + 2 * H, ny + 2 * H, nx + 2 * H], [nz, ny, nx]
    tf = "tensor<%dx%dx%dxf64>" % tuple(full)
    ti = "tensor<%dx%dx%dxf64>" % tuple(inner)
    lines, k, c = ["    %z = stablehlo.constant dense<0.000000e+00> : tensor<f64>"], [0], "%arg0"

    def new():
        k[0] += 1
        return "%%v%d" % k[0]

    def sl(x, d):
        r, st = new(), [H + d[0], H + d[1], H + d[2]]
        lines.append("    %s = stablehlo.slice %s [%s] : (%s) -> %s" % (
            r, x, ", ".join("%d:%d" % (a, a + n) for a, n in zip(st, inner)), tf, ti))
        return r

    u = sl("%arg1", (0, 0, 0))
    for _ in range(steps):
        acc = u
        for d in offsets:
            t, r = sl(c, d), new()
            lines.append("    %s = stablehlo.add %s, %s : %s" % (r, acc, t, ti))
            acc = r
        c = new()
        lines.append("    %s = stablehlo.pad %s, %%z, low = [%d, %d, %d], high = [%d, %d, %d], interior = [0, 0, 0] : (%s, tensor<f64>) -> %s"
                     % (c, acc, H, H, H, H, H, H, ti, tf))
    return ("module @reactant_lopsided {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n%s\n    return %s : %s\n  }\n}\n"
            % (tf, tf, tf, "\n".join(lines), c, tf))


@pytest.mark.parametrize("march", ["1", "0"])
@pytest.mark.parametrize("offsets", [[(0, 0, 0), (-1, 0, 0), (0, 1, 0), (0, 0, -2)],
                                     [(0, 0, 0), (2, 0, 0), (0, -2, 0), (0, 0, 1), (0, 0, 3)],
                                     [(0, 0, 0), (0, -1, 0), (0, 1, 0), (0, 0, 1)]])
def test_two_step_kernels_with_one_sided_neighbourhoods(rx, client, monkeypatch, offsets, march):
    """Halos that differ per side and per dimension (including none in z): ring sizes, shell
    enumeration and tile halos follow the offsets the module actually uses."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    monkeypatch.setenv("RX_STENCIL_MARCH2", march)
    nx, ny, nz = 70, 19, 7
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(11)
    args = [I.Tensor(rng.uniform(-1, 1, full), "f64") for _ in range(2)]
    text = _lopsided_stencil(nx, ny, nz, 3, offsets)
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["map_stencil_lds2", "map_stencil_lds"]
    assert np.array_equal(got[0].a, oracle_run(text, args)[0].a)


@pytest.mark.parametrize("elt", ["f64", "f32"])
def test_stencil_with_two_fields_read_at_offsets(rx, client, monkeypatch, elt):
    """Both inputs are read at several offsets: both get an LDS halo tile in the one-step kernel,
    and steps are not paired (a pair needs a single field carried from step to step)."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    nx, ny, nz, H = 72, 20, 6, 3
    full, inner = [nz + 2 * H, ny + 2 * H, nx + 2 * H], [nz, ny, nx]
    tf = "tensor<%dx%dx%dx%s>" % (*full, elt)
    ti = "tensor<%dx%dx%dx%s>" % (*inner, elt)
    lines, k = ["    %%z = stablehlo.constant dense<0.000000e+00> : tensor<%s>" % elt], [0]

    def sl(x, d):
        k[0] += 1
        r, st = "%%s%d" % k[0], [H + d[0], H + d[1], H + d[2]]
        lines.append("    %s = stablehlo.slice %s [%s] : (%s) -> %s" % (
            r, x, ", ".join("%d:%d" % (a, a + n) for a, n in zip(st, inner)), tf, ti))
        return r

    c = "%arg0"
    for step in range(2):
        terms = [sl(c, d) for d in [(0, 0, -1), (0, 0, 1), (0, 1, 0), (-1, 0, 0)]] + \
                [sl("%arg1", d) for d in [(1, 0, 0), (-1, 0, 0), (0, -1, 0), (0, 0, 2)]]
        acc = terms[0]
        for t in terms[1:]:
            k[0] += 1
            r = "%%a%d" % k[0]
            lines.append("    %s = stablehlo.multiply %s, %s : %s" % (r, acc, t, ti) if step and t is terms[4] else
                         "    %s = stablehlo.add %s, %s : %s" % (r, acc, t, ti))
            acc = r
        k[0] += 1
        c = "%%p%d" % k[0]
        lines.append("    %s = stablehlo.pad %s, %%z, low = [3, 3, 3], high = [3, 3, 3], interior = [0, 0, 0] : (%s, tensor<%s>) -> %s"
                     % (c, acc, ti, elt, tf))
    text = ("module @reactant_two_fields {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n%s\n    return %s : %s\n  }\n}\n"
            % (tf, tf, tf, "\n".join(lines), c, tf))
    rng = np.random.default_rng(4)
    np_t = np.float64 if elt == "f64" else np.float32
    args = [I.Tensor(rng.uniform(-1, 1, full).astype(np_t), elt) for _ in range(2)]
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["map_stencil_lds", "map_stencil_lds"]
    assert np.array_equal(got[0].a, oracle_run(text, args)[0].a)


@pytest.mark.parametrize("planes,tile", [("3", "8,64"), ("5", "16,32"), ("100", "4,128"), ("7", "32,16")])
def test_stencil_marching_chunks_and_tiles(rx, client, monkeypatch, planes, tile):
    """The marching kernel with chunks shorter and longer than the grid and other plane tiles."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    monkeypatch.setenv("RX_MARCH2_PLANES", planes)
    monkeypatch.setenv("RX_MARCH2_TILE", tile)
    for shape, embed in [((70, 21, 9), "pad"), ((20, 130, 11), "dus")]:
        got, ref, exe = _stencil_case(rx, client, shape, embed, 2)
        assert exe.launches()[0]["kernel"].endswith("_stencil2m")
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("shape,elt,tile", [((134, 70, 9), "f64", "8,64"), ((200, 33, 5), "f32", "8,64"), ((390, 20, 12), "f32", "8,64"),
                                            ((262, 9, 30), "f64", "8,64")])
def test_stencil_edge_columns_in_tiles_of_their_own(rx, client, monkeypatch, shape, elt, tile):
    """A nearly empty last tile column is covered by tiles a quarter as wide and four times as tall in the same launch:
    same bits as the oracle's and as the kernel with one tile shape."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    monkeypatch.setenv("RX_MARCH2_TILE", tile)
    monkeypatch.setenv("RX_MARCH2_PLANES", "4")
    text = P.stencil(*shape, steps=2, elt=elt)
    assert "columns in tiles of" in rx.compile_offline(text, with_source=True)
    got, ref, exe = _stencil_case(rx, client, shape, "pad", 2, elt=elt)
    assert exe.launches()[0]["kernel"].endswith("_stencil2m")
    assert np.array_equal(got, ref)
    monkeypatch.setenv("RX_MARCH2_EDGE", "0")
    assert "columns in tiles of" not in rx.compile_offline(text, with_source=True)
    one, _, exe1 = _stencil_case(rx, client, shape, "pad", 2, elt=elt)
    assert np.array_equal(one, got)


def test_stencil_two_steps_f32_and_unfused_agree(rx, client, monkeypatch):
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    got, ref, exe = _stencil_case(rx, client, (72, 24, 10), "pad", 2, elt="f32")
    assert [l["kind"] for l in exe.launches()] == ["map_stencil_lds2"]
    assert np.array_equal(got, ref)
    monkeypatch.setenv("RX_STENCIL_FUSE", "0")
    got1, _, exe1 = _stencil_case(rx, client, (72, 24, 10), "pad", 2, elt="f32")
    assert [l["kind"] for l in exe1.launches()] == ["map_stencil_lds", "map_stencil_lds"]
    assert np.array_equal(got1, got)


@pytest.mark.parametrize("embed", ["pad", "dus"])
def test_stencil_traced_loop_form(rx, client, monkeypatch, embed):
    """`@trace for`: the ten steps arrive as one stablehlo.while; same bits as the oracle's loop."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    nx, ny, nz = 40, 21, 9
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(3)
    args = [I.Tensor(rng.uniform(-1, 1, full), "f64") for _ in range(4)]
    text = P.stencil(nx, ny, nz, steps=5, embed=embed, loop="while")
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["map_stencil_lds2", "map_stencil_lds2", "map_stencil_lds"]
    assert np.array_equal(got[0].a, oracle_run(text, args)[0].a)


def test_stencil_xcd_slab_order(rx, client, monkeypatch):
    """Same parity with the XCD-slab tile order forced on a small grid."""
    monkeypatch.setenv("RX_SLAB_MIN_NUMEL", "1")
    test_stencil(rx, client, (64, 40, 20), "pad")
    test_stencil(rx, client, (30, 33, 9), "dus")


@pytest.mark.parametrize("m,n,k,form", [(5, 7, 3, "propagated"), (5, 7, 3, "transposed"), (64, 48, 32, "propagated"),
                                        (256, 256, 256, "propagated"), (128, 256, 64, "transposed")])
def test_gemm_f32(rx, client, m, n, k, form):
    A = np.random.default_rng(0).normal(size=(m, k)).astype(np.float32)
    B = np.random.default_rng(1).normal(size=(k, n)).astype(np.float32)
    C = np.random.default_rng(2).normal(size=(m, n)).astype(np.float32)
    args = [I.Tensor(A.T.copy(), "f32"), I.Tensor(B.T.copy(), "f32"), I.Tensor(C.T.copy(), "f32")]
    text = P.gemm(m, n, k, form=form)
    got, _ = gpu_run(rx, client, text, args)
    ref = 1.5 * (A.astype(np.float64) @ B.astype(np.float64)) + 1.2 * C.astype(np.float64)
    # componentwise: against 1.5 |A| |B| + 1.2 |C|, entry by entry
    bound = 1.5 * (np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64)) + 1.2 * np.abs(C).astype(np.float64)
    assert contraction_err(got[0].a.T, ref, bound) <= 1e-6
    assert max_rel_to_scale(got[0].a.T, ref) <= 1e-5 * np.sqrt(k)
    orc = oracle_run(text, args, hifi=True)
    assert max_rel_to_scale(orc[0].a.T, ref) <= 1e-6


def _mlp_args(batch, widths, seed=0):
    rng = np.random.default_rng(seed)
    args = [I.tensor(rng.normal(size=(batch, widths[0])), "bf16")]
    for l in range(len(widths) - 1):
        lim = np.sqrt(6.0 / (widths[l] + widths[l + 1]))
        args.append(I.tensor(np.random.default_rng(seed + 1 + l).uniform(-lim, lim, size=(widths[l], widths[l + 1])), "bf16"))
        args.append(I.tensor(np.random.default_rng(seed + 4 + l).normal(size=(widths[l + 1],)) * 0.01, "bf16"))
    return args


@pytest.mark.parametrize("batch,widths,gelu", [(8, (16, 32, 32, 16), "chain"), (64, (32, 64, 64, 32), "op"),
                                               (256, (128, 256, 256, 128), "chain")])
def test_mlp_bf16(rx, client, batch, widths, gelu):
    args = _mlp_args(batch, widths)
    text = P.mlp(batch, widths, gelu=gelu)
    got, _ = gpu_run(rx, client, text, args)
    # The GPU path keeps bf16 arithmetic in f32 inside a kernel (as XLA does by default) and rounds
    # where values are written: compare with the oracle evaluated the same way at 1e-2 of the
    # output scale; the oracle that rounds after every op is a second valid evaluation of the
    # module, three bf16 layers deep, and must agree within a few bf16 ulps (2e-2).
    ref = oracle_run(text, args, hifi=True, excess=True)
    strict = oracle_run(text, args, hifi=True)
    assert np.allclose(got[0].a.sum(axis=1), 1.0, atol=2e-2)   # softmax rows sum to one
    # outputs are bf16: one ulp is up to 0.8% of a value, and three chained bf16 layers can move a
    # result by two ulps, so the end-to-end bound is 2e-2 (single dot_generals are held to 1e-2
    # in test_gpu_dot.py)
    assert max_rel_to_scale(got[0].a, ref[0].a) <= 2e-2
    assert max_rel_to_scale(got[0].a, strict[0].a) <= 3e-2
    # every layer on its own, fed with the oracle's activations of the layer before, is held to 1e-2 componentwise:
    # |got - ref|_ij <= 1e-2 (|h| . |W| + |b|)_ij  (gelu has slope <= 1.13 and is rounded to bf16 once)
    h = args[0]
    for l in range(len(widths) - 1):
        layer = P.mlp(batch, widths[l:l + 2], gelu=gelu, softmax=False)
        largs = [h, args[1 + 2 * l], args[2 + 2 * l]]
        got_l, _ = gpu_run(rx, client, layer, largs)
        ref_l = oracle_run(layer, largs, hifi=True, excess=True)
        bound = (np.abs(h.a.astype(np.float64)) @ np.abs(largs[1].a.astype(np.float64))) + np.abs(largs[2].a.astype(np.float64))[None, :]
        assert contraction_err(got_l[0].a, ref_l[0].a, bound) <= 1e-2, l
        h = ref_l[0]


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_gelu_chain_on_every_value(rx, client, dt):
    """The tanh chain that gelu lowers to, as a map of its own over every 16-bit pattern (infinities, NaNs, zeros and
    subnormals included): the kernel evaluates it in the logistic form with folded constants.  Each result is within
    one ulp of the chain evaluated in float64 and rounded once (plus |x| 2^-22, what one float32 rounding of
    1 + tanh costs the chain itself: where that sum cancels, the logistic form is the more accurate of the two);
    non-finite results agree in kind."""
    n = 1 << 16
    b = P._B()
    b.types["%arg0"] = P._tt([n], dt)
    h = P._gelu_tanh(b, "%arg0", [n], dt)
    text = ("module {\n  func.func @main(%%arg0: %s) -> %s {\n" % (P._tt([n], dt), P._tt([n], dt)) + b.text()
            + "    return %s : %s\n  }\n}\n" % (h, P._tt([n], dt)))
    bits = np.arange(n, dtype=np.uint16)
    x = I.Tensor.from_bytes(bits.tobytes(), dt, (n,))
    got, exe = gpu_run(rx, client, text, [x])
    assert "rx_gelu_chain_fast" in rx.compile_offline(text, with_source=True)
    with np.errstate(all="ignore"):
        xv = x.a.astype(np.float64)
    c0 = float(I.tensor(np.array([np.sqrt(2.0 / np.pi)]), dt).a[0])
    c1 = float(I.tensor(np.array([0.044715]), dt).a[0])
    with np.errstate(all="ignore"):
        exact = 0.5 * xv * (1.0 + np.tanh(c0 * (xv + c1 * xv * xv * xv)))
        ref = I.tensor(exact, dt).a.astype(np.float64)
    g = got[0].a.astype(np.float64)
    assert np.array_equal(np.isnan(g), np.isnan(ref))
    fin = np.isfinite(ref)
    assert np.array_equal(g[~fin & ~np.isnan(ref)], ref[~fin & ~np.isnan(ref)])
    ulp = np.spacing(np.abs(ref[fin]).astype(np.float32)).astype(np.float64) * (2.0 ** (24 - (8 if dt == "bf16" else 11)))
    tiny = 2.0 ** (-133 if dt == "bf16" else -24)
    assert np.all(np.abs(g[fin] - ref[fin]) <= np.maximum(ulp, tiny) + np.abs(xv[fin]) * 2.0 ** -22)


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_exponential_of_every_narrow_value(rx, client, dt):
    """exp over every 16-bit pattern: narrow results take the hardware 2^y on y = x log2(e).  Within one ulp of the
    exponential evaluated in float64 and rounded once; overflow to inf, underflow to zero and NaN as the exact result;
    results below the smallest normal float32 (bf16 subnormals) may be flushed to zero."""
    n = 1 << 16
    ty = P._tt([n], dt)
    text = "module {\n  func.func @main(%%arg0: %s) -> %s {\n    %%0 = stablehlo.exponential %%arg0 : %s\n    return %%0 : %s\n  }\n}\n" % (ty, ty, ty, ty)
    x = I.Tensor.from_bytes(np.arange(n, dtype=np.uint16).tobytes(), dt, (n,))
    got, _ = gpu_run(rx, client, text, [x])
    assert "rx_exp_fast" in rx.compile_offline(text, with_source=True)
    with np.errstate(all="ignore"):
        xv = x.a.astype(np.float64)
        exact = np.exp(xv)
        ref = I.tensor(exact, dt).a.astype(np.float64)
    g = got[0].a.astype(np.float64)
    assert np.array_equal(np.isnan(g), np.isnan(ref))
    ok = ~np.isnan(ref)
    inf = ok & np.isinf(ref)
    # at the overflow threshold the rounded exact result may be the largest finite value where the GPU gives inf, or the reverse
    big = np.finfo(np.float32).max if dt == "bf16" else 65504.0
    assert np.all((g[inf] == np.inf) | (g[inf] >= big * 0.99))
    fin = ok & np.isfinite(ref)
    ulp = np.spacing(np.abs(ref[fin]).astype(np.float32)).astype(np.float64) * (2.0 ** (24 - (8 if dt == "bf16" else 11)))
    tiny = 2.0 ** -126 if dt == "bf16" else 2.0 ** -24
    d = np.abs(g[fin] - ref[fin])
    assert np.all((d <= np.maximum(ulp, tiny)) | (np.isinf(g[fin]) & (ref[fin] >= big * 0.99)))


def test_division_by_a_row_value_special_cases(rx, client):
    """bf16 rows divided by a per-row value (the reciprocal form): divisors that are zero, infinite, NaN, huge, tiny and
    subnormal against dividends of every kind.  Finite quotients within an ulp of the exact one (or both zero / both
    beyond the largest bf16), infinities and NaNs where IEEE division has them."""
    big, tiny = 3.0e38, 1.2e-38
    divisors = np.array([1.0, -3.0, 0.0, -0.0, np.inf, -np.inf, np.nan, big, -big, tiny, 4.0e-39, 2.0e-39, 1.0e-39, 1.0e-40, 9.2e-41, -9.2e-41, 1.0e-30, 5.0e-20, 7.0e20, 0.333], dtype=np.float64)
    dividends = np.array([0.0, -0.0, 1.0, -1.0, 2.5, np.inf, -np.inf, np.nan, big, -big, tiny, 1.0e-20, 6.0e15, 0.1, 100.0, -7.0, 1.0e-35, 9.2e-41, 3.0e-39], dtype=np.float64)
    rows, cols = len(divisors), 64
    x = np.tile(np.resize(dividends, cols), (rows, 1))
    ty, tr = P._tt([rows, cols], "bf16"), P._tt([rows], "bf16")
    text = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%0 = stablehlo.broadcast_in_dim %%arg1, dims = [0] : (%s) -> %s\n"
            "    %%1 = stablehlo.divide %%arg0, %%0 : %s\n    return %%1 : %s\n  }\n}\n" % (ty, tr, ty, tr, ty, ty, ty))
    assert "rx_div_minor_uniform(" in rx.compile_offline(text, with_source=True)
    a, b = I.tensor(x, "bf16"), I.tensor(divisors, "bf16")
    got, _ = gpu_run(rx, client, text, [a, b])
    g = got[0].a.astype(np.float64)
    with np.errstate(all="ignore"):
        exact = a.a.astype(np.float64) / b.a.astype(np.float64)[:, None]
        ref = I.tensor(exact, "bf16").a.astype(np.float64)
    assert np.array_equal(np.isnan(g), np.isnan(ref)), (g[np.isnan(g) != np.isnan(ref)], ref[np.isnan(g) != np.isnan(ref)])
    ok = ~np.isnan(ref)
    top = 3.3895313892515355e38          # the largest bf16
    both_huge = ok & (np.abs(g) >= top) & (np.abs(ref) >= top) & (np.sign(g) == np.sign(ref))
    fin = ok & np.isfinite(ref) & ~both_huge
    assert np.array_equal(np.isinf(g[ok & ~both_huge]), np.isinf(ref[ok & ~both_huge]))
    ulp = np.spacing(np.abs(ref[fin]).astype(np.float32)).astype(np.float64) * 2.0 ** 16
    assert np.all(np.abs(g[fin] - ref[fin]) <= np.maximum(ulp, 2.0 ** -126)), (g[fin][np.abs(g[fin] - ref[fin]) > np.maximum(ulp, 2.0 ** -126)], ref[fin][np.abs(g[fin] - ref[fin]) > np.maximum(ulp, 2.0 ** -126)])
    assert np.array_equal(np.signbit(g[fin & (ref == 0)]), np.signbit(ref[fin & (ref == 0)]))


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_logistic_of_every_narrow_value(rx, client, dt):
    """1 / (1 + e^-x) over every 16-bit pattern (narrow results: hardware 2^y and reciprocal): one ulp of the float64
    result rounded once, exactly 0 and 1 at the ends, NaN where the input is NaN; results below the smallest normal
    float32 may be flushed to zero."""
    n = 1 << 16
    ty = P._tt([n], dt)
    text = "module {\n  func.func @main(%%arg0: %s) -> %s {\n    %%0 = stablehlo.logistic %%arg0 : %s\n    return %%0 : %s\n  }\n}\n" % (ty, ty, ty, ty)
    x = I.Tensor.from_bytes(np.arange(n, dtype=np.uint16).tobytes(), dt, (n,))
    got, _ = gpu_run(rx, client, text, [x])
    assert "rx_logistic_fast" in rx.compile_offline(text, with_source=True)
    with np.errstate(all="ignore"):
        xv = x.a.astype(np.float64)
        exact = 1.0 / (1.0 + np.exp(-xv))
        ref = I.tensor(exact, dt).a.astype(np.float64)
    g = got[0].a.astype(np.float64)
    assert np.array_equal(np.isnan(g), np.isnan(ref))
    fin = ~np.isnan(ref)
    ulp = np.spacing(np.abs(ref[fin]).astype(np.float32)).astype(np.float64) * (2.0 ** (24 - (8 if dt == "bf16" else 11)))
    tiny = 2.0 ** -126 if dt == "bf16" else 2.0 ** -24
    assert np.all(np.abs(g[fin] - ref[fin]) <= np.maximum(ulp, tiny))
    assert g[fin].min() >= 0.0 and g[fin].max() <= 1.0


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_softmax_rows_with_extreme_sums(rx, client, dt):
    """Softmax over rows whose sums of exponentials are tiny, ordinary and huge: the division by the row's sum is a
    multiplication by its reciprocal (computed once per row by a true division) for narrow results; against the oracle,
    one ulp of the exact quotient."""
    rows, cols = 64, 1000
    rng = np.random.default_rng(5)
    x = rng.normal(size=(rows, cols))
    hi = 80.0 if dt == "bf16" else 3.0
    x += np.linspace(-hi, hi, rows)[:, None]          # sums from e^-80 * 1000 to e^80 * 1000 (bf16); f16 holds no more than 65504
    ty, tr = P._tt([rows, cols], dt), P._tt([rows], dt)
    text = ("module {\n  func.func @main(%%arg0: %s) -> %s {\n"
            "    %%c = stablehlo.constant dense<0.0> : tensor<%s>\n"
            "    %%0 = stablehlo.exponential %%arg0 : %s\n"
            "    %%1 = stablehlo.reduce(%%0 init: %%c) applies stablehlo.add across dimensions = [1] : (%s, tensor<%s>) -> %s\n"
            "    %%2 = stablehlo.broadcast_in_dim %%1, dims = [0] : (%s) -> %s\n"
            "    %%3 = stablehlo.divide %%0, %%2 : %s\n    return %%3 : %s\n  }\n}\n" % (ty, ty, dt, ty, ty, dt, tr, tr, ty, ty, ty))
    a = I.tensor(x, dt)
    got, exe = gpu_run(rx, client, text, [a])
    assert "rx_div_minor_uniform(" in rx.compile_offline(text, with_source=True)
    xv = a.a.astype(np.float64)
    e = np.exp(xv)
    exact = e / e.sum(axis=1, keepdims=True)
    g = got[0].a.astype(np.float64)
    rel = 2.0 ** -7 if dt == "bf16" else 2.0 ** -10
    # the kernel keeps the exponentials and the row's sum in float32 and rounds once: one ulp of the exact quotient
    assert np.all(np.abs(g - exact) <= 1.01 * rel * exact + (1e-40 if dt == "bf16" else 2.0 ** -24))
    # the oracle may round the row's sum to the narrow type before it is broadcast (it is a tensor of that type)
    ref = oracle_run(text, [a], hifi=True, excess=True)[0].a.astype(np.float64)
    assert np.all(np.abs(g - ref) <= 2.5 * rel * np.maximum(np.abs(ref), np.abs(g)) + (1e-40 if dt == "bf16" else 2.0 ** -24))


@pytest.mark.parametrize("batch,k,n,layout,form", [(8, 32, 16, "nk", "convert"), (8, 32, 16, "kn", "direct"),
                                                   (64, 128, 256, "nk", "convert"), (128, 256, 128, "kn", "convert")])
def test_fp8_linear(rx, client, batch, k, n, layout, form):
    a = I.tensor(np.random.default_rng(0).normal(size=(batch, k)), "bf16")
    wq = I.tensor(np.random.default_rng(1).normal(size=(n, k) if layout == "nk" else (k, n)), "f8E4M3FN")
    sw = I.Tensor(np.float32(0.0123), "f32")
    text = P.fp8_linear(batch, k, n, weight_layout=layout, dot_form=form)
    got, _ = gpu_run(rx, client, text, [a, wq, sw])
    ref = oracle_run(text, [a, wq, sw], hifi=True, excess=True)
    assert max_rel_to_scale(got[0].a, ref[0].a) <= 1e-2
    # rows are normalised one by one: each row against its own largest entry
    g64, r64 = got[0].a.astype(np.float64), ref[0].a.astype(np.float64)
    assert float(np.max(np.max(np.abs(g64 - r64), axis=1) / np.max(np.abs(r64), axis=1))) <= 1e-2
    # RMSNorm invariant: mean square of every row is 1 (up to bf16 rounding)
    assert np.allclose((got[0].a.astype(np.float64) ** 2).mean(axis=1), 1.0, atol=2e-2)
