"""CPU tests that pin the oracle (no GPU): the reference's own known-answer tests
and fixtures for the hot path, closed forms, library routines and brute force on
tiny inputs.  Each check is chosen so that a plausible mistake in the oracle (a
wrong index convention, a dropped term, a transposed operand) fails it."""
import json
import math
import os

import numpy as np
import pytest

from oracle import lowfloat as lf
from oracle import stablehlo_interp as I
from _loader import load_programs
import _while_modules as W

P = load_programs()
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def run(text, args, **kw):
    return I.run_text(text, args, **kw)


def jl_fixture(dtype, *dims):
    """Reactant.TestUtils.construct_test_array: reshape(collect(1:prod) ./ prod, dims), column-major
    (reference src/TestUtils.jl:9-23)."""
    n = int(np.prod(dims))
    flat = np.arange(1, n + 1)
    a = (flat / n).astype(dtype) if np.issubdtype(dtype, np.floating) else flat.astype(dtype)
    return a.reshape(dims, order="F")


def wire(a):
    """Julia array -> dense row-major buffer with reversed dims (src/xla/PJRT/Buffer.jl:9-17)."""
    return np.ascontiguousarray(a.T)


def test_golden_vectors_file():
    """Vectors transcribed from the reference's tests (inputs and expected outputs only)."""
    with open(os.path.join(GOLD, "reference_kats.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 10
    for c in cases:
        args = [I.Tensor(np.array(a["data"], dtype=I.NP_OF[a["dtype"]]).reshape(a["shape"]), a["dtype"]) for a in c["args"]]
        out = run(c["module"], args, hifi=True)
        exp = np.array(c["expect"]["data"], dtype=np.float64).reshape(c["expect"]["shape"])
        got = np.asarray(out[0].a, dtype=np.float64)
        if c["expect"].get("exact", False):
            assert np.array_equal(got, exp), c["name"]
        else:
            assert np.allclose(got, exp, rtol=c["expect"].get("rtol", 1e-12), atol=c["expect"].get("atol", 1e-12)), c["name"]


def test_dims_reversal_and_layout():
    # x == Array(to_rarray(x)) for a 2x2 (test/core/layout.jl:35-48): the wire buffer of Julia [1 2; 3 4]
    # is the bytes 1,3,2,4 viewed as a row-major 2x2, i.e. the transpose
    x = np.array([[1.0, 2.0], [3.0, 4.0]])
    t = I.Tensor(wire(x), "f64")
    assert t.to_bytes() == np.array([1.0, 3.0, 2.0, 4.0]).tobytes()
    # a Julia 3x4 array is typed tensor<4x3xf64> on the wire (test/core/buffer_donation.jl:64-72)
    assert wire(jl_fixture(np.float64, 3, 4)).shape == (4, 3)


def test_reductions_closed_forms():
    A = jl_fixture(np.float64, 2, 10)
    t = "tensor<10x2xf64>"
    text = ("module { func.func @main(%%a: %s) -> tensor<f64> {\n %%c = stablehlo.constant dense<0.0> : tensor<f64>\n"
            " %%0 = stablehlo.reduce(%%a init: %%c) applies stablehlo.add across dimensions = [0, 1] : (%s, tensor<f64>) -> tensor<f64>\n"
            " return %%0 : tensor<f64> } }" % (t, t))
    assert abs(float(run(text, [I.Tensor(wire(A), "f64")])[0].a) - 10.5) < 1e-13     # 210/20
    # sum over Julia dims=1 of a 2x10: wire dims [1] -> 10 values (k + k+1)/20 for k = 1,3,5...
    text2 = ("module { func.func @main(%%a: %s) -> tensor<10xf64> {\n %%c = stablehlo.constant dense<0.0> : tensor<f64>\n"
             " %%0 = stablehlo.reduce(%%a init: %%c) applies stablehlo.add across dimensions = [1] : (%s, tensor<f64>) -> tensor<10xf64>\n"
             " return %%0 : tensor<10xf64> } }" % (t, t))
    got = run(text2, [I.Tensor(wire(A), "f64")])[0].a
    assert np.allclose(got, A.sum(axis=0))
    assert np.allclose(got, [(4 * k + 3) / 20 for k in range(10)])


def test_sinsum_against_library():
    n = 4097
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
    got = run(P.sinsum_add(n), [I.Tensor(x, "f32"), I.Tensor(y, "f32")], hifi=True)
    exact = math.fsum(np.sin(x.astype(np.float64)) + y.astype(np.float64))
    # sin is evaluated in f32 (then widened): each term carries an f32 rounding
    assert abs(float(got[0].a) - exact) <= 1e-6 * n
    # the reduce adds the init value: a dropped init would change this
    t = P.sinsum_add(4).replace("dense<0.000000e+00>", "dense<2.500000e+00>")
    z = np.zeros(4, np.float32)
    assert float(run(t, [I.Tensor(z, "f32"), I.Tensor(z, "f32")])[0].a) == 2.5


def brute_stencil(c, u, v, w, steps, dt=0.05, dx=1.0, kappa=1.0, H=3):
    c = c.copy()
    nz, ny, nx = (s - 2 * H for s in c.shape)
    for _ in range(steps):
        new = np.zeros_like(c)
        for k in range(H, H + nz):
            for j in range(H, H + ny):
                for i in range(H, H + nx):
                    ci = c[k, j, i]
                    s = c[k, j, i - 1] + c[k, j, i + 1]
                    s = s + c[k, j - 1, i]
                    s = s + c[k, j + 1, i]
                    s = s + c[k - 1, j, i]
                    s = s + c[k + 1, j, i]
                    lap = (s - 6.0 * ci) * (kappa / (dx * dx))
                    adv = None
                    for vel, cm, cp in ((u[k, j, i], c[k, j, i - 1], c[k, j, i + 1]), (v[k, j, i], c[k, j - 1, i], c[k, j + 1, i]),
                                        (w[k, j, i], c[k - 1, j, i], c[k + 1, j, i])):
                        a = (vel * (ci - cm) if vel > 0 else vel * (cp - ci)) * (1.0 / dx)
                        adv = a if adv is None else adv + a
                    new[k, j, i] = ci + dt * (lap - adv)
        c = new
    return c


@pytest.mark.parametrize("embed", ["pad", "dus"])
def test_stencil_against_brute_force(embed):
    nx, ny, nz = 5, 4, 3
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(0)
    c = np.zeros(full)
    c[3:-3, 3:-3, 3:-3] = rng.uniform(0, 1, (nz, ny, nx))
    u, v, w = [rng.uniform(-1, 1, full) for _ in range(3)]
    got = run(P.stencil(nx, ny, nz, steps=3, embed=embed), [I.Tensor(a, "f64") for a in (c, u, v, w)])[0].a
    ref = brute_stencil(c, u, v, w, 3)
    assert np.array_equal(got, ref)       # same operation order: bit-exact
    # invariants: halos stay zero; pure diffusion (zero velocity) conserves nothing here but is symmetric
    assert np.all(got[:3] == 0) and np.all(got[:, :3] == 0) and np.all(got[:, :, -3:] == 0)


def test_gemm_alpha_beta_reference_case():
    # 5-arg mul!(C, A, B, alpha=2, beta=1) on construct_test_array 4x4 * 4x2 (test/integration/linear_algebra.jl:50-62)
    A, B, C = jl_fixture(np.float64, 4, 4), jl_fixture(np.float64, 4, 2), jl_fixture(np.float64, 4, 2)
    expect = np.zeros((4, 2))
    for i in range(4):
        for j in range(2):
            acc = 0.0
            for k in range(4):
                acc += A[i, k] * B[k, j]
            expect[i, j] = 2.0 * acc + 1.0 * C[i, j]
    for form in ("propagated", "transposed"):
        text = P.gemm(4, 2, 4, alpha=2.0, beta=1.0, dt="f64", form=form)
        got = run(text, [I.Tensor(wire(A), "f64"), I.Tensor(wire(B), "f64"), I.Tensor(wire(C), "f64")])[0].a.T
        assert np.allclose(got, expect, rtol=1e-14), form
    # a transposed operand must fail: A is not symmetric
    assert not np.allclose(2.0 * (A.T @ B) + C, expect)


def test_gelu_and_softmax_closed_forms():
    from scipy.special import erf, softmax
    x = np.linspace(-4, 4, 41)
    assert np.allclose(I.gelu(x, "NONE"), 0.5 * x * (1 + erf(x / np.sqrt(2))))
    assert np.allclose(I.gelu(x, "TANH"), 0.5 * x * (1 + np.tanh(np.sqrt(2 / np.pi) * (x + 0.044715 * x ** 3))))
    assert abs(I.gelu(np.array(1.0), "TANH") - 0.8411919906082768) < 1e-12
    assert np.allclose(I.gelu(x, "SIGMOID"), x / (1 + np.exp(-1.702 * x)))
    # softmax chain of the MLP program in f32 on a 12x5 input (shape of test/nn/nnlib.jl:85-92)
    X = jl_fixture(np.float32, 12, 5)
    text = P.mlp(5, (12, 12), dt="f32", softmax=True)
    # identity weights and zero bias; gelu is applied before the softmax
    W = np.eye(12, dtype=np.float32)
    got = run(text, [I.Tensor(wire(X), "f32"), I.Tensor(W, "f32"), I.Tensor(np.zeros(12, np.float32), "f32")], hifi=True)[0].a
    h = I.gelu(wire(X).astype(np.float64), "TANH")
    assert np.allclose(got, softmax(h, axis=1), rtol=2e-6)
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-6)


def test_fused_dense_bias_activation_case():
    # fused_dense_bias_activation 9x10 * 10x12 + bias 9 (test/nn/nnlib.jl:103-149), gelu variant, rtol 1e-2 there
    W, X, b = jl_fixture(np.float32, 9, 10), jl_fixture(np.float32, 10, 12), jl_fixture(np.float32, 9)
    text = P.mlp(12, (10, 9), dt="f32", softmax=False)
    got = run(text, [I.Tensor(wire(X), "f32"), I.Tensor(wire(W), "f32"), I.Tensor(b, "f32")], hifi=True)[0].a.T
    ref = I.gelu((W.astype(np.float64) @ X.astype(np.float64)) + b.astype(np.float64)[:, None], "TANH")
    assert np.allclose(got, ref, rtol=1e-5)


def test_fp8_tables_and_rounding():
    # closed form of the OCP e4m3 format: bias 7, max 448, S.1111.111 = NaN, no inf
    t = lf.E4M3FN_TABLE
    assert t[0x7E] == 448.0 and np.isnan(t[0x7F]) and np.isnan(t[0xFF]) and t[0x01] == 2.0 ** -9 and t[0x08] == 2.0 ** -6
    assert t[0x38] == 1.0 and t[0xB8] == -1.0 and not np.isinf(t).any()
    t5 = lf.E5M2_TABLE
    assert t5[0x7B] == 57344.0 and np.isinf(t5[0x7C]) and np.isnan(t5[0x7D]) and t5[0x01] == 2.0 ** -16
    # round trip of every finite code
    codes = np.arange(256, dtype=np.uint8)
    fin = np.isfinite(t)
    assert np.array_equal(lf.f32_to_e4m3fn_bits(t[fin]), codes[fin] & np.where(t[fin] == 0, 0x80 | 0x00, 0xFF).astype(np.uint8))
    # ties to even and overflow to NaN
    assert lf.f32_to_e4m3fn_bits(np.float32([464.0, 465.0, 2.0 ** -10, 3 * 2.0 ** -10]))[:].tolist() == [0x7E, 0x7F, 0x00, 0x02]
    # 10x3 table of test/core/custom_number_types.jl uses values exactly representable in e4m3
    vals = np.float32([[1, 2, 3], [0.5, 1.5, 2.5], [4, 8, 16]])
    assert np.array_equal(lf.round_e4m3fn(vals), vals)


def test_narrow_float_casts_match_torch():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(size=20000) * s for s in (1e-3, 1, 100, 1e4)]).astype(np.float32)
    x = np.concatenate([x, np.float32([448, 464, 465, 2.0 ** -10, 61440, 61439, 65504, 1e6, 0, -0.0])])
    tx = torch.from_numpy(x)
    assert np.array_equal(lf.f32_to_bf16_bits(x), tx.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(lf.f32_to_e4m3fn_bits(x), tx.to(torch.float8_e4m3fn).view(torch.uint8).numpy())
    a = lf.f32_to_e5m2_bits(x)
    b = tx.to(torch.float8_e5m2).view(torch.uint8).numpy()
    assert np.array_equal(a, b)
    # product-side packers (hostfloat) agree with the oracle's
    from _loader import load_pkg
    import importlib
    load_pkg()
    hf = importlib.import_module("reactant_jl_amd.hostfloat")
    assert np.array_equal(hf.f32_to_bf16_bits(x), lf.f32_to_bf16_bits(x))
    assert np.array_equal(hf.f32_to_f8e4m3fn_bits(x), lf.f32_to_e4m3fn_bits(x))
    assert np.array_equal(hf.f32_to_f8e5m2_bits(x), lf.f32_to_e5m2_bits(x))


def test_bf16_and_fp8_dot_exact_products():
    # inputs exactly representable in bf16 / e4m3; f64 triple loop; products of two e4m3 numbers are exact in f32
    rng = np.random.default_rng(0)
    a = lf.round_e4m3fn(rng.normal(size=(5, 16)).astype(np.float32))
    b = lf.round_e4m3fn(rng.normal(size=(7, 16)).astype(np.float32))
    text = ("module { func.func @main(%a: tensor<5x16xf8E4M3FN>, %b: tensor<7x16xf8E4M3FN>) -> tensor<5x7xf32> {\n"
            " %0 = stablehlo.dot_general %a, %b, contracting_dims = [1] x [1] : (tensor<5x16xf8E4M3FN>, tensor<7x16xf8E4M3FN>) -> tensor<5x7xf32>\n"
            " return %0 : tensor<5x7xf32> } }")
    got = run(text, [I.Tensor(a, "f8E4M3FN"), I.Tensor(b, "f8E4M3FN")], hifi=True)[0].a
    ref = np.zeros((5, 7))
    for i in range(5):
        for j in range(7):
            ref[i, j] = math.fsum(float(a[i, k]) * float(b[j, k]) for k in range(16))
    assert np.array_equal(got, ref.astype(np.float32))
    # the whole fp8-linear program: RMSNorm invariant and absmax scale
    x = I.tensor(rng.normal(size=(6, 32)), "bf16")
    w = I.tensor(rng.normal(size=(8, 32)), "f8E4M3FN")
    out = run(P.fp8_linear(6, 32, 8), [x, w, I.Tensor(np.float32(0.02), "f32")], hifi=True)[0].a
    assert np.allclose((out.astype(np.float64) ** 2).mean(axis=1), 1.0, atol=2e-2)
    sa = np.float32(np.abs(x.a).max()) / np.float32(448.0)
    q = lf.round_e4m3fn(np.clip(x.a / sa, -448, 448))
    y = lf.round_bf16(((q.astype(np.float64) @ w.a.astype(np.float64).T) * float(sa * np.float32(0.02))).astype(np.float32))
    ref = y / np.sqrt((y.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6)
    assert np.allclose(out, ref, rtol=2e-2, atol=1e-2)


def test_parser_accepts_reference_text_samples():
    # whole modules that appear in the reference (test/core/ops.jl:1054-1059,1071-1076,1154-1166; src/Ops.jl:1986-2020)
    m1 = """
    module {
      func.func @main(%arg0: tensor<3xf32>, %arg1: tensor<3xf32>) -> tensor<3xf32> {
        %0 = stablehlo.add %arg0, %arg1 : tensor<3xf32>
        return %0 : tensor<3xf32>
      }
    }"""
    x, y = np.float32([1.0, 2.0, 50.0]), np.float32([-4.0, 0.001, 2.0])
    assert np.array_equal(run(m1, [I.Tensor(x, "f32"), I.Tensor(y, "f32")])[0].a, x + y)
    m2 = """
    module {
      func.func @main(%arg0: tensor<3xf32>, %arg1: tensor<3xf32>) -> tensor<3xf32> {
        %0 = func.call @add(%arg0, %arg1) : (tensor<3xf32>, tensor<3xf32>) -> tensor<3xf32>
        return %0 : tensor<3xf32>
      }
      func.func @add(%arg0: tensor<3xf32>, %arg1: tensor<3xf32>) -> tensor<3xf32> {
        %0 = stablehlo.add %arg0, %arg1 : tensor<3xf32>
        return %0 : tensor<3xf32>
      }
    }"""
    o = np.float32([1, 2, 3])
    assert run(m2, [I.Tensor(o, "f32"), I.Tensor(o, "f32")])[0].a.tolist() == [2, 4, 6]
    # argument attributes, locations, multi-result barrier (test/core/buffer_donation.jl:64-72, test/core/compile.jl:653-661)
    m3 = """
    module @reactant_f attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
      func.func @main(%arg0: tensor<4x3xf64> {tf.aliasing_output = 0 : i32} loc("arg1 (path=(:args, 1))"), %arg1: tensor<4x3xf64>) -> (tensor<4x3xf64>, tensor<4x3xf64>) {
        %0:2 = stablehlo.optimization_barrier %arg0, %arg1 : tensor<4x3xf64>, tensor<4x3xf64>
        %1 = stablehlo.multiply %0#0, %0#1 : tensor<4x3xf64> loc(#loc1)
        return %1, %0#1 : tensor<4x3xf64>, tensor<4x3xf64>
      }
    }
    #loc1 = loc("mul")
    """
    a = np.arange(12.0).reshape(4, 3)
    r = run(m3, [I.Tensor(a, "f64"), I.Tensor(a + 1, "f64")])
    assert np.array_equal(r[0].a, a * (a + 1)) and np.array_equal(r[1].a, a + 1)
    # attribute text of test/core/config.jl:9-12,76-78
    m4 = """
    module {
      func.func @main(%arg0: tensor<2x3xf32>, %arg1: tensor<3x2xf32>) -> tensor<2x2xf32> {
        %0 = stablehlo.dot_general %arg0, %arg1, contracting_dims = [1] x [0], precision = [HIGH, DEFAULT], algorithm = <lhs_precision_type = f16, rhs_precision_type = f16, accumulation_type = f32, lhs_component_count = 1, rhs_component_count = 1, num_primitive_operations = 1, allow_imprecise_accumulation = false> : (tensor<2x3xf32>, tensor<3x2xf32>) -> tensor<2x2xf32>
        return %0 : tensor<2x2xf32>
      }
    }"""
    A = np.float32([[1, 2, 3], [4, 5, 6]])
    assert np.array_equal(run(m4, [I.Tensor(A, "f32"), I.Tensor(A.T.copy(), "f32")])[0].a, A @ A.T)
    # generic-form reduce with a region (src/mlir/Dialects/StableHLO.jl docstring form)
    m5 = """
    module {
      func.func @main(%arg0: tensor<2x3xi64>) -> tensor<2xi64> {
        %c = stablehlo.constant dense<0> : tensor<i64>
        %0 = "stablehlo.reduce"(%arg0, %c) ({
          ^bb0(%a: tensor<i64>, %b: tensor<i64>):
            %1 = "stablehlo.add"(%a, %b) : (tensor<i64>, tensor<i64>) -> tensor<i64>
            "stablehlo.return"(%1) : (tensor<i64>) -> ()
        }) {dimensions = array<i64: 1>} : (tensor<2x3xi64>, tensor<i64>) -> tensor<2xi64>
        return %0 : tensor<2xi64>
      }
    }"""
    assert run(m5, [I.Tensor(np.array([[1, 2, 3], [4, 5, 6]]), "i64")])[0].a.tolist() == [6, 15]
    # hex and splat constants
    m6 = """
    module {
      func.func @main() -> (tensor<3xf32>, tensor<2xf32>) {
        %cst = stablehlo.constant dense<0.000000e+00> : tensor<3xf32>
        %c2 = stablehlo.constant dense<"0x0000803F00000040"> : tensor<2xf32>
        return %cst, %c2 : tensor<3xf32>, tensor<2xf32>
      }
    }"""
    r = run(m6, [])
    assert r[0].a.tolist() == [0, 0, 0] and r[1].a.tolist() == [1.0, 2.0]


def test_while_loops_against_plain_loops():
    """`stablehlo.while` in the oracle: the example of the reference's binding docstring
    (src/mlir/Dialects/StableHLO.jl:4850-4861) against a Python loop for several starting
    points (including one where the body never runs), a counter-indexed update-slice loop
    against its closed form, the generic form, and a data-dependent trip count."""
    for i0, s0 in [(1, 0), (0, 0), (7, -3), (10, 5), (12, 1)]:
        i, acc = i0, s0
        while i < 10:
            acc, i = acc + 1, i + 1
        r = I.run_text(W.COUNT, [I.Tensor(np.int64(i0), "i64"), I.Tensor(np.int64(s0), "i64")])
        assert (int(r[0].a), int(r[1].a)) == (i, acc)
    x = np.array([10, 20, 30, 40], dtype=np.int64)
    r = I.run_text(W.SETINDEX, [I.Tensor(x, "i64")])
    assert np.array_equal(r[0].a, x + 2 * np.arange(1, 5))
    v = np.array([0.5, -1.0, 3.0, 0.0], dtype=np.float32)
    r = I.run_text(W.GENERIC, [I.Tensor(v, "f32")])
    assert int(r[0].a) == 3 and np.array_equal(r[1].a, 8 * v)
    for n in (0, 1, 5):
        r = I.run_text(W.DATA_DEPENDENT, [I.Tensor(x, "i64"), I.Tensor(np.int64(n), "i64")])
        assert np.array_equal(r[0].a, x * 2 ** n)


@pytest.mark.parametrize("embed", ["pad", "dus"])
def test_while_form_of_the_stencil_equals_the_unrolled_form(embed):
    """`@trace for` (one stablehlo.while carrying a counter and the field) and a plain `for`
    (steps traced one after another) are the same computation: same bits."""
    rng = np.random.default_rng(5)
    full = (4 + 6, 5 + 6, 6 + 6)
    args = [I.Tensor(rng.uniform(-1, 1, full), "f64") for _ in range(4)]
    a = I.run_text(P.stencil(6, 5, 4, steps=4, embed=embed, loop="while"), args)[0].a
    b = I.run_text(P.stencil(6, 5, 4, steps=4, embed=embed), args)[0].a
    assert np.array_equal(a, b)


@pytest.mark.parametrize("embed", ["pad", "dus"])
def test_c_restatement_of_the_stencil_matches_the_interpreter(embed):
    """oracle/stencil_cpu.c (the CPU baseline of the benchmark) against the numpy interpreter:
    same bits, on a grid with odd extents and for several steps."""
    from oracle import build_c
    lib = build_c.load() if os.path.exists(build_c.SO) else None
    if lib is None:
        build_c.build()
        lib = build_c.load()
    nx, ny, nz = 13, 9, 7
    full = (nz + 6, ny + 6, nx + 6)
    rng = np.random.default_rng(2)
    a = [rng.uniform(-1, 1, full) for _ in range(4)]
    ref = I.run_text(P.stencil(nx, ny, nz, steps=3, embed=embed), [I.Tensor(x, "f64") for x in a])[0].a
    got = build_c.stencil_steps(lib, *a, nx, ny, nz, 3, embed=embed)
    assert np.array_equal(got, ref)
    assert lib.rx_oracle_threads() >= 1


def test_c_restatement_of_sinsum_add_is_pinned():
    """oracle/reduce_cpu.c (a CPU baseline of the benchmark): closed forms that a dropped term, a wrong sign or a swapped
    operand would miss (sum over a whole period of sine is the sum of y alone; sin(pi/2) = 1 counts the elements), and
    the numpy interpreter's float64 evaluation of the same module on seeded data."""
    from oracle import build_c
    if not os.path.exists(build_c.SO) or os.path.getmtime(build_c.SO) < os.path.getmtime(os.path.join(os.path.dirname(build_c.SO), "..", "reduce_cpu.c")):
        build_c.build(force=True)
    lib = build_c.load()
    n = 1 << 12
    half_pi = np.full(n, np.pi / 2, dtype=np.float32)
    assert build_c.sinsum_add(lib, half_pi, np.zeros(n, dtype=np.float32)) == pytest.approx(n, rel=1e-7)
    assert build_c.sinsum_add(lib, half_pi, np.full(n, -3.0, dtype=np.float32)) == pytest.approx(-2.0 * n, rel=1e-7)
    period = (2 * np.pi * np.arange(n) / n).astype(np.float32)
    y = np.arange(n, dtype=np.float32) / n
    assert build_c.sinsum_add(lib, period, y) == pytest.approx(float(y.astype(np.float64).sum()), abs=1e-3)
    assert build_c.sinsum_add(lib, -half_pi, y) == pytest.approx(float(y.astype(np.float64).sum()) - n, rel=1e-6)   # sine is odd
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, 100003).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, 100003).astype(np.float32)
    ref = float(I.run_text(P.sinsum_add(100003), [I.tensor(x, "f32"), I.tensor(y, "f32")], hifi=True)[0].a)
    mag = float(np.sum(np.abs(np.sin(x.astype(np.float64)) + y.astype(np.float64))))
    assert abs(build_c.sinsum_add(lib, x, y) - ref) <= 1e-6 * mag


def _c_oracle():
    from oracle import build_c
    srcs = [os.path.join(os.path.dirname(build_c.SO), "..", f) for f in ("stencil_cpu.c", "reduce_cpu.c", "dense_cpu.c")]
    if not os.path.exists(build_c.SO) or any(os.path.getmtime(build_c.SO) < os.path.getmtime(f) for f in srcs):
        build_c.build(force=True)
    return build_c, build_c.load()


def test_c_restatement_of_the_dense_layers_is_pinned():
    """oracle/dense_cpu.c (bias + gelu, softmax, dequantizing scale + RMSNorm: the elementwise parts of the CPU baselines
    of the two dense programs).  Closed forms that a wrong constant, a dropped term or a swapped operand would miss --
    gelu(0) = 0, gelu(x) - gelu(-x) = x, gelu(large) = x, a softmax row sums to one and keeps the order of its inputs, a
    constant row gives 1/n, RMSNorm output has unit mean square and the input's signs, and both are invariant under what
    they should be (softmax under a shift, RMSNorm under a positive factor) -- and the numpy interpreter's evaluation of
    the same modules on seeded bf16 / e4m3 data (float64 accumulation, rounding where the module stores)."""
    build_c, lib = _c_oracle()
    bf = lambda a: lf.bf16_bits_to_f32(lf.f32_to_bf16_bits(np.asarray(a, dtype=np.float32)))
    ones = np.eye(8, dtype=np.float32)
    # one layer with identity weights: bias + gelu alone
    x = bf(np.array([[0.0, 1.0, -1.0, 3.0, -3.0, 20.0, -20.0, 0.5]], dtype=np.float32))
    g = build_c.mlp_f32(lib, x, [ones], [np.zeros(8, np.float32)], softmax=False)[0]
    assert g[0] == 0.0 and g[5] == 20.0 and abs(g[6]) == 0.0
    assert abs((g[1] - g[2]) - 1.0) <= 2.0 ** -7 and abs((g[3] - g[4]) - 3.0) <= 2.0 ** -6      # gelu(x) - gelu(-x) = x
    assert abs(g[1] - 0.8411919906082768) <= 2.0 ** -8 and abs(g[7] - 0.34571400982514394) <= 2.0 ** -9   # tanh form, float64 values
    gb = build_c.mlp_f32(lib, np.zeros((1, 8), np.float32), [ones], [x[0].copy()], softmax=False)[0]
    assert np.array_equal(gb, g)                                                               # the bias enters like the product
    # softmax
    fp = __import__("ctypes").POINTER(__import__("ctypes").c_float)
    r = np.array([[1.0, 2.0, 3.0, 4.0], [7.0, 7.0, 7.0, 7.0], [101.0, 102.0, 103.0, 104.0]], dtype=np.float32)
    lib.rx_oracle_softmax_rows_bf16(r.ctypes.data_as(fp), 3, 4)
    assert np.all(np.abs(r.sum(axis=1) - 1.0) <= 2.0 ** -7) and np.all(np.diff(r[0]) > 0)
    assert np.array_equal(r[1], np.full(4, 0.25, np.float32)) and np.array_equal(r[0], r[2])    # shift invariance
    assert abs(r[0][3] - 0.6439142598879724) <= 2.0 ** -9
    # RMSNorm
    v = np.array([[3.0, -4.0, 0.0, 0.0], [30.0, -40.0, 0.0, 0.0]], dtype=np.float32)
    lib.rx_oracle_scale_rmsnorm_bf16(v.ctypes.data_as(fp), 1.0, 0.0, 2, 4)
    assert np.array_equal(v[0], v[1]) and abs(v[0][0] - 1.2) <= 2.0 ** -8 and abs(v[0][1] + 1.6) <= 2.0 ** -8
    v2 = np.array([[3.0, -4.0, 0.0, 0.0]], dtype=np.float32)
    lib.rx_oracle_scale_rmsnorm_bf16(v2.ctypes.data_as(fp), 2.0, 0.0, 1, 4)
    assert np.array_equal(v2[0], v[0])                                                          # the scale cancels in the norm
    # against the interpreter: the whole dense network and the FP8 layer on seeded data
    batch, widths = 24, (32, 64, 48, 40)
    rng = np.random.default_rng(0)
    raw = [lf.f32_to_bf16_bits(rng.normal(size=(batch, widths[0])).astype(np.float32))]
    for l in range(3):
        lim = np.sqrt(6.0 / (widths[l] + widths[l + 1]))
        raw.append(lf.f32_to_bf16_bits(rng.uniform(-lim, lim, size=(widths[l], widths[l + 1])).astype(np.float32)))
        raw.append(lf.f32_to_bf16_bits((rng.normal(size=(widths[l + 1],)) * 0.1).astype(np.float32)))
    args = [I.Tensor.from_bytes(a.tobytes(), "bf16", a.shape) for a in raw]
    ref = run(P.mlp(batch, widths), args, hifi=True, excess=True)[0].a.astype(np.float64)
    f32 = [lf.bf16_bits_to_f32(a) for a in raw]
    got = build_c.mlp_f32(lib, f32[0], f32[1::2], f32[2::2])
    assert np.max(np.abs(got - ref)) <= 2e-2 * np.max(np.abs(ref))
    n, k = 40, 64
    act = lf.f32_to_bf16_bits(rng.normal(size=(batch, k)).astype(np.float32))
    codes = rng.integers(0, 256, size=(n, k), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38
    sw = np.float32(0.0123)
    ref = run(P.fp8_linear(batch, k, n), [I.Tensor.from_bytes(act.tobytes(), "bf16", (batch, k)), I.Tensor.from_bytes(codes.tobytes(), "f8E4M3FN", (n, k)),
                                          I.Tensor(sw, "f32")], hifi=True, excess=True)[0].a.astype(np.float64)
    a32 = lf.bf16_bits_to_f32(act)
    sa = np.float32(np.abs(a32).max()) / np.float32(448.0)
    q = lf.e4m3fn_bits_to_f32(lf.f32_to_e4m3fn_bits(np.clip(a32 / sa, -448.0, 448.0).astype(np.float32)))
    got = build_c.fp8_linear_f32(lib, q, lf.e4m3fn_bits_to_f32(codes), sa * sw)
    assert np.max(np.abs(got - ref)) <= 1e-2 * np.max(np.abs(ref))


def test_conditionals_against_plain_python():
    x = np.arange(8, dtype=np.float32) / 4
    for s in (2.0, -3.0):
        a, b = I.run_text(W.IF, [I.tensor(x, "f32"), I.tensor(np.float32(s), "f32")])
        if s > 0:
            assert np.allclose(a.a, np.sin(x), rtol=1e-6) and float(b.a) == 1.0
        else:
            assert np.array_equal(a.a, x * np.float32(s)) and float(b.a) == -s
    y = np.random.default_rng(0).normal(size=(4, 5))
    for idx, want in ((0, np.exp(y)), (1, y * y), (2, -y), (7, -y), (-1, -y)):
        got = I.run_text(W.CASE, [I.tensor(y, "f64"), I.Tensor(np.int32(idx), "i32")])[0].a
        assert np.allclose(got, want, rtol=1e-14)
    assert np.allclose(I.run_text(W.IF_CONST, [I.tensor(x, "f32")])[0].a, np.cos(x), rtol=1e-6)


def test_chlo_math_ops_satisfy_their_identities():
    """The oracle's chlo unary ops (scipy / numpy routines, reference src/Ops.jl:398-436) against what the
    mathematics fixes: inverse pairs, the hyperbolic identity, digamma's recurrence and psi(1) = -gamma,
    lgamma at the integers, erfc = 1 - erf; popcnt / count_leading_zeros on known values."""
    import math
    from oracle import stablehlo_interp as I

    def run(op, x, dt="f64"):
        t = "tensor<%dx%s>" % (len(x), dt)
        text = "module {\n func.func @main(%%arg0: %s) -> %s {\n  %%0 = %s %%arg0 : %s%s\n  return %%0 : %s\n }\n}\n" % (
            t, t, op, t, " -> " + t if op.startswith("chlo.") else "", t)
        return I.run_text(text, [I.Tensor(np.asarray(x, dtype=I.NP_OF[dt]), dt)])[0].a

    x = np.linspace(0.05, 0.95, 19)
    assert np.allclose(np.cos(run("chlo.acos", x)), x) and np.allclose(np.sin(run("chlo.asin", x)), x) and np.allclose(np.tan(run("chlo.atan", x)), x)
    assert np.allclose(np.cosh(run("chlo.acosh", 1 + x)), 1 + x) and np.allclose(np.sinh(run("chlo.asinh", x)), x) and np.allclose(np.tanh(run("chlo.atanh", x)), x)
    assert np.allclose(run("chlo.cosh", x) ** 2 - run("chlo.sinh", x) ** 2, 1.0)
    assert np.allclose(run("chlo.erf", run("chlo.erf_inv", x)), x) and np.allclose(run("chlo.erfc", x), 1 - run("chlo.erf", x))
    assert np.allclose(run("chlo.lgamma", [1.0, 2.0, 5.0, 11.0]), [0.0, 0.0, math.log(24.0), math.log(3628800.0)])
    assert np.allclose(run("chlo.digamma", [1.0]), [-0.5772156649015329])
    assert np.allclose(run("chlo.digamma", x + 1) - run("chlo.digamma", x), 1 / x)
    assert run("stablehlo.popcnt", [0, 1, 255, -1, 1 << 20], "i32").tolist() == [0, 1, 8, 32, 1]
    assert run("stablehlo.count_leading_zeros", [0, 1, 255, -1, 1 << 20], "i32").tolist() == [32, 31, 24, 0, 11]
    assert run("stablehlo.count_leading_zeros", [0, 1, 127, -1], "i8").tolist() == [8, 7, 1, 0]


def test_integer_division_rules_against_python_integers():
    """Quotients truncate toward zero and remainders take the dividend's sign (C and XLA alike);
    x / 0 is all ones and x % 0 is x; MIN / -1 wraps to MIN and MIN % -1 is 0; the all-ones divisor
    of an unsigned type is an ordinary number."""
    for dt in ("i8", "i16", "i32", "i64", "ui8", "ui16", "ui32", "ui64"):
        info = np.iinfo(I.NP_OF[dt])
        bits = info.bits
        vals = sorted({0, 1, 2, 3, 7, 100, info.max, info.max - 1, info.min, info.min + 1, -1 if info.min else info.max, -7 if info.min else 9})
        a = np.array([x for x in vals for _ in vals], dtype=I.NP_OF[dt])
        b = np.array([y for _ in vals for y in vals], dtype=I.NP_OF[dt])
        q = I._binary("divide", I.Tensor(a, dt), I.Tensor(b, dt), dt).a
        r = I._binary("remainder", I.Tensor(a, dt), I.Tensor(b, dt), dt).a

        def wrap(v):
            v &= (1 << bits) - 1
            return v - (1 << bits) if info.min and v >> (bits - 1) else v
        for x, y, qq, rr in zip(a.tolist(), b.tolist(), q.tolist(), r.tolist()):
            if y == 0:
                eq, er = wrap(-1), x
            else:
                t = abs(x) // abs(y) * (1 if (x < 0) == (y < 0) else -1)
                eq, er = wrap(t), x - t * y
            assert (qq, rr) == (eq, er), (dt, x, y, qq, rr, eq, er)


def test_float_to_integer_conversion_against_python_int():
    """In range: Python's int() (truncation).  Beyond the range the oracle saturates and maps NaN to 0,
    which is XLA's choice and not fixed by the specification (parity unpinned there)."""
    rng = np.random.default_rng(5)
    for dt in ("i8", "ui8", "i16", "ui16", "i32", "ui32", "i64", "ui64"):
        info = np.iinfo(I.NP_OF[dt])
        x = rng.uniform(max(info.min, -2.0 ** 52), min(info.max, 2.0 ** 52), 500)
        got = I._convert(I.Tensor(x, "f64"), dt).a.tolist()
        assert got == [int(v) for v in x.tolist()], dt
        edge = I._convert(I.Tensor(np.array([1e30, -1e30, np.nan, np.inf, -np.inf]), "f64"), dt).a.tolist()
        assert edge == [info.max, info.min, 0, info.max, info.min], (dt, edge)
