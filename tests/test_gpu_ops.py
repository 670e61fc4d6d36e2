"""Op-level GPU parity: the reference's own known-answer tests for the ops on the
hot path (test/core/ops.jl, test/core/map_reduction.jl, test/core/math_ops.jl,
src/TestUtils.jl fixture generator), plus bit-exact checks of conversions and
index ops against the oracle."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run, rel_err, max_rel_to_scale
from oracle import stablehlo_interp as I
from oracle import lowfloat as lf

pytestmark = pytest.mark.gpu


def _tt(shape, dt):
    return "tensor<" + "x".join([str(s) for s in shape] + [dt]) + ">"


def mod(args, ret, body):
    sig = ", ".join("%%arg%d: %s" % (k, t) for k, t in enumerate(args))
    return "module {\n  func.func @main(%s) -> %s {\n%s  }\n}\n" % (sig, ret, body)


def construct_test_array(dtype, *dims):
    """Reactant.TestUtils.construct_test_array (src/TestUtils.jl:9-23), Julia (column-major) order."""
    n = int(np.prod(dims))
    flat = np.arange(1, n + 1)
    a = (flat / n).astype(dtype) if np.issubdtype(dtype, np.floating) else flat.astype(dtype)
    return a.reshape(dims, order="F")


def both(rx, client, text, args, hifi=True):
    got, _ = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=hifi)
    return got, ref


# ---- pad (test/core/ops.jl:534-557) -----------------------------------------------
@pytest.mark.parametrize("low,high,interior,expect", [
    ([1], [0], [0], [0, 1, 2, 3, 4]), ([0], [1], [0], [1, 2, 3, 4, 0]), ([0], [0], [1], [1, 0, 2, 0, 3, 0, 4])])
def test_pad_1d_reference_vectors(rx, client, low, high, interior, expect):
    n = len(expect)
    text = mod([_tt([4], "i64"), "tensor<i64>"], _tt([n], "i64"),
               "    %%0 = stablehlo.pad %%arg0, %%arg1, low = %s, high = %s, interior = %s : (tensor<4xi64>, tensor<i64>) -> %s\n"
               "    return %%0 : %s\n" % (low, high, interior, _tt([n], "i64"), _tt([n], "i64")))
    got, ref = both(rx, client, text, [I.Tensor(np.array([1, 2, 3, 4]), "i64"), I.Tensor(np.array(0), "i64")])
    assert got[0].a.tolist() == expect and ref[0].a.tolist() == expect


@pytest.mark.parametrize("low,high,interior,expect", [
    ([1, 2], [0, 0], [0, 0], [[0, 0, 0, 0], [0, 0, 1, 2], [0, 0, 3, 4]]),
    ([0, 0], [1, 2], [0, 0], [[1, 2, 0, 0], [3, 4, 0, 0], [0, 0, 0, 0]]),
    ([0, 0], [0, 0], [1, 2], [[1, 0, 0, 2], [0, 0, 0, 0], [3, 0, 0, 4]])])
def test_pad_2d_reference_vectors(rx, client, low, high, interior, expect):
    # Julia [1 2; 3 4] arrives as raw [[1,3],[2,4]]; Julia dims (low etc.) are reversed on the wire
    E = np.array(expect)
    raw_in = np.array([[1, 2], [3, 4]]).T.copy()
    rl, rh, ri = low[::-1], high[::-1], interior[::-1]
    oshape = list(E.T.shape)
    text = mod([_tt([2, 2], "i64"), "tensor<i64>"], _tt(oshape, "i64"),
               "    %%0 = stablehlo.pad %%arg0, %%arg1, low = %s, high = %s, interior = %s : (tensor<2x2xi64>, tensor<i64>) -> %s\n"
               "    return %%0 : %s\n" % (rl, rh, ri, _tt(oshape, "i64"), _tt(oshape, "i64")))
    got, ref = both(rx, client, text, [I.Tensor(raw_in, "i64"), I.Tensor(np.array(0), "i64")])
    assert np.array_equal(got[0].a.T, E) and np.array_equal(ref[0].a.T, E)


def test_slice_reference_vectors(rx, client):
    # Ops.slice(x, [2], [3]) == [2, 3]  (1-based inclusive -> [1:3])   test/core/ops.jl:815-819
    text = mod([_tt([4], "i64")], _tt([2], "i64"),
               "    %0 = stablehlo.slice %arg0 [1:3] : (tensor<4xi64>) -> tensor<2xi64>\n    return %0 : tensor<2xi64>\n")
    got, ref = both(rx, client, text, [I.Tensor(np.array([1, 2, 3, 4]), "i64")])
    assert got[0].a.tolist() == [2, 3] == ref[0].a.tolist()


# ---- elementwise known answers (test/core/ops.jl:788-824) ------------------------
def test_sine_sqrt_reference_vectors(rx, client):
    x = np.array([0.0, np.pi / 2, np.pi, 3 * np.pi / 2, 2 * np.pi])
    text = mod([_tt([5], "f64")], _tt([5], "f64"), "    %0 = stablehlo.sine %arg0 : tensor<5xf64>\n    return %0 : tensor<5xf64>\n")
    got, ref = both(rx, client, text, [I.Tensor(x, "f64")])
    assert np.allclose(got[0].a, [0, 1, 0, -1, 0], atol=1e-15) and np.allclose(ref[0].a, [0, 1, 0, -1, 0], atol=1e-15)
    text = mod([_tt([4], "f64")], _tt([4], "f64"), "    %0 = stablehlo.sqrt %arg0 : tensor<4xf64>\n    return %0 : tensor<4xf64>\n")
    got, ref = both(rx, client, text, [I.Tensor(np.array([1.0, 4.0, 9.0, 16.0]), "f64")])
    assert got[0].a.tolist() == [1.0, 2.0, 3.0, 4.0] == ref[0].a.tolist()


UNARY_F32 = ["sine", "cosine", "tanh", "exponential", "log", "sqrt", "rsqrt", "abs", "negate", "logistic", "floor", "ceil",
             "sign", "exponential_minus_one", "log_plus_one", "cbrt", "round_nearest_even"]


@pytest.mark.parametrize("op", UNARY_F32)
def test_unary_f32_maps(rx, client, op):
    """fp32 maps agree with the f64-evaluated library routine to 1e-6 relative (trig sweep on the
    reference's fixture array, test/core/math_ops.jl:33-43, plus a seeded wide sweep)."""
    fix = construct_test_array(np.float32, 4, 16)[:, :7]
    rng = np.random.default_rng(0)
    wide = rng.uniform(0.05, 8.0, 4096).astype(np.float32) if op in ("log", "sqrt", "rsqrt", "log_plus_one") \
        else rng.uniform(-8.0, 8.0, 4096).astype(np.float32)
    for x in (np.ascontiguousarray(fix.T), wide):
        t = _tt(x.shape, "f32")
        text = mod([t], t, "    %%0 = stablehlo.%s %%arg0 : %s\n    return %%0 : %s\n" % (op, t, t))
        got, _ = gpu_run(rx, client, text, [I.Tensor(x, "f32")])
        ref64 = oracle_run(text.replace("f32", "f64"), [I.Tensor(x.astype(np.float64), "f64")])[0].a
        err = np.abs(got[0].a.astype(np.float64) - ref64) / np.maximum(np.abs(ref64), 1e-30)
        ok = (err <= 1e-6) | (np.abs(got[0].a.astype(np.float64) - ref64) <= 1e-7)
        assert ok.all(), (op, float(err.max()))


BINARY = ["add", "subtract", "multiply", "divide", "maximum", "minimum", "power", "remainder"]


@pytest.mark.parametrize("op", BINARY)
@pytest.mark.parametrize("dt", ["f32", "f64", "i32", "i64", "ui8"])
def test_binary_ops(rx, client, op, dt):
    rng = np.random.default_rng(1)
    n = 1000
    if dt.startswith("f"):
        a = rng.uniform(0.5, 4.0, n).astype(I.NP_OF[dt])
        b = rng.uniform(0.5, 3.0, n).astype(I.NP_OF[dt])
    else:
        a = rng.integers(0 if dt == "ui8" else -50, 50, n).astype(I.NP_OF[dt])
        b = rng.integers(1, 5, n).astype(I.NP_OF[dt])
        if op == "power":
            a = (np.abs(a) % 6).astype(I.NP_OF[dt])
            b = (b % 4).astype(I.NP_OF[dt])
    t = _tt([n], dt)
    text = mod([t, t], t, "    %%0 = stablehlo.%s %%arg0, %%arg1 : %s\n    return %%0 : %s\n" % (op, t, t))
    got, ref = both(rx, client, text, [I.Tensor(a, dt), I.Tensor(b, dt)])
    if dt.startswith("f"):
        tol = 1e-6 if dt == "f32" else 1e-14
        assert rel_err(got[0].a, ref[0].a) <= tol
    else:
        assert np.array_equal(got[0].a, ref[0].a)   # integers: bit-exact


# ---- reductions (test/core/ops.jl:1207-1235, test/core/map_reduction.jl) ---------
@pytest.mark.parametrize("dims,body,init", [([1], "multiply", 1), ([0, 2], "add", 0), ([0, 1, 2], "add", 0)])
def test_int_reduce_reference(rx, client, dims, body, init):
    A = construct_test_array(np.int64, 3, 4, 5)       # Julia 3x4x5
    raw = np.ascontiguousarray(A.T)                   # wire layout 5x4x3
    jd = [d + 1 for d in dims]                        # these are the Julia dims of the reference test ...
    wire = sorted(2 - d for d in dims)                # ... which are reversed on the wire
    oshape = [s for k, s in enumerate(raw.shape) if k not in wire]
    text = mod([_tt(raw.shape, "i64"), "tensor<i64>"], _tt(oshape, "i64"),
               "    %%0 = stablehlo.reduce(%%arg0 init: %%arg1) applies stablehlo.%s across dimensions = %s : (%s, tensor<i64>) -> %s\n"
               "    return %%0 : %s\n" % (body, wire, _tt(raw.shape, "i64"), _tt(oshape, "i64"), _tt(oshape, "i64")))
    got, ref = both(rx, client, text, [I.Tensor(raw, "i64"), I.Tensor(np.array(init), "i64")])
    f = np.multiply.reduce if body == "multiply" else np.add.reduce
    expect = A
    for d in sorted(dims, reverse=True):
        expect = f(expect, axis=d)
    assert np.array_equal(np.asarray(got[0].a).T, np.asarray(expect))
    assert np.array_equal(np.asarray(ref[0].a).T, np.asarray(expect))
    assert jd


def test_float_sum_closed_form(rx, client):
    # sum(construct_test_array(Float64, 2, 10)) == 210/20 == 10.5   (test/core/map_reduction.jl:8-19)
    A = construct_test_array(np.float64, 2, 10)
    raw = np.ascontiguousarray(A.T)
    text = mod([_tt(raw.shape, "f64")], "tensor<f64>",
               "    %%c = stablehlo.constant dense<0.000000e+00> : tensor<f64>\n"
               "    %%0 = stablehlo.reduce(%%arg0 init: %%c) applies stablehlo.add across dimensions = [0, 1] : (%s, tensor<f64>) -> tensor<f64>\n"
               "    return %%0 : tensor<f64>\n" % _tt(raw.shape, "f64"))
    got, ref = both(rx, client, text, [I.Tensor(raw, "f64")])
    assert abs(float(got[0].a) - 10.5) < 1e-12 and abs(float(ref[0].a) - 10.5) < 1e-12


@pytest.mark.parametrize("shape,dims", [((64, 1000), [1]), ((1000, 64), [0]), ((7, 33, 65), [2]), ((7, 33, 65), [1, 2]),
                                        ((7, 33, 65), [0]), ((5, 6, 7), [0, 2]), ((300, 4096), [1]), ((3, 70), [1]),
                                        # few outputs, long reductions: the reduced dimension is cut into chunks
                                        ((1000, 520), [0]), ((37, 130, 9), [0, 1]), ((130, 37, 9), [0, 1]), ((3, 1030, 2), [1]),
                                        ((2049, 3), [0])])
@pytest.mark.parametrize("body", ["add", "maximum", "minimum"])
def test_partial_reductions_f32(rx, client, shape, dims, body):
    x = np.random.default_rng(3).normal(size=shape).astype(np.float32)
    oshape = [s for k, s in enumerate(shape) if k not in dims]
    init = {"add": "0.000000e+00", "maximum": "0xFF800000", "minimum": "0x7F800000"}[body]
    text = mod([_tt(shape, "f32")], _tt(oshape, "f32"),
               "    %%c = stablehlo.constant dense<%s> : tensor<f32>\n"
               "    %%0 = stablehlo.reduce(%%arg0 init: %%c) applies stablehlo.%s across dimensions = %s : (%s, tensor<f32>) -> %s\n"
               "    return %%0 : %s\n" % (init, body, dims, _tt(shape, "f32"), _tt(oshape, "f32"), _tt(oshape, "f32")))
    got, ref = both(rx, client, text, [I.Tensor(x, "f32")])
    n = int(np.prod([shape[d] for d in dims]))
    if body == "add":
        scale = np.abs(x).sum(axis=tuple(dims))
        assert np.all(np.abs(got[0].a.astype(np.float64) - ref[0].a) <= 1e-5 * np.sqrt(n) * np.maximum(scale / n, 1e-30) + 1e-6)
    else:
        assert np.array_equal(got[0].a, ref[0].a)


def test_bool_and_int_widening_sum(rx, client):
    # sum(::Array{Bool}) widens to Int64 before the reduce (src/TracedRArray.jl:200-216)
    x = (np.random.default_rng(0).uniform(size=(17, 9)) > 0.5)
    text = mod([_tt(x.shape, "i1")], "tensor<i64>",
               "    %%c = stablehlo.constant dense<0> : tensor<i64>\n"
               "    %%0 = stablehlo.convert %%arg0 : (%s) -> %s\n"
               "    %%1 = stablehlo.reduce(%%0 init: %%c) applies stablehlo.add across dimensions = [0, 1] : (%s, tensor<i64>) -> tensor<i64>\n"
               "    return %%1 : tensor<i64>\n" % (_tt(x.shape, "i1"), _tt(x.shape, "i64"), _tt(x.shape, "i64")))
    got, ref = both(rx, client, text, [I.Tensor(x, "i1")])
    assert int(got[0].a) == int(x.sum()) == int(ref[0].a)


# ---- conversions: bit-exact --------------------------------------------------------
def _interesting_f32():
    vals = [0.0, -0.0, np.inf, -np.inf, np.nan, 448.0, 449.0, 463.99, 464.0, 464.01, 480.0, 1e9, 2.0 ** -6, 2.0 ** -9,
            2.0 ** -10, 2.0 ** -10 * 1.0001, 2.0 ** -11, 57344.0, 61439.0, 61440.0, 65504.0, 1e-30, 3.0e38]
    codes = np.arange(256, dtype=np.uint8)
    rep = lf.e4m3fn_bits_to_f32(codes)
    rep = rep[np.isfinite(rep)]
    mids = (np.sort(rep)[1:] + np.sort(rep)[:-1]) / 2           # ties
    rng = np.random.default_rng(0)
    rnd = np.concatenate([rng.normal(size=20000) * s for s in (1e-3, 1.0, 100.0, 1000.0)])
    bits = rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = np.concatenate([np.array(vals, dtype=np.float32), -np.array(vals, dtype=np.float32), rep, mids,
                        np.nextafter(mids.astype(np.float32), np.float32(np.inf)), np.nextafter(mids.astype(np.float32), np.float32(-np.inf)),
                        rnd.astype(np.float32), bits]).astype(np.float32)
    return x


@pytest.mark.parametrize("dt", ["bf16", "f8E4M3FN", "f8E5M2", "f16"])
def test_convert_f32_to_narrow_bit_exact(rx, client, dt):
    x = _interesting_f32()
    t, o = _tt(x.shape, "f32"), _tt(x.shape, dt)
    text = mod([t], o, "    %%0 = stablehlo.convert %%arg0 : (%s) -> %s\n    return %%0 : %s\n" % (t, o, o))
    got, ref = both(rx, client, text, [I.Tensor(x, "f32")])
    gb, rb = np.frombuffer(got[0].to_bytes(), np.uint8), np.frombuffer(ref[0].to_bytes(), np.uint8)
    nan = np.isnan(got[0].a) & np.isnan(ref[0].a)
    esz = I.ITEMSIZE[dt]
    same = (gb.reshape(-1, esz) == rb.reshape(-1, esz)).all(axis=1)
    assert (same | nan).all(), x[~(same | nan)][:10]


def test_convert_of_a_clamped_value_to_e4m3_bit_exact(rx, client):
    """clamp(x, -448, 448) followed by the conversion to e4m3 (a quantization): the conversion is the hardware
    instruction alone there; the same bytes as the oracle's on every interesting float32 (ties, subnormals, both
    zeros, values far outside the range), NaN stays NaN."""
    x = _interesting_f32()
    t, o = _tt(x.shape, "f32"), _tt(x.shape, "f8E4M3FN")
    text = mod([t], o, "    %%lo = stablehlo.constant dense<-448.0> : %s\n    %%hi = stablehlo.constant dense<448.0> : %s\n"
               "    %%0 = stablehlo.clamp %%lo, %%arg0, %%hi : %s\n    %%1 = stablehlo.convert %%0 : (%s) -> %s\n    return %%1 : %s\n" % (t, t, t, t, o, o))
    assert "rx_f32_to_e4m3_inrange" in rx.compile_offline(text, with_source=True)
    got, ref = both(rx, client, text, [I.Tensor(x, "f32")])
    gb, rb = np.frombuffer(got[0].to_bytes(), np.uint8), np.frombuffer(ref[0].to_bytes(), np.uint8)
    nan = np.isnan(got[0].a) & np.isnan(ref[0].a)
    assert ((gb == rb) | nan).all(), x[~((gb == rb) | nan)][:10]
    assert np.array_equal(np.isnan(got[0].a), np.isnan(ref[0].a))


@pytest.mark.parametrize("dt", ["bf16", "f8E4M3FN", "f8E5M2", "f16"])
def test_convert_narrow_to_f32_exact(rx, client, dt):
    n = 65536 if I.ITEMSIZE[dt] == 2 else 256
    raw = np.arange(n, dtype=np.uint16 if n > 256 else np.uint8)
    x = I.Tensor.from_bytes(raw.tobytes(), dt, (n,))
    t, o = _tt([n], dt), _tt([n], "f32")
    text = mod([t], o, "    %%0 = stablehlo.convert %%arg0 : (%s) -> %s\n    return %%0 : %s\n" % (t, o, o))
    got, ref = both(rx, client, text, [x])
    assert np.array_equal(got[0].a.view(np.uint32)[~np.isnan(ref[0].a)], ref[0].a.view(np.uint32)[~np.isnan(ref[0].a)])
    assert np.array_equal(np.isnan(got[0].a), np.isnan(ref[0].a))


# ---- index ops: bit-exact on integers --------------------------------------------------
def test_index_op_chain(rx, client):
    x = np.arange(4 * 6 * 8, dtype=np.int32).reshape(4, 6, 8)
    t = _tt(x.shape, "i32")
    body = ("    %%0 = stablehlo.transpose %%arg0, dims = [2, 0, 1] : (%s) -> tensor<8x4x6xi32>\n"
            "    %%1 = stablehlo.slice %%0 [1:7:2, 0:4, 2:6] : (tensor<8x4x6xi32>) -> tensor<3x4x4xi32>\n"
            "    %%2 = stablehlo.reshape %%1 : (tensor<3x4x4xi32>) -> tensor<12x4xi32>\n"
            "    %%3 = stablehlo.iota dim = 1 : tensor<12x4xi32>\n"
            "    %%4 = stablehlo.add %%2, %%3 : tensor<12x4xi32>\n"
            "    %%5 = stablehlo.broadcast_in_dim %%arg1, dims = [1] : (tensor<4xi32>) -> tensor<12x4xi32>\n"
            "    %%6 = stablehlo.multiply %%4, %%5 : tensor<12x4xi32>\n"
            "    %%7 = stablehlo.concatenate %%6, %%2, dim = 0 : (tensor<12x4xi32>, tensor<12x4xi32>) -> tensor<24x4xi32>\n"
            "    %%c = stablehlo.constant dense<-1> : tensor<i32>\n"
            "    %%8 = stablehlo.pad %%7, %%c, low = [1, -1], high = [2, 1], interior = [0, 1] : (tensor<24x4xi32>, tensor<i32>) -> tensor<27x7xi32>\n"
            "    return %%8 : tensor<27x7xi32>\n" % t)
    text = mod([t, _tt([4], "i32")], "tensor<27x7xi32>", body)
    got, ref = both(rx, client, text, [I.Tensor(x, "i32"), I.Tensor(np.array([3, -2, 7, 1], dtype=np.int32), "i32")])
    assert np.array_equal(got[0].a, ref[0].a)


def test_compare_select_clamp(rx, client):
    rng = np.random.default_rng(5)
    a = rng.normal(size=(33, 17)).astype(np.float32)
    b = rng.normal(size=(33, 17)).astype(np.float32)
    t, tb = _tt(a.shape, "f32"), _tt(a.shape, "i1")
    body = ("    %%0 = stablehlo.compare  GT, %%arg0, %%arg1,  FLOAT : (%s, %s) -> %s\n"
            "    %%1 = stablehlo.select %%0, %%arg0, %%arg1 : %s, %s\n"
            "    %%lo = stablehlo.constant dense<-5.000000e-01> : tensor<f32>\n"
            "    %%hi = stablehlo.constant dense<5.000000e-01> : tensor<f32>\n"
            "    %%2 = stablehlo.clamp %%lo, %%1, %%hi : (tensor<f32>, %s, tensor<f32>) -> %s\n"
            "    return %%2 : %s\n" % (t, t, tb, tb, t, t, t, t))
    got, ref = both(rx, client, mod([t, t], t, body), [I.Tensor(a, "f32"), I.Tensor(b, "f32")])
    assert np.array_equal(got[0].a, ref[0].a)


def test_map_op_generic_form(rx, client):
    """stablehlo.map in generic form (src/mlir/Dialects/StableHLO.jl:2686-2705 spec example)."""
    a = np.arange(6, dtype=np.int64).reshape(2, 3)
    b = np.arange(6, 12, dtype=np.int64).reshape(2, 3)
    text = ('module {\n  func.func @main(%arg0: tensor<2x3xi64>, %arg1: tensor<2x3xi64>) -> tensor<2x3xi64> {\n'
            '    %0 = "stablehlo.map"(%arg0, %arg1) ({\n'
            '      ^bb0(%a: tensor<i64>, %b: tensor<i64>):\n'
            '        %1 = stablehlo.multiply %a, %b : tensor<i64>\n'
            '        stablehlo.return %1 : tensor<i64>\n'
            '    }) {dimensions = array<i64: 0, 1>} : (tensor<2x3xi64>, tensor<2x3xi64>) -> tensor<2x3xi64>\n'
            '    return %0 : tensor<2x3xi64>\n  }\n}\n')
    got, ref = both(rx, client, text, [I.Tensor(a, "i64"), I.Tensor(b, "i64")])
    assert np.array_equal(got[0].a, a * b) and np.array_equal(ref[0].a, a * b)


def test_empty_and_scalar_shapes(rx, client):
    t0 = _tt([0], "f32")
    text = mod([t0], "tensor<f32>",
               "    %%c = stablehlo.constant dense<1.500000e+00> : tensor<f32>\n"
               "    %%0 = stablehlo.reduce(%%arg0 init: %%c) applies stablehlo.add across dimensions = [0] : (%s, tensor<f32>) -> tensor<f32>\n"
               "    return %%0 : tensor<f32>\n" % t0)
    got, ref = both(rx, client, text, [I.Tensor(np.zeros(0, np.float32), "f32")])
    assert float(got[0].a) == 1.5 == float(ref[0].a)
    text = mod(["tensor<f32>", "tensor<f32>"], "tensor<f32>", "    %0 = stablehlo.add %arg0, %arg1 : tensor<f32>\n    return %0 : tensor<f32>\n")
    got, _ = gpu_run(rx, client, text, [I.Tensor(np.float32(2.0), "f32"), I.Tensor(np.float32(2.0), "f32")])
    assert float(got[0].a) == 4.0   # test/core/ops.jl:1066-1082


# ---- stablehlo.while with a static trip count ------------------------------------------------
def test_while_counter_indexed_update_slice(rx, client):
    import _while_modules as W
    x = np.array([10, 20, 30, 40], dtype=np.int64)
    got, ref = both(rx, client, W.SETINDEX, [I.Tensor(x, "i64")])
    assert np.array_equal(got[0].a, x + 2 * np.arange(1, 5)) and np.array_equal(got[0].a, ref[0].a)


def test_while_generic_form_returns_counter_and_value(rx, client):
    import _while_modules as W
    v = np.array([0.5, -1.0, 3.0, 0.0], dtype=np.float32)
    got, ref = both(rx, client, W.GENERIC, [I.Tensor(v, "f32")])
    assert int(got[0].a) == 3 and np.array_equal(got[1].a, 8 * v)
    assert np.array_equal(got[1].a, ref[1].a)


# ---- division by a broadcast scalar ------------------------------------------------------------
@pytest.mark.parametrize("divisor", [3.0, 0.1, 448.0, 1e-40, 3.4e38, 0.0, -7.25, float("inf"), 1.9999999, 0.99999994, 0.012125223,
                                     3.6379788e-12, 3.63797e-12, 5.4975581e11, 5.49756e11, -1.0000001])
def test_divide_by_a_broadcast_scalar_is_correctly_rounded(rx, client, divisor):
    """x / s with s one value for the whole tensor is evaluated as a product with the double
    reciprocal; it must round exactly like the IEEE division (bit-for-bit against numpy),
    including subnormal and huge divisors, divisors with an all-ones mantissa, zeros, infinities
    and quotients next to a tie."""
    n = 1 << 20
    rng = np.random.default_rng(5)
    x = rng.integers(0, 2 ** 32, n, dtype=np.uint64).astype(np.uint32).view(np.float32).copy()
    x[: n // 2] = rng.normal(size=n // 2).astype(np.float32) * np.float32(100)
    # numerators that put the quotient half an ulp away from a float: (2k+1) * s in float
    s32 = np.float32(divisor)
    if np.isfinite(s32) and s32 != 0:
        k = (rng.integers(2 ** 23, 2 ** 24, 4096) * 2 + 1).astype(np.float64)
        with np.errstate(all="ignore"):
            x[-4096:] = (k * np.float64(s32)).astype(np.float32)
    text = mod([_tt([n], "f32"), "tensor<f32>"], _tt([n], "f32"),
               "    %0 = stablehlo.broadcast_in_dim %arg1, dims = [] : (tensor<f32>) -> tensor<{n}xf32>\n".replace("{n}", str(n)) +
               "    %1 = stablehlo.divide %arg0, %0 : tensor<{n}xf32>\n    return %1 : tensor<{n}xf32>\n".replace("{n}", str(n)))
    got, _ = gpu_run(rx, client, text, [I.Tensor(x, "f32"), I.Tensor(s32, "f32")])
    with np.errstate(all="ignore"):
        want = x / s32
    same = got[0].a.view(np.uint32) == want.view(np.uint32)
    both_nan = np.isnan(got[0].a) & np.isnan(want)
    assert (same | both_nan).all(), (x[~(same | both_nan)][:5], got[0].a[~(same | both_nan)][:5], want[~(same | both_nan)][:5])


# ---- maps with transposed reads (64x64 tiles through LDS) ---------------------------------------
def _tt_(shape, dt):
    return "tensor<" + "".join("%dx" % d for d in shape) + dt + ">"


@pytest.mark.parametrize("shape,perm,dt", [((300, 257), (1, 0), "f32"), ((257, 300), (1, 0), "f64"), ((64, 1030), (1, 0), "i32"),
                                           ((9, 130, 70), (0, 2, 1), "f32"), ((70, 33, 129), (2, 1, 0), "f32"),
                                           ((3, 66, 5, 80), (0, 3, 2, 1), "bf16"), ((130, 20, 70), (1, 2, 0), "f32"),
                                           # both dimensions whole 16-byte vectors: the vector form, tiles of 64 x 128 (64 x 64 for f64) cut by the edges
                                           ((300, 260), (1, 0), "f32"), ((520, 264), (1, 0), "f64"), ((1000, 1000), (1, 0), "i32"),
                                           ((3, 72, 5, 80), (0, 3, 2, 1), "bf16"), ((132, 20, 68), (1, 2, 0), "f32"), ((256, 256), (1, 0), "f32"),
                                           ((5, 128, 192), (0, 2, 1), "f16")])
def test_transpose_through_lds_tiles(rx, client, shape, perm, dt):
    """Pure transposes of every kind that moves the minor dimension, with tiles cut by the edges;
    bit-exact (a transpose moves values, it does not compute)."""
    out_shape = tuple(shape[p] for p in perm)
    text = ("module { func.func @main(%%a: %s) -> %s {\n  %%0 = stablehlo.transpose %%a, dims = [%s] : (%s) -> %s\n  return %%0 : %s } }"
            % (_tt_(shape, dt), _tt_(out_shape, dt), ", ".join(map(str, perm)), _tt_(shape, dt), _tt_(out_shape, dt), _tt_(out_shape, dt)))
    rng = np.random.default_rng(0)
    x = I.tensor(rng.integers(-1000, 1000, size=shape), dt) if dt == "i32" else I.tensor(rng.normal(size=shape), dt)
    got, exe = gpu_run(rx, client, text, [x])
    assert [l["kind"] for l in exe.launches()] == ["map_transposed"]
    want = np.transpose(x.a, perm)
    assert got[0].a.shape == want.shape and np.array_equal(got[0].a, want)
    assert np.array_equal(got[0].a, oracle_run(text, [x])[0].a)


@pytest.mark.parametrize("shape,low,high,perm,dt", [
    ((6, 200, 121), (0, 2, 1), (0, 1, 3), (0, 2, 1), "f32"),          # scalar tiles, padding on both tiled dimensions
    ((4, 128, 30, 26), (0, 0, 1, 1), (0, 0, 1, 1), (0, 2, 3, 1), "bf16"),   # [B, C, H, W] -> padded [B, H, W, C]: vector tiles, rows that start at odd elements
    ((2, 64, 40, 56), (0, 0, 0, 3), (0, 64, 2, 0), (0, 2, 3, 1), "f16"),    # zero channels after the last one, columns before the first
    ((5, 72, 200), (1, 0, 0), (0, 8, 5), (0, 2, 1), "f64"),
    ((250, 300), (0, 7), (32, 0), (1, 0), "i32")])
def test_transpose_of_a_padded_operand_through_lds_tiles(rx, client, shape, low, high, perm, dt):
    """transpose(pad(x)): the tiles are read at positions clamped into x (a vector inside a row of x at any element
    address, one that crosses the row's ends element by element) and the pad's test guards the read of the tile; bit-exact."""
    padded = tuple(s + l + h for s, l, h in zip(shape, low, high))
    out_shape = tuple(padded[p] for p in perm)
    zero = "0" if dt == "i32" else "0.000000e+00"
    lst = lambda v: ", ".join(str(x) for x in v)
    text = ("module { func.func @main(%%a: %s) -> %s {\n  %%z = stablehlo.constant dense<%s> : tensor<%s>\n"
            "  %%p = stablehlo.pad %%a, %%z, low = [%s], high = [%s], interior = [%s] : (%s, tensor<%s>) -> %s\n"
            "  %%0 = stablehlo.transpose %%p, dims = [%s] : (%s) -> %s\n  return %%0 : %s } }"
            % (_tt_(shape, dt), _tt_(out_shape, dt), zero, dt, lst(low), lst(high), lst([0] * len(shape)), _tt_(shape, dt), dt, _tt_(padded, dt),
               lst(perm), _tt_(padded, dt), _tt_(out_shape, dt), _tt_(out_shape, dt)))
    rng = np.random.default_rng(3)
    x = I.tensor(rng.integers(-1000, 1000, size=shape), dt) if dt == "i32" else I.tensor(rng.normal(size=shape), dt)
    got, exe = gpu_run(rx, client, text, [x])
    assert [l["kind"] for l in exe.launches()] == ["map_transposed"]
    want = np.transpose(np.pad(x.a, list(zip(low, high))), perm)
    assert got[0].a.shape == want.shape and np.array_equal(got[0].a, want)
    assert np.array_equal(got[0].a, oracle_run(text, [x])[0].a)


def test_transpose_of_a_slice_through_lds_tiles(rx, client):
    """transpose(x[1:, 3:131, 8:200]): offsets without any guard."""
    shape, start, limit, perm = (4, 140, 210), (1, 3, 8), (4, 131, 200), (0, 2, 1)
    sl = tuple(l - s for s, l in zip(start, limit))
    out_shape = tuple(sl[p] for p in perm)
    lst = lambda v: ", ".join(str(x) for x in v)
    text = ("module { func.func @main(%%a: %s) -> %s {\n  %%s = stablehlo.slice %%a [%s] : (%s) -> %s\n"
            "  %%0 = stablehlo.transpose %%s, dims = [%s] : (%s) -> %s\n  return %%0 : %s } }"
            % (_tt_(shape, "f32"), _tt_(out_shape, "f32"), ", ".join("%d:%d" % (a, b) for a, b in zip(start, limit)), _tt_(shape, "f32"), _tt_(sl, "f32"),
               lst(perm), _tt_(sl, "f32"), _tt_(out_shape, "f32"), _tt_(out_shape, "f32")))
    x = I.tensor(np.random.default_rng(4).normal(size=shape), "f32")
    got, exe = gpu_run(rx, client, text, [x])
    assert [l["kind"] for l in exe.launches()] == ["map_transposed"]
    assert np.array_equal(got[0].a, np.transpose(x.a[1:, 3:131, 8:200], perm))


@pytest.mark.parametrize("block", ["1", "3", "16"])
@pytest.mark.parametrize("shape,perm,dt", [((1100, 1300), (1, 0), "f32"), ((3, 700, 129), (0, 2, 1), "f32"), ((2, 1000, 72), (0, 2, 1), "f64")])
def test_transposing_tiles_in_blocks_of_other_sizes(rx, client, monkeypatch, block, shape, perm, dt):
    """The order in which the tiles are taken (blocks of B x B, ragged at the edges of the tile grid) does not change a value."""
    monkeypatch.setenv("RX_TRANSPOSE_BLOCK", block)
    test_transpose_through_lds_tiles(rx, client, shape, perm, dt)


def test_map_with_transposed_and_plain_operands(rx, client):
    """sin(a') * b + c' in one kernel: two transposed reads share the tiling, one operand is read in place."""
    m, n = 200, 330
    ta, tb = _tt_((n, m), "f32"), _tt_((m, n), "f32")
    text = ("module { func.func @main(%%a: %s, %%b: %s, %%c: %s) -> %s {\n"
            "  %%0 = stablehlo.transpose %%a, dims = [1, 0] : (%s) -> %s\n  %%1 = stablehlo.sine %%0 : %s\n"
            "  %%2 = stablehlo.multiply %%1, %%b : %s\n  %%3 = stablehlo.transpose %%c, dims = [1, 0] : (%s) -> %s\n"
            "  %%4 = stablehlo.add %%2, %%3 : %s\n  return %%4 : %s } }" % (ta, tb, ta, tb, ta, tb, tb, tb, ta, tb, tb, tb))
    rng = np.random.default_rng(1)
    a, b, c = I.tensor(rng.normal(size=(n, m)), "f32"), I.tensor(rng.normal(size=(m, n)), "f32"), I.tensor(rng.normal(size=(n, m)), "f32")
    got, exe = gpu_run(rx, client, text, [a, b, c])
    assert [l["kind"] for l in exe.launches()] == ["map_transposed"]
    ref = oracle_run(text, [a, b, c])
    assert max_rel_to_scale(got[0].a, ref[0].a) <= 1e-6


def test_transposed_reads_with_different_pairings_fall_back_per_operand(rx, client):
    """out[i,j,k] = a[k,j,i] + b[i,k,j]: the minor dimensions of a and b pair with different output
    dimensions; one of them is staged, the other is read with a stride -- same values either way."""
    s = (40, 48, 56)
    ta, tb, to = _tt_((56, 48, 40), "f32"), _tt_((40, 56, 48), "f32"), _tt_(s, "f32")
    text = ("module { func.func @main(%%a: %s, %%b: %s) -> %s {\n"
            "  %%0 = stablehlo.transpose %%a, dims = [2, 1, 0] : (%s) -> %s\n  %%1 = stablehlo.transpose %%b, dims = [0, 2, 1] : (%s) -> %s\n"
            "  %%2 = stablehlo.add %%0, %%1 : %s\n  return %%2 : %s } }" % (ta, tb, to, ta, to, tb, to, to, to))
    rng = np.random.default_rng(2)
    a, b = I.tensor(rng.normal(size=(56, 48, 40)), "f32"), I.tensor(rng.normal(size=(40, 56, 48)), "f32")
    got, exe = gpu_run(rx, client, text, [a, b])
    assert [l["kind"] for l in exe.launches()] == ["map_transposed"]
    assert np.array_equal(got[0].a, np.transpose(a.a, (2, 1, 0)) + np.transpose(b.a, (0, 2, 1)))


def test_chunked_integer_reduction_with_an_init_value(rx, client):
    """A column sum whose reduced dimension is cut into chunks: exact in i32, the init value is
    applied once (by the combining kernel), chunk sizes that do not divide the extent."""
    shape = (1001, 77)
    x = np.random.default_rng(8).integers(-1000, 1000, size=shape).astype(np.int32)
    text = mod([_tt(shape, "i32"), "tensor<i32>"], _tt([77], "i32"),
               "    %%0 = stablehlo.reduce(%%arg0 init: %%arg1) applies stablehlo.add across dimensions = [0] : (%s, tensor<i32>) -> %s\n"
               "    return %%0 : %s\n" % (_tt(shape, "i32"), _tt([77], "i32"), _tt([77], "i32")))
    got, exe = gpu_run(rx, client, text, [I.Tensor(x, "i32"), I.Tensor(np.int32(12345), "i32")])
    assert [l["kind"] for l in exe.launches()] == ["reduce_generic", "reduce_final"]
    assert np.array_equal(got[0].a, x.sum(axis=0, dtype=np.int32) + np.int32(12345))


# ---- row groups on short rows: several rows share a wavefront --------------------------------------
@pytest.mark.parametrize("rows,cols", [(1000, 3), (777, 5), (4099, 10), (300, 17), (129, 33), (515, 48), (64, 64), (9, 2)])
def test_softmax_over_short_rows(rx, client, rows, cols):
    """max / exp-sum / divide fused in one row kernel; rows of 2..64 elements are handled by
    aligned groups of 1..32 lanes.  Against scipy-style softmax in float64 and the row-sum invariant."""
    ty, to = _tt_((rows, cols), "f32"), _tt_((rows,), "f32")
    text = ("module { func.func @main(%%a: %s) -> %s {\n"
            " %%ninf = stablehlo.constant dense<0xFF800000> : tensor<f32>\n %%z = stablehlo.constant dense<0.0> : tensor<f32>\n"
            " %%m = stablehlo.reduce(%%a init: %%ninf) applies stablehlo.maximum across dimensions = [1] : (%s, tensor<f32>) -> %s\n"
            " %%mb = stablehlo.broadcast_in_dim %%m, dims = [0] : (%s) -> %s\n %%d = stablehlo.subtract %%a, %%mb : %s\n %%e = stablehlo.exponential %%d : %s\n"
            " %%s = stablehlo.reduce(%%e init: %%z) applies stablehlo.add across dimensions = [1] : (%s, tensor<f32>) -> %s\n"
            " %%sb = stablehlo.broadcast_in_dim %%s, dims = [0] : (%s) -> %s\n %%r = stablehlo.divide %%e, %%sb : %s\n return %%r : %s } }"
            % (ty, ty, ty, to, to, ty, ty, ty, ty, to, to, ty, ty, ty))
    x = np.random.default_rng(rows + cols).normal(size=(rows, cols)).astype(np.float32) * 3
    got, exe = gpu_run(rx, client, text, [I.Tensor(x, "f32")])
    assert [l["kind"] for l in exe.launches()] == ["row"]
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    assert np.max(np.abs(got[0].a - want)) <= 2e-6
    assert np.allclose(got[0].a.sum(axis=1), 1.0, atol=1e-5)
    ref = oracle_run(text, [I.Tensor(x, "f32")], hifi=True)
    assert np.max(np.abs(got[0].a - ref[0].a)) <= 2e-6


def test_reshapes_that_share_a_buffer(rx, client):
    """A reshape of a value that owns a buffer costs no launch; results stay independent buffers."""
    t = ("module {\n func.func @main(%arg0: tensor<6x4xf32>) -> (tensor<24xf32>, tensor<3x8xf32>, tensor<2x12xf32>, tensor<4x6xf32>, tensor<6x4xf32>) {\n"
         "  %0 = stablehlo.reshape %arg0 : (tensor<6x4xf32>) -> tensor<24xf32>\n"             # reshape of an argument: a copy
         "  %1 = stablehlo.exponential %arg0 : tensor<6x4xf32>\n"
         "  %2 = stablehlo.reshape %1 : (tensor<6x4xf32>) -> tensor<3x8xf32>\n"              # shares the temporary
         "  %3 = stablehlo.reshape %1 : (tensor<6x4xf32>) -> tensor<2x12xf32>\n"             # second result on the same value: its own copy
         "  %4 = stablehlo.negate %arg0 : tensor<6x4xf32>\n"
         "  %5 = stablehlo.reshape %4 : (tensor<6x4xf32>) -> tensor<4x6xf32>\n"              # the value itself is returned too
         "  return %0, %2, %3, %5, %4 : tensor<24xf32>, tensor<3x8xf32>, tensor<2x12xf32>, tensor<4x6xf32>, tensor<6x4xf32>\n }\n}\n")
    x = I.tensor(np.random.default_rng(0).normal(size=(6, 4)), "f32")
    got, exe = gpu_run(rx, client, t, [x])
    ref = oracle_run(t, [x])
    for g, r in zip(got, ref):
        assert g.a.shape == r.a.shape
        assert np.allclose(g.a, r.a, rtol=1e-6)
    assert len(exe.launches()) == 5          # copy, exp, copy of exp, negate, copy of negate; one reshape is free
    # a reshape between two kernels is always free
    t2 = ("module {\n func.func @main(%arg0: tensor<64x32xf32>, %arg1: tensor<16x128xf32>) -> tensor<16x16xf32> {\n"
          "  %0 = stablehlo.exponential %arg0 : tensor<64x32xf32>\n"
          "  %1 = stablehlo.reshape %0 : (tensor<64x32xf32>) -> tensor<16x128xf32>\n"
          "  %2 = stablehlo.dot_general %1, %arg1, contracting_dims = [1] x [1] : (tensor<16x128xf32>, tensor<16x128xf32>) -> tensor<16x16xf32>\n"
          "  return %2 : tensor<16x16xf32>\n }\n}\n")
    a = [I.tensor(np.random.default_rng(1).normal(size=(64, 32)), "f32"), I.tensor(np.random.default_rng(2).normal(size=(16, 128)), "f32")]
    got, exe = gpu_run(rx, client, t2, a)
    assert len(exe.launches()) == 2
    assert max_rel_to_scale(got[0].a, oracle_run(t2, a, hifi=True)[0].a) <= 1e-5


def test_conditionals(rx, client):
    """stablehlo.if / stablehlo.case: every branch is evaluated and the results selected."""
    import _while_modules as W
    x = I.tensor(np.arange(8) / 4, "f32")
    exe = None
    for s in (2.0, -3.0, 0.0):
        args = [x, I.tensor(np.float32(s), "f32")]
        got, exe = gpu_run(rx, client, W.IF, args, exe=exe)
        ref = oracle_run(W.IF, args)
        assert rel_err(got[0].a, ref[0].a) <= 1e-6 and float(got[1].a) == float(ref[1].a)
    y = I.tensor(np.random.default_rng(0).normal(size=(4, 5)), "f64")
    exe = None
    for idx in (0, 1, 2, 7, -1):
        args = [y, I.Tensor(np.int32(idx), "i32")]
        got, exe = gpu_run(rx, client, W.CASE, args, exe=exe)
        assert rel_err(got[0].a, oracle_run(W.CASE, args)[0].a) <= 1e-14
    got, exe = gpu_run(rx, client, W.IF_CONST, [x])
    assert rel_err(got[0].a, np.cos(x.a)) <= 1e-6
    assert "select" not in exe.report() and ":: cosine" in exe.report()


CHLO_UNARY = {   # op -> range of the sweep
    "acos": (-0.99, 0.99), "asin": (-0.99, 0.99), "atan": (-20.0, 20.0), "acosh": (1.01, 50.0), "asinh": (-50.0, 50.0),
    "atanh": (-0.99, 0.99), "cosh": (-8.0, 8.0), "sinh": (-8.0, 8.0), "erfc": (-3.0, 3.0), "lgamma": (2.5, 30.0),
    "digamma": (0.1, 30.0), "erf_inv": (-0.999, 0.999), "erf": (-3.0, 3.0),
}


@pytest.mark.parametrize("op", sorted(CHLO_UNARY))
@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_chlo_unary_maps(rx, client, op, dt):
    """The `chlo` math ops of reference src/Ops.jl:398-436 against scipy / numpy in float64: 1e-6 relative for
    f32 (5e-6 for digamma near its zero), 1e-12 for f64."""
    lo, hi = CHLO_UNARY[op]
    x = np.random.default_rng(5).uniform(lo, hi, 4096).astype(I.NP_OF[dt])
    t = _tt(x.shape, dt)
    text = mod([t], t, "    %%0 = chlo.%s %%arg0 : %s -> %s\n    return %%0 : %s\n" % (op, t, t, t))
    got, _ = gpu_run(rx, client, text, [I.Tensor(x, dt)])
    ref64 = oracle_run(text.replace(dt, "f64"), [I.Tensor(x.astype(np.float64), "f64")])[0].a
    diff = np.abs(got[0].a.astype(np.float64) - ref64)
    rel = (5e-6 if op == "digamma" else 1e-6) if dt == "f32" else 1e-12
    assert ((diff <= rel * np.maximum(np.abs(ref64), 1e-30)) | (diff <= rel)).all(), (op, float((diff / np.maximum(np.abs(ref64), 1e-30)).max()))


def test_digamma_below_zero_and_classification_ops(rx, client):
    x = np.array([-2.5, -0.5, -1.25, -7.75, 0.25], np.float64)
    t = _tt(x.shape, "f64")
    text = mod([t], t, "    %%0 = chlo.digamma %%arg0 : %s -> %s\n    return %%0 : %s\n" % (t, t, t))
    got, ref = both(rx, client, text, [I.Tensor(x, "f64")])
    assert np.allclose(got[0].a, ref[0].a, rtol=1e-11)
    y = np.array([1.0, np.inf, -np.inf, np.nan, 0.0], np.float32)
    t, tb = _tt(y.shape, "f32"), _tt(y.shape, "i1")
    for op, want in (("is_inf", [0, 1, 1, 0, 0]), ("is_pos_inf", [0, 1, 0, 0, 0]), ("is_neg_inf", [0, 0, 1, 0, 0])):
        text = mod([t], tb, "    %%0 = chlo.%s %%arg0 : %s -> %s\n    return %%0 : %s\n" % (op, t, tb, tb))
        got, ref = both(rx, client, text, [I.Tensor(y, "f32")])
        assert got[0].a.astype(int).tolist() == want == ref[0].a.astype(int).tolist()


@pytest.mark.parametrize("dt", ["i8", "ui16", "i32", "ui32", "i64"])
def test_popcnt_and_count_leading_zeros(rx, client, dt):
    """stablehlo.popcnt / count_leading_zeros at the element's own width, bit for bit."""
    npdt = I.NP_OF[dt]
    bits = 8 * np.dtype(npdt).itemsize
    rng = np.random.default_rng(9)
    raw = rng.integers(0, 1 << 62, 3000, dtype=np.uint64) >> rng.integers(0, 62, 3000).astype(np.uint64)
    x = np.concatenate([np.array([0, 1, (1 << bits) - 1, 1 << (bits - 1)], dtype=np.uint64), raw & np.uint64((1 << bits) - 1)]).astype(
        {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[bits // 8]).view(npdt)
    t = _tt(x.shape, dt)
    for op in ("popcnt", "count_leading_zeros"):
        text = mod([t], t, "    %%0 = stablehlo.%s %%arg0 : %s\n    return %%0 : %s\n" % (op, t, t))
        got, ref = both(rx, client, text, [I.Tensor(x, dt)])
        assert np.array_equal(got[0].a, ref[0].a), op
    # known answers at this width
    text = mod([t], t, "    %%0 = stablehlo.count_leading_zeros %%arg0 : %s\n    return %%0 : %s\n" % (t, t))
    assert oracle_run(text, [I.Tensor(x, dt)])[0].a[:4].tolist() == [bits, bits - 1, 0, 0]


def test_bitcast_convert_and_get_dimension_size(rx, client):
    """bitcast_convert between types of one width (known bit patterns: 1.0f = 0x3F800000, -2.0 = 0xC000...), and
    get_dimension_size, which folds to a constant."""
    x = np.array([1.0, -2.0, 0.0, np.inf, 1e-45], np.float32)
    t, ti = _tt(x.shape, "f32"), _tt(x.shape, "ui32")
    text = mod([t], ti, "    %%0 = stablehlo.bitcast_convert %%arg0 : (%s) -> %s\n    return %%0 : %s\n" % (t, ti, ti))
    got, ref = both(rx, client, text, [I.Tensor(x, "f32")])
    assert got[0].a.tolist() == [0x3F800000, 0xC0000000, 0, 0x7F800000, 1] == ref[0].a.tolist()
    y = np.random.default_rng(2).integers(-2 ** 62, 2 ** 62, 1000)
    t, tf = _tt(y.shape, "i64"), _tt(y.shape, "f64")
    text = mod([t], tf, "    %%0 = stablehlo.bitcast_convert %%arg0 : (%s) -> %s\n    return %%0 : %s\n" % (t, tf, tf))
    got, ref = both(rx, client, text, [I.Tensor(y, "i64")])
    assert np.array_equal(got[0].a.view(np.int64), y) and np.array_equal(ref[0].a.view(np.int64), y)
    t = _tt([7, 5, 3], "f32")
    text = mod([t], "tensor<i32>", "    %%0 = stablehlo.get_dimension_size %%arg0, dim = 1 : (%s) -> tensor<i32>\n    return %%0 : tensor<i32>\n" % t)
    got, ref = both(rx, client, text, [I.Tensor(np.zeros((7, 5, 3), np.float32), "f32")])
    assert int(got[0].a) == 5 == int(ref[0].a)


# ---- integer division at the edges, float -> integer conversion beyond the range -------------
@pytest.mark.parametrize("dt", ["ui8", "ui16", "ui32", "ui64", "i8", "i16", "i32", "i64"])
@pytest.mark.parametrize("op", ["divide", "remainder"])
def test_integer_division_edge_cases(rx, client, op, dt):
    """Divisors 0, 1 and the all-ones pattern (the largest value of an unsigned type, -1 of a signed
    one), dividends including the type's limits; bit-exact against the oracle, whose rules are pinned
    against Python integers in tests/test_oracle_golden.py."""
    info = np.iinfo(I.NP_OF[dt])
    av = [0, 1, 2, 5, 100, info.max, info.max - 1, info.min, info.min + 1 if info.min else 7]
    bv = [0, 1, 2, 3, info.max, info.max - 1, -1 if info.min else info.max, info.min if info.min else 4]
    a = np.array([x for x in av for _ in bv], dtype=I.NP_OF[dt])
    b = np.array([y for _ in av for y in bv], dtype=I.NP_OF[dt])
    t = _tt([a.size], dt)
    text = mod([t, t], t, "    %%0 = stablehlo.%s %%arg0, %%arg1 : %s\n    return %%0 : %s\n" % (op, t, t))
    got, ref = both(rx, client, text, [I.Tensor(a, dt), I.Tensor(b, dt)])
    assert np.array_equal(got[0].a, ref[0].a), (got[0].a.tolist(), ref[0].a.tolist())


@pytest.mark.parametrize("dst", ["i8", "ui8", "i16", "ui16", "i32", "ui32", "i64", "ui64"])
@pytest.mark.parametrize("src", ["f32", "f64", "bf16"])
def test_convert_float_to_integer_saturates(rx, client, src, dst):
    """Truncation toward zero inside the range, the nearest limit beyond it, 0 for NaN."""
    vals = [0.0, 0.9, -0.9, 3.9, -3.9, 127.0, 128.0, -128.0, -129.0, 255.0, 256.0, 300.0, -200.0, 32767.0, 32768.0, -32769.0, 65535.0,
            65536.0, 2147483520.0, 2147483648.0, -2147483648.0, -2147483904.0, 4294967040.0, 4294967296.0, 9.2233715e18, 9.3e18,
            -9.3e18, 1.8446743e19, 1.9e19, 1e30, -1e30, float("inf"), float("-inf"), float("nan")]
    x = I.tensor(np.array(vals, dtype=np.float64), src)
    ts, td = _tt([len(vals)], src), _tt([len(vals)], dst)
    text = mod([ts], td, "    %%0 = stablehlo.convert %%arg0 : (%s) -> %s\n    return %%0 : %s\n" % (ts, td, td))
    got, ref = both(rx, client, text, [x])
    assert np.array_equal(got[0].a, ref[0].a), (got[0].a.tolist(), ref[0].a.tolist())


# ---- an update in place must wait for every reader of the buffer it takes over ---------------
@pytest.mark.parametrize("name", ["dot_epilogue_after_update", "row_reduce_after_update", "update_after_all_readers"])
def test_update_slice_and_late_readers(rx, client, name):
    import _inplace_modules as M
    text, nargs, shapes = M.CASES[name]
    rng = np.random.default_rng(11)
    args = [I.Tensor(rng.uniform(0.5, 1.5, s).astype(np.float32), "f32") for s in shapes]
    got, ref = both(rx, client, text, args)
    assert np.array_equal(got[0].a[:16], args[nargs - 2].a)           # the updated rows: copies
    assert rel_err(got[0].a, ref[0].a) <= 1e-5, name                  # the rest: a sum or a product of positive numbers
    assert max_rel_to_scale(got[1].a, ref[1].a) <= 1e-5, name        # positive operands: no cancellation
    assert rel_err(got[1].a, ref[1].a) <= 1e-4, name
