"""Writes tests/golden/reference_kats.json: known-answer vectors transcribed by hand from the
reference's own tests (inputs and expected outputs only; the reference was read, not run --
Julia is not available).  Each case names the reference file:line it comes from.  Julia arrays
are given in wire layout (row-major, dims reversed) and Julia's 1-based dims are mapped to wire
dims (d -> N - d).

    python tests/golden/make_reference_kats.py
"""
import json
import os

import numpy as np


def T(shape, dt):
    return "tensor<" + "x".join([str(s) for s in shape] + [dt]) + ">"


def case(name, src, module, args, expect, **kw):
    e = {"shape": list(np.shape(expect)), "data": np.asarray(expect, dtype=np.float64).reshape(-1).tolist()}
    e.update(kw)
    return {"name": name, "source": src, "module": module,
            "args": [{"dtype": dt, "shape": list(np.shape(a)), "data": np.asarray(a).reshape(-1).tolist()} for a, dt in args],
            "expect": e}


def unary(op, n, dt):
    t = T([n], dt)
    return "module { func.func @main(%%a: %s) -> %s { %%0 = stablehlo.%s %%a : %s\n return %%0 : %s } }" % (t, t, op, t, t)


def pad1(n_out, low, high, interior):
    return ("module { func.func @main(%%x: tensor<4xi64>, %%v: tensor<i64>) -> %s { %%0 = stablehlo.pad %%x, %%v, low = [%d], high = [%d], "
            "interior = [%d] : (tensor<4xi64>, tensor<i64>) -> %s\n return %%0 : %s } }" % (T([n_out], "i64"), low, high, interior, T([n_out], "i64"), T([n_out], "i64")))


def fixture(dims, integer):
    n = int(np.prod(dims))
    flat = np.arange(1, n + 1)
    a = flat.astype(np.int64) if integer else flat / n
    return a.reshape(dims, order="F")


cases = []
pi = np.pi
cases.append(case("sine at multiples of pi/2", "test/core/ops.jl:788-793", unary("sine", 5, "f64"),
                  [([0.0, pi / 2, pi, 3 * pi / 2, 2 * pi], "f64")], [0, 1, 0, -1, 0], atol=1e-15, rtol=0))
cases.append(case("sqrt of squares", "test/core/ops.jl:821-824", unary("sqrt", 4, "f64"), [([1.0, 4.0, 9.0, 16.0], "f64")], [1, 2, 3, 4], exact=True))
cases.append(case("pad low", "test/core/ops.jl:538-539", pad1(5, 1, 0, 0), [([1, 2, 3, 4], "i64"), (0, "i64")], [0, 1, 2, 3, 4], exact=True))
cases.append(case("pad high", "test/core/ops.jl:541-542", pad1(5, 0, 1, 0), [([1, 2, 3, 4], "i64"), (0, "i64")], [1, 2, 3, 4, 0], exact=True))
cases.append(case("pad interior", "test/core/ops.jl:544-545", pad1(7, 0, 0, 1), [([1, 2, 3, 4], "i64"), (0, "i64")], [1, 0, 2, 0, 3, 0, 4], exact=True))
# 2-D pads: Julia x = [1 2; 3 4]; wire buffer is x', Julia dims (a, b) become wire dims (b, a)
xw = np.array([[1, 2], [3, 4]]).T
for nm, src, low, high, inter, exp in (
        ("pad 2d low", "test/core/ops.jl:549-550", [1, 2], [0, 0], [0, 0], [[0, 0, 0, 0], [0, 0, 1, 2], [0, 0, 3, 4]]),
        ("pad 2d high", "test/core/ops.jl:552-553", [0, 0], [1, 2], [0, 0], [[1, 2, 0, 0], [3, 4, 0, 0], [0, 0, 0, 0]]),
        ("pad 2d interior", "test/core/ops.jl:555-556", [0, 0], [0, 0], [1, 2], [[1, 0, 0, 2], [0, 0, 0, 0], [3, 0, 0, 4]])):
    ew = np.array(exp).T
    to = T(ew.shape, "i64")
    m = ("module { func.func @main(%%x: tensor<2x2xi64>, %%v: tensor<i64>) -> %s { %%0 = stablehlo.pad %%x, %%v, low = %s, high = %s, interior = %s : "
         "(tensor<2x2xi64>, tensor<i64>) -> %s\n return %%0 : %s } }" % (to, low[::-1], high[::-1], inter[::-1], to, to))
    cases.append(case(nm, src, m, [(xw, "i64"), (0, "i64")], ew, exact=True))
cases.append(case("slice [2:3]", "test/core/ops.jl:815-817",
                  "module { func.func @main(%x: tensor<4xi64>) -> tensor<2xi64> { %0 = stablehlo.slice %x [1:3] : (tensor<4xi64>) -> tensor<2xi64>\n return %0 : tensor<2xi64> } }",
                  [([1, 2, 3, 4], "i64")], [2, 3], exact=True))
cases.append(case("slice [1:1]", "test/core/ops.jl:818",
                  "module { func.func @main(%x: tensor<4xi64>) -> tensor<1xi64> { %0 = stablehlo.slice %x [0:1] : (tensor<4xi64>) -> tensor<1xi64>\n return %0 : tensor<1xi64> } }",
                  [([1, 2, 3, 4], "i64")], [1], exact=True))
dotv = ("module { func.func @main(%%a: %s, %%b: %s) -> %s { %%0 = stablehlo.dot_general %%a, %%b, contracting_dims = [0] x [0] : (%s, %s) -> %s\n return %%0 : %s } }")
for dt in ("i32", "f64"):
    t4, t0 = T([4], dt), T([], dt)
    cases.append(case("dot of vectors " + dt, "test/core/ops.jl:260-270", dotv % (t4, t4, t0, t4, t4, t0, t0),
                      [([1, 2, 3, 4], dt), ([5, 6, -7, -8], dt)], -36, exact=True))
t4, t44 = T([4], "i32"), T([4, 4], "i32")
cases.append(case("outer product", "test/core/ops.jl:253,268-269",
                  "module { func.func @main(%%a: %s, %%b: %s) -> %s { %%0 = stablehlo.dot_general %%a, %%b, contracting_dims = [] x [] : (%s, %s) -> %s\n return %%0 : %s } }"
                  % (t4, t4, t44, t4, t4, t44, t44), [([1, 2, 3, 4], "i32"), ([5, 6, -7, -8], "i32")],
                  np.outer([1, 2, 3, 4], [5, 6, -7, -8]), exact=True))
cases.append(case("batched elementwise product", "test/core/ops.jl:256-258,270",
                  "module { func.func @main(%%a: %s, %%b: %s) -> %s { %%0 = stablehlo.dot_general %%a, %%b, batching_dims = [0] x [0], contracting_dims = [] x [] : (%s, %s) -> %s\n return %%0 : %s } }"
                  % (t4, t4, t4, t4, t4, t4, t4), [([1, 2, 3, 4], "i32"), ([5, 6, -7, -8], "i32")], [5, 12, -21, -32], exact=True))
# Int32[1 2; 3 4]' * Int32[5 6; -7 -8]: contraction over Julia dim 1 == wire dim 1 of both buffers
A, B = np.array([[1, 2], [3, 4]]), np.array([[5, 6], [-7, -8]])
t22 = T([2, 2], "i32")
cases.append(case("transposed matrix product", "test/core/ops.jl:273-276",
                  "module { func.func @main(%%a: %s, %%b: %s) -> %s { %%0 = stablehlo.dot_general %%a, %%b, contracting_dims = [1] x [1] : (%s, %s) -> %s\n return %%0 : %s } }"
                  % (t22, t22, t22, t22, t22, t22, t22), [(A.T, "i32"), (B.T, "i32")], [[-16, -18], [-18, -20]], exact=True))
# Int64 3x4x5 reduce (test/core/ops.jl:1207-1235): Julia dims -> wire dims 3 - d
Aj = fixture((3, 4, 5), True)
Aw = np.ascontiguousarray(Aj.T)
for nm, jdims, body, init, f in (("prod over dims [2]", [2], "multiply", 1, np.multiply), ("sum over dims [1,3]", [1, 3], "add", 0, np.add),
                                 ("sum over all dims", [1, 2, 3], "add", 0, np.add)):
    wd = sorted(3 - d for d in jdims)
    e = Aj
    for d in sorted(jdims, reverse=True):
        e = f.reduce(e, axis=d - 1)
    ew = np.asarray(e).T
    to = T(ew.shape, "i64")
    m = ("module { func.func @main(%%x: %s, %%i: tensor<i64>) -> %s { %%0 = stablehlo.reduce(%%x init: %%i) applies stablehlo.%s across dimensions = %s : "
         "(%s, tensor<i64>) -> %s\n return %%0 : %s } }" % (T(Aw.shape, "i64"), to, body, wd, T(Aw.shape, "i64"), to, to))
    cases.append(case(nm, "test/core/ops.jl:1214-1234", m, [(Aw, "i64"), (init, "i64")], ew, exact=True))
F = fixture((2, 10), False)
cases.append(case("sum of fixture 2x10 is 10.5", "test/core/map_reduction.jl:8-19, src/TestUtils.jl:9-13",
                  "module { func.func @main(%x: tensor<10x2xf64>) -> tensor<f64> { %c = stablehlo.constant dense<0.0> : tensor<f64>\n %0 = stablehlo.reduce(%x init: %c) applies stablehlo.add across dimensions = [0, 1] : (tensor<10x2xf64>, tensor<f64>) -> tensor<f64>\n return %0 : tensor<f64> } }",
                  [(np.ascontiguousarray(F.T), "f64")], 10.5, rtol=1e-14, atol=0))
cases.append(case("hlo_call add", "test/core/ops.jl:1046-1064",
                  "module {\n  func.func @main(%arg0: tensor<3xf32>, %arg1: tensor<3xf32>) -> tensor<3xf32> {\n    %0 = stablehlo.add %arg0, %arg1 : tensor<3xf32>\n    return %0 : tensor<3xf32>\n  }\n}",
                  [([1.0, 2.0, 50.0], "f32"), ([-4.0, 0.001, 2.0], "f32")], np.float32([1.0, 2.0, 50.0]) + np.float32([-4.0, 0.001, 2.0]), exact=True))
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_kats.json")
with open(out, "w") as f:
    json.dump({"cases": cases}, f, indent=1)
print("wrote", out, len(cases), "cases")
