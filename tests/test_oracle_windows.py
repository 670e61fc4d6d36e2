"""Pins for the oracle's windowed ops (reverse, reduce_window, convolution): the reference's own
known answers, library routines and brute-force loops.  CPU only."""
import itertools

import numpy as np
import pytest
from scipy import signal

from oracle import stablehlo_interp as I
import _nn_modules as NN


def run(text, arrays, dt="f32", hifi=False):
    return I.run_text(text, [I.tensor(a, dt) if dt[0] in "fb" else I.Tensor(np.asarray(a), dt) for a in arrays], hifi=hifi)[0].a


def test_reverse_reference_vectors():
    """test/core/ops.jl:609-618; Julia matrices arrive with their dims reversed."""
    t = ("module {\n func.func @main(%arg0: tensor<4xi64>) -> tensor<4xi64> {\n"
         "  %0 = stablehlo.reverse %arg0, dims = [0] : tensor<4xi64>\n  return %0 : tensor<4xi64>\n }\n}\n")
    assert run(t, [np.array([1, 2, 3, 4])], "i64").tolist() == [4, 3, 2, 1]
    x = np.array([[1, 2], [3, 4]])                       # Julia [1 2; 3 4]
    for jdim, want in ((1, [[3, 4], [1, 2]]), (2, [[2, 1], [4, 3]])):
        raw_dim = 2 - jdim
        t = ("module {\n func.func @main(%%arg0: tensor<2x2xi64>) -> tensor<2x2xi64> {\n"
             "  %%0 = stablehlo.reverse %%arg0, dims = [%d] : tensor<2x2xi64>\n  return %%0 : tensor<2x2xi64>\n }\n}\n" % raw_dim)
        got = run(t, [x.T.copy()], "i64").T
        assert got.tolist() == want


def test_conv_1d_flip_reference_vectors():
    """test/nn/convolution.jl:206-217: x = W = [1, 2, 3], pad 1, flipped and not."""
    x = np.array([[[1.0, 2.0, 3.0]]])
    for flip, want in ((False, [0 * 1 + 1 * 2 + 2 * 3, 1 * 1 + 2 * 2 + 3 * 3, 1 * 2 + 2 * 3 + 3 * 0]),
                       (True, [3 * 0 + 2 * 1 + 1 * 2, 3 * 1 + 2 * 2 + 1 * 3, 3 * 2 + 2 * 3 + 1 * 0])):
        text, out = NN.convolution([1, 1, 3], [1, 1, 3], "f32", dims="[b, f, 0]x[o, i, 0]->[b, f, 0]", padding=[[1, 1]], flip=flip)
        assert out == [1, 1, 3]
        assert run(text, [x, x]).reshape(-1).tolist() == want
        text, _ = NN.convolution([1, 1, 3], [1, 1, 3], "f32", dims="[b, f, 0]x[o, i, 0]->[b, f, 0]", padding=[[1, 1]], flip=flip, generic=True)
        assert run(text, [x, x]).reshape(-1).tolist() == want


def test_cumulative_reference_cases():
    """test/core/map_reduction.jl:165-229: cumsum / cumprod of 1:10 ./ 10 and of a 3x4x5 array along
    each Julia dim (raw dim = 3 - Julia dim) against numpy's accumulate."""
    a = (np.arange(1, 11) / 10).astype(np.float32)
    assert np.allclose(run(NN.cumulative([10], "f32", 0), [a]), np.cumsum(a), rtol=1e-6)
    assert np.allclose(run(NN.cumulative([10], "f32", 0, "multiply"), [a]), np.cumprod(a), rtol=1e-6)
    b = (np.arange(1, 61).reshape(5, 4, 3) / 60).astype(np.float32)      # raw view of reshape(1:60, (3, 4, 5)) ./ 60
    for raw in range(3):
        assert np.allclose(run(NN.cumulative([5, 4, 3], "f32", raw), [b]), np.cumsum(b, axis=raw), rtol=1e-6)
        assert np.allclose(run(NN.cumulative([5, 4, 3], "f32", raw, "multiply"), [b]), np.cumprod(b, axis=raw), rtol=1e-6)


def test_prefix_fast_path_equals_the_general_window_form():
    rng = np.random.default_rng(0)
    for shape, dim, body, rev in (([37], 0, "add", False), ([6, 11], 0, "maximum", True), ([6, 11], 1, "multiply", False),
                                  ([3, 5, 4], 1, "minimum", True), ([9, 2], 0, "add", True)):
        x = rng.uniform(0.5, 1.5, size=shape)
        text = NN.cumulative(shape, "f64", dim, body, rev)
        fast = I.Interpreter(I.parse_module(text)).run([I.tensor(x, "f64")])[0].a
        # force the general path: pad with the init value, gather every window, reduce
        funcs = I.parse_module(text)
        for fn in funcs.values():
            for op in fn.ops:
                if op.name == "reduce_window":
                    op.attrs["__general__"] = True
        slow = I.Interpreter(funcs).run([I.tensor(x, "f64")])[0].a
        assert np.allclose(fast, slow, rtol=1e-13, atol=0), (shape, dim, body, rev)
    ints = rng.integers(-50, 50, size=(7, 13)).astype(np.int32)
    assert np.array_equal(run(NN.cumulative([7, 13], "i32", 1), [ints], "i32"), np.cumsum(ints, axis=1, dtype=np.int32))


def brute_pool(x, body, window, strides, padding, base_dil, win_dil):
    r = x.ndim
    ident = {"add": 0.0, "maximum": -np.inf, "minimum": np.inf, "multiply": 1.0}[body]
    f = {"add": lambda p, q: p + q, "maximum": max, "minimum": min, "multiply": lambda p, q: p * q}[body]
    dil = [n + max(n - 1, 0) * (base_dil[d] - 1) for d, n in enumerate(x.shape)]
    big = np.full([dil[d] + padding[d][0] + padding[d][1] for d in range(r)], ident)
    for idx in itertools.product(*[range(n) for n in x.shape]):
        big[tuple(padding[d][0] + idx[d] * base_dil[d] for d in range(r))] = x[idx]
    out_shape = NN.window_out_shape(list(x.shape), window, strides, padding, base_dil, win_dil)
    out = np.zeros(out_shape)
    for o in itertools.product(*[range(n) for n in out_shape]):
        acc = ident
        for k in itertools.product(*[range(w) for w in window]):
            acc = f(acc, big[tuple(o[d] * strides[d] + k[d] * win_dil[d] for d in range(r))])
        out[o] = acc
    return out


@pytest.mark.parametrize("body", ["add", "maximum", "minimum"])
def test_reduce_window_against_brute_force(body):
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 3, 7, 9))
    for window, strides, padding, bd, wd in (
            ([1, 1, 2, 2], [1, 1, 2, 2], [[0, 0]] * 4, [1] * 4, [1] * 4),
            ([1, 1, 3, 3], [1, 1, 2, 1], [[0, 0], [0, 0], [1, 1], [2, 0]], [1] * 4, [1] * 4),
            ([1, 2, 3, 2], [1, 1, 1, 2], [[0, 0], [1, 0], [2, 1], [0, 3]], [1, 1, 2, 1], [1, 1, 2, 3])):
        text, out_shape = NN.reduce_window(list(x.shape), "f64", body, window, strides, padding, bd, wd)
        got = run(text, [x], "f64")
        want = brute_pool(x, body, window, strides, padding, bd, wd)
        assert list(got.shape) == out_shape
        assert np.array_equal(np.isinf(got), np.isinf(want))
        fin = np.isfinite(want)
        assert np.allclose(got[fin], want[fin], rtol=1e-13)


def brute_conv(x, w, strides, padding, lhs_dil, rhs_dil, groups):
    """x [b, c, s...], w [o, i, k...] -> [b, o, s...]: plain loops."""
    nsp = x.ndim - 2
    B, C = x.shape[:2]
    O, Ich = w.shape[:2]
    dil = [n + max(n - 1, 0) * (lhs_dil[d] - 1) for d, n in enumerate(x.shape[2:])]
    big = np.zeros([B, C] + [dil[d] + padding[d][0] + padding[d][1] for d in range(nsp)])
    for idx in itertools.product(*[range(n) for n in x.shape[2:]]):
        big[(slice(None), slice(None)) + tuple(padding[d][0] + idx[d] * lhs_dil[d] for d in range(nsp))] = x[(slice(None), slice(None)) + idx]
    osp = NN.conv_out_shape(list(x.shape[2:]), list(w.shape[2:]), strides, padding, lhs_dil, rhs_dil)
    out = np.zeros([B, O] + osp)
    og = O // groups
    for b in range(B):
        for o in range(O):
            g = o // og
            for pos in itertools.product(*[range(n) for n in osp]):
                acc = 0.0
                for i in range(Ich):
                    for k in itertools.product(*[range(n) for n in w.shape[2:]]):
                        acc += big[(b, g * Ich + i) + tuple(pos[d] * strides[d] + k[d] * rhs_dil[d] for d in range(nsp))] * w[(o, i) + k]
                out[(b, o) + pos] = acc
    return out


def test_convolution_against_brute_force_and_scipy():
    rng = np.random.default_rng(4)
    # the grid of test/nn/convolution.jl:165-181 on a smaller image: groups, strides, padding, dilation
    for groups in (1, 2, 4):
        x = rng.normal(size=(2, 8, 9, 10))
        w = rng.normal(size=(4, 8 // groups, 3, 2))
        for strides, padding, rd in (([1, 1], [[0, 0], [0, 0]], [1, 1]), ([2, 2], [[2, 2], [0, 0]], [1, 2]),
                                     ([3, 3], [[0, 0], [2, 2]], [1, 1]), ([1, 2], [[2, 1], [0, 3]], [2, 1])):
            text, out_shape = NN.convolution(list(x.shape), list(w.shape), "f64", strides=strides, padding=padding,
                                             rhs_dil=rd, groups=groups, dims="[b, f, 0, 1]x[o, i, 0, 1]->[b, f, 0, 1]")
            got = run(text, [x, w], "f64")
            want = brute_conv(x, w, strides, padding, [1, 1], rd, groups)
            assert list(got.shape) == out_shape
            assert np.allclose(got, want, rtol=1e-12, atol=1e-12), (groups, strides, padding, rd)
    # input dilation (what the gradient with respect to the input uses), one spatial dim
    x = rng.normal(size=(2, 3, 11))
    w = rng.normal(size=(5, 3, 4))
    text, _ = NN.convolution([2, 3, 11], [5, 3, 4], "f64", dims="[b, f, 0]x[o, i, 0]->[b, f, 0]", lhs_dil=[3], padding=[[3, 2]])
    assert np.allclose(run(text, [x, w], "f64"), brute_conv(x, w, [1], [[3, 2]], [3], [1], 1), rtol=1e-12, atol=1e-12)
    # one channel, no padding: scipy's cross-correlation; flipped kernel: scipy's convolution
    img = rng.normal(size=(12, 13))
    ker = rng.normal(size=(3, 4))
    for flip, lib in ((False, signal.correlate2d), (True, signal.convolve2d)):
        text, _ = NN.convolution([1, 1, 12, 13], [1, 1, 3, 4], "f64", dims="[b, f, 0, 1]x[o, i, 0, 1]->[b, f, 0, 1]", flip=flip)
        assert np.allclose(run(text, [img[None, None], ker[None, None]], "f64")[0, 0], lib(img, ker, mode="valid"), rtol=1e-12, atol=1e-12)


def test_convolution_layouts_agree():
    """The same convolution written with the reference's Julia-order dimension numbers
    ([0, 1, f, b]-style, src/Ops.jl:1029-1043 on unreversed dims) and in the reversed raw order."""
    rng = np.random.default_rng(5)
    x = rng.normal(size=(2, 3, 7, 6))          # [b, f, h, w]
    w = rng.normal(size=(4, 3, 3, 2))          # [o, i, kh, kw]
    t1, _ = NN.convolution([2, 3, 7, 6], [4, 3, 3, 2], "f64", dims="[b, f, 1, 0]x[o, i, 1, 0]->[b, f, 1, 0]", strides=[1, 2], padding=[[0, 1], [1, 0]])
    a = run(t1, [x, w], "f64")
    # the same data seen as [w, h, f, b]; spatial dim 0 is still the image's w
    xt, wt = np.ascontiguousarray(x.transpose(3, 2, 1, 0)), np.ascontiguousarray(w.transpose(3, 2, 1, 0))
    t2, _ = NN.convolution(list(xt.shape), list(wt.shape), "f64", dims="[0, 1, f, b]x[0, 1, i, o]->[0, 1, f, b]", strides=[1, 2], padding=[[0, 1], [1, 0]])
    b = run(t2, [xt, wt], "f64")
    assert np.allclose(a, b.transpose(3, 2, 1, 0), rtol=1e-13, atol=1e-13)


def test_batch_norm_closed_forms():
    """Normalizing with a batch's own statistics gives zero mean and unit (biased) variance per
    feature; inference with mean 0, variance 1 - eps, scale s, offset b is s * x + b."""
    rng = np.random.default_rng(8)
    x = rng.normal(2.0, 3.0, size=(6, 5, 7))
    ones, zeros = np.ones(5), np.zeros(5)
    out, mean, var = [t.a for t in I.run_text(NN.batch_norm([6, 5, 7], "f64", 1, 1e-5, training=True),
                                              [I.tensor(a, "f64") for a in (x, ones, zeros)])]
    assert np.allclose(mean, x.mean(axis=(0, 2)), rtol=1e-13)
    assert np.allclose(var, x.var(axis=(0, 2)), rtol=1e-12)
    assert np.allclose(out.mean(axis=(0, 2)), 0, atol=1e-12)
    assert np.allclose(out.var(axis=(0, 2)), var / (var + 1e-5), rtol=1e-10)
    s, b = rng.normal(size=5), rng.normal(size=5)
    got = I.run_text(NN.batch_norm([6, 5, 7], "f64", 1, 0.25), [I.tensor(a, "f64") for a in (x, s, b, zeros, ones * 0.75)])[0].a
    assert np.allclose(got, x * s[None, :, None] + b[None, :, None], rtol=1e-13, atol=1e-13)


def test_argmax_reduce_against_numpy():
    """findmax / argmax arrive as a reduce over (value, index) pairs (src/Ops.jl:1571-1596); the
    folded region must agree with numpy's max / argmax (first index on ties) along every dim."""
    rng = np.random.default_rng(9)
    x = rng.integers(0, 5, size=(4, 6, 5)).astype(np.float64)        # many ties
    for dim in range(3):
        for generic in (False, True):
            v, i = [t.a for t in I.run_text(NN.argreduce([4, 6, 5], "f64", dim, "GE", generic=generic), [I.tensor(x, "f64")])]
            assert np.array_equal(v, x.max(axis=dim)) and np.array_equal(i, x.argmax(axis=dim))
        v, i = [t.a for t in I.run_text(NN.argreduce([4, 6, 5], "f64", dim, "LE"), [I.tensor(x, "f64")])]
        assert np.array_equal(v, x.min(axis=dim)) and np.array_equal(i, x.argmin(axis=dim))
        # the strict comparison keeps the later of two equal values
        v, i = [t.a for t in I.run_text(NN.argreduce([4, 6, 5], "f64", dim, "GT"), [I.tensor(x, "f64")])]
        last = x.shape[dim] - 1 - np.flip(x, axis=dim).argmax(axis=dim)
        assert np.array_equal(v, x.max(axis=dim)) and np.array_equal(i, last)


def test_gather_reference_vectors():
    """test/nn/scatter_gather.jl:5-99 (NNlib.gather known answers) with the dimension numbers of
    ext/ReactantNNlibExt/Implementations.jl:426-438, written on the tensors as the traced program
    sees them (Julia dim order, one-based indices)."""
    src = np.array([3, 4, 5, 6, 7], dtype=np.float32)
    index = np.array([[1, 2, 3, 4], [4, 2, 1, 3], [3, 5, 5, 3]])
    output = np.array([[3, 4, 5, 6], [6, 4, 3, 5], [5, 7, 7, 5]], dtype=np.float32)
    t = NN.gather([5], [1, 3, 4], [3, 4], "f32", [], [0], [0], 0, [1], one_based=True)
    got = I.run_text(t, [I.tensor(src, "f32"), I.Tensor(index.reshape(1, 3, 4), "i64")])[0].a
    assert np.array_equal(got, output)
    # 2-d source, columns gathered: output[:, i, j] = src[:, index[i, j]]
    src2 = np.array([[3, 5, 7], [4, 6, 8]], dtype=np.float32)
    index2 = np.array([[1, 2, 3], [2, 2, 1], [3, 1, 3]])
    want = np.zeros((2, 3, 3), dtype=np.float32)
    want[:, :, 0] = [[3, 5, 7], [4, 6, 8]]
    want[:, :, 1] = [[5, 5, 3], [6, 6, 4]]
    want[:, :, 2] = [[7, 3, 7], [8, 4, 8]]
    t = NN.gather([2, 3], [1, 3, 3], [2, 3, 3], "f32", [0], [1], [1], 0, [2, 1], one_based=True)
    got = I.run_text(t, [I.tensor(src2, "f32"), I.Tensor(index2.reshape(1, 3, 3), "i64")])[0].a
    assert np.array_equal(got, want)


def test_gather_against_numpy_indexing():
    rng = np.random.default_rng(12)
    x = rng.normal(size=(7, 5, 6))
    # x[idx] on a flattened view: the reference's gather_getindex (src/Ops.jl:2269-2298)
    idx = rng.integers(0, 7, size=(11, 3))
    idx[:, 1] = rng.integers(0, 5, size=11)
    idx[:, 2] = rng.integers(0, 6, size=11)
    t = NN.gather([7, 5, 6], [11, 3], [11, 1], "f64", [1], [0, 1], [0, 1, 2], 1, [1, 1, 1])
    got = I.run_text(t, [I.tensor(x, "f64"), I.Tensor(idx, "i64")])[0].a
    assert np.array_equal(got[:, 0], x[idx[:, 0], idx[:, 1], idx[:, 2]])
    # rows of a table (an embedding lookup), out-of-range rows clamped
    table = rng.normal(size=(10, 4))
    ids = np.array([[0, 9, 3], [12, -2, 5]])
    t = NN.gather([10, 4], [2, 3], [2, 3, 4], "f64", [2], [0], [0], 2, [1, 4])
    got = I.run_text(t, [I.tensor(table, "f64"), I.Tensor(ids, "i64")])[0].a
    assert np.array_equal(got, table[np.clip(ids, 0, 9)])
    # windows: slices of 3 starting at given offsets, with a batching dimension
    y = rng.normal(size=(4, 20))
    starts = rng.integers(-2, 22, size=(4, 5))
    t = NN.gather([4, 20], [4, 5], [4, 5, 3], "f64", [2], [], [1], 2, [1, 3], operand_batching_dims=[0], start_indices_batching_dims=[0])
    got = I.run_text(t, [I.tensor(y, "f64"), I.Tensor(starts, "i64")])[0].a
    want = np.stack([[y[b, np.clip(s, 0, 17):np.clip(s, 0, 17) + 3] for s in starts[b]] for b in range(4)])
    assert np.array_equal(got, want)


def _grad_cases():
    """x [w, h, cin, b], w [kw, kh, cin, cout] (Julia dim order, as the traced program sees them), forward
    cross-correlation with stride s, padding p (symmetric per dim), dilation d."""
    return [dict(W=9, H=8, ci=3, co=4, B=2, kw=3, kh=2, s=(1, 1), p=(0, 0), d=(1, 1)),
            dict(W=10, H=9, ci=2, co=3, B=2, kw=3, kh=3, s=(2, 1), p=(1, 2), d=(1, 1)),
            dict(W=11, H=10, ci=2, co=2, B=3, kw=2, kh=3, s=(1, 2), p=(2, 0), d=(2, 1))]


def _dil(n, d):
    return max(0, 1 + d * (n - 1))


def conv_grad_modules(c, dt):
    """The two gradient convolutions as ext/ReactantNNlibExt/Implementations.jl:85-251 builds them."""
    ow = (c["W"] + 2 * c["p"][0] - _dil(c["kw"], c["d"][0])) // c["s"][0] + 1
    oh = (c["H"] + 2 * c["p"][1] - _dil(c["kh"], c["d"][1])) // c["s"][1] + 1
    xs, ws, ys = [c["W"], c["H"], c["ci"], c["B"]], [c["kw"], c["kh"], c["ci"], c["co"]], [ow, oh, c["co"], c["B"]]
    lhs_shape, k_shape, o_shape = (c["W"], c["H"]), (_dil(c["kw"], c["d"][0]), _dil(c["kh"], c["d"][1])), (_dil(ow, c["s"][0]), _dil(oh, c["s"][1]))
    # filter gradient: x is the input with batch = cin, feature = b; dy is the kernel with o = cout, i = b
    padf = [[c["p"][i], o_shape[i] - lhs_shape[i] + k_shape[i] - c["p"][i] - 1] for i in range(2)]
    tf, outf = NN.convolution(xs, ys, dt, dims="[0, 1, b, f]x[0, 1, o, i]->[0, 1, b, f]", strides=list(c["d"]), padding=padf, rhs_dil=list(c["s"]))
    assert outf == ws, (outf, ws)
    # data gradient: dy is the input (dilated by the stride), the reversed kernel has o = cin, i = cout
    padd = []
    for i in range(2):
        before = k_shape[i] - c["p"][i] - 1
        padd.append([before, lhs_shape[i] + k_shape[i] - 1 - o_shape[i] - before])
    td, outd = NN.convolution(ys, ws, dt, dims="[0, 1, f, b]x[0, 1, o, i]->[0, 1, f, b]", padding=padd, lhs_dil=list(c["s"]), rhs_dil=list(c["d"]), flip=True)
    assert outd == xs, (outd, xs)
    return tf, td, xs, ws, ys


def conv_grads_brute(c, x, w, dy):
    """Derivatives of sum(y * dy), y the forward cross-correlation, from the definition."""
    ow, oh = dy.shape[0], dy.shape[1]
    dw, dx = np.zeros_like(w), np.zeros_like(x)
    for kx in range(c["kw"]):
        for ky in range(c["kh"]):
            for ox in range(ow):
                ix = ox * c["s"][0] + kx * c["d"][0] - c["p"][0]
                if not 0 <= ix < c["W"]:
                    continue
                for oy in range(oh):
                    iy = oy * c["s"][1] + ky * c["d"][1] - c["p"][1]
                    if not 0 <= iy < c["H"]:
                        continue
                    dw[kx, ky] += x[ix, iy] @ dy[ox, oy].T                 # [ci, b] x [b, co]
                    dx[ix, iy] += w[kx, ky] @ dy[ox, oy]                   # [ci, co] x [co, b]
    return dw, dx


def test_convolution_gradient_forms_against_the_definition():
    """The dimension-number forms of the filter and data gradients (batch and feature roles swapped,
    input dilation, reversed kernel) give the derivatives of the forward pass."""
    rng = np.random.default_rng(6)
    for c in _grad_cases():
        tf, td, xs, ws, ys = conv_grad_modules(c, "f64")
        x, w, dy = rng.normal(size=xs), rng.normal(size=ws), rng.normal(size=ys)
        dw, dx = conv_grads_brute(c, x, w, dy)
        got_w = I.run_text(tf, [I.tensor(x, "f64"), I.tensor(dy, "f64")])[0].a
        got_x = I.run_text(td, [I.tensor(dy, "f64"), I.tensor(w, "f64")])[0].a
        assert np.allclose(got_w, dw, rtol=1e-12, atol=1e-12), c
        assert np.allclose(got_x, dx, rtol=1e-12, atol=1e-12), c


def grouped_filter_grad_module(c, groups, dt):
    """Filter gradient of a grouped convolution: `batch_group_count = groups`
    (ext/ReactantNNlibExt/Implementations.jl:85-140)."""
    ow = (c["W"] + 2 * c["p"][0] - _dil(c["kw"], c["d"][0])) // c["s"][0] + 1
    oh = (c["H"] + 2 * c["p"][1] - _dil(c["kh"], c["d"][1])) // c["s"][1] + 1
    xs, ys = [c["W"], c["H"], c["ci"], c["B"]], [ow, oh, c["co"], c["B"]]
    ws = [c["kw"], c["kh"], c["ci"] // groups, c["co"]]
    lhs_shape, k_shape, o_shape = (c["W"], c["H"]), (_dil(c["kw"], c["d"][0]), _dil(c["kh"], c["d"][1])), (_dil(ow, c["s"][0]), _dil(oh, c["s"][1]))
    padf = [[c["p"][i], o_shape[i] - lhs_shape[i] + k_shape[i] - c["p"][i] - 1] for i in range(2)]
    tf, outf = NN.convolution(xs, ys, dt, dims="[0, 1, b, f]x[0, 1, o, i]->[0, 1, b, f]", strides=list(c["d"]), padding=padf,
                              rhs_dil=list(c["s"]), batch_groups=groups)
    assert outf == ws, (outf, ws)
    return tf, xs, ws, ys


def test_grouped_filter_gradient_against_the_definition():
    rng = np.random.default_rng(7)
    for groups, c in ((2, dict(W=9, H=8, ci=4, co=6, B=2, kw=3, kh=2, s=(1, 1), p=(1, 0), d=(1, 1))),
                      (3, dict(W=10, H=7, ci=6, co=3, B=3, kw=2, kh=2, s=(2, 1), p=(0, 1), d=(1, 2)))):
        tf, xs, ws, ys = grouped_filter_grad_module(c, groups, "f64")
        x, dy = rng.normal(size=xs), rng.normal(size=ys)
        cpg, opg = c["ci"] // groups, c["co"] // groups
        dw = np.zeros(ws)
        for g in range(groups):
            cg = dict(c, ci=cpg, co=opg)
            dwg, _ = conv_grads_brute(cg, x[:, :, g * cpg:(g + 1) * cpg], np.zeros([c["kw"], c["kh"], cpg, opg]), dy[:, :, g * opg:(g + 1) * opg])
            dw[:, :, :, g * opg:(g + 1) * opg] = dwg
        got = I.run_text(tf, [I.tensor(x, "f64"), I.tensor(dy, "f64")])[0].a
        assert np.allclose(got, dw, rtol=1e-12, atol=1e-12), (groups, c)


def test_scatter_against_numpy():
    """setindex! with index arrays (src/Ops.jl:2150-2172) and scatter-add, against numpy's indexed
    assignment / np.add.at; out-of-range updates are dropped."""
    rng = np.random.default_rng(14)
    dest = rng.normal(size=(6, 7))
    idx = np.array([[0, 0], [5, 6], [2, 3], [9, 1], [3, -1], [4, 4]])          # two of them out of range
    upd = rng.normal(size=6)
    t = NN.scatter([6, 7], [6, 2], [6], "f64", [], [0, 1], [0, 1], 1)
    got = I.run_text(t, [I.tensor(dest, "f64"), I.Tensor(idx, "i64"), I.tensor(upd, "f64")])[0].a
    want = dest.copy()
    for k in (0, 1, 2, 5):
        want[idx[k, 0], idx[k, 1]] = upd[k]
    assert np.array_equal(got, want)
    # rows added into a table, with repeated rows (what the gradient of an embedding lookup is)
    table = rng.normal(size=(10, 4))
    ids = np.array([3, 3, 0, 9, 3, 11])
    rows = rng.normal(size=(6, 4))
    t = NN.scatter([10, 4], [6], [6, 4], "f64", [1], [0], [0], 1, body="add")
    got = I.run_text(t, [I.tensor(table, "f64"), I.Tensor(ids, "i64"), I.tensor(rows, "f64")])[0].a
    want = table.copy()
    np.add.at(want, ids[:5], rows[:5])
    assert np.allclose(got, want, rtol=1e-14)
    # a window that sticks out of the operand is dropped as a whole
    base = np.zeros((8,))
    t = NN.scatter([8], [3, 1], [3, 3], "f64", [1], [], [0], 1, body="add")
    got = I.run_text(t, [I.tensor(base, "f64"), I.Tensor(np.array([[0], [6], [4]]), "i64"), I.tensor(np.ones((3, 3)), "f64")])[0].a
    assert got.tolist() == [1, 1, 1, 0, 1, 1, 1, 0]


def _nnlib_scatter_cases():
    import _nnlib_scatter_cases as C
    return [pytest.param(*c[1:], id=c[0]) for c in C.cases()]


@pytest.mark.parametrize("op,dst,src,idx,want", _nnlib_scatter_cases())
def test_scatter_nnlib_reference_vectors(op, dst, src, idx, want):
    """NNlib.scatter! / scatter known answers (test/nn/scatter_gather.jl:254-428) through the module the
    reference's lowering builds (ext/ReactantNNlibExt/Implementations.jl:477-530): pins the roles of
    update_window_dims, inserted_window_dims, scatter_dims_to_operand_dims and index_vector_dim, and
    the argument order of the update computation (element first: subtract and divide)."""
    text = NN.nnlib_scatter(op, list(dst.shape), list(src.shape), list(idx.shape))
    got = I.run_text(text, [I.tensor(dst, "f32"), I.Tensor(idx.reshape((1,) + idx.shape), "i64"), I.tensor(src, "f32")])[0].a
    np.testing.assert_allclose(got, want, rtol=1e-6)


def test_polybench_stencil_modules_follow_the_julia_loops():
    """The four vectorized polybench programs (benchmark/polybench/stencil.jl) as `stablehlo.while`
    modules over dim-reversed tensors, against loop nests written from the Julia source on arrays
    indexed like the Julia ones: pins the module builders (offsets, update boxes, the reversal of
    dims) and the oracle's while / dynamic_update_slice on them, bit for bit."""
    import _polybench_cases as C
    rng = np.random.default_rng(5)
    f = lambda *s: rng.random(s, dtype=np.float32)
    rt = lambda a: I.tensor(np.ascontiguousarray(a.T), "f32")          # Julia array -> dim-reversed tensor
    A, B = f(37), f(37)
    out = I.run_text(C.P.jacobi_1d(37, 5), [rt(A), rt(B)])
    for got, want in zip(out, C.jacobi_1d(5, A, B)):
        assert np.array_equal(got.a.T, want)
    A, B = f(13, 13), f(13, 13)
    out = I.run_text(C.P.jacobi_2d(13, 4), [rt(A), rt(B)])
    for got, want in zip(out, C.jacobi_2d(4, A, B)):
        assert np.array_equal(got.a.T, want)
    A, B = f(9, 9, 9), f(9, 9, 9)
    out = I.run_text(C.P.heat_3d(9, 3), [rt(A), rt(B)])
    for got, want in zip(out, C.heat_3d(3, A, B)):
        assert np.array_equal(got.a.T, want)
    EX, EY, HZ, fict = f(11, 7), f(11, 7), f(11, 7), f(6)
    out = I.run_text(C.P.fdtd_2d(11, 7, 6), [rt(EX), rt(EY), rt(HZ), I.tensor(fict, "f32")])
    assert np.array_equal(out[0].a.T, C.fdtd_2d(EX, EY, HZ, fict))


def _linalg_names():
    import _polybench_cases as C
    return sorted(C.LINALG_SMALL)


@pytest.mark.parametrize("name", _linalg_names())
def test_polybench_linalg_modules_follow_the_julia_formulas(name):
    """The vectorized BLAS / linear-algebra / data-mining programs of benchmark/polybench as modules over
    dim-reversed tensors, against the Julia formulas evaluated by numpy in float64: pins the builders
    (which operand of a dot_general is which, the adjoints, Julia's broadcasting of row and column vectors)."""
    import _polybench_cases as C
    text, shapes = C.P.linalg(name, **C.LINALG_SMALL[name])
    args = C.linalg_args(shapes, seed=len(name))
    got = I.run_text(text, [C.to_tensor(I, a) for a in args], hifi=True)
    want = C.LINALG_REFERENCE[name](*C._f64(args))
    assert len(got) == len(want)
    for g_, w_ in zip(got, want):
        g_ = C.from_tensor(g_)
        assert g_.shape == w_.shape
        assert np.max(np.abs(g_ - w_)) <= 2e-6 * max(1.0, np.max(np.abs(w_)))


SAS_CASES = [
    # x shape, window, strides, padding
    ([2, 3, 8, 8], [1, 1, 2, 2], [1, 1, 2, 2], None),
    ([2, 3, 9, 11], [1, 1, 3, 3], [1, 1, 2, 2], [[0, 0], [0, 0], [1, 1], [1, 1]]),
    ([1, 2, 7, 7], [1, 1, 3, 3], [1, 1, 1, 1], None),                              # overlapping windows
    ([3, 1, 10, 6], [1, 1, 2, 3], [1, 1, 2, 3], [[0, 0], [0, 0], [1, 1], [0, 0]]),
]


@pytest.mark.parametrize("xs,w,st,pd", SAS_CASES)
def test_select_and_scatter_is_the_gradient_of_max_pooling(xs, w, st, pd):
    """The oracle's select_and_scatter (GE select, add scatter) against torch's max_pool2d backward, a
    library routine; ties are rare in random data, the tie rule is pinned below."""
    import torch
    rng = np.random.default_rng(3)
    text, ss = NN.select_and_scatter(xs, "f32", w, st, pd)
    x, dy = rng.normal(size=xs).astype(np.float32), rng.normal(size=ss).astype(np.float32)
    got = I.run_text(text, [I.tensor(x, "f32"), I.tensor(dy, "f32")])[0].a
    xt = torch.tensor(x, requires_grad=True)
    y = torch.nn.functional.max_pool2d(xt, kernel_size=(w[2], w[3]), stride=(st[2], st[3]), padding=(pd[2][0], pd[3][0]) if pd else 0)
    assert list(y.shape) == ss
    y.backward(torch.tensor(dy))
    np.testing.assert_allclose(got, xt.grad.numpy(), rtol=0, atol=1e-6)


def test_select_and_scatter_ties_and_padding():
    """On a constant operand GE keeps the first element of a window (row-major) and GT moves on to the
    last; elements of the padding are never selected; LE / LT select minima the same way."""
    x = np.ones((1, 1, 4, 4), np.float32)
    dy = np.arange(1, 5, dtype=np.float32).reshape(1, 1, 2, 2)
    for direction, corner in (("GE", (0, 0)), ("GT", (1, 1)), ("LE", (0, 0)), ("LT", (1, 1))):
        text, ss = NN.select_and_scatter([1, 1, 4, 4], "f32", [1, 1, 2, 2], [1, 1, 2, 2], None, direction=direction)
        got = I.run_text(text, [I.tensor(x, "f32"), I.tensor(dy, "f32")])[0].a[0, 0]
        want = np.zeros((4, 4), np.float32)
        for i in range(2):
            for j in range(2):
                want[2 * i + corner[0], 2 * j + corner[1]] = dy[0, 0, i, j]
        assert np.array_equal(got, want), direction
    # one row of padding above and below: windows (rows -1..0) and (rows 3..4) select inside the operand
    text, ss = NN.select_and_scatter([1, 1, 4, 2], "f32", [1, 1, 2, 2], [1, 1, 2, 2], [[0, 0], [0, 0], [1, 1], [0, 0]])
    assert ss == [1, 1, 3, 1]
    x = -np.arange(8, dtype=np.float32).reshape(1, 1, 4, 2) - 100.0            # all far below zero
    got = I.run_text(text, [I.tensor(x, "f32"), I.tensor(np.array([1, 10, 100], np.float32).reshape(1, 1, 3, 1), "f32")])[0].a[0, 0]
    assert np.array_equal(got, np.array([[1, 0], [10, 0], [0, 0], [100, 0]], np.float32))
