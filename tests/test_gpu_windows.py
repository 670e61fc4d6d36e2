"""Windowed ops on the GPU against the oracle: reverse, reduce_window in its pooling forms (window
view + reduction) and its cumulative forms (prefix scans), convolution (window matrix + matrix
product).  Cases follow the reference's tests: test/core/ops.jl:609-618 (reverse),
test/core/map_reduction.jl:165-229 (cumsum / cumprod), test/nn/convolution.jl:160-217 (groups x
stride x padding x dilation grid, 1-d flip vectors)."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run, max_rel_to_scale
from oracle import stablehlo_interp as I
import _nn_modules as NN

pytestmark = pytest.mark.gpu


def _args(shapes, dt, seed=0, lo=None):
    rng = np.random.default_rng(seed)
    out = []
    for sh in shapes:
        if dt[0] == "i":
            out.append(I.Tensor(rng.integers(-1000, 1000, size=sh).astype(I.NP_OF[dt]), dt))
        elif lo is not None:
            out.append(I.tensor(rng.uniform(lo[0], lo[1], size=sh), dt))
        else:
            out.append(I.tensor(rng.normal(size=sh), dt))
    return out


def _close(got, ref, tol):
    assert got.shape == ref.shape
    same_inf = np.array_equal(np.isinf(got), np.isinf(ref)) and np.array_equal(np.isnan(got), np.isnan(ref))
    assert same_inf
    fin = np.isfinite(ref)
    if fin.any():
        scale = max(float(np.max(np.abs(ref[fin]))), 1e-30)
        assert float(np.max(np.abs(got[fin].astype(np.float64) - ref[fin].astype(np.float64)))) / scale <= tol


def test_reverse_reference_vectors(rx, client):
    t = ("module {\n func.func @main(%arg0: tensor<4xi64>) -> tensor<4xi64> {\n"
         "  %0 = stablehlo.reverse %arg0, dims = [0] : tensor<4xi64>\n  return %0 : tensor<4xi64>\n }\n}\n")
    got, _ = gpu_run(rx, client, t, [I.Tensor(np.array([1, 2, 3, 4]), "i64")])
    assert got[0].a.tolist() == [4, 3, 2, 1]
    t2 = ("module {\n func.func @main(%arg0: tensor<3x5x4xf32>) -> tensor<3x5x4xf32> {\n"
          "  %0 = stablehlo.reverse %arg0, dims = [0, 2] : tensor<3x5x4xf32>\n"
          "  %1 = stablehlo.negate %0 : tensor<3x5x4xf32>\n  return %1 : tensor<3x5x4xf32>\n }\n}\n")
    a = _args([(3, 5, 4)], "f32")
    got, _ = gpu_run(rx, client, t2, a)
    assert np.array_equal(got[0].a, -a[0].a[::-1, :, ::-1])


def test_cumulative_reference_cases(rx, client):
    a = I.tensor(np.arange(1, 11) / 10, "f32")
    for body, lib in (("add", np.cumsum), ("multiply", np.cumprod)):
        got, exe = gpu_run(rx, client, NN.cumulative([10], "f32", 0, body), [a])
        assert [l["kind"] for l in exe.launches()] == ["scan"]
        assert np.allclose(got[0].a, lib(a.a.astype(np.float64)), rtol=1e-6)
    b = I.tensor(np.arange(1, 61).reshape(5, 4, 3) / 60, "f32")
    for raw in range(3):
        for body, lib in (("add", np.cumsum), ("multiply", np.cumprod)):
            got, _ = gpu_run(rx, client, NN.cumulative([5, 4, 3], "f32", raw, body), [b])
            assert np.allclose(got[0].a, lib(b.a.astype(np.float64), axis=raw), rtol=1e-6)


# (shape, dtype, dim, body, from the end, launch kinds)
SCANS = [
    ([1 << 22], "f32", 0, "add", False, ["scan"]),               # long rows: one launch
    ([100003], "f64", 0, "add", False, ["scan"]),
    ([100003], "i32", 0, "add", True, ["scan"]),
    ([512, 3000], "f32", 1, "add", False, ["scan"]),
    ([3, 70001], "f32", 1, "maximum", True, None),
    ([3000, 512], "f32", 0, "add", False, None),
    ([100000, 8], "f32", 0, "add", False, ["scan_totals", "scan"]),
    ([7, 300, 33], "f32", 1, "add", True, None),
    ([64, 1000], "f64", 1, "multiply", True, ["scan"]),
    ([1000, 64], "f32", 0, "minimum", False, None),
    ([300, 1000], "i32", 1, "add", False, ["scan"]),
    ([300, 1000], "i64", 0, "add", False, None),
    ([100000, 10], "f32", 1, "add", False, ["scan"]),
    ([2, 1500], "bf16", 1, "add", False, ["scan"]),
    ([2, 300], "bf16", 0, "maximum", False, ["scan"]),
]


@pytest.mark.parametrize("shape,dt,dim,body,rev,kinds", SCANS)
def test_prefix_scans(rx, client, shape, dt, dim, body, rev, kinds):
    text = NN.cumulative(shape, dt, dim, body, rev)
    args = _args([shape], dt, seed=7, lo=(0.98, 1.02) if body == "multiply" else None)
    got, exe = gpu_run(rx, client, text, args)
    got_kinds = [l["kind"] for l in exe.launches()]
    assert set(got_kinds) <= {"scan_totals", "scan"}, got_kinds
    if kinds is not None:
        assert got_kinds == kinds
    ref = oracle_run(text, args, hifi=True)
    if dt[0] == "i" or body in ("maximum", "minimum"):
        assert np.array_equal(got[0].a, ref[0].a)
    elif dt == "bf16":
        _close(got[0].a, ref[0].a, 1e-2)
    elif dt == "f64":
        _close(got[0].a, ref[0].a, 1e-12)
    else:
        _close(got[0].a, ref[0].a, 1e-5 * np.sqrt(shape[dim]))


# long rows in one launch: chunks of 16 tiles (16384 elements of 4 bytes), totals per chunk / 32 chunks / 1024 chunks
ONE_LAUNCH_SCANS = [
    ([1 << 25], "f32", 0, "add", False),         # 2048 chunks: 8 groups of 256; carries use group totals from two groups back
    ([3000001], "f32", 0, "add", False),          # ragged last chunk, partial last group, scalar loads (odd length)
    ([3000000], "i32", 0, "add", True),           # from the end; integers are exact
    ([9000000], "i64", 0, "add", False),          # two flagged words per total; 1099 chunks, five groups
    ([1200000], "f64", 0, "multiply", False),
    ([3, 700000], "f32", 1, "maximum", True),     # several rows, each with its own slots
    ([5, 40000], "bf16", 1, "add", False),
    ([2, 16385], "f32", 1, "add", False),         # two chunks, the second of one element
]


@pytest.mark.parametrize("shape,dt,dim,body,rev", ONE_LAUNCH_SCANS)
def test_prefix_scans_of_long_rows_in_one_launch(rx, client, monkeypatch, shape, dt, dim, body, rev):
    """The one-launch form of a scan over long rows against the oracle and against the two-launch form (bit for bit where
    the operation is exact), three runs of one executable: the slots are cleared by the run that used them."""
    text = NN.cumulative(shape, dt, dim, body, rev)
    args = _args([shape], dt, seed=9, lo=(0.999999, 1.000001) if body == "multiply" else None)
    monkeypatch.setenv("RX_SINGLE_PASS_SCAN", "0")
    two, exe2 = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe2.launches()] == ["scan_totals", "scan"]
    monkeypatch.setenv("RX_SINGLE_PASS_SCAN", "1")
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["scan"]
    ref = oracle_run(text, args, hifi=True)
    exact = dt[0] == "i" or body in ("maximum", "minimum")
    for run in range(3):
        if exact:
            assert np.array_equal(got[0].a, ref[0].a) and got[0].a.tobytes() == two[0].a.tobytes()
        elif dt == "bf16":
            _close(got[0].a, ref[0].a, 1e-2)
        elif dt == "f64":
            _close(got[0].a, ref[0].a, 1e-12)
        else:
            _close(got[0].a, ref[0].a, 1e-5 * np.sqrt(shape[dim]))
        if run == 0:
            first = got[0].a.tobytes()
        else:
            assert got[0].a.tobytes() == first        # fixed combination order: the same bits every run
        got, _ = gpu_run(rx, client, text, args, exe=exe)


def test_a_wait_that_expires_is_reported(rx, client, monkeypatch):
    """A workgroup of the one-launch scan waits, for a bounded number of polls, for totals that lower-numbered workgroups
    publish.  With the bound forced to zero polls from the host some wait expires (every kernel still runs to its end): the
    kernel sets the device's fault word and the next call that waits for the device raises instead of returning the result.
    The same executable is then rebuilt in the two-launch form on its next execution and gives the right answer, as does
    every executable compiled through that client afterwards (a client of its own: the switch is per client)."""
    client = rx.Client()
    text = NN.cumulative([1 << 24], "f32", 0, "add", False)
    args = _args([[1 << 24]], "f32", seed=3)
    ref = np.cumsum(args[0].a.astype(np.float64))
    monkeypatch.setenv("RX_SCAN_SPIN_LIMIT", "0")
    exe = rx.xla_compile(client, text)
    assert [l["kind"] for l in exe.launches()] == ["scan"]
    with pytest.raises(rx.ReactantInternalError, match="bounded wait for another workgroup"):
        for _ in range(3):       # a run in which every slot happens to be there in time is possible, three in a row are not
            gpu_run(rx, client, text, args, exe=exe)
    # the same executable again, the zero bound still set: it no longer waits
    for _ in range(2):
        got, _ = gpu_run(rx, client, text, args, exe=exe)
        _close(got[0].a, ref, 1e-5 * np.sqrt(1 << 24))
    assert [l["kind"] for l in exe.launches()] == ["scan_totals", "scan"]
    monkeypatch.delenv("RX_SCAN_SPIN_LIMIT")
    got, exe2 = gpu_run(rx, client, text, args)          # the device is usable afterwards and the word was cleared
    assert [l["kind"] for l in exe2.launches()] == ["scan_totals", "scan"]
    _close(got[0].a, ref, 1e-5 * np.sqrt(1 << 24))


def test_scan_of_a_fused_producer_and_into_a_consumer(rx, client):
    """cumsum(abs2.(x)) ./ sum: the producer is evaluated inside the scan kernels, the consumer reads its result."""
    t = ("module {\n func.func @main(%arg0: tensor<64x5000xf32>) -> tensor<64x5000xf32> {\n"
         "  %sq = stablehlo.multiply %arg0, %arg0 : tensor<64x5000xf32>\n"
         "  %c = stablehlo.constant dense<0.000000e+00> : tensor<f32>\n"
         "  %0 = \"stablehlo.reduce_window\"(%sq, %c) <{base_dilations = array<i64: 1, 1>, padding = dense<[[0, 0], [4999, 0]]> : tensor<2x2xi64>, "
         "window_dilations = array<i64: 1, 1>, window_dimensions = array<i64: 1, 5000>, window_strides = array<i64: 1, 1>}> ({\n"
         "  ^bb0(%a: tensor<f32>, %b: tensor<f32>):\n    %s = stablehlo.add %a, %b : tensor<f32>\n    stablehlo.return %s : tensor<f32>\n"
         "  }) : (tensor<64x5000xf32>, tensor<f32>) -> tensor<64x5000xf32>\n"
         "  %h = stablehlo.constant dense<5.000000e-01> : tensor<64x5000xf32>\n"
         "  %1 = stablehlo.multiply %0, %h : tensor<64x5000xf32>\n"
         "  return %1 : tensor<64x5000xf32>\n }\n}\n")
    args = _args([(64, 5000)], "f32", seed=2)
    got, exe = gpu_run(rx, client, t, args)
    assert [l["kind"] for l in exe.launches()] in (["scan_totals", "scan", "map"], ["scan", "map"])
    ref = np.cumsum(args[0].a.astype(np.float64) ** 2, axis=1) * 0.5
    _close(got[0].a, ref, 1e-5 * np.sqrt(5000))


POOLS = [
    ([8, 16, 32, 32], "f32", "maximum", [1, 1, 2, 2], [1, 1, 2, 2], None, None, None),
    ([8, 16, 32, 32], "f32", "add", [1, 1, 2, 2], [1, 1, 2, 2], None, None, None),
    ([2, 3, 17, 19], "f32", "add", [1, 1, 3, 3], [1, 1, 2, 2], [[0, 0], [0, 0], [1, 1], [1, 1]], None, None),
    ([2, 3, 17, 19], "f32", "maximum", [1, 1, 3, 2], [1, 1, 1, 2], [[0, 0], [0, 0], [2, 1], [0, 3]], [1, 1, 2, 1], [1, 1, 2, 3]),
    ([4, 6, 40], "f64", "minimum", [1, 1, 5], [1, 1, 3], [[0, 0], [0, 0], [2, 2]], None, None),
    ([2, 4, 9, 10, 11], "f32", "maximum", [1, 1, 2, 2, 2], [1, 1, 2, 2, 2], None, None, None),
    ([4, 4, 28, 28], "bf16", "maximum", [1, 1, 3, 3], [1, 1, 2, 2], [[0, 0], [0, 0], [1, 1], [1, 1]], None, None),
    ([6, 50, 50], "i32", "add", [1, 3, 3], [1, 1, 1], [[0, 0], [1, 1], [1, 1]], None, None),
]


@pytest.mark.parametrize("shape,dt,body,window,strides,padding,bd,wd", POOLS)
def test_pooling_windows(rx, client, shape, dt, body, window, strides, padding, bd, wd):
    text, out_shape = NN.reduce_window(shape, dt, body, window, strides, padding, bd, wd)
    args = _args([shape], dt, seed=11)
    got, exe = gpu_run(rx, client, text, args)
    assert all(l["kind"] in ("reduce_generic", "reduce_final", "row") for l in exe.launches())
    ref = oracle_run(text, args, hifi=True)
    assert list(got[0].a.shape) == out_shape
    if dt[0] == "i" or body in ("maximum", "minimum"):
        assert np.array_equal(got[0].a, ref[0].a)
    else:
        _close(got[0].a, ref[0].a, 1e-6 * np.prod(window))


def test_conv_1d_flip_reference_vectors(rx, client):
    x = I.tensor(np.array([[[1.0, 2.0, 3.0]]]), "f32")
    for flip, want in ((False, [8.0, 14.0, 8.0]), (True, [4.0, 10.0, 12.0])):
        for generic in (False, True):
            text, _ = NN.convolution([1, 1, 3], [1, 1, 3], "f32", dims="[b, f, 0]x[o, i, 0]->[b, f, 0]", padding=[[1, 1]], flip=flip, generic=generic)
            got, _ = gpu_run(rx, client, text, [x, x])
            assert got[0].a.reshape(-1).tolist() == want


CONV_GRID = [(g, s, p, d) for g in (1, 2, 4) for s in ((1, 1), (2, 2), (3, 3))
             for p in ((0, 0), (2, 2), (0, 2), (2, 0)) for d in ((1, 1), (1, 2))]


@pytest.mark.parametrize("groups", [1, 2, 4])
def test_convolution_reference_grid(rx, client, groups):
    """x 16x16x8x2, weight 4x4x(8/groups)x4 in Julia order, i.e. raw [2, 8, 16, 16] and [4, 8/groups, 4, 4]."""
    xs, ws = [2, 8, 16, 16], [4, 8 // groups, 4, 4]
    args = _args([xs, ws], "f32", seed=groups)
    for (g, s, p, d) in CONV_GRID:
        if g != groups:
            continue
        # Julia's dim 1 is the raw minor dim: spatial dim 0 sits at raw position 3
        text, out_shape = NN.convolution(xs, ws, "f32", strides=list(s), padding=[[p[0], p[0]], [p[1], p[1]]],
                                         rhs_dil=list(d), groups=g, flip=True)
        got, _ = gpu_run(rx, client, text, args)
        ref = oracle_run(text, args, hifi=True)
        assert list(got[0].a.shape) == out_shape
        _close(got[0].a, ref[0].a, 1e-5 * np.sqrt(8 // g * 16))


CONVS = [
    # x, w, dtype, dims, kwargs, expected kind of the product
    # f32, unit strides and dilations, at least 33 output features: the direct-convolution kernel (bias + relu in its epilogue)
    ([4, 64, 56, 56], [64, 64, 3, 3], "f32", None, dict(padding=[[1, 1], [1, 1]], epilogue="bias_relu"), "conv"),
    # the same as a matrix product on the window matrix
    ([4, 64, 56, 56], [64, 64, 3, 3], "f32", None, dict(padding=[[1, 1], [1, 1]], epilogue="bias_relu", env={"RX_CONV_DIRECT": "0"}), "gemm_f32"),
    # a 5x3 filter, uneven padding, channels that are not whole slabs of 8, 48 features (three of the four wavefronts), a ragged last tile
    ([3, 20, 30, 36], [48, 20, 5, 3], "f32", None, dict(padding=[[2, 1], [0, 2]]), "conv"),
    # rows of the image and of the result that are not whole 16-byte vectors, no padding, 40 features
    ([2, 9, 21, 23], [40, 9, 3, 3], "f32", None, dict(), "conv"),
    # channels-last images and [rows, columns, in, out] filters: transposes around the kernel
    ([2, 16, 20, 8], [3, 3, 8, 64], "f32", "[b, 0, 1, f]x[0, 1, i, o]->[b, 0, 1, f]", dict(padding=[[1, 1], [1, 1]]), "conv"),
    # strides: a 7x7/2 stem with three channels (one slab, one LDS stage) and a 3x3/2 layer with two groups of 64 features
    ([2, 3, 64, 64], [64, 3, 7, 7], "f32", None, dict(strides=[2, 2], padding=[[3, 3], [3, 3]]), "conv"),
    ([3, 24, 30, 28], [128, 24, 3, 3], "f32", None, dict(strides=[2, 1], padding=[[1, 1], [1, 0]], epilogue="bias_relu"), "conv"),
    # a dilated filter with unequal strides, flipped (NNlib's true convolution)
    ([2, 16, 24, 28], [48, 16, 3, 3], "f32", None, dict(strides=[1, 2], rhs_dil=[2, 3], padding=[[2, 2], [3, 3]], flip=True), "conv"),
    # a 1x1 filter (a product over the channels), 7x7 images, bias + relu
    ([8, 128, 16, 16], [96, 128, 1, 1], "f32", None, dict(epilogue="bias_relu"), "conv"),
    # fewer than 16 channels in 16 bits (a network's first layer): converted to f32 for the direct kernel, back in its epilogue
    ([2, 8, 28, 28], [64, 8, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]]), "conv"),
    ([2, 3, 64, 64], [64, 3, 7, 7], "f16", None, dict(strides=[2, 2], padding=[[3, 3], [3, 3]], epilogue="bias_relu"), "conv"),
    # 32 channels: zero channels up to 64
    ([2, 32, 28, 28], [64, 32, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]]), "conv_bf16"),
    # 16-bit images with whole 128-byte runs of channels, unit strides: a product over the zero-padded [image, row, column,
    # channel] data with one row shift per tap (no window matrix) -- 64 x 64 and 128 x 64 tiles of the direct-to-LDS skeleton,
    ([2, 64, 40, 40], [128, 64, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]], epilogue="bias_relu"), "conv_bf16"),
    ([4, 64, 64, 64], [64, 64, 5, 5], "bf16", None, dict(padding=[[2, 2], [2, 2]], flip=True), "conv_bf16"),
    # f16, a dilated 2 x 3 filter, uneven padding; a 1 x 1 filter; channels-last images and [rows, columns, in, out] filters
    ([2, 128, 30, 26], [64, 128, 2, 3], "f16", None, dict(padding=[[0, 1], [2, 0]], rhs_dil=[2, 1]), "conv_f16"),
    ([2, 64, 24, 24], [128, 64, 1, 1], "bf16", None, dict(), "conv_bf16"),
    ([2, 20, 16, 64], [3, 3, 64, 128], "bf16", "[b, 0, 1, f]x[0, 1, i, o]->[b, 0, 1, f]", dict(padding=[[1, 1], [1, 1]]), "conv_bf16"),
    # a strided 1 x 1 filter: the images are sliced, then the product (one tap)
    ([8, 64, 57, 56], [128, 64, 1, 1], "bf16", None, dict(strides=[2, 3]), "conv_bf16"),
    # 96 channels: zero channels up to 128
    ([8, 96, 48, 48], [64, 96, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]]), "conv_bf16"),
    # the streaming skeletons: 256 x 128 tiles, and 256 x 256 tiles in the ping-pong form
    ([8, 64, 94, 94], [128, 64, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]]), "conv_bf16"),
    ([4, 64, 90, 90], [512, 64, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]], epilogue="bias_relu"), "conv_bf16"),
    # the same data through the window matrix
    ([2, 64, 40, 40], [128, 64, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]], epilogue="bias_relu", env={"RX_CONV_SHIFT": "0"}), "gemm_bf16"),
    ([1, 3, 33, 35], [16, 3, 5, 5], "f32", None, dict(strides=[2, 2], padding=[[2, 2], [2, 2]]), "gemm_f32"),
    ([16, 16, 8, 2], [4, 4, 8, 4], "f32", "[1, 0, f, b]x[1, 0, i, o]->[1, 0, f, b]", dict(), None),
    ([2, 16, 16, 8], [4, 4, 8, 4], "f32", "[b, 1, 0, f]x[1, 0, i, o]->[b, 1, 0, f]", dict(padding=[[1, 2], [0, 1]]), None),
    ([3, 5, 40], [7, 5, 3], "f32", "[b, f, 0]x[o, i, 0]->[b, f, 0]", dict(lhs_dil=[2], padding=[[2, 2]]), None),
    ([2, 3, 8, 8, 8], [3, 3, 3, 3, 3], "f32", "[b, f, 2, 1, 0]x[o, i, 2, 1, 0]->[b, f, 2, 1, 0]", dict(padding=[[1, 1], [1, 1], [1, 1]]), None),
    ([2, 6, 20, 20], [12, 3, 3, 3], "f64", None, dict(groups=2, generic=True), None),
    ([8, 32, 14, 14], [32, 1, 3, 3], "f32", None, dict(groups=32, padding=[[1, 1], [1, 1]]), None),
    # 160 output features: three groups of 64 features in the direct kernel's grid
    ([2, 160, 20, 20], [160, 160, 3, 3], "f32", None, dict(padding=[[1, 1], [1, 1]]), "conv"),
    # small images: the matrix product, whose tiles span images (more than 128 output features: the window matrix is written to memory)
    ([2, 160, 10, 10], [160, 160, 3, 3], "f32", None, dict(padding=[[1, 1], [1, 1]]), "gemm_f32"),
    # 14 x 14 images: 13 blocks of 16 pixels per image in the direct kernel
    ([3, 96, 14, 14], [96, 96, 3, 3], "f32", None, dict(padding=[[1, 1], [1, 1]]), "conv"),
    # bf16 with more than 128 output features: the window matrix is written to memory instead of being evaluated by the product
    ([2, 160, 14, 14], [160, 160, 3, 3], "bf16", None, dict(padding=[[1, 1], [1, 1]]), "gemm_bf16"),
]


@pytest.mark.parametrize("xs,ws,dt,dims,kw,kind", CONVS)
def test_convolution_layouts_and_types(rx, client, xs, ws, dt, dims, kw, kind, monkeypatch):
    kw = dict(kw)
    for k, v in kw.pop("env", {}).items():
        monkeypatch.setenv(k, v)
    if kind == "conv":
        # the direct kernel wherever it covers the case: at these sizes the planner's estimate may prefer the matrix product
        monkeypatch.setenv("RX_CONV_DIRECT", "2")
    if dims:
        kw["dims"] = dims
    text, out_shape = NN.convolution(xs, ws, dt, **kw)
    shapes = [xs, ws] + ([[out_shape[1]]] if kw.get("epilogue") else [])
    args = _args(shapes, dt, seed=21)
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    if kind:
        assert kind in kinds, kinds
    ref = oracle_run(text, args, hifi=True)
    assert list(got[0].a.shape) == out_shape
    taps = int(np.prod(ws[1:])) if not dims or dims.startswith("[b, f") else int(np.prod(ws)) // max(ws)
    tol = 1e-2 if dt == "bf16" else (1e-3 if dt == "f16" else (1e-12 if dt == "f64" else 1e-5 * np.sqrt(taps)))   # 16 bits: an ulp or two of the largest result
    _close(got[0].a, ref[0].a, tol)


@pytest.mark.parametrize("shape,dt,feature,training", [([4, 16, 14, 14], "f32", 1, False), ([14, 14, 16, 4], "f32", 2, False),
                                                       ([64, 33], "f32", 1, True), ([8, 6, 30, 30], "f32", 1, True),
                                                       ([4, 16, 14, 14], "bf16", 1, False), ([5, 7, 9], "f64", 0, True)])
def test_batch_norm(rx, client, shape, dt, feature, training):
    text = NN.batch_norm(shape, dt, feature, 1e-3, training)
    rng = np.random.default_rng(13)
    nf = shape[feature]
    args = [I.tensor(rng.normal(1.0, 2.0, size=shape), dt), I.tensor(rng.uniform(0.5, 1.5, size=nf), dt), I.tensor(rng.normal(size=nf), dt)]
    if not training:
        args += [I.tensor(rng.normal(size=nf), dt), I.tensor(rng.uniform(0.5, 2.0, size=nf), dt)]
    got, exe = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True, excess=(dt == "bf16"))
    assert len(got) == (3 if training else 1)
    tol = {"f32": 2e-5, "bf16": 1e-2, "f64": 1e-12}[dt]
    for g, r in zip(got, ref):
        _close(g.a, r.a, tol)


@pytest.mark.parametrize("dt,kind,chained", [("bf16", "conv_bf16", True), ("bf16", "conv_bf16", False), ("f16", "conv_f16", True), ("f16", "conv_f16", False), ("f32", "conv", True)])
def test_chain_of_convolutions_with_bias_and_relu(rx, client, monkeypatch, dt, kind, chained):
    """Three 3x3 layers of 64 -> 64 features with bias + relu.  In 16 bits the products with row shifts: chained, a product
    writes bias + relu of its results straight into the next one's zero-padded operand (same grid, rows moved by the
    padding, zeros where a row is not a result), so nothing lies between the products (the filters' layout maps run first, as one launch); unchained
    (RX_CHAIN_CONVS=0), one map between them does that.  In f32 the direct kernel with its epilogue.  Against the oracle."""
    if not chained:
        monkeypatch.setenv("RX_CHAIN_CONVS", "0")
    text, shapes = NN.conv_chain(3, 64, 40, 3, dt)
    rng = np.random.default_rng(5)
    args = [I.tensor((rng.normal(size=s) * (0.05 if len(s) == 4 and k > 0 else 1.0)).astype(np.float32), dt) for k, s in enumerate(shapes)]
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    assert kinds.count(kind) == 3, kinds
    if dt != "f32" and chained:
        assert kinds == ["map", "map_transposed", kind, kind, kind, "map_transposed"], kinds     # the first map: the three filters' layouts in one launch
    elif dt != "f32":
        assert kinds == ["map", "map_transposed", kind, "map", kind, "map", kind, "map_transposed"], kinds
    ref = oracle_run(text, args, hifi=True)
    _close(got[0].a, ref[0].a, 2e-2 if dt == "bf16" else (4e-3 if dt == "f16" else 1e-4))


def test_chain_of_convolutions_when_the_kernels_take_no_epilogues(rx, client, monkeypatch):
    """RX_EPILOGUES=0: bias + relu run as a map after each product, so a product cannot write the next one's operand;
    the module is planned without the chaining and the results are the same."""
    monkeypatch.setenv("RX_EPILOGUES", "0")
    text, shapes = NN.conv_chain(2, 64, 24, 2, "bf16")
    rng = np.random.default_rng(6)
    args = [I.tensor((rng.normal(size=s) * (0.05 if len(s) == 4 and k > 0 else 1.0)).astype(np.float32), "bf16") for k, s in enumerate(shapes)]
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    assert kinds == ["map", "map_transposed", "conv_bf16", "map", "conv_bf16", "map_transposed"], kinds
    _close(got[0].a, oracle_run(text, args, hifi=True)[0].a, 2e-2)


@pytest.mark.parametrize("sizes", [dict(batch=2, cin=3, cmid=8, hw=16, classes=10), dict(batch=4, cin=3, cmid=64, hw=32, classes=100)])
def test_vgg_style_forward_pass(rx, client, sizes):
    text, shapes = NN.vgg_block(**sizes)
    rng = np.random.default_rng(17)
    args = []
    for k, sh in enumerate(shapes):
        if k == 5:      # running variance
            args.append(I.tensor(rng.uniform(0.5, 2.0, size=sh), "f32"))
        elif len(sh) == 4 and k > 0:
            args.append(I.tensor(rng.normal(size=sh) / np.sqrt(np.prod(sh[1:])), "f32"))
        else:
            args.append(I.tensor(rng.normal(size=sh), "f32"))
    got, exe = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True)
    assert got[0].a.shape == (sizes["batch"], sizes["classes"])
    assert np.allclose(got[0].a.sum(axis=1), 1.0, atol=1e-5)
    _close(got[0].a, ref[0].a, 1e-4)
    if sizes["cmid"] >= 64:
        assert any(l["kind"] == "conv" for l in exe.launches())


def test_vgg_style_forward_pass_in_bf16(rx, client):
    """The same op sequence on bf16 images of 64 channels: both convolutions are products with row shifts, whose
    channels-last results the batch norm, the pooling window and the mean pool read through the transposes' index maps."""
    sizes = dict(batch=4, cin=64, cmid=64, hw=32, classes=100)
    text, shapes = NN.vgg_block(dt="bf16", **sizes)
    rng = np.random.default_rng(19)
    args = []
    for k, sh in enumerate(shapes):
        if k == 5:      # running variance
            args.append(I.tensor(rng.uniform(0.5, 2.0, size=sh), "bf16"))
        elif len(sh) == 4 and k > 0:
            args.append(I.tensor(rng.normal(size=sh) / np.sqrt(np.prod(sh[1:])), "bf16"))
        else:
            args.append(I.tensor(rng.normal(size=sh), "bf16"))
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    assert kinds.count("conv_bf16") == 2, kinds
    ref = oracle_run(text, args, hifi=True)
    assert got[0].a.shape == (sizes["batch"], sizes["classes"])
    assert np.allclose(got[0].a.astype(np.float64).sum(axis=1), 1.0, atol=2e-2)
    _close(got[0].a, ref[0].a, 3e-2)


def _vgg11_args(shapes, dt, seed=23):
    rng = np.random.default_rng(seed)
    args = []
    for k, sh in enumerate(shapes):
        if len(sh) == 1 and 0 < k <= 40 and (k - 1) % 5 == 4:       # running variances
            args.append(I.tensor(rng.uniform(0.5, 2.0, size=sh), dt))
        elif len(sh) == 1 and 0 < k <= 40 and (k - 1) % 5 == 1:     # batch norm scales
            args.append(I.tensor(rng.uniform(0.8, 1.6, size=sh), dt))
        elif len(sh) == 4 and k > 0:
            args.append(I.tensor(rng.normal(size=sh) * np.sqrt(2.0 / np.prod(sh[1:])), dt))
        elif len(sh) == 2:
            args.append(I.tensor(rng.normal(size=sh) * np.sqrt(2.0 / sh[0]), dt))
        else:
            args.append(I.tensor(rng.normal(size=sh) * (1.0 if k == 0 else 0.3), dt))
    return args


@pytest.mark.parametrize("dt,nhwc", [("f32", True), ("bf16", True), ("bf16", False), ("f16", True)])
def test_vgg11_forward_pass(rx, client, monkeypatch, dt, nhwc):
    """The whole VGG-11 forward pass with batch norm in test mode (eight 3x3 convolutions + batch norm + relu, five
    2x2 max pools, three dense layers) at small sizes.  In 16 bits the pooling windows between two products with row
    shifts run on the channel-minor layout (no transposes between them; RX_NHWC_POOLS=0: through the transposes),
    the batch norm + relu as the products' epilogues.  Against the oracle."""
    if not nhwc:
        monkeypatch.setenv("RX_NHWC_POOLS", "0")
    layers = (64, "M", 64, "M", 64, 64, "M", 64, 64, "M", 64, 64, "M")
    text, shapes, _ = NN.vgg11(batch=4, hw=64, classes=10, dt=dt, layers=layers, dense=96, cin=3)
    args = _vgg11_args(shapes, dt)
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    if dt != "f32":
        assert kinds.count("conv_" + dt) == 7, kinds
        pools = [ln.split("::")[1] for ln in rx.compile_offline(text).splitlines() if "kind=reduce_generic" in ln and "window" in ln]
        assert len(pools) == 5
        # the pools between two products: pure window reductions on the channel-minor layout when the rewrite is on
        assert sum("divide" not in d for d in pools) == (4 if nhwc else 1), pools
    ref = oracle_run(text, args, hifi=True)
    assert got[0].a.shape == (4, 10)
    _close(got[0].a, ref[0].a, {"f32": 2e-4, "bf16": 5e-2, "f16": 8e-3}[dt])


@pytest.mark.parametrize("dt,regions", [("bf16", True), ("bf16", False), ("f16", True), ("f32", True)])
def test_residual_stage(rx, client, monkeypatch, dt, regions):
    """Three basic residual blocks (convolution + batch norm + relu + convolution + batch norm, the block's input added,
    relu).  In 16 bits the products with row shifts keep the values channel-minor through the whole stage: a block is
    two products -- batch norm + relu, and batch norm + the addition + relu, as their epilogues -- and a padding map; the
    stage's input is transposed once on the way in, its result once on the way out (RX_NHWC_REGIONS=0: a transposing
    map on either side of every second product).  Against the oracle."""
    if not regions:
        monkeypatch.setenv("RX_NHWC_REGIONS", "0")
    text, shapes, _ = NN.resnet_stage(batch=3, channels=64, hw=24, blocks=3, dt=dt)
    rng = np.random.default_rng(31)
    args = []
    for k, sh in enumerate(shapes):
        if len(sh) == 1 and (k - 1) % 5 == 4:
            args.append(I.tensor(rng.uniform(0.5, 2.0, size=sh), dt))
        elif len(sh) == 1 and (k - 1) % 5 == 1:
            args.append(I.tensor(rng.uniform(0.5, 1.0, size=sh), dt))
        elif len(sh) == 4 and k > 0:
            args.append(I.tensor(rng.normal(size=sh) * np.sqrt(1.0 / np.prod(sh[1:])), dt))
        else:
            args.append(I.tensor(rng.normal(size=sh) * (1.0 if k == 0 else 0.2), dt))
    got, exe = gpu_run(rx, client, text, args)
    kinds = [l["kind"] for l in exe.launches()]
    if dt != "f32":
        kind = "conv_" + dt
        assert kinds.count(kind) == 6, kinds
        if regions:
            assert kinds == ["map", "map_transposed", kind, "map_transposed", kind, "map", kind, kind, "map", kind, kind, "map_transposed"], kinds
        else:
            assert kinds.count("map_transposed") == 6, kinds
    ref = oracle_run(text, args, hifi=True)
    _close(got[0].a, ref[0].a, {"f32": 1e-4, "bf16": 3e-2, "f16": 5e-3}[dt])


@pytest.mark.parametrize("bh,seq,dim,dt,tol", [(6, 40, 16, "f32", 1e-5), (8, 256, 64, "f32", 1e-4), (8, 256, 64, "bf16", 2e-2)])
def test_attention_block(rx, client, bh, seq, dim, dt, tol):
    text, shapes = NN.attention_block(bh, seq, dim, dt)
    args = _args(shapes, dt, seed=19)
    got, exe = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True, excess=(dt == "bf16"))
    _close(got[0].a, ref[0].a, tol)


EDGES = [
    ("scan of an empty tensor", lambda: (NN.cumulative([5, 0], "f32", 0), [[5, 0]])),
    ("scan along a dimension of one element", lambda: (NN.cumulative([1, 7], "f32", 0), [[1, 7]])),
    ("scan of two elements", lambda: (NN.cumulative([2], "f32", 0), [[2]])),
    ("window larger than the operand", lambda: (NN.reduce_window([2, 3], "f32", "add", [3, 1])[0], [[2, 3]])),
    ("window of one element", lambda: (NN.reduce_window([4, 5], "f32", "maximum", [1, 1])[0], [[4, 5]])),
    ("convolution of an empty batch", lambda: (NN.convolution([0, 3, 8, 8], [4, 3, 3, 3], "f32")[0], [[0, 3, 8, 8], [4, 3, 3, 3]])),
    ("1x1 convolution", lambda: (NN.convolution([2, 16, 9, 9], [8, 16, 1, 1], "f32")[0], [[2, 16, 9, 9], [8, 16, 1, 1]])),
    ("kernel larger than the image", lambda: (NN.convolution([1, 2, 3, 3], [2, 2, 5, 5], "f32")[0], [[1, 2, 3, 3], [2, 2, 5, 5]])),
    ("convolution without spatial dims", lambda: (NN.convolution([5, 7], [3, 7], "f32", dims="[b, f]x[o, i]->[b, f]")[0], [[5, 7], [3, 7]])),
]


@pytest.mark.parametrize("name,make", EDGES, ids=[e[0] for e in EDGES])
def test_degenerate_windows(rx, client, name, make):
    text, shapes = make()
    args = _args(shapes, "f32", seed=23)
    got, _ = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True)
    assert got[0].a.shape == ref[0].a.shape
    assert np.allclose(got[0].a, ref[0].a, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape,dt,dim,direction,generic", [
    ([2, 3], "f64", 0, "GE", False), ([2, 3], "f64", 1, "LE", False),          # the shapes of test/core/sorting.jl:109-139
    ([4, 3, 2], "f64", 0, "GE", False), ([4, 3, 2], "f64", 1, "GE", True), ([4, 3, 2], "f64", 2, "LE", False),
    ([4096, 1000], "f32", 1, "GE", False), ([4096, 1000], "f32", 0, "LE", True), ([100000], "f32", 0, "GE", False),
    ([64, 50, 30], "bf16", 1, "GT", False), ([300, 70], "i32", 1, "LT", False),
])
def test_argmax_and_argmin(rx, client, shape, dt, dim, direction, generic):
    """The (value, index) reduce of argmax / argmin / findmax (src/Ops.jl:1571-1596), with many ties."""
    text = NN.argreduce(shape, dt, dim, direction, generic=generic)
    rng = np.random.default_rng(31)
    if dt == "i32":
        x = I.Tensor(rng.integers(-3, 4, size=shape).astype(np.int32), dt)
    else:
        x = I.tensor(rng.integers(-8, 9, size=shape) / 4.0, dt)
    got, exe = gpu_run(rx, client, text, [x])
    ref = oracle_run(text, [x])
    assert len(got) == 2
    assert np.array_equal(got[0].a, ref[0].a)
    assert np.array_equal(got[1].a, ref[1].a)
    lib = np.argmax if direction in ("GE", "GT") else np.argmin
    if direction in ("GE", "LE"):
        assert np.array_equal(got[1].a, lib(x.a, axis=dim))


def test_gather_reference_vectors(rx, client):
    """NNlib.gather known answers (test/nn/scatter_gather.jl:5-99)."""
    src = I.tensor(np.array([3, 4, 5, 6, 7]), "f32")
    index = np.array([[1, 2, 3, 4], [4, 2, 1, 3], [3, 5, 5, 3]])
    t = NN.gather([5], [1, 3, 4], [3, 4], "f32", [], [0], [0], 0, [1], one_based=True)
    got, _ = gpu_run(rx, client, t, [src, I.Tensor(index.reshape(1, 3, 4), "i64")])
    assert got[0].a.tolist() == [[3, 4, 5, 6], [6, 4, 3, 5], [5, 7, 7, 5]]
    src2 = I.tensor(np.array([[3, 5, 7], [4, 6, 8]]), "f32")
    index2 = np.array([[1, 2, 3], [2, 2, 1], [3, 1, 3]])
    t = NN.gather([2, 3], [1, 3, 3], [2, 3, 3], "f32", [0], [1], [1], 0, [2, 1], one_based=True)
    got, _ = gpu_run(rx, client, t, [src2, I.Tensor(index2.reshape(1, 3, 3), "i64")])
    assert got[0].a[:, :, 1].tolist() == [[5, 5, 3], [6, 6, 4]] and got[0].a[:, :, 2].tolist() == [[7, 3, 7], [8, 4, 8]]


GATHERS = [
    # operand, start indices, result, dtype, offset_dims, collapsed, start_index_map, index_vector_dim, slice_sizes, batching
    ([7, 5, 6], [1000, 3], [1000, 1], "f32", [1], [0, 1], [0, 1, 2], 1, [1, 1, 1], None),          # x[idx] (gather_getindex)
    ([50000, 64], [32, 128], [32, 128, 64], "bf16", [2], [0], [0], 2, [1, 64], None),               # embedding lookup
    ([50000, 64], [4096], [4096, 64], "f32", [1], [0], [0], 1, [1, 64], None),                      # index vector dim past the end
    ([64, 50000], [1, 3000], [64, 3000], "f32", [0], [1], [1], 0, [64, 1], None),                   # columns (NNlib.gather layout)
    ([4, 2000], [4, 50], [4, 50, 33], "f64", [2], [], [1], 2, [1, 33], ([0], [0])),                 # windows with a batching dim
    ([30, 40], [17, 2], [17, 5, 7], "i32", [1, 2], [], [0, 1], 1, [5, 7], None),                    # 2-d patches
]


@pytest.mark.parametrize("os_,ss,rs,dt,od,cd,sim,ivd,sz,bat", GATHERS)
def test_gather(rx, client, os_, ss,rs, dt, od, cd, sim, ivd, sz, bat):
    kw = {} if bat is None else dict(operand_batching_dims=bat[0], start_indices_batching_dims=bat[1])
    text = NN.gather(os_, ss, rs, dt, od, cd, sim, ivd, sz, idt="i32" if dt == "i32" else "i64", **kw)
    rng = np.random.default_rng(37)
    x = _args([os_], dt, seed=37)[0]
    hi = max(os_)
    idt = "i32" if dt == "i32" else "i64"
    idx = I.Tensor(rng.integers(-3, hi + 3, size=ss).astype(I.NP_OF[idt]), idt)     # some starts out of range: clamped
    got, exe = gpu_run(rx, client, text, [x, idx])
    ref = oracle_run(text, [x, idx])
    assert got[0].a.shape == ref[0].a.shape
    assert np.array_equal(got[0].a, ref[0].a)
    assert [l["kind"] for l in exe.launches()] == ["map"]


def test_convolution_gradient_forms(rx, client):
    """Filter and data gradients of a convolution as the reference builds them
    (ext/ReactantNNlibExt/Implementations.jl:85-251): batch and feature roles swapped, input
    dilation, reversed kernel.  The oracle's values for these forms are pinned against the
    definition of the derivative in tests/test_oracle_windows.py."""
    from test_oracle_windows import _grad_cases, conv_grad_modules
    rng = np.random.default_rng(41)
    cases = _grad_cases() + [dict(W=28, H=28, ci=16, co=32, B=8, kw=3, kh=3, s=(1, 1), p=(1, 1), d=(1, 1)),
                             dict(W=32, H=32, ci=8, co=16, B=4, kw=5, kh=5, s=(2, 2), p=(2, 2), d=(1, 1))]
    for c in cases:
        tf, td, xs, ws, ys = conv_grad_modules(c, "f32")
        x, w, dy = I.tensor(rng.normal(size=xs), "f32"), I.tensor(rng.normal(size=ws), "f32"), I.tensor(rng.normal(size=ys), "f32")
        got, _ = gpu_run(rx, client, tf, [x, dy])
        _close(got[0].a, oracle_run(tf, [x, dy], hifi=True)[0].a, 1e-5 * np.sqrt(ys[0] * ys[1] * ys[3]))
        got, _ = gpu_run(rx, client, td, [dy, w])
        _close(got[0].a, oracle_run(td, [dy, w], hifi=True)[0].a, 1e-5 * np.sqrt(ws[0] * ws[1] * ws[3]))


def test_grouped_filter_gradient(rx, client):
    """`batch_group_count`: the filter gradient of a grouped convolution, one product per group."""
    from test_oracle_windows import grouped_filter_grad_module
    rng = np.random.default_rng(43)
    for groups, c in ((2, dict(W=9, H=8, ci=4, co=6, B=2, kw=3, kh=2, s=(1, 1), p=(1, 0), d=(1, 1))),
                      (4, dict(W=28, H=28, ci=32, co=64, B=8, kw=3, kh=3, s=(1, 1), p=(1, 1), d=(1, 1)))):
        tf, xs, ws, ys = grouped_filter_grad_module(c, groups, "f32")
        x, dy = I.tensor(rng.normal(size=xs), "f32"), I.tensor(rng.normal(size=ys), "f32")
        got, _ = gpu_run(rx, client, tf, [x, dy])
        _close(got[0].a, oracle_run(tf, [x, dy], hifi=True)[0].a, 1e-5 * np.sqrt(ys[0] * ys[1] * ys[3]))


SCATTERS = [
    # operand, indices, updates, dtype, update_window_dims, inserted_window_dims, scatter_dims_to_operand_dims, index_vector_dim, body, batching
    ([600, 700], [5000, 2], [5000], "f32", [], [0, 1], [0, 1], 1, "assign", None),        # setindex! with index pairs
    ([600, 700], [5000, 2], [5000], "f32", [], [0, 1], [0, 1], 1, "add", None),
    ([1000, 64], [4096], [4096, 64], "f32", [1], [0], [0], 1, "add", None),                # gradient of an embedding lookup
    ([1000, 64], [4096], [4096, 64], "f64", [1], [0], [0], 1, "add", None),
    ([50, 40], [300, 1], [300, 40], "i32", [1], [0], [0], 1, "maximum", None),
    ([200], [77, 1], [77, 5], "f32", [1], [], [0], 1, "add", None),                         # windows, some sticking out
    ([8, 300], [8, 60], [8, 60], "i64", [], [1], [1], 2, "add", ([0], [0])),              # a batching dim
    ([300], [1000, 1], [1000], "i8", [], [0], [0], 1, "add", None),
    ([300], [1000, 1], [1000], "f32", [], [0], [0], 1, "minimum", None),
]


@pytest.mark.parametrize("os_,is_,us,dt,uwd,iwd,sdo,ivd,body,bat", SCATTERS)
def test_scatter(rx, client, os_, is_, us, dt, uwd, iwd, sdo, ivd, body, bat):
    kw = {} if bat is None else dict(input_batching_dims=bat[0], scatter_indices_batching_dims=bat[1])
    text = NN.scatter(os_, is_, us, dt, uwd, iwd, sdo, ivd, body=body, **kw)
    rng = np.random.default_rng(47)
    dest = _args([os_], dt, seed=47)[0] if dt[0] == "f" else I.Tensor(rng.integers(-50, 50, size=os_).astype(I.NP_OF[dt]), dt)
    upd = _args([us], dt, seed=48)[0] if dt[0] == "f" else I.Tensor(rng.integers(-3, 4, size=us).astype(I.NP_OF[dt]), dt)
    hi = max(os_)
    idx = rng.integers(-2, hi + 2, size=is_)
    if body == "assign":
        # colliding assignments may leave either value: use distinct in-range targets (plus some out of range)
        flat = rng.permutation(os_[0] * os_[1])[: is_[0]]
        idx = np.stack([flat // os_[1], flat % os_[1]], axis=1)
        idx[::50] = [os_[0] + 3, 0]
    idx = I.Tensor(idx.astype(np.int64), "i64")
    got, exe = gpu_run(rx, client, text, [dest, idx, upd])
    assert [l["kind"] for l in exe.launches()] == ["map", "scatter"]
    ref = oracle_run(text, [dest, idx, upd])
    if dt[0] == "f" and body == "add":
        _close(got[0].a, ref[0].a, 1e-5 if dt == "f32" else 1e-13)
    else:
        assert np.array_equal(got[0].a, ref[0].a)


def _nnlib_scatter_cases():
    import _nnlib_scatter_cases as C
    return [pytest.param(*c[1:], id=c[0]) for c in C.cases()]


@pytest.mark.parametrize("op,dst,src,idx,want", _nnlib_scatter_cases())
def test_scatter_nnlib_reference_vectors(rx, client, op, dst, src, idx, want):
    """NNlib.scatter! / scatter known answers (test/nn/scatter_gather.jl:254-428), all seven operations
    (element - update and element / update included) through the module the reference's lowering builds."""
    text = NN.nnlib_scatter(op, list(dst.shape), list(src.shape), list(idx.shape))
    args = [I.tensor(dst, "f32"), I.Tensor(idx.reshape((1,) + idx.shape), "i64"), I.tensor(src, "f32")]
    got, _ = gpu_run(rx, client, text, args)
    np.testing.assert_allclose(got[0].a, want, rtol=1e-6)
    assert np.array_equal(got[0].a, oracle_run(text, args)[0].a) or op in ("add", "subtract", "multiply", "divide", "mean")


def test_scatter_subtract_divide_large(rx, client):
    """element - update and element / update with many colliding updates, against the oracle."""
    rng = np.random.default_rng(53)
    for body, tol in (("subtract", 1e-5), ("divide", 1e-5)):
        text = NN.scatter([1000, 64], [4096], [4096, 64], "f32", [1], [0], [0], 1, body=body)
        dest = I.tensor(rng.normal(size=(1000, 64)), "f32")
        upd = I.tensor(rng.uniform(0.5, 1.5, size=(4096, 64)), "f32")
        idx = I.Tensor(rng.integers(-2, 1002, size=(4096,)).astype(np.int64), "i64")
        got, exe = gpu_run(rx, client, text, [dest, idx, upd])
        assert [l["kind"] for l in exe.launches()] == ["map", "scatter"]
        _close(got[0].a, oracle_run(text, [dest, idx, upd])[0].a, tol)


SELECT_AND_SCATTER = [
    # x shape, dtype, window, strides, padding, direction
    ([8, 16, 32, 32], "f32", [1, 1, 2, 2], [1, 1, 2, 2], None, "GE"),                               # 2x2 max pooling, VGG
    ([4, 8, 33, 29], "f32", [1, 1, 3, 3], [1, 1, 2, 2], [[0, 0], [0, 0], [1, 1], [1, 1]], "GE"),   # overlapping, padded
    ([2, 4, 20, 20], "f64", [1, 1, 3, 3], [1, 1, 1, 1], None, "GE"),                                # every element in nine windows
    ([3, 5, 40], "f32", [1, 1, 4], [1, 1, 4], None, "GT"),
    ([2, 3, 8, 9, 10], "f32", [1, 1, 2, 2, 2], [1, 1, 2, 2, 2], None, "LE"),                        # 3-d min pooling
    ([64, 64, 56, 56], "f32", [1, 1, 2, 2], [1, 1, 2, 2], None, "GE"),
]


@pytest.mark.parametrize("xs,dt,w,st,pd,direction", SELECT_AND_SCATTER)
def test_select_and_scatter(rx, client, xs, dt, w, st, pd, direction):
    """The gradient of pooling: the window's extreme found by an index reduction over the window view,
    then a scatter-add; against the oracle (itself checked against torch's max_pool2d backward)."""
    text, ss = NN.select_and_scatter(xs, dt, w, st, pd, direction=direction)
    x, dy = _args([xs], dt, seed=61)[0], _args([ss], dt, seed=62)[0]
    got, exe = gpu_run(rx, client, text, [x, dy])
    assert [l["kind"] for l in exe.launches()][-1] == "scatter"
    ref = oracle_run(text, [x, dy])
    _close(got[0].a, ref[0].a, 1e-5 if dt == "f32" else 1e-13)


def test_select_and_scatter_ties(rx, client):
    x = I.tensor(np.ones((2, 3, 8, 8)), "f32")
    dy = _args([[2, 3, 4, 4]], "f32", seed=63)[0]
    for direction in ("GE", "GT", "LE", "LT"):
        text, _ = NN.select_and_scatter([2, 3, 8, 8], "f32", [1, 1, 2, 2], [1, 1, 2, 2], None, direction=direction)
        got, _ = gpu_run(rx, client, text, [x, dy])
        assert np.array_equal(got[0].a, oracle_run(text, [x, dy])[0].a), direction
