"""dot_general against the f64-accumulating oracle.  On the MFMA skeletons: every operand order,
element type and the batched form, at shapes chosen so that the MFMA path is taken (the plan's
launch kind is asserted), including tile edges.  With a vector-like operand (matrix-vector,
inner products, a few right-hand sides): the multiply + reduce form, every layout."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run, max_rel_to_scale, contraction_err, dot_bound
from oracle import stablehlo_interp as I

pytestmark = pytest.mark.gpu


def cw_tol(dt, out_dt):
    """Bound on |got - ref|_ij / (|A| . |B|)_ij, the componentwise error of a contraction accumulated in f32 (f64 for f64
    operands): the rounding of the result type for 16-bit results (half an ulp of bf16 is 2^-9, of f16 2^-12, relative to
    the entry, which is at most the bound), the accumulation for wider ones.  All are below the 1e-2 (16- and 8-bit
    operands) and 1e-5 sqrt(K) (f32) the specification of this backend allows."""
    if out_dt == "bf16":
        return 4e-3
    if out_dt == "f16":
        return 1e-3
    if dt == "f64":
        return 1e-14
    return 1e-4 if dt.startswith("f8") else 1e-6


def _tt(shape, dt):
    return "tensor<" + "x".join([str(s) for s in shape] + [dt]) + ">"


def dot_module(M, N, K, dt, out_dt, a_kc, b_kc, batch=0):
    bs = [batch] if batch else []
    a_shape = bs + ([M, K] if a_kc else [K, M])
    b_shape = bs + ([N, K] if b_kc else [K, N])
    nb = len(bs)
    lc = nb + (1 if a_kc else 0)
    rc = nb + (1 if b_kc else 0)
    battr = "batching_dims = [0] x [0], " if batch else ""
    ta, tb, to = _tt(a_shape, dt), _tt(b_shape, dt), _tt(bs + [M, N], out_dt)
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%0 = stablehlo.dot_general %%arg0, %%arg1, %scontracting_dims = [%d] x [%d], "
            "precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s\n    return %%0 : %s\n  }\n}\n"
            % (ta, tb, to, battr, lc, rc, ta, tb, to, to)), a_shape, b_shape


CASES = []
for a_kc in (True, False):
    for b_kc in (True, False):
        CASES += [("f32", "f32", 128, 128, 64, a_kc, b_kc, 0), ("f32", "f32", 200, 136, 48, a_kc, b_kc, 0),
                  ("bf16", "bf16", 128, 256, 128, a_kc, b_kc, 0), ("bf16", "f32", 136, 200, 64, a_kc, b_kc, 0),
                  ("f16", "f16", 128, 128, 64, a_kc, b_kc, 0),
                  ("f8E4M3FN", "f32", 128, 128, 256, a_kc, b_kc, 0), ("f8E4M3FN", "f32", 144, 208, 128, a_kc, b_kc, 0)]
# contracted dimension that is not a multiple of the K step (tail zero-filled), any operand order
for a_kc in (True, False):
    for b_kc in (True, False):
        CASES += [("f32", "f32", 200, 136, 52, a_kc, b_kc, 0), ("bf16", "f32", 136, 200, 72, a_kc, b_kc, 0),
                  ("f8E4M3FN", "f32", 144, 208, 176, a_kc, b_kc, 0)]
# f64 on v_mfma_f64_16x16x4_f64: every operand order, tile edges, a K tail, batched
for a_kc in (True, False):
    for b_kc in (True, False):
        CASES += [("f64", "f64", 128, 128, 64, a_kc, b_kc, 0), ("f64", "f64", 200, 136, 50, a_kc, b_kc, 0),
                  ("f64", "f64", 72, 64, 16, a_kc, b_kc, 3)]
CASES += [("f64", "f64", 512, 384, 256, True, False, 0), ("f64", "f64", 1000, 1000, 300, True, True, 0)]
CASES += [("f32", "f32", 96, 128, 37, False, False, 0), ("bf16", "bf16", 128, 136, 1000, True, False, 0),
          ("f32", "f32", 1000, 1000, 1000, True, False, 0), ("f32", "f32", 128, 128, 8, True, True, 0)]
CASES += [("f32", "f32", 128, 128, 32, True, False, 3), ("bf16", "bf16", 128, 128, 64, True, True, 2),
          ("f8E4M3FN", "f32", 128, 128, 128, True, True, 2), ("bf16", "bf16", 256, 384, 512, True, False, 0)]


# dimensions that are not whole 16-byte vectors: operands are zero-padded, the product sliced
CASES += [("f32", "f32", 301, 1001, 999, True, True, 0), ("f32", "f32", 301, 1001, 999, False, False, 0),
          ("bf16", "bf16", 256, 100, 512, True, False, 0), ("bf16", "f32", 250, 130, 777, False, True, 0),
          ("f64", "f64", 129, 131, 1027, True, False, 0), ("f32", "f32", 130, 66, 150, True, False, 5)]


@pytest.mark.parametrize("dt,out_dt,M,N,K,a_kc,b_kc,batch", CASES)
def test_dot_general_mfma(rx, client, dt, out_dt, M, N, K, a_kc, b_kc, batch):
    text, a_shape, b_shape = dot_module(M, N, K, dt, out_dt, a_kc, b_kc, batch)
    a = I.tensor(np.random.default_rng(0).normal(size=a_shape), dt)
    b = I.tensor(np.random.default_rng(1).normal(size=b_shape), dt)
    got, exe = gpu_run(rx, client, text, [a, b])
    kinds = [l["kind"] for l in exe.launches() if l["kind"] != "map"]     # maps: the padding copies and the final slice
    assert kinds == ["gemm_" + {"f32": "f32", "bf16": "bf16", "f16": "f16", "f8E4M3FN": "f8", "f64": "f64"}[dt]], kinds
    ref = oracle_run(text, [a, b], hifi=True)
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, [a, b])) <= cw_tol(dt, out_dt)
    err = max_rel_to_scale(got[0].a, ref[0].a)     # second figure: the error against the largest entry
    if out_dt in ("bf16", "f16"):
        assert err <= 1e-2
    elif out_dt == "f64":
        assert err <= 1e-14 * np.sqrt(K)
    else:
        assert err <= 1e-5 * np.sqrt(K)


STREAM_CASES = [
    # dt, out, M, N, K, a_kc, b_kc, batch: 256 or more eight-wavefront tiles, ragged last tiles, one to five K tiles of 128 bytes
    ("f8E4M3FN", "f32", 4000, 4112, 128, True, True, 0),
    ("f8E4M3FN", "bf16", 4000, 4112, 256, True, False, 0),
    ("f8E4M3FN", "f32", 4000, 4112, 384, False, False, 0),
    ("f8E4M3FN", "bf16", 4016, 4100, 640, False, True, 0),
    ("f8E4M3FN", "f32", 2048, 2064, 512, True, True, 4),
    ("f8E4M3FN", "bf16", 2040, 2064, 256, True, False, 5),
    ("f8E4M3FN", "bf16", 4000, 4112, 512, True, True, 0),
    ("f8E4M3FN", "f32", 4016, 4100, 256, False, True, 0),
    ("bf16", "bf16", 4000, 4104, 64, True, False, 0),
    ("bf16", "f32", 4000, 4104, 128, True, True, 0),
    ("bf16", "bf16", 4000, 4104, 192, False, False, 0),
    ("f16", "f16", 4008, 4100, 320, False, True, 0),
    ("f16", "f32", 2040, 2056, 256, True, False, 5),
    # an even number of K tiles on 256x256 tiles: 16-bit operands take the ping-pong form, in every operand order
    ("bf16", "bf16", 4000, 4104, 256, True, False, 0),
    ("bf16", "f32", 4000, 4104, 384, False, False, 0),
    ("f16", "f16", 4008, 4100, 768, False, True, 0),
    ("bf16", "bf16", 2040, 2056, 128, False, True, 5),
    # 256x128 tiles (the tall products whose 256x256 tiles would not fill the chip)
    ("bf16", "bf16", 8000, 1032, 192, True, False, 0),
    ("bf16", "f32", 8000, 1028, 128, True, True, 0),
    ("f16", "f16", 8000, 1032, 64, False, False, 0),
    ("bf16", "bf16", 8000, 1028, 320, False, True, 0),
]


@pytest.mark.parametrize("dt,out_dt,M,N,K,a_kc,b_kc,batch", STREAM_CASES)
def test_streaming_skeleton(rx, client, dt, out_dt, M, N, K, a_kc, b_kc, batch):
    """8- and 16-bit operands on the eight-wavefront tiles take the skeleton that streams one operand through the 16x16
    MFMA shapes, or its ping-pong form: every operand order, batched, rows past the end of an operand (read as zero by the
    buffer loads), odd and even tile counts along K."""
    text, a_shape, b_shape = dot_module(M, N, K, dt, out_dt, a_kc, b_kc, batch)
    # 256x256 tiles with an even number of K tiles: the ping-pong form of the same tiles (8-bit operands: when B is [n][k])
    pingpong = N > 2000 and (K * (1 if dt == "f8E4M3FN" else 2) // 128) % 2 == 0 and (dt != "f8E4M3FN" or b_kc)
    assert ("rx_gemm_body_pp<" if pingpong else "rx_gemm_body_s<") in rx.compile_offline(text, with_source=True)
    a = I.tensor(np.random.default_rng(5).normal(size=a_shape), dt)
    b = I.tensor(np.random.default_rng(6).normal(size=b_shape), dt)
    got, exe = gpu_run(rx, client, text, [a, b])
    assert [l["kind"] for l in exe.launches()] == ["gemm_" + {"bf16": "bf16", "f16": "f16", "f8E4M3FN": "f8"}[dt]], exe.report()
    ref = oracle_run(text, [a, b], hifi=True)
    assert got[0].a.shape == ref[0].a.shape
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, [a, b])) <= cw_tol(dt, out_dt)
    assert max_rel_to_scale(got[0].a, ref[0].a) <= (1e-2 if out_dt in ("bf16", "f16") else 1e-5 * np.sqrt(K))


@pytest.mark.parametrize("dt,M,N,K", [("bf16", 4000, 4104, 256), ("f16", 8000, 1032, 192)])
def test_bias_as_the_accumulators_first_values(rx, client, monkeypatch, dt, M, N, K):
    """relu(x W + b) on the streaming skeletons, ragged last tiles in both directions: the bias is the accumulators' first
    values (the epilogue functor's `init`), which must give what adding it in the epilogue gives, up to the order of the
    float32 additions, and what the oracle gives."""
    t = lambda s: "tensor<" + "x".join(str(v) for v in s) + "x" + dt + ">"
    text = ("module {\n  func.func @main(%%x: %s, %%w: %s, %%b: %s) -> %s {\n"
            "    %%0 = stablehlo.dot_general %%x, %%w, contracting_dims = [1] x [0] : (%s, %s) -> %s\n"
            "    %%1 = stablehlo.broadcast_in_dim %%b, dims = [1] : (%s) -> %s\n    %%2 = stablehlo.add %%0, %%1 : %s\n"
            "    %%z = stablehlo.constant dense<0.000000e+00> : %s\n    %%3 = stablehlo.maximum %%2, %%z : %s\n    return %%3 : %s\n  }\n}\n"
            % (t([M, K]), t([K, N]), t([N]), t([M, N]), t([M, K]), t([K, N]), t([M, N]), t([N]), t([M, N]), t([M, N]), t([M, N]), t([M, N]), t([M, N])))
    rng = np.random.default_rng(9)
    args = [I.tensor(rng.normal(size=(M, K)), dt), I.tensor(rng.normal(size=(K, N)) / np.sqrt(K), dt), I.tensor(rng.normal(size=(N,)) * 3.0, dt)]
    src = rx.compile_offline(text, with_source=True)
    assert "has_init = true" in src and "void init(float (&v)[NV], int n)" in src
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["gemm_" + dt]
    monkeypatch.setenv("RX_EPILOGUE_INIT", "0")
    assert "has_init" not in rx.compile_offline(text, with_source=True)
    plain, _ = gpu_run(rx, client, text, args)
    ref = oracle_run(text, args, hifi=True)
    tol = 1e-2 if dt == "bf16" else 2e-3
    assert max_rel_to_scale(got[0].a, ref[0].a) <= tol and max_rel_to_scale(plain[0].a, ref[0].a) <= tol
    # the two forms differ by float32 rounding of the sums only: at most an ulp of the narrow result here and there
    g, p = got[0].a.astype(np.float64), plain[0].a.astype(np.float64)
    assert np.mean(g != p) < 0.02 and np.max(np.abs(g - p)) <= (2.0 ** -7 if dt == "bf16" else 2.0 ** -10) * np.abs(p).max()


def test_int_dot_general_reference_vectors(rx, client):
    """Known answers of the reference's own test (test/core/ops.jl:249-278)."""
    t = ("module {\n  func.func @main(%arg0: tensor<4xi32>, %arg1: tensor<4xi32>) -> tensor<i32> {\n"
         "    %0 = stablehlo.dot_general %arg0, %arg1, contracting_dims = [0] x [0] : (tensor<4xi32>, tensor<4xi32>) -> tensor<i32>\n"
         "    return %0 : tensor<i32>\n  }\n}\n")
    a = I.Tensor(np.array([1, 2, 3, 4], dtype=np.int32), "i32")
    b = I.Tensor(np.array([5, 6, -7, -8], dtype=np.int32), "i32")
    got, _ = gpu_run(rx, client, t, [a, b])
    assert int(got[0].a) == -36
    # Int32[1 2; 3 4]' * Int32[5 6; -7 -8] == [-16 -18; -18 -20]; Julia matrices arrive transposed
    t2 = ("module {\n  func.func @main(%arg0: tensor<2x2xi32>, %arg1: tensor<2x2xi32>) -> tensor<2x2xi32> {\n"
          "    %0 = stablehlo.dot_general %arg0, %arg1, contracting_dims = [1] x [1] : (tensor<2x2xi32>, tensor<2x2xi32>) -> tensor<2x2xi32>\n"
          "    return %0 : tensor<2x2xi32>\n  }\n}\n")
    A = np.array([[1, 2], [3, 4]], dtype=np.int32)
    B = np.array([[5, 6], [-7, -8]], dtype=np.int32)
    # Julia f1(x, y) contracts dim 1 of both: result[i, j] = sum_k A[k, i] * B[k, j]; raw buffers are A.T, B.T
    # and raw dim 1 is Julia dim 1.
    got, _ = gpu_run(rx, client, t2, [I.Tensor(A.T.copy(), "i32"), I.Tensor(B.T.copy(), "i32")])
    assert np.array_equal(got[0].a, A.T @ B)
    assert np.array_equal(A.T @ B, np.array([[-16, -18], [-18, -20]]))


def _dot_text(ls, rs, os_, attrs, dt, out_dt=None):
    lt, rt, ot = _tt(ls, dt), _tt(rs, dt), _tt(os_, out_dt or dt)
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%0 = stablehlo.dot_general %%arg0, %%arg1, %s : (%s, %s) -> %s\n    return %%0 : %s\n  }\n}\n"
            % (lt, rt, ot, attrs, lt, rt, ot, ot))


# products with a vector-like operand run as multiply + reduce: (lhs, rhs, out, attributes, type, kinds)
VECTOR_CASES = [
    ((300, 1000), (1000,), (300,), "contracting_dims = [1] x [0]", "f32", ["row"]),
    ((1000, 300), (1000,), (300,), "contracting_dims = [0] x [0]", "f32", ["reduce_generic"]),
    ((1000,), (1000, 300), (300,), "contracting_dims = [0] x [0]", "f32", ["reduce_generic"]),
    ((1000,), (300, 1000), (300,), "contracting_dims = [0] x [1]", "f32", ["row"]),
    ((100003,), (100003,), (), "contracting_dims = [0] x [0]", "f32", ["reduce", "reduce_final"]),
    ((100003,), (100003,), (), "contracting_dims = [0] x [0]", "f64", ["reduce", "reduce_final"]),
    ((100003,), (100003,), (), "contracting_dims = [0] x [0]", "i32", ["reduce", "reduce_final"]),
    ((130, 70), (130, 70), (), "contracting_dims = [0, 1] x [0, 1]", "f64", ["reduce", "reduce_final"]),
    ((130, 70), (70, 130), (), "contracting_dims = [0, 1] x [1, 0]", "f32", ["reduce", "reduce_final"]),
    ((256, 520), (520, 3), (256, 3), "contracting_dims = [1] x [0]", "f32", ["row"]),
    ((256, 520), (3, 520), (256, 3), "contracting_dims = [1] x [1]", "bf16", ["row", "map"]),
    ((3, 520), (256, 520), (3, 256), "contracting_dims = [1] x [1]", "f32", ["row", "map"]),
    ((2, 520), (520, 256), (2, 256), "contracting_dims = [1] x [0]", "f16", None),
    ((520, 256), (520, 5), (256, 5), "contracting_dims = [0] x [0]", "f32", ["reduce_generic"]),
    ((6, 200, 300), (6, 300), (6, 200), "batching_dims = [0] x [0], contracting_dims = [2] x [1]", "f32", ["row"]),
    ((6, 300, 200), (6, 300), (6, 200), "batching_dims = [0] x [0], contracting_dims = [1] x [1]", "f32", ["reduce_generic"]),
    ((6, 300), (6, 200, 300), (6, 200), "batching_dims = [0] x [0], contracting_dims = [1] x [2]", "bf16", ["row", "map"]),
    ((200, 6, 300), (300, 6), (6, 200), "batching_dims = [1] x [1], contracting_dims = [2] x [0]", "f32", None),
    ((300, 700), (700,), (300,), "contracting_dims = [1] x [0]", "i32", ["row"]),
    ((300, 700), (700,), (300,), "contracting_dims = [1] x [0]", "f8E4M3FN", None),
    # four rows times a wide matrix (a dense layer on a batch of four): 4 x 4 blocks of the result per thread
    ((4, 1003), (1003, 2048), (4, 2048), "contracting_dims = [1] x [0]", "f32", ["reduce_generic"]),
    ((4, 4100), (4100, 1024), (4, 1024), "contracting_dims = [1] x [0]", "i32", ["reduce_generic"]),
]


@pytest.mark.parametrize("ls,rs,os_,attrs,dt,kinds", VECTOR_CASES)
def test_dot_general_with_a_vector_like_operand(rx, client, ls, rs, os_, attrs, dt, kinds):
    out_dt = "f32" if dt == "f8E4M3FN" else dt
    text = _dot_text(list(ls), list(rs), list(os_), attrs, dt, out_dt)
    rng = np.random.default_rng(5)
    if dt == "i32":
        a = I.Tensor(rng.integers(-2**20, 2**20, size=ls).astype(np.int32), dt)
        b = I.Tensor(rng.integers(-2**20, 2**20, size=rs).astype(np.int32), dt)
    else:
        a = I.tensor(rng.normal(size=ls), dt)
        b = I.tensor(rng.normal(size=rs), dt)
    got, exe = gpu_run(rx, client, text, [a, b])
    got_kinds = [l["kind"] for l in exe.launches()]
    assert "dot_scalar" not in got_kinds and not any(k.startswith("gemm") for k in got_kinds), got_kinds
    if kinds is not None:
        assert got_kinds[0] == kinds[0], got_kinds
    ref = oracle_run(text, [a, b], hifi=True)
    assert got[0].a.shape == ref[0].a.shape
    if dt == "i32":
        assert np.array_equal(got[0].a, ref[0].a)
        return
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, [a, b])) <= cw_tol(dt, out_dt)
    err = max_rel_to_scale(got[0].a, ref[0].a)
    if out_dt in ("bf16", "f16"):
        assert err <= 1e-2
    elif dt == "f64":
        assert err <= 1e-12
    else:
        assert err <= 1e-5 * np.sqrt(100003 if not os_ else 1000)


def test_four_rows_times_a_wide_matrix_plan():
    """x[4][k] w[k][n] as a reduction over k with the result as [n][4]: a thread owns four n and the four rows, and reads
    w sixteen bytes at a time for eight k ahead of the arithmetic (RX_REDUCE_ROW_BLOCKS=0: one n per thread)."""
    from _loader import load_pkg
    rep = load_pkg().compile_offline(_dot_text([4, 1003], [1003, 2048], [4, 2048], "contracting_dims = [1] x [0]", "f32"), with_source=True)
    assert "threadIdx.x) * 16;" in rep and "float wq[32];" in rep and "for (; r0s + 8 <= r0_end; r0s += 8)" in rep, rep


def test_short_contractions_keep_the_scalar_loop(rx, client):
    text = _dot_text([4096, 16], [16], [4096], "contracting_dims = [1] x [0]", "f32")
    a = I.tensor(np.random.default_rng(0).normal(size=(4096, 16)), "f32")
    b = I.tensor(np.random.default_rng(1).normal(size=(16,)), "f32")
    got, exe = gpu_run(rx, client, text, [a, b])
    assert [l["kind"] for l in exe.launches()] == ["dot_scalar"]
    ref = oracle_run(text, [a, b], hifi=True)
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, [a, b])) <= cw_tol("f32", "f32")
    assert max_rel_to_scale(got[0].a, ref[0].a) <= 1e-5


@pytest.mark.parametrize("dt", ["f32", "bf16"])
def test_operand_evaluated_inside_the_product_with_an_epilogue(rx, client, dt):
    """A dot operand that expands smaller data (here a broadcast vector, scaled) is a functor of the
    GEMM, on either side, next to an epilogue with an operand of its own."""
    M, K, N = 64, 256, 4096
    tA, tw, tB, tC, ts = _tt([M, K], dt), _tt([K], dt), _tt([K, N], dt), _tt([M, N], dt), _tt([N], dt)
    text = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg2: %s, %%arg3: %s) -> %s {\n"
            "    %%wb = stablehlo.broadcast_in_dim %%arg1, dims = [0] : (%s) -> %s\n"
            "    %%sb = stablehlo.broadcast_in_dim %%arg3, dims = [1] : (%s) -> %s\n"
            "    %%b = stablehlo.multiply %%wb, %%sb : %s\n"
            "    %%0 = stablehlo.dot_general %%arg0, %%b, contracting_dims = [1] x [0] : (%s, %s) -> %s\n"
            "    %%1 = stablehlo.add %%0, %%arg2 : %s\n"
            "    %%z = stablehlo.constant dense<0.000000e+00> : %s\n"
            "    %%2 = stablehlo.maximum %%1, %%z : %s\n"
            "    return %%2 : %s\n  }\n}\n" % (tA, tw, tC, ts, tC, tw, tB, ts, tB, tB, tA, tB, tC, tC, tC, tC, tC))
    rng = np.random.default_rng(3)
    args = [I.tensor(rng.normal(size=(M, K)), dt), I.tensor(rng.normal(size=(K,)), dt), I.tensor(rng.normal(size=(M, N)), dt),
            I.tensor(rng.uniform(0.5, 1.5, size=(N,)), dt)]
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["gemm_" + dt], exe.report()
    ref = oracle_run(text, args, hifi=True, excess=(dt == "bf16"))
    # on magnitudes the module is |A| . (|w| |s|) + |C| (the maximum with zero changes nothing): the bound with the epilogue's term;
    # the expanded operand is rounded to bf16 before the product, which doubles the allowance
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, args)) <= (2 if dt == "bf16" else 1) * cw_tol(dt, dt)
    assert max_rel_to_scale(got[0].a, ref[0].a) <= (2e-2 if dt == "bf16" else 1e-5 * np.sqrt(K))
    # the same product transposed: the expanded operand is now the left one
    text2 = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s, %%arg3: %s) -> %s {\n"
             "    %%wb = stablehlo.broadcast_in_dim %%arg1, dims = [0] : (%s) -> %s\n"
             "    %%sb = stablehlo.broadcast_in_dim %%arg3, dims = [1] : (%s) -> %s\n"
             "    %%b = stablehlo.multiply %%wb, %%sb : %s\n"
             "    %%0 = stablehlo.dot_general %%b, %%arg0, contracting_dims = [0] x [1] : (%s, %s) -> %s\n"
             "    return %%0 : %s\n  }\n}\n" % (tA, tw, ts, _tt([N, M], dt), tw, tB, ts, tB, tB, tB, tA, _tt([N, M], dt), _tt([N, M], dt)))
    args2 = [args[0], args[1], args[3]]
    got, exe = gpu_run(rx, client, text2, args2)
    assert [l["kind"] for l in exe.launches()] == ["gemm_" + dt], exe.report()
    ref = oracle_run(text2, args2, hifi=True, excess=(dt == "bf16"))
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text2, args2)) <= (2 if dt == "bf16" else 1) * cw_tol(dt, dt)
    assert max_rel_to_scale(got[0].a, ref[0].a) <= (2e-2 if dt == "bf16" else 1e-5 * np.sqrt(K))


GENERAL_DOTS = [
    # lhs, rhs, out, attributes, dtype: forms that are reshaped (and where needed transposed) into batched matrix products
    ([64, 96, 12], [96, 80, 12], [12, 64, 80], "batching_dims = [2] x [2], contracting_dims = [1] x [0]", "f32"),       # NNlib.batched_mul layout
    ([3, 4, 64, 96], [3, 4, 96, 80], [3, 4, 64, 80], "batching_dims = [0, 1] x [0, 1], contracting_dims = [3] x [2]", "bf16"),
    ([128, 8, 16], [8, 16, 192], [128, 192], "contracting_dims = [1, 2] x [0, 1]", "f32"),
    ([16, 8, 128], [128, 12, 16], [16, 8, 12, 16], "contracting_dims = [2] x [0]", "f32"),
    ([128, 8, 16], [16, 8, 192], [128, 192], "contracting_dims = [1, 2] x [1, 0]", "f64"),
    ([5, 64, 7, 32], [32, 5, 96], [5, 64, 7, 96], "batching_dims = [0] x [1], contracting_dims = [3] x [0]", "f32"),
]


@pytest.mark.parametrize("ls,rs,os_,attrs,dt", GENERAL_DOTS)
def test_dot_general_with_grouped_or_permuted_dims(rx, client, ls, rs, os_, attrs, dt):
    text = _dot_text(ls, rs, os_, attrs, dt)
    rng = np.random.default_rng(11)
    a, b = I.tensor(rng.normal(size=ls), dt), I.tensor(rng.normal(size=rs), dt)
    got, exe = gpu_run(rx, client, text, [a, b])
    kinds = [l["kind"] for l in exe.launches()]
    assert any(k.startswith("gemm_") for k in kinds) and "dot_scalar" not in kinds, kinds
    ref = oracle_run(text, [a, b], hifi=True)
    assert got[0].a.shape == ref[0].a.shape
    assert contraction_err(got[0].a, ref[0].a, dot_bound(text, [a, b])) <= cw_tol(dt, dt)
    err = max_rel_to_scale(got[0].a, ref[0].a)
    assert err <= {"bf16": 1e-2, "f64": 1e-13, "f32": 1e-4}[dt]


SPLIT_CASES = [
    # dt, out, M, N, K, a_kc, b_kc, slices
    ("f32", "f32", 256, 256, 2048, True, False, 8),
    ("f32", "f32", 128, 192, 8192, False, True, 16),
    ("f32", "f32", 256, 2048, 4096, True, True, 2),
    ("bf16", "bf16", 128, 128, 16384, True, False, 16),
    ("bf16", "f32", 320, 192, 4096, False, False, 16),
    ("f16", "f16", 64, 512, 4096, True, True, 16),
    ("f8E4M3FN", "f32", 256, 128, 8192, True, True, 16),
    ("f8E4M3FN", "bf16", 128, 128, 4096, False, True, 16),
]


@pytest.mark.parametrize("dt,out_dt,M,N,K,a_kc,b_kc,slices", SPLIT_CASES)
def test_long_contractions_with_few_output_tiles_are_cut_along_k(rx, client, monkeypatch, dt, out_dt, M, N, K, a_kc, b_kc, slices):
    """Few 64x64 output tiles and a long K: partial products of K slices in f32 ([S, M, N]), then a
    reduction over the slices (and the rounding to the result type)."""
    text, a_shape, b_shape = dot_module(M, N, K, dt, out_dt, a_kc, b_kc)
    a = I.tensor(np.random.default_rng(0).normal(size=a_shape), dt)
    b = I.tensor(np.random.default_rng(1).normal(size=b_shape), dt)
    got, exe = gpu_run(rx, client, text, [a, b])
    L = exe.launches()
    assert [l["kind"] for l in L][:2] == ["gemm_" + {"f32": "f32", "bf16": "bf16", "f16": "f16", "f8E4M3FN": "f8"}[dt], "reduce_generic"], L
    import re
    assert int(re.search(r"kind=gemm_\w+ grid=\d+x(\d+)x1", exe.report()).group(1)) in (slices // 4, slices // 2, slices, 2 * slices)
    ref = oracle_run(text, [a, b], hifi=True)
    bound = dot_bound(text, [a, b])
    assert contraction_err(got[0].a, ref[0].a, bound) <= cw_tol(dt, out_dt)
    err = max_rel_to_scale(got[0].a, ref[0].a)
    assert err <= (1e-2 if out_dt in ("bf16", "f16") else 1e-5 * np.sqrt(K))
    monkeypatch.setenv("RX_SPLIT_K", "0")
    whole, exe1 = gpu_run(rx, client, text, [a, b])
    assert len(exe1.launches()) == 1
    assert contraction_err(whole[0].a, ref[0].a, bound) <= cw_tol(dt, out_dt)
    assert max_rel_to_scale(whole[0].a, ref[0].a) <= (1e-2 if out_dt in ("bf16", "f16") else 1e-5 * np.sqrt(K))


def test_a_root_fed_by_several_products(rx, client):
    """(A*B + C*D) .* (E'*F'): one product joins the elementwise root's kernel, the others run on their own
    and are read back (syr2k of the reference's polybench suite is the two-product case)."""
    t = _tt([256, 256], "f32")
    text = ("module {\n func.func @main(%a: T, %b: T, %c: T, %d: T, %e: T, %f: T) -> T {\n"
            "  %0 = stablehlo.dot_general %a, %b, contracting_dims = [1] x [0] : (T, T) -> T\n"
            "  %1 = stablehlo.dot_general %c, %d, contracting_dims = [1] x [0] : (T, T) -> T\n"
            "  %2 = stablehlo.dot_general %e, %f, contracting_dims = [0] x [1] : (T, T) -> T\n"
            "  %3 = stablehlo.add %0, %1 : T\n  %4 = stablehlo.multiply %3, %2 : T\n  return %4 : T\n }\n}\n").replace("T", t)
    rng = np.random.default_rng(0)
    args = [I.tensor(rng.normal(size=(256, 256)), "f32") for _ in range(6)]
    got, exe = gpu_run(rx, client, text, args)
    assert [l["kind"] for l in exe.launches()] == ["gemm_f32"] * 3
    ref = oracle_run(text, args, hifi=True)[0].a
    # on magnitudes the module is (|A||B| + |C||D|) (|E||F|): the first-order bound of the product of the two factors' errors
    assert contraction_err(got[0].a, ref, dot_bound(text, args)) <= 2 * cw_tol("f32", "f32")
    assert max_rel_to_scale(got[0].a, ref) <= 1e-5 * 16
