"""The five benchmark configs at their full sizes on the GPU.

The numpy interpreter is too slow for these shapes, so each config is checked the way its
structure allows: the stencil bit for bit against the oracle's C restatement (which the CPU
tests pin to the interpreter); the reduction and the f32 GEMM against float64 numpy; the MLP and
the FP8 linear layer, whose rows are independent, on a sample of rows recomputed by the
interpreter with the same weights (plus the row invariants of softmax and RMSNorm on every row)."""
import numpy as np
import pytest

from _harness import gpu_run, oracle_run, max_rel_to_scale, contraction_err
from _loader import load_programs
from oracle import stablehlo_interp as I
from oracle import lowfloat as lf

pytestmark = pytest.mark.gpu
P = load_programs()


def _upload(rx, client, raw, dt):
    return rx.Buffer.from_host(client, raw, dt)


def _download(buf):
    return buf.synced_buffer().to_host()


def test_sinsum_add_2_pow_26(rx, client):
    n = 1 << 26
    x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
    exe = rx.xla_compile(client, P.sinsum_add(n))
    out = exe.execute_sharded([_upload(rx, client, x, "f32"), _upload(rx, client, y, "f32")])
    got = float(_download(out[0]))
    terms = np.sin(x.astype(np.float64)) + y.astype(np.float64)
    exact, scale = float(terms.sum()), float(np.abs(terms).sum())
    # fp32 reduction: 1e-5 * sqrt(n) relative to the mean magnitude of the summands
    assert abs(got - exact) <= 1e-5 * np.sqrt(n) * scale / n


def test_stencil_512x512x256_ten_steps_bit_exact(rx, client):
    from oracle import build_c
    lib = build_c.load()
    nx, ny, nz, H = 512, 512, 256, 3
    full = (nz + 2 * H, ny + 2 * H, nx + 2 * H)
    c = np.zeros(full)
    c[H:-H, H:-H, H:-H] = np.random.default_rng(0).random((nz, ny, nx))
    u = 2.0 * np.random.default_rng(1).random(full) - 1.0
    v = np.ascontiguousarray(u[::-1])
    w = 0.5 * (u - v)
    exe = rx.xla_compile(client, P.stencil(nx, ny, nz, steps=10))
    assert [l["kind"] for l in exe.launches()] == ["map_stencil_lds2"] * 5
    out = exe.execute_sharded([_upload(rx, client, a, "f64") for a in (c, u, v, w)])
    got = _download(out[0])
    want = build_c.stencil_steps(lib, c, u, v, w, nx, ny, nz, 10)
    assert got.shape == want.shape and np.array_equal(got, want)
    assert not np.any(got[:H]) and not np.any(got[:, :H]) and not np.any(got[:, :, -H:])   # halos stay zero


def test_gemm_4096_f32_alpha_beta(rx, client):
    n = 4096
    A, B, C = [np.random.default_rng(s).normal(size=(n, n)).astype(np.float32) for s in (0, 1, 2)]
    exe = rx.xla_compile(client, P.gemm(n, n, n))
    out = exe.execute_sharded([_upload(rx, client, a, "f32") for a in (A, B, C)])
    got = _download(out[0])
    # buffers are the Julia arrays with dims reversed: C_raw = alpha * B_raw @ A_raw + beta * C_raw
    want = 1.5 * (B.astype(np.float64) @ A.astype(np.float64)) + 1.2 * C.astype(np.float64)
    bound = 1.5 * (np.abs(B).astype(np.float64) @ np.abs(A).astype(np.float64)) + 1.2 * np.abs(C).astype(np.float64)
    assert contraction_err(got, want, bound) <= 1e-6                       # entry by entry against 1.5 |B| |A| + 1.2 |C|
    assert max_rel_to_scale(got, want) <= 1e-5


def _bf16(a):
    return lf.f32_to_bf16_bits(np.asarray(a, dtype=np.float32))


def test_mlp_8192_rows_sampled(rx, client):
    batch, widths, rows = 8192, (1024, 4096, 4096, 1024), 48
    rng = np.random.default_rng(0)
    raw = [_bf16(rng.normal(size=(batch, widths[0])))]
    for l in range(3):
        lim = np.sqrt(6.0 / (widths[l] + widths[l + 1]))
        raw.append(_bf16(np.random.default_rng(1 + l).uniform(-lim, lim, size=(widths[l], widths[l + 1]))))
        raw.append(_bf16(np.random.default_rng(4 + l).normal(size=(widths[l + 1],)) * 0.01))
    exe = rx.xla_compile(client, P.mlp(batch, widths))
    out = exe.execute_sharded([_upload(rx, client, a, "bf16") for a in raw])
    got = lf.bf16_bits_to_f32(_download(out[0])).reshape(batch, widths[-1])
    assert np.allclose(got.sum(axis=1), 1.0, atol=2e-2)                    # every softmax row sums to one
    pick = np.linspace(0, batch - 1, rows).astype(int)                     # rows are independent: recompute a sample
    args = [I.Tensor.from_bytes(raw[0][pick].tobytes(), "bf16", (rows, widths[0]))]
    args += [I.Tensor.from_bytes(a.tobytes(), "bf16", a.shape) for a in raw[1:]]
    ref = oracle_run(P.mlp(rows, widths), args, hifi=True, excess=True)
    assert max_rel_to_scale(got[pick], ref[0].a) <= 2e-2


@pytest.mark.parametrize("k,n", [(1024, 4096), (4096, 4096), (4096, 1024)])
def test_mlp_layers_8192_componentwise(rx, client, k, n):
    """Each dense layer of the MLP at its full size (the three GEMM shapes with their bias + gelu epilogue) on its own:
    |got - ref|_ij <= 1e-2 (|x| . |W| + |b|)_ij on a sample of rows, the bound that the 2e-2 allowance of the whole
    three-layer network rests on."""
    batch, rows = 8192, 64
    x = _bf16(np.random.default_rng(0).normal(size=(batch, k)))
    lim = np.sqrt(6.0 / (k + n))
    w = _bf16(np.random.default_rng(1).uniform(-lim, lim, size=(k, n)))
    b = _bf16(np.random.default_rng(2).normal(size=(n,)) * 0.01)
    exe = rx.xla_compile(client, P.mlp(batch, (k, n), softmax=False))
    out = exe.execute_sharded([_upload(rx, client, a, "bf16") for a in (x, w, b)])
    got = lf.bf16_bits_to_f32(_download(out[0])).reshape(batch, n)
    pick = np.concatenate([np.arange(4), np.linspace(4, batch - 5, rows - 8).astype(int), np.arange(batch - 4, batch)])
    args = [I.Tensor.from_bytes(x[pick].tobytes(), "bf16", (rows, k)), I.Tensor.from_bytes(w.tobytes(), "bf16", (k, n)),
            I.Tensor.from_bytes(b.tobytes(), "bf16", (n,))]
    ref = oracle_run(P.mlp(rows, (k, n), softmax=False), args, hifi=True, excess=True)
    xf, wf, bf = [t.a.astype(np.float64) for t in args]
    assert contraction_err(got[pick], ref[0].a, np.abs(xf) @ np.abs(wf) + np.abs(bf)[None, :]) <= 1e-2


def test_fp8_linear_8192_rows_sampled(rx, client):
    n, rows = 8192, 32
    act = np.random.default_rng(0).normal(size=(n, n)).astype(np.float32)
    act[0, 0] = 9.0                                                        # the per-tensor absmax sits in a sampled row
    a_raw = _bf16(act)
    codes = np.random.default_rng(1).integers(0, 256, size=(n, n), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38                                   # no NaN codes among the weights
    sw = np.float32(0.0123)
    exe = rx.xla_compile(client, P.fp8_linear(n, n, n))
    out = exe.execute_sharded([_upload(rx, client, a_raw, "bf16"), _upload(rx, client, codes, "f8E4M3FN"), _upload(rx, client, sw, "f32")])
    got = lf.bf16_bits_to_f32(_download(out[0])).reshape(n, n)
    assert np.allclose((got.astype(np.float64) ** 2).mean(axis=1), 1.0, atol=2e-2)   # RMSNorm: unit mean square per row
    args = [I.Tensor.from_bytes(a_raw[:rows].tobytes(), "bf16", (rows, n)),
            I.Tensor.from_bytes(codes.tobytes(), "f8E4M3FN", (n, n)), I.Tensor(sw, "f32")]
    ref = oracle_run(P.fp8_linear(rows, n, n), args, hifi=True, excess=True)
    assert max_rel_to_scale(got[:rows], ref[0].a) <= 1e-2
    # rows are normalised one by one: each sampled row against its own largest entry
    g64, r64 = got[:rows].astype(np.float64), ref[0].a.astype(np.float64)
    assert float(np.max(np.max(np.abs(g64 - r64), axis=1) / np.max(np.abs(r64), axis=1))) <= 1e-2


def test_fp8_dot_8192_componentwise(rx, client):
    """The 8192-long e4m3 contraction of the FP8 layer on its own at full size (both operands [rows][k], f32 result, no
    scale, no norm), on sampled rows: |got - ref|_ij <= 1e-2 (|A8| . |W8|)_ij with the reference accumulated in float64.
    Products of two e4m3 values are exact in float32, so what this bounds is the f32 accumulation over 8192 terms in the
    order the kernel takes them, and a dropped K tile or a wrong fragment shows as an entry of its own."""
    n, rows = 8192, 48
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, size=(n, n), dtype=np.uint8)
    w = rng.integers(0, 256, size=(n, n), dtype=np.uint8)
    for c in (a, w):
        c[(c & 0x7F) == 0x7F] = 0x38                                       # no NaN codes
    ta, to = "tensor<%dx%dxf8E4M3FN>" % (n, n), "tensor<%dx%dxf32>" % (n, n)
    text = ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%0 = stablehlo.dot_general %%arg0, %%arg1, contracting_dims = [1] x [1], precision = [DEFAULT, DEFAULT] : (%s, %s) -> %s\n"
            "    return %%0 : %s\n  }\n}\n" % (ta, ta, to, ta, ta, to, to))
    exe = rx.xla_compile(client, text)
    assert [l["kind"] for l in exe.launches()] == ["gemm_f8"], exe.report()
    out = exe.execute_sharded([_upload(rx, client, a, "f8E4M3FN"), _upload(rx, client, w, "f8E4M3FN")])
    got = _download(out[0]).reshape(n, n)
    pick = np.concatenate([np.arange(4), np.linspace(4, n - 5, rows - 8).astype(int), np.arange(n - 4, n)])
    af = lf.e4m3fn_bits_to_f32(a[pick]).astype(np.float64)
    wf = lf.e4m3fn_bits_to_f32(w).astype(np.float64)
    ref, bound = af @ wf.T, np.abs(af) @ np.abs(wf).T
    assert contraction_err(got[pick], ref, bound) <= 1e-2
    # and far inside it: float32 accumulation of exact products
    assert contraction_err(got[pick], ref, bound) <= 1e-4


def test_tensors_of_more_than_2_31_elements(rx, client):
    """Index arithmetic switches to 64 bits when a tensor has 2^31 elements or more: an elementwise
    map with a shifted slice and a pad, a full reduction, a row and a column reduction, bit for bit
    on i8 data (2 GiB per tensor)."""
    n = (1 << 31) + 4096
    t = "tensor<%dxi8>" % n
    mapped = ("module { func.func @main(%%a: %s) -> %s {\n %%c = stablehlo.constant dense<3> : %s\n %%0 = stablehlo.multiply %%a, %%c : %s\n"
              " %%1 = stablehlo.slice %%0 [5:%d] : (%s) -> tensor<%dxi8>\n %%z = stablehlo.constant dense<7> : tensor<i8>\n"
              " %%2 = stablehlo.pad %%1, %%z, low = [2], high = [3], interior = [0] : (tensor<%dxi8>, tensor<i8>) -> %s\n return %%2 : %s } }"
              % (t, t, t, t, n, t, n - 5, n - 5, t, t))
    summed = ("module { func.func @main(%%a: %s) -> tensor<i64> {\n %%0 = stablehlo.convert %%a : (%s) -> tensor<%dxi64>\n"
              " %%z = stablehlo.constant dense<0> : tensor<i64>\n"
              " %%1 = stablehlo.reduce(%%0 init: %%z) applies stablehlo.add across dimensions = [0] : (tensor<%dxi64>, tensor<i64>) -> tensor<i64>\n"
              " return %%1 : tensor<i64> } }" % (t, t, n, n))
    rng = np.random.default_rng(0)
    x = rng.integers(-20, 21, size=n, dtype=np.int8)
    bx = rx.Buffer.from_host(client, x, "i8")
    out = rx.xla_compile(client, mapped).execute_sharded([bx])[0].synced_buffer().to_host()
    assert np.array_equal(out[2:n - 3], (x[5:] * np.int8(3)).astype(np.int8)) and (out[:2] == 7).all() and (out[n - 3:] == 7).all()
    del out
    total = rx.xla_compile(client, summed).execute_sharded([bx])[0].synced_buffer().to_host()
    assert int(total) == int(x.sum(dtype=np.int64))
    del bx, x
    R, C = (1 << 16) + 1, 1 << 15
    t2 = "tensor<%dx%dxi8>" % (R, C)
    sums = ("module { func.func @main(%%a: %s) -> (tensor<%dxi32>, tensor<%dxi32>) {\n %%0 = stablehlo.convert %%a : (%s) -> tensor<%dx%dxi32>\n"
            " %%z = stablehlo.constant dense<0> : tensor<i32>\n"
            " %%1 = stablehlo.reduce(%%0 init: %%z) applies stablehlo.add across dimensions = [1] : (tensor<%dx%dxi32>, tensor<i32>) -> tensor<%dxi32>\n"
            " %%2 = stablehlo.reduce(%%0 init: %%z) applies stablehlo.add across dimensions = [0] : (tensor<%dx%dxi32>, tensor<i32>) -> tensor<%dxi32>\n"
            " return %%1, %%2 : tensor<%dxi32>, tensor<%dxi32> } }" % (t2, R, C, t2, R, C, R, C, R, R, C, C, R, C))
    x2 = rng.integers(-20, 21, size=(R, C), dtype=np.int8)
    outs = rx.xla_compile(client, sums).execute_sharded([rx.Buffer.from_host(client, x2, "i8")])
    assert np.array_equal(outs[0].synced_buffer().to_host(), x2.sum(axis=1, dtype=np.int32))
    assert np.array_equal(outs[1].synced_buffer().to_host(), x2.sum(axis=0, dtype=np.int32))
