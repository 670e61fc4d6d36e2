"""RxExecuteNoAlloc: the launch list of an executable with caller-owned result buffers and every
temporary of the plan inside the library's static device array.  Checked against XLAExecuteSharded
(same kernels, so bit for bit) on two calls in a row, the second with a smaller input."""
import ctypes

import numpy as np
import pytest

from _loader import load_programs

pytestmark = pytest.mark.gpu


def _no_alloc(rx, exe, bufs, outs):
    """Straight through the C ABI: handles in, return code and RxLastError out."""
    a = (ctypes.c_void_p * len(bufs))(*[b.handle for b in bufs])
    r = (ctypes.c_void_p * len(outs))(*[b.handle for b in outs])
    rx.lib.RxClearError()
    rc = rx.lib.RxExecuteNoAlloc(exe.handle, len(bufs), a, len(outs), r)
    msg = (rx.lib.RxLastError() or b"").decode()
    rx.lib.RxClearError()
    if rc != 0:
        raise rx.ReactantInternalError(msg)


def _compare(rx, client, text, arrays, dtypes):
    exe = rx.xla_compile(client, text)
    bufs = [rx.Buffer.from_host(client, a, dt) for a, dt in zip(arrays, dtypes)]
    ref = [r.synced_buffer() for r in exe.execute_sharded(bufs)]
    outs = [rx.Buffer.uninitialized(client, b.shape(), b.dtype()) for b in ref]
    stats0 = client.default_device().allocator_stats()
    _no_alloc(rx, exe, bufs, outs)
    client.default_device().synchronize()
    stats1 = client.default_device().allocator_stats()
    assert stats1["num_allocs"] == stats0["num_allocs"]          # nothing came from the allocator
    for o, r in zip(outs, ref):
        assert o.to_host().tobytes() == r.to_host().tobytes()
    return exe, bufs, outs


def test_no_alloc_matches_execute_sharded_on_two_calls_in_a_row(rx, client):
    P = load_programs()
    assert rx.lib.RxNoAllocScratchBytes() == 4 << 20
    for n in (1 << 22, 100003):                                   # the second call is smaller
        x = np.random.default_rng(0).uniform(-np.pi, np.pi, n).astype(np.float32)
        y = np.random.default_rng(1).uniform(-np.pi, np.pi, n).astype(np.float32)
        exe, _, _ = _compare(rx, client, P.sinsum_add(n), [x, y], ["f32", "f32"])
        assert [l["kind"] for l in exe.launches()] == ["reduce", "reduce_final"]   # partials live in the scratch array
    # several temporaries: absmax partials, the scale, the quantized activations, the product
    for m in (256, 128):
        a = rx.encode(np.random.default_rng(2).normal(size=(m, 256)).astype(np.float32), "bf16")
        w = rx.encode(np.random.default_rng(3).normal(size=(256, 256)).astype(np.float32), "f8E4M3FN")
        sw = np.float32(0.01).reshape(())
        _compare(rx, client, P.fp8_linear(m, 256, 256), [a, w, sw], ["bf16", "f8E4M3FN", "f32"])
    # a pass-through argument, a constant and a computed result in one module
    t = """module {
  func.func @main(%a: tensor<300xf32>) -> (tensor<300xf32>, tensor<4xi32>, tensor<300xf32>, tensor<300xf32>) {
    %c = stablehlo.constant dense<[1, 2, 3, 4]> : tensor<4xi32>
    %0 = stablehlo.add %a, %a : tensor<300xf32>
    return %a, %c, %0, %0 : tensor<300xf32>, tensor<4xi32>, tensor<300xf32>, tensor<300xf32>
  }
}
"""
    _compare(rx, client, t, [np.arange(300, dtype=np.float32)], ["f32"])
    # two chained 16-bit convolutions: the filters' layout maps as one launch with two results, the padded images, the
    # first product's result on the second one's padded grid -- all of them temporaries in the array
    import importlib
    NN = importlib.import_module("reactant_jl_amd.nn_programs")
    text, shapes = NN.conv_chain(2, 64, 24, 2, "bf16")
    rng = np.random.default_rng(4)
    arrays = [rx.encode((rng.normal(size=sh) * (0.05 if len(sh) == 4 and k > 0 else 1.0)).astype(np.float32), "bf16") for k, sh in enumerate(shapes)]
    exe, _, _ = _compare(rx, client, text, arrays, ["bf16"] * len(shapes))
    assert [l["kind"] for l in exe.launches()] == ["map", "map_transposed", "conv_bf16", "conv_bf16", "map_transposed"]


def test_no_alloc_rejects_what_does_not_fit(rx, client):
    P = load_programs()
    # the hidden activations of this MLP are 2 x 8 MB: more than the scratch array holds
    text = P.mlp(1024, (1024, 4096, 4096, 1024))
    exe = rx.xla_compile(client, text)
    import re
    params = re.findall(r"%arg\d+: tensor<([^>]*)>", text)
    bufs = [rx.Buffer.uninitialized(client, [int(s) for s in p.split("x")[:-1]], p.split("x")[-1]) for p in params]
    out = [rx.Buffer.uninitialized(client, [1024, 1024], "bf16")]
    with pytest.raises(rx.ReactantInternalError, match="RESOURCE_EXHAUSTED.*RxExecuteNoAlloc"):
        _no_alloc(rx, exe, bufs, out)
    # wrong result type, result aliasing an argument
    exe2 = rx.xla_compile(client, P.sinsum_add(4096))
    x = rx.Buffer.uninitialized(client, [4096], "f32")
    with pytest.raises(rx.ReactantInternalError, match="result buffer 0 has type"):
        _no_alloc(rx, exe2, [x, x], [x])
