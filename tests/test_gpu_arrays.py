"""Operations on device arrays that compile a small function behind the scenes, as the reference
does for arrays that do not live in host memory: `fill!`, scalar `setindex!`/`getindex`
(src/ConcreteRArray.jl:423-446,783-805), `similar`/`copy` (src/xla/PJRT/Buffer.jl:19-103,170-182),
and the same modules with run-time start indices against the oracle."""
import numpy as np
import pytest

import _while_modules as W
from _harness import gpu_run, oracle_run
from oracle import stablehlo_interp as I

pytestmark = pytest.mark.gpu


def test_fill_setindex_getindex_on_a_device_array(rx, client):
    a = np.arange(12, dtype=np.float64).reshape(3, 4)
    x = rx.to_rarray(a, client=client)
    assert x.getindex(2, 3) == a[1, 2]
    x.setindex(-5.0, 2, 4)
    x.setindex(7.5, 3, 1)
    a[1, 3], a[2, 0] = -5.0, 7.5
    assert np.array_equal(np.asarray(x), a)
    assert [x.getindex(i + 1, j + 1) for i in range(3) for j in range(4)] == list(a.reshape(-1))
    y = x.copy()
    x.fill(2.0)
    assert np.array_equal(np.asarray(x), np.full((3, 4), 2.0)) and np.array_equal(np.asarray(y), a)
    z = x.similar()
    assert z.shape == (3, 4) and z.dtype == "f64" and np.asarray(z).shape == (3, 4)
    w = x.similar(dtype="i32", shape=(5,))
    w.fill(9)
    assert np.array_equal(np.asarray(w), np.full(5, 9, dtype=np.int32))
    with pytest.raises(IndexError):
        x.setindex(1.0, 4, 1)
    with pytest.raises(IndexError):
        x.getindex(0, 1)


def test_one_executable_serves_every_position(rx, client):
    x = rx.to_rarray(np.zeros((2, 3, 4), dtype=np.float32), client=client)
    before = len(rx._THUNKS)
    for i in range(2):
        for j in range(3):
            for k in range(4):
                x.setindex(100 * i + 10 * j + k, i + 1, j + 1, k + 1)
    assert len(rx._THUNKS) == before + 1
    want = np.fromfunction(lambda i, j, k: 100 * i + 10 * j + k, (2, 3, 4)).astype(np.float32)
    assert np.array_equal(np.asarray(x), want)


@pytest.mark.parametrize("i,j", [(1, 1), (3, 4), (2, 3)])
def test_update_slice_with_runtime_indices_matches_the_oracle(rx, client, i, j):
    a = np.arange(12, dtype=np.float64).reshape(4, 3)
    args = [I.Tensor(a, "f64"), I.Tensor(np.float64(-5), "f64"), I.Tensor(np.int64(i), "i64"), I.Tensor(np.int64(j), "i64")]
    got, _ = gpu_run(rx, client, W.SETINDEX_SCALAR, args)
    want = a.copy()
    want[j - 1, i - 1] = -5
    assert np.array_equal(got[0].a, want) and np.array_equal(got[0].a, oracle_run(W.SETINDEX_SCALAR, args)[0].a)


@pytest.mark.parametrize("i,j,ei,ej", [(0, 0, 0, 0), (1, 2, 1, 2), (7, -2, 1, 0), (-3, 9, 0, 2)])
def test_slice_with_runtime_indices_clamps_like_the_specification(rx, client, i, j, ei, ej):
    """Start indices are clamped so that the slice stays inside the operand."""
    a = np.arange(12, dtype=np.float64).reshape(4, 3)
    args = [I.Tensor(a, "f64"), I.Tensor(np.int32(i), "i32"), I.Tensor(np.int32(j), "i32")]
    got, _ = gpu_run(rx, client, W.GETINDEX_BLOCK, args)
    assert np.array_equal(got[0].a, a[ej:ej + 2, ei:ei + 2])
    assert np.array_equal(got[0].a, oracle_run(W.GETINDEX_BLOCK, args)[0].a)


def test_fill_module(rx, client):
    args = [I.Tensor(np.zeros((4, 3), np.float32), "f32"), I.Tensor(np.float32(1.25), "f32")]
    got, _ = gpu_run(rx, client, W.FILL, args)
    assert np.array_equal(got[0].a, np.full((4, 3), 1.25, np.float32))


def test_profiled_execution_does_not_block_and_reports_every_launch(rx, client):
    """RxExecuteProfiled / RxExecutableTakeTimings: same results as a plain execution, one timing
    per kernel launch, summed over the executions queued since the last read."""
    from _loader import load_programs
    P = load_programs()
    n = 1 << 16
    x = np.random.default_rng(0).uniform(-3, 3, n).astype(np.float32)
    y = np.random.default_rng(1).uniform(-3, 3, n).astype(np.float32)
    exe = rx.xla_compile(client, P.sinsum_add(n))
    bufs = [rx.Buffer.from_host(client, a, "f32") for a in (x, y)]
    want = exe.execute_sharded(bufs)[0].synced_buffer().to_host()
    outs = [exe.execute_profiled(bufs)[0] for _ in range(5)]
    runs, ms = exe.take_timings()
    assert runs == 5 and len(ms) == len(exe.launches()) >= 1 and all(m > 0 for m in ms)
    assert all(np.array_equal(o.to_host(), want) for o in outs)
    assert exe.take_timings()[0] == 0


def test_calls_from_several_host_threads(rx, client):
    """Calls arrive from any host thread (Julia tasks) and frees from finalizer threads: uploads,
    executions of one shared executable, downloads and frees from four threads at once."""
    import threading
    from _loader import load_programs
    P = load_programs()
    n = 1 << 14
    exe = rx.xla_compile(client, P.sinsum_add(n))
    errors, results = [], {}

    def work(k):
        try:
            rng = np.random.default_rng(k)
            for rep in range(20):
                x = rng.uniform(-3, 3, n).astype(np.float32)
                y = rng.uniform(-3, 3, n).astype(np.float32)
                bx, by = rx.Buffer.from_host(client, x, "f32"), rx.Buffer.from_host(client, y, "f32")
                out = exe.execute_sharded([bx, by])[0].synced_buffer().to_host()
                want = float((np.sin(x.astype(np.float64)) + y).sum())
                if abs(float(out) - want) > 1e-5 * np.sqrt(n) * 4:
                    errors.append((k, rep, float(out), want))
                bx.free()
                by.free()
            results[k] = True
        except Exception as e:      # noqa: BLE001 - reported below
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]
    assert len(results) == 4


PASS_THROUGH = """module {
  func.func @main(%a: tensor<256xf32>, %b: tensor<256xf32>) -> (tensor<256xf32>, tensor<256xf32>) {
    %0 = stablehlo.add %a, %b : tensor<256xf32>
    return %a, %0 : tensor<256xf32>, tensor<256xf32>
  }
}
"""


def test_an_argument_returned_unchanged_is_a_buffer_of_its_own_unless_donated(rx, client):
    a = np.arange(256, dtype=np.float32)
    exe = rx.xla_compile(client, PASS_THROUGH)
    ba, bb = rx.Buffer.from_host(client, a, "f32"), rx.Buffer.from_host(client, a, "f32")
    out = [r.synced_buffer() for r in exe.execute_sharded([ba, bb])]
    assert out[0].unsafe_pointer() != ba.unsafe_pointer()
    out[0].copy_from_host(np.full(256, -1.0, dtype=np.float32))          # writes the result only
    assert np.array_equal(ba.to_host(), a) and np.array_equal(out[0].to_host(), np.full(256, -1.0, dtype=np.float32))
    assert np.array_equal(out[1].to_host(), 2 * a)
    # donated: the result takes the argument's storage over, the argument can no longer be read
    p = ba.unsafe_pointer()
    out = [r.synced_buffer() for r in exe.execute_sharded([ba, bb], donated=[True, False])]
    assert out[0].unsafe_pointer() == p and np.array_equal(out[0].to_host(), a)
    with pytest.raises(rx.ReactantInternalError, match="donated"):
        ba.to_host()


def test_memory_limit_is_enforced_and_a_failed_execution_keeps_donated_arguments(rx):
    """A client with a small memory fraction: an allocation beyond it fails with RESOURCE_EXHAUSTED
    (src/accelerators/GPU.jl:7-37 passes the fraction), and an execution that fails that way leaves
    the argument it was asked to donate readable."""
    small = rx.Client(memory_fraction=2e-4)                                # about 58 MB of 288 GB
    try:
        limit = small.default_device().allocator_stats()["bytes_limit"]
        assert 0 < limit < (1 << 28)
        n = int(limit // 4 * 0.6)
        x = np.ones(n, dtype=np.float32)
        bx = rx.Buffer.from_host(small, x, "f32")                          # 60 % of the limit: fits
        with pytest.raises(rx.ReactantInternalError, match="RESOURCE_EXHAUSTED"):
            rx.Buffer.from_host(small, x, "f32")                           # a second one does not
        t = "tensor<%dxf32>" % n
        exe = rx.xla_compile(small, "module { func.func @main(%%a: %s) -> %s { %%0 = stablehlo.add %%a, %%a : %s\n return %%0 : %s } }" % (t, t, t, t))
        with pytest.raises(rx.ReactantInternalError, match="RESOURCE_EXHAUSTED"):
            exe.execute_sharded([bx], donated=[True])                      # the result does not fit beside the argument
        assert float(bx.to_host()[n - 1]) == 1.0                           # still the caller's
        exe.free()
        bx.free()
    finally:
        small.close()


def test_futures_are_asked_late_or_never(rx):
    """A future records its event when it is first asked (src/xla/PJRT/Future.jl:1-28 only ever polls or awaits): asking
    after more work was queued, asking twice, never asking, and asking after the client was freed all behave."""
    own = rx.Client()
    try:
        n = 1 << 22
        t = "tensor<%dxf32>" % n
        exe = rx.xla_compile(own, "module { func.func @main(%%a: %s) -> %s { %%0 = stablehlo.add %%a, %%a : %s\n return %%0 : %s } }" % (t, t, t, t))
        x = np.arange(n, dtype=np.float32)
        bx = rx.Buffer.from_host(own, x, "f32")
        first = exe.execute_sharded([bx])[0]
        later = [exe.execute_sharded([bx])[0] for _ in range(20)]          # more work behind the first call
        assert first.future is not None
        first.future.wait()                                                # waits for a point at or after the first call's end
        assert first.future.is_ready()                                     # asked again: the same event
        assert np.array_equal(first.buffer.to_host(), 2 * x)
        while not later[-1].future.is_ready():                             # polling alone makes progress
            pass
        assert np.array_equal(later[-1].buffer.to_host(), 2 * x)
        unasked = later[3].future                                          # never asked before the client goes away
    finally:
        own.close()
    assert unasked.is_ready()                                              # FreeClient waited for the stream
    unasked.wait()


def test_cost_analysis_of_an_executable(rx, client):
    from _loader import load_programs
    P = load_programs()
    """XLA.cost_analysis(exec) (reference src/xla/Stats.jl:86-115): the eleven HloCostAnalysisProperties fields through the
    C ABI, for the fused sin + add + sum and for a matrix product."""
    n = 1 << 20
    exe = rx.xla_compile(client, P.sinsum_add(n))
    c = exe.cost_analysis()
    assert c["flops"] == 2.0 * n and c["transcendentals"] == float(n)
    assert c["operand0_bytes_accessed"] == 4.0 * n and c["operand1_bytes_accessed"] == 4.0 * n and c["output_root_bytes_accessed"] == 4.0
    assert c["bytes_accessed"] >= 8.0 * n and 0.0 < c["utilization"] <= 1.0
    assert c["optimal_seconds"] == pytest.approx(8.0 * n / 8.0e12, rel=0.05)      # one pass over both vectors at the HBM peak
    exe = rx.xla_compile(client, P.gemm(512, 512, 512))
    c = exe.cost_analysis()
    assert c["flops"] == 2.0 * 512 ** 3 + 3.0 * 512 ** 2 and c["transcendentals"] == 0.0
