"""CPU tests of the boundary and the host logic (no compute calls without a GPU):
the shared library loads and exports every symbol the header declares, the error
convention works, the StableHLO importer and the fusion planner accept what the
reference prints and reject what they cannot run, and the kernel text written for
each benchmark program compiles for gfx950 (hiprtc needs no device)."""
import ctypes
import os
import re

import numpy as np

import pytest

from _loader import load_pkg, load_programs, ROOT
import _while_modules as W

rx = load_pkg()
P = load_programs()
HEADER = os.path.join(ROOT, "include", "reactant_mi355x.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text))
    names -= {"defined", "void"}
    funcs = {n for n in names if re.search(r"\b%s\s*\([^;{]*\)\s*;" % n, text)}
    return funcs


def test_library_exports_every_declared_symbol():
    funcs = declared_symbols()
    assert len(funcs) >= 45
    lib = ctypes.CDLL(rx.LIB_PATH)
    missing = [f for f in sorted(funcs) if not hasattr(lib, f)]
    assert not missing, missing
    # the throw hook is an exported data symbol (reference API.cpp:262)
    hook = ctypes.c_void_p.in_dll(lib, "ReactantThrowError")
    assert hook.value is None
    # every declared function has a ctypes signature in the host mirror, and vice versa
    assert funcs == set(rx.SIGNATURES), funcs ^ set(rx.SIGNATURES)


def test_handles_are_validated_without_a_device():
    assert rx.lib.RxOwns(None) == 0
    assert rx.lib.RxOwns(ctypes.c_void_p(0x1234)) == 0
    # calls on foreign handles fail cleanly with a message instead of dereferencing them
    rx.lib.RxClearError()
    assert rx.lib.ClientNumDevices(ctypes.c_void_p(0x1234)) == 0
    assert b"client handle" in rx.lib.RxLastError()
    rx.lib.RxClearError()
    rx.lib.PjRtBufferFree(ctypes.c_void_p(0x1234))      # finalizer path: silently ignored
    rx.lib.FreeFuture(None)
    rx.lib.ExecutableFree(None)
    assert rx.lib.RxLastError() == b""


def test_throw_callback_is_invoked():
    seen = []
    CB = ctypes.CFUNCTYPE(None, ctypes.c_char_p)
    cb = CB(lambda m: seen.append(m))
    lib = ctypes.CDLL(rx.LIB_PATH)
    hook = ctypes.c_void_p.in_dll(lib, "ReactantThrowError")
    hook.value = ctypes.cast(cb, ctypes.c_void_p).value
    try:
        lib.BufferNDimensions.restype = ctypes.c_int64
        lib.BufferNDimensions(ctypes.c_void_p(0x42))
        assert seen and b"buffer handle" in seen[0]
    finally:
        hook.value = None
        rx.lib.RxClearError()


def test_client_creation_reports_errors_through_the_error_pointer():
    import subprocess, sys
    # in a child process: a machine without a GPU must get NULL + a message, not a crash
    code = ("import sys; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
            "from _loader import load_pkg\nrx = load_pkg()\n"
            "try:\n    rx.Client()\n    print('CLIENT-OK')\n"
            "except rx.ReactantInternalError as e:\n    print('ERR:', e)\n" % (ROOT, os.path.join(ROOT, "tests")))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert "CLIENT-OK" in out.stdout or "ERR:" in out.stdout, out.stdout + out.stderr
    # multi-node requests are refused before any device is touched
    err = ctypes.c_char_p()
    h = rx.lib.MakeGPUClient(0, 2, None, 0, 0.75, False, b"rocm", ctypes.byref(err), None)
    assert not h and b"one process" in err.value
    rx.lib.RxClearError()


PROGRAMS = {
    "sinsum_add": (lambda: P.sinsum_add(1 << 20), ["reduce", "reduce_final"]),
    # a small grid (below 2^18 cells): two of the three steps share a chain kernel, the third is a map
    "stencil": (lambda: P.stencil(64, 64, 32, steps=3), ["map_chain", "map"]),
    "stencil_full": (lambda: P.stencil(512, 512, 256, steps=3), ["map_stencil_lds2", "map_stencil_lds"]),
    "gemm": (lambda: P.gemm(512, 512, 512), ["gemm_f32"]),
    "gemm_transposed": (lambda: P.gemm(512, 256, 128, form="transposed"), ["gemm_f32"]),
    "mlp": (lambda: P.mlp(512, (256, 512, 512, 256)), ["gemm_bf16", "gemm_bf16", "gemm_bf16", "row"]),
    "mlp_gelu_op": (lambda: P.mlp(512, (256, 512, 512, 256), gelu="op"), ["gemm_bf16", "gemm_bf16", "gemm_bf16", "row"]),
    "fp8_linear": (lambda: P.fp8_linear(512, 512, 512), ["reduce", "reduce_final", "map", "gemm_f8", "row"]),
    "fp8_linear_kn": (lambda: P.fp8_linear(512, 512, 512, weight_layout="kn", dot_form="direct"),
                      ["reduce", "reduce_final", "map", "gemm_f8", "row"]),
}


@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_benchmark_programs_plan_and_compile_for_gfx950(name):
    make, kinds = PROGRAMS[name]
    report = rx.compile_offline(make())
    got = re.findall(r"kind=(\w+)", report)
    assert got == kinds, report
    assert "code object:" in report


def test_fusion_plan_of_the_full_size_stencil_is_one_kernel_per_two_timesteps():
    report = rx.compile_offline(P.stencil(512, 512, 256, steps=10))
    launches = re.findall(r"\] (\w+) kind=(\w+)", report)
    assert len(launches) == 5 and {k for _, k in launches} == {"map_stencil_lds2"}
    assert len({k for k, _ in launches}) == 1           # five launches of one compiled kernel
    # compulsory traffic of two timesteps on the halo'd arrays: 2 x (4 reads + 1 write) of 262*518*518 doubles
    assert "algo_bytes=%d" % (2 * 5 * 262 * 518 * 518 * 8) in report
    assert "buffers: 9," in report                      # 4 arguments + 5 fields; the odd steps own no buffer


def test_fusion_plan_of_the_stencil_without_step_pairing(monkeypatch):
    monkeypatch.setenv("RX_STENCIL_FUSE", "0")
    report = rx.compile_offline(P.stencil(512, 512, 256, steps=10))
    launches = re.findall(r"\] (\w+) kind=(\w+)", report)
    assert len(launches) == 10 and {k for _, k in launches} == {"map_stencil_lds"}
    assert "algo_bytes=%d" % (5 * 262 * 518 * 518 * 8) in report


def test_generated_source_is_inspectable():
    report = rx.compile_offline(P.sinsum_add(4096), with_source=True)
    assert "rx_wave_reduce" in report or "rx_block_reduce" in report
    assert "sinf(" in report and "extern \"C\" __global__" in report


@pytest.mark.parametrize("text,needle", [
    ("module { func.func @main(%a: tensor<4xf32>) -> tensor<4xf32> { %0 = stablehlo.frobnicate %a : tensor<4xf32>\n return %0 : tensor<4xf32> } }", "unsupported operation"),
    ("module { func.func @main(%a: tensor<4xf32>) -> tensor<4xf32> { %0 = stablehlo.add %a, %b : tensor<4xf32>\n return %0 : tensor<4xf32> } }", "undefined value"),
    ("module { func.func @main(%a: tensor<4xf32>, %b: tensor<5xf32>) -> tensor<4xf32> { %0 = stablehlo.add %a, %b : tensor<4xf32>\n return %0 : tensor<4xf32> } }", "type mismatch"),
    ("module { func.func @main(%a: tensor<4xc64>) -> tensor<4xc64> { return %a : tensor<4xc64> } }", "unsupported element type"),
    ("module { func.func @main(%a: tensor<4x3xf32>) -> tensor<2x2xf32> { %0 = stablehlo.slice %a [0:2, 2:4] : (tensor<4x3xf32>) -> tensor<2x2xf32>\n return %0 : tensor<2x2xf32> } }", "bounds out of range"),
    ("module { func.func @main(%a: tensor<4xf32>) -> tensor<f32> { return %a : tensor<4xf32> } }", "declared"),
    ("module { func.func @main(%a: tensor<4xf32> -> tensor<4xf32> { return %a : tensor<4xf32> } }", "parse error"),
])
def test_importer_rejects_bad_modules_with_a_message(text, needle):
    with pytest.raises(rx.ReactantInternalError) as e:
        rx.compile_offline(text)
    assert needle in str(e.value)


def test_host_side_array_conventions():
    import numpy as np
    # dims reversal: a Julia array of size (3, 4) travels as a row-major [4][3] buffer (src/xla/PJRT/Buffer.jl:9-17)
    x = np.arange(12.0).reshape(3, 4)
    raw = np.ascontiguousarray(rx.encode(x, "f64").T)
    assert raw.shape == (4, 3) and raw[1, 2] == x[2, 1]
    # narrow floats are packed to their storage bits and back
    v = np.float32([1.0, -2.5, 0.3333, 448.0, 1e-3])
    assert np.array_equal(rx.decode(rx.encode(v, "bf16"), "bf16"), np.float32([1.0, -2.5, 0.333984375, 448.0, 0.00099945068359375]))
    assert rx.decode(rx.encode(v, "f8E4M3FN"), "f8E4M3FN").tolist() == [1.0, -2.5, 0.34375, 448.0, 0.001953125]
    assert rx.PRIMITIVE_TYPE["f32"] == 11 and rx.PRIMITIVE_TYPE["bf16"] == 16 and rx.PRIMITIVE_TYPE["f8E4M3FN"] == 20
    with pytest.raises(rx.ReactantInternalError):
        rx.set_default_backend("tpu")


def test_enzymejax_export_files_are_read_in_argument_order(tmp_path):
    """`<fn>_<id>.mlir` + `<fn>_<id>_inputs.npz` with keys arr_1.. (reference
    src/serialization/EnzymeJAX.jl:124-172); no device needed to read them and plan the module."""
    text = P.sinsum_add(8)
    (tmp_path / "f_0.mlir").write_text(text)
    a, b = np.arange(8, dtype=np.float32), -np.arange(8, dtype=np.float32)
    np.savez(tmp_path / "f_0_inputs.npz", arr_2=b, arr_1=a)
    got_text, arrays = rx.load_enzymejax_export(str(tmp_path / "f_0.mlir"))
    assert got_text == text and len(arrays) == 2
    assert np.array_equal(arrays[0], a) and np.array_equal(arrays[1], b)
    assert "kind=reduce" in rx.compile_offline(got_text)
    np.savez(tmp_path / "g_0_inputs.npz", x=a)
    (tmp_path / "g_0.mlir").write_text(text)
    with pytest.raises(rx.ReactantInternalError, match="arr_1"):
        rx.load_enzymejax_export(str(tmp_path / "g_0.mlir"))


def test_while_with_a_static_trip_count_is_unrolled_at_import():
    """The `@trace for` form of the stencil plans exactly like the unrolled form (five launches of
    the two-step kernel); counters fold to constants, so counter-indexed slices plan too."""
    strip = lambda rep: re.sub(r"code object: \d+ bytes", "", rep)
    assert strip(rx.compile_offline(P.stencil(512, 512, 256, steps=10, loop="while"))) == \
        strip(rx.compile_offline(P.stencil(512, 512, 256, steps=10)))
    rep = rx.compile_offline(W.SETINDEX)
    assert rep.count("dynamic_update_slice") >= 1 and "kind=map" in rep
    assert "launches: 2" in rx.compile_offline(W.GENERIC)


@pytest.mark.parametrize("text", [W.DATA_DEPENDENT, W.COUNT])
def test_while_with_a_data_dependent_trip_count_is_rejected(text):
    """A bound or a starting value that is an argument: the loop cannot be unrolled."""
    with pytest.raises(rx.ReactantInternalError, match="static trip count"):
        rx.compile_offline(text)


def test_single_launch_reduction_is_an_option(monkeypatch):
    monkeypatch.setenv("RX_SINGLE_PASS_REDUCE", "1")
    rep = rx.compile_offline(P.sinsum_add(1 << 20), with_source=True)
    # partials travel as flagged 64-bit words (no fence, no ticket); the last workgroup collects them
    assert re.findall(r"kind=(\w+)", rep) == ["reduce"] and "rx_publish_partial<float>" in rep and "rx_await_partial<float>" in rep
    f64 = P.sinsum_add(1 << 20).replace("f32", "f64")
    rep = rx.compile_offline(f64, with_source=True)
    assert "rx_publish_partial<double>(slots + (size_t)blockIdx.x * 2" in rep      # two 32-bit pieces per partial


def _dot(lt, rt, ot, attrs):
    return ("module {\n  func.func @main(%%arg0: %s, %%arg1: %s) -> %s {\n"
            "    %%0 = stablehlo.dot_general %%arg0, %%arg1, %s : (%s, %s) -> %s\n    return %%0 : %s\n  }\n}\n"
            % (lt, rt, ot, attrs, lt, rt, ot, ot))


def test_products_with_a_vector_like_operand_plan_as_reductions(monkeypatch):
    mv = _dot("tensor<8192x8192xf32>", "tensor<8192xf32>", "tensor<8192xf32>", "contracting_dims = [1] x [0]")
    rep = rx.compile_offline(mv)
    assert "kind=row" in rep and "launches: 1" in rep and "dot" not in rep.split("code object")[0].replace("dot_general", "")
    # contracting the slow dimension walks the matrix in storage order: a column reduction cut into chunks
    mtv = _dot("tensor<8192x8192xf32>", "tensor<8192xf32>", "tensor<8192xf32>", "contracting_dims = [0] x [0]")
    assert "kind=reduce_generic" in rx.compile_offline(mtv)
    inner = _dot("tensor<67108864xf32>", "tensor<67108864xf32>", "tensor<f32>", "contracting_dims = [0] x [0]")
    rep = rx.compile_offline(inner)
    assert "kind=reduce " in rep and "kind=reduce_final" in rep
    # a real matrix product is left to the MFMA skeleton, a short contraction to the scalar loop
    assert "kind=gemm_f32" in rx.compile_offline(P.gemm(256, 256, 256))
    short = _dot("tensor<4096x16xf32>", "tensor<16xf32>", "tensor<4096xf32>", "contracting_dims = [1] x [0]")
    assert "kind=dot_scalar" in rx.compile_offline(short)
    # without the rewrite the product is padded to four columns and runs on the MFMA skeleton
    monkeypatch.setenv("RX_DOT_AS_REDUCE", "0")
    assert "kind=gemm_f32" in rx.compile_offline(mv)


def test_windowed_ops_plan(monkeypatch):
    import _nn_modules as NN
    # cumsum over 2^24 elements: one launch whose workgroups hand their chunk totals on as flagged words
    rep = rx.compile_offline(NN.cumulative([1 << 24], "f32", 0), with_source=True)
    assert "kind=scan " in rep and "launches: 1" in rep and "rx_peek_partial<float>" in rep and "unsigned* __restrict__ fault" in rep
    # the form that does not wait for other workgroups: chunk totals, then the scan proper
    monkeypatch.setenv("RX_SINGLE_PASS_SCAN", "0")
    rep = rx.compile_offline(NN.cumulative([1 << 24], "f32", 0))
    assert "kind=scan_totals" in rep and "kind=scan " in rep and "launches: 2" in rep
    monkeypatch.delenv("RX_SINGLE_PASS_SCAN")
    # rows of a matrix: one workgroup per row chunk, no totals needed when a row is one chunk
    assert "launches: 1" in rx.compile_offline(NN.cumulative([4096, 4096], "f32", 1))
    # pooling: the window view is index arithmetic inside a reduction kernel
    rep = rx.compile_offline(NN.reduce_window([8, 16, 32, 32], "f32", "maximum", [1, 1, 2, 2], strides=[1, 1, 2, 2])[0])
    assert "launches: 1" in rep and "window reduce" in rep
    # f32 convolution, unit strides, 64 output features: the direct-convolution kernel with bias + relu as its epilogue,
    # seven rows of the result per workgroup (256 workgroups)
    conv = NN.convolution([32, 64, 56, 56], [64, 64, 3, 3], "f32", padding=[[1, 1], [1, 1]], epilogue="bias_relu")[0]
    kinds = lambda rep: [ln.split("kind=")[1].split()[0] for ln in rep.splitlines() if "kind=" in ln]
    rep = rx.compile_offline(conv, with_source=True)
    assert kinds(rep) == ["conv"] and "grid=256x1x1" in rep, rep
    assert "rx_conv_body<32, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1, 56, 56, 7, 8, " in rep
    # without it: one MFMA product (64-row tiles) that evaluates the window matrix while it loads its tiles, then
    # bias + relu + layout in one map; the reshaped weights share the argument's buffer
    monkeypatch.setenv("RX_CONV_DIRECT", "0")
    rep = rx.compile_offline(conv, with_source=True)
    assert kinds(rep) == ["gemm_f32", "map"], rep
    assert "rx_gemm_body<rx_mma_f32, 64, 128" in rep and "dot operand B computed on the fly" in rep
    # many output features: every tile row would evaluate the window matrix again, so it is written once instead
    rep = rx.compile_offline(NN.convolution([32, 256, 14, 14], [256, 256, 3, 3], "f32", padding=[[1, 1], [1, 1]])[0])
    assert kinds(rep) == ["map", "gemm_f32", "map"], rep
    monkeypatch.setenv("RX_FUSE_DOT_OPERANDS", "0")
    rep = rx.compile_offline(conv, with_source=True)
    assert kinds(rep) == ["map", "gemm_f32", "map"] and "rx_gemm_body_dl<rx_mma_f32, 64, 128" in rep
    monkeypatch.delenv("RX_FUSE_DOT_OPERANDS")
    monkeypatch.delenv("RX_CONV_DIRECT")
    # a strided stem (three channels: one slab, one LDS stage): two rows of the result per workgroup
    rep = rx.compile_offline(NN.convolution([32, 3, 224, 224], [64, 3, 7, 7], "f32", strides=[2, 2], padding=[[3, 3], [3, 3]])[0], with_source=True)
    assert kinds(rep) == ["conv"] and "rx_conv_body<32, 3, 224, 224, 64, 7, 7, 2, 2, 1, 1, 3, 3, 112, 112, 2, 4, " in rep, rep
    # few output features, input dilation, other element types: the matrix product
    assert "kind=conv" not in rx.compile_offline(NN.convolution([1, 3, 33, 35], [16, 3, 5, 5], "f32", strides=[2, 2], padding=[[2, 2], [2, 2]])[0])
    assert "kind=conv" not in rx.compile_offline(NN.convolution([2, 8, 20, 20], [64, 8, 3, 3], "f32", lhs_dil=[2, 2], padding=[[2, 2], [2, 2]])[0])
    assert "kind=conv " not in rx.compile_offline(NN.convolution([2, 32, 28, 28], [64, 32, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0])
    with pytest.raises(Exception, match="batch_group_count and feature_group_count"):
        rx.compile_offline(NN.convolution([2, 8, 16, 16], [4, 4, 4, 4], "f32", groups=2)[0].replace("batch_group_count = 1", "batch_group_count = 2"))
    # 16-bit images, whole 128-byte runs of channels, unit strides: pad + layout map, filter layout map, the product with
    # one row shift per tap on the skeleton the product's shape gets, and the transposing map of the result
    rep = rx.compile_offline(NN.convolution([32, 256, 56, 56], [256, 256, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0], with_source=True)
    assert kinds(rep) == ["map_transposed", "map", "conv_bf16", "map_transposed"], rep
    assert "rx_gemm_body_pp<rx_el_bf16, 256, 256, 2, 4, true, true, 107648, 256, 2304, " in rep and "rx_tap_shift<256, 3, 58, 1, 2>>(A, B, epi)" in rep
    rep = rx.compile_offline(NN.convolution([32, 64, 112, 112], [128, 64, 3, 3], "f16", padding=[[1, 1], [1, 1]], rhs_dil=[1, 2])[0], with_source=True)
    assert kinds(rep) == ["map_transposed", "map", "conv_f16", "map_transposed"] and "rx_gemm_body_s<rx_el_f16, 256, 128, 4, 2, true, true, " in rep and "rx_tap_shift<64, 3, 228, 1, 2>>" in rep, rep
    rep = rx.compile_offline(NN.convolution([4, 256, 56, 56], [256, 256, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0], with_source=True)
    assert "conv_bf16" in kinds(rep) and "rx_gemm_body_dl<rx_mma_bf16_16, 128, 128, 64, " in rep and ", 1, rx_tap_shift<256, 3, 58, 1, 2>>" in rep, rep
    # not that form: strides, channels that are not whole 128-byte runs, a product that is cut along K, the switch
    assert "conv_bf16" not in kinds(rx.compile_offline(NN.convolution([32, 64, 56, 56], [128, 64, 3, 3], "bf16", strides=[2, 2], padding=[[1, 1], [1, 1]])[0]))
    assert "conv_bf16" not in kinds(rx.compile_offline(NN.convolution([32, 8, 56, 56], [128, 8, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0]))
    # 96 channels: padded with zero channels to 128, in the images' layout map and in the filter's (up to four times the channels)
    rep = rx.compile_offline(NN.convolution([32, 96, 56, 56], [128, 96, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0], with_source=True)
    assert "conv_bf16" in kinds(rep) and "rx_tap_shift<128, 3, 58, 1, 2>>" in rep, rep
    assert "conv_bf16" not in kinds(rx.compile_offline(NN.convolution([4, 512, 14, 14], [512, 512, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0]))
    monkeypatch.setenv("RX_CONV_SHIFT", "0")
    assert "conv_bf16" not in kinds(rx.compile_offline(NN.convolution([32, 256, 56, 56], [256, 256, 3, 3], "bf16", padding=[[1, 1], [1, 1]])[0]))
    monkeypatch.delenv("RX_CONV_SHIFT")
    # two such convolutions with bias + relu between them share the padded grid: the first one's kernel writes the
    # second one's zero-padded operand and no map runs between them; the switch, and a first convolution whose kernel
    # does not hold the ops between them (then the module is planned again without it), leave the maps in
    text = NN.conv_chain(32, 256, 56, 2, "bf16")[0]
    # (the two filters' layout maps read arguments only: they run first, as one launch)
    chained = ["map", "map_transposed", "conv_bf16", "conv_bf16", "map_transposed"]
    unchained = ["map", "map_transposed", "conv_bf16", "map", "conv_bf16", "map_transposed"]
    rep = rx.compile_offline(text, with_source=True)
    assert kinds(rep) == chained and "zero_" in rep, rep
    monkeypatch.setenv("RX_CHAIN_CONVS", "0")
    rep = rx.compile_offline(text, with_source=True)
    assert kinds(rep) == unchained and "zero_" not in rep, rep
    monkeypatch.delenv("RX_CHAIN_CONVS")
    monkeypatch.setenv("RX_EPILOGUES", "0")
    rep = rx.compile_offline(text, with_source=True)
    assert kinds(rep) == unchained and "zero_" not in rep, rep
    monkeypatch.delenv("RX_EPILOGUES")


def test_vgg11_forward_pass_plans(monkeypatch):
    """VGG-11 with batch norm in test mode (benchmark/nn/vision.jl:24-34).  In f32 on 4 images: the direct kernel where it
    covers the layer; batch norm + relu run in the pooling kernel that reads the convolution (RX_CONV_TAILS=2: in the
    convolution's epilogue, the pools as pure window reductions).  In bf16 on 32 images: seven products with row shifts
    with batch norm + relu as their epilogues (results narrower than the accumulators are written where a window reads
    them); the pools between two of them run channel-minor -- no transposing map on either side, a padding map after
    them -- and take eight outputs per thread; convolutions that follow one another directly are chained."""
    import _nn_modules as NN
    parse = lambda rep: [(ln.split("kind=")[1].split()[0], ln.split("::")[1].strip()) for ln in rep.splitlines() if "kind=" in ln]
    f32 = parse(rx.compile_offline(NN.vgg11(batch=4, dt="f32")[0]))
    assert [k for k, _ in f32].count("conv") == 6
    assert [d for k, d in f32 if k == "conv"].count("convolution") == 4 and sum("window" in d and "divide" in d for _, d in f32) >= 4, f32
    monkeypatch.setenv("RX_CONV_TAILS", "2")
    f32 = parse(rx.compile_offline(NN.vgg11(batch=4, dt="f32")[0]))
    assert all("divide" in d and "maximum" in d for k, d in f32 if k == "conv")
    assert [d for k, d in f32 if k == "reduce_generic" and "window" in d][:4] == ["window reduce"] * 4
    monkeypatch.delenv("RX_CONV_TAILS")
    text = NN.vgg11(batch=32, dt="bf16")[0]
    rep = rx.compile_offline(text, with_source=True)
    bf16 = parse(rep)
    kinds = [k for k, _ in bf16]
    assert kinds.count("conv_bf16") == 7 and kinds.count("conv") == 1 and kinds.count("map_transposed") == 1, kinds
    # the zero padding of the next product's operand sits in the pooling kernel's reads (the windows do not overlap): no padding maps
    assert [d for k, d in bf16 if "window" in d][:4] == ["window reduce"] + ["pad window reduce"] * 3
    assert [d for k, d in bf16 if k == "map" and d.startswith("pad")] == []
    assert "static constexpr bool masks_rows = true;" in rep and "rx_keep_value(res);" in rep and "rx_load_const(in0, " in rep
    i = rep.index("// reduce (generic): pad window over dims -> tensor<32x58x58x128xbf16>")
    assert "threadIdx.x) * 8;" in rep[i:i + 400]
    # the conversions of the first images and filter and the seven filter layout maps read arguments only: one launch, first
    assert kinds[0] == "map" and "_maps kind=map grid=9211x1x1" in rep and rep.count("_map_part(blockIdx.x - ") == 9, kinds
    assert len(kinds) == 24
    monkeypatch.setenv("RX_MERGE_MAPS", "0")
    assert len(parse(rx.compile_offline(text))) == 32
    monkeypatch.delenv("RX_MERGE_MAPS")
    monkeypatch.setenv("RX_PAD_INTO_POOLS", "0")
    off = parse(rx.compile_offline(text))
    assert len(off) == 27 and [d for k, d in off if k == "map" and d.startswith("pad")] == ["pad"] * 3
    monkeypatch.delenv("RX_PAD_INTO_POOLS")
    monkeypatch.setenv("RX_NHWC_POOLS", "0")
    off = parse(rx.compile_offline(text))
    assert [k for k, _ in off].count("map_transposed") == 4 and sum("transpose window" in d for _, d in off) == 4, off
    monkeypatch.delenv("RX_NHWC_POOLS")
    monkeypatch.setenv("RX_CONV_TAILS", "0")
    off = parse(rx.compile_offline(text))
    assert sum("window" in d and "divide" in d for _, d in off) == 5, off
    monkeypatch.delenv("RX_CONV_TAILS")


def test_residual_blocks_plan_channel_minor(monkeypatch):
    """Three basic residual blocks in bf16: the filters' layout maps as one launch, the first product's padded operand
    and the block input's layout (two transposing maps), then per block two products (the second one's epilogue adds
    the block's input) and one padding map; the result is transposed once.  Without the regions: a transposing map
    after and before every second product."""
    import _nn_modules as NN
    kinds = lambda rep: [ln.split("kind=")[1].split()[0] for ln in rep.splitlines() if "kind=" in ln]
    text = NN.resnet_stage(batch=32, channels=128, hw=28, blocks=3, dt="bf16")[0]
    c = "conv_bf16"
    assert kinds(rx.compile_offline(text)) == ["map", "map_transposed", c, "map_transposed", c, "map", c, c, "map", c, c, "map_transposed"]
    monkeypatch.setenv("RX_NHWC_REGIONS", "0")
    off = kinds(rx.compile_offline(text))
    assert off.count(c) == 6 and off.count("map_transposed") == 6, off
    monkeypatch.delenv("RX_NHWC_REGIONS")
    # f32 runs on the direct kernel in the module's own layout: nothing to do
    assert "map_transposed" not in kinds(rx.compile_offline(NN.resnet_stage(batch=4, channels=64, hw=28, blocks=2, dt="f32")[0]))


def test_time_loops_over_small_arrays_plan_as_chain_kernels(monkeypatch):
    """The reference's polybench stencils (benchmark/polybench/stencil.jl) at its sizes: 1024 or 256
    trips of a `stablehlo.while` unroll into runs of update steps, which share chain kernels."""
    import importlib
    PB = importlib.import_module("reactant_jl_amd.polybench_programs")
    kinds = lambda rep: [ln.split("kind=")[1].split()[0] for ln in rep.splitlines() if "kind=" in ln]
    k = kinds(rx.compile_offline(PB.build("jacobi_1d")))            # 2048 half steps, 64 per launch
    assert k == ["map_chain"] * 32
    rep = rx.compile_offline(PB.build("jacobi_2d"), with_source=True)
    assert kinds(rep) == ["map_chain"] * 128 and "16 update steps through LDS tiles (32x32 outputs per workgroup, box 64x64, 2 fields)" in rep
    k = kinds(rx.compile_offline(PB.build("fdtd_2d", tmax=32)))      # 96 updates, the last three fused into one step
    assert k == ["map_chain"] * len(k) and len(k) <= 8
    # rank 3: one launch per step; once the arrays are temporaries each step writes only its box, in place
    assert kinds(rx.compile_offline(PB.build("heat_3d", tsteps=8))) == ["map"] * 2 + ["map_in_place"] * 14
    monkeypatch.setenv("RX_CHAIN_STEPS", "1")
    assert kinds(rx.compile_offline(PB.build("jacobi_1d", tsteps=16))) == ["map"] * 2 + ["map_in_place"] * 30
    monkeypatch.setenv("RX_IN_PLACE", "0")
    assert kinds(rx.compile_offline(PB.build("jacobi_1d", tsteps=16))) == ["map"] * 32


def test_long_time_loops_import_and_plan_in_linear_time():
    """8192 trips of a two-step loop body (16384 update steps): import, planning and compilation stay
    linear in the trip count (a few seconds); more than 65536 trips are refused with a message."""
    import importlib
    import time
    PB = importlib.import_module("reactant_jl_amd.polybench_programs")
    t0 = time.time()
    rep = rx.compile_offline(PB.build("jacobi_2d", tsteps=8192))
    assert "launches: 1024" in rep
    assert time.time() - t0 < 60
    with pytest.raises(Exception, match="more than 65536 iterations"):
        rx.compile_offline(PB.build("jacobi_1d", n=64, tsteps=70000))


def test_update_in_place_waits_for_readers_that_are_launched_late():
    """A product absorbed by its epilogue is launched at the epilogue, a reduction fused into a row
    kernel at that kernel's root: when either comes after a `dynamic_update_slice` of the value it
    reads, the update must write a buffer of its own (kind map, not map_in_place)."""
    import _inplace_modules as M
    kinds = lambda rep: re.findall(r"kind=(\w+)", rep)
    assert kinds(rx.compile_offline(M.DOT_EPILOGUE_AFTER_UPDATE)) == ["map", "map", "gemm_f32"]
    assert kinds(rx.compile_offline(M.ROW_REDUCE_AFTER_UPDATE)) == ["gemm_f32", "map", "row"]
    assert kinds(rx.compile_offline(M.UPDATE_AFTER_ALL_READERS)) == ["map", "gemm_f32", "map_in_place"]


def test_gemm_tuning_overrides_are_honoured_or_refused(monkeypatch):
    # a K step whose two LDS stages exceed 160 KB used to end in the scalar loop without a word
    fp8 = P.fp8_linear(512, 512, 512)
    monkeypatch.setenv("RX_GEMM_TILE", "256,256,2,4")
    monkeypatch.setenv("RX_GEMM_BK", "256")
    with pytest.raises(rx.ReactantInternalError, match="tuning override cannot be honoured"):
        rx.compile_offline(fp8)
    monkeypatch.setenv("RX_GEMM_BK", "100")   # not a multiple of the MFMA k step
    with pytest.raises(rx.ReactantInternalError, match="multiple of the MFMA k step"):
        rx.compile_offline(fp8)
    monkeypatch.setenv("RX_GEMM_BK", "128")
    assert "kind=gemm_f8" in rx.compile_offline(fp8)
    monkeypatch.delenv("RX_GEMM_BK")
    monkeypatch.setenv("RX_GEMM_TILE", "96,96,2,2")
    with pytest.raises(rx.ReactantInternalError, match="32x32 blocks"):
        rx.compile_offline(fp8)


def test_gelu_chain_is_recognised_for_narrow_results(monkeypatch):
    """0.5 x (1 + tanh(a (x + b x^3))) in a bf16 program is evaluated as x / (1 + e^(...)) with folded constants; the
    f32 program, and a bf16 program that must round after every op, keep the chain."""
    P = load_programs()
    src = rx.compile_offline(P.mlp(64, (32, 64, 64, 32)), with_source=True)
    assert src.count("rx_gelu_chain_fast(") == 3 and "rx_tanh_fast" not in src
    src32 = rx.compile_offline(P.mlp(64, (32, 64, 64, 32), dt="f32"), with_source=True)
    assert "rx_gelu_chain_fast" not in src32 and "tanhf(" in src32
    monkeypatch.setenv("RX_EXCESS_PRECISION", "0")
    strict = rx.compile_offline(P.mlp(64, (32, 64, 64, 32)), with_source=True)
    assert "rx_gelu_chain_fast" not in strict


def test_gemm_takes_the_streaming_skeleton_where_it_fits(monkeypatch):
    # 8- and 16-bit operands on eight-wavefront tiles with whole K tiles of 128 bytes: the 16x16 MFMA skeleton that streams
    # one operand (with_source shows the call)
    big = P.fp8_linear(8192, 8192, 8192)
    # 256x256 tiles, an even number of K tiles, B stored [n][k]: the ping-pong form of those tiles; B stored [k][n]: the interleaved form
    assert "rx_gemm_body_pp<rx_el_f8, 256, 256, 2, 4, true, true, 8192, 8192, 8192" in rx.compile_offline(big, with_source=True)
    assert "rx_gemm_body_s<rx_el_f8, 256, 256, 2, 4, true, false, 8192, 8192, 8192" in rx.compile_offline(P.fp8_linear(8192, 8192, 8192, weight_layout="kn"), with_source=True)
    mlp = rx.compile_offline(P.mlp(8192, [1024, 4096, 4096, 1024]), with_source=True)
    # 16-bit operands on 256x256 tiles with an even number of K tiles: the ping-pong form of the same tiles
    assert "rx_gemm_body_pp<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 4096" in mlp     # the 4096^2 layer
    assert "rx_gemm_body_pp<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 1024" in mlp     # the first layer
    assert "rx_gemm_body_s<rx_el_bf16, 256, 128, 4, 2, true, false, 8192, 1024, 4096" in mlp      # the last layer: 256x128 tiles, wavefronts of 64x64
    monkeypatch.setenv("RX_GEMM_PINGPONG", "0")
    assert "rx_gemm_body_s<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 4096" in rx.compile_offline(P.mlp(8192, [1024, 4096, 4096, 1024]), with_source=True)
    assert "rx_gemm_body_s<rx_el_f8, 256, 256, 2, 4, true, true, 8192, 8192, 8192" in rx.compile_offline(big, with_source=True)
    monkeypatch.setenv("RX_GEMM_PINGPONG", "1")
    assert "rx_gemm_body_pp<rx_el_f8, 256, 256, 2, 4, true, false, 8192, 8192, 8192" in rx.compile_offline(P.fp8_linear(8192, 8192, 8192, weight_layout="kn"), with_source=True)
    monkeypatch.delenv("RX_GEMM_PINGPONG")
    # an odd number of K tiles (K = 64 * 65) stays with the interleaved form
    odd_kt = rx.compile_offline(_dot("tensor<8192x4160xbf16>", "tensor<4160x4096xbf16>", "tensor<8192x4096xf32>", "contracting_dims = [1] x [0]"), with_source=True)
    assert "rx_gemm_body_s<rx_el_bf16, 256, 256, 2, 4, true, false, 8192, 4096, 4160" in odd_kt
    monkeypatch.setenv("RX_GEMM_STREAM", "0")
    src = rx.compile_offline(big, with_source=True)
    assert "rx_gemm_body_s<" not in src and "rx_gemm_body_dl<rx_mma_f8, 256, 256, 128" in src
    monkeypatch.delenv("RX_GEMM_STREAM")
    # K = 8256 is whole 16-byte vectors but not whole K tiles of 128: not the direct-to-LDS skeletons
    odd = rx.compile_offline(P.fp8_linear(8192, 8256, 8192), with_source=True)
    assert "rx_gemm_body_s<" not in odd and "kind=gemm_f8" in odd
    # an operand of 4 GB or more is beyond the 32-bit buffer offsets of the streaming skeleton: the ring skeleton takes it
    huge = rx.compile_offline(_dot("tensor<65536x65536xf8E4M3FN>", "tensor<8192x65536xf8E4M3FN>", "tensor<65536x8192xf32>", "contracting_dims = [1] x [1]"),
                              with_source=True)
    assert "rx_gemm_body_s<" not in huge and "rx_gemm_body_dl<rx_mma_f8, 256, 256, 128" in huge
    below = rx.compile_offline(_dot("tensor<32768x65536xf8E4M3FN>", "tensor<8192x65536xf8E4M3FN>", "tensor<32768x8192xf32>", "contracting_dims = [1] x [1]"),
                               with_source=True)
    assert "rx_gemm_body_pp<rx_el_f8, 256, 256, 2, 4, true, true, 32768, 8192, 65536" in below
    # the 32x32 MFMA shapes are a request for the ring skeleton
    monkeypatch.setenv("RX_GEMM_MFMA32", "1")
    assert "rx_gemm_body_dl<rx_mma_bf16, 256, 256, 64" in rx.compile_offline(P.mlp(8192, [1024, 4096, 4096, 1024]), with_source=True)


def test_cost_analysis_counts_of_the_module(rx):
    """The counts behind RxExecutableCostAnalysis (the reference's cost_analysis, src/xla/Stats.jl:86-115), in the plan
    report: sum(sin.(x) .+ y) over n elements is n additions + n reduced elements, n transcendentals, and every op reads
    its operands and writes its result once; a product counts 2 M N K."""
    import re
    n = 1 << 16
    rep = rx.compile_offline(P.sinsum_add(n))
    m = re.search(r"module costs: flops=(\d+) transcendentals=(\d+) bytes_accessed=(\d+) output_bytes=(\d+)", rep)
    assert m, rep
    flops, trans, nbytes, out = map(int, m.groups())
    assert flops == 2 * n and trans == n and out == 4
    assert nbytes == (4 * n + 4 * n) + (8 * n + 4 * n) + (4 * n + 4 + 4)      # sine, add, reduce (operand + init + result)
    rep = rx.compile_offline(P.gemm(64, 128, 256))
    flops = int(re.search(r"module costs: flops=(\d+)", rep).group(1))
    assert flops == 2 * 64 * 128 * 256 + 3 * 64 * 128                            # the product, alpha, beta, the sum
