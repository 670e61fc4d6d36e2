"""The importer, the fusion planner, the code generator and the GEMM chooser under AddressSanitizer and
UndefinedBehaviorSanitizer, as a host-only program (reactant.jl_amd/csrc/rx_hostcheck.cpp, built by
`python reactant.jl_amd/build.py --sanitize`).  The corpus is the module text of every program builder of the
package (the five benchmark programs at small and full sizes, the polybench suites, the windowed / NN programs),
the hand-written modules of the CPU tests, and modules that must be rejected with a message.  Skipped when the
sanitizer program has not been built (the build takes about a minute)."""
import importlib
import os
import subprocess

import pytest

from _loader import load_pkg, load_programs, ROOT
import _while_modules as W
import _inplace_modules as M

load_pkg()
P = load_programs()
NN = importlib.import_module("reactant_jl_amd.nn_programs")
PB = importlib.import_module("reactant_jl_amd.polybench_programs")
HOSTCHECK = os.path.join(ROOT, "reactant.jl_amd", "csrc", "build", "rx_hostcheck_asan")


def corpus():
    mods = {
        "sinsum_small": P.sinsum_add(4096), "sinsum_full": P.sinsum_add(1 << 26),
        "stencil_small": P.stencil(20, 12, 9, steps=3), "stencil_dus": P.stencil(16, 16, 8, steps=2, embed="dus"),
        "stencil_while": P.stencil(32, 16, 8, steps=4, loop="while"), "stencil_full": P.stencil(512, 512, 256, steps=10),
        "gemm_small": P.gemm(64, 48, 32), "gemm_transposed": P.gemm(128, 256, 64, form="transposed"), "gemm_full": P.gemm(4096, 4096, 4096),
        "mlp_small": P.mlp(8, (16, 32, 32, 16)), "mlp_op": P.mlp(64, (32, 64, 64, 32), gelu="op"), "mlp_full": P.mlp(8192, (1024, 4096, 4096, 1024)),
        "fp8_small": P.fp8_linear(8, 32, 16), "fp8_kn": P.fp8_linear(128, 256, 128, weight_layout="kn"),
        "fp8_direct": P.fp8_linear(8, 32, 16, weight_layout="kn", dot_form="direct"), "fp8_full": P.fp8_linear(8192, 8192, 8192),
        "cumsum": NN.cumulative([1 << 20], "f32", 0), "cumsum_rows": NN.cumulative([512, 384], "f32", 1, reverse=True),
        "cumsum_long": NN.cumulative([1 << 26], "f32", 0), "cumsum_long_rows": NN.cumulative([3, 9000000], "i64", 1),
        "transpose": "module { func.func @main(%a: tensor<520x264xf64>) -> tensor<264x520xf64> { %0 = stablehlo.transpose %a, dims = [1, 0] : "
                     "(tensor<520x264xf64>) -> tensor<264x520xf64>\n return %0 : tensor<264x520xf64> } }",
        "transpose_batched": "module { func.func @main(%a: tensor<5x1000x72xf32>) -> tensor<5x72x1000xf32> { %0 = stablehlo.transpose %a, dims = [0, 2, 1] : "
                             "(tensor<5x1000x72xf32>) -> tensor<5x72x1000xf32>\n return %0 : tensor<5x72x1000xf32> } }",
        "stencil_edge": P.stencil(134, 70, 9, steps=2), "stencil_edge_f32": P.stencil(390, 20, 12, steps=3, elt="f32"),
        "maxpool": NN.reduce_window([4, 8, 32, 32], "f32", "maximum", [1, 1, 2, 2], strides=[1, 1, 2, 2])[0],
        "conv": NN.convolution([2, 8, 16, 16], [4, 8, 3, 3], "f32", padding=[[1, 1], [1, 1]])[0],
        "conv_groups": NN.convolution([2, 8, 16, 16], [4, 4, 3, 3], "f32", groups=2)[0],
        "conv_direct": NN.convolution([32, 64, 56, 56], [64, 64, 3, 3], "f32", padding=[[1, 1], [1, 1]], epilogue="bias_relu")[0],
        "conv_shifted": NN.convolution([32, 256, 56, 56], [256, 256, 3, 3], "bf16", padding=[[1, 1], [1, 1]], epilogue="bias_relu")[0],
        "conv_shifted_small": NN.convolution([2, 20, 16, 64], [3, 3, 64, 128], "f16", padding=[[1, 0], [2, 1]], rhs_dil=[1, 2], dims="[b, 0, 1, f]x[0, 1, i, o]->[b, 0, 1, f]")[0],
        "vgg": NN.vgg_block(), "attention": NN.attention_block(),
        "conv_chain": NN.conv_chain(32, 256, 56, 3, "bf16")[0], "vgg11_f32": NN.vgg11(batch=4, dt="f32")[0], "vgg11_bf16": NN.vgg11(batch=32, dt="bf16")[0],
        "resnet_stage": NN.resnet_stage(batch=32, channels=128, hw=28, blocks=3, dt="bf16")[0], "resnet_stage_f32": NN.resnet_stage(batch=2, channels=64, hw=16, blocks=2, dt="f32")[0],
        "vgg11_small": NN.vgg11(batch=4, hw=64, classes=10, dt="f16", layers=(64, "M", 64, "M", 64, 64, "M", 64, 64, "M", 64, 64, "M"), dense=96)[0],
        "argmax": NN.argreduce([64, 100], "f32", 1),
        "pool_grad": NN.select_and_scatter([2, 4, 16, 16], "f32", [1, 1, 2, 2], strides=[1, 1, 2, 2]),
        "while_setindex": W.SETINDEX, "while_generic": W.GENERIC, "setindex_scalar": W.SETINDEX_SCALAR,
        "getindex_block": W.GETINDEX_BLOCK, "fill": W.FILL, "if": W.IF, "case": W.CASE, "if_const": W.IF_CONST,
        "inplace_dot": M.DOT_EPILOGUE_AFTER_UPDATE, "inplace_row": M.ROW_REDUCE_AFTER_UPDATE, "inplace_ok": M.UPDATE_AFTER_ALL_READERS,
    }
    for name in ("jacobi_1d", "jacobi_2d", "heat_3d", "fdtd_2d"):
        sz = dict(PB.POLYBENCH_SIZES[name])
        for key in ("tsteps", "tmax"):
            if key in sz:
                sz[key] = 24
        mods["polybench_" + name] = PB.build(name, **sz)
    for name in PB.LINALG_SIZES:
        mods["linalg_" + name] = PB.linalg(name, **{k: max(8, v // 8) for k, v in PB.LINALG_SIZES[name].items()})[0]
    rejected = {
        "reject_data_dependent_while": W.DATA_DEPENDENT, "reject_while_runtime_init": W.COUNT,
        "reject_sort": "module { func.func @main(%a: tensor<8xf32>) -> tensor<8xf32> {\n %0 = \"stablehlo.sort\"(%a) ({\n ^bb0(%x: tensor<f32>, %y: tensor<f32>):\n"
                       "  %c = stablehlo.compare LT, %x, %y : (tensor<f32>, tensor<f32>) -> tensor<i1>\n  stablehlo.return %c : tensor<i1>\n }) {dimension = 0 : i64} : (tensor<8xf32>) -> tensor<8xf32>\n"
                       " return %0 : tensor<8xf32> } }",
        "reject_truncated": P.mlp(8, (16, 32, 32, 16))[:700],
        "reject_shape_mismatch": P.gemm(64, 48, 32).replace("tensor<32x64xf32>", "tensor<31x64xf32>", 1),
        "reject_empty": "",
    }
    return mods, rejected


@pytest.mark.skipif(not os.path.exists(HOSTCHECK), reason="sanitizer program not built (python reactant.jl_amd/build.py --sanitize)")
def test_importer_and_planner_are_clean_under_asan_and_ubsan(tmp_path):
    mods, rejected = corpus()
    files = []
    for name, text in mods.items():
        f = tmp_path / (name + ".mlir")
        f.write_text(text if isinstance(text, str) else text[0])   # some builders return (text, shapes)
        files.append(str(f))
    for name, text in rejected.items():
        f = tmp_path / (name + ".mlir")
        f.write_text("// expect-error\n" + text)
        files.append(str(f))
    # once with the default plan options, once with the optional one-launch reductions and scans
    for extra in ({}, {"RX_SINGLE_PASS_REDUCE": "1", "RX_SINGLE_PASS_SCAN": "1"}):
        env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1", **extra)
        r = subprocess.run([HOSTCHECK] + files, capture_output=True, text=True, timeout=900, env=env)
        report = r.stdout[-3000:] + "\n" + r.stderr[-6000:]
        assert "AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr and "LeakSanitizer" not in r.stderr, report
        assert r.returncode == 0, report
        assert r.stdout.count("launches") == len(mods) and r.stdout.count("rejected as expected") == len(rejected), report
