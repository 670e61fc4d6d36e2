"""The hand-off format of Reactant.Serialization.export_to_enzymejax (`<fn>_<id>.mlir` +
`<fn>_<id>_inputs.npz`) run on the GPU.  The two cases are the ones the reference tests
(test/integration/enzymejax.jl:20-104): `sin.(x) .+ cos.(x)` on construct_test_array(Float32, 4, 5)
and `x * y` for 3x4 by 4x5, both checked against the plain formula (atol = rtol = 1e-5 there)."""
import numpy as np
import pytest

from oracle import stablehlo_interp as I

pytestmark = pytest.mark.gpu


def construct_test_array(dtype, *dims):
    """Reactant.TestUtils.construct_test_array (src/TestUtils.jl:9-23), Julia (column-major) order."""
    n = int(np.prod(dims))
    return (np.arange(1, n + 1) / n).astype(dtype).reshape(dims, order="F")


def write_export(tmp_path, name, text, julia_arrays):
    """What export_to_enzymejax leaves in its output directory: the module text and the inputs with
    their dims reversed (ext/ReactantNPZExt.jl:9-22)."""
    mlir = tmp_path / ("%s_0.mlir" % name)
    mlir.write_text(text)
    np.savez(tmp_path / ("%s_0_inputs.npz" % name),
             **{"arr_%d" % (i + 1): np.ascontiguousarray(a.T) if np.ndim(a) else a for i, a in enumerate(julia_arrays)})
    return str(mlir)


F_SIMPLE = """module @reactant_f_simple attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<5x4xf32>) -> tensor<5x4xf32> {
    %0 = stablehlo.sine %arg0 : tensor<5x4xf32>
    %1 = stablehlo.cosine %arg0 : tensor<5x4xf32>
    %2 = stablehlo.add %0, %1 : tensor<5x4xf32>
    return %2 : tensor<5x4xf32>
  }
}
"""

MATMUL = """module @reactant_matmul attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<4x3xf32>, %arg1: tensor<5x4xf32>) -> tensor<5x3xf32> {
    %0 = stablehlo.dot_general %arg1, %arg0, contracting_dims = [1] x [0], precision = [DEFAULT, DEFAULT] : (tensor<5x4xf32>, tensor<4x3xf32>) -> tensor<5x3xf32>
    return %0 : tensor<5x3xf32>
  }
}
"""

SCALED = """module @reactant_scaled attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<3x2xi64>, %arg1: tensor<i64>) -> tensor<3x2xi64> {
    %0 = stablehlo.broadcast_in_dim %arg1, dims = [] : (tensor<i64>) -> tensor<3x2xi64>
    %1 = stablehlo.multiply %arg0, %0 : tensor<3x2xi64>
    return %1 : tensor<3x2xi64>
  }
}
"""


def test_exported_elementwise_function(rx, client, tmp_path):
    x = construct_test_array(np.float32, 4, 5)
    path = write_export(tmp_path, "f_simple", F_SIMPLE, [x])
    (res,) = rx.run_enzymejax_export(path, client=client)
    assert res.shape == (5, 4)
    np.testing.assert_allclose(res.T, np.sin(x.astype(np.float64)) + np.cos(x.astype(np.float64)), atol=1e-5, rtol=1e-5)
    # and the same bytes through the oracle
    ref = I.run_text(F_SIMPLE, [I.Tensor(np.ascontiguousarray(x.T), "f32")])
    np.testing.assert_allclose(res, ref[0].a, rtol=1e-6, atol=1e-7)


def test_exported_matmul(rx, client, tmp_path):
    x, y = construct_test_array(np.float32, 3, 4), construct_test_array(np.float32, 4, 5)
    path = write_export(tmp_path, "matmul", MATMUL, [x, y])
    (res,) = rx.run_enzymejax_export(path, client=client)
    np.testing.assert_allclose(res.T, x.astype(np.float64) @ y.astype(np.float64), atol=1e-5, rtol=1e-5)


def test_exported_function_with_a_number_argument(rx, client, tmp_path):
    x = np.arange(1, 7, dtype=np.int64).reshape((2, 3), order="F")
    path = write_export(tmp_path, "scaled", SCALED, [x, np.int64(-3)])
    (res,) = rx.run_enzymejax_export(path, client=client)
    assert res.dtype == np.int64 and np.array_equal(res.T, -3 * x)


def test_exported_inputs_of_the_wrong_shape_are_rejected(rx, client, tmp_path):
    x = construct_test_array(np.float32, 5, 4)          # not reversed
    path = write_export(tmp_path, "f_simple", F_SIMPLE, [x])
    with pytest.raises(rx.ReactantInternalError, match="executable expects"):
        rx.run_enzymejax_export(path, client=client)
