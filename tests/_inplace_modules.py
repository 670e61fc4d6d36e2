"""Modules in which a value that `dynamic_update_slice` overwrites is also read by a kernel that is
launched later than the reader's own position in the module: a product whose epilogue follows the
update, a row reduction fused into a kernel that follows it, and a stencil pair whose second step
follows it.  The update must not take over the buffer in any of them."""

_T = "tensor<64x64xf32>"

# the product reads `base`; its bias epilogue (where the product is launched) comes after the update
DOT_EPILOGUE_AFTER_UPDATE = """module {
  func.func @main(%a: T, %b: T, %w: T, %u: tensor<16x64xf32>, %bias: T) -> (T, T) {
    %c0 = stablehlo.constant dense<0> : tensor<i32>
    %base = stablehlo.add %a, %b : T
    %d = stablehlo.dot_general %base, %w, contracting_dims = [1] x [0] : (T, T) -> T
    %r = stablehlo.dynamic_update_slice %base, %u, %c0, %c0 : (T, tensor<16x64xf32>, tensor<i32>, tensor<i32>) -> T
    %e = stablehlo.add %d, %bias : T
    return %r, %e : T, T
  }
}
""".replace("T", _T)

# the row sum of `base` is computed inside the kernel of the division, which comes after the update
ROW_REDUCE_AFTER_UPDATE = """module {
  func.func @main(%a: T, %b: T, %u: tensor<16x64xf32>, %o: T) -> (T, T) {
    %c0 = stablehlo.constant dense<0> : tensor<i32>
    %z = stablehlo.constant dense<0.0> : tensor<f32>
    %base = stablehlo.dot_general %a, %b, contracting_dims = [1] x [0] : (T, T) -> T
    %m = stablehlo.reduce(%base init: %z) applies stablehlo.add across dimensions = [1] : (T, tensor<f32>) -> tensor<64xf32>
    %r = stablehlo.dynamic_update_slice %base, %u, %c0, %c0 : (T, tensor<16x64xf32>, tensor<i32>, tensor<i32>) -> T
    %mb = stablehlo.broadcast_in_dim %m, dims = [0] : (tensor<64xf32>) -> T
    %e = stablehlo.divide %o, %mb : T
    return %r, %e : T, T
  }
}
""".replace("T", _T)

# the same update with every reader of `base` launched before it: this one may work in place
UPDATE_AFTER_ALL_READERS = """module {
  func.func @main(%a: T, %b: T, %w: T, %u: tensor<16x64xf32>, %bias: T) -> (T, T) {
    %c0 = stablehlo.constant dense<0> : tensor<i32>
    %base = stablehlo.add %a, %b : T
    %d = stablehlo.dot_general %base, %w, contracting_dims = [1] x [0] : (T, T) -> T
    %e = stablehlo.add %d, %bias : T
    %r = stablehlo.dynamic_update_slice %base, %u, %c0, %c0 : (T, tensor<16x64xf32>, tensor<i32>, tensor<i32>) -> T
    return %r, %e : T, T
  }
}
""".replace("T", _T)

CASES = {"dot_epilogue_after_update": (DOT_EPILOGUE_AFTER_UPDATE, 5, [(64, 64)] * 3 + [(16, 64), (64, 64)]),
         "row_reduce_after_update": (ROW_REDUCE_AFTER_UPDATE, 4, [(64, 64)] * 2 + [(16, 64), (64, 64)]),
         "update_after_all_readers": (UPDATE_AFTER_ALL_READERS, 5, [(64, 64)] * 3 + [(16, 64), (64, 64)])}
