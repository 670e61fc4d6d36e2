"""StableHLO text of small `stablehlo.while` loops shared by the CPU and GPU tests."""

# The example in the docstring of the reference's binding (src/mlir/Dialects/StableHLO.jl:4850-4861):
# count to ten, adding one to a second value each time.
COUNT = """module { func.func @main(%init_i: tensor<i64>, %init_sum: tensor<i64>) -> (tensor<i64>, tensor<i64>) {
  %one = stablehlo.constant dense<1> : tensor<i64>
  %ten = stablehlo.constant dense<10> : tensor<i64>
  %results0, %results1 = stablehlo.while(%arg0 = %init_i, %arg1 = %init_sum) : tensor<i64>, tensor<i64>
  cond {
    %cond = stablehlo.compare LT, %arg0, %ten : (tensor<i64>, tensor<i64>) -> tensor<i1>
    stablehlo.return %cond : tensor<i1>
  } do {
    %new_sum = stablehlo.add %arg1, %one : tensor<i64>
    %new_i = stablehlo.add %arg0, %one : tensor<i64>
    stablehlo.return %new_i, %new_sum : tensor<i64>, tensor<i64>
  }
  return %results0, %results1 : tensor<i64>, tensor<i64>
} }"""

# x[i] += 2i for i in 1:4, the in-place `setindex!` of a traced loop (src/Indexing.jl:438-443):
# the loop counter is the start index of a dynamic_slice / dynamic_update_slice pair.
SETINDEX = """module { func.func @main(%x: tensor<4xi64>) -> tensor<4xi64> {
  %c0 = stablehlo.constant dense<0> : tensor<i64>
  %c1 = stablehlo.constant dense<1> : tensor<i64>
  %c4 = stablehlo.constant dense<4> : tensor<i64>
  %c2 = stablehlo.constant dense<2> : tensor<i64>
  %r:2 = stablehlo.while(%iterArg = %c0, %iterArg_0 = %x) : tensor<i64>, tensor<4xi64>
   cond {
    %p = stablehlo.compare  LT, %iterArg, %c4,  SIGNED : (tensor<i64>, tensor<i64>) -> tensor<i1>
    stablehlo.return %p : tensor<i1>
  } do {
    %n = stablehlo.add %iterArg, %c1 : tensor<i64>
    %v = stablehlo.multiply %n, %c2 : tensor<i64>
    %s = stablehlo.dynamic_slice %iterArg_0, %iterArg, sizes = [1] : (tensor<4xi64>, tensor<i64>) -> tensor<1xi64>
    %vb = stablehlo.reshape %v : (tensor<i64>) -> tensor<1xi64>
    %w = stablehlo.add %s, %vb : tensor<1xi64>
    %u = stablehlo.dynamic_update_slice %iterArg_0, %w, %iterArg : (tensor<4xi64>, tensor<1xi64>, tensor<i64>) -> tensor<4xi64>
    stablehlo.return %n, %u : tensor<i64>, tensor<4xi64>
  }
  return %r#1 : tensor<4xi64>
} }"""

# generic form: three doublings of a vector, counter returned as well
GENERIC = """module { func.func @main(%x: tensor<4xf32>) -> (tensor<i64>, tensor<4xf32>) {
  %c0 = "stablehlo.constant"() {value = dense<0> : tensor<i64>} : () -> tensor<i64>
  %c1 = "stablehlo.constant"() {value = dense<1> : tensor<i64>} : () -> tensor<i64>
  %c3 = "stablehlo.constant"() {value = dense<3> : tensor<i64>} : () -> tensor<i64>
  %r:2 = "stablehlo.while"(%c0, %x) ({
  ^bb0(%a: tensor<i64>, %b: tensor<4xf32>):
    %p = "stablehlo.compare"(%a, %c3) {comparison_direction = #stablehlo<comparison_direction LT>} : (tensor<i64>, tensor<i64>) -> tensor<i1>
    "stablehlo.return"(%p) : (tensor<i1>) -> ()
  }, {
  ^bb0(%a: tensor<i64>, %b: tensor<4xf32>):
    %n = "stablehlo.add"(%a, %c1) : (tensor<i64>, tensor<i64>) -> tensor<i64>
    %m = "stablehlo.add"(%b, %b) : (tensor<4xf32>, tensor<4xf32>) -> tensor<4xf32>
    "stablehlo.return"(%n, %m) : (tensor<i64>, tensor<4xf32>) -> ()
  }) : (tensor<i64>, tensor<4xf32>) -> (tensor<i64>, tensor<4xf32>)
  return %r#0, %r#1 : tensor<i64>, tensor<4xf32>
} }"""

# a trip count read from the data: not a static loop
DATA_DEPENDENT = """module { func.func @main(%x: tensor<4xi64>, %n: tensor<i64>) -> tensor<4xi64> {
  %c0 = stablehlo.constant dense<0> : tensor<i64>
  %c1 = stablehlo.constant dense<1> : tensor<i64>
  %r:2 = stablehlo.while(%iterArg = %c0, %iterArg_0 = %x) : tensor<i64>, tensor<4xi64>
   cond {
    %p = stablehlo.compare  LT, %iterArg, %n,  SIGNED : (tensor<i64>, tensor<i64>) -> tensor<i1>
    stablehlo.return %p : tensor<i1>
  } do {
    %i = stablehlo.add %iterArg, %c1 : tensor<i64>
    %u = stablehlo.add %iterArg_0, %iterArg_0 : tensor<4xi64>
    stablehlo.return %i, %u : tensor<i64>, tensor<4xi64>
  }
  return %r#1 : tensor<4xi64>
} }"""

# scalar `setindex!` / `getindex` on a device array (src/ConcreteRArray.jl:423-446): Julia a is 3x4,
# the indices arrive as 1-based numbers, the module works on the dim-reversed 4x3 tensor
SETINDEX_SCALAR = """module @reactant_mysetindex attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<4x3xf64> {tf.aliasing_output = 0 : i32}, %arg1: tensor<f64>, %arg2: tensor<i64>, %arg3: tensor<i64>) -> tensor<4x3xf64> {
    %c = stablehlo.constant dense<1> : tensor<i64>
    %0 = stablehlo.subtract %arg2, %c : tensor<i64>
    %1 = stablehlo.subtract %arg3, %c : tensor<i64>
    %2 = stablehlo.reshape %arg1 : (tensor<f64>) -> tensor<1x1xf64>
    %3 = stablehlo.dynamic_update_slice %arg0, %2, %1, %0 : (tensor<4x3xf64>, tensor<1x1xf64>, tensor<i64>, tensor<i64>) -> tensor<4x3xf64>
    return %3 : tensor<4x3xf64>
  }
}"""
GETINDEX_BLOCK = """module @reactant_getblock attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<4x3xf64>, %arg1: tensor<i32>, %arg2: tensor<i32>) -> tensor<2x2xf64> {
    %0 = stablehlo.dynamic_slice %arg0, %arg2, %arg1, sizes = [2, 2] : (tensor<4x3xf64>, tensor<i32>, tensor<i32>) -> tensor<2x2xf64>
    return %0 : tensor<2x2xf64>
  }
}"""
FILL = """module @reactant_fill attributes {mhlo.num_partitions = 1 : i64, mhlo.num_replicas = 1 : i64} {
  func.func @main(%arg0: tensor<4x3xf32> {tf.aliasing_output = 0 : i32}, %arg1: tensor<f32>) -> tensor<4x3xf32> {
    %0 = stablehlo.broadcast_in_dim %arg1, dims = [] : (tensor<f32>) -> tensor<4x3xf32>
    return %0 : tensor<4x3xf32>
  }
}"""


# `@trace if` (reference src/Ops.jl:2449-2470, 2838): both regions see the enclosing values
IF = """module {
  func.func @main(%arg0: tensor<8xf32>, %arg1: tensor<f32>) -> (tensor<8xf32>, tensor<f32>) {
    %z = stablehlo.constant dense<0.000000e+00> : tensor<f32>
    %p = stablehlo.compare GT, %arg1, %z : (tensor<f32>, tensor<f32>) -> tensor<i1>
    %0:2 = "stablehlo.if"(%p) ({
      %1 = stablehlo.sine %arg0 : tensor<8xf32>
      %one = stablehlo.constant dense<1.000000e+00> : tensor<f32>
      stablehlo.return %1, %one : tensor<8xf32>, tensor<f32>
    }, {
      %b = stablehlo.broadcast_in_dim %arg1, dims = [] : (tensor<f32>) -> tensor<8xf32>
      %2 = stablehlo.multiply %arg0, %b : tensor<8xf32>
      %3 = stablehlo.negate %arg1 : tensor<f32>
      stablehlo.return %2, %3 : tensor<8xf32>, tensor<f32>
    }) : (tensor<i1>) -> (tensor<8xf32>, tensor<f32>)
    return %0#0, %0#1 : tensor<8xf32>, tensor<f32>
  }
}
"""

# `stablehlo.case` (src/Ops.jl:2890-3210): three branches on an i32 index; out-of-range indices take the last one
CASE = """module {
  func.func @main(%arg0: tensor<4x5xf64>, %arg1: tensor<i32>) -> tensor<4x5xf64> {
    %0 = "stablehlo.case"(%arg1) ({
      %1 = stablehlo.exponential %arg0 : tensor<4x5xf64>
      stablehlo.return %1 : tensor<4x5xf64>
    }, {
      %2 = stablehlo.multiply %arg0, %arg0 : tensor<4x5xf64>
      stablehlo.return %2 : tensor<4x5xf64>
    }, {
      %3 = stablehlo.negate %arg0 : tensor<4x5xf64>
      stablehlo.return %3 : tensor<4x5xf64>
    }) : (tensor<i32>) -> tensor<4x5xf64>
    return %0 : tensor<4x5xf64>
  }
}
"""

# a predicate that is a constant selects its branch while the module is imported
IF_CONST = """module {
  func.func @main(%arg0: tensor<8xf32>) -> tensor<8xf32> {
    %p = stablehlo.constant dense<false> : tensor<i1>
    %0 = "stablehlo.if"(%p) ({
      %1 = stablehlo.sine %arg0 : tensor<8xf32>
      stablehlo.return %1 : tensor<8xf32>
    }, {
      %2 = stablehlo.cosine %arg0 : tensor<8xf32>
      stablehlo.return %2 : tensor<8xf32>
    }) : (tensor<i1>) -> tensor<8xf32>
    return %0 : tensor<8xf32>
  }
}
"""
