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
