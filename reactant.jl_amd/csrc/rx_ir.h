// Graph form of the StableHLO subset that the backend executes, and the parser
// from MLIR text (what `string(mod)` prints on the Julia side, reference
// src/compiler/Compiler.jl:1318-1321) into it.
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace rx {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Element types.  `code` is the value used on the wire by the reference
// (xla::PrimitiveType, src/xla/Utils.jl:18-40).
enum class DT : uint8_t { I1, I8, I16, I32, I64, U8, U16, U32, U64, F16, BF16, F32, F64, F8E4M3FN, F8E5M2, INVALID };

struct DTInfo {
  const char* mlir;     // element type spelling in MLIR text
  int code;             // xla::PrimitiveType
  int size;             // bytes in a buffer
  const char* ctype;    // type values are computed in inside kernels
  const char* stype;    // type values are stored as in buffers
  bool is_float;
  bool is_signed;
};
const DTInfo& info(DT t);
DT dt_from_mlir(const std::string& s);
DT dt_from_code(int code);
inline bool is_float(DT t) { return info(t).is_float; }
inline bool is_narrow_float(DT t) { return t == DT::F16 || t == DT::BF16 || t == DT::F8E4M3FN || t == DT::F8E5M2; }

struct TType {
  DT dt = DT::INVALID;
  std::vector<int64_t> dims;
  int64_t numel() const {
    int64_t n = 1;
    for (auto d : dims) n *= d;
    return n;
  }
  int64_t bytes() const { return numel() * info(dt).size; }
  int rank() const { return (int)dims.size(); }
  bool operator==(const TType& o) const { return dt == o.dt && dims == o.dims; }
  std::string str() const;
};

enum class OpK : uint8_t {
  Param, Constant, Iota,
  Unary, Binary, Compare, Select, Clamp, Convert, Gelu,
  BroadcastInDim, Reshape, Transpose, Slice, Pad, DynamicUpdateSlice, DynamicSlice, Concatenate,
  Reverse, Window, Gather,
  Reduce, DotGeneral, Scan, Scatter, Conv,
};

enum class Red : uint8_t { Add, Mul, Max, Min, And, Or };

struct Node {
  int id = -1;
  OpK k = OpK::Param;
  std::string op;             // short op name: "sine", "add", "GT", gelu approximation, ...
  TType ty;
  std::vector<int> in;        // operand node ids
  // integer attributes; meaning depends on the op
  //   BroadcastInDim: a0 = broadcast dims            Transpose: a0 = permutation
  //   Slice: a0/a1/a2 = start/limit/stride           Pad: a0/a1/a2 = low/high/interior
  //   DynamicSlice: a0 = sizes                       Concatenate, Iota: a0[0] = dimension
  //   Reduce: a0 = dimensions                        Param: a0[0] = argument index
  //   DotGeneral: a0/a1 = lhs/rhs batching, a2/a3 = lhs/rhs contracting
  //   Reverse: a0 = dimensions
  //   Window (rank r -> 2r): a0/a1/a2 = window sizes/strides/dilations;
  //       out[k_0..k_{r-1}, o_0..o_{r-1}] = in[o_i * stride_i + k_i * dilation_i]
  //   Gather (operand, start_indices): a0 = offset_dims, a1 = collapsed_slice_dims, a2 = start_index_map,
  //       a3 = slice_sizes, a4[0] = index_vector_dim, a5 = operand_batching_dims, a6 = start_indices_batching_dims
  //   Scatter (operand, scatter_indices, updates): a0 = update_window_dims, a1 = inserted_window_dims,
  //       a2 = scatter_dims_to_operand_dims, a4[0] = index_vector_dim, a5 = input_batching_dims,
  //       a6 = scatter_indices_batching_dims; op = "assign", "subtract", "divide" or "combine" (then `red` is the monoid)
  //   Scan (inclusive prefix combine with `red`): a0[0] = dimension, a1[0] = 1 if it runs from the end
  //   Conv (image [B, C, H, W], filter [O, C, KH, KW]) -> [B, O, HO, WO]: zero padding a0 = {rows before, rows after,
  //       columns before, columns after}, a1 = strides, a2 = filter dilations (the direct-convolution kernel's operation)
  //   Conv with a3 = {KW, SY, SX, HP, WP} (product with row shifts): operands [M, C] with M = B * HP * WP (or [B, HP, WP, C]) and
  //       [O, taps * C]; p[m][o] = sum over taps t = (ty, tx), tx < KW, and c of in0[m + ty * SY + tx * SX][c] * in1[o][t * C + c]
  //       (rows beyond M read as zeros): a unit-stride convolution of zero-padded [image, row, column, channel] data on
  //       the padded grid; the result [B, HO, WO, O] keeps p at m = (b * HP + y) * WP + x for y < HO, x < WO
  //       with a3 = {KW, SY, SX, HP, WP, HO, WO, shift} the result is [B, HP, WP, O]: row m of p, zero where it is not a
  //       result, at row m + shift, and zeros in the rows before `shift` (the next such product's zero-padded operand)
  std::vector<int64_t> a0, a1, a2, a3, a4, a5, a6;
  Red red = Red::Add;
  // Constant payload: either one splat element or dense bytes in storage format
  bool splat = false;
  std::vector<uint8_t> data;  // splat: one element; dense: ty.bytes()
  bool cmp_unsigned = false;
};

struct Graph {
  std::string name;
  std::string module_name;            // symbol of the module ("reactant_<fn>" in what Reactant prints), may be empty
  std::vector<Node> nodes;            // topologically ordered
  std::vector<int> params;            // node ids of @main arguments
  std::vector<int> results;           // node ids returned
  std::vector<int> aliasing_output;   // per argument: result index it may alias, or -1
  int add(Node n) {
    n.id = (int)nodes.size();
    nodes.push_back(std::move(n));
    return nodes.back().id;
  }
};

// Parse a module; functions called from @main are inlined.  Throws rx::Error.
Graph parse_module(const char* text, size_t len);

// Constant payload helpers
double splat_as_double(const Node& n);
int64_t splat_as_int(const Node& n);

}  // namespace rx
