// Expression emitter: writes HIP text that evaluates a fused cone of StableHLO
// nodes at one symbolic index.  Index-transforming ops (slice, pad, broadcast,
// transpose, reshape, dynamic_update_slice, concatenate) become index arithmetic
// on the producer side, so a stencil written as a slice/pad/add chain turns into
// loads at constant offsets from the output index.
#pragma once
#include <functional>
#include <map>
#include <set>
#include <sstream>

#include "rx_ir.h"

namespace rx {

// One index component: value = var + off (var empty -> constant `off`), known to lie in [lo, hi].
struct Ix {
  std::string var;
  int64_t off = 0;
  int64_t lo = 0, hi = 0;
  // `var` is known to be a multiple of `align` (the first lane of a vector of `align` consecutive elements, off = lane):
  // a reshape then splits var alone and adds the lane to the innermost component, so the divisions are shared by the lanes
  int64_t align = 1;
  bool is_const() const { return var.empty(); }
  std::string str() const;
  std::string key() const { return var + "+" + std::to_string(off) + (align > 1 ? "@" + std::to_string(align) : ""); }
};
using Index = std::vector<Ix>;

struct LoadRecord {
  int node;                     // materialized node that is read
  std::vector<int64_t> off;     // constant offsets relative to the root index (valid if `affine`)
  bool affine = false;          // index is root identity + constant offsets
  // per input dimension: which root variable indexes it with offset 0 (-1: anything else).  A
  // permutation of the root variables that is not the identity marks a transposed read.
  std::vector<int> root_var;
  bool minor_follows = false;   // the input's minor dimension is indexed by the root's minor variable (any offset)
  std::vector<int64_t> root_off;   // with root_var: constant offset of every input dimension's index (offset_perms)
};

class Emitter {
 public:
  Emitter(const Graph& g, std::function<bool(int)> is_input) : g_(g), is_input_(std::move(is_input)) {}

  // kernel parameter order of inputs, filled as loads are emitted
  std::vector<int> inputs;
  std::map<int, std::string> bound;          // node id -> expression already in scope
  std::vector<LoadRecord> loads;
  bool idx64 = false;
  int indent = 2;

  // direct (vectorizable) loads: root dims + names of the root index variables
  void set_root(const std::vector<int64_t>& dims, const std::vector<std::string>& vars, bool allow_direct) {
    root_dims_ = dims;
    root_vars_ = vars;
    allow_direct_ = allow_direct;
  }
  // Vector preloads.  (slot, D): the aligned vector of input `slot` at element offset D from the
  // vector of the output element; D != 0 arises from loads at constant offsets (stencils) and is
  // only produced when `allow_shifted` is set.  `direct_expr(slot, D)` names the preloaded vector.
  std::set<std::pair<int, int64_t>> direct_vecs;
  std::function<std::string(int slot, int64_t D)> direct_expr;
  bool allow_shifted = false;
  int vec = 1;
  // Arithmetic on bf16/f16/f8 tensors is carried in f32 inside a kernel and rounded once, when a
  // value is stored or explicitly converted (what XLA does under its default
  // xla_allow_excess_precision).  With this off every op result is rounded to its element type.
  bool excess_precision = true;
  // Loads of an input at root-index + constant offsets can be redirected (to an LDS halo tile):
  // the hook returns true and the expression to read instead of global memory.
  std::function<bool(int slot, const std::vector<int64_t>& off, std::string* expr)> tile_hook;
  // Loads whose index is a non-identity permutation of the root variables (a transposed read) can
  // be redirected too; `root_var[d]` is the root variable that indexes input dimension d.
  std::function<bool(int slot, const std::vector<int>& root_var, std::string* expr)> perm_hook;

  // pad / dynamic_update_slice guards: when everything read under a guard comes from a tile or a
  // preloaded vector (so evaluating it at a point the guard excludes cannot fault), evaluate both
  // sides and select, instead of branching per element
  bool branchless_guards = false;
  bool offset_perms = false;   // a transposed read may carry constant offsets and read an input of other extents (a padded or sliced transpose)
  bool const_vectors = false;  // vectors and scalars are read through the constant address space (nothing in the kernel writes them): equal reads merge across stores
  bool columns_reused = false; // the code runs for many rows of the same columns in one thread (a product's epilogue): values that vary along the minor dimension only are computed once
  bool clamp_guards = false;   // pad: read at positions clamped into the operand and select, instead of a branch around the read

  std::string emit(int node, const Index& ix);
  std::string take_code() { std::string s = out_.str(); out_.str(""); return s; }
  void line(const std::string& s) { out_ << std::string(indent, ' ') << s << "\n"; }
  int slot_of(int node);
  std::string load_conv(DT dt, const std::string& raw) const;          // storage -> compute
  static std::string store_conv(DT dt, const std::string& val);        // compute -> storage
  // same, for a value this emitter produced: a value that was just rounded to `dt` is converted
  // from its unrounded form (one conversion instead of round-trip plus conversion)
  std::string store_value(DT dt, const std::string& val) const;
  static std::string literal(const Node& n);
  static std::string round_narrow(DT dt, const std::string& e);
  std::string idx_t() const { return idx64 ? "long long" : "int"; }
  std::string fresh(const char* p = "v") { return std::string(p) + std::to_string(tmp_++); }
  void push_scope() { scopes_.emplace_back(); }
  void pop_scope() { scopes_.pop_back(); }
  std::string linear(const Index& ix, const std::vector<int64_t>& dims) const;
  bool minor_uniform(int node, int depth = 0) const;   // the value does not vary along the node's last dimension

 private:
  const Graph& g_;
  std::function<bool(int)> is_input_;
  std::ostringstream out_;
  std::vector<std::map<std::string, std::string>> scopes_{1};
  int tmp_ = 0;
  std::map<std::string, std::pair<DT, std::string>> rounded_;   // variable -> (type it was rounded to, unrounded expression)
  std::set<std::string> e4m3_range_;   // float values known to lie in [-448, 448] (or to be NaN)
  int unsafe_loads_ = 0;   // loads emitted as plain global reads at a computed index
  std::vector<int64_t> root_dims_;
  std::vector<std::string> root_vars_;
  bool allow_direct_ = false;

  bool is_uniform(int node, int depth = 0) const;
  bool minor_only(int node, int depth = 0) const;   // the value varies along the minor dimension at most
  std::string emit_load(int node, const Index& ix);
  std::string emit_op(const Node& n, const Index& ix);
  bool match_gelu_chain(const Node& n, int* xnode, double* ka, double* kb) const;
  bool lookup(const std::string& key, std::string* out) const;
  Ix temp_index(const std::string& expr, int64_t lo, int64_t hi);
};

}  // namespace rx
