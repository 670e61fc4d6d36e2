#include "rx_emit.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace rx {

std::string Ix::str() const {
  if (var.empty()) return std::to_string(off);
  if (off == 0) return var;
  if (off > 0) return "(" + var + " + " + std::to_string(off) + ")";
  return "(" + var + " - " + std::to_string(-off) + ")";
}

static Ix const_ix(int64_t v) {
  Ix i;
  i.off = v;
  i.lo = i.hi = v;
  return i;
}

static Ix shifted(const Ix& a, int64_t d) {
  Ix r = a;
  r.off += d;
  r.lo += d;
  r.hi += d;
  return r;
}

bool Emitter::lookup(const std::string& key, std::string* out) const {
  for (auto it = scopes_.rbegin(); it != scopes_.rend(); ++it) {
    auto f = it->find(key);
    if (f != it->end()) {
      *out = f->second;
      return true;
    }
  }
  return false;
}

int Emitter::slot_of(int node) {
  for (size_t k = 0; k < inputs.size(); ++k)
    if (inputs[k] == node) return (int)k;
  inputs.push_back(node);
  return (int)inputs.size() - 1;
}

std::string Emitter::linear(const Index& ix, const std::vector<int64_t>& dims) const {
  int64_t stride = 1, c = 0;
  std::vector<std::string> terms;
  for (int d = (int)dims.size() - 1; d >= 0; --d) {
    c += ix[d].off * stride;
    if (!ix[d].var.empty() && dims[d] > 1) {
      std::string v = idx64 ? "(long long)" + ix[d].var : ix[d].var;
      terms.push_back(stride == 1 ? v : v + " * " + std::to_string(stride) + (idx64 ? "LL" : ""));
    } else if (!ix[d].var.empty()) {
      // dimension of size 1: index is 0 whatever the variable says (range-checked by the caller)
      c -= ix[d].off * stride;
    }
    stride *= dims[d];
  }
  std::string s;
  for (auto& t : terms) s += (s.empty() ? "" : " + ") + t;
  if (s.empty()) return std::to_string(c) + (idx64 ? "LL" : "");
  if (c > 0) s += " + " + std::to_string(c) + (idx64 ? "LL" : "");
  if (c < 0) s += " - " + std::to_string(-c) + (idx64 ? "LL" : "");
  return s;
}

std::string Emitter::load_conv(DT dt, const std::string& raw) const {
  switch (dt) {
    case DT::BF16: return "rx_bf16_to_f32(" + raw + ")";
    case DT::F16: return "rx_f16_to_f32(" + raw + ")";
    case DT::F8E4M3FN: return "rx_e4m3_to_f32(" + raw + ")";
    case DT::F8E5M2: return "rx_e5m2_to_f32(" + raw + ")";
    case DT::I1: return "(" + raw + " != 0)";
    default: return raw;
  }
}

std::string Emitter::store_conv(DT dt, const std::string& val) {
  switch (dt) {
    case DT::BF16: return "rx_f32_to_bf16(" + val + ")";
    case DT::F16: return "rx_f32_to_f16(" + val + ")";
    case DT::F8E4M3FN: return "rx_f32_to_e4m3(" + val + ")";
    case DT::F8E5M2: return "rx_f32_to_e5m2(" + val + ")";
    case DT::I1: return "(rx_u8)((" + val + ") ? 1 : 0)";
    default: return val;
  }
}

// `e` with casts to float and enclosing parentheses taken off
static std::string bare_name(std::string e) {
  for (;;) {
    if (e.size() >= 2 && e.front() == '(' && e.back() == ')' && e.find(')') == e.size() - 1) e = e.substr(1, e.size() - 2);
    else if (e.compare(0, 7, "(float)") == 0) e = e.substr(7);
    else return e;
  }
}

std::string Emitter::store_value(DT dt, const std::string& val) const {
  // a value that a clamp has just put inside the range of e4m3 (what a quantization does): the hardware conversion
  // by itself, without the range handling around it
  if (dt == DT::F8E4M3FN) {
    auto r = rounded_.find(val);
    const std::string src = bare_name(r != rounded_.end() && r->second.first == dt ? r->second.second : val);
    if (e4m3_range_.count(src)) return "rx_f32_to_e4m3_inrange(" + src + ")";
  }
  auto it = rounded_.find(val);
  if (it != rounded_.end() && it->second.first == dt) return store_conv(dt, "(" + it->second.second + ")");
  return store_conv(dt, val);
}

std::string Emitter::round_narrow(DT dt, const std::string& e) {
  switch (dt) {
    case DT::BF16: return "rx_round_bf16(" + e + ")";
    case DT::F16: return "rx_round_f16(" + e + ")";
    case DT::F8E4M3FN: return "rx_round_e4m3(" + e + ")";
    case DT::F8E5M2: return "rx_round_e5m2(" + e + ")";
    default: return e;
  }
}

static std::string float_lit(double v, bool dbl) {
  if (std::isnan(v)) return dbl ? "__builtin_nan(\"\")" : "__builtin_nanf(\"\")";
  if (std::isinf(v)) return std::string(v < 0 ? "(-" : "(") + (dbl ? "__builtin_inf()" : "__builtin_inff()") + ")";
  char buf[64];
  snprintf(buf, sizeof buf, "%a", v);
  std::string s = buf;
  if (!dbl) s += "f";
  return "(" + s + ")";
}

std::string Emitter::literal(const Node& n) {
  DT dt = n.ty.dt;
  if (is_float(dt)) return float_lit(splat_as_double(n), dt == DT::F64);
  if (dt == DT::I1) return splat_as_int(n) ? "true" : "false";
  int64_t v = splat_as_int(n);
  if (dt == DT::U64) return "(rx_u64)" + std::to_string((uint64_t)v) + "ULL";
  if (dt == DT::I64) {
    if (v == INT64_MIN) return "(rx_i64)(-9223372036854775807LL - 1)";
    return "(rx_i64)" + std::to_string(v) + "LL";
  }
  return std::string("(") + info(dt).ctype + ")" + "(" + std::to_string(v) + ")";
}

Ix Emitter::temp_index(const std::string& expr, int64_t lo, int64_t hi) {
  Ix r;
  r.var = fresh("t");
  r.lo = lo;
  r.hi = hi;
  line("const " + idx_t() + " " + r.var + " = " + expr + ";");
  return r;
}

std::string Emitter::emit(int node, const Index& ix) {
  auto b = bound.find(node);
  if (b != bound.end()) return b->second;
  const Node& n = g_.nodes[node];
  if ((int)ix.size() != n.ty.rank()) throw Error("internal: index rank mismatch at node " + std::to_string(node));
  std::string key = std::to_string(node) + ":";
  for (auto& i : ix) key += i.key() + ",";
  std::string r;
  if (lookup(key, &r)) return r;
  if (is_input_(node)) r = emit_load(node, ix);
  else r = emit_op(n, ix);
  scopes_.back()[key] = r;
  return r;
}

std::string Emitter::emit_load(int node, const Index& ix) {
  const Node& n = g_.nodes[node];
  const auto& dims = n.ty.dims;
  for (size_t d = 0; d < dims.size(); ++d) {
    if (dims[d] == 1) continue;
    if (ix[d].lo < 0 || ix[d].hi > dims[d] - 1)
      throw Error("internal: index range check failed reading node " + std::to_string(node) + " dim " + std::to_string(d) +
                  " range [" + std::to_string(ix[d].lo) + "," + std::to_string(ix[d].hi) + "] size " + std::to_string(dims[d]));
  }
  int slot = slot_of(node);
  LoadRecord rec;
  rec.node = node;
  rec.minor_follows = !dims.empty() && !root_vars_.empty() && ix[dims.size() - 1].var == root_vars_.back();
  if (dims.size() == root_vars_.size() && !dims.empty()) {
    rec.affine = true;
    for (size_t d = 0; d < dims.size(); ++d) {
      if (ix[d].var != root_vars_[d]) { rec.affine = false; break; }
      rec.off.push_back(ix[d].off);
    }
  }
  bool permuted = false;
  if (!rec.affine && dims.size() == root_vars_.size() && dims.size() >= 2) {
    std::vector<char> used(dims.size(), 0);
    permuted = true;
    for (size_t d = 0; d < dims.size() && permuted; ++d) {
      int which = -1;
      for (size_t v = 0; v < root_vars_.size(); ++v)
        if (ix[d].var == root_vars_[v] && (ix[d].off == 0 || offset_perms)) which = (int)v;
      if (which < 0 || used[which] || (root_dims_[which] != dims[d] && !offset_perms)) permuted = false;
      else { used[which] = 1; rec.root_var.push_back(which); rec.root_off.push_back(ix[d].off); }
    }
    if (!permuted) { rec.root_var.clear(); rec.root_off.clear(); }
  }
  loads.push_back(rec);
  if (permuted && perm_hook) {
    std::string hooked;
    if (perm_hook(slot, rec.root_var, &hooked)) {
      std::string v = fresh();
      line(std::string("const ") + info(n.ty.dt).ctype + " " + v + " = " + load_conv(n.ty.dt, hooked) + ";");
      return v;
    }
  }
  bool direct = allow_direct_ && rec.affine && dims == root_dims_;
  bool shifted = false;
  if (direct)
    for (auto o : rec.off) shifted = shifted || o != 0;
  if (shifted && !(allow_shifted && vec > 1)) direct = false;
  std::string raw;
  std::string hooked;
  if (tile_hook && rec.affine && dims == root_dims_ && tile_hook(slot, rec.off, &hooked)) {
    raw = hooked;
  } else if (direct) {
    // element (l + o) of the row, o = offset in the minor dimension; outer offsets move whole vectors
    const int nd = (int)dims.size();
    int64_t stride = 1, delta = 0;
    for (int d = nd - 1; d >= 0; --d) {
      if (d < nd - 1) delta += rec.off[d] * stride;
      stride *= dims[d];
    }
    const int64_t o = rec.off[nd - 1];
    int64_t q = o >= 0 ? o / vec : -((-o + vec - 1) / vec);
    const int64_t r = o - q * vec;
    const int64_t D0 = delta + q * vec;
    direct_vecs.insert({slot, D0});
    std::string A = direct_expr(slot, D0);
    if (r == 0) {
      raw = A + ".v[l]";
    } else {
      direct_vecs.insert({slot, D0 + vec});
      std::string B = direct_expr(slot, D0 + vec);
      const std::string lr = "(l + " + std::to_string(r) + ")";
      raw = "(" + lr + " < " + std::to_string(vec) + " ? " + A + ".v[" + lr + " % " + std::to_string(vec) + "] : " + B + ".v[" + lr + " % " +
            std::to_string(vec) + "])";
    }
  } else {
    const std::string at = dims.empty() ? std::string("0") : linear(ix, dims);
    if (const_vectors && dims.size() <= 1) raw = "rx_load_const(in" + std::to_string(slot) + ", " + at + ")";
    else raw = "in" + std::to_string(slot) + "[" + at + "]";
    if (!dims.empty()) ++unsafe_loads_;
  }
  std::string v = fresh();
  line(std::string("const ") + info(n.ty.dt).ctype + " " + v + " = " + load_conv(n.ty.dt, raw) + ";");
  return v;
}

static std::string fn(const std::string& base, bool dbl) { return dbl ? base : base + "f"; }

// The same value at every index: a rank-0 value, or broadcasts / elementwise ops of such values.
bool Emitter::is_uniform(int node, int depth) const {
  const Node& n = g_.nodes[node];
  if (n.ty.rank() == 0) return true;
  if (depth > 8) return false;
  switch (n.k) {
    case OpK::Constant: return n.splat;
    case OpK::BroadcastInDim:
    case OpK::Reshape:
    case OpK::Convert:
    case OpK::Unary:
      return is_uniform(n.in[0], depth + 1);
    case OpK::Binary:
      return is_uniform(n.in[0], depth + 1) && is_uniform(n.in[1], depth + 1);
    default:
      return false;
  }
}

// The value does not vary along the node's last dimension (a row's reduction result broadcast back over the row).
bool Emitter::minor_uniform(int node, int depth) const {
  const Node& n = g_.nodes[node];
  if (n.ty.rank() == 0) return true;
  if (depth > 8) return false;
  switch (n.k) {
    case OpK::Constant: return n.splat;
    case OpK::BroadcastInDim: {
      const Node& o = g_.nodes[n.in[0]];
      for (size_t d = 0; d < n.a0.size(); ++d)
        if (n.a0[d] == n.ty.rank() - 1 && o.ty.dims[d] != 1) return false;
      return true;
    }
    case OpK::Convert:
    case OpK::Unary:
      return minor_uniform(n.in[0], depth + 1);
    case OpK::Binary:
      return minor_uniform(n.in[0], depth + 1) && minor_uniform(n.in[1], depth + 1);
    default:
      return false;
  }
}

bool Emitter::minor_only(int node, int depth) const {
  const Node& n = g_.nodes[node];
  if (n.ty.rank() == 0) return true;
  if (depth > 8) return false;
  switch (n.k) {
    case OpK::Constant: return n.splat;
    case OpK::BroadcastInDim: {
      const Node& o = g_.nodes[n.in[0]];
      for (size_t d = 0; d < n.a0.size(); ++d)
        if (n.a0[d] != n.ty.rank() - 1 && o.ty.dims[d] != 1) return false;
      return true;
    }
    case OpK::Convert:
    case OpK::Unary:
      return minor_only(n.in[0], depth + 1);
    case OpK::Binary:
      return minor_only(n.in[0], depth + 1) && minor_only(n.in[1], depth + 1);
    default:
      return false;
  }
}

// n = (0.5 * x) * (1 + tanh(a * (x + b * ((x * x) * x)))) in any operand order, every intermediate value computed in
// this kernel and of n's type; a, b constants.
bool Emitter::match_gelu_chain(const Node& n, int* xnode, double* ka, double* kb) const {
  auto constant = [&](int id, double* v) {
    const Node* c = &g_.nodes[id];
    while (c->k == OpK::BroadcastInDim || c->k == OpK::Reshape) c = &g_.nodes[c->in[0]];
    if (c->k != OpK::Constant || !c->splat || !is_float(c->ty.dt)) return false;
    *v = splat_as_double(*c);
    return true;
  };
  auto inner = [&](int id, const char* op) -> const Node* {
    const Node& m = g_.nodes[id];
    if (is_input_(id) || bound.count(id) || m.k != OpK::Binary || m.op != op || !(m.ty == n.ty)) return nullptr;
    return &m;
  };
  // (constant, other) of a commutative node
  auto with_constant = [&](const Node& m, double* c, int* other) {
    for (int k = 0; k < 2; ++k)
      if (constant(m.in[k], c)) { *other = m.in[1 - k]; return true; }
    return false;
  };
  for (int k = 0; k < 2; ++k) {
    const Node* half = inner(n.in[k], "multiply");
    const Node* one = inner(n.in[1 - k], "add");
    if (!half || !one) continue;
    double c;
    int x, t;
    if (!with_constant(*half, &c, &x) || c != 0.5) continue;
    if (!with_constant(*one, &c, &t) || c != 1.0) continue;
    const Node& th = g_.nodes[t];
    if (is_input_(t) || bound.count(t) || th.k != OpK::Unary || th.op != "tanh" || !(th.ty == n.ty)) continue;
    const Node* y = inner(th.in[0], "multiply");
    int sum_id;
    if (!y || !with_constant(*y, ka, &sum_id)) continue;
    const Node* sum = inner(sum_id, "add");
    if (!sum) continue;
    for (int j = 0; j < 2; ++j) {
      if (sum->in[j] != x) continue;
      const Node* bx3 = inner(sum->in[1 - j], "multiply");
      int cube_id;
      if (!bx3 || !with_constant(*bx3, kb, &cube_id)) continue;
      const Node* cube = inner(cube_id, "multiply");
      if (!cube) continue;
      for (int i = 0; i < 2; ++i) {
        if (cube->in[i] != x) continue;
        const Node* sq = inner(cube->in[1 - i], "multiply");
        if (sq && sq->in[0] == x && sq->in[1] == x) { *xnode = x; return true; }
      }
    }
  }
  return false;
}

std::string Emitter::emit_op(const Node& n, const Index& ix) {
  const DT dt = n.ty.dt;
  const std::string CT = info(dt).ctype;
  const bool dbl = dt == DT::F64;
  auto def = [&](const std::string& expr, bool force_round = false) {
    std::string v = fresh();
    const bool rnd = is_narrow_float(dt) && (force_round || !excess_precision);
    line("const " + CT + " " + v + " = " + (rnd ? round_narrow(dt, expr) : expr) + ";");
    if (rnd) rounded_[v] = {dt, expr};
    return v;
  };
  // index of a rank-0 or same-shape operand
  auto opnd = [&](int k) {
    const Node& o = g_.nodes[n.in[k]];
    if (o.ty.rank() == 0 && n.ty.rank() != 0) return emit(n.in[k], Index{});
    return emit(n.in[k], ix);
  };
  switch (n.k) {
    case OpK::Param:
      throw Error("internal: parameter reached the emitter without a buffer");
    case OpK::Constant:
      if (!n.splat) throw Error("internal: dense constant must be materialized");
      return literal(n);
    case OpK::Iota: {
      std::string e = "(" + CT + ")" + ix[n.a0[0]].str();
      return is_narrow_float(dt) ? def(e, true) : e;
    }
    case OpK::Unary: {
      const DT sdt = g_.nodes[n.in[0]].ty.dt;
      std::string x = opnd(0);
      const std::string& op = n.op;
      if (op == "is_finite") return def("isfinite(" + x + ")");
      if (op == "bitcast") return sdt == dt ? x : def("__builtin_bit_cast(" + CT + ", " + x + ")");
      if (op == "is_inf") return def("isinf(" + x + ")");
      if (op == "is_pos_inf") return def("(isinf(" + x + ") && " + x + " > 0)");
      if (op == "is_neg_inf") return def("(isinf(" + x + ") && " + x + " < 0)");
      if (is_float(dt)) {
        for (const char* m : {"acos", "acosh", "asin", "asinh", "atan", "atanh", "cosh", "sinh", "erfc", "lgamma"})
          if (op == m) return def(fn(m, dbl) + "(" + x + ")");
        if (op == "erf_inv") return def(fn("erfinv", dbl) + "(" + x + ")");
        if (op == "digamma") return def("rx_digamma(" + x + ")");
        if (op == "sine") return def(fn("sin", dbl) + "(" + x + ")");
        if (op == "cosine") return def(fn("cos", dbl) + "(" + x + ")");
        if (op == "tan") return def(fn("tan", dbl) + "(" + x + ")");
        if (op == "tanh") return def((is_narrow_float(dt) ? std::string("rx_tanh_fast") : fn("tanh", dbl)) + "(" + x + ")");
        if (op == "exponential") return def((is_narrow_float(dt) ? std::string("rx_exp_fast") : fn("exp", dbl)) + "(" + x + ")");
        if (op == "exponential_minus_one") return def(fn("expm1", dbl) + "(" + x + ")");
        if (op == "log") return def(fn("log", dbl) + "(" + x + ")");
        if (op == "log_plus_one") return def(fn("log1p", dbl) + "(" + x + ")");
        if (op == "sqrt") return def(fn("sqrt", dbl) + "(" + x + ")");
        if (op == "cbrt") return def(fn("cbrt", dbl) + "(" + x + ")");
        if (op == "rsqrt") return def("rx_rsqrt(" + x + ")");
        if (op == "abs") return def(fn("fabs", dbl) + "(" + x + ")");
        if (op == "negate") return def("(-" + x + ")");
        if (op == "logistic") return def((is_narrow_float(dt) ? "rx_logistic_fast(" : "rx_logistic(") + x + ")");
        if (op == "floor") return def(fn("floor", dbl) + "(" + x + ")");
        if (op == "ceil") return def(fn("ceil", dbl) + "(" + x + ")");
        if (op == "sign") return def("rx_sign(" + x + ")");
        if (op == "round_nearest_even") return def(fn("rint", dbl) + "(" + x + ")");
        if (op == "round_nearest_afz") return def(fn("round", dbl) + "(" + x + ")");
        if (op == "erf") return def(fn("erf", dbl) + "(" + x + ")");
      } else if (dt == DT::I1) {
        if (op == "not") return def("(!" + x + ")");
        if (op == "abs" || op == "negate" || op == "sign") return x;
      } else {
        if (op == "not") return def("(" + CT + ")(~" + x + ")");
        if (op == "negate") return def("(" + CT + ")(0 - " + x + ")");
        if (op == "abs") return info(dt).is_signed ? def("(" + CT + ")(" + x + " < 0 ? 0 - " + x + " : " + x + ")") : x;
        if (op == "sign") return def("(" + CT + ")((" + x + " > 0) - (" + x + " < 0))");
        if (op == "popcnt") return def("(" + CT + ")rx_popcnt(" + x + ")");
        if (op == "count_leading_zeros") return def("(" + CT + ")rx_clz(" + x + ")");
      }
      (void)sdt;
      throw Error("unsupported unary op '" + op + "' on " + info(dt).mlir);
    }
    case OpK::Gelu: {
      std::string x = opnd(0);
      if (!is_float(dt)) throw Error("gelu on a non-float type");
      if (n.op == "TANH" && is_narrow_float(dt)) {
        const double k1 = -2.0 * 1.4426950408889634 * 0.7978845608028654;
        return def("rx_gelu_chain_fast(" + x + ", " + float_lit(k1, false) + ", " + float_lit(k1 * 0.044715, false) + ")");
      }
      std::string f = n.op == "TANH" ? "rx_gelu_tanh" : (n.op == "SIGMOID" ? "rx_gelu_sigmoid" : "rx_gelu_erf");
      return def(f + "(" + x + ")");
    }
    case OpK::Binary: {
      if (n.op == "multiply" && is_narrow_float(dt) && excess_precision) {
        // 0.5 x (1 + tanh(a (x + b x^3))), the chain that `gelu_tanh` lowers to, for a result that is rounded to a
        // narrow float: x / (1 + e^(-2 a (x + b x^3))) with the two constants folded (8 instructions instead of 15;
        // in the epilogue of a matrix product the difference is a quarter of the epilogue's time)
        double ka, kb;
        int xnode;
        if (match_gelu_chain(n, &xnode, &ka, &kb)) {
          const Node& xo = g_.nodes[xnode];
          const std::string x = emit(xnode, xo.ty.rank() == 0 && n.ty.rank() != 0 ? Index{} : ix);
          const double k1 = -2.0 * 1.4426950408889634 * ka;
          return def("rx_gelu_chain_fast(" + x + ", " + float_lit(k1, false) + ", " + float_lit(k1 * kb, false) + ")");
        }
      }
      std::string a = opnd(0), b = opnd(1);
      const std::string& op = n.op;
      if (is_float(dt)) {
        if (op == "add") return def("(" + a + " + " + b + ")");
        if (op == "subtract") return def("(" + a + " - " + b + ")");
        if (op == "multiply") return def("(" + a + " * " + b + ")");
        if (op == "divide") {
          // a divisor that is one value for the whole tensor (a broadcast scalar, e.g. a
          // quantization scale): its reciprocal in double is loop-invariant, and the product in
          // double rounds to the same float as the division (see rx_div_uniform)
          // a result that is rounded to a narrow float, divided by a value that is the same along the minor dimension
          // (the sum of a softmax row, a quantization scale): its reciprocal, a division of its own that the compiler
          // computes once per row, times the dividend -- within an ulp of float32 of the quotient (rx_div_minor_uniform, which
          // also covers subnormal divisors whose reciprocal would overflow)
          // (in a product's epilogue a thread handles many rows of the same columns: there the same holds for a divisor
          // that varies along the minor dimension only, a per-feature standard deviation)
          if (CT == "float" && is_narrow_float(dt) && excess_precision && n.ty.rank() > 0 && (minor_uniform(n.in[1]) || (columns_reused && n.ty.rank() >= 2 && minor_only(n.in[1]))))
            return def("rx_div_minor_uniform(" + a + ", " + b + ")");
          if (CT == "float" && n.ty.rank() > 0 && is_uniform(n.in[1])) return def("rx_div_uniform(" + a + ", " + b + ")");
          return def("(" + a + " / " + b + ")");
        }
        if (op == "maximum") return def("rx_max(" + a + ", " + b + ")");
        if (op == "minimum") return def("rx_min(" + a + ", " + b + ")");
        if (op == "power") return def(fn("pow", dbl) + "(" + a + ", " + b + ")");
        if (op == "remainder") return def(fn("fmod", dbl) + "(" + a + ", " + b + ")");
        if (op == "atan2") return def(fn("atan2", dbl) + "(" + a + ", " + b + ")");
      } else if (dt == DT::I1) {
        if (op == "add" || op == "or" || op == "maximum") return def("(" + a + " || " + b + ")");
        if (op == "multiply" || op == "and" || op == "minimum") return def("(" + a + " && " + b + ")");
        if (op == "xor" || op == "subtract") return def("(" + a + " != " + b + ")");
      } else {
        auto c = [&](const std::string& e) { return def("(" + CT + ")(" + e + ")"); };
        if (op == "add") return c(a + " + " + b);
        if (op == "subtract") return c(a + " - " + b);
        if (op == "multiply") return c(a + " * " + b);
        if (op == "divide") return def("rx_idiv<" + CT + ">(" + a + ", " + b + ")");
        if (op == "remainder") return def("rx_irem<" + CT + ">(" + a + ", " + b + ")");
        if (op == "maximum") return c(a + " > " + b + " ? " + a + " : " + b);
        if (op == "minimum") return c(a + " < " + b + " ? " + a + " : " + b);
        if (op == "and") return c(a + " & " + b);
        if (op == "or") return c(a + " | " + b);
        if (op == "xor") return c(a + " ^ " + b);
        if (op == "power") return def("rx_ipow<" + CT + ">(" + a + ", " + b + ")");
        const int bits = info(dt).size * 8;
        const std::string oob = "((rx_u64)" + b + " >= " + std::to_string(bits) + ")";
        if (op == "shift_left") return c(oob + " ? 0 : (" + a + " << " + b + ")");
        if (op == "shift_right_logical") {
          std::string U = std::string("rx_u") + std::to_string(bits);
          return c(oob + " ? 0 : (" + CT + ")((" + U + ")" + a + " >> " + b + ")");
        }
        if (op == "shift_right_arithmetic") return c(oob + " ? (" + a + " < 0 ? -1 : 0) : (" + a + " >> " + b + ")");
      }
      throw Error("unsupported binary op '" + op + "' on " + info(dt).mlir);
    }
    case OpK::Compare: {
      std::string a = opnd(0), b = opnd(1);
      const char* o = n.op == "EQ" ? "==" : n.op == "NE" ? "!=" : n.op == "LT" ? "<" : n.op == "LE" ? "<=" : n.op == "GT" ? ">" : n.op == "GE" ? ">=" : nullptr;
      if (!o) throw Error("unknown comparison direction " + n.op);
      return def("(" + a + " " + o + " " + b + ")");
    }
    case OpK::Select: {
      std::string p = opnd(0), a = opnd(1), b = opnd(2);
      return def("(" + p + " ? " + a + " : " + b + ")");
    }
    case OpK::Clamp: {
      std::string lo = opnd(0), x = opnd(1), hi = opnd(2);
      if (is_float(dt)) {
        // constant finite bounds in order: one median instruction, NaN of the operand passed through
        auto const_bound = [&](int k, double* v) {
          const Node* c = &g_.nodes[n.in[k]];
          while (c->k == OpK::BroadcastInDim || c->k == OpK::Reshape) c = &g_.nodes[c->in[0]];
          if (c->k != OpK::Constant || !c->splat) return false;
          *v = splat_as_double(*c);
          return true;
        };
        double lv, hv;
        if (CT == "float" && const_bound(0, &lv) && const_bound(2, &hv) && lv <= hv) {
          const std::string v = def("rx_clamp_ordered(" + x + ", " + lo + ", " + hi + ")");
          if (lv >= -448.0 && hv <= 448.0 && dt == DT::F32) e4m3_range_.insert(v);
          return v;
        }
        return def("rx_min(rx_max(" + x + ", " + lo + "), " + hi + ")");
      }
      return def("(" + CT + ")((" + x + " < " + lo + " ? " + lo + " : " + x + ") > " + hi + " ? " + hi + " : (" + x + " < " + lo + " ? " + lo + " : " + x + "))");
    }
    case OpK::Convert: {
      const DT sdt = g_.nodes[n.in[0]].ty.dt;
      std::string x = opnd(0);
      if (sdt == dt) return x;
      if (dt == DT::I1) return def("(" + x + " != 0)");
      if (is_narrow_float(sdt) && is_narrow_float(dt)) return def(x, true);
      if (is_narrow_float(sdt) && dt == DT::F32) return x;
      // float -> integer: toward zero, saturating at the type's limits, NaN -> 0 (a plain cast is undefined there)
      if (is_float(sdt) && !is_float(dt)) return def("rx_f2i<" + CT + ">(" + x + ")", true);
      return def("(" + CT + ")" + x, true);
    }
    case OpK::BroadcastInDim: {
      const Node& o = g_.nodes[n.in[0]];
      Index oi(o.ty.rank());
      for (int k = 0; k < o.ty.rank(); ++k) {
        if (o.ty.dims[k] == 1 && n.ty.dims[n.a0[k]] != 1) oi[k] = const_ix(0);
        else oi[k] = ix[n.a0[k]];
      }
      return emit(n.in[0], oi);
    }
    case OpK::Transpose: {
      Index oi(ix.size());
      for (size_t i = 0; i < ix.size(); ++i) oi[n.a0[i]] = ix[i];
      return emit(n.in[0], oi);
    }
    case OpK::Reshape: {
      const Node& o = g_.nodes[n.in[0]];
      // fast path: shapes equal after dropping unit dims
      std::vector<int> rn, ro;
      for (int k = 0; k < n.ty.rank(); ++k) if (n.ty.dims[k] != 1) rn.push_back(k);
      for (int k = 0; k < o.ty.rank(); ++k) if (o.ty.dims[k] != 1) ro.push_back(k);
      bool same = rn.size() == ro.size();
      for (size_t k = 0; same && k < rn.size(); ++k) same = n.ty.dims[rn[k]] == o.ty.dims[ro[k]];
      Index oi(o.ty.rank(), const_ix(0));
      if (same) {
        for (size_t k = 0; k < rn.size(); ++k) oi[ro[k]] = ix[rn[k]];
        return emit(n.in[0], oi);
      }
      // Dims that regroup independently ([C*T, B*P] <-> [C, T, B, P]) are converted group by group:
      // a group's index arithmetic involves only its own variables, so the part that does not
      // depend on the minor output index is computed once per thread, not once per element.
      {
        const auto& nd = n.ty.dims;
        const auto& od = o.ty.dims;
        struct Grp { size_t a0, a1, b0, b1; };
        std::vector<Grp> groups;
        size_t a = 0, b = 0;
        bool ok = n.ty.numel() > 0;
        while (ok && a < nd.size() && b < od.size()) {
          Grp gq{a, a, b, b};
          int64_t pa = nd[a++], pb = od[b++];
          while (pa != pb) {
            if (pa < pb) { if (a >= nd.size()) { ok = false; break; } pa *= nd[a++]; }
            else { if (b >= od.size()) { ok = false; break; } pb *= od[b++]; }
          }
          gq.a1 = a; gq.b1 = b;
          groups.push_back(gq);
        }
        for (; ok && a < nd.size(); ++a) ok = nd[a] == 1;     // trailing unit dims carry no index
        for (; ok && b < od.size(); ++b) ok = od[b] == 1;
        if (ok && groups.size() > 1) {
          for (auto& gq : groups) {
            if (gq.a1 - gq.a0 == 1 && gq.b1 - gq.b0 == 1) { oi[gq.b0] = ix[gq.a0]; continue; }
            // One source dimension whose index is lane `off` of an aligned vector (var a multiple of `align`), split into
            // dimensions the innermost of which is a whole number of vectors: var splits by itself and the lane is added
            // to the innermost component -- the lanes of a vector then share every division.
            {
              int k0 = -1, nz = 0, last = -1;
              for (size_t k = gq.a0; k < gq.a1; ++k) if (nd[k] != 1) { k0 = (int)k; ++nz; }
              for (size_t k = gq.b0; k < gq.b1; ++k) if (od[k] != 1) last = (int)k;
              if (nz == 1 && last >= 0) {
                const Ix& sx = ix[k0];
                if (!sx.is_const() && sx.align > 1 && sx.off >= 0 && sx.off < sx.align && od[last] % sx.align == 0) {
                  int64_t stride = nd[k0];
                  for (size_t k = gq.b0; k < gq.b1; ++k) {
                    stride /= std::max<int64_t>(od[k], 1);
                    if (od[k] == 1) continue;
                    std::string c2 = sx.var;
                    if (stride > 1) c2 = "(" + c2 + " / " + std::to_string(stride) + ")";
                    bool first = true;
                    for (size_t q = gq.b0; q < k; ++q) first = first && od[q] == 1;
                    if (!first) c2 = c2 + " % " + std::to_string(od[k]);
                    oi[k] = temp_index(c2, 0, od[k] - 1);
                    if ((int)k == last) { oi[k].off = sx.off; oi[k].align = sx.align; oi[k].hi = od[k] - sx.align; oi[k].lo = 0; oi[k].lo += sx.off; oi[k].hi += sx.off; }
                  }
                  continue;
                }
              }
            }
            // linear index inside the group
            std::string e;
            int64_t total = 1, lo = 0, hi = 0;
            bool all_const = true;
            for (size_t k = gq.a0; k < gq.a1; ++k) {
              total *= nd[k];
              if (nd[k] == 1) continue;
              all_const = all_const && ix[k].is_const();
            }
            {
              int64_t stride = total;
              for (size_t k = gq.a0; k < gq.a1; ++k) {
                stride /= std::max<int64_t>(nd[k], 1);
                if (nd[k] == 1) continue;
                const std::string term = stride == 1 ? "(" + ix[k].str() + ")" : "(" + ix[k].str() + ") * " + std::to_string(stride);
                e += (e.empty() ? "" : " + ") + term;
                lo += ix[k].lo * stride;
                hi += ix[k].hi * stride;
              }
            }
            if (e.empty()) e = "0";
            Ix lin = temp_index(e, lo, hi);
            int64_t stride = total;
            for (size_t k = gq.b0; k < gq.b1; ++k) {
              stride /= std::max<int64_t>(od[k], 1);
              if (od[k] == 1) continue;
              std::string c2 = lin.var;
              if (stride > 1) c2 = "(" + c2 + " / " + std::to_string(stride) + ")";
              bool first = true;
              for (size_t q = gq.b0; q < k; ++q) first = first && od[q] == 1;
              if (!first) c2 = c2 + " % " + std::to_string(od[k]);
              oi[k] = temp_index(c2, 0, od[k] - 1);
            }
            (void)all_const;
          }
          return emit(n.in[0], oi);
        }
      }
      Ix lin = temp_index(linear(ix, n.ty.dims), 0, n.ty.numel() - 1);
      int64_t stride = o.ty.numel();
      for (int k = 0; k < o.ty.rank(); ++k) {
        stride /= std::max<int64_t>(o.ty.dims[k], 1);
        if (o.ty.dims[k] == 1) continue;
        std::string e = lin.var;
        if (stride > 1) e = "(" + e + " / " + std::to_string(stride) + ")";
        if (k > 0) e = e + " % " + std::to_string(o.ty.dims[k]);
        oi[k] = temp_index(e, 0, o.ty.dims[k] - 1);
      }
      return emit(n.in[0], oi);
    }
    case OpK::Slice: {
      Index oi(ix.size());
      for (size_t d = 0; d < ix.size(); ++d) {
        if (n.a2[d] == 1) oi[d] = shifted(ix[d], n.a0[d]);
        else if (ix[d].is_const()) oi[d] = const_ix(ix[d].off * n.a2[d] + n.a0[d]);
        else oi[d] = temp_index(ix[d].str() + " * " + std::to_string(n.a2[d]) + " + " + std::to_string(n.a0[d]),
                                ix[d].lo * n.a2[d] + n.a0[d], ix[d].hi * n.a2[d] + n.a0[d]);
      }
      return emit(n.in[0], oi);
    }
    case OpK::Reverse: {
      const Node& o = g_.nodes[n.in[0]];
      Index oi = ix;
      for (auto d : n.a0) {
        const int64_t last = o.ty.dims[d] - 1;
        if (ix[d].is_const()) oi[d] = const_ix(last - ix[d].off);
        else oi[d] = temp_index(std::to_string(last) + " - (" + ix[d].str() + ")", last - ix[d].hi, last - ix[d].lo);
      }
      return emit(n.in[0], oi);
    }
    case OpK::Window: {
      const Node& o = g_.nodes[n.in[0]];
      const int r = o.ty.rank();
      Index oi(r);
      for (int d = 0; d < r; ++d) {
        const Ix& k = ix[d];
        const Ix& p = ix[r + d];
        const int64_t st = n.a1[d], dl = n.a2[d];
        if (k.is_const() && p.is_const()) oi[d] = const_ix(p.off * st + k.off * dl);
        else if (k.is_const() && st == 1) oi[d] = shifted(p, k.off * dl);
        else if (p.is_const() && dl == 1) oi[d] = shifted(k, p.off * st);
        else {
          std::string e = st == 1 ? p.str() : "(" + p.str() + ") * " + std::to_string(st);
          e += " + " + (dl == 1 ? k.str() : "(" + k.str() + ") * " + std::to_string(dl));
          oi[d] = temp_index(e, p.lo * st + k.lo * dl, p.hi * st + k.hi * dl);
        }
      }
      return emit(n.in[0], oi);
    }
    case OpK::Gather: {
      // result index -> (batch index into start_indices, offset index into the slice); the operand
      // index is the clamped start read at the batch index, plus the offset
      const Node& o = g_.nodes[n.in[0]];
      const Node& st = g_.nodes[n.in[1]];
      const int r = o.ty.rank(), rs = st.ty.rank();
      const int ivd = (int)n.a4[0];
      auto has = [](const std::vector<int64_t>& v, int x) { return std::find(v.begin(), v.end(), (int64_t)x) != v.end(); };
      std::vector<Ix> batch;   // result index components of the non-offset dims, in order
      for (int d = 0; d < n.ty.rank(); ++d) if (!has(n.a0, d)) batch.push_back(ix[d]);
      // offset component per operand dim
      Index off(r, const_ix(0));
      {
        size_t j = 0;
        for (int d = 0; d < r; ++d) {
          if (has(n.a1, d) || has(n.a5, d)) continue;
          off[d] = ix[n.a0[j++]];
        }
      }
      Index oi = off;
      // operand batching dims take the batch index component of their start_indices dim
      for (size_t b = 0; b < n.a5.size(); ++b) {
        const int ds = (int)n.a6[b];
        oi[n.a5[b]] = batch[ds - (ds < ivd ? 0 : 1)];
      }
      for (size_t k = 0; k < n.a2.size(); ++k) {
        const int d = (int)n.a2[k];
        Index si(rs);
        size_t bi = 0;
        for (int q = 0; q < rs; ++q) si[q] = q == ivd ? const_ix((int64_t)k) : batch[bi++];
        const std::string e = emit(n.in[1], si);
        const int64_t room = o.ty.dims[d] - n.a3[d];
        const Ix& f = off[d];
        oi[d] = temp_index("(" + idx_t() + ")rx_clamp_idx<long long>((long long)(" + e + "), " + std::to_string(room) + "LL)" +
                               (f.is_const() && f.off == 0 ? std::string() : " + " + f.str()),
                           f.lo, f.hi + room);
      }
      return emit(n.in[0], oi);
    }
    case OpK::DynamicSlice: {
      const Node& o = g_.nodes[n.in[0]];
      Index oi(ix.size());
      for (size_t d = 0; d < ix.size(); ++d) {
        const Node& s = g_.nodes[n.in[1 + d]];
        const int64_t room = o.ty.dims[d] - n.a0[d];   // start indices are clamped into [0, room]
        if (s.k == OpK::Constant && s.splat) {
          oi[d] = shifted(ix[d], std::min(std::max<int64_t>(splat_as_int(s), 0), room));
        } else {
          // start index computed at run time (a 0-d integer value): clamp, then offset
          const std::string e = emit(n.in[1 + d], Index{});
          oi[d] = temp_index("(" + idx_t() + ")rx_clamp_idx<long long>((long long)(" + e + "), " + std::to_string(room) + "LL) + " + ix[d].str(),
                             ix[d].lo, ix[d].hi + room);
        }
      }
      return emit(n.in[0], oi);
    }
    case OpK::Pad: {
      const Node& o = g_.nodes[n.in[0]];
      std::string pv = emit(n.in[1], Index{});
      Index oi(ix.size());
      std::vector<std::string> conds;
      std::vector<std::string> pre;
      bool never = false;
      for (size_t d = 0; d < ix.size(); ++d) {
        const int64_t low = n.a0[d], q = n.a2[d] + 1, sd = o.ty.dims[d];
        Ix p = shifted(ix[d], -low);
        if (q == 1) {
          if (p.lo < 0) conds.push_back(p.str() + " >= 0");
          if (p.hi > sd - 1) conds.push_back(p.str() + " < " + std::to_string(sd));
          p.lo = std::max<int64_t>(p.lo, 0);
          p.hi = std::min<int64_t>(p.hi, sd - 1);
          if (p.lo > p.hi) never = true;
          oi[d] = p;
        } else {
          if (p.lo < 0) conds.push_back(p.str() + " >= 0");
          conds.push_back(p.str() + " % " + std::to_string(q) + " == 0");
          if (p.hi / q > sd - 1) conds.push_back(p.str() + " / " + std::to_string(q) + " < " + std::to_string(sd));
          Ix t;
          t.var = fresh("t");
          t.lo = std::max<int64_t>(0, p.lo / q);
          t.hi = std::min<int64_t>(sd - 1, std::max<int64_t>(p.hi, 0) / q);
          pre.push_back("const " + idx_t() + " " + t.var + " = " + p.str() + " / " + std::to_string(q) + ";");
          if (t.lo > t.hi) never = true;
          oi[d] = t;
        }
      }
      if (never || o.ty.numel() == 0) return pv;
      if (conds.empty() && pre.empty()) return emit(n.in[0], oi);
      std::string v = fresh();
      std::string cond;
      for (auto& c : conds) cond += (cond.empty() ? "" : " && ") + c;
      if (cond.empty()) cond = "true";
      if (clamp_guards && pre.empty()) {
        // Reads at positions clamped into the operand and a select instead of a branch: the loads of a lane's
        // consecutive elements are then unconditional and at consecutive addresses, and the compiler combines them
        // into one vector load (under a branch of their own, eight 16-bit elements are eight loads).
        Index ci = oi;
        for (size_t d = 0; d < ix.size(); ++d) {
          const int64_t sd = o.ty.dims[d];
          const Ix q0 = shifted(ix[d], -n.a0[d]);
          if (q0.lo >= 0 && q0.hi <= sd - 1) continue;
          Ix t;
          t.var = fresh("t");
          t.lo = std::max<int64_t>(q0.lo, 0);
          t.hi = std::min<int64_t>(q0.hi, sd - 1);
          line("const " + idx_t() + " " + t.var + " = rx_min<" + idx_t() + ">(rx_max<" + idx_t() + ">(" + q0.str() + ", 0), " + std::to_string(sd - 1) + ");");
          ci[d] = t;
        }
        std::string inner = emit(n.in[0], ci);
        line("const " + CT + " " + v + " = (" + cond + ") ? " + inner + " : " + pv + ";");
        return v;
      }
      if (branchless_guards) {
        const int unsafe0 = unsafe_loads_;
        const std::string before = take_code();
        push_scope();
        for (auto& p : pre) line(p);
        std::string inner = emit(n.in[0], oi);
        const std::string code = take_code();
        out_ << before;
        if (unsafe_loads_ == unsafe0) {
          // straight-line: the values stay in scope of the enclosing block
          out_ << code;
          auto top = scopes_.back();
          scopes_.pop_back();
          for (auto& kv : top) scopes_.back().insert(kv);
          line("const " + CT + " " + v + " = (" + cond + ") ? " + inner + " : " + pv + ";");
          return v;
        }
        line(CT + " " + v + " = " + pv + ";");
        line("if (" + cond + ") {");
        out_ << code;
        line("  " + v + " = " + inner + ";");
        pop_scope();
        line("}");
        return v;
      }
      line(CT + " " + v + " = " + pv + ";");
      line("if (" + cond + ") {");
      indent += 2;
      push_scope();
      for (auto& p : pre) line(p);
      std::string inner = emit(n.in[0], oi);
      line(v + " = " + inner + ";");
      pop_scope();
      indent -= 2;
      line("}");
      return v;
    }
    case OpK::DynamicUpdateSlice: {
      const Node& o = g_.nodes[n.in[0]];
      const Node& u = g_.nodes[n.in[1]];
      Index ui(ix.size()), oi = ix;
      std::vector<std::string> conds;
      bool never = false;
      for (size_t d = 0; d < ix.size(); ++d) {
        const Node& s = g_.nodes[n.in[2 + d]];
        const int64_t room = o.ty.dims[d] - u.ty.dims[d];   // start indices are clamped into [0, room]
        Ix p;
        if (s.k == OpK::Constant && s.splat) {
          p = shifted(ix[d], -std::min(std::max<int64_t>(splat_as_int(s), 0), room));
        } else {
          const std::string e = emit(n.in[2 + d], Index{});
          p = temp_index(ix[d].str() + " - (" + idx_t() + ")rx_clamp_idx<long long>((long long)(" + e + "), " + std::to_string(room) + "LL)",
                         ix[d].lo - room, ix[d].hi);
        }
        if (p.lo < 0) conds.push_back(p.str() + " >= 0");
        if (p.hi > u.ty.dims[d] - 1) conds.push_back(p.str() + " < " + std::to_string(u.ty.dims[d]));
        p.lo = std::max<int64_t>(p.lo, 0);
        p.hi = std::min<int64_t>(p.hi, u.ty.dims[d] - 1);
        if (p.lo > p.hi) never = true;
        ui[d] = p;
      }
      if (never || u.ty.numel() == 0) return emit(n.in[0], oi);
      if (conds.empty()) return emit(n.in[1], ui);
      std::string v = fresh();
      std::string cond;
      for (auto& c : conds) cond += (cond.empty() ? "" : " && ") + c;
      if (branchless_guards) {
        const int unsafe0 = unsafe_loads_;
        const std::string before = take_code();
        push_scope();
        std::string a = emit(n.in[1], ui);
        const std::string code_a = take_code();
        pop_scope();
        push_scope();
        std::string b = emit(n.in[0], oi);
        const std::string code_b = take_code();
        pop_scope();
        out_ << before;
        if (unsafe_loads_ == unsafe0) {
          out_ << code_a << code_b;
          line("const " + CT + " " + v + " = (" + cond + ") ? " + a + " : " + b + ";");
          return v;
        }
        line(CT + " " + v + ";");
        line("if (" + cond + ") {");
        out_ << code_a;
        line("  " + v + " = " + a + ";");
        line("} else {");
        out_ << code_b;
        line("  " + v + " = " + b + ";");
        line("}");
        return v;
      }
      line(CT + " " + v + ";");
      line("if (" + cond + ") {");
      indent += 2;
      push_scope();
      std::string a = emit(n.in[1], ui);
      line(v + " = " + a + ";");
      pop_scope();
      indent -= 2;
      line("} else {");
      indent += 2;
      push_scope();
      std::string b = emit(n.in[0], oi);
      line(v + " = " + b + ";");
      pop_scope();
      indent -= 2;
      line("}");
      return v;
    }
    case OpK::Concatenate: {
      const int d = (int)n.a0[0];
      // static choice when the index range falls inside one operand
      int64_t base = 0;
      std::vector<int64_t> starts;
      for (int id : n.in) { starts.push_back(base); base += g_.nodes[id].ty.dims[d]; }
      for (size_t k = 0; k < n.in.size(); ++k) {
        int64_t sz = g_.nodes[n.in[k]].ty.dims[d];
        if (ix[d].lo >= starts[k] && ix[d].hi < starts[k] + sz) {
          Index oi = ix;
          oi[d] = shifted(ix[d], -starts[k]);
          return emit(n.in[k], oi);
        }
      }
      std::string v = fresh();
      line(CT + " " + v + ";");
      bool first = true;
      for (size_t k = 0; k < n.in.size(); ++k) {
        int64_t sz = g_.nodes[n.in[k]].ty.dims[d];
        if (sz == 0) continue;
        if (ix[d].hi < starts[k] || ix[d].lo >= starts[k] + sz) continue;
        bool last = true;
        for (size_t k2 = k + 1; k2 < n.in.size(); ++k2)
          if (g_.nodes[n.in[k2]].ty.dims[d] > 0 && ix[d].hi >= starts[k2]) last = false;
        std::string head = first ? "if (" : "} else if (";
        if (last && !first) line("} else {");
        else line(head + ix[d].str() + " < " + std::to_string(starts[k] + sz) + ") {");
        first = false;
        indent += 2;
        push_scope();
        Index oi = ix;
        oi[d] = shifted(ix[d], -starts[k]);
        oi[d].lo = std::max<int64_t>(oi[d].lo, 0);
        oi[d].hi = std::min<int64_t>(oi[d].hi, sz - 1);
        std::string a = emit(n.in[k], oi);
        line(v + " = " + a + ";");
        pop_scope();
        indent -= 2;
      }
      line("}");
      return v;
    }
    case OpK::Reduce:
    case OpK::Scan:
    case OpK::Scatter:
    case OpK::Conv:
    case OpK::DotGeneral:
      throw Error("internal: reduce/dot_general reached the emitter without a buffer or binding");
  }
  throw Error("internal: unhandled op kind");
}

}  // namespace rx
