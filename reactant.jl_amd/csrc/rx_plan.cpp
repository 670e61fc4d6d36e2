// Fusion partitioner and kernel writer.
//
// Every live node is either MATERIALIZED (it owns a buffer: parameters, dense
// constants, results, reduce and dot_general results, and producers whose
// duplication into several consumers would be expensive) or FUSED into the
// kernels of the materialized nodes that consume it.  Group classes:
//   map      one elementwise/broadcast/slice/pad cone per output element
//            (stencils are maps whose loads sit at constant offsets)
//   reduce   cone -> full reduction: per-thread partials, wavefront DPP stage,
//            LDS across the workgroup, then a second single-workgroup pass
//   row      reductions over the minor dimension fused with the elementwise ops
//            that consume them (softmax, RMSNorm): one workgroup or one
//            wavefront per row, the row stays in registers between phases
//   dot      dot_general with its elementwise epilogue (MFMA skeletons for
//            f32/bf16/f16/f8, a scalar loop for everything else)
#include "rx_plan.h"

#include <algorithm>
#include <array>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <set>
#include <sstream>

#include "rx_emit.h"
#include "rx_gemm.h"

namespace rx {
namespace {

constexpr int kBlock = 256;

using Ctx = std::pair<int, std::string>;

bool is_index_op(OpK k) {
  switch (k) {
    case OpK::BroadcastInDim: case OpK::Reshape: case OpK::Transpose: case OpK::Slice: case OpK::Pad:
    case OpK::DynamicUpdateSlice: case OpK::DynamicSlice: case OpK::Concatenate: case OpK::Reverse: case OpK::Window: case OpK::Gather:
      return true;
    default:
      return false;
  }
}

bool is_arith(OpK k) {
  switch (k) {
    case OpK::Unary: case OpK::Binary: case OpK::Compare: case OpK::Select: case OpK::Clamp: case OpK::Gelu:
      return true;
    default:
      return false;
  }
}

const char* acc_ctype(DT dt) {
  if (dt == DT::F64) return "double";
  if (is_float(dt)) return "float";
  return info(dt).ctype;
}

std::string red_identity(Red r, DT dt) {
  const bool f = is_float(dt), d = dt == DT::F64;
  switch (r) {
    case Red::Add: case Red::Or: return dt == DT::I1 ? "false" : (f ? (d ? "0.0" : "0.0f") : "0");
    case Red::Mul: case Red::And:
      if (dt == DT::I1) return "true";
      if (r == Red::And) return std::string("(") + info(dt).ctype + ")(~0ull)";
      return f ? (d ? "1.0" : "1.0f") : "1";
    case Red::Max:
      if (f) return d ? "(-__builtin_inf())" : "(-__builtin_inff())";
      if (dt == DT::I1) return "false";
      if (!info(dt).is_signed) return "0";
      switch (info(dt).size) { case 1: return "(rx_i8)(-128)"; case 2: return "(rx_i16)(-32768)"; case 4: return "(-2147483647 - 1)"; default: return "(-9223372036854775807LL - 1)"; }
    case Red::Min:
      if (f) return d ? "__builtin_inf()" : "__builtin_inff()";
      if (dt == DT::I1) return "true";
      if (!info(dt).is_signed) return std::string("(") + info(dt).ctype + ")(~0ull)";
      switch (info(dt).size) { case 1: return "(rx_i8)127"; case 2: return "(rx_i16)32767"; case 4: return "2147483647"; default: return "9223372036854775807LL"; }
  }
  return "0";
}

const char* red_functor(Red r) {
  switch (r) {
    case Red::Add: return "rx_op_add()";
    case Red::Mul: return "rx_op_mul()";
    case Red::Max: return "rx_op_max()";
    case Red::Min: return "rx_op_min()";
    case Red::And: return "rx_op_and()";
    case Red::Or: return "rx_op_or()";
  }
  return "rx_op_add()";
}

std::string red_apply(Red r, DT dt, const std::string& a, const std::string& b) {
  if (dt == DT::I1) {
    if (r == Red::Add || r == Red::Or || r == Red::Max) return "(" + a + " || " + b + ")";
    return "(" + a + " && " + b + ")";
  }
  switch (r) {
    case Red::Add: return "(" + a + " + " + b + ")";
    case Red::Mul: return "(" + a + " * " + b + ")";
    case Red::Max: return "rx_max(" + a + ", " + b + ")";
    case Red::Min: return "rx_min(" + a + ", " + b + ")";
    case Red::And: return "(" + a + " & " + b + ")";
    case Red::Or: return "(" + a + " | " + b + ")";
  }
  return a;
}

// Thrown while planning when a convolution in the grid form did not take the whole elementwise chain that follows
// it into its kernel: the module is then planned again without that rewrite.
struct ChainNotAbsorbed {};

struct Planner {
  Graph g;  // canonicalized copy
  PlanOptions opt;
  Plan plan;
  std::vector<char> live, mat;
  std::vector<std::vector<int>> users;
  std::vector<std::set<Ctx>> ctx;
  std::vector<char> prev_mat;       // materialization decided by the previous analysis sweep (used for producers)
  std::vector<char> force_mat;      // chosen cut points below a dot_general with several consumers
  std::set<int> layout_entries;     // transposes that bring a tensor into a channel-minor region: written by a transposing map, not read across the layout by their readers
  std::vector<int> buf_of;          // node -> buffer id (materialized nodes)
  std::map<int, int> fuse_prev;     // stencil root -> the stencil step it evaluates in LDS instead of reading from memory
  std::set<int> lds_only;           // the steps absorbed that way: no launch, no buffer
  std::map<int, int> reshape_alias; // materialized reshape of a materialized value: the same bytes, no launch
  std::set<std::pair<int, int>> fused_operands;   // (dot_general, side): the operand is evaluated inside the GEMM's tile loads
  std::map<int, int> epilogue_of;   // dot_general -> the elementwise root that absorbs it (the product is launched there)
  std::map<int, int> row_anchor;    // reduction fused into a row kernel -> the root of that kernel
  std::ostringstream src;
  int kcount = 0;

  Planner(const Graph& gin, const PlanOptions& o) : g(gin), opt(o) {}

  // ------------------------------------------------------------------ rewrites
  void canonicalize() {
    const int N = (int)g.nodes.size();
    std::vector<int> nuse(N, 0);
    for (auto& n : g.nodes) for (int i : n.in) nuse[i]++;
    for (int r : g.results) nuse[r]++;
    for (auto& n : g.nodes) {
      // dot_general(transpose(X), Y): read X directly
      if (n.k == OpK::DotGeneral) {
        for (int side = 0; side < 2; ++side) {
          const Node& o = g.nodes[n.in[side]];
          auto& batch = side == 0 ? n.a0 : n.a1;
          auto& contr = side == 0 ? n.a2 : n.a3;
          if (o.k == OpK::Transpose && o.ty.rank() == 2 && batch.empty() && contr.size() == 1) {
            contr[0] = o.a0[contr[0]];
            n.in[side] = o.in[0];
          }
        }
        // operands widened from one narrow float type: contract the narrow data directly
        const Node &a = g.nodes[n.in[0]], &b = g.nodes[n.in[1]];
        if (a.k == OpK::Convert && b.k == OpK::Convert && n.ty.dt == DT::F32) {
          DT sa = g.nodes[a.in[0]].ty.dt, sb = g.nodes[b.in[0]].ty.dt;
          if (sa == sb && is_narrow_float(sa) && a.ty.dt == DT::F32 && b.ty.dt == DT::F32) {
            n.in[0] = a.in[0];
            n.in[1] = b.in[0];
          }
        }
      }
      // transpose(dot_general(X, Y)) on matrices: swap the operands instead
      if (n.k == OpK::Transpose && n.ty.rank() == 2 && n.a0 == std::vector<int64_t>{1, 0}) {
        const Node& d = g.nodes[n.in[0]];
        if (d.k == OpK::DotGeneral && nuse[d.id] == 1 && d.a0.empty() && g.nodes[d.in[0]].ty.rank() == 2 &&
            g.nodes[d.in[1]].ty.rank() == 2 && d.a2.size() == 1) {
          Node nd = d;
          nd.id = n.id;
          nd.ty = n.ty;
          nd.in = {d.in[1], d.in[0]};
          nd.a2 = d.a3;
          nd.a3 = d.a2;
          n = nd;
        }
      }
    }
    dots_to_reductions();
    normalize_dots();
    align_dots();
    split_dots();
    pools_between_convs();
    chain_convs();
    channel_minor_regions();
    pad_into_pools();
  }

  // Zero padding of a pooled value, where the windows do not overlap (size = stride, no dilation, the extent a whole
  // number of windows), is the pooling of the operand padded by that many windows: a window made of padding alone
  // reduces to zero -- the maximum of -inf and zeros, or a sum of zeros -- and the other windows are the same ones.
  // The padding then sits in the pooling kernel's reads and the padding map of the pooled value (the operand of the
  // next convolution) disappears.
  void pad_into_pools() {
    if (!opt.pad_into_pools) return;
    const int N = (int)g.nodes.size();
    std::vector<int> nuse(N, 0);
    for (auto& n : g.nodes) for (int i : n.in) nuse[i]++;
    for (int r : g.results) nuse[r]++;
    auto zero = [&](int x) {
      const Node& c = g.nodes[x];
      if (c.k != OpK::Constant || !c.splat || c.ty.rank() != 0) return false;
      for (uint8_t b : c.data) if (b) return false;
      return true;
    };
    std::map<int, int> pad_of_win, pad_of_red;   // window / reduction -> the padding that moves
    std::set<int> moved;
    for (const Node& p : g.nodes) {
      if (p.k != OpK::Pad || !zero(p.in[1]) || !is_float(p.ty.dt)) continue;
      const Node& r = g.nodes[p.in[0]];
      if (r.k != OpK::Reduce || nuse[r.id] != 1 || (r.red != Red::Max && r.red != Red::Add)) continue;
      const Node& w = g.nodes[r.in[0]];
      const int rank = p.ty.rank();
      if (w.k != OpK::Window || nuse[w.id] != 1 || g.nodes[w.in[0]].ty.rank() != rank || (int)r.a0.size() != rank) continue;
      // (not along the minor dimension: the pooling kernel's vectors of outputs would no longer be whole)
      bool ok = p.a0[rank - 1] == 0 && p.a1[rank - 1] == 0;
      for (int d = 0; d < rank; ++d) {
        ok = ok && r.a0[d] == d && w.a0[d] == w.a1[d] && w.a2[d] == 1 && g.nodes[w.in[0]].ty.dims[d] % w.a0[d] == 0 && p.a0[d] >= 0 && p.a1[d] >= 0 && p.a2[d] == 0;
      }
      // the reduction starts from the identity: -inf for a maximum, zero for a sum
      const Node& init = g.nodes[r.in[1]];
      if (init.k != OpK::Constant || !init.splat || init.ty.rank() != 0) continue;
      const double iv = splat_as_double(init);
      ok = ok && (r.red == Red::Max ? (std::isinf(iv) && iv < 0) : iv == 0.0);
      if (!ok) continue;
      pad_of_win[w.id] = p.id;
      pad_of_red[r.id] = p.id;
      moved.insert(p.id);
    }
    if (moved.empty()) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(N, -1);
    for (const Node& n : g.nodes) {
      Node c = n;
      for (int& i : c.in) i = remap[i];
      if (pad_of_win.count(n.id)) {
        const Node& p = g.nodes[pad_of_win[n.id]];
        const int rank = p.ty.rank();
        Node np = p;            // the padding, on the operand, in units of windows
        np.in = {remap[n.in[0]], remap[p.in[1]] >= 0 ? remap[p.in[1]] : -1};
        if (np.in[1] < 0) {     // the zero comes later in the list than the window: give the new padding one of its own
          Node z = g.nodes[p.in[1]];
          np.in[1] = out.add(z);
        }
        np.ty = g.nodes[n.in[0]].ty;
        for (int d = 0; d < rank; ++d) {
          np.a0[d] = p.a0[d] * n.a0[d];
          np.a1[d] = p.a1[d] * n.a0[d];
          np.ty.dims[d] += np.a0[d] + np.a1[d];
        }
        c.in = {out.add(np)};
        for (int d = 0; d < rank; ++d) c.ty.dims[rank + d] = p.ty.dims[d];
      } else if (pad_of_red.count(n.id)) {
        c.ty.dims = g.nodes[pad_of_red[n.id]].ty.dims;
      } else if (moved.count(n.id)) {
        remap[n.id] = remap[n.in[0]];
        continue;
      }
      remap[n.id] = out.add(c);
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // What pools_between_convs does for a chain, for a region: a connected set of values between products with row
  // shifts in which every op can run on either layout -- elementwise ops on tensors of one shape (residual additions
  // among them) whose other operands vary along the channels only, padding with a scalar, pooling windows -- with any
  // number of readers.  The region is rebuilt on [image, row, column, channel]; the transposes after the products
  // that feed it and before the products that read it disappear, a tensor that enters it from elsewhere is transposed
  // once on the way in, and a value that something outside reads (a reduction over the pixels, the module's result) is
  // transposed once on the way out.  Done when the transposes that disappear move at least one and a half times the
  // bytes of those that are added.
  void channel_minor_regions() {
    if (!opt.nhwc_regions || !opt.nhwc_pools || !opt.mfma) return;
    const int N = (int)g.nodes.size();
    std::vector<std::vector<int>> use(N);
    std::vector<char> is_res(N, 0);
    for (auto& n : g.nodes) for (int i : n.in) use[i].push_back(n.id);
    for (int r : g.results) is_res[r] = 1;
    auto elementwise = [](OpK k) { return k == OpK::Unary || k == OpK::Binary || k == OpK::Clamp || k == OpK::Gelu || k == OpK::Convert || k == OpK::Select || k == OpK::Compare; };
    std::vector<signed char> vec_memo(N, -1);
    std::function<bool(int, int)> channel_only = [&](int x, int depth) -> bool {
      if (vec_memo[x] >= 0) return vec_memo[x] != 0;
      const Node& n = g.nodes[x];
      bool ok = false;
      if (n.k == OpK::Constant) ok = n.splat;
      else if (n.k == OpK::BroadcastInDim) {
        const TType& st = g.nodes[n.in[0]].ty;
        ok = n.ty.rank() == 4 && (st.rank() == 0 || (st.rank() == 1 && n.a0.size() == 1 && n.a0[0] == 1 && st.dims[0] == n.ty.dims[1]));
      } else if (elementwise(n.k) && depth < 12) {
        ok = !n.in.empty();
        for (int i : n.in) ok = ok && channel_only(i, depth + 1);
      }
      vec_memo[x] = ok ? 1 : 0;
      return ok;
    };
    auto shifted_conv = [&](int x) { return g.nodes[x].k == OpK::Conv && !g.nodes[x].a3.empty(); };
    enum Role : char { None = 0, T1, Elem, PadOp, Win, Red, T2 };
    std::vector<char> role(N, None);
    for (const Node& n : g.nodes) {
      if (n.k == OpK::Transpose && n.ty.rank() == 4) {
        if (n.a0 == std::vector<int64_t>{0, 3, 1, 2} && g.nodes[n.in[0]].k == OpK::Conv && g.nodes[n.in[0]].a3.size() == 5 && use[n.in[0]].size() == 1 && !is_res[n.in[0]])
          role[n.id] = T1;
        else if (n.a0 == std::vector<int64_t>{0, 2, 3, 1} && !is_res[n.id] && !use[n.id].empty()) {
          bool all = true;
          for (int u : use[n.id]) all = all && shifted_conv(u) && g.nodes[u].in[0] == n.id && g.nodes[u].in[1] != n.id;
          if (all) role[n.id] = T2;
        }
      } else if (n.ty.rank() == 4 && elementwise(n.k) && n.k != OpK::Compare && n.k != OpK::Select && !channel_only(n.id, 0)) {
        bool ok = !n.in.empty();
        for (int i : n.in) ok = ok && (channel_only(i, 0) || (g.nodes[i].ty.rank() == 4 && g.nodes[i].ty.dims == n.ty.dims));
        if (ok) role[n.id] = Elem;
      } else if (n.k == OpK::Pad && n.ty.rank() == 4 && g.nodes[n.in[1]].ty.rank() == 0 && n.in[0] != n.in[1] && !channel_only(n.in[0], 0)) {
        role[n.id] = PadOp;
      } else if (n.k == OpK::Window && g.nodes[n.in[0]].ty.rank() == 4 && use[n.id].size() == 1 && !is_res[n.id]) {
        const Node& r = g.nodes[use[n.id][0]];
        if (r.k == OpK::Reduce && r.in[0] == n.id && r.a0 == std::vector<int64_t>{0, 1, 2, 3} && g.nodes[r.in[1]].ty.rank() == 0) { role[n.id] = Win; role[r.id] = Red; }
      }
    }
    // the tensor operands of a member
    auto tensor_ins = [&](const Node& n) {
      std::vector<int> t;
      if (role[n.id] == Elem) { for (int i : n.in) if (!channel_only(i, 0)) t.push_back(i); }
      else if (role[n.id] == PadOp || role[n.id] == Win || role[n.id] == Red || role[n.id] == T2) t.push_back(n.in[0]);
      return t;
    };
    // components over tensor edges between members
    std::vector<int> comp(N);
    for (int i = 0; i < N; ++i) comp[i] = i;
    std::function<int(int)> find = [&](int x) { while (comp[x] != x) x = comp[x] = comp[comp[x]]; return x; };
    for (const Node& n : g.nodes) {
      if (role[n.id] == None) continue;
      for (int i : tensor_ins(n)) if (role[i] != None && role[i] != T2) comp[find(n.id)] = find(i);
    }
    struct Tally { double saved = 0, added = 0; int t1 = 0, t2 = 0; std::set<int> entries, exits; };
    std::map<int, Tally> tally;
    for (const Node& n : g.nodes) {
      if (role[n.id] == None) continue;
      Tally& t = tally[find(n.id)];
      if (role[n.id] == T1) { t.saved += (double)n.ty.bytes(); ++t.t1; }
      if (role[n.id] == T2) { t.saved += (double)n.ty.bytes(); ++t.t2; }
      for (int i : tensor_ins(n))
        if (role[i] == None || role[i] == T2) { if (t.entries.insert(i).second) t.added += (double)g.nodes[i].ty.bytes(); }
      if (role[n.id] == T2 || role[n.id] == Win) continue;      // read by the products / by its reduction only
      bool outside = is_res[n.id];
      for (int u : use[n.id]) {
        bool inside = role[u] != None && role[u] != T1;
        if (inside) { bool reads = false; for (int i : tensor_ins(g.nodes[u])) reads = reads || i == n.id; inside = reads; }
        outside = outside || !inside;
      }
      if (outside && t.exits.insert(n.id).second) t.added += (double)n.ty.bytes();
    }
    std::set<int> chosen;
    for (auto& kv : tally)
      if (kv.second.t1 >= 1 && kv.second.t2 >= 1 && kv.second.saved >= opt.nhwc_region_ratio * kv.second.added) chosen.insert(kv.first);
    if (chosen.empty()) return;
    auto member = [&](int x) { return role[x] != None && chosen.count(find(x)) > 0; };
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(N, -1), nhwc(N, -1);
    static const int P[4] = {0, 3, 1, 2};      // old dimension i is new dimension P[i]
    auto permuted = [&](const std::vector<int64_t>& v) { std::vector<int64_t> r(4); for (int i = 0; i < 4; ++i) r[P[i]] = v[i]; return r; };
    std::map<std::pair<int, std::vector<int64_t>>, int> memo;
    std::function<int(int, const std::vector<int64_t>&)> rebuild_vec = [&](int x, const std::vector<int64_t>& dims) -> int {
      auto it = memo.find({x, dims});
      if (it != memo.end()) return it->second;
      Node c = g.nodes[x];
      c.ty.dims = dims;
      if (c.k == OpK::BroadcastInDim) {
        c.in = {remap[c.in[0]]};
        if (!c.a0.empty()) c.a0 = {3};
      } else if (c.k != OpK::Constant) {
        for (int& i : c.in) i = rebuild_vec(i, dims);
      }
      return memo[{x, dims}] = out.add(c);
    };
    // the value of old node x in the old layout (members of a chosen region exist in the new layout only)
    std::function<int(int)> old_layout = [&](int x) -> int {
      if (remap[x] >= 0) return remap[x];
      Node t;
      t.k = OpK::Transpose;
      t.in = {nhwc[x]};
      t.a0 = {0, 3, 1, 2};
      t.ty = g.nodes[x].ty;
      return remap[x] = out.add(t);
    };
    std::function<int(int)> new_layout = [&](int x) -> int {
      if (nhwc[x] >= 0) return nhwc[x];
      Node t;
      t.k = OpK::Transpose;
      t.in = {old_layout(x)};
      t.a0 = {0, 2, 3, 1};
      t.ty.dt = g.nodes[x].ty.dt;
      t.ty.dims = permuted(g.nodes[x].ty.dims);
      nhwc[x] = out.add(t);
      layout_entries.insert(nhwc[x]);
      return nhwc[x];
    };
    layout_entries.clear();
    for (const Node& n : g.nodes) {
      Node c = n;
      if (!member(n.id)) {
        for (int& i : c.in) i = old_layout(i);
        remap[n.id] = out.add(c);
        continue;
      }
      switch (role[n.id]) {
        case T1:
          nhwc[n.id] = old_layout(n.in[0]);      // the product's own result
          continue;
        case T2:
          remap[n.id] = new_layout(n.in[0]);     // what the products read
          continue;
        case Elem:
          c.ty.dims = permuted(n.ty.dims);
          for (int& i : c.in) i = channel_only(i, 0) ? rebuild_vec(i, c.ty.dims) : new_layout(i);
          break;
        case PadOp:
          c.ty.dims = permuted(n.ty.dims);
          c.a0 = permuted(n.a0); c.a1 = permuted(n.a1); c.a2 = permuted(n.a2);
          c.in = {new_layout(n.in[0]), old_layout(n.in[1])};
          break;
        case Win: {
          c.a0 = permuted(n.a0); c.a1 = permuted(n.a1); c.a2 = permuted(n.a2);
          const std::vector<int64_t> k = permuted(std::vector<int64_t>(n.ty.dims.begin(), n.ty.dims.begin() + 4));
          const std::vector<int64_t> o = permuted(std::vector<int64_t>(n.ty.dims.begin() + 4, n.ty.dims.end()));
          c.ty.dims = k;
          c.ty.dims.insert(c.ty.dims.end(), o.begin(), o.end());
          c.in = {new_layout(n.in[0])};
          break;
        }
        case Red:
          c.ty.dims = permuted(n.ty.dims);
          c.in = {nhwc[n.in[0]], old_layout(n.in[1])};
          break;
        default:
          break;
      }
      nhwc[n.id] = out.add(c);
    }
    for (int p : g.params) out.params.push_back(old_layout(p));
    for (int r : g.results) out.results.push_back(old_layout(r));
    g = std::move(out);
  }

  // Between two convolutions in the product-with-row-shifts form the values live as [image, row, column, channel]: the
  // first one's result is transposed to [image, channel, row, column] for the ops of the module and the second one's
  // operand is transposed back.  When everything in between can run in either layout -- elementwise ops whose other
  // operands vary along the channels only, padding with a scalar, pooling windows (a window view and its reduction)
  // -- and a pooling window is among them, those ops are rebuilt on the channel-minor layout and both transposes
  // disappear: the elementwise ops before the first window become the first product's epilogue, the window's reads
  // run along the channels (16-byte loads) instead of across a transposed operand, and the layout map of the second
  // product's operand is a plain padding map of the pooled values.  (Chains without a window are chain_convs's.)
  void pools_between_convs() {
    if (!opt.nhwc_pools || !opt.mfma) return;
    const int N = (int)g.nodes.size();
    std::vector<int> nuse(N, 0);
    std::vector<std::vector<int>> use(N);
    for (auto& n : g.nodes) for (int i : n.in) { nuse[i]++; use[i].push_back(n.id); }
    for (int r : g.results) nuse[r]++;
    auto elementwise = [](OpK k) { return k == OpK::Unary || k == OpK::Binary || k == OpK::Clamp || k == OpK::Gelu || k == OpK::Convert || k == OpK::Select || k == OpK::Compare; };
    std::vector<signed char> vec_memo(N, -1);
    std::function<bool(int, int)> channel_only = [&](int x, int depth) -> bool {
      if (vec_memo[x] >= 0) return vec_memo[x] != 0;
      const Node& n = g.nodes[x];
      bool ok = false;
      if (n.k == OpK::Constant) ok = n.splat;
      else if (n.k == OpK::BroadcastInDim) {
        const TType& st = g.nodes[n.in[0]].ty;
        ok = n.ty.rank() == 4 && (st.rank() == 0 || (st.rank() == 1 && n.a0.size() == 1 && n.a0[0] == 1 && st.dims[0] == n.ty.dims[1]));
      } else if (elementwise(n.k) && depth < 12) {
        ok = !n.in.empty();
        for (int i : n.in) ok = ok && channel_only(i, depth + 1);
      }
      vec_memo[x] = ok ? 1 : 0;
      return ok;
    };
    enum Role : char { None = 0, T1, Elem, PadOp, Win, Red, T2 };
    std::vector<char> role(N, None);
    bool any = false;
    for (const Node& t1 : g.nodes) {
      if (t1.k != OpK::Transpose || t1.a0 != std::vector<int64_t>{0, 3, 1, 2} || nuse[t1.id] != 1) continue;
      const Node& c1 = g.nodes[t1.in[0]];
      if (c1.k != OpK::Conv || c1.a3.size() != 5 || nuse[c1.id] != 1) continue;
      std::vector<std::pair<int, char>> found{{t1.id, T1}};
      int cur = t1.id;
      bool ok = false, pooled = false;
      for (int depth = 0; depth < 24; ++depth) {
        if (nuse[cur] != 1 || use[cur].size() != 1) break;
        const Node& u = g.nodes[use[cur][0]];
        if (u.k == OpK::Transpose) {
          ok = u.a0 == std::vector<int64_t>{0, 2, 3, 1} && nuse[u.id] == 1 && use[u.id].size() == 1 && g.nodes[use[u.id][0]].k == OpK::Conv &&
               g.nodes[use[u.id][0]].a3.size() == 5 && g.nodes[use[u.id][0]].in[0] == u.id;
          found.push_back({u.id, T2});
          break;
        }
        if (u.ty.rank() != 4 && u.k != OpK::Window) break;
        if (elementwise(u.k) && u.k != OpK::Compare && u.k != OpK::Select) {
          int tensors = 0;
          for (int i : u.in) if (i == cur) ++tensors; else if (!channel_only(i, 0)) tensors = 99;
          if (tensors != 1) break;
          found.push_back({u.id, Elem});
          cur = u.id;
        } else if (u.k == OpK::Pad) {
          if (u.in[0] != cur || u.in[1] == cur || g.nodes[u.in[1]].ty.rank() != 0) break;
          found.push_back({u.id, PadOp});
          cur = u.id;
        } else if (u.k == OpK::Window) {
          if (g.nodes[cur].ty.rank() != 4 || nuse[u.id] != 1 || use[u.id].size() != 1) break;
          const Node& r = g.nodes[use[u.id][0]];
          if (r.k != OpK::Reduce || r.in[0] != u.id || r.a0 != std::vector<int64_t>{0, 1, 2, 3} || g.nodes[r.in[1]].ty.rank() != 0) break;
          found.push_back({u.id, Win});
          found.push_back({r.id, Red});
          pooled = true;
          cur = r.id;
        } else break;
      }
      if (!ok || !pooled) continue;
      for (auto& f : found) role[f.first] = f.second;
      any = true;
    }
    if (!any) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(N, -1);
    // old dimension i is new dimension P[i]
    static const int P[4] = {0, 3, 1, 2};
    auto permuted = [&](const std::vector<int64_t>& v) { std::vector<int64_t> r(4); for (int i = 0; i < 4; ++i) r[P[i]] = v[i]; return r; };
    std::map<std::pair<int, std::vector<int64_t>>, int> memo;
    std::function<int(int, const std::vector<int64_t>&)> rebuild_vec = [&](int x, const std::vector<int64_t>& dims) -> int {
      auto it = memo.find({x, dims});
      if (it != memo.end()) return it->second;
      Node c = g.nodes[x];
      c.ty.dims = dims;
      if (c.k == OpK::BroadcastInDim) {
        c.in = {remap[c.in[0]]};
        if (!c.a0.empty()) c.a0 = {3};
      } else if (c.k != OpK::Constant) {
        for (int& i : c.in) i = rebuild_vec(i, dims);
      }
      return memo[{x, dims}] = out.add(c);
    };
    for (const Node& n : g.nodes) {
      Node c = n;
      switch (role[n.id]) {
        case T1: case T2:
          remap[n.id] = remap[n.in[0]];
          continue;
        case Elem: {
          c.ty.dims = permuted(n.ty.dims);
          for (int& i : c.in) i = role[i] != None ? remap[i] : rebuild_vec(i, c.ty.dims);
          break;
        }
        case PadOp:
          c.ty.dims = permuted(n.ty.dims);
          c.a0 = permuted(n.a0); c.a1 = permuted(n.a1); c.a2 = permuted(n.a2);
          for (int& i : c.in) i = remap[i];
          break;
        case Win: {
          c.a0 = permuted(n.a0); c.a1 = permuted(n.a1); c.a2 = permuted(n.a2);
          const std::vector<int64_t> k = permuted(std::vector<int64_t>(n.ty.dims.begin(), n.ty.dims.begin() + 4));
          const std::vector<int64_t> o = permuted(std::vector<int64_t>(n.ty.dims.begin() + 4, n.ty.dims.end()));
          c.ty.dims = k;
          c.ty.dims.insert(c.ty.dims.end(), o.begin(), o.end());
          for (int& i : c.in) i = remap[i];
          break;
        }
        case Red:
          c.ty.dims = permuted(n.ty.dims);
          for (int& i : c.in) i = remap[i];
          break;
        default:
          for (int& i : c.in) i = remap[i];
      }
      remap[n.id] = out.add(c);
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // Two convolutions in the product-with-row-shifts form (OpK::Conv with a3) with nothing between them but elementwise
  // ops whose other operands vary along the channels only (bias, batch norm, activation) and the zero padding of the
  // second one, on the same padded grid (same batch, HP x WP): the first product keeps its rows on that grid instead of
  // packing the results -- the epilogue writes row m to row m + (top padding * WP + left padding), zero where row m is
  // not a result, and zeros to the rows before that offset -- which is the second product's zero-padded operand: a
  // result's grid position (y, x) moves to (y + top, x + left), and the positions that are not results (the last rows
  // and columns of every image's grid) move onto the borders, each border position exactly once.  The elementwise ops
  // become the first product's epilogue; the map between the two products disappears.
  void chain_convs() {
    if (!opt.chain_convs || !opt.mfma) return;
    const int N = (int)g.nodes.size();
    std::vector<int> nuse(N, 0);
    for (auto& n : g.nodes) for (int i : n.in) nuse[i]++;
    for (int r : g.results) nuse[r]++;
    auto elementwise = [](OpK k) { return k == OpK::Unary || k == OpK::Binary || k == OpK::Clamp || k == OpK::Gelu || k == OpK::Convert || k == OpK::Select || k == OpK::Compare; };
    // value varies along dimension 1 (the channels of [B, C, H, W]) only
    std::vector<signed char> vec_memo(N, -1);
    std::function<bool(int, int)> channel_only = [&](int x, int depth) -> bool {
      if (vec_memo[x] >= 0) return vec_memo[x] != 0;
      const Node& n = g.nodes[x];
      bool ok = false;
      if (n.k == OpK::Constant) ok = n.splat;
      else if (n.k == OpK::BroadcastInDim) {
        const TType& st = g.nodes[n.in[0]].ty;
        ok = n.ty.rank() == 4 && (st.rank() == 0 || (st.rank() == 1 && n.a0.size() == 1 && n.a0[0] == 1 && st.dims[0] == n.ty.dims[1]));
      } else if (elementwise(n.k) && depth < 12) {
        ok = !n.in.empty();
        for (int i : n.in) ok = ok && channel_only(i, depth + 1);
      }
      vec_memo[x] = ok ? 1 : 0;
      return ok;
    };
    struct Match { int c1, t1, pad, t2, c2; std::vector<int> chain; int64_t shift; };
    std::vector<Match> matches;
    std::vector<char> taken(N, 0);
    for (const Node& c2 : g.nodes) {
      if (c2.k != OpK::Conv || c2.a3.size() != 5) continue;
      Match m;
      m.c2 = c2.id;
      m.t2 = c2.in[0];
      const Node& t2 = g.nodes[m.t2];
      if (t2.k != OpK::Transpose || t2.a0 != std::vector<int64_t>{0, 2, 3, 1} || nuse[m.t2] != 1) continue;
      int cur = t2.in[0];
      m.pad = -1;
      int64_t pt = 0, pl = 0;
      if (g.nodes[cur].k == OpK::Pad) {
        const Node& p = g.nodes[cur];
        const Node& pv = g.nodes[p.in[1]];
        bool zero = pv.k == OpK::Constant && pv.splat;
        for (uint8_t b : pv.data) zero = zero && b == 0;
        if (!zero || nuse[cur] != 1 || p.a0.size() != 4 || p.a0[0] || p.a0[1] || p.a1[0] || p.a1[1] || p.a2 != std::vector<int64_t>{0, 0, 0, 0} ||
            p.a0[2] < 0 || p.a0[3] < 0 || p.a1[2] < 0 || p.a1[3] < 0) continue;
        m.pad = cur;
        pt = p.a0[2];
        pl = p.a0[3];
        cur = p.in[0];
      }
      bool ok = true;
      m.t1 = -1;
      for (int depth = 0; depth < 16 && ok; ++depth) {
        const Node& n = g.nodes[cur];
        if (nuse[cur] != 1 || taken[cur]) { ok = false; break; }
        if (n.k == OpK::Transpose) {
          ok = n.a0 == std::vector<int64_t>{0, 3, 1, 2};
          m.t1 = cur;
          break;
        }
        if (!elementwise(n.k) || n.k == OpK::Compare || n.k == OpK::Select || n.ty.rank() != 4) { ok = false; break; }
        int tensor = -1;
        for (int i : n.in) {
          if (channel_only(i, 0)) continue;
          if (tensor >= 0) ok = false;
          tensor = i;
        }
        if (tensor < 0) ok = false;
        m.chain.push_back(cur);
        cur = tensor;
      }
      if (!ok || m.t1 < 0) continue;
      m.c1 = g.nodes[m.t1].in[0];
      const Node& c1 = g.nodes[m.c1];
      if (c1.k != OpK::Conv || c1.a3.size() != 5 || nuse[m.c1] != 1 || taken[m.c1] || m.c1 == m.c2) continue;
      // the same grid, the second operand's channels as the first product delivers them, results where the padding puts them
      const TType& x2 = t2.ty;   // [B, HP, WP, C]
      if (x2.rank() != 4 || c1.ty.rank() != 4 || x2.dims[0] != c1.ty.dims[0] || x2.dims[1] != c1.a3[3] || x2.dims[2] != c1.a3[4] || x2.dims[3] != c1.ty.dims[3] ||
          c2.a3[3] != c1.a3[3] || c2.a3[4] != c1.a3[4] || x2.dims[1] - c1.ty.dims[1] < pt || x2.dims[2] - c1.ty.dims[2] < pl)
        continue;
      if (m.pad >= 0) {
        const Node& p = g.nodes[m.pad];
        if (c1.ty.dims[1] + pt + p.a1[2] != x2.dims[1] || c1.ty.dims[2] + pl + p.a1[3] != x2.dims[2]) continue;
      } else if (c1.ty.dims[1] != x2.dims[1] || c1.ty.dims[2] != x2.dims[2]) continue;
      m.shift = pt * c1.a3[4] + pl;
      for (int x : m.chain) taken[x] = 1;
      taken[m.c1] = taken[m.t1] = taken[m.t2] = 1;
      if (m.pad >= 0) taken[m.pad] = 1;
      matches.push_back(m);
    }
    if (matches.empty()) return;
    std::map<int, const Match*> by_c1, by_t1, by_chain, by_pad, by_t2;
    for (auto& m : matches) {
      by_c1[m.c1] = &m; by_t1[m.t1] = &m; by_t2[m.t2] = &m;
      if (m.pad >= 0) by_pad[m.pad] = &m;
      for (int x : m.chain) by_chain[x] = &m;
    }
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(N, -1);
    // a channel-only value rebuilt on [B, HP, WP, C]
    std::function<int(int, const std::vector<int64_t>&, std::map<int, int>&)> rebuild_vec = [&](int x, const std::vector<int64_t>& dims, std::map<int, int>& memo) -> int {
      auto it = memo.find(x);
      if (it != memo.end()) return it->second;
      Node c = g.nodes[x];
      c.ty.dims = dims;
      if (c.k == OpK::BroadcastInDim) {
        c.in = {remap[c.in[0]]};
        if (!c.a0.empty()) c.a0 = {3};
      } else if (c.k != OpK::Constant) {
        for (int& i : c.in) i = rebuild_vec(i, dims, memo);
      }
      return memo[x] = out.add(c);
    };
    std::map<const Match*, std::map<int, int>> memos;
    for (const Node& n : g.nodes) {
      if (by_c1.count(n.id)) {
        const Match& m = *by_c1[n.id];
        Node c = n;
        for (int& i : c.in) i = remap[i];
        c.a3 = {n.a3[0], n.a3[1], n.a3[2], n.a3[3], n.a3[4], n.ty.dims[1], n.ty.dims[2], m.shift};
        c.ty.dims = {n.ty.dims[0], n.a3[3], n.a3[4], n.ty.dims[3]};
        remap[n.id] = out.add(c);
        continue;
      }
      if (by_t1.count(n.id)) { remap[n.id] = remap[n.in[0]]; continue; }
      if (by_chain.count(n.id)) {
        const Match& m = *by_chain[n.id];
        const Node& c1 = g.nodes[m.c1];
        const std::vector<int64_t> dims{c1.ty.dims[0], c1.a3[3], c1.a3[4], c1.ty.dims[3]};
        Node c = n;
        c.ty.dims = dims;
        for (int& i : c.in) i = channel_only(i, 0) ? rebuild_vec(i, dims, memos[&m]) : remap[i];
        remap[n.id] = out.add(c);
        continue;
      }
      if (by_pad.count(n.id)) { remap[n.id] = remap[n.in[0]]; continue; }
      if (by_t2.count(n.id)) { remap[n.id] = remap[n.in[0]]; continue; }
      Node c = n;
      for (int& i : c.in) i = remap[i];
      remap[n.id] = out.add(c);
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // A dot_general with several batch, free or contracting dims, or with them in another order than
  // [batch, rows, k] / [batch, k, rows], is brought to the (batched) matrix form the GEMM skeletons
  // understand: each operand is reshaped when its dims are already grouped that way (free of
  // charge) and transposed first when they are not; the result is reshaped back.
  void normalize_dots() {
    if (!opt.mfma) return;
    struct Form {
      std::vector<int64_t> perm[2];   // operand dims in the order batch.., free.., contract.. (or batch.., contract.., free..)
      bool kc[2];                     // contract dims last
      bool transpose[2];
      int64_t B, M, N, K;
    };
    std::map<int, Form> forms;
    for (const Node& d : g.nodes) {
      if (d.k != OpK::DotGeneral || d.a2.empty()) continue;
      if (dot_form(d).ok) continue;
      const TType &lt = g.nodes[d.in[0]].ty, &rt = g.nodes[d.in[1]].ty;
      if (lt.numel() == 0 || rt.numel() == 0 || d.ty.numel() == 0) continue;
      Form f;
      // contracting pairs in the order of the lhs dims
      std::vector<std::pair<int64_t, int64_t>> cp;
      for (size_t k = 0; k < d.a2.size(); ++k) cp.push_back({d.a2[k], d.a3[k]});
      std::sort(cp.begin(), cp.end());
      auto isin = [](const std::vector<int64_t>& v, int64_t x) { return std::find(v.begin(), v.end(), x) != v.end(); };
      f.B = f.M = f.N = f.K = 1;
      for (auto b : d.a0) f.B *= lt.dims[b];
      for (auto& c : cp) f.K *= lt.dims[c.first];
      for (int side = 0; side < 2; ++side) {
        const TType& t = side == 0 ? lt : rt;
        const auto& batch = side == 0 ? d.a0 : d.a1;
        const auto& contr = side == 0 ? d.a2 : d.a3;
        std::vector<int64_t> fr, ct;
        for (int k = 0; k < t.rank(); ++k) if (!isin(batch, k) && !isin(contr, k)) fr.push_back(k);
        for (auto& c : cp) ct.push_back(side == 0 ? c.first : c.second);
        for (auto k : fr) (side == 0 ? f.M : f.N) *= t.dims[k];
        std::vector<int64_t> p_kc = batch, p_tr = batch;
        p_kc.insert(p_kc.end(), fr.begin(), fr.end());
        p_kc.insert(p_kc.end(), ct.begin(), ct.end());
        p_tr.insert(p_tr.end(), ct.begin(), ct.end());
        p_tr.insert(p_tr.end(), fr.begin(), fr.end());
        auto identity = [](const std::vector<int64_t>& p) { for (size_t k = 0; k < p.size(); ++k) if (p[k] != (int64_t)k) return false; return true; };
        if (identity(p_kc)) { f.perm[side] = p_kc; f.kc[side] = true; f.transpose[side] = false; }
        else if (identity(p_tr)) { f.perm[side] = p_tr; f.kc[side] = false; f.transpose[side] = false; }
        else { f.perm[side] = p_kc; f.kc[side] = true; f.transpose[side] = true; }
      }
      // worth it only if the matrix form reaches a skeleton (possibly after padding to whole vectors) or the reduction form
      const DT a = lt.dt, b = rt.dt;
      const int64_t ve = 16 / info(a).size;
      auto up = [](int64_t x, int64_t m) { return (x + m - 1) / m * m; };
      if (!choose_gemm(a, b, d.ty.dt, f.B, f.kc[0] ? f.M : up(f.M, ve), up(f.N, std::max<int64_t>(4, ve)), up(f.K, ve), f.kc[0], f.kc[1]).ok) continue;
      forms[d.id] = f;
    }
    if (forms.empty()) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(g.nodes.size(), -1);
    for (const Node& n : g.nodes) {
      Node c = n;
      for (int& i : c.in) i = remap[i];
      auto fi = forms.find(n.id);
      if (fi == forms.end()) { remap[n.id] = out.add(c); continue; }
      const Form& f = fi->second;
      const bool batched = !n.a0.empty();
      int opnd[2];
      for (int side = 0; side < 2; ++side) {
        int cur = c.in[side];
        const TType t = out.nodes[cur].ty;
        if (f.transpose[side]) {
          Node tr;
          tr.k = OpK::Transpose;
          tr.in = {cur};
          tr.a0 = f.perm[side];
          tr.ty.dt = t.dt;
          for (auto pdim : f.perm[side]) tr.ty.dims.push_back(t.dims[pdim]);
          cur = out.add(tr);
        }
        const int64_t rows = side == 0 ? f.M : f.N;
        std::vector<int64_t> md;
        if (batched) md.push_back(f.B);
        if (f.kc[side]) { md.push_back(rows); md.push_back(f.K); } else { md.push_back(f.K); md.push_back(rows); }
        if (out.nodes[cur].ty.dims != md) {
          Node rs;
          rs.k = OpK::Reshape;
          rs.in = {cur};
          rs.ty = TType{t.dt, md};
          cur = out.add(rs);
        }
        opnd[side] = cur;
      }
      Node dn;
      dn.k = OpK::DotGeneral;
      dn.op = n.op;
      dn.in = {opnd[0], opnd[1]};
      const int64_t nb = batched ? 1 : 0;
      if (batched) { dn.a0 = {0}; dn.a1 = {0}; }
      dn.a2 = {nb + (f.kc[0] ? 1 : 0)};
      dn.a3 = {nb + (f.kc[1] ? 1 : 0)};
      dn.ty.dt = n.ty.dt;
      if (batched) dn.ty.dims.push_back(f.B);
      dn.ty.dims.push_back(f.M);
      dn.ty.dims.push_back(f.N);
      int cur = out.add(dn);
      if (out.nodes[cur].ty.dims != n.ty.dims) {
        Node rs;
        rs.k = OpK::Reshape;
        rs.in = {cur};
        rs.ty = n.ty;
        cur = out.add(rs);
      }
      remap[n.id] = cur;
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // A dot_general operand that is a cheap expansion of much smaller data -- the window matrix of a
  // convolution, a broadcast -- is not written to memory: the GEMM evaluates it while it loads
  // its tiles (a functor in place of the operand pointer), reading the small data through the caches.
  void decide_fused_operands() {
    fused_operands.clear();
    if (!opt.mfma || !opt.fuse_dot_operands) return;
    const int N = (int)g.nodes.size();
    std::vector<int> nuse(N, 0);
    for (auto& n : g.nodes) for (int i : n.in) nuse[i]++;
    for (int r : g.results) nuse[r]++;
    auto is_leaf = [](const Node& n) {
      return n.k == OpK::Param || (n.k == OpK::Constant && !n.splat) || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv || n.k == OpK::DotGeneral;
    };
    for (const Node& d : g.nodes) {
      if (d.k != OpK::DotGeneral || d.ty.rank() < 2 || !d.a4.empty()) continue;
      DotForm f = dot_form(d);
      if (!f.ok) continue;
      const DT a = g.nodes[d.in[0]].ty.dt, b = g.nodes[d.in[1]].ty.dt;
      if (!choose_gemm(a, b, d.ty.dt, f.batch, f.M, f.N, f.K, f.a_k_contig, f.b_k_contig, true).ok) continue;
      for (int side = 0; side < 2; ++side) {
        const int x = d.in[side];
        const Node& xn = g.nodes[x];
        if (is_leaf(xn) || xn.k == OpK::Constant || nuse[x] != 1) continue;
        // every tile row (column) of the product evaluates the operand again; with more than one or two
        // of them the expanded matrix is cheaper (3x3 256 -> 256 features on 14x14 images: 0.12 ms
        // with the window matrix in memory, 0.15 ms evaluated four times over)
        if ((side == 1 ? f.M : f.N) > 128) continue;
        std::set<int> seen;
        std::vector<int> st{x};
        double leaf = 0;
        int count = 0;
        bool ok = true;
        while (!st.empty() && ok) {
          const int y = st.back();
          st.pop_back();
          if (!seen.insert(y).second) continue;
          const Node& yn = g.nodes[y];
          if (is_leaf(yn)) { leaf += (double)yn.ty.numel(); continue; }
          if (yn.k == OpK::Constant) continue;
          if (yn.k == OpK::Gather) { ok = false; break; }   // data-dependent addresses: keep the plain path
          if (++count > 48) ok = false;
          for (int i : yn.in) st.push_back(i);
        }
        if (!ok || (double)xn.ty.numel() < 3.0 * leaf) continue;
        fused_operands.insert({d.id, side});
      }
    }
  }

  // A matrix product that misses the MFMA path only because a dimension is not a whole number of
  // 16-byte vectors (an odd N, a K of 27) is padded with zeros to the next multiple and the
  // padding sliced off the result: two small copies instead of the scalar loop.
  void align_dots() {
    if (!opt.mfma) return;
    struct Fix { int64_t Mp, Np, Kp; };
    std::map<int, Fix> fixes;
    for (const Node& d : g.nodes) {
      if (d.k != OpK::DotGeneral) continue;
      DotForm f = dot_form(d);
      if (!f.ok || d.ty.rank() < 2) continue;
      const DT a = g.nodes[d.in[0]].ty.dt, b = g.nodes[d.in[1]].ty.dt;
      if (a != b || !is_float(a) || a == DT::F8E5M2) continue;
      if (choose_gemm(a, b, d.ty.dt, f.batch, f.M, f.N, f.K, f.a_k_contig, f.b_k_contig).ok) continue;
      if ((double)f.M * (double)f.N * (double)f.K * (double)f.batch < (double)(1 << 22)) continue;   // small: the scalar loop will do
      const int64_t ve = 16 / info(a).size;
      auto up = [](int64_t x, int64_t m) { return (x + m - 1) / m * m; };
      Fix fx;
      fx.Kp = up(f.K, ve);
      fx.Mp = f.a_k_contig ? f.M : up(f.M, ve);
      fx.Np = up(f.N, f.b_k_contig ? 4 : std::max<int64_t>(4, ve));
      if (fx.Kp == f.K && fx.Mp == f.M && fx.Np == f.N) continue;
      if (!choose_gemm(a, b, d.ty.dt, f.batch, fx.Mp, fx.Np, fx.Kp, f.a_k_contig, f.b_k_contig).ok) continue;
      fixes[d.id] = fx;
    }
    if (fixes.empty()) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(g.nodes.size(), -1);
    for (const Node& n : g.nodes) {
      Node c = n;
      for (int& i : c.in) i = remap[i];
      auto fi = fixes.find(n.id);
      if (fi == fixes.end()) { remap[n.id] = out.add(c); continue; }
      const Fix& fx = fi->second;
      DotForm f = dot_form(n);
      const int nb = (int)n.a0.size();
      auto padded = [&](int node, bool kc, int64_t rows_to, int64_t k_to) {
        // operand dims [batch.., rows, K] (kc) or [batch.., K, rows]
        const TType t = out.nodes[node].ty;
        std::vector<int64_t> want = t.dims;
        want[nb + (kc ? 0 : 1)] = rows_to;
        want[nb + (kc ? 1 : 0)] = k_to;
        if (want == t.dims) return node;
        Node z;
        z.k = OpK::Constant;
        z.splat = true;
        z.ty = TType{t.dt, {}};
        z.data.assign((size_t)info(t.dt).size, 0);
        const int zi = out.add(z);
        Node pn;
        pn.k = OpK::Pad;
        pn.in = {node, zi};
        pn.a0.assign(t.rank(), 0);
        pn.a2.assign(t.rank(), 0);
        for (int k = 0; k < t.rank(); ++k) pn.a1.push_back(want[k] - t.dims[k]);
        pn.ty = TType{t.dt, want};
        return out.add(pn);
      };
      c.in[0] = padded(c.in[0], f.a_k_contig, fx.Mp, fx.Kp);
      c.in[1] = padded(c.in[1], f.b_k_contig, fx.Np, fx.Kp);
      c.ty.dims[nb] = fx.Mp;
      c.ty.dims[nb + 1] = fx.Np;
      int cur = out.add(c);
      Node sl;
      sl.k = OpK::Slice;
      sl.in = {cur};
      sl.a0.assign(n.ty.rank(), 0);
      sl.a1 = n.ty.dims;
      sl.a2.assign(n.ty.rank(), 1);
      sl.ty = n.ty;
      remap[n.id] = out.add(sl);
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // A matrix product with few output tiles and a long contraction (the last product of a chain, a
  // Gram matrix of tall data, the filter gradient of a convolution) leaves most compute units idle:
  // K is cut into S slices, workgroup (tile, s) contracts slice s into a partial product
  // [S, M, N] in f32, and a reduction over the leading index adds the slices up.
  void split_dots() {
    if (!opt.mfma || !opt.split_k) return;
    std::map<int, int> splits;
    for (const Node& d : g.nodes) {
      if (d.k != OpK::DotGeneral || d.ty.rank() != 2 || !d.a0.empty()) continue;
      DotForm f = dot_form(d);
      if (!f.ok || f.batch != 1) continue;
      const DT a = g.nodes[d.in[0]].ty.dt, b = g.nodes[d.in[1]].ty.dt;
      if (a != b || !is_float(a) || a == DT::F64 || !is_float(d.ty.dt)) continue;
      if (!choose_gemm(a, b, d.ty.dt, 1, f.M, f.N, f.K, f.a_k_contig, f.b_k_contig).ok) continue;
      const int64_t tiles = ((f.M + 63) / 64) * ((f.N + 63) / 64);
      if (tiles >= 256 || f.K < 1024) continue;
      // enough slices for two workgroups per compute unit, each slice at least 512 long
      int S = 1;
      while (S < 256 && tiles * S < 512 && f.K / (2 * S) >= 512) S *= 2;
      for (; S > 1; S /= 2) {
        if (f.K % S) continue;
        GemmChoice c = choose_gemm(a, b, DT::F32, 1, f.M, f.N, f.K, f.a_k_contig, f.b_k_contig, false, S);
        if (c.ok && c.split == S) break;
      }
      if (S > 1) splits[d.id] = S;
    }
    if (splits.empty()) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(g.nodes.size(), -1);
    for (const Node& n : g.nodes) {
      Node c = n;
      for (int& i : c.in) i = remap[i];
      auto si = splits.find(n.id);
      if (si == splits.end()) { remap[n.id] = out.add(c); continue; }
      const int S = si->second;
      c.a4 = {S};
      c.ty = TType{DT::F32, {S, n.ty.dims[0], n.ty.dims[1]}};
      const int part = out.add(c);
      Node zero;
      zero.k = OpK::Constant;
      zero.splat = true;
      zero.ty = TType{DT::F32, {}};
      zero.data.assign(4, 0);
      const int pz = out.add(zero);
      Node red;
      red.k = OpK::Reduce;
      red.red = Red::Add;
      red.in = {part, pz};
      red.a0 = {0};
      red.ty = TType{DT::F32, n.ty.dims};
      int cur = out.add(red);
      if (n.ty.dt != DT::F32) {
        Node cv;
        cv.k = OpK::Convert;
        cv.ty = n.ty;
        cv.in = {cur};
        cur = out.add(cv);
      }
      remap[n.id] = cur;
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // A dot_general whose smaller operand has at most 8 free elements (matrix-vector, vector-matrix,
  // inner products, a handful of right-hand sides) moves every element of the larger operand once and
  // does a few flops on it: it is a reduction, not a matrix product.  It is rewritten into
  // reduce(multiply(broadcast(big), broadcast(small))) laid out in the large operand's own dimension
  // order, so that the row / column / full reduction kernels stream that operand with coalesced
  // vector loads.  Narrow floats are multiplied and summed in f32 and rounded once.
  struct DotAsReduce {
    bool ok = false;
    bool big_is_lhs = true;
    std::vector<int> lfree, rfree;
  };
  DotAsReduce dot_as_reduction(const Node& d) const {
    DotAsReduce r;
    if (!opt.dot_as_reduce || d.k != OpK::DotGeneral || d.a2.empty()) return r;
    const TType &lt = g.nodes[d.in[0]].ty, &rt = g.nodes[d.in[1]].ty;
    if (lt.dt != rt.dt || lt.dt == DT::I1 || d.ty.dt == DT::I1) return r;
    if (is_float(lt.dt) != is_float(d.ty.dt)) return r;
    auto isin = [](const std::vector<int64_t>& v, int x) { return std::find(v.begin(), v.end(), (int64_t)x) != v.end(); };
    int64_t mfree = 1, nfree = 1, kprod = 1;
    for (int k = 0; k < lt.rank(); ++k) if (!isin(d.a0, k) && !isin(d.a2, k)) { r.lfree.push_back(k); mfree *= lt.dims[k]; }
    for (int k = 0; k < rt.rank(); ++k) if (!isin(d.a1, k) && !isin(d.a3, k)) { r.rfree.push_back(k); nfree *= rt.dims[k]; }
    for (auto c : d.a2) kprod *= lt.dims[c];
    r.big_is_lhs = lt.numel() >= rt.numel();
    if ((r.big_is_lhs ? nfree : mfree) > 8) return r;
    if (kprod < 1 || d.ty.numel() < 1) return r;
    // short contractions: one thread per output element walks them as fast
    if (kprod < 128) return r;
    r.ok = true;
    return r;
  }

  void dots_to_reductions() {
    bool any = false;
    for (auto& n : g.nodes) any = any || dot_as_reduction(n).ok;
    if (!any) return;
    Graph out;
    out.name = g.name;
    out.module_name = g.module_name;
    out.aliasing_output = g.aliasing_output;
    std::vector<int> remap(g.nodes.size(), -1);
    for (const Node& n : g.nodes) {
      DotAsReduce f = dot_as_reduction(n);
      if (!f.ok) {
        Node c = n;
        for (int& i : c.in) i = remap[i];
        remap[n.id] = out.add(c);
        continue;
      }
      const Node& d = n;
      const int bigside = f.big_is_lhs ? 0 : 1;
      const TType bt = g.nodes[d.in[bigside]].ty, st = g.nodes[d.in[1 - bigside]].ty;
      const auto& bbatch = bigside == 0 ? d.a0 : d.a1;
      const auto& sbatch = bigside == 0 ? d.a1 : d.a0;
      const auto& bcontr = bigside == 0 ? d.a2 : d.a3;
      const auto& scontr = bigside == 0 ? d.a3 : d.a2;
      const auto& bfree = bigside == 0 ? f.lfree : f.rfree;
      const auto& sfree = bigside == 0 ? f.rfree : f.lfree;
      // product dims: the big operand's dims in order, the small operand's free dims after the big
      // operand's last kept dim
      int ins = 0;
      for (int k = 0; k < bt.rank(); ++k)
        if (std::find(bcontr.begin(), bcontr.end(), (int64_t)k) == bcontr.end()) ins = k + 1;
      struct PD { int64_t size; int role; int idx; };  // role 0 batch(j) 1 lhs free(dim) 2 rhs free(dim) 3 contract(j)
      std::vector<PD> pd;
      std::vector<int64_t> bmap(bt.rank()), smap(st.rank(), -1);
      auto push_big = [&](int k) {
        PD e{bt.dims[k], 0, 0};
        auto bi = std::find(bbatch.begin(), bbatch.end(), (int64_t)k);
        auto ci = std::find(bcontr.begin(), bcontr.end(), (int64_t)k);
        if (bi != bbatch.end()) { e.role = 0; e.idx = (int)(bi - bbatch.begin()); smap[sbatch[e.idx]] = (int64_t)pd.size(); }
        else if (ci != bcontr.end()) { e.role = 3; e.idx = (int)(ci - bcontr.begin()); smap[scontr[e.idx]] = (int64_t)pd.size(); }
        else { e.role = bigside == 0 ? 1 : 2; e.idx = k; }
        bmap[k] = (int64_t)pd.size();
        pd.push_back(e);
      };
      for (int k = 0; k < ins; ++k) push_big(k);
      for (int k : sfree) { smap[k] = (int64_t)pd.size(); pd.push_back({st.dims[k], bigside == 0 ? 2 : 1, k}); }
      for (int k = ins; k < bt.rank(); ++k) push_big(k);
      (void)bfree;
      std::vector<int64_t> pdims;
      for (auto& e : pd) pdims.push_back(e.size);

      const DT CT = (is_narrow_float(bt.dt) || is_narrow_float(d.ty.dt)) ? DT::F32 : d.ty.dt;
      auto unary_node = [&](OpK k, int in, TType ty) {
        Node c;
        c.k = k;
        c.ty = ty;
        c.in = {in};
        return c;
      };
      auto operand = [&](int src_old, const TType& sty, const std::vector<int64_t>& map) {
        int cur = remap[src_old];
        if (sty.dt != CT) cur = out.add(unary_node(OpK::Convert, cur, TType{CT, sty.dims}));
        bool identity = sty.dims == pdims;
        for (size_t k = 0; k < map.size(); ++k) identity = identity && map[k] == (int64_t)k;
        if (!identity) {
          Node b = unary_node(OpK::BroadcastInDim, cur, TType{CT, pdims});
          b.a0 = map;
          cur = out.add(b);
        }
        return cur;
      };
      const int pb = operand(d.in[bigside], bt, bmap);
      const int ps = operand(d.in[1 - bigside], st, smap);
      Node mul;
      mul.k = OpK::Binary;
      mul.op = "multiply";
      mul.ty = TType{CT, pdims};
      mul.in = bigside == 0 ? std::vector<int>{pb, ps} : std::vector<int>{ps, pb};
      const int pm = out.add(mul);
      Node zero;
      zero.k = OpK::Constant;
      zero.splat = true;
      zero.ty = TType{CT, {}};
      zero.data.assign((size_t)info(CT).size, 0);
      const int pz = out.add(zero);
      Node red;
      red.k = OpK::Reduce;
      red.red = Red::Add;
      red.in = {pm, pz};
      std::vector<PD> kept;
      for (size_t k = 0; k < pd.size(); ++k) {
        if (pd[k].role == 3) red.a0.push_back((int64_t)k);
        else kept.push_back(pd[k]);
      }
      std::vector<int64_t> kdims;
      for (auto& e : kept) kdims.push_back(e.size);
      red.ty = TType{CT, kdims};
      int cur = out.add(red);
      if (CT != d.ty.dt) cur = out.add(unary_node(OpK::Convert, cur, TType{d.ty.dt, kdims}));
      // result order of dot_general: batch dims, lhs free dims, rhs free dims
      std::vector<std::pair<int, int>> want;
      for (size_t j = 0; j < d.a0.size(); ++j) want.push_back({0, (int)j});
      for (int k : f.lfree) want.push_back({1, k});
      for (int k : f.rfree) want.push_back({2, k});
      std::vector<int64_t> perm;
      for (auto& w : want)
        for (size_t k = 0; k < kept.size(); ++k)
          if (kept[k].role == w.first && kept[k].idx == w.second) perm.push_back((int64_t)k);
      if (perm.size() != kept.size() || (int)perm.size() != d.ty.rank()) throw Error("dot_general: internal error in the reduction form");
      bool identity = true, same_order = true;
      int64_t last = -1;
      for (size_t k = 0; k < perm.size(); ++k) {
        identity = identity && perm[k] == (int64_t)k;
        if (kept[perm[k]].size != 1) { same_order = same_order && perm[k] > last; last = perm[k]; }
      }
      if (!identity) {
        Node t = unary_node(same_order ? OpK::Reshape : OpK::Transpose, cur, d.ty);
        if (!same_order) t.a0 = perm;
        cur = out.add(t);
      }
      if (!(out.nodes[cur].ty == d.ty)) throw Error("dot_general: internal error in the reduction form (type)");
      remap[n.id] = cur;
    }
    for (int p : g.params) out.params.push_back(remap[p]);
    for (int r : g.results) out.results.push_back(remap[r]);
    g = std::move(out);
  }

  // ------------------------------------------------------------------ analysis
  int cone_cost(int id, int cap = 16) {
    std::set<int> seen;
    std::vector<int> st{id};
    int cost = 0;
    while (!st.empty() && cost <= cap) {
      int x = st.back();
      st.pop_back();
      if (!seen.insert(x).second) continue;
      const Node& n = g.nodes[x];
      if (n.k == OpK::Param || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv || n.k == OpK::DotGeneral) continue;
      if (n.k == OpK::Constant) continue;
      if (x != id && prev_mat[x]) continue;
      if (is_arith(n.k)) cost += (n.k == OpK::Unary || n.k == OpK::Gelu) ? 2 : 1;
      for (int i : n.in) st.push_back(i);
    }
    return cost;
  }

  bool reaches_dot(int id) const {
    std::set<int> seen;
    std::vector<int> st{id};
    while (!st.empty()) {
      int x = st.back();
      st.pop_back();
      if (!seen.insert(x).second || seen.size() > 64) continue;
      const Node& n = g.nodes[x];
      if (n.k == OpK::DotGeneral) return true;
      if (n.k == OpK::Param || n.k == OpK::Constant || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv) continue;
      if (x != id && prev_mat[x]) continue;
      for (int i : n.in) st.push_back(i);
    }
    return false;
  }

  void analyze() {
    const int N = (int)g.nodes.size();
    live.assign(N, 0);
    mat.assign(N, 0);
    force_mat.assign(N, 0);
    users.assign(N, {});
    ctx.assign(N, {});
    std::vector<int> st(g.results.begin(), g.results.end());
    while (!st.empty()) {
      int x = st.back();
      st.pop_back();
      if (live[x]) continue;
      live[x] = 1;
      for (int i : g.nodes[x].in) st.push_back(i);
    }
    for (int x = 0; x < N; ++x)
      if (live[x]) for (int i : g.nodes[x].in) users[i].push_back(x);
    std::vector<char> is_result(N, 0);
    for (int r : g.results) is_result[r] = 1;

    // The elementwise ops that follow a convolution one after the other (conversion to the images' type, batch norm,
    // bias, activation) end where something reads their value at other positions (a pooling window, a layout change):
    // the value is written there, so that the chain runs once per element in the convolution's kernel, in the
    // type it ends in, instead of once per read in the reader's.
    for (int x : layout_entries)
      if (x < N && live[x] && !users[x].empty()) force_mat[x] = 1;
    if (opt.product_epilogues && opt.conv_tails) {
      auto pointwise = [](OpK k) { return k == OpK::Unary || k == OpK::Binary || k == OpK::Clamp || k == OpK::Convert || k == OpK::Select || k == OpK::Gelu; };
      for (int c = 0; c < N; ++c) {
        if (!live[c] || g.nodes[c].k != OpK::Conv) continue;
        int cur = c;
        while (!is_result[cur] && users[cur].size() == 1) {
          const Node& un = g.nodes[users[cur][0]];
          if (!pointwise(un.k) || un.ty.dims != g.nodes[c].ty.dims) break;
          cur = un.id;
        }
        if (cur == c || is_result[cur]) continue;
        // (measured on VGG-11: with 16-bit results the readers, bound by memory, get twice as fast and the convolutions
        // pay less than that; with f32 results the division and square root of a batch norm cost the convolution
        // kernels more than the pooling kernels gain)
        if (opt.conv_tails < 2 && info(g.nodes[cur].ty.dt).size >= 4) continue;
        bool index_reader = !users[cur].empty();
        for (int u : users[cur]) index_reader = index_reader && (is_index_op(g.nodes[u].k) || g.nodes[u].k == OpK::Reduce);
        if (index_reader) force_mat[cur] = 1;
      }
    }

    for (int x = N - 1; x >= 0; --x) {
      if (!live[x]) continue;
      const Node& n = g.nodes[x];
      // contexts in which x is evaluated
      std::set<Ctx> U;
      bool forced = is_result[x] || n.k == OpK::Param || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv || n.k == OpK::DotGeneral ||
                    (n.k == OpK::Constant && !n.splat);
      for (int u : users[x]) {
        const Node& un = g.nodes[u];
        if (un.k == OpK::Conv) { forced = true; continue; }   // the direct-convolution kernel reads its operands from memory
        if (un.k == OpK::DotGeneral) {
          const int side = un.in[0] == x ? 0 : 1;
          if (fused_operands.count({u, side})) U.insert({u, "/operand" + std::to_string(side)});
          else forced = true;
          continue;
        }
        // start indices of dynamic slices must be constants; they are read at plan time
        std::vector<Ctx> base;
        if (mat[u]) base.push_back({u, ""});
        else base.assign(ctx[u].begin(), ctx[u].end());
        for (auto& c : base) {
          std::string sig = c.second;
          if (is_index_op(un.k)) {
            for (size_t k = 0; k < un.in.size(); ++k)
              if (un.in[k] == x) U.insert({c.first, sig + "/" + std::to_string(u) + ":" + std::to_string(k)});
          } else if (n.ty.rank() == 0 && un.ty.rank() != 0) {
            U.insert({c.first, sig + "/s"});
          } else {
            U.insert({c.first, sig});
          }
        }
      }
      if (n.ty.rank() == 0) {  // a 0-d value has a single index whatever the path
        std::set<Ctx> V;
        for (auto& c : U) V.insert({c.first, "0d"});
        U.swap(V);
      }
      ctx[x] = U;
      if (forced || force_mat[x]) { mat[x] = 1; continue; }
      if (U.size() <= 1) continue;
      // A value computed from a dot_general and read by several kernels: write it once, at the
      // narrowest point of the single-consumer chain under it, so the dot keeps its epilogue.
      {
        std::set<int> roots;
        for (auto& c : U) roots.insert(c.first);
        if (roots.size() > 1 && reaches_dot(x)) {
          int best = x, cur = x;
          while (true) {
            const Node& cn = g.nodes[cur];
            if (!(cn.k == OpK::Convert || cn.k == OpK::Unary)) break;
            int p = cn.in[0];
            const Node& pn = g.nodes[p];
            if (pn.k == OpK::DotGeneral || pn.k == OpK::Param || pn.k == OpK::Constant || pn.k == OpK::Reduce || pn.k == OpK::Scan || pn.k == OpK::Scatter || pn.k == OpK::Conv) break;
            if (users[p].size() != 1 || is_result[p]) break;
            cur = p;
            if (info(pn.ty.dt).size < info(g.nodes[best].ty.dt).size) best = cur;
          }
          force_mat[best] = 1;
          if (best == x) { mat[x] = 1; continue; }
          continue;
        }
      }
      int cost = cone_cost(x);
      if (cost == 0) continue;
      if (cost * ((int)U.size() - 1) <= 6) continue;
      mat[x] = 1;
    }
  }

  // Plain maps that read nothing but arguments and constants of the module (the layout maps of a network's filters, a
  // conversion of its first images) depend on no other launch: they go to the front of the launch list, and when
  // there are several they run as one launch -- each map's kernel becomes a device function that takes the workgroup
  // number as its first parameter, and one kernel sends ranges of workgroup numbers to them.  Small maps cost a launch
  // each (4 us between dependent launches) for a microsecond of work.
  void merge_parameter_maps() {
    if (!opt.merge_parameter_maps) return;
    std::map<std::string, std::string> text_of;   // kernel symbol prefix -> its text
    for (auto& kv : dedupe) text_of[kv.second] = named(kv.first, kv.second);
    std::vector<size_t> picked;
    std::vector<char> written(plan.buffers.size(), 0);
    for (auto& L : plan.launches)
      for (int k = 0; k < L.n_outputs; ++k) written[L.args[L.args.size() - 1 - k]] = 1;
    for (size_t li = 0; li < plan.launches.size(); ++li) {
      const Launch& L = plan.launches[li];
      if (L.kind != "map" || L.grid[1] != 1 || L.grid[2] != 1 || L.block[0] != (unsigned)kBlock || L.lds_bytes != 0 || L.n_outputs != 1 || L.args.empty()) continue;
      bool ok = L.grid[0] <= 16384;
      for (size_t a = 0; a + 1 < L.args.size(); ++a) {
        const BufferDesc& B = plan.buffers[L.args[a]];
        ok = ok && (B.kind == BufferDesc::Param || B.kind == BufferDesc::Const) && !written[L.args[a]];
      }
      const BufferDesc& O = plan.buffers[L.args.back()];
      ok = ok && O.kind == BufferDesc::Temp && !O.is_result;   // operands prepared for later launches, not results of the module
      // the only launch that writes its result
      int writers = 0;
      for (auto& M : plan.launches)
        for (int k = 0; k < M.n_outputs; ++k) writers += M.args[M.args.size() - 1 - k] == L.args.back();
      ok = ok && writers == 1;
      const size_t us = L.kernel.rfind("_map");
      if (!ok || us == std::string::npos || us + 4 != L.kernel.size()) continue;
      auto it = text_of.find(L.kernel.substr(0, us));
      if (it == text_of.end()) continue;
      const std::string& t = it->second;
      const std::string sig = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void " + L.kernel + "(";
      const size_t at = t.find(sig);
      if (at == std::string::npos || t.find("__global__", at + sig.size()) != std::string::npos || t.find("__global__") != at + 11 ||
          t.find("gridDim") != std::string::npos || t.find("blockIdx.y") != std::string::npos || t.find("blockIdx.z") != std::string::npos || t.find("__shared__") != std::string::npos)
        continue;
      picked.push_back(li);
    }
    if (picked.size() < 2) return;
    if (picked.size() > 64) picked.resize(64);   // the merged kernel takes every map's pointers as parameters
    std::vector<Launch> front, rest;
    for (size_t li = 0, q = 0; li < plan.launches.size(); ++li) {
      if (q < picked.size() && picked[q] == li) { front.push_back(plan.launches[li]); ++q; }
      else rest.push_back(plan.launches[li]);
    }
    {
      std::ostringstream o;
      o << "// " << front.size() << " maps of the module's arguments in one launch\n";
      std::set<std::string> defined;
      std::vector<std::vector<std::pair<std::string, std::string>>> params(front.size());   // per map: (type, name)
      for (size_t f = 0; f < front.size(); ++f) {
        const Launch& L = front[f];
        const std::string& t = text_of[L.kernel.substr(0, L.kernel.size() - 4)];
        const std::string sig = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void " + L.kernel + "(";
        const size_t at = t.find(sig), close = t.find(") {", at);
        const std::string plist = t.substr(at + sig.size(), close - at - sig.size());
        for (size_t q = 0; q < plist.size();) {
          size_t e = plist.find(", ", q);
          if (e == std::string::npos) e = plist.size();
          const std::string d = plist.substr(q, e - q);
          const size_t sp = d.rfind(' ');
          params[f].push_back({d.substr(0, sp), d.substr(sp + 1)});
          q = e + 2;
        }
        if (params[f].size() != L.args.size()) return;   // not the text this pass understands: leave the plan as it is
        if (!defined.insert(L.kernel).second) continue;
        std::string body = t.substr(close + 3);
        for (size_t q; (q = body.find("blockIdx.x")) != std::string::npos;) body.replace(q, 10, "bid_");
        o << "static __device__ __forceinline__ void " << L.kernel << "_part(const unsigned bid_, " << plist << ") {" << body;
      }
      o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void @K@_maps(";
      for (size_t f = 0; f < front.size(); ++f)
        for (size_t a = 0; a < params[f].size(); ++a) o << (f + a ? ", " : "") << params[f][a].first << " m" << f << "_" << params[f][a].second;
      o << ") {\n";
      Launch F;
      unsigned first = 0;
      for (size_t f = 0; f < front.size(); ++f) {
        const Launch& L = front[f];
        o << "  if (blockIdx.x < " << first + L.grid[0] << "u) { " << L.kernel << "_part(blockIdx.x - " << first << "u";
        for (size_t a = 0; a < params[f].size(); ++a) o << ", m" << f << "_" << params[f][a].second;
        o << "); return; }\n";
        first += L.grid[0];
        // results last, as every launch has them
        for (size_t a = 0; a + 1 < L.args.size(); ++a) F.args.push_back(L.args[a]);
        F.algo_bytes += L.algo_bytes;
        F.desc += (f ? " | " : "") + L.desc;
      }
      o << "}\n\n";
      // the kernel's parameters are in the maps' order (inputs and result of each map together); the launch's argument
      // list must follow that order too, so it is rebuilt here and all results count as outputs only for the liveness
      F.args.clear();
      for (auto& L : front) for (int a : L.args) F.args.push_back(a);
      const std::string base = finalize(o.str());
      F.kernel = named("@K@_maps", base);
      F.kind = "map";
      F.grid[0] = first;
      F.block[0] = kBlock;
      F.n_outputs = 1;
      front.assign(1, F);
    }
    plan.launches = front;
    plan.launches.insert(plan.launches.end(), rest.begin(), rest.end());
  }

  // ------------------------------------------------------------------ buffers
  int buffer_for(int node) {
    if (buf_of[node] >= 0) return buf_of[node];
    {
      auto al = reshape_alias.find(node);
      if (al != reshape_alias.end()) return buf_of[node] = buffer_for(al->second);
    }
    const Node& n = g.nodes[node];
    BufferDesc b;
    b.ty = n.ty;
    b.bytes = std::max<int64_t>(n.ty.bytes(), 1);
    if (n.k == OpK::Param) { b.kind = BufferDesc::Param; b.param_index = (int)n.a0[0]; }
    else if (n.k == OpK::Constant && !n.splat) { b.kind = BufferDesc::Const; b.data = n.data; }
    else b.kind = BufferDesc::Temp;
    plan.buffers.push_back(b);
    return buf_of[node] = (int)plan.buffers.size() - 1;
  }
  int scratch(int64_t bytes) {
    BufferDesc b;
    b.kind = BufferDesc::Scratch;
    b.bytes = bytes;
    plan.buffers.push_back(b);
    return (int)plan.buffers.size() - 1;
  }

  bool is_input(int root_or_self, int node) const {
    (void)root_or_self;
    return mat[node];
  }

  // ------------------------------------------------------------------ helpers
  // Kernel text is written with the placeholder "@K@" in its symbol names; identical texts
  // (the unrolled steps of a time loop) share one compiled kernel.
  std::map<std::string, std::string> dedupe;
  std::string finalize(const std::string& text) {
    auto it = dedupe.find(text);
    if (it != dedupe.end()) return it->second;
    // kernel symbols carry the module's name so that profiles of several programs stay readable
    std::string mod;
    for (char ch : g.module_name) mod += (isalnum((unsigned char)ch) ? ch : '_');
    if (mod.rfind("reactant_", 0) == 0) mod = mod.substr(9);
    if (mod.size() > 24) mod.resize(24);
    std::string base = "rx_" + (mod.empty() ? std::string("mod") : mod) + "_k" + std::to_string(kcount++);
    dedupe[text] = base;
    src << named(text, base);
    return base;
  }
  static std::string named(std::string text, const std::string& base) {
    size_t p = 0;
    while ((p = text.find("@K@", p)) != std::string::npos) text.replace(p, 3, base);
    return text;
  }

  static std::string ptr_decl(const std::string& stype, bool is_const, const std::string& name) {
    return std::string(is_const ? "const " : "") + stype + "* __restrict__ " + name;
  }

  std::string signature(const std::string& kname, const std::vector<int>& inputs, const std::vector<std::pair<std::string, std::string>>& outs,
                        int launch_bounds = kBlock) {
    std::string s = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(launch_bounds) + ") void " + kname + "(";
    bool first = true;
    for (size_t k = 0; k < inputs.size(); ++k) {
      s += (first ? "" : ", ") + ptr_decl(info(g.nodes[inputs[k]].ty.dt).stype, true, "in" + std::to_string(k));
      first = false;
    }
    for (auto& o : outs) {
      s += (first ? "" : ", ") + ptr_decl(o.first, false, o.second);
      first = false;
    }
    return s + ")";
  }

  std::string describe(int root, const std::vector<int>& extra_roots = {}) {
    std::set<int> seen;
    std::vector<int> st{root};
    for (int r : extra_roots) st.push_back(r);
    std::map<std::string, int> cnt;
    while (!st.empty()) {
      int x = st.back();
      st.pop_back();
      if (!seen.insert(x).second) continue;
      const Node& n = g.nodes[x];
      if (x != root && mat[x] && std::find(extra_roots.begin(), extra_roots.end(), x) == extra_roots.end()) continue;
      std::string nm;
      switch (n.k) {
        case OpK::Unary: case OpK::Binary: nm = n.op; break;
        case OpK::Compare: nm = "compare"; break;
        case OpK::Select: nm = "select"; break;
        case OpK::Clamp: nm = "clamp"; break;
        case OpK::Convert: nm = "convert"; break;
        case OpK::Gelu: nm = "gelu"; break;
        case OpK::BroadcastInDim: nm = "broadcast_in_dim"; break;
        case OpK::Reshape: nm = "reshape"; break;
        case OpK::Transpose: nm = "transpose"; break;
        case OpK::Slice: nm = "slice"; break;
        case OpK::Pad: nm = "pad"; break;
        case OpK::DynamicUpdateSlice: nm = "dynamic_update_slice"; break;
        case OpK::DynamicSlice: nm = "dynamic_slice"; break;
        case OpK::Concatenate: nm = "concatenate"; break;
        case OpK::Reverse: nm = "reverse"; break;
        case OpK::Window: nm = "window"; break;
        case OpK::Gather: nm = "gather"; break;
        case OpK::Scan: nm = "scan"; break;
        case OpK::Scatter: nm = "scatter"; break;
        case OpK::Conv: nm = "convolution"; break;
        case OpK::Reduce: nm = "reduce"; break;
        case OpK::DotGeneral: nm = "dot_general"; break;
        case OpK::Iota: nm = "iota"; break;
        default: break;
      }
      if (!nm.empty()) cnt[nm]++;
      for (int i : n.in) st.push_back(i);
    }
    std::string s;
    for (auto& kv : cnt) s += (s.empty() ? "" : " ") + kv.first + (kv.second > 1 ? "x" + std::to_string(kv.second) : "");
    return s;
  }

  double algo_bytes(const std::vector<int>& inputs, const std::vector<int>& outs) {
    double b = 0;
    for (int i : inputs) b += (double)g.nodes[i].ty.bytes();
    for (int o : outs) b += (double)g.nodes[o].ty.bytes();
    return b;
  }

  static std::string vec_name(int slot, int64_t D) {
    if (D == 0) return "d" + std::to_string(slot);
    return "d" + std::to_string(slot) + (D < 0 ? "_m" + std::to_string(-D) : "_p" + std::to_string(D));
  }

  static int pick_vec(const TType& t) {
    if (t.rank() == 0) return 1;
    int v = std::max(1, 16 / info(t.dt).size);
    int64_t minor = t.dims.back();
    while (v > 1 && minor % v != 0) v >>= 1;
    return v;
  }

  // Decode a linear vector id into the root index variables (row-major, minor dim in vectors).
  // Declares i0..i{n-2} and i{n-1}b (first lane of the vector).
  static void decode_index(std::ostringstream& o, const std::string& it, const std::string& vid, const std::vector<int64_t>& dims, int vec,
                           const std::string& pad) {
    const int n = (int)dims.size();
    if (n == 0) return;
    std::string rest = vid;
    const int64_t mv = dims[n - 1] / vec;
    if (n == 1) {
      o << pad << "const " << it << " i0b = " << rest << " * " << vec << ";\n";
      return;
    }
    o << pad << "const " << it << " i" << n - 1 << "b = (" << rest << " % " << mv << ") * " << vec << ";\n";
    o << pad << it << " rr = " << rest << " / " << mv << ";\n";
    for (int d = n - 2; d >= 1; --d) {
      o << pad << "const " << it << " i" << d << " = rr % " << dims[d] << ";\n";
      o << pad << "rr /= " << dims[d] << ";\n";
    }
    o << pad << "const " << it << " i0 = rr;\n";
  }

  static Index root_index(const std::vector<int64_t>& dims) {
    Index ix(dims.size());
    for (size_t d = 0; d < dims.size(); ++d) {
      ix[d].var = "i" + std::to_string(d);
      ix[d].lo = 0;
      ix[d].hi = dims[d] - 1;
    }
    return ix;
  }

  bool needs64(const std::vector<int>& nodes_touched) const {
    for (int x : nodes_touched)
      if (g.nodes[x].ty.numel() >= (int64_t)1 << 31) return true;
    return false;
  }

  std::vector<int> cone_nodes(int root) const {
    std::set<int> seen;
    std::vector<int> st{root}, out;
    while (!st.empty()) {
      int x = st.back();
      st.pop_back();
      if (!seen.insert(x).second) continue;
      out.push_back(x);
      if (x != root && mat[x]) continue;
      for (int i : g.nodes[x].in) st.push_back(i);
    }
    return out;
  }

  // Tile order of the stencil kernels.  Workgroups are dealt round-robin to the 8 XCDs, each with
  // its own L2.  The y-tiles are cut into slabs of `sy` tiles; XCD k owns slabs k, k+8, ... and
  // walks each of them layer by layer in z, so the planes that consecutive layers share (and the
  // rows that neighbouring tiles of a layer share) are still in that XCD's L2 when they are asked
  // for again.  Declares x0, y0, z0; returns the number of workgroups to launch.
  // `bid` is the expression of the block number within the region (a launch can hold two regions with tile shapes of
  // their own), `x_base` the region's first column.
  int64_t emit_tile_order(std::ostringstream& o, int64_t ntx, int64_t nty, int64_t ntz, int TX, int TY, int TZ, int64_t default_sy = 0,
                          const std::string& bid = "blockIdx.x", int64_t x_base = 0) {
    const int64_t nblocks = ntx * nty * ntz;
    const std::string xb = x_base ? std::to_string(x_base) + " + " : std::string();
    if (!(opt.xcd_slabs && nty >= 16)) {
      o << "  const unsigned tile = rx_xcd_remap(" << bid << ", " << nblocks << "u);\n";
      o << "  const int x0 = " << xb << "(int)(tile % " << ntx << "u) * " << TX << ";\n";
      o << "  const int y0 = (int)((tile / " << ntx << "u) % " << nty << "u) * " << TY << ";\n";
      o << "  const int z0 = (int)(tile / " << ntx * nty << "u) * " << TZ << ";\n";
      return nblocks;
    }
    int64_t sy = opt.slab_ytiles > 0 ? opt.slab_ytiles : default_sy > 0 ? default_sy : (nty + 7) / 8;
    sy = std::min<int64_t>(sy, (nty + 7) / 8);
    const int64_t nslabs = (nty + sy - 1) / sy, rounds = (nslabs + 7) / 8;
    const int64_t per_slab = ntz * ntx * sy;
    o << "  const unsigned xcd = " << bid << " & 7u, j = " << bid << " >> 3;\n";
    o << "  const unsigned slab = (j / " << per_slab << "u) * 8u + xcd, r = j % " << per_slab << "u;\n";
    o << "  const unsigned tz = r / " << ntx * sy << "u, rr = r % " << ntx * sy << "u;\n";
    o << "  const unsigned ty = slab * " << sy << "u + rr / " << ntx << "u;\n";
    o << "  if (ty >= " << nty << "u) return;\n";
    o << "  const int x0 = " << xb << "(int)(rr % " << ntx << "u) * " << TX << ";\n";
    o << "  const int y0 = (int)ty * " << TY << ";\n";
    o << "  const int z0 = (int)tz * " << TZ << ";\n";
    return 8 * rounds * per_slab;
  }

  struct Halo { int64_t lo[3] = {0, 0, 0}, hi[3] = {0, 0, 0}; bool ok = true; };
  struct StencilProbe {
    int vec = 1;
    std::vector<int> staged;       // same-shape inputs read at three or more constant offsets
    std::map<int, Halo> halos;     // per staged input: how far the offsets reach in each dimension
  };
  void stencil_emitter(Emitter& em, int root, int vec, const std::vector<std::string>& vars) {
    em.idx64 = needs64(cone_nodes(root));
    em.set_root(g.nodes[root].ty.dims, vars, true);
    em.vec = vec;
    em.allow_shifted = false;
    em.excess_precision = opt.excess_precision;
    em.branchless_guards = opt.branchless_guards;
    em.indent = 8;
  }
  bool probe_stencil(int root, StencilProbe* sp) {
    const Node& rn = g.nodes[root];
    const auto& dims = rn.ty.dims;
    if (!opt.lds_stencil || rn.ty.rank() != 3 || rn.k == OpK::Reduce || rn.k == OpK::Scan || rn.k == OpK::Scatter || rn.k == OpK::Conv || rn.k == OpK::DotGeneral) return false;
    sp->vec = pick_vec(rn.ty);
    if (rn.ty.numel() < opt.slab_min_numel || sp->vec < 2) return false;
    Emitter probe(g, [&](int x) { return x != root && mat[x]; });
    stencil_emitter(probe, root, sp->vec, {"i0", "i1", "i2"});
    probe.direct_expr = vec_name;
    probe.emit(root, root_index(dims));
    std::map<int, std::set<std::vector<int64_t>>> offs;
    std::map<int, Halo> halos;
    for (auto& l : probe.loads) {
      const Node& ln = g.nodes[l.node];
      if (ln.ty.dims != dims) continue;
      if (!l.affine) { halos[l.node].ok = false; continue; }
      offs[l.node].insert(l.off);
    }
    for (auto& kv : offs) {
      if (kv.second.size() < 3 || !halos[kv.first].ok) continue;
      Halo& h = halos[kv.first];
      for (auto& o : kv.second)
        for (int d = 0; d < 3; ++d) { h.lo[d] = std::max<int64_t>(h.lo[d], -o[d]); h.hi[d] = std::max<int64_t>(h.hi[d], o[d]); }
      if (h.lo[0] > 4 || h.hi[0] > 4 || h.lo[1] > 4 || h.hi[1] > 4 || h.lo[2] > 8 || h.hi[2] > 8) continue;
      const int es = info(g.nodes[kv.first].ty.dt).size;
      if (es != 4 && es != 8) continue;
      if (es != info(rn.ty.dt).size) continue;  // same vector width as the output
      sp->staged.push_back(kv.first);
      sp->halos[kv.first] = h;
    }
    return !sp->staged.empty();
  }

  // ------------------------------------------------------------------ stencil maps through LDS halo tiles
  // A rank-3 map that reads some input at several constant offsets (a stencil): the workgroup
  // owns a TZ x TY x TX block of outputs, loads that input's block plus halo into LDS once with
  // aligned 16-byte loads, and every neighbour access becomes an LDS read.  Inputs read only at
  // the output's own position are still streamed from global memory with vector loads.
  bool emit_map_lds(int root) {
    const Node& rn = g.nodes[root];
    const auto& dims = rn.ty.dims;
    StencilProbe sp;
    if (!probe_stencil(root, &sp)) return false;
    const int vec = sp.vec;
    const int64_t Z = dims[0], Y = dims[1], X = dims[2];
    auto make_emitter = [&](Emitter& em) {
      stencil_emitter(em, root, vec, {"i0", "i1", "i2"});
      em.direct_expr = vec_name;
    };
    std::vector<int>& staged = sp.staged;
    std::map<int, Halo>& halos = sp.halos;
    {
      auto pf = fuse_prev.find(root);
      if (pf != fuse_prev.end()) {
        const int prev = pf->second;
        if (opt.stencil_march2 && emit_map_march2(root, prev, sp)) return true;
        if (emit_map_lds2(root, prev, sp)) return true;
        // not fused after all: the producer gets its own launch first
        fuse_prev.erase(pf);
        lds_only.erase(prev);
        emit_map(prev);
      }
    }
    int TZ = opt.lds_tile[0], TY = opt.lds_tile[1], TX = opt.lds_tile[2];
    // the tile is given for 8-byte elements (two per vector); with more elements per vector the rows
    // take fewer threads, so the tile gets more rows
    if (TX % vec == 0 && (TX / vec) * TY != kBlock && kBlock % (TX / vec) == 0) TY = kBlock / (TX / vec);
    if (TX % vec || (TX / vec) * TY != kBlock) return false;
    const int TXV = TX / vec;
    // LDS geometry per staged input
    struct Geo { int64_t pz, py, lx, hxl; int64_t bytes; };
    std::map<int, Geo> geo;
    int64_t lds_total = 0;
    for (int s : staged) {
      Halo& h = halos[s];
      Geo ge;
      ge.hxl = (h.lo[2] + vec - 1) / vec * vec;
      const int64_t hxh = (h.hi[2] + vec - 1) / vec * vec;
      ge.pz = TZ + h.lo[0] + h.hi[0];
      ge.py = TY + h.lo[1] + h.hi[1];
      ge.lx = TX + ge.hxl + hxh;
      ge.bytes = ge.pz * ge.py * ge.lx * info(g.nodes[s].ty.dt).size;
      geo[s] = ge;
      lds_total += ge.bytes;
    }
    if (lds_total > 64 * 1024) return false;

    // pass 2: emit with the staged inputs redirected to LDS
    Emitter em(g, [&](int x) { return x != root && mat[x]; });
    make_emitter(em);
    em.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
      const int node = em.inputs[slot];
      auto it = geo.find(node);
      if (it == geo.end()) return false;
      const Halo& h = halos[node];
      const Geo& ge = it->second;
      // position inside the tile: (lz + dz + hz_lo, ly + dy + hy_lo, hxl + lx + l + dx)
      std::ostringstream e;
      e << "lds" << slot << "[((lz + " << (off[0] + h.lo[0]) << ") * " << ge.py << " + (ly + " << (off[1] + h.lo[1]) << ")) * " << ge.lx << " + lxe + l + "
        << (ge.hxl + off[2]) << "]";
      *expr = e.str();
      return true;
    };
    std::string val = em.emit(root, root_index(dims));
    std::string body = em.take_code();
    const std::string it = em.idx_t();
    const std::string kname = "@K@_stencil";
    const int64_t ntx = (X + TX - 1) / TX, nty = (Y + TY - 1) / TY, ntz = (Z + TZ - 1) / TZ;
    std::ostringstream o;
    o << "// stencil map through LDS halo tiles (" << TZ << "x" << TY << "x" << TX << " outputs per workgroup): " << describe(root) << " -> " << rn.ty.str() << "\n";
    o << signature(kname, em.inputs, {{info(rn.ty.dt).stype, "out0"}}) << " {\n";
    for (int s : staged) {
      const int slot = em.slot_of(s);
      const Geo& ge = geo[s];
      o << "  __shared__ __attribute__((aligned(16))) " << info(g.nodes[s].ty.dt).stype << " lds" << slot << "[" << ge.pz * ge.py * ge.lx << "];\n";
    }
    const int64_t launch_blocks = emit_tile_order(o, ntx, nty, ntz, TX, TY, TZ);
    for (int s : staged) {
      const int slot = em.slot_of(s);
      const Geo& ge = geo[s];
      const Halo& h = halos[s];
      const std::string st = info(g.nodes[s].ty.dt).stype;
      const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
      const int64_t lxv = ge.lx / vec;
      const int64_t total = ge.pz * ge.py * lxv;
      const int64_t nit = (total + kBlock - 1) / kBlock;
      // all global loads of the tile are issued before the first LDS write
      o << "  {\n    " << vt << " t[" << nit << "];\n";
      o << "#pragma unroll\n    for (int q = 0; q < " << nit << "; ++q) {\n";
      o << "      const int v = threadIdx.x + q * " << kBlock << ";\n";
      o << "      const int xv = v % " << lxv << ", rw = v / " << lxv << ";\n";
      o << "      const int yy = rw % " << ge.py << ", zz = rw / " << ge.py << ";\n";
      // halo cells outside the array are clamped to valid addresses; their values are never used
      o << "      const " << it << " gz = rx_clamp_idx<" << it << ">(z0 - " << h.lo[0] << " + zz, " << Z - 1 << ");\n";
      o << "      const " << it << " gy = rx_clamp_idx<" << it << ">(y0 - " << h.lo[1] << " + yy, " << Y - 1 << ");\n";
      o << "      const " << it << " gx = rx_clamp_idx<" << it << ">(x0 - " << ge.hxl << " + xv * " << vec << ", " << X - vec << ");\n";
      o << "      t[q] = rx_load<" << vt << ">(in" << slot << " + (gz * " << Y << " + gy) * " << X << (em.idx64 ? "LL" : "") << " + gx);\n";
      o << "    }\n";
      o << "#pragma unroll\n    for (int q = 0; q < " << nit << "; ++q) {\n";
      o << "      const int v = threadIdx.x + q * " << kBlock << ";\n";
      o << "      if (v < " << total << ") rx_store(lds" << slot << " + v * " << vec << ", t[q]);\n";
      o << "    }\n  }\n";
    }
    o << "  const int ly = threadIdx.x / " << TXV << ", lxe = (threadIdx.x % " << TXV << ") * " << vec << ";\n";
    o << "  const " << it << " i1 = y0 + ly, i2b = x0 + lxe;\n";
    o << "  const bool live = i1 < " << Y << " && i2b < " << X << ";\n";
    // inputs read only at the output position: their loads for every plane of the tile are in
    // flight while the halo tile settles in LDS
    for (auto& sd : em.direct_vecs) {
      const int slot = sd.first;
      const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
      const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
      o << "  " << vt << " " << vec_name(slot, 0) << "z[" << TZ << "];\n";
    }
    if (!em.direct_vecs.empty()) {
      o << "  if (live) {\n#pragma unroll\n    for (int lz = 0; lz < " << TZ << "; ++lz) {\n";
      o << "      const " << it << " i0c = rx_clamp_idx<" << it << ">(z0 + lz, " << Z - 1 << ");\n";
      o << "      const " << it << " linc = (i0c * " << Y << " + i1) * " << X << (em.idx64 ? "LL" : "") << " + i2b;\n";
      for (auto& sd : em.direct_vecs) {
        const int slot = sd.first;
        const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
        const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
        o << "      " << vec_name(slot, 0) << "z[lz] = " << (opt.nt_loads ? "rx_load_nt" : "rx_load") << "<" << vt << ">(in" << slot << " + linc);\n";
      }
      o << "    }\n  }\n";
    }
    o << "  rx_lds_barrier();\n";
    o << "  if (!live) return;\n";
    o << "#pragma unroll\n  for (int lz = 0; lz < " << TZ << "; ++lz) {\n";
    o << "    const " << it << " i0 = z0 + lz;\n";
    o << "    if (i0 >= " << Z << ") break;\n";
    o << "    const " << it << " lin0 = (i0 * " << Y << " + i1) * " << X << (em.idx64 ? "LL" : "") << " + i2b;\n";
    for (auto& sd : em.direct_vecs) {
      const int slot = sd.first;
      const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
      const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
      o << "    const " << vt << " " << vec_name(slot, 0) << " = " << vec_name(slot, 0) << "z[lz];\n";
    }
    const std::string ost = info(rn.ty.dt).stype;
    o << "    rx_vec<" << ost << ", " << vec << "> res;\n";
    o << "#pragma unroll\n    for (int l = 0; l < " << vec << "; ++l) {\n";
    o << "      const " << it << " i2 = i2b + l;\n";
    o << body;
    o << "      res.v[l] = " << em.store_value(rn.ty.dt, val) << ";\n    }\n";
    o << "    " << (opt.nt_stores ? "rx_store_nt" : "rx_store") << "(out0 + lin0, res);\n";
    o << "  }\n}\n\n";
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = "map_stencil_lds";
    L.grid[0] = (unsigned)launch_blocks;
    L.block[0] = kBlock;
    for (int i : em.inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    L.algo_bytes = algo_bytes(em.inputs, {root});
    L.desc = describe(root);
    plan.launches.push_back(L);
    return true;
  }

  // ------------------------------------------------------------------ two stencil steps in one kernel
  // `root` is a stencil of `prev`, which is itself a stencil of some array A and has no other
  // reader.  The workgroup loads A's tile with both halos into LDS, evaluates `prev` on the
  // output tile plus root's halo into registers, writes those values over the A tile (after a
  // barrier), and evaluates `root` from them.  `prev` never reaches global memory.  The values of
  // `prev` are computed by the same expression at the same points as in a kernel of its own, so
  // the result is bit-identical to the two-kernel form.
  bool emit_map_lds2(int root, int prev, const StencilProbe& spR) {
    const Node& rn = g.nodes[root];
    const Node& pn = g.nodes[prev];
    const auto& dims = rn.ty.dims;
    if (pn.ty.dims != dims || pn.ty.dt != rn.ty.dt) return false;
    StencilProbe spP;
    if (!probe_stencil(prev, &spP) || spP.staged.size() != 1 || spP.vec != spR.vec) return false;
    const int src = spP.staged[0];
    if (g.nodes[src].ty.dims != dims) return false;
    const int vec = spR.vec;
    const Halo hR = spR.halos.at(prev), hP = spP.halos.at(src);
    const int TZ = opt.lds_tile2[0], TY = opt.lds_tile2[1], TX = opt.lds_tile2[2];
    if (TZ < 1 || TX % vec) return false;
    const int TXV = TX / vec;
    // NB threads cover PZ planes of the output tile at a time
    const int NB = opt.lds2_threads;
    if (NB < 64 || NB > 1024 || NB % 64 || NB % (TXV * TY)) return false;
    const int PZ = NB / (TXV * TY);
    if (TZ % PZ) return false;
    const int64_t Z = dims[0], Y = dims[1], X = dims[2];
    auto up = [&](int64_t v) { return (v + vec - 1) / vec * vec; };
    // region of `prev` values (B) and of A values (A), relative to the output tile origin
    const int64_t bxl = up(hR.lo[2]), bxh = up(hR.hi[2]);
    const int64_t BZ = TZ + hR.lo[0] + hR.hi[0], BY = TY + hR.lo[1] + hR.hi[1], BX = TX + bxl + bxh;
    const int64_t axl = up(hP.lo[2]), axh = up(hP.hi[2]);
    const int64_t AZ = BZ + hP.lo[0] + hP.hi[0], AY = BY + hP.lo[1] + hP.hi[1], AX = BX + axl + axh;
    const int64_t BXV = BX / vec, AXV = AX / vec;
    const int64_t totalA = AZ * AY * AXV, totalB = BZ * BY * BXV;
    const int es = info(rn.ty.dt).size;
    const int64_t lds_bytes = std::max(totalA, totalB) * vec * es;
    if (lds_bytes > 80 * 1024) return false;
    const int64_t nitA = (totalA + NB - 1) / NB, nitB = (totalB + NB - 1) / NB;
    if (nitB * vec * es / 4 > 96) return false;   // registers that hold the first step's values
    const std::string st = info(rn.ty.dt).stype;
    const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";

    // first step, evaluated at (j0, j1, j2) = a point of region B (clamped into the array)
    Emitter eb(g, [&](int x) { return x != prev && mat[x]; });
    stencil_emitter(eb, prev, vec, {"j0", "j1", "j2"});
    eb.direct_expr = [](int slot, int64_t D) { return "b" + vec_name(slot, D); };
    eb.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
      if (eb.inputs[slot] != src) return false;
      std::ostringstream e;
      e << "lds[((bz + " << (off[0] + hP.lo[0]) << ") * " << AY << " + (by + " << (off[1] + hP.lo[1]) << ")) * " << AX << " + bxe + l + " << (axl + off[2]) << "]";
      *expr = e.str();
      return true;
    };
    Index jb(3);
    for (int d = 0; d < 3; ++d) { jb[d].var = "j" + std::to_string(d); jb[d].lo = 0; jb[d].hi = dims[d] - 1; }
    std::string valB = eb.emit(prev, jb);
    std::string bodyB = eb.take_code();
    for (auto& dv : eb.direct_vecs) if (dv.second != 0) return false;

    // second step, evaluated at the output point; slots continue the first step's numbering
    Emitter ec(g, [&](int x) { return x != root && mat[x]; });
    stencil_emitter(ec, root, vec, {"i0", "i1", "i2"});
    ec.idx64 = ec.idx64 || eb.idx64;
    ec.inputs = eb.inputs;
    ec.direct_expr = vec_name;
    ec.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
      if (ec.inputs[slot] != prev) return false;
      std::ostringstream e;
      e << "lds[((lz + " << (off[0] + hR.lo[0]) << ") * " << BY << " + (ly + " << (off[1] + hR.lo[1]) << ")) * " << BX << " + lxe + l + " << (bxl + off[2]) << "]";
      *expr = e.str();
      return true;
    };
    std::string valC = ec.emit(root, root_index(dims));
    std::string bodyC = ec.take_code();
    for (auto& dv : ec.direct_vecs) if (dv.second != 0) return false;
    // every read of `prev` must have gone to the tile
    for (auto& l : ec.loads) if (l.node == prev && !l.affine) return false;
    const std::string it = ec.idx_t();
    const bool i64 = ec.idx64;
    const int prev_slot = ec.slot_of(prev);

    const std::string kname = "@K@_stencil2";
    const int64_t ntx = (X + TX - 1) / TX, nty = (Y + TY - 1) / TY, ntz = (Z + TZ - 1) / TZ;
    std::ostringstream o;
    o << "// two stencil steps through one LDS tile (" << TZ << "x" << TY << "x" << TX << " outputs per workgroup): " << describe(prev) << " ; " << describe(root)
      << " -> " << rn.ty.str() << "\n";
    {
      std::string s = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(NB) + ") void " + kname + "(";
      for (size_t k = 0; k < ec.inputs.size(); ++k) {
        if ((int)k == prev_slot) continue;
        s += ptr_decl(info(g.nodes[ec.inputs[k]].ty.dt).stype, true, "in" + std::to_string(k)) + ", ";
      }
      s += ptr_decl(st, false, "out0") + ")";
      o << s << " {\n";
    }
    o << "  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];\n";
    o << "  " << st << "* const lds = reinterpret_cast<" << st << "*>(rx_smem);\n";
    const int64_t launch_blocks = emit_tile_order(o, ntx, nty, ntz, TX, TY, TZ, std::max(1, 16 / TY));
    const std::string LL = i64 ? "LL" : "";
    // stage A: the source tile with both halos; out-of-array cells are clamped (never used)
    {
      const int sslot = ec.slot_of(src);
      o << "  {\n    " << vt << " t[" << nitA << "];\n";
      o << "#pragma unroll\n    for (int q = 0; q < " << nitA << "; ++q) {\n";
      o << "      const int v = threadIdx.x + q * " << NB << ";\n";
      o << "      const int xv = v % " << AXV << ", rw = v / " << AXV << ";\n";
      o << "      const int yy = rw % " << AY << ", zz = rw / " << AY << ";\n";
      o << "      const " << it << " gz = rx_clamp_idx<" << it << ">(z0 - " << (hR.lo[0] + hP.lo[0]) << " + zz, " << Z - 1 << ");\n";
      o << "      const " << it << " gy = rx_clamp_idx<" << it << ">(y0 - " << (hR.lo[1] + hP.lo[1]) << " + yy, " << Y - 1 << ");\n";
      o << "      const " << it << " gx = rx_clamp_idx<" << it << ">(x0 - " << (bxl + axl) << " + xv * " << vec << ", " << X - vec << ");\n";
      o << "      t[q] = rx_load<" << vt << ">(in" << sslot << " + (gz * " << Y << " + gy) * " << X << LL << " + gx);\n";
      o << "    }\n";
      o << "#pragma unroll\n    for (int q = 0; q < " << nitA << "; ++q) {\n";
      o << "      const int v = threadIdx.x + q * " << NB << ";\n";
      o << "      if (v < " << totalA << ") rx_store(lds + v * " << vec << ", t[q]);\n";
      o << "    }\n  }\n";
    }
    // loads of the streamed inputs of both steps are issued while the tile settles in LDS; points
    // of region B outside the array are evaluated at clamped coordinates (their values are never used)
    auto vts_of = [&](Emitter& em, int slot) { return "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vec) + ">"; };
    for (auto& dv : eb.direct_vecs) o << "  " << vts_of(eb, dv.first) << " b" << vec_name(dv.first, 0) << "q[" << nitB << "];\n";
    if (!eb.direct_vecs.empty()) {
      o << "#pragma unroll\n  for (int q = 0; q < " << nitB << "; ++q) {\n";
      o << "    const int v = rx_min((int)threadIdx.x + q * " << NB << ", " << totalB - 1 << ");\n";
      o << "    const int bxv = v % " << BXV << ", brw = v / " << BXV << ";\n";
      o << "    const int by = brw % " << BY << ", bz = brw / " << BY << ";\n";
      o << "    const " << it << " j0 = rx_clamp_idx<" << it << ">(z0 - " << hR.lo[0] << " + bz, " << Z - 1 << ");\n";
      o << "    const " << it << " j1 = rx_clamp_idx<" << it << ">(y0 - " << hR.lo[1] << " + by, " << Y - 1 << ");\n";
      o << "    const " << it << " j2b = rx_clamp_idx<" << it << ">(x0 - " << bxl << " + bxv * " << vec << ", " << X - vec << ");\n";
      o << "    const " << it << " linb = (j0 * " << Y << " + j1) * " << X << LL << " + j2b;\n";
      for (auto& dv : eb.direct_vecs)
        o << "    b" << vec_name(dv.first, 0) << "q[q] = " << "rx_load" << "<" << vts_of(eb, dv.first) << ">(in" << dv.first << " + linb);\n";
      o << "  }\n";
    }
    o << "  const int lzb = threadIdx.x / " << TXV * TY << ", lrem = threadIdx.x % " << TXV * TY << ";\n";
    o << "  const int ly = lrem / " << TXV << ", lxe = (lrem % " << TXV << ") * " << vec << ";\n";
    o << "  const " << it << " i1 = rx_min<" << it << ">(y0 + ly, " << Y - 1 << "), i2b = rx_min<" << it << ">(x0 + lxe, " << X - vec << ");\n";
    o << "  const bool live = y0 + ly < " << Y << " && x0 + lxe < " << X << ";\n";
    o << "  rx_lds_barrier();\n";
    // stage B: first step on region B, kept in registers until every wavefront has read the tile
    o << "  " << vt << " sb[" << nitB << "];\n";
    o << "#pragma unroll\n  for (int q = 0; q < " << nitB << "; ++q) {\n";
    o << "    const int v = rx_min((int)threadIdx.x + q * " << NB << ", " << totalB - 1 << ");\n";
    o << "    const int bxv = v % " << BXV << ", brw = v / " << BXV << ";\n";
    o << "    const int by = brw % " << BY << ", bz = brw / " << BY << ", bxe = bxv * " << vec << ";\n";
    o << "    const " << it << " j0 = rx_clamp_idx<" << it << ">(z0 - " << hR.lo[0] << " + bz, " << Z - 1 << ");\n";
    o << "    const " << it << " j1 = rx_clamp_idx<" << it << ">(y0 - " << hR.lo[1] << " + by, " << Y - 1 << ");\n";
    o << "    const " << it << " j2b = rx_clamp_idx<" << it << ">(x0 - " << bxl << " + bxe, " << X - vec << ");\n";
    for (auto& dv : eb.direct_vecs)
      o << "    const " << vts_of(eb, dv.first) << " b" << vec_name(dv.first, 0) << " = b" << vec_name(dv.first, 0) << "q[q];\n";
    o << "#pragma unroll\n    for (int l = 0; l < " << vec << "; ++l) {\n";
    o << "      const " << it << " j2 = j2b + l;\n";
    o << bodyB;
    o << "      sb[q].v[l] = " << Emitter::store_conv(pn.ty.dt, valB) << ";\n    }\n";
    o << "  }\n";
    // streamed inputs of the second step: in flight across the barriers
    for (auto& dv : ec.direct_vecs) o << "  " << vts_of(ec, dv.first) << " " << vec_name(dv.first, 0) << "z[" << TZ / PZ << "];\n";
    if (!ec.direct_vecs.empty()) {
      o << "#pragma unroll\n  for (int lk = 0; lk < " << TZ / PZ << "; ++lk) {\n";
      o << "    const int lz = lk * " << PZ << " + lzb;\n";
      o << "    const " << it << " i0c = rx_clamp_idx<" << it << ">(z0 + lz, " << Z - 1 << ");\n";
      o << "    const " << it << " linc = (i0c * " << Y << " + i1) * " << X << LL << " + i2b;\n";
      for (auto& dv : ec.direct_vecs)
        o << "    " << vec_name(dv.first, 0) << "z[lk] = " << "rx_load" << "<" << vts_of(ec, dv.first) << ">(in" << dv.first << " + linc);\n";
      o << "  }\n";
    }
    o << "  rx_lds_barrier();\n";
    o << "#pragma unroll\n  for (int q = 0; q < " << nitB << "; ++q) {\n";
    o << "    const int v = threadIdx.x + q * " << NB << ";\n";
    o << "    if (v < " << totalB << ") rx_store(lds + v * " << vec << ", sb[q]);\n";
    o << "  }\n";
    o << "  rx_lds_barrier();\n";
    // stage C: second step on the output tile
    o << "  if (!live) return;\n";
    o << "#pragma unroll\n  for (int lk = 0; lk < " << TZ / PZ << "; ++lk) {\n";
    o << "    const int lz = lk * " << PZ << " + lzb;\n";
    o << "    const " << it << " i0 = z0 + lz;\n";
    o << "    if (i0 >= " << Z << ") break;\n";
    o << "    const " << it << " lin0 = (i0 * " << Y << " + i1) * " << X << LL << " + i2b;\n";
    for (auto& dv : ec.direct_vecs)
      o << "    const " << vts_of(ec, dv.first) << " " << vec_name(dv.first, 0) << " = " << vec_name(dv.first, 0) << "z[lk];\n";
    o << "    " << vt << " res;\n";
    o << "#pragma unroll\n    for (int l = 0; l < " << vec << "; ++l) {\n";
    o << "      const " << it << " i2 = i2b + l;\n";
    o << bodyC;
    o << "      res.v[l] = " << Emitter::store_conv(rn.ty.dt, valC) << ";\n    }\n";
    o << "    " << (opt.nt_stores ? "rx_store_nt" : "rx_store") << "(out0 + lin0, res);\n";
    o << "  }\n}\n\n";
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = "map_stencil_lds2";
    L.grid[0] = (unsigned)launch_blocks;
    L.block[0] = NB;
    L.lds_bytes = (unsigned)lds_bytes;
    std::vector<int> ins;
    for (size_t k = 0; k < ec.inputs.size(); ++k) {
      if ((int)k == prev_slot) continue;
      ins.push_back(ec.inputs[k]);
      L.args.push_back(buffer_for(ec.inputs[k]));
    }
    L.args.push_back(buffer_for(root));
    // both steps' compulsory traffic: the first step's inputs and output, then the second's
    std::set<int> read2;
    for (auto& l : ec.loads) read2.insert(l.node);
    L.algo_bytes = algo_bytes(eb.inputs, {prev}) + algo_bytes(std::vector<int>(read2.begin(), read2.end()), {root});
    L.desc = describe(prev) + " ; " + describe(root);
    plan.launches.push_back(L);
    return true;
  }

  // ------------------------------------------------------------------ two stencil steps, marching
  // Same pairing as emit_map_lds2, other traversal: a workgroup owns TY x TX output columns and
  // walks ZC planes along the slowest dimension.  Two rings of planes live in LDS: the source
  // field A (with both halos in y/x) and the first step's values B (with the second step's halo).
  // Every iteration t brings one new plane of A (requested one iteration earlier into registers),
  // evaluates one plane of B from the ring of A, and evaluates one output plane from the ring
  // of B.  Halo planes in z are therefore read and computed once per workgroup, not once per
  // tile, and only the y/x surface of the column is recomputed.
  bool emit_map_march2(int root, int prev, const StencilProbe& spR) {
    const Node& rn = g.nodes[root];
    const Node& pn = g.nodes[prev];
    const auto& dims = rn.ty.dims;
    if (pn.ty.dims != dims || pn.ty.dt != rn.ty.dt) return false;
    StencilProbe spP;
    if (!probe_stencil(prev, &spP) || spP.staged.size() != 1 || spP.vec != spR.vec) return false;
    const int src = spP.staged[0];
    if (g.nodes[src].ty.dims != dims) return false;
    const int vec = spR.vec;
    const Halo hR = spR.halos.at(prev), hP = spP.halos.at(src);
    const int64_t Z = dims[0], Y = dims[1], X = dims[2];
    // planes per workgroup: the extent is cut into equal chunks of about march2_planes
    const int64_t nchunks = std::max<int64_t>(1, (Z + opt.march2_planes - 1) / opt.march2_planes);
    const int64_t ZC = (Z + nchunks - 1) / nchunks;
    // A launch holds one or two regions of columns [x_lo, x_hi), each with a tile shape of its own (same number of
    // threads); `bid` is the block number within the region.
    struct Region {
      std::string text, note;
      int64_t blocks = 0, lds_a = 0, lds_b = 0;
      int nb = 0, prev_slot = -1;
      std::vector<int> inputs, first_inputs, reads2;
    };
    auto gen = [&](int TY, int TX, int64_t x_lo, int64_t x_hi, const std::string& bid, Region* R) -> bool {
    if (TX % vec) return false;
    const int TXV = TX / vec, NB = TXV * TY;
    if (NB < 64 || NB > 1024 || NB % 64) return false;
    auto up = [&](int64_t v) { return (v + vec - 1) / vec * vec; };
    const int64_t bxl = up(hR.lo[2]), bxh = up(hR.hi[2]);
    const int64_t BY = TY + hR.lo[1] + hR.hi[1], BX = TX + bxl + bxh, BXV = BX / vec;
    const int64_t axl = up(hP.lo[2]), axh = up(hP.hi[2]);
    const int64_t AY = BY + hP.lo[1] + hP.hi[1], AX = BX + axl + axh, AXV = AX / vec;
    const int64_t APLANE = AY * AX, BPLANE = BY * BX, AV = AY * AXV;
    const int64_t RA = hP.lo[0] + hP.hi[0] + 2, RB = hR.lo[0] + hR.hi[0] + 2;   // a stencil's reach plus the plane being written
    const int es = info(rn.ty.dt).size;
    if ((RA * APLANE + RB * BPLANE) * es > 80 * 1024) return false;   // two workgroups per compute unit at least
    const int64_t NLA = (AV + NB - 1) / NB;   // 16-byte loads per thread for one source plane
    if (NLA > 8) return false;
    const std::string st = info(rn.ty.dt).stype;
    const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
    const int64_t dA = hP.lo[0] + hP.hi[0], dB = hR.lo[0] + hR.hi[0];

    Emitter eb(g, [&](int x) { return x != prev && mat[x]; });
    stencil_emitter(eb, prev, vec, {"j0", "j1", "j2"});
    eb.indent = 12;
    eb.direct_expr = [](int slot, int64_t D) { return "b" + vec_name(slot, D); };
    eb.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
      if (eb.inputs[slot] != src) return false;
      std::ostringstream e;   // plane b + off0 is the plane brought in (hi0 - off0) iterations ago
      e << "ldsA[sa" << (hP.hi[0] - off[0]) << " + (by + " << (off[1] + hP.lo[1]) << ") * " << AX << " + bxe + l + " << (axl + off[2]) << "]";
      *expr = e.str();
      return true;
    };
    Index jb(3);
    for (int d = 0; d < 3; ++d) { jb[d].var = "j" + std::to_string(d); jb[d].lo = 0; jb[d].hi = dims[d] - 1; }
    std::string valB = eb.emit(prev, jb);
    std::string bodyB = eb.take_code();
    for (auto& dv : eb.direct_vecs) if (dv.second != 0) return false;

    Emitter ec(g, [&](int x) { return x != root && mat[x]; });
    stencil_emitter(ec, root, vec, {"i0", "i1", "i2"});
    ec.indent = 10;
    ec.idx64 = ec.idx64 || eb.idx64;
    ec.inputs = eb.inputs;
    ec.direct_expr = vec_name;
    ec.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
      if (ec.inputs[slot] != prev) return false;
      std::ostringstream e;
      e << "ldsB[sb" << (hR.hi[0] - off[0]) << " + (ly + " << (off[1] + hR.lo[1]) << ") * " << BX << " + lxe + l + " << (bxl + off[2]) << "]";
      *expr = e.str();
      return true;
    };
    std::string valC = ec.emit(root, root_index(dims));
    std::string bodyC = ec.take_code();
    for (auto& dv : ec.direct_vecs) if (dv.second != 0) return false;
    for (auto& l : ec.loads) if (l.node == prev && !l.affine) return false;
    const std::string it = ec.idx_t();
    const std::string LL = ec.idx64 ? "LL" : "";
    const int prev_slot = ec.slot_of(prev), sslot = ec.slot_of(src);
    auto vts_of = [&](Emitter& em, int slot) { return "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vec) + ">"; };

    const int64_t ntx = (x_hi - x_lo + TX - 1) / TX, nty = (Y + TY - 1) / TY, ntz = (Z + ZC - 1) / ZC;
    std::ostringstream o;
    const int64_t launch_blocks = emit_tile_order(o, ntx, nty, ntz, TX, TY, (int)ZC, std::max(1, 32 / TY), bid, x_lo);
    o << "  const int zend = z0 + " << ZC << " < " << Z << " ? z0 + " << ZC << " : " << Z << ";\n";
    // The first step is evaluated in two passes.  The inner pass maps thread -> point exactly as
    // the second step does, so the streamed inputs it loads for plane b are still in its registers
    // when the second step reaches that plane.  The shell pass covers the rest of region B (the
    // second step's halo in y/x): NSH vectors, enumerated row by row.
    const int64_t nTop = hR.lo[1] * BXV, nBot = hR.hi[1] * BXV, nL = bxl / vec, nR = bxh / vec, nS = nL + nR;
    const int64_t NSH = nTop + nBot + (int64_t)TY * nS, NSP = (NSH + NB - 1) / NB;
    if (NSP > 2) return false;
    const int64_t h = hR.hi[0];   // the second step's plane z is the first step's plane b - h
    // plane-independent parts of the addresses (clamped into the array; clamped cells are never used)
    o << "  " << it << " poffA[" << NLA << "];\n";
    o << "#pragma unroll\n  for (int q = 0; q < " << NLA << "; ++q) {\n";
    o << "    const int v = rx_min((int)threadIdx.x + q * " << NB << ", " << AV - 1 << ");\n";
    o << "    const int xv = v % " << AXV << ", yy = v / " << AXV << ";\n";
    o << "    poffA[q] = rx_clamp_idx<" << it << ">(y0 - " << (hR.lo[1] + hP.lo[1]) << " + yy, " << Y - 1 << ") * " << X << " + rx_clamp_idx<" << it << ">(x0 - "
      << (bxl + axl) << " + xv * " << vec << ", " << X - vec << ");\n  }\n";
    o << "  const int ly = threadIdx.x / " << TXV << ", lxe = (threadIdx.x % " << TXV << ") * " << vec << ";\n";
    o << "  const " << it << " i1 = rx_min<" << it << ">(y0 + ly, " << Y - 1 << "), i2b = rx_min<" << it << ">(x0 + lxe, " << X - vec << ");\n";
    o << "  const bool live = y0 + ly < " << Y << " && x0 + lxe < " << X << ";\n";
    o << "  const " << it << " colc = i1 * " << X << " + i2b;\n";
    if (NSP > 0) {
      o << "  int sby[" << NSP << "], sbxe[" << NSP << "];\n  " << it << " soff[" << NSP << "];\n";
      o << "#pragma unroll\n  for (int q = 0; q < " << NSP << "; ++q) {\n";
      o << "    const int s = rx_min((int)threadIdx.x + q * " << NB << ", " << NSH - 1 << ");\n";
      o << "    int yy, xv;\n";
      o << "    if (s < " << nTop << ") { yy = s / " << BXV << "; xv = s % " << BXV << "; }\n";
      o << "    else if (s < " << nTop + nBot << ") { const int r = s - " << nTop << "; yy = " << hR.lo[1] + TY << " + r / " << BXV << "; xv = r % " << BXV << "; }\n";
      if (nS > 0)
        o << "    else { const int r = s - " << nTop + nBot << ", c = r % " << nS << "; yy = " << hR.lo[1] << " + r / " << nS << "; xv = c < " << nL << " ? c : c + " << TXV << "; }\n";
      else
        o << "    else { yy = 0; xv = 0; }\n";
      o << "    sby[q] = yy; sbxe[q] = xv * " << vec << ";\n";
      o << "    soff[q] = rx_clamp_idx<" << it << ">(y0 - " << hR.lo[1] << " + yy, " << Y - 1 << ") * " << X << " + rx_clamp_idx<" << it << ">(x0 - " << bxl
        << " + xv * " << vec << ", " << X - vec << ");\n  }\n";
    }
    // Schedule: iteration n evaluates first-step plane n (from source planes that were in the ring
    // before the iteration began), the output plane whose first-step planes were all finished
    // before the iteration began, and puts the next source plane into the ring -- three pieces of
    // work that touch disjoint ring slots, so one barrier per iteration is enough.  The rings hold
    // one plane more than a stencil's reach for that.
    o << "  const int tA0 = z0 - " << (hR.lo[0] + hP.lo[0]) << ", zb0 = z0 - " << hR.lo[0] << ";\n";
    o << "  const int nB = zend - z0 + " << dB << ", nit = nB + 1;\n";
    o << "  auto plane = [&](int p) { return (" << it << ")rx_clamp_idx<int>(p, " << Z - 1 << ") * " << Y * X << LL << "; };\n";
    // Requests run PD planes ahead of their use: with one plane ahead the bytes in flight (3 workgroups of 256 threads
    // per CU, about 90 bytes each) divided by the memory latency are what the kernel moves, not what the memory
    // system can (measured: 5.3 TB/s against 6.5 for a plain copy).  Registers that receive a request are named by the
    // iteration's parity, so the loop body is instantiated for both.
    const int PD = opt.march2_prefetch == 2 ? 2 : 1;
    auto par = [&](const std::string& e) { return PD == 2 ? "[" + e + "]" : std::string(); };
    // prologue: the source planes the first first-step plane needs
    o << "  " << vt << " preA" << (PD == 2 ? "[2]" : "") << "[" << NLA << "];\n";
    o << "  {\n    " << vt << " pro[" << dA + 1 << "][" << NLA << "];\n";
    for (int64_t k = 0; k <= dA; ++k)
      o << "#pragma unroll\n    for (int q = 0; q < " << NLA << "; ++q) pro[" << k << "][q] = rx_load<" << vt << ">(in" << sslot << " + plane(tA0 + " << k
        << ") + poffA[q]);\n";
    o << "#pragma unroll\n    for (int q = 0; q < " << NLA << "; ++q) preA" << par("0") << "[q] = rx_load<" << vt << ">(in" << sslot << " + plane(tA0 + " << dA + 1 << ") + poffA[q]);\n";
    if (PD == 2)
      o << "#pragma unroll\n    for (int q = 0; q < " << NLA << "; ++q) preA[1][q] = rx_load<" << vt << ">(in" << sslot << " + plane(tA0 + " << dA + 2 << ") + poffA[q]);\n";
    std::set<int> stream_slots;
    for (auto& dv : eb.direct_vecs) stream_slots.insert(dv.first);
    for (auto& dv : ec.direct_vecs) stream_slots.insert(dv.first);
    const int64_t QL = h + 2;   // plane b of the first step is plane b - h - 1 ... of the second, one iteration later
    for (int64_t k = 0; k <= dA; ++k) {
      o << "#pragma unroll\n    for (int q = 0; q < " << NLA << "; ++q) {\n";
      o << "      const int v = threadIdx.x + q * " << NB << ";\n";
      o << "      if (v < " << AV << ") rx_store(ldsA + " << k * APLANE << " + v * " << vec << ", pro[" << k << "][q]);\n    }\n";
    }
    o << "  }\n";
    for (int sl : stream_slots) {
      const std::string vts = vts_of(ec, sl);
      o << "  " << vts << " uq" << sl << "[" << QL << "], un" << sl << (PD == 2 ? "[2]" : "") << ";\n";
      o << "  uq" << sl << "[0] = rx_load<" << vts << ">(in" << sl << " + plane(zb0) + colc);\n";
      if (PD == 2) o << "  un" << sl << "[1] = rx_load<" << vts << ">(in" << sl << " + plane(zb0 + 1) + colc);\n";
      if (NSP > 0 && eb.direct_vecs.count({sl, 0})) {
        o << "  " << vts << " us" << sl << "[" << NSP << "], usn" << sl << (PD == 2 ? "[2]" : "") << "[" << NSP << "];\n";
        o << "#pragma unroll\n  for (int q = 0; q < " << NSP << "; ++q) us" << sl << "[q] = rx_load<" << vts << ">(in" << sl << " + plane(zb0) + soff[q]);\n";
        if (PD == 2)
          o << "#pragma unroll\n  for (int q = 0; q < " << NSP << "; ++q) usn" << sl << "[1][q] = rx_load<" << vts << ">(in" << sl << " + plane(zb0 + 1) + soff[q]);\n";
      }
    }
    o << "  rx_lds_barrier();\n";
    // body of the first step for one vector of region B
    auto emit_B = [&](const std::string& pad, const std::string& by, const std::string& bxe, const std::string& j1, const std::string& j2b,
                      const std::function<std::string(int)>& stream, const std::string& ldsoff) {
      o << pad << "{\n";
      o << pad << "  const int by = " << by << ", bxe = " << bxe << ";\n";
      o << pad << "  const " << it << " j1 = " << j1 << ", j2b = " << j2b << ";\n";
      for (auto& dv : eb.direct_vecs) o << pad << "  const " << vts_of(eb, dv.first) << " b" << vec_name(dv.first, 0) << " = " << stream(dv.first) << ";\n";
      o << pad << "  " << vt << " res;\n";
      o << "#pragma unroll\n" << pad << "  for (int l = 0; l < " << vec << "; ++l) {\n";
      o << pad << "    const " << it << " j2 = j2b + l;\n";
      o << bodyB;
      o << pad << "    res.v[l] = " << Emitter::store_conv(pn.ty.dt, valB) << ";\n" << pad << "  }\n";
      o << pad << "  rx_store(dstb + " << ldsoff << ", res);\n";
      o << pad << "}\n";
    };
    if (PD == 2) o << "  auto iter = [&](auto PAR, const int n) __attribute__((always_inline)) {\n    constexpr int P = decltype(PAR)::value;\n";
    else o << "  for (int n = 0; n < nit; ++n) {\n";
    // requests for the iteration PD ahead
    o << "    if (n + " << PD << " < nB) {\n";
    for (int sl : stream_slots) {
      const std::string vts = vts_of(ec, sl);
      o << "      un" << sl << par("P") << " = rx_load<" << vts << ">(in" << sl << " + plane(zb0 + n + " << PD << ") + colc);\n";
      if (NSP > 0 && eb.direct_vecs.count({sl, 0}))
        o << "#pragma unroll\n      for (int q = 0; q < " << NSP << "; ++q) usn" << sl << par("P") << "[q] = rx_load<" << vts << ">(in" << sl << " + plane(zb0 + n + " << PD << ") + soff[q]);\n";
    }
    o << "    }\n";
    // the source plane requested last iteration goes to the ring; request the one after it
    o << "    if (n + 1 < nB) {\n";
    o << "      " << st << "* dst = ldsA + ((n + " << dA + 1 << ") % " << RA << ") * " << APLANE << ";\n";
    o << "#pragma unroll\n      for (int q = 0; q < " << NLA << "; ++q) {\n";
    o << "        const int v = threadIdx.x + q * " << NB << ";\n";
    o << "        if (v < " << AV << ") rx_store(dst + v * " << vec << ", preA" << par("P") << "[q]);\n      }\n";
    o << "      if (n + " << PD + 1 << " < nB) {\n";
    o << "#pragma unroll\n        for (int q = 0; q < " << NLA << "; ++q) preA" << par("P") << "[q] = rx_load<" << vt << ">(in" << sslot << " + plane(tA0 + n + " << dA + 1 + PD
      << ") + poffA[q]);\n";
    o << "      }\n    }\n";
    // one output plane of the second step
    o << "    const int iz = n - " << dB + 1 << ";\n";
    o << "    if (iz >= 0 && live) {\n";
    o << "      const int z = z0 + iz;\n";
    for (int64_t k = 0; k <= dB; ++k) o << "      const int sb" << k << " = ((n + " << (2 * RB - 1 - k) << ") % " << RB << ") * " << BPLANE << ";\n";
    o << "      const " << it << " i0 = z;\n";
    o << "      const " << it << " lin0 = (i0 * " << Y << " + i1) * " << X << LL << " + i2b;\n";
    for (auto& dv : ec.direct_vecs) o << "      const " << vts_of(ec, dv.first) << " " << vec_name(dv.first, 0) << " = uq" << dv.first << "[" << h + 1 << "];\n";
    o << "      " << vt << " res;\n";
    o << "#pragma unroll\n      for (int l = 0; l < " << vec << "; ++l) {\n";
    o << "        const " << it << " i2 = i2b + l;\n";
    o << bodyC;
    o << "        res.v[l] = " << ec.store_value(rn.ty.dt, valC) << ";\n      }\n";
    o << "      " << (opt.nt_stores ? "rx_store_nt" : "rx_store") << "(out0 + lin0, res);\n";
    o << "    }\n";
    // one plane of the first step
    o << "    if (n < nB) {\n";
    o << "      const int b = zb0 + n;\n";
    for (int64_t k = 0; k <= dA; ++k) o << "      const int sa" << k << " = ((n + " << (dA - k) << ") % " << RA << ") * " << APLANE << ";\n";
    o << "      " << st << "* dstb = ldsB + (n % " << RB << ") * " << BPLANE << ";\n";
    o << "      const " << it << " j0 = rx_clamp_idx<" << it << ">(b, " << Z - 1 << ");\n";
    emit_B("      ", "ly + " + std::to_string(hR.lo[1]), "lxe + " + std::to_string(bxl), "i1", "i2b",
           [&](int sl) { return "uq" + std::to_string(sl) + "[0]"; }, "by * " + std::to_string(BX) + " + bxe");
    for (int64_t q = 0; q < NSP; ++q) {
      o << "      if ((int)threadIdx.x + " << q * NB << " < " << NSH << ") {\n";
      const std::string qs = std::to_string(q);
      emit_B("        ", "sby[" + qs + "]", "sbxe[" + qs + "]",
             "rx_clamp_idx<" + it + ">(y0 - " + std::to_string(hR.lo[1]) + " + sby[" + qs + "], " + std::to_string(Y - 1) + ")",
             "rx_clamp_idx<" + it + ">(x0 - " + std::to_string(bxl) + " + sbxe[" + qs + "], " + std::to_string(X - vec) + ")",
             [&](int sl) { return "us" + std::to_string(sl) + "[" + qs + "]"; }, "by * " + std::to_string(BX) + " + bxe");
      o << "      }\n";
    }
    o << "    }\n";
    // the streamed inputs move one plane on
    for (int sl : stream_slots) {
      for (int64_t k = QL - 1; k >= 1; --k) o << "    uq" << sl << "[" << k << "] = uq" << sl << "[" << k - 1 << "];\n";
      o << "    uq" << sl << "[0] = un" << sl << par("P ^ 1") << ";\n";
      if (NSP > 0 && eb.direct_vecs.count({sl, 0}))
        o << "#pragma unroll\n    for (int q = 0; q < " << NSP << "; ++q) us" << sl << "[q] = usn" << sl << par("P ^ 1") << "[q];\n";
    }
    o << "    rx_lds_barrier();\n";
    if (PD == 2) o << "  };\n  for (int n = 0; n < nit; n += 2) {\n    iter(rx_int<0>{}, n);\n    if (n + 1 < nit) iter(rx_int<1>{}, n + 1);\n  }\n";
    else o << "  }\n";
    R->text = o.str();
    R->blocks = launch_blocks;
    R->lds_a = RA * APLANE;
    R->lds_b = RB * BPLANE;
    R->nb = (int)NB;
    R->prev_slot = prev_slot;
    R->inputs = ec.inputs;
    R->first_inputs = eb.inputs;
    std::set<int> read2;
    for (auto& l : ec.loads) read2.insert(l.node);
    R->reads2.assign(read2.begin(), read2.end());
    std::ostringstream note;
    note << TY << "x" << TX << " outputs per plane, " << ZC << " planes per workgroup, rings of " << RA << " and " << RB << " planes in LDS";
    R->note = note.str();
    return true;
    };
    const int TY0 = opt.march2_tile[0], TX0 = opt.march2_tile[1];
    std::vector<Region> regions(1);
    // A last tile column that is nearly empty (518 columns in tiles of 64: eight full ones and six columns) costs as
    // many workgroups as a full one, each as long-lived.  Those columns go to tiles a quarter as wide and four times as
    // tall instead: the same number of threads, and for symmetric halos the same planes in LDS.
    const int64_t rem = X % TX0;
    bool split = false;
    if (opt.march2_edge && rem > 0 && rem * 4 <= TX0 && X / TX0 >= 2 && (TX0 / 4) % spR.vec == 0 && TX0 / 4 >= 2 * spR.vec) {
      std::vector<Region> two(2);
      if (gen(TY0, TX0, 0, X - rem, "blockIdx.x", &two[0]) &&
          gen(TY0 * 4, TX0 / 4, X - rem, X, "(blockIdx.x - " + std::to_string(two[0].blocks) + "u)", &two[1]) &&
          two[0].nb == two[1].nb && two[0].inputs == two[1].inputs && two[0].prev_slot == two[1].prev_slot &&
          std::max(two[0].lds_a, two[1].lds_a) + std::max(two[0].lds_b, two[1].lds_b) <= (two[0].lds_a + two[0].lds_b) * 5 / 4) {
        regions = two;
        split = true;
      }
    }
    if (!split && !gen(TY0, TX0, 0, X, "blockIdx.x", &regions[0])) return false;
    const Region& R0 = regions[0];
    const std::string st = info(rn.ty.dt).stype;
    const std::string kname = "@K@_stencil2m";
    std::ostringstream o;
    o << "// two stencil steps, marching along dim 0 (" << R0.note;
    if (split) o << "; the last " << rem << " columns in tiles of " << regions[1].note;
    o << "): " << describe(prev) << " ; " << describe(root) << " -> " << rn.ty.str() << "\n";
    {
      std::string sg = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(R0.nb) + ") void " + kname + "(";
      for (size_t k = 0; k < R0.inputs.size(); ++k) {
        if ((int)k == R0.prev_slot) continue;
        sg += ptr_decl(info(g.nodes[R0.inputs[k]].ty.dt).stype, true, "in" + std::to_string(k)) + ", ";
      }
      sg += ptr_decl(st, false, "out0") + ")";
      o << sg << " {\n";
    }
    int64_t lds_a = 0, lds_b = 0, launch_blocks = 0;
    for (auto& R : regions) { lds_a = std::max(lds_a, R.lds_a); lds_b = std::max(lds_b, R.lds_b); launch_blocks += R.blocks; }
    // the two rings: static LDS up to the 64 KB that a static array may take, dynamic beyond
    const int es_k = info(rn.ty.dt).size;
    const bool dyn_lds = (lds_a + lds_b) * es_k > 64 * 1024;
    if (dyn_lds) {
      o << "  extern __shared__ __attribute__((aligned(16))) " << st << " rx_rings[];\n";
      o << "  " << st << "* const ldsA = rx_rings;\n  " << st << "* const ldsB = rx_rings + " << lds_a << ";\n";
    } else {
      o << "  __shared__ __attribute__((aligned(16))) " << st << " ldsA[" << lds_a << "];\n";
      o << "  __shared__ __attribute__((aligned(16))) " << st << " ldsB[" << lds_b << "];\n";
    }
    if (split) o << "  if (blockIdx.x < " << R0.blocks << "u) {\n" << R0.text << "  } else {\n" << regions[1].text << "  }\n";
    else o << R0.text;
    o << "}\n\n";
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = "map_stencil_lds2";
    L.grid[0] = (unsigned)launch_blocks;
    L.block[0] = R0.nb;
    L.lds_bytes = (unsigned)((dyn_lds ? (lds_a + lds_b) * es_k : 0) + opt.march2_lds_ballast);   // the ballast (occupancy experiments) is never touched
    for (size_t k = 0; k < R0.inputs.size(); ++k) {
      if ((int)k == R0.prev_slot) continue;
      L.args.push_back(buffer_for(R0.inputs[k]));
    }
    L.args.push_back(buffer_for(root));
    // both steps' compulsory traffic: the first step's inputs and output, then the second's
    L.algo_bytes = algo_bytes(R0.first_inputs, {prev}) + algo_bytes(R0.reads2, {root});
    L.desc = describe(prev) + " ; " + describe(root);
    plan.launches.push_back(L);
    return true;
  }

  // ------------------------------------------------------------------ maps with transposed reads
  // A map that reads an input with its two fastest-varying roles swapped (out[.., a, b] uses
  // in[.., b, .., a]: the output's minor index selects a slow dimension of the input) would read
  // that input with a large stride per lane.  Here a workgroup owns a 64 x 64 tile of the two
  // dimensions involved: the input tile is read along the input's own minor dimension
  // (coalesced), parked in LDS with a one-element row pad, and read back transposed.
  bool emit_map_transposed(int root) {
    const Node& rn = g.nodes[root];
    const auto& dims = rn.ty.dims;
    const int n = rn.ty.rank();
    if (!opt.lds_transpose || n < 2 || rn.ty.numel() < (1 << 16)) return false;
    const int TS = 64, ROWS = kBlock / TS;
    auto fresh_emitter = [&](Emitter& em) {
      em.excess_precision = opt.excess_precision;
      em.idx64 = needs64(cone_nodes(root));
      std::vector<std::string> vars;
      for (int d = 0; d < n; ++d) vars.push_back("i" + std::to_string(d));
      em.set_root(dims, vars, false);
      em.vec = 1;
      em.indent = 6;
      em.offset_perms = opt.transpose_offsets;
    };
    // pass 1: which reads are transposed, and against which root dimension
    Emitter probe(g, [&](int x) { return x != root && mat[x]; });
    fresh_emitter(probe);
    probe.emit(root, root_index(dims));
    int q = -1;                      // root dimension that indexes the staged inputs' minor dimension
    std::map<int, std::vector<int>> staged;   // node -> root_var
    // constant offsets of the staged reads (a transpose of a padded or sliced operand): the tile is then read at
    // positions clamped into the operand, and whatever guards the read in the map (the pad's test) guards the tile read
    std::map<int, std::vector<int64_t>> staged_off;
    std::set<int> conflicting;
    for (auto& l : probe.loads) {
      if (l.root_var.empty()) continue;
      {
        auto so = staged_off.find(l.node);
        if (so != staged_off.end() && so->second != l.root_off) conflicting.insert(l.node);
        staged_off[l.node] = l.root_off;
      }
      const int in_minor_var = l.root_var.back();
      if (in_minor_var == n - 1) continue;                     // its minor dim already follows the output's
      if (dims[in_minor_var] < 16 || dims[n - 1] < 16) continue;
      const int es = info(g.nodes[l.node].ty.dt).size;
      if (es != 2 && es != 4 && es != 8) continue;
      if (q < 0) q = in_minor_var;
      if (in_minor_var != q) continue;                          // one tiling serves one pairing
      auto it2 = staged.find(l.node);
      if (it2 != staged.end() && it2->second != l.root_var) continue;
      staged[l.node] = l.root_var;
    }
    for (int c : conflicting) staged.erase(c);   // read at several offsets: not one tile
    if (staged.empty()) return false;
    auto plain = [&](int node) {   // the read is a pure permutation of an operand of the root's extents
      const Node& in = g.nodes[node];
      const auto& rv = staged[node];
      for (int d = 0; d < in.ty.rank(); ++d)
        if (staged_off[node][d] != 0 || in.ty.dims[d] != dims[rv[d]]) return false;
      return true;
    };
    // Whole 16-byte vectors on both sides where the two dimensions allow it: a tile of 64 input columns x 128 input
    // rows (64 x 64 for 8-byte elements) is read with 16-byte loads, parked with a row pitch of 64 + V, and written as
    // output rows of 512 bytes, each lane storing the V elements it gathered from V tile rows (8192^2 f32 transpose:
    // 134 -> 105 us; the 4-byte form moves a 256-byte row segment per wavefront instruction).
    const int es_out = info(rn.ty.dt).size;
    int V = (es_out == 2 || es_out == 4 || es_out == 8) ? 16 / es_out : 1;
    for (auto& kv : staged) if ((int)info(g.nodes[kv.first].ty.dt).size != es_out || (!plain(kv.first) && g.nodes[kv.first].ty.dims.back() < 16 / es_out)) V = 1;
    bool all_offset = true;   // every staged read carries offsets: its vectors are tested against the operand's row one by one
    for (auto& kv : staged) all_offset = all_offset && !plain(kv.first);
    if (V > 1 && (q < 0 || dims[n - 1] % V != 0 || dims[n - 1] < 32 || !opt.transpose_vectors)) V = 1;
    if (V > 1 && !all_offset && (dims[q] % V != 0 || dims[q] < 64)) V = 1;
    if (V > 1 && all_offset && dims[q] < 16) V = 1;
    // a minor dimension of at most 64 (the rows of a 56 x 56 image) takes tiles of 64 rows: 128 would be half empty
    const int TQ = TS, TM = V > 1 ? ((es_out == 8 || dims[n - 1] <= 64) ? 64 : 128) : TS, LD = V > 1 ? TQ + V : TS + 1;
    int64_t lds_total = 0;
    for (auto& kv : staged) lds_total += (int64_t)TM * LD * info(g.nodes[kv.first].ty.dt).size;
    if (lds_total > 64 * 1024) return false;

    // pass 2: emit with the transposed reads redirected to the tiles
    Emitter em(g, [&](int x) { return x != root && mat[x]; });
    fresh_emitter(em);
    em.perm_hook = [&](int slot, const std::vector<int>& rv, std::string* expr) {
      auto it2 = staged.find(em.inputs[slot]);
      if (it2 == staged.end() || it2->second != rv) return false;
      *expr = "tile" + std::to_string(slot) + "[tb * " + std::to_string(LD) + " + ta]";
      return true;
    };
    std::string val = em.emit(root, root_index(dims));
    std::string body = em.take_code();
    const std::string it = em.idx_t();
    const int64_t DQ = dims[q], DM = dims[n - 1];
    const int64_t ntq = (DQ + TQ - 1) / TQ, ntm = (DM + TM - 1) / TM;
    int64_t outer = 1;
    for (int d = 0; d < n - 1; ++d) if (d != q) outer *= dims[d];
    const int64_t nblocks = outer * ntq * ntm;
    if (nblocks >= ((int64_t)1 << 31)) return false;
    const std::string kname = "@K@_map_t";
    std::ostringstream o;
    o << "// map with transposed reads staged through 64x64 LDS tiles: " << describe(root) << " -> " << rn.ty.str() << "\n";
    o << signature(kname, em.inputs, {{info(rn.ty.dt).stype, "out0"}}) << " {\n";
    for (auto& kv : staged) {
      const int slot = em.slot_of(kv.first);
      o << "  __shared__ __attribute__((aligned(16))) " << info(g.nodes[kv.first].ty.dt).stype << " tile" << slot << "[" << TM * LD << "];\n";
    }
    // block -> (outer coordinates, tile of dimension q, tile of the minor dimension)
    // Tiles are taken in blocks of B x B (B along the output's minor dimension first, then bands of B tiles of
    // dimension q), so that the workgroups running at one time read and write runs of B neighbouring row segments
    // instead of one: 8192^2 f32, 102 us with tiles in plain order down the input, 89 us with B = 8 (4: 103, 16: 91,
    // Morton order: 95).  Ragged edges keep the scheme with narrower blocks.
    o << "  unsigned rest = blockIdx.x;\n";
    const int B = opt.transpose_block;
    if (B > 1 && ntm > 1 && ntq > 1) {
      o << "  const unsigned pair = rest % " << ntm * ntq << "u; rest /= " << ntm * ntq << "u;\n";
      o << "  const unsigned band = pair / " << ntm * B << "u, wq = rx_min<unsigned>(" << B << "u, " << ntq << "u - band * " << B << "u);\n";
      o << "  const unsigned idx = pair - band * " << ntm * B << "u, mblk = idx / (" << B << "u * wq), wi = idx - mblk * " << B << "u * wq;\n";
      o << "  const unsigned hm = rx_min<unsigned>(" << B << "u, " << ntm << "u - mblk * " << B << "u);\n";
      o << "  const " << it << " m0 = (" << it << ")(mblk * " << B << "u + wi % hm) * " << TM << ";\n";
      o << "  const " << it << " q0 = (" << it << ")(band * " << B << "u + wi / hm) * " << TQ << ";\n";
    } else {
      o << "  const " << it << " m0 = (" << it << ")(rest % " << ntm << "u) * " << TM << "; rest /= " << ntm << "u;\n";
      o << "  const " << it << " q0 = (" << it << ")(rest % " << ntq << "u) * " << TQ << "; rest /= " << ntq << "u;\n";
    }
    for (int d = n - 2; d >= 0; --d) {
      if (d == q) continue;
      o << "  const " << it << " i" << d << " = (" << it << ")(rest % " << dims[d] << "u); rest /= " << dims[d] << "u;\n";
    }
    o << "  const int lane = threadIdx.x % " << TS << ", grp = threadIdx.x / " << TS << ";\n";
    // phase 1: read each staged input along its own minor dimension.  A tile that sticks out of the array reads the
    // last row / vector again instead of skipping the load (what it parks there is never used): a load under its own
    // condition is a branch of its own, and the loads of a workgroup then wait for one another (8192^2 f32: three of
    // the eight loads of a lane were issued one after the other's data had arrived, 105 us; all eight at once, 92)
    const bool full_m = DM % TM == 0, full_q = DQ % TQ == 0;
    auto row_of = [&](const std::string& e) { return full_m ? "(" + e + ")" : "rx_min<" + it + ">(" + e + ", " + std::to_string(DM - 1) + ")"; };
    auto col_of = [&](const std::string& e, int v) { return full_q ? "(" + e + ")" : "rx_min<" + it + ">(" + e + ", " + std::to_string(DQ - v) + ")"; };
    for (auto& kv : staged) {
      const int slot = em.slot_of(kv.first);
      const Node& in = g.nodes[kv.first];
      const auto& rv = kv.second;
      // linear offset of the tile origin's row: every input dim d is indexed by root var rv[d]
      std::vector<int64_t> stride(in.ty.rank(), 1);
      for (int d = in.ty.rank() - 2; d >= 0; --d) stride[d] = stride[d + 1] * in.ty.dims[d + 1];
      std::string base = "0";
      int64_t stride_m = 0;
      const bool pl = plain(kv.first);
      const auto& off = staged_off[kv.first];
      int64_t off_m = 0, off_q = 0, dim_m = 0, dim_q = 0;
      for (int d = 0; d < in.ty.rank(); ++d) {
        if (rv[d] == n - 1) { stride_m = stride[d]; off_m = off[d]; dim_m = in.ty.dims[d]; continue; }
        if (rv[d] == q) { off_q = off[d]; dim_q = in.ty.dims[d]; continue; }   // the input's minor dimension
        std::string coord = "i" + std::to_string(rv[d]);
        if (!pl && (off[d] != 0 || in.ty.dims[d] < dims[rv[d]]))
          coord = "rx_min<" + it + ">(rx_max<" + it + ">(" + coord + " + (" + std::to_string(off[d]) + "), 0), " + std::to_string(in.ty.dims[d] - 1) + ")";
        base += " + " + coord + " * " + std::to_string(stride[d]) + (em.idx64 ? "LL" : "");
      }
      o << "  {\n    const " << it << " base = " << base << ";\n";
      if (!pl) {
        // offsets: rows and columns of the operand at clamped positions; a vector that lies inside the operand's row
        // is one load (at any element address), one that crosses its ends is read element by element
        const std::string st = info(in.ty.dt).stype;
        if (V > 1) {
          const int LPR = TQ / V, RPP = kBlock / LPR;
          const std::string vts = "rx_vec<" + st + ", " + std::to_string(V) + ">";
          o << "#pragma unroll\n    for (int r = 0; r < " << TM / RPP << "; ++r) {\n";
          o << "      const int tb = r * " << RPP << " + (int)threadIdx.x / " << LPR << ", ta = ((int)threadIdx.x % " << LPR << ") * " << V << ";\n";
          o << "      const " << it << " rr = rx_min<" << it << ">(rx_max<" << it << ">(m0 + tb + (" << off_m << "), 0), " << dim_m - 1 << ");\n";
          o << "      const " << it << " cc = q0 + ta + (" << off_q << ");\n";
          o << "      const " << st << "* src = in" << slot << " + base + rr * " << stride_m << (em.idx64 ? "LL" : "") << ";\n";
          o << "      if (cc >= 0 && cc + " << V << " <= " << dim_q << ") {\n";
          o << "        rx_store(tile" << slot << " + tb * " << LD << " + ta, rx_load_unaligned<" << vts << ">(src + cc));\n";
          o << "      } else {\n#pragma unroll\n        for (int e = 0; e < " << V << "; ++e) tile" << slot << "[tb * " << LD << " + ta + e] = src[rx_min<" << it << ">(rx_max<" << it << ">(cc + e, 0), " << dim_q - 1 << ")];\n      }\n";
          o << "    }\n  }\n";
        } else {
          o << "#pragma unroll\n    for (int r = 0; r < " << TS / ROWS << "; ++r) {\n";
          o << "      const int tb = r * " << ROWS << " + grp, ta = lane;\n";
          o << "      const " << it << " rr = rx_min<" << it << ">(rx_max<" << it << ">(m0 + tb + (" << off_m << "), 0), " << dim_m - 1 << ");\n";
          o << "      const " << it << " cc = rx_min<" << it << ">(rx_max<" << it << ">(q0 + ta + (" << off_q << "), 0), " << dim_q - 1 << ");\n";
          o << "      tile" << slot << "[tb * " << TS + 1 << " + ta] = in" << slot << "[base + rr * " << stride_m << (em.idx64 ? "LL" : "") << " + cc];\n";
          o << "    }\n  }\n";
        }
        continue;
      }
      if (V > 1) {
        const int LPR = TQ / V, RPP = kBlock / LPR;    // lanes per input row, rows per pass
        const std::string vts = "rx_vec<" + std::string(info(in.ty.dt).stype) + ", " + std::to_string(V) + ">";
        o << "#pragma unroll\n    for (int r = 0; r < " << TM / RPP << "; ++r) {\n";
        o << "      const int tb = r * " << RPP << " + (int)threadIdx.x / " << LPR << ", ta = ((int)threadIdx.x % " << LPR << ") * " << V << ";\n";
        o << "      rx_store(tile" << slot << " + tb * " << LD << " + ta, rx_load_nt<" << vts << ">(in" << slot << " + base + " << row_of("m0 + tb") << " * " << stride_m << (em.idx64 ? "LL" : "")
          << " + " << col_of("q0 + ta", V) << "));\n";
        o << "    }\n  }\n";
        continue;
      }
      o << "#pragma unroll\n    for (int r = 0; r < " << TS / ROWS << "; ++r) {\n";
      o << "      const int tb = r * " << ROWS << " + grp, ta = lane;\n";
      o << "      tile" << slot << "[tb * " << TS + 1 << " + ta] = in" << slot << "[base + " << row_of("m0 + tb") << " * " << stride_m << (em.idx64 ? "LL" : "") << " + " << col_of("q0 + ta", 1) << "];\n";
      o << "    }\n  }\n";
    }
    o << "  __syncthreads();\n";
    if (V > 1) {
      // phase 2 on vectors: a lane owns V consecutive elements of an output row
      const int OPR = TM / V, ORP = kBlock / OPR;      // lanes per output row, output rows per pass
      const std::string vto = "rx_vec<" + std::string(info(rn.ty.dt).stype) + ", " + std::to_string(V) + ">";
      o << "#pragma unroll 4\n  for (int r = 0; r < " << TQ / ORP << "; ++r) {\n";
      o << "    const int ta = r * " << ORP << " + (int)threadIdx.x / " << OPR << ", tbv = ((int)threadIdx.x % " << OPR << ") * " << V << ";\n";
      o << "    const " << it << " i" << q << " = q0 + ta;\n";
      o << "    if (" << (full_q ? std::string("true") : "i" + std::to_string(q) + " < " + std::to_string(DQ)) << " && " << (full_m ? std::string("true") : "m0 + tbv < " + std::to_string(DM)) << ") {\n";
      o << "      " << vto << " res;\n";
      o << "#pragma unroll\n      for (int e = 0; e < " << V << "; ++e) {\n";
      o << "      const int tb = tbv + e;\n";
      o << "      const " << it << " i" << n - 1 << " = m0 + tb;\n";
      o << body;
      o << "      res.v[e] = " << em.store_value(rn.ty.dt, val) << ";\n      }\n";
      {
        Index rix = root_index(dims);
        rix[n - 1].var = "(m0 + tbv)";
        o << "      " << (opt.nt_stores ? "rx_store_nt" : "rx_store") << "(out0 + " << em.linear(rix, dims) << ", res);\n";
      }
      o << "    }\n  }\n}\n\n";
    } else {
    // phase 2: the map itself, lanes along the output's minor dimension
    o << "#pragma unroll 4\n  for (int r = 0; r < " << TS / ROWS << "; ++r) {\n";
    o << "    const int ta = r * " << ROWS << " + grp, tb = lane;\n";
    o << "    const " << it << " i" << q << " = q0 + ta, i" << n - 1 << " = m0 + tb;\n";
    o << "    if (" << (full_q ? std::string("true") : "i" + std::to_string(q) + " < " + std::to_string(DQ)) << " && " << (full_m ? std::string("true") : "i" + std::to_string(n - 1) + " < " + std::to_string(DM)) << ") {\n";
    o << body;
    Index rix = root_index(dims);
    o << "      out0[" << em.linear(rix, dims) << "] = " << em.store_value(rn.ty.dt, val) << ";\n";
    o << "    }\n  }\n}\n\n";
    }
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = "map_transposed";
    L.grid[0] = (unsigned)nblocks;
    L.block[0] = kBlock;
    for (int i : em.inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    L.algo_bytes = algo_bytes(em.inputs, {root});
    L.desc = describe(root);
    plan.launches.push_back(L);
    return true;
  }

  // ------------------------------------------------------------------ chains of update steps through LDS
  // A time loop over small arrays (the reference's polybench stencils, benchmark/polybench/stencil.jl)
  // unrolls into a run of steps, each a dynamic_update_slice over one array (a "field") with values
  // computed from neighbouring elements of the others.  With one launch per step such a loop is bound
  // by the gap between dependent launches, not by memory.  A chain kernel runs K consecutive steps per
  // launch: a workgroup loads its tile of every field plus a halo as wide as the K steps reach,
  // updates the fields in LDS step by step on regions that shrink by each step's reach (neighbouring
  // workgroups recompute each other's halos), and writes its tile of the fields that changed.
  // Versions of a field that are superseded inside the kernel never reach memory.
  struct ChainProbe {
    int base = -1;                 // the array the step's update is written over
    std::map<int, Halo> reads;     // inputs of the field's shape and type, and how far the step reads around a point
    std::vector<int> others;       // every other input (read from memory as in a map kernel)
  };
  std::map<int, std::vector<int>> chain_at;   // first step of a chain -> all its steps
  std::set<int> chain_member;                 // steps emitted by a chain kernel

  // steps per kernel: a 1-d tile's halo grows by a cell or two per step, so long chains stay cheap
  int chain_cap(int rank) const { return opt.chain_steps > 0 ? opt.chain_steps : rank == 1 ? 64 : rank == 2 ? 16 : 4; }

  bool probe_chain_step(int x, ChainProbe* cp) {
    const Node& n = g.nodes[x];
    const int r = n.ty.rank();
    // rank 3: only small arrays, whose steps are bound by the launch gap (32^3 and 64^3 heat steps: 1.6x and 1.4x
    // faster in chains of four); at 128^3 the redundant halo cells cost more than the launches saved
    if (r < 1 || r > 3 || (r > opt.chain_max_rank && !(r == 3 && n.ty.numel() <= opt.chain_rank3_numel))) return false;
    if (n.k == OpK::Param || n.k == OpK::Constant || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv || n.k == OpK::DotGeneral) return false;
    const int es = info(n.ty.dt).size;
    if (es != 4 && es != 8) return false;
    if (n.ty.numel() < 2 || n.ty.numel() >= opt.slab_min_numel) return false;
    // an update (x[r] = ...) supersedes the array it is written over; any other step (u = f(u), a pad
    // around a computed interior) supersedes the array it reads the farthest around a point
    int b = -1;
    if (n.k == OpK::DynamicUpdateSlice) {
      b = n.in[0];
      while (!mat[b] && g.nodes[b].k == OpK::DynamicUpdateSlice) b = g.nodes[b].in[0];
      if (!mat[b] || !(g.nodes[b].ty == n.ty)) return false;
    }
    Emitter probe(g, [&](int y) { return y != x && mat[y]; });
    std::vector<std::string> vars;
    Index ix(r);
    for (int d = 0; d < r; ++d) {
      vars.push_back("g" + std::to_string(d));
      ix[d].var = vars[d]; ix[d].lo = 0; ix[d].hi = n.ty.dims[d] - 1;
    }
    probe.set_root(n.ty.dims, vars, false);
    probe.excess_precision = opt.excess_precision;
    try { probe.emit(x, ix); } catch (const Error&) { return false; }
    cp->base = b;
    bool saw_base = false;
    for (auto& l : probe.loads) {
      const Node& ln = g.nodes[l.node];
      if (ln.ty == n.ty) {
        if (!l.affine) return false;
        Halo& h = cp->reads[l.node];
        for (int d = 0; d < r; ++d) { h.lo[d] = std::max<int64_t>(h.lo[d], -l.off[d]); h.hi[d] = std::max<int64_t>(h.hi[d], l.off[d]); }
        saw_base = saw_base || l.node == b;
      } else cp->others.push_back(l.node);
    }
    if (b < 0) {
      int64_t best = -1;
      for (auto& kv : cp->reads) {
        int64_t reach = 0;
        for (int d = 0; d < r; ++d) reach += kv.second.lo[d] + kv.second.hi[d];
        if (reach > best) { best = reach; b = kv.first; }
      }
      if (b < 0 || best == 0) return false;   // a plain elementwise step gains nothing from a tile
      cp->base = b;
      saw_base = true;
    }
    if (!saw_base) return false;
    for (auto& kv : cp->reads)
      for (int d = 0; d < r; ++d) if (kv.second.lo[d] > 4 || kv.second.hi[d] > 4) return false;
    return true;
  }

  // every kernel that reads `v` is one of `group` (or `also`)
  bool read_only_by(int v, const std::set<int>& group, int also) {
    std::vector<int> st{v};
    std::set<int> seen;
    while (!st.empty()) {
      int y = st.back();
      st.pop_back();
      for (int u : users[y]) {
        if (!live[u]) continue;
        if (mat[u]) { if (!group.count(u) && u != also) return false; }
        else if (seen.insert(u).second) st.push_back(u);
      }
    }
    return true;
  }

  // Kernel for a prefix of `steps`; returns how many steps it covers (0: none, nothing emitted).
  size_t emit_chain(const std::vector<int>& steps, const std::vector<ChainProbe>& probes) {
    const Node& n0 = g.nodes[steps[0]];
    const int r = n0.ty.rank();
    const auto& D = n0.ty.dims;
    const int es = info(n0.ty.dt).size;
    const std::string st = info(n0.ty.dt).stype;
    int64_t T[3] = {1, 1, 1};
    {
      // vectors: one cell per thread (a step costs an LDS round trip and a barrier, whatever the tile);
      // matrices: 32x64 tiles, 32x32 when that is what it takes to give every compute unit a tile
      int64_t dflt[3][3] = {{128, 1, 1}, {32, 64, 1}, {8, 8, 16}};
      if (r == 2 && ((D[0] + 31) / 32) * ((D[1] + 63) / 64) < 256) dflt[1][1] = 32;
      for (int d = 0; d < r; ++d) {
        T[d] = opt.chain_tile[d] > 0 && opt.chain_tile[r - 1] > 0 ? opt.chain_tile[d] : dflt[r - 1][d];
        T[d] = std::min<int64_t>(T[d], D[d]);
      }
    }
    for (size_t k = std::min<size_t>(steps.size(), (size_t)chain_cap(r)); k >= 2; --k) {
      // fields of the first k steps: version at kernel entry, and which field each node is a version of
      std::vector<int> entry;
      std::map<int, int> field_of;
      for (size_t i = 0; i < k; ++i) {
        for (auto& kv : probes[i].reads)
          if (!field_of.count(kv.first)) { field_of[kv.first] = (int)entry.size(); entry.push_back(kv.first); }
        field_of[steps[i]] = field_of[probes[i].base];
      }
      const int nf = (int)entry.size();
      // a step that reads the array it supersedes at other positions than its own cannot update it in
      // place: such arrays get a second tile, written and read in turns
      std::vector<char> two_tiles(nf, 0);
      for (size_t i = 0; i < k; ++i) {
        const Halo& hb = probes[i].reads.at(probes[i].base);
        for (int d = 0; d < r; ++d) if (hb.lo[d] || hb.hi[d]) two_tiles[field_of[probes[i].base]] = 1;
      }
      // an array that no step writes and every step reads at its own position only stays in memory
      std::vector<char> has_tile(nf, 0);
      for (size_t i = 0; i < k; ++i) {
        has_tile[field_of[probes[i].base]] = 1;
        for (auto& kv : probes[i].reads)
          for (int d = 0; d < r; ++d) if (kv.second.lo[d] || kv.second.hi[d]) has_tile[field_of[kv.first]] = 1;
      }
      int ntiles_lds = 0;
      for (int f = 0; f < nf; ++f) ntiles_lds += has_tile[f] ? 1 + two_tiles[f] : 0;
      std::vector<std::array<int64_t, 3>> lo(k), hi(k);
      int64_t HL[3] = {0, 0, 0}, HH[3] = {0, 0, 0};
      for (size_t i = 0; i < k; ++i) {
        lo[i] = {0, 0, 0}; hi[i] = {0, 0, 0};
        for (auto& kv : probes[i].reads)
          for (int d = 0; d < r; ++d) { lo[i][d] = std::max(lo[i][d], kv.second.lo[d]); hi[i][d] = std::max(hi[i][d], kv.second.hi[d]); }
        for (int d = 0; d < r; ++d) { HL[d] += lo[i][d]; HH[d] += hi[i][d]; }
      }
      int64_t E[3] = {1, 1, 1}, box = 1, tile = 1;
      for (int d = 0; d < r; ++d) { E[d] = T[d] + HL[d] + HH[d]; box *= E[d]; tile *= T[d]; }
      const int64_t lds_bytes = box * ntiles_lds * es;
      if (getenv("RX_CHAIN_DEBUG")) fprintf(stderr, "[chain] k=%zu box=%lld tile=%lld tiles_in_lds=%d bytes=%lld\n", k, (long long)box, (long long)tile, ntiles_lds, (long long)lds_bytes);
      if (lds_bytes > opt.chain_lds_bytes || (double)box > (r == 3 ? 2.0 : 1.0) * opt.chain_redundancy * (double)tile) continue;
      const int NB = opt.chain_threads > 0 ? opt.chain_threads : (int)std::min<int64_t>(1024, (box + 63) / 64 * 64);
      if (NB < 64 || NB > 1024 || NB % 64) continue;

      // the steps' bodies, evaluated at the array position (g0, g1, g2) whose cell in the box is `li`
      std::vector<std::string> vars;
      Index ix(r);
      for (int d = 0; d < r; ++d) {
        vars.push_back("g" + std::to_string(d));
        ix[d].var = vars[d]; ix[d].lo = 0; ix[d].hi = D[d] - 1;
      }
      std::vector<int> inputs, cur = entry, writes(k);
      std::vector<std::string> bodies(k), vals(k), wname(k);
      // tile that holds the current version of a field: lds<f> or its twin lds<f>b
      std::vector<char> side(nf, 0);
      auto tile_name = [&](int f) { return "lds" + std::to_string(f) + (side[f] ? "b" : ""); };
      int64_t margin = 0;   // farthest neighbour read, in cells: the tiles sit that far inside the LDS allocation
      std::set<int> group(steps.begin(), steps.begin() + k);
      bool ok = true;
      for (size_t i = 0; i < k && ok; ++i) {
        const int x = steps[i];
        Emitter em(g, [&, x](int y) { return y != x && mat[y]; });
        em.inputs = inputs;
        em.set_root(D, vars, false);
        em.excess_precision = opt.excess_precision;
        em.branchless_guards = opt.branchless_guards;
        em.indent = 6;
        em.tile_hook = [&](int slot, const std::vector<int64_t>& off, std::string* expr) {
          const int node = em.inputs[slot];
          auto f = field_of.find(node);
          if (f == field_of.end() || !(g.nodes[node].ty == n0.ty)) return false;
          if (cur[f->second] != node) { ok = false; return false; }
          if (!has_tile[f->second]) return false;
          int64_t delta = 0, stride = 1;
          for (int d = r - 1; d >= 0; --d) { delta += off[d] * stride; stride *= E[d]; }
          margin = std::max<int64_t>(margin, delta < 0 ? -delta : delta);
          *expr = tile_name(f->second) + "[li + (" + std::to_string(delta) + ")]";
          return true;
        };
        vals[i] = em.store_value(n0.ty.dt, em.emit(x, ix));
        bodies[i] = em.take_code();
        for (auto& l : em.loads) if (group.count(l.node) && !(l.affine && g.nodes[l.node].ty == n0.ty)) ok = false;
        inputs = em.inputs;
        writes[i] = field_of[probes[i].base];
        {
          const Halo& hb = probes[i].reads.at(probes[i].base);
          bool self = false;
          for (int d = 0; d < r; ++d) self = self || hb.lo[d] || hb.hi[d];
          if (self) side[writes[i]] = !side[writes[i]];
          wname[i] = tile_name(writes[i]);
        }
        cur[writes[i]] = x;
      }
      if (!ok) continue;

      std::ostringstream o;
      const std::string kname = "@K@_chain";
      o << "// " << k << " update steps through LDS tiles (";
      for (int d = 0; d < r; ++d) o << (d ? "x" : "") << T[d];
      o << " outputs per workgroup, box ";
      for (int d = 0; d < r; ++d) o << (d ? "x" : "") << E[d];
      o << ", " << nf << " fields): " << describe(steps[0]) << " ... -> " << n0.ty.str() << "\n";
      std::vector<int> arg_nodes;
      {
        std::string s = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(NB) + ") void " + kname + "(";
        bool first = true;
        for (size_t q = 0; q < inputs.size(); ++q) {
          if (group.count(inputs[q])) continue;
          s += (first ? "" : ", ") + ptr_decl(info(g.nodes[inputs[q]].ty.dt).stype, true, "in" + std::to_string(q));
          first = false;
          arg_nodes.push_back(inputs[q]);
        }
        for (int f = 0; f < nf; ++f)
          if (cur[f] != entry[f]) { s += (first ? "" : ", ") + ptr_decl(st, false, "out" + std::to_string(f)); first = false; }
        o << s << ") {\n";
      }
      auto slot_in = [&](int node) {
        for (size_t q = 0; q < inputs.size(); ++q) if (inputs[q] == node) return (int)q;
        return -1;
      };
      o << "  extern __shared__ __attribute__((aligned(16))) unsigned char rx_smem[];\n";
      {
        int slot = 0;
        for (int f = 0; f < nf; ++f) {
          if (!has_tile[f]) continue;
          o << "  " << st << "* const lds" << f << " = reinterpret_cast<" << st << "*>(rx_smem) + " << margin + slot++ * box << ";\n";
          if (two_tiles[f]) o << "  " << st << "* const lds" << f << "b = reinterpret_cast<" << st << "*>(rx_smem) + " << margin + slot++ * box << ";\n";
        }
      }
      int64_t nt[3] = {1, 1, 1}, ntiles = 1;
      for (int d = 0; d < r; ++d) { nt[d] = (D[d] + T[d] - 1) / T[d]; ntiles *= nt[d]; }
      o << "  int tb = blockIdx.x;\n";
      for (int d = r - 1; d >= 0; --d) {
        o << "  const int t" << d << " = (tb % " << nt[d] << ") * " << T[d] << ";\n";
        if (d) o << "  tb /= " << nt[d] << ";\n";
      }
      const int64_t R = (box + NB - 1) / NB;   // box cells per thread
      const bool fixed = R <= 8 && opt.chain_fixed_cells;
      if (!fixed) {
      // Loops over the cells of a region run a fixed number of rounds per thread without branches
      // (cells past the end repeat the last one, array positions are clamped into the array, and
      // only the final LDS or global store is predicated), so that the compiler can keep the loads
      // of several rounds in flight.
      // decode cell p of a region with extents ext[] whose first cell sits at (t - back[]) in the array
      auto open_loop = [&](int64_t total, const int64_t* ext, const int64_t* back, const char* ind) {
        const int64_t rounds = (total + NB - 1) / NB;
        o << "#pragma unroll " << std::min<int64_t>(rounds, 8) << "\n";
        o << "  for (int q = 0; q < " << rounds << "; ++q) {\n";
        o << ind << "const int p = threadIdx.x + q * " << NB << ";\n";
        o << ind << "int rr = rx_min(p, " << total - 1 << ");\n";
        for (int d = r - 1; d >= 0; --d) {
          if (d) { o << ind << "const int c" << d << " = rr % " << ext[d] << ";\n" << ind << "rr /= " << ext[d] << ";\n"; }
          else o << ind << "const int c0 = rr;\n";
        }
        std::string in_arr = "p < " + std::to_string(total);
        for (int d = 0; d < r; ++d) {
          o << ind << "const int a" << d << " = t" << d << " - " << back[d] << " + c" << d << ";\n";
          o << ind << "const int g" << d << " = rx_clamp_idx<int>(a" << d << ", " << D[d] - 1 << ");\n";
          in_arr += " && a" + std::to_string(d) + " == g" + std::to_string(d);
        }
        o << ind << "const bool live = " << in_arr << ";\n";
      };
      auto box_index = [&](const int64_t* back) {   // cell of the box that holds array position a
        std::string e;
        for (int d = 0; d < r; ++d) {
          const std::string c = "(c" + std::to_string(d) + " + " + std::to_string(HL[d] - back[d]) + ")";
          e = d ? "(" + e + ") * " + std::to_string(E[d]) + " + " + c : c;
        }
        return e;
      };
      auto array_index = [&]() {
        std::string e;
        for (int d = 0; d < r; ++d) e = d ? "(" + e + ") * " + std::to_string(D[d]) + " + g" + std::to_string(d) : "g0";
        return e;
      };
      // stage every field's box
      {
        open_loop(box, E, HL, "    ");
        o << "    const int lin = " << array_index() << ";\n";
        for (int f = 0; f < nf; ++f) if (has_tile[f]) o << "    const " << st << " s" << f << " = in" << slot_in(entry[f]) << "[lin];\n";
        o << "    if (p < " << box << ") {\n";
        for (int f = 0; f < nf; ++f) if (has_tile[f]) o << "      lds" << f << "[p] = s" << f << ";\n";
        o << "    }\n  }\n  __syncthreads();\n";
      }
      for (size_t i = 0; i < k; ++i) {
        int64_t back[3] = {0, 0, 0}, ext[3] = {1, 1, 1}, total = 1;
        for (int d = 0; d < r; ++d) {
          int64_t fwd = 0;
          for (size_t j = i + 1; j < k; ++j) { back[d] += lo[j][d]; fwd += hi[j][d]; }
          ext[d] = T[d] + back[d] + fwd;
          total *= ext[d];
        }
        o << "  // step " << i << ": " << describe(steps[i]) << "\n";
        open_loop(total, ext, back, "    ");
        o << "    {\n      const int li = " << box_index(back) << ";\n";
        o << bodies[i];
        o << "      if (live) " << wname[i] << "[li] = " << vals[i] << ";\n    }\n  }\n  __syncthreads();\n";
      }
      {
        const int64_t zero[3] = {0, 0, 0};
        open_loop(tile, T, zero, "    ");
        o << "    if (live) {\n      const int li = " << box_index(zero) << ";\n      const int lin = " << array_index() << ";\n";
        for (int f = 0; f < nf; ++f) if (cur[f] != entry[f]) o << "      out" << f << "[lin] = " << tile_name(f) << "[li];\n";
        o << "    }\n  }\n}\n\n";
      }
      } else {
        // Every thread owns the box cells p = threadIdx.x + q * NB for the whole kernel: their array
        // coordinates are worked out once and kept in registers, a step only tests whether a cell lies
        // in its region, and a cell's index in an LDS tile is p itself.  Rounds that cannot meet a
        // step's region are left out when the text is written.  Nothing branches inside a round (only
        // the final store is predicated), so the loads of several rounds stay in flight.
        auto array_index = [&]() {
          std::string e;
          for (int d = 0; d < r; ++d) e = d ? "(" + e + ") * " + std::to_string(D[d]) + " + g" + std::to_string(d) : "g0";
          return e;
        };
        for (int d = 0; d < r; ++d) o << "  int C" << d << "[" << R << "], G" << d << "[" << R << "];\n";
        o << "  bool IN[" << R << "];\n";
        o << "#pragma unroll\n  for (int q = 0; q < " << R << "; ++q) {\n";
        o << "    const int p = threadIdx.x + q * " << NB << ";\n    int rr = rx_min(p, " << box - 1 << ");\n";
        for (int d = r - 1; d >= 0; --d) {
          if (d) o << "    const int c" << d << " = rr % " << E[d] << ";\n    rr /= " << E[d] << ";\n";
          else o << "    const int c0 = rr;\n";
        }
        std::string in_arr = "p < " + std::to_string(box);
        for (int d = 0; d < r; ++d) {
          o << "    const int a" << d << " = t" << d << " - " << HL[d] << " + c" << d << ";\n";
          o << "    const int g" << d << " = rx_clamp_idx<int>(a" << d << ", " << D[d] - 1 << ");\n";
          o << "    C" << d << "[q] = c" << d << "; G" << d << "[q] = g" << d << ";\n";
          in_arr += " && a" + std::to_string(d) + " == g" + std::to_string(d);
        }
        o << "    IN[q] = " << in_arr << ";\n";
        o << "    const int lin = " << array_index() << ";\n";
        for (int f = 0; f < nf; ++f) if (has_tile[f]) o << "    const " << st << " s" << f << " = in" << slot_in(entry[f]) << "[lin];\n";
        o << "    if (p < " << box << ") {\n";
        for (int f = 0; f < nf; ++f) if (has_tile[f]) o << "      lds" << f << "[p] = s" << f << ";\n";
        o << "    }\n  }\n  __syncthreads();\n";
        const int64_t plane = box / E[0];
        auto rounds_of = [&](int64_t r0, int64_t r1, int64_t* qlo, int64_t* qhi) {   // rounds that hold cells of box rows [r0, r1)
          *qlo = r0 * plane / NB;
          *qhi = std::min<int64_t>(R, (r1 * plane + NB - 1) / NB);
        };
        auto open_round = [&](const int64_t* first, const int64_t* ext) {
          int64_t qlo, qhi;
          rounds_of(first[0], first[0] + ext[0], &qlo, &qhi);
          o << "#pragma unroll\n  for (int q = " << qlo << "; q < " << qhi << "; ++q) {\n";
          o << "    const int li = rx_min((int)threadIdx.x + q * " << NB << ", " << box - 1 << ");\n";
          std::string live = "IN[q]";
          for (int d = 0; d < r; ++d) {
            o << "    const int g" << d << " = G" << d << "[q];\n";
            live += " && (unsigned)(C" + std::to_string(d) + "[q] - " + std::to_string(first[d]) + ") < " + std::to_string(ext[d]) + "u";
          }
          o << "    const bool live = " << live << ";\n";
        };
        for (size_t i = 0; i < k; ++i) {
          int64_t first[3] = {0, 0, 0}, ext[3] = {1, 1, 1};
          for (int d = 0; d < r; ++d) {
            int64_t back = 0, fwd = 0;
            for (size_t j = i + 1; j < k; ++j) { back += lo[j][d]; fwd += hi[j][d]; }
            first[d] = HL[d] - back;
            ext[d] = T[d] + back + fwd;
          }
          o << "  // step " << i << ": " << describe(steps[i]) << "\n";
          open_round(first, ext);
          o << "    {\n" << bodies[i];
          o << "      if (live) " << wname[i] << "[li] = " << vals[i] << ";\n    }\n  }\n  __syncthreads();\n";
        }
        {
          open_round(HL, T);
          o << "    if (live) {\n      const int lin = " << array_index() << ";\n";
          for (int f = 0; f < nf; ++f) if (cur[f] != entry[f]) o << "      out" << f << "[lin] = " << tile_name(f) << "[li];\n";
          o << "    }\n  }\n}\n\n";
        }
      }
      const std::string kb_final = finalize(o.str());
      Launch L;
      L.kernel = named(kname, kb_final);
      L.kind = "map_chain";
      L.grid[0] = (unsigned)ntiles;
      L.block[0] = NB;
      L.lds_bytes = (unsigned)(lds_bytes + 2 * margin * es);
      for (int a : arg_nodes) L.args.push_back(buffer_for(a));
      std::vector<int> outs;
      for (int f = 0; f < nf; ++f) if (cur[f] != entry[f]) { L.args.push_back(buffer_for(cur[f])); outs.push_back(cur[f]); }
      L.n_outputs = (int)outs.size();
      L.algo_bytes = algo_bytes(arg_nodes, outs);
      L.desc = std::to_string(k) + " steps: " + describe(steps[0]) + " ...";
      plan.launches.push_back(L);
      return k;
    }
    return 0;
  }

  // ------------------------------------------------------------------ updates in place
  // root = dynamic_update_slice(base, update, constant starts) where `base` is a temporary that no
  // later kernel reads: the result takes over base's buffer and the kernel touches only the box
  // that changes (range `setindex!` on a traced array, src/Indexing.jl:438-443, costs the bytes of
  // the range, not of the array).  Returns the box as (start, length) per dimension.
  bool update_in_place_box(int root, std::vector<std::pair<int64_t, int64_t>>* box) {
    if (!opt.in_place_updates) return false;
    const Node& n = g.nodes[root];
    if (n.k != OpK::DynamicUpdateSlice) return false;
    const int base = n.in[0];
    const Node& bn = g.nodes[base];
    if (!mat[base] || !(bn.ty == n.ty) || bn.k == OpK::Param || bn.k == OpK::Constant) return false;
    if (reshape_alias.count(base) || reshape_alias.count(root)) return false;
    for (auto& kv : reshape_alias) if (kv.second == base) return false;
    for (int r : g.results) if (r == base) return false;
    const Node& un = g.nodes[n.in[1]];
    if (un.ty.numel() == 0) return false;
    box->clear();
    for (int d = 0; d < n.ty.rank(); ++d) {
      const Node& sn = g.nodes[n.in[2 + d]];
      if (sn.k != OpK::Constant || !sn.splat) return false;
      const int64_t room = n.ty.dims[d] - un.ty.dims[d];
      box->push_back({std::min(std::max<int64_t>(splat_as_int(sn), 0), room), un.ty.dims[d]});
    }
    // every other kernel that reads base is launched before this one
    std::vector<int> st{base};
    std::set<int> seen;
    while (!st.empty()) {
      int y = st.back();
      st.pop_back();
      for (int u : users[y]) {
        if (!live[u] || u == root) continue;
        if (mat[u]) { if (launch_position(u) > root) return false; }
        else if (seen.insert(u).second) st.push_back(u);
      }
    }
    return true;
  }

  // Kernels are launched in the node order of their jobs, but some values are computed by a job
  // that comes later than their own node: a product absorbed by its epilogue runs at the
  // epilogue's root, a reduction fused into a row kernel at the row anchor, a stencil step that
  // lives in LDS only inside the kernel of the step that reads it.
  int launch_position(int u) const {
    auto e = epilogue_of.find(u);
    if (e != epilogue_of.end()) return e->second;
    auto r = row_anchor.find(u);
    if (r != row_anchor.end()) return r->second;
    if (lds_only.count(u))
      for (auto& kv : fuse_prev) if (kv.second == u) return kv.first;
    return u;
  }

  // ------------------------------------------------------------------ map kernels
  // `value` >= 0: write that node's values (same type as `root`) into root's buffer instead of
  // evaluating root itself (the copy of the operand a scatter starts from).
  void emit_map(int root, int value = -1) {
    if (value < 0) {
      if (lds_only.count(root)) return;   // evaluated inside its only reader's kernel
      if (emit_map_lds(root)) return;
      if (emit_map_transposed(root)) return;
    }
    const Node& rn = g.nodes[root];
    const auto& dims = rn.ty.dims;
    const int n = rn.ty.rank();
    const int vec = pick_vec(rn.ty);
    const int64_t numel = rn.ty.numel();
    if (numel == 0) return;
    const int64_t nv = numel / vec;
    const std::string kname = "@K@_map";
    Emitter em(g, [&](int x) { return x != root && mat[x]; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(value >= 0 ? value : root)) || numel >= ((int64_t)1 << 31);
    const std::string it = em.idx_t();
    std::vector<std::string> vars;
    for (int d = 0; d < n; ++d) vars.push_back("i" + std::to_string(d));
    em.set_root(dims, vars, vec > 1);
    em.vec = vec;
    em.allow_shifted = opt.shifted_vector_loads;
    // narrow elements, several per lane: padded reads at clamped positions, so that a lane's loads combine (the map
    // between two 16-bit convolutions, 107 MB: 54 -> 24 us)
    // where every read runs along the root's minor dimension (a padded copy in the same layout; not a transposing read,
    // whose loads cannot combine and which the clamps only slow down: 42 -> 60 us)
    if (opt.clamp_pad_reads && vec > 1 && info(rn.ty.dt).size <= 2) {
      Emitter probe(g, [&](int x) { return x != root && mat[x]; });
      probe.excess_precision = opt.excess_precision;
      probe.idx64 = em.idx64;
      probe.set_root(dims, vars, true);
      probe.vec = vec;
      probe.allow_shifted = opt.shifted_vector_loads;
      probe.direct_expr = vec_name;
      probe.emit(value >= 0 ? value : root, root_index(dims));
      bool follows = !probe.loads.empty();
      for (auto& l : probe.loads) follows = follows && (l.minor_follows || g.nodes[l.node].ty.rank() == 0);
      em.clamp_guards = follows;
    }
    em.direct_expr = vec_name;
    em.indent = 4;
    Index ix = root_index(dims);
    // evaluate the root op itself (it is materialized, so bypass the input test by emitting its op)
    std::string val = em.emit(value >= 0 ? value : root, ix);
    std::string body = em.take_code();
    // an update that can take over its operand's buffer: the kernel reads that operand only at the
    // position it writes
    std::vector<std::pair<int64_t, int64_t>> box;
    bool inplace = value < 0 && n >= 1 && update_in_place_box(root, &box);
    if (inplace)
      for (auto& l : em.loads)
        if (l.node == rn.in[0]) {
          bool own = l.affine;
          for (auto off : l.off) own = own && off == 0;
          inplace = inplace && own;
        }

    // does the update itself use the old values (x[r] .+= ...), or only the copy around the box?
    bool update_reads_base = false;
    if (inplace) {
      std::vector<int> st{rn.in[1]};
      std::set<int> seen;
      while (!st.empty() && !update_reads_base) {
        int y = st.back();
        st.pop_back();
        if (y == rn.in[0]) { update_reads_base = true; break; }
        if (mat[y] || !seen.insert(y).second) continue;
        for (int i : g.nodes[y].in) st.push_back(i);
      }
    }

    // shifted loads along the slowest dimension -> XCD slab order
    bool slab = false;
    if (opt.xcd_slabs && n >= 3 && dims[0] >= 8 && dims[1] >= 8 && numel >= opt.slab_order_min_numel) {
      std::map<int, std::set<int64_t>> offs0;
      for (auto& l : em.loads)
        if (l.affine && (int)l.off.size() == n) offs0[l.node].insert(l.off[0]);
      for (auto& kv : offs0) slab = slab || kv.second.size() > 1;
    }

    std::ostringstream o;
    std::vector<std::pair<std::string, std::string>> outs{{info(rn.ty.dt).stype, "out0"}};
    o << "// map: " << (value >= 0 ? "copy of " + describe(value) : describe(root)) << " -> " << rn.ty.str() << "\n";
    o << signature(kname, em.inputs, outs) << " {\n";
    unsigned grid;
    if (!slab) {
      const int64_t nblocks = (nv + kBlock - 1) / kBlock;
      grid = (unsigned)nblocks;
      o << "  const " << it << " vid = (" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x;\n";
      o << "  if (vid >= " << nv << ") return;\n";
      decode_index(o, it, "vid", dims, vec, "  ");
      o << "  const " << it << " lin0 = vid * " << vec << ";\n";
    } else {
      // XCD x owns rows [y0, y1) of dimension 1 for every index of dimension 0; inside an
      // XCD the tiles advance along dimension 0 so that its L2 keeps the neighbouring planes.
      int64_t plane = numel / dims[0];
      int64_t rowlen = plane / dims[1];
      int64_t ymax = (dims[1] + 7) / 8;
      int64_t bps = (ymax * rowlen / vec + kBlock - 1) / kBlock;
      grid = (unsigned)(8 * dims[0] * bps);
      o << "  const unsigned xcd = blockIdx.x & 7u, lb = blockIdx.x >> 3;\n";
      o << "  const " << it << " i0 = lb / " << bps << "u;\n";
      o << "  const " << it << " cb = lb % " << bps << "u;\n";
      o << "  const " << it << " y0 = (" << it << ")xcd * " << dims[1] << " / 8, y1 = (" << it << ")(xcd + 1) * " << dims[1] << " / 8;\n";
      o << "  const " << it << " e = (cb * " << kBlock << " + threadIdx.x) * " << vec << ";\n";
      o << "  if (e >= (y1 - y0) * " << rowlen << ") return;\n";
      o << "  const " << it << " pe = y0 * " << rowlen << " + e;\n";
      // decode pe inside the plane: dims[1..n-1]
      {
        std::string rest = "pe";
        o << "  const " << it << " i" << n - 1 << "b = " << rest << " % " << dims[n - 1] << ";\n";
        o << "  " << it << " rr = " << rest << " / " << dims[n - 1] << ";\n";
        for (int d = n - 2; d >= 2; --d) {
          o << "  const " << it << " i" << d << " = rr % " << dims[d] << ";\n";
          o << "  rr /= " << dims[d] << ";\n";
        }
        if (n >= 3) o << "  const " << it << " i1 = rr;\n";
      }
      o << "  const " << it << " lin0 = i0 * " << plane << (em.idx64 ? "LL" : "") << " + pe;\n";
    }
    if (inplace) {
      std::string outside;
      for (int d = 0; d < n; ++d) {
        const std::string v = "i" + std::to_string(d) + (d == n - 1 ? "b" : "");
        const int64_t lo = box[d].first, hi = box[d].first + box[d].second;
        outside += (d ? " || " : "") + (d == n - 1 ? v + " + " + std::to_string(vec) + " <= " + std::to_string(lo) : v + " < " + std::to_string(lo)) + " || " + v +
                   " >= " + std::to_string(hi);
      }
      o << "  if (" << outside << ") return;   // outside the box that changes: the buffer already holds the operand\n";
    }
    {
      // inputs read once, at the output's own position, stream through (non-temporal hint);
      // inputs read at several offsets stay cacheable
      std::map<int, int> nvec, nload;
      for (auto& sd : em.direct_vecs) nvec[sd.first]++;
      for (auto& l : em.loads) nload[em.slot_of(l.node)]++;
      for (auto& sd : em.direct_vecs) {
        const int slot = sd.first;
        const int64_t D = sd.second;
        const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
        const std::string vt = "rx_vec<" + st + ", " + std::to_string(vec) + ">";
        std::string addr = "lin0";
        if (D != 0) {
          // neighbours of elements on the boundary fall outside the array; their values are never
          // used (the pad / update-slice guard selects them away), so the address is clamped
          const std::string sfx = em.idx64 ? "LL" : "";
          addr = "rx_clamp_idx<" + it + ">(lin0 + " + std::to_string(D) + sfx + ", " + std::to_string(numel - vec) + sfx + ")";
        }
        const bool stream = opt.nt_loads && nvec[slot] == 1 && D == 0 && nload[slot] == 1;
        if (inplace && !update_reads_base && em.inputs[slot] == rn.in[0] && D == 0) {
          // the old values matter only where a vector sticks out of the box
          const std::string v = "i" + std::to_string(n - 1) + "b";
          o << "  const " << vt << " " << vec_name(slot, D) << " = (" << v << " < " << box[n - 1].first << " || " << v << " + " << vec << " > "
            << box[n - 1].first + box[n - 1].second << ") ? rx_load<" << vt << ">(in" << slot << " + lin0) : " << vt << "{};\n";
          continue;
        }
        o << "  const " << vt << " " << vec_name(slot, D) << " = " << (stream ? "rx_load_nt" : "rx_load") << "<" << vt << ">(in" << slot << " + " << addr
          << ");\n";
      }
    }
    const std::string ost = info(rn.ty.dt).stype;
    if (n == 0) {
      o << "  {\n" << body << "    out0[0] = " << em.store_value(rn.ty.dt, val) << ";\n  }\n";
    } else {
      o << "  rx_vec<" << ost << ", " << vec << "> res;\n";
      o << "#pragma unroll\n  for (int l = 0; l < " << vec << "; ++l) {\n";
      o << "    const " << it << " i" << n - 1 << " = i" << n - 1 << "b + l;\n";
      o << body;
      o << "    res.v[l] = " << em.store_value(rn.ty.dt, val) << ";\n  }\n";
      o << "  " << (opt.nt_stores ? "rx_store_nt" : "rx_store") << "(out0 + lin0, res);\n";
    }
    o << "}\n\n";
    std::string ktext = o.str();
    if (inplace) {
      // the operand and the result are the same memory
      for (size_t q; (q = ktext.find("* __restrict__ ")) != std::string::npos;) ktext.replace(q, 15, "* ");
      buf_of[root] = buffer_for(rn.in[0]);
    }
    const std::string kb_final = finalize(ktext);

    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = inplace ? "map_in_place" : slab ? "map_stencil" : "map";
    L.grid[0] = n == 0 ? 1 : grid;
    L.block[0] = kBlock;
    for (int i : em.inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    L.algo_bytes = algo_bytes(em.inputs, {root});
    if (inplace) {
      // the operand is not copied: its box is written (and read, if the update uses the old values)
      std::vector<int> others;
      bool reads_base = false;
      for (int i : em.inputs) { if (i == rn.in[0]) reads_base = true; else others.push_back(i); }
      (void)reads_base;   // unless the update uses them, old values are read only where a vector straddles the edge of the box
      double boxb = info(rn.ty.dt).size;
      for (auto& b : box) boxb *= (double)b.second;
      L.algo_bytes = algo_bytes(others, {}) + boxb * (update_reads_base ? 2 : 1);
    }
    L.desc = value >= 0 ? "copy of the scatter operand" : describe(root);
    plan.launches.push_back(L);
  }

  // ------------------------------------------------------------------ scatter
  // The result starts as a copy of the operand (a map kernel); then one thread per element of
  // `updates` finds its target -- the start index read from the index tensor at its scatter
  // position, plus its offset inside the update window -- skips it if the window leaves the
  // operand (the specification drops such updates, it does not clamp them), and stores or
  // combines.  Combining uses the hardware atomics (the order of colliding float additions is
  // not fixed); colliding assignments leave one of the values, as the specification allows.
  void emit_scatter(int root) {
    const Node& rn = g.nodes[root];
    const TType& ot = rn.ty;
    const TType& st = g.nodes[rn.in[1]].ty;
    const TType& ut = g.nodes[rn.in[2]].ty;
    emit_map(root, rn.in[0]);
    if (ut.numel() == 0 || ot.numel() == 0) return;
    const int r = ot.rank(), rs = st.rank(), ru = ut.rank();
    const int ivd = (int)rn.a4[0];
    auto has = [](const std::vector<int64_t>& v, int x) { return std::find(v.begin(), v.end(), (int64_t)x) != v.end(); };
    Emitter em(g, [&](int x) { return mat[x] != 0; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(rn.in[1])) || needs64(cone_nodes(rn.in[2])) || ot.numel() >= ((int64_t)1 << 31) || ut.numel() >= ((int64_t)1 << 31);
    const std::string it = em.idx_t();
    em.set_root({}, {}, false);
    em.indent = 2;
    Index ux(ru);
    for (int d = 0; d < ru; ++d) { ux[d].var = "u" + std::to_string(d); ux[d].hi = ut.dims[d] - 1; }
    // scatter position = update index without the window dims
    std::vector<Ix> spos;
    for (int d = 0; d < ru; ++d) if (!has(rn.a0, d)) spos.push_back(ux[d]);
    // window offset per operand dim
    std::vector<std::string> off(r, "0");
    {
      size_t j = 0;
      for (int d = 0; d < r; ++d) {
        if (has(rn.a1, d) || has(rn.a5, d)) continue;
        off[d] = ux[rn.a0[j++]].str();
      }
    }
    for (size_t b = 0; b < rn.a5.size(); ++b) {
      const int ds = (int)rn.a6[b];
      off[rn.a5[b]] = spos[ds - (ds < ivd ? 0 : 1)].str();
    }
    std::ostringstream body;
    std::vector<std::string> target(r);
    std::string guard;
    std::vector<std::string> start_code;
    for (int d = 0; d < r; ++d) target[d] = "(long long)(" + off[d] + ")";
    for (size_t k = 0; k < rn.a2.size(); ++k) {
      const int d = (int)rn.a2[k];
      Index si(rs);
      size_t bi = 0;
      for (int q = 0; q < rs; ++q) {
        if (q == ivd) { si[q].off = (int64_t)k; si[q].lo = si[q].hi = (int64_t)k; }
        else si[q] = spos[bi++];
      }
      const std::string e = em.emit(rn.in[1], si);
      target[d] = "((long long)(" + e + ") + (long long)(" + off[d] + "))";
    }
    const std::string val = em.emit(rn.in[2], ux);
    const std::string code = em.take_code();
    std::ostringstream o;
    const std::string ost = info(ot.dt).stype;
    o << "// scatter (" << rn.op << "): " << describe(rn.in[2]) << " -> " << ot.str() << "\n";
    o << signature("@K@_scatter", em.inputs, {{ost, "out0"}}) << " {\n";
    o << "  const " << it << " uid = (" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x;\n";
    o << "  if (uid >= " << ut.numel() << ") return;\n";
    o << "  " << it << " rr = uid;\n";
    for (int d = ru - 1; d >= 0; --d) {
      o << "  const " << it << " u" << d << " = rr % " << ut.dims[d] << ";\n";
      o << "  rr /= " << ut.dims[d] << ";\n";
    }
    o << "  (void)rr;\n" << code;
    std::string lin = "0";
    int64_t stride = 1;
    for (int d = r - 1; d >= 0; --d) {
      o << "  const long long t" << d << "_ = " << target[d] << ";\n";
      guard += (guard.empty() ? "" : " && ") + std::string("t") + std::to_string(d) + "_ >= 0 && t" + std::to_string(d) + "_ < " + std::to_string(ot.dims[d]) + "LL";
      lin += " + t" + std::to_string(d) + "_ * " + std::to_string(stride) + "LL";
      stride *= ot.dims[d];
    }
    // The whole update window must lie inside the operand, not just this element: test the window's corners.
    {
      std::string wguard;
      size_t j = 0;
      for (int d = 0; d < r; ++d) {
        if (has(rn.a1, d) || has(rn.a5, d)) continue;
        const int ud = (int)rn.a0[j++];
        // start of the window in dim d = target - own offset; the window spans ut.dims[ud] elements
        wguard += (wguard.empty() ? "" : " && ") + std::string("(t") + std::to_string(d) + "_ - (long long)u" + std::to_string(ud) + ") >= 0 && (t" +
                  std::to_string(d) + "_ - (long long)u" + std::to_string(ud) + ") + " + std::to_string(ut.dims[ud]) + "LL <= " + std::to_string(ot.dims[d]) + "LL";
      }
      if (!wguard.empty()) guard += " && " + wguard;
    }
    if (guard.empty()) guard = "true";
    o << "  if (" << guard << ") {\n";
    o << "    " << ost << "* p = out0 + (" << lin << ");\n";
    const std::string sv = em.store_value(ot.dt, val);
    if (rn.op == "assign") {
      o << "    *p = " << sv << ";\n";
    } else if (rn.op == "subtract") {
      o << "    rx_atomic_add(p, (" << ost << ")(-(" << sv << ")));\n";
    } else if (rn.op == "divide") {
      o << "    rx_atomic_div(p, " << sv << ");\n";
    } else {
      const char* fn = rn.red == Red::Add ? "rx_atomic_add" : rn.red == Red::Mul ? "rx_atomic_mul" : rn.red == Red::Max ? "rx_atomic_max"
                       : rn.red == Red::Min ? "rx_atomic_min" : rn.red == Red::And ? "rx_atomic_and" : "rx_atomic_or";
      o << "    " << fn << "(p, " << sv << ");\n";
    }
    o << "  }\n}\n\n";
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named("@K@_scatter", kb_final);
    L.kind = "scatter";
    L.grid[0] = (unsigned)((ut.numel() + kBlock - 1) / kBlock);
    L.block[0] = kBlock;
    for (int i : em.inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    L.algo_bytes = algo_bytes(em.inputs, {});
    L.desc = describe(rn.in[2]) + " scatter";
    plan.launches.push_back(L);
  }

  // ------------------------------------------------------------------ direct convolution
  // `root` is the convolution itself or the elementwise root that consumes it at the identity index (a bias, an
  // activation): that cone becomes the kernel's epilogue functor, as for a dot_general.
  void emit_conv(int root, int conv) {
    const Node& cn = g.nodes[conv];
    const Node& rn = g.nodes[root];
    const TType& xt = g.nodes[cn.in[0]].ty;
    const TType& wt = g.nodes[cn.in[1]].ty;
    const bool shifted = !cn.a3.empty();   // the product with row shifts (16-bit images)
    ConvChoice cc;
    if (!shifted) {
      cc = choose_conv(xt.dims[0], xt.dims[1], xt.dims[2], xt.dims[3], wt.dims[0], wt.dims[2], wt.dims[3], cn.ty.dims[2], cn.ty.dims[3], cn.a0[2],
                       cn.a1[0], cn.a1[1], cn.a2[0], cn.a2[1]);
      if (!cc.ok) throw Error("internal: convolution node without a tiling");
    }
    const int n = rn.ty.rank();
    if (shifted && cn.a3.size() == 8) {
      // The grid form zeroes the rows that are not results and moves the rows inside this kernel, after the
      // elementwise ops it has taken in.  That is only right when nothing elementwise is left to run
      // afterwards (it would turn the zeros into f(0)) and when every reader expects the moved rows.
      bool whole = !std::count(g.results.begin(), g.results.end(), root) && !users[root].empty();
      for (int u : users[root]) {
        const Node& un = g.nodes[u];
        whole = whole && un.k == OpK::Conv && !un.a3.empty() && un.in[0] == root && un.in[1] != root;
      }
      if (!whole) throw ChainNotAbsorbed();
    }
    Emitter em(g, [&](int x) { return mat[x] && x != root; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(root));
    const std::string it = em.idx_t();
    std::vector<std::string> vars;
    for (int k = 0; k < n; ++k) vars.push_back("i" + std::to_string(k));
    em.set_root(rn.ty.dims, vars, true);
    em.vec = 4;
    em.direct_expr = vec_name;
    em.indent = 6;
    em.bound[conv] = "accv";
    em.columns_reused = shifted;
    em.const_vectors = true;
    const std::string val = root == conv ? std::string("accv") : em.emit(root, root_index(rn.ty.dims));
    const std::string ebody = em.take_code();
    const std::string ost = info(rn.ty.dt).stype;
    // The compact form of the shifted product drops the rows that are not results.  When the epilogue reads per-feature
    // vectors only (bias, batch norm) the test guards the store alone: the arithmetic is then straight-line code over all
    // the rows a thread handles, and what depends on the column only (the vectors' loads and conversions, a square root,
    // a reciprocal) is computed once per column instead of once per row.
    // (Tensors of the result's own shape that are read at the result's position -- the other operand of a residual
    // addition -- may take part in the compact form: their vectors are read at a position clamped into the tensor.)
    bool vectors_only = shifted && !em.inputs.empty(), clamped_reads = false;
    for (auto& l : em.loads) {
      const Node& ln = g.nodes[l.node];
      bool ok = ln.ty.rank() == 0 || (ln.ty.rank() <= 1 && l.minor_follows);      // read at the column only: in range on every row
      if (!ok && cn.a3.size() == 5 && l.affine && ln.ty.dims == rn.ty.dims && std::all_of(l.off.begin(), l.off.end(), [](int64_t v) { return v == 0; })) ok = clamped_reads = true;
      vectors_only = vectors_only && ok;
    }
    for (auto& sd : em.direct_vecs) vectors_only = vectors_only && sd.second == 0;
    if (clamped_reads) for (int i : em.inputs) vectors_only = vectors_only && (g.nodes[i].ty.rank() <= 1 || g.nodes[i].ty.dims == rn.ty.dims);
    else for (int i : em.inputs) vectors_only = vectors_only && g.nodes[i].ty.rank() <= 1;
    const bool late_mask = vectors_only && cn.a3.size() == 5;
    // The direct kernel: a lane holds one feature for all its pixels.  An epilogue that reads nothing but per-feature
    // vectors (broadcast along the result's feature dimension) takes the kernel's bounds test as an argument and guards
    // its store with it, for the same reason.
    bool direct_mask = !shifted && !em.inputs.empty() && n == 4;
    for (int i : em.inputs) {
      const Node& in = g.nodes[i];
      direct_mask = direct_mask && in.ty.rank() <= 1;
      if (in.ty.rank() == 1)
        for (int u : users[i]) {
          const Node& un = g.nodes[u];
          direct_mask = direct_mask && un.k == OpK::BroadcastInDim && un.ty.rank() == 4 && un.a0 == std::vector<int64_t>{1} && in.ty.dims[0] == rn.ty.dims[1];
        }
    }
    // (the grid form computes every row anyway and guards its stores by the row number: it takes the rows past the last one too)
    const bool grid_all_rows = vectors_only && cn.a3.size() == 8;
    std::ostringstream o;
    o << "// convolution epilogue: " << describe(root) << "\n";
    o << "struct @K@_epi {\n";
    for (size_t k = 0; k < em.inputs.size(); ++k)
      o << "  const " << info(g.nodes[em.inputs[k]].ty.dt).stype << "* __restrict__ in" << k << ";\n";
    o << "  " << ost << "* __restrict__ out0;\n";
    if (late_mask || grid_all_rows || direct_mask) o << "  static constexpr bool masks_rows = true;\n";
    o << "  template <int NV>\n  __device__ __forceinline__ void operator()(const float (&acc)[NV]";
    if (shifted) {
      // called with (row of the product, first column): the row is a position of the padded grid, of which the
      // result keeps the first HO rows and WO columns of every image
      if (n != 4) throw Error("internal: shifted product with a result of another rank");
      o << ", " << it << " row_, " << it << " i3b) const {\n";
      o << "    const " << it << " i2 = row_ % " << cn.a3[4] << ", i1 = (row_ / " << cn.a3[4] << ") % " << cn.a3[3] << ", i0 = row_ / " << cn.a3[3] * cn.a3[4] << ";\n";
      if (cn.a3.size() == 8) {
        // the grid form (chain_convs): every row is written, the ones that are not results as zeros
        o << "    const bool result_ = i1 < " << cn.a3[5] << " && i2 < " << cn.a3[6] << ";\n";
      } else if (late_mask) {
        o << "    const bool keep_ = i0 < " << rn.ty.dims[0] << " && i1 < " << rn.ty.dims[1] << " && i2 < " << rn.ty.dims[2] << ";\n";
      } else {
        o << "    if (i1 >= " << rn.ty.dims[1] << " || i2 >= " << rn.ty.dims[2] << ") return;\n";
      }
    } else {
      for (int k = 0; k < n; ++k) o << ", " << it << " i" << k << (k == n - 1 ? "b" : "");
      if (direct_mask) o << ", const bool keep_";
      o << ") const {\n";
    }
    {
      Index rix = root_index(rn.ty.dims);
      rix[n - 1].var = "i" + std::to_string(n - 1) + "b";
      o << "    const " << it << " lin0 = " << em.linear(rix, rn.ty.dims) << ";\n";
    }
    if (late_mask && !em.direct_vecs.empty()) o << "    const " << it << " lin0c = rx_min<" << it << ">(lin0, " << rn.ty.numel() << " - NV);\n";
    for (auto& sd : em.direct_vecs) {
      const int slot = sd.first;
      const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
      o << "    const rx_vec<" << st << ", NV> d" << slot << " = *reinterpret_cast<const rx_vec<" << st << ", NV>*>(in" << slot << " + " << (late_mask ? "lin0c" : "lin0") << ");\n";
    }
    o << "    rx_vec<" << ost << ", NV> res;\n";
    o << "#pragma unroll\n    for (int l = 0; l < NV; ++l) {\n";
    o << "      const " << it << " i" << n - 1 << " = i" << n - 1 << "b + l;\n";
    o << "      const float accv = acc[l];\n";
    o << ebody;
    o << "      res.v[l] = " << em.store_value(rn.ty.dt, val) << ";\n    }\n";
    if (shifted && cn.a3.size() == 8) {
      // row m goes to row m + shift (the position of the same pixel in the next product's zero-padded operand); rows that
      // are not results carry zeros onto the borders; the rows before the shift are zeros too, written by the call for the
      // product row of the same number
      const int64_t rows = cn.ty.dims[0] * cn.a3[3] * cn.a3[4], ncol = cn.ty.dims[3];
      o << "    rx_vec<" << ost << ", NV> zero_;\n#pragma unroll\n    for (int l = 0; l < NV; ++l) zero_.v[l] = 0;\n";
      o << "    if (!result_) res = zero_;\n";
      if (grid_all_rows) o << "    rx_keep_value(res);\n";
      o << "    if (row_ + " << cn.a3[7] << " < " << rows << ") *reinterpret_cast<rx_vec<" << ost << ", NV>*>(out0 + lin0 + " << cn.a3[7] * ncol << ") = res;\n";
      if (cn.a3[7] > 0) o << "    if (row_ < " << cn.a3[7] << ") *reinterpret_cast<rx_vec<" << ost << ", NV>*>(out0 + lin0) = zero_;\n";
    } else {
      if (late_mask || direct_mask) o << "    rx_keep_value(res);\n";
      o << "    " << (late_mask || direct_mask ? "if (keep_) " : "") << "*reinterpret_cast<rx_vec<" << ost << ", NV>*>(out0 + lin0) = res;\n";
    }
    o << "  }\n};\n\n";
    if (shifted) {
      // [rows of the padded images, C] x [O, taps * C] -> [rows, O] on a streaming GEMM skeleton whose K tiles of the
      // first operand carry the tap's row shift (rx_tap_shift)
      const int64_t xrows = xt.numel() / xt.dims.back(), xcols = xt.dims.back();   // the first operand as a matrix (its leading dimensions are the rows)
      if (rn.ty.dims != cn.ty.dims || cn.ty.dims[0] * cn.a3[3] * cn.a3[4] != xrows) throw Error("internal: shifted product with a result of another shape");
      const GemmChoice gc = choose_gemm(xt.dt, wt.dt, cn.ty.dt, 1, xrows, wt.dims[0], wt.dims[1], true, true);
      const bool dl = gc.skeleton == "rx_gemm_body_dl";
      if (!gc.ok || (gc.skeleton != "rx_gemm_body_pp" && gc.skeleton != "rx_gemm_body_s" && !(dl && gc.bk * (int)info(xt.dt).size == 128 && gc.split == 1)))
        throw Error("internal: shifted product without a skeleton that loads tiles straight into LDS");
      o << "// convolution as a product with row shifts: " << xt.str() << " x " << wt.str() << " -> " << cn.ty.str() << ", window " << wt.dims[1] / xcols / cn.a3[0] << " x " << cn.a3[0]
        << ", row shifts " << cn.a3[1] << " / " << cn.a3[2] << "\n";
      o << "extern \"C\" __global__ __launch_bounds__(" << gc.block << ") void @K@_conv(const " << gc.stype_a << "* __restrict__ A, const " << gc.stype_a << "* __restrict__ B";
      for (size_t k = 0; k < em.inputs.size(); ++k) o << ", const " << info(g.nodes[em.inputs[k]].ty.dt).stype << "* __restrict__ e" << k;
      o << ", " << ost << "* __restrict__ out0) {\n";
      o << "  @K@_epi epi{";
      for (size_t k = 0; k < em.inputs.size(); ++k) o << "e" << k << ", ";
      o << "out0};\n";
      o << "  " << gc.skeleton << "<" << gc.targs << ", false, @K@_epi";
      if (gc.depth > 0) o << ", " << gc.depth;
      if (gc.stream_stages > 0) o << ", " << gc.stream_stages;
      o << (dl ? ", 1" : ", rx_no_fn") << ", rx_tap_shift<" << xcols << ", " << cn.a3[0] << ", " << cn.a3[1] << ", " << cn.a3[2] << ", " << info(xt.dt).size << ">>(A, B, epi);\n}\n\n";
      const std::string kb = finalize(o.str());
      Launch L;
      L.kernel = named("@K@_conv", kb);
      L.kind = "conv_" + gc.kind.substr(5);   // conv_bf16, conv_f16
      L.grid[0] = gc.grid[0]; L.grid[1] = gc.grid[1]; L.grid[2] = gc.grid[2];
      L.block[0] = gc.block;
      L.lds_bytes = gc.lds_bytes;
      L.args.push_back(buffer_for(cn.in[0]));
      L.args.push_back(buffer_for(cn.in[1]));
      for (int i : em.inputs) L.args.push_back(buffer_for(i));
      L.args.push_back(buffer_for(root));
      std::vector<int> all_in{cn.in[0], cn.in[1]};
      for (int i : em.inputs) if (std::find(all_in.begin(), all_in.end(), i) == all_in.end()) all_in.push_back(i);
      L.algo_bytes = algo_bytes(all_in, {root});
      // of the results that are kept
      L.flops = 2.0 * (double)(cn.a3.size() == 8 ? cn.ty.dims[0] * cn.a3[5] * cn.a3[6] * cn.ty.dims[3] : cn.ty.numel()) * (double)wt.dims[1];
      L.desc = describe(root);
      plan.launches.push_back(L);
      return;
    }
    o << "// direct convolution: " << xt.str() << " * " << wt.str() << " -> " << cn.ty.str() << ", " << cc.rows << " rows of the result per workgroup, channels in slabs of " << cc.slab << "\n";
    o << "extern \"C\" __global__ __launch_bounds__(256) void @K@_conv(const float* __restrict__ X, const float* __restrict__ Wt";
    for (size_t k = 0; k < em.inputs.size(); ++k) o << ", const " << info(g.nodes[em.inputs[k]].ty.dt).stype << "* __restrict__ e" << k;
    o << ", " << ost << "* __restrict__ out0) {\n";
    o << "  @K@_epi epi{";
    for (size_t k = 0; k < em.inputs.size(); ++k) o << "e" << k << ", ";
    o << "out0};\n";
    o << "  rx_conv_body<" << xt.dims[0] << ", " << xt.dims[1] << ", " << xt.dims[2] << ", " << xt.dims[3] << ", " << wt.dims[0] << ", " << wt.dims[2] << ", " << wt.dims[3] << ", "
      << cn.a1[0] << ", " << cn.a1[1] << ", " << cn.a2[0] << ", " << cn.a2[1] << ", " << cn.a0[0] << ", " << cn.a0[2] << ", " << cn.ty.dims[2] << ", " << cn.ty.dims[3] << ", " << cc.rows << ", " << cc.slab << ", @K@_epi>(X, Wt, epi);\n}\n\n";
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named("@K@_conv", kb_final);
    L.kind = "conv";
    L.grid[0] = cc.grid[0];
    L.grid[1] = cc.grid[1];
    L.block[0] = 256;
    L.lds_bytes = cc.lds_bytes;
    L.args.push_back(buffer_for(cn.in[0]));
    L.args.push_back(buffer_for(cn.in[1]));
    for (int i : em.inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    std::vector<int> all_in{cn.in[0], cn.in[1]};
    for (int i : em.inputs) if (std::find(all_in.begin(), all_in.end(), i) == all_in.end()) all_in.push_back(i);
    L.algo_bytes = algo_bytes(all_in, {root});
    L.flops = 2.0 * (double)cn.ty.numel() * (double)(wt.dims[1] * wt.dims[2] * wt.dims[3]);
    L.desc = describe(root);
    plan.launches.push_back(L);
  }

  // ------------------------------------------------------------------ reductions
  struct RedShape {
    bool trailing = false;   // reduced dims are exactly the trailing dims
    int64_t rows = 1, cols = 1;
    int nkeep = 0;
  };
  RedShape red_shape(const Node& r) const {
    const TType& in = g.nodes[r.in[0]].ty;
    RedShape s;
    std::vector<int64_t> dd = r.a0;
    std::sort(dd.begin(), dd.end());
    s.nkeep = in.rank() - (int)dd.size();
    s.trailing = true;
    for (size_t k = 0; k < dd.size(); ++k) s.trailing = s.trailing && dd[k] == s.nkeep + (int)k;
    for (int d = 0; d < in.rank(); ++d) (d < s.nkeep ? s.rows : s.cols) *= in.dims[d];
    return s;
  }

  // full reduction (all dims): two kernels
  void emit_reduce_full(int root) {
    const Node& rn = g.nodes[root];
    const Node& inn = g.nodes[rn.in[0]];
    const auto& dims = inn.ty.dims;
    const int n = inn.ty.rank();
    const DT dt = rn.ty.dt;
    const std::string ACC = acc_ctype(dt);
    const int vec = pick_vec(inn.ty);
    const int64_t nv = inn.ty.numel() / vec;
    const int U = 4;
    int64_t tiles = (nv + (int64_t)kBlock * U - 1) / ((int64_t)kBlock * U);
    const int G = (int)std::max<int64_t>(1, std::min<int64_t>(tiles, 2048));
    const std::string k1 = "@K@_reduce", k2 = "@K@_reduce_final";

    Emitter em(g, [&](int x) { return mat[x]; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(rn.in[0]));
    const std::string it = em.idx_t();
    std::vector<std::string> vars;
    for (int d = 0; d < n; ++d) vars.push_back("i" + std::to_string(d));
    em.set_root(dims, vars, vec > 1);
    em.vec = vec;
    em.direct_expr = vec_name;
    em.indent = 10;
    std::string val = em.emit(rn.in[0], root_index(dims));
    std::string body = em.take_code();

    std::ostringstream o;
    o << "// reduce (pass 1): " << describe(rn.in[0]) << " -> partials\n";
    o << signature(k1, em.inputs, {{ACC, "partial"}}) << " {\n";
    o << "  " << ACC << " acc[" << U << "];\n";
    o << "#pragma unroll\n  for (int u = 0; u < " << U << "; ++u) acc[u] = " << red_identity(rn.red, dt) << ";\n";
    o << "  for (" << it << " base = (" << it << ")blockIdx.x * " << kBlock * U << "; base < " << nv << "; base += (" << it << ")gridDim.x * " << kBlock * U
      << ") {\n";
    o << "#pragma unroll\n    for (int u = 0; u < " << U << "; ++u) {\n";
    o << "      const " << it << " vid = base + u * " << kBlock << " + threadIdx.x;\n";
    o << "      if (vid < " << nv << ") {\n";
    decode_index(o, it, "vid", dims, vec, "        ");
    o << "        const " << it << " lin0 = vid * " << vec << ";\n";
    for (auto& sd : em.direct_vecs) {
      const int slot = sd.first;
      const std::string vt = "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vec) + ">";
      o << "        const " << vt << " " << vec_name(slot, 0) << " = " << (opt.nt_loads ? "rx_load_nt" : "rx_load") << "<" << vt << ">(in" << slot
        << " + lin0);\n";
    }
    o << "#pragma unroll\n        for (int l = 0; l < " << vec << "; ++l) {\n";
    if (n > 0) o << "          const " << it << " i" << n - 1 << " = i" << n - 1 << "b + l;\n";
    o << body;
    o << "          acc[u] = " << red_apply(rn.red, dt, "acc[u]", "(" + ACC + ")" + val) << ";\n";
    o << "        }\n      }\n    }\n  }\n";
    o << "  " << ACC << " a = acc[0];\n";
    o << "#pragma unroll\n  for (int u = 1; u < " << U << "; ++u) a = " << red_apply(rn.red, dt, "a", "acc[u]") << ";\n";
    o << "  __shared__ " << ACC << " lds[" << kBlock / 64 << "];\n";
    o << "  a = rx_block_reduce<" << ACC << ", decltype(" << red_functor(rn.red) << "), " << kBlock / 64 << ">(a, " << red_functor(rn.red) << ", lds);\n";
    // the init value and the final store, evaluated by one thread
    Emitter e2(g, [&](int x) { return mat[x]; });
    e2.excess_precision = opt.excess_precision;
    e2.indent = 4;
    std::string initv = e2.emit(rn.in[1], Index{});
    std::string ibody = e2.take_code();
    std::vector<int> in2 = e2.inputs;
    std::string rv = is_narrow_float(dt) ? Emitter::round_narrow(dt, "r") : std::string("(") + info(dt).ctype + ")r";
    auto combine = [&](std::ostringstream& oo, const std::string& src) {
      // partials are combined in index order by a fixed tree: the result does not depend on
      // which workgroup finished last
      oo << "  " << ACC << " c = " << red_identity(rn.red, dt) << ";\n";
      oo << "  for (int i = threadIdx.x; i < " << G << "; i += " << kBlock << ") c = " << red_apply(rn.red, dt, "c", src + "[i]") << ";\n";
      oo << "  c = rx_block_reduce<" << ACC << ", decltype(" << red_functor(rn.red) << "), " << kBlock / 64 << ">(c, " << red_functor(rn.red) << ", lds);\n";
      oo << "  if (threadIdx.x == 0) {\n" << ibody;
      oo << "    const " << ACC << " r = " << red_apply(rn.red, dt, "c", "(" + ACC + ")" + initv) << ";\n";
      oo << "    out0[0] = " << Emitter::store_conv(dt, rv) << ";\n";
    };
    const bool single = opt.single_pass_reduce && G > 1;
    const int NW = (dt == DT::F64 || info(dt).size == 8) ? 2 : 1;   // 32-bit words of one partial
    if (single) {
      // One launch.  Every workgroup publishes its partial as self-validating 64-bit words -- 32 bits of the value
      // under a flag, written by one relaxed device-scope atomic store each, so no fence (an L2 write-back on this
      // multi-die part) is needed to order value and flag.  The workgroup with the last index then waits for every
      // slot, clears it for the next run, and combines the partials in index order by the same fixed tree as the
      // two-launch form: the result is bit-identical to it and does not depend on timing.  The slots live in a
      // buffer that is zero when the executable is loaded.  The wait is bounded: a slot that never arrives (which
      // no correct run produces) ends it after about a second with whatever the slot holds.
      std::string sig = signature(k1, em.inputs, {{ACC, "partial"}});
      sig.pop_back();
      sig += ", unsigned long long* __restrict__ slots";
      for (size_t k = 0; k < in2.size(); ++k) sig += ", " + ptr_decl(info(g.nodes[in2[k]].ty.dt).stype, true, "fin" + std::to_string(k));
      sig += ", " + ptr_decl(info(dt).stype, false, "out0") + ")";
      // the pass-1 text was written against `signature(k1, ...)`; swap the header
      std::string text = o.str();
      const std::string old_sig = signature(k1, em.inputs, {{ACC, "partial"}});
      const size_t at = text.find(old_sig);
      text.replace(at, old_sig.size(), sig);
      o.str("");
      o << text;
      o << "  if (threadIdx.x == 0) rx_publish_partial<" << ACC << ">(slots + (size_t)blockIdx.x * " << NW << ", a);\n";
      o << "  if (blockIdx.x != gridDim.x - 1u) return;\n";
      // the combining workgroup keeps what it collected in the partials buffer: it reads that buffer alone
      o << "  " << ACC << "* all = partial;\n";
      o << "  for (int i = threadIdx.x; i < " << G << "; i += " << kBlock << ") all[i] = rx_await_partial<" << ACC << ">(slots + (size_t)i * " << NW << ");\n";
      // the init-value operands were numbered for a kernel of their own
      std::ostringstream oc;
      combine(oc, "all");
      std::string ctext = oc.str();
      for (size_t k = in2.size(); k-- > 0;) {
        const std::string from = "in" + std::to_string(k) + "[", to = "fin" + std::to_string(k) + "[";
        for (size_t p = ctext.find(from); p != std::string::npos; p = ctext.find(from, p + to.size())) {
          if (p > 0 && (isalnum((unsigned char)ctext[p - 1]) || ctext[p - 1] == '_')) continue;
          ctext.replace(p, from.size(), to);
        }
      }
      o << ctext;
      o << "  }\n}\n\n";
    } else {
      o << "  if (threadIdx.x == 0) partial[blockIdx.x] = a;\n";
      o << "}\n\n";
      o << "// reduce (pass 2): combine " << G << " partials, apply init -> " << rn.ty.str() << "\n";
      {
        std::string s2 = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void " + k2 + "(const " + ACC + "* __restrict__ partial";
        for (size_t k = 0; k < in2.size(); ++k) s2 += ", " + ptr_decl(info(g.nodes[in2[k]].ty.dt).stype, true, "in" + std::to_string(k));
        s2 += ", " + ptr_decl(info(dt).stype, false, "out0") + ")";
        o << s2 << " {\n";
      }
      o << "  __shared__ " << ACC << " lds[" << kBlock / 64 << "];\n";
      combine(o, "partial");
      o << "  }\n}\n\n";
    }
    const std::string kb_final = finalize(o.str());

    int sc = scratch((int64_t)G * (dt == DT::F64 || info(dt).size == 8 ? 8 : 4));
    Launch L1;
    L1.kernel = named(k1, kb_final);
    L1.kind = "reduce";
    L1.grid[0] = G;
    L1.block[0] = kBlock;
    for (int i : em.inputs) L1.args.push_back(buffer_for(i));
    L1.args.push_back(sc);
    L1.algo_bytes = algo_bytes(em.inputs, {}) + info(dt).size;
    L1.desc = describe(rn.in[0]) + " reduce";
    if (single) {
      BufferDesc cb;
      cb.kind = BufferDesc::Const;          // lives with the executable; zero when loaded
      cb.ty.dt = DT::U64;
      cb.ty.dims = {(int64_t)G * NW};
      cb.bytes = (int64_t)G * NW * 8;
      cb.data.assign((size_t)cb.bytes, 0);
      plan.buffers.push_back(cb);
      L1.args.push_back((int)plan.buffers.size() - 1);
      for (int i : in2) L1.args.push_back(buffer_for(i));
      L1.args.push_back(buffer_for(root));
      plan.launches.push_back(L1);
      return;
    }
    plan.launches.push_back(L1);
    Launch L2;
    L2.kernel = named(k2, kb_final);
    L2.kind = "reduce_final";
    L2.grid[0] = 1;
    L2.block[0] = kBlock;
    L2.args.push_back(sc);
    for (int i : in2) L2.args.push_back(buffer_for(i));
    L2.args.push_back(buffer_for(root));
    L2.desc = "combine partials";
    plan.launches.push_back(L2);
  }

  // generic reduction: one thread per output element, sequential loops over reduced dims
  void emit_reduce_generic(int root) {
    const Node& rn = g.nodes[root];
    const Node& inn = g.nodes[rn.in[0]];
    const DT dt = rn.ty.dt;
    const std::string ACC = acc_ctype(dt);
    const int64_t nout = rn.ty.numel();
    const std::string kname = "@K@_reduce_generic";
    Emitter em(g, [&](int x) { return mat[x]; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(rn.in[0]));
    const std::string it = em.idx_t();
    em.set_root({}, {}, false);
    std::vector<int> kept, red;
    for (int d = 0; d < inn.ty.rank(); ++d)
      (std::find(rn.a0.begin(), rn.a0.end(), d) == rn.a0.end() ? kept : red).push_back(d);
    Index ix(inn.ty.rank());
    for (size_t k = 0; k < kept.size(); ++k) { ix[kept[k]].var = "o" + std::to_string(k); ix[kept[k]].hi = inn.ty.dims[kept[k]] - 1; }
    for (size_t k = 0; k < red.size(); ++k) { ix[red[k]].var = "r" + std::to_string(k); ix[red[k]].hi = inn.ty.dims[red[k]] - 1; }
    em.indent = 4 + 2 * (int)red.size();
    // 16-bit elements whose minor dimension is kept (eight outputs per thread, below): padded reads at clamped
    // positions and a select, so that the eight loads of a window element stay one 16-byte load
    em.clamp_guards = opt.clamp_pad_reads && opt.window_reduce_vectors && info(inn.ty.dt).size == 2 && !kept.empty() && kept.back() == inn.ty.rank() - 1;
    std::string val = em.emit(rn.in[0], ix);
    std::string body = em.take_code();
    em.indent = 2;
    std::string initv = em.emit(rn.in[1], Index{});
    std::string ibody = em.take_code();
    // Few outputs and a long reduction: one thread per output would leave most of the chip idle
    // (a column sum of an 8192 x 8192 matrix has 8192 outputs).  The largest reduced dimension is
    // then cut into `split` chunks (blockIdx.y); each chunk writes a partial per output and a
    // second small kernel combines the partials in chunk order and applies the init value.
    int64_t red_len = 1;
    size_t ks = 0;
    for (size_t k = 0; k < red.size(); ++k) {
      red_len *= inn.ty.dims[red[k]];
      if (inn.ty.dims[red[k]] > inn.ty.dims[red[ks]]) ks = k;
    }
    // When the input's minor dimension is kept, a thread owns VEC consecutive outputs, so that its VEC loads of a row
    // are one 16-byte access (the per-output order of the sum does not change); the chunk loop is unrolled to keep
    // eight such loads in flight (column sum of an 8192 x 8192 f32 matrix: 4.1 -> 6.3 TB/s).
    int VEC = 1;
    // 16-bit elements take it for short reductions too (pooling windows: eight outputs per thread, 16-byte loads where the
    // window view's minor dimension is the operand's).
    const int esz = info(inn.ty.dt).size;
    if (!kept.empty() && !red.empty() && kept.back() == inn.ty.rank() - 1 && (esz == 2 || esz == 4 || esz == 8) && info(dt).size == esz) {
      const int v = 16 / esz;
      // (not when the reads are transposed or gathered: eight outputs along the minor dimension would be eight strides apart)
      bool short_ok = esz == 2 && opt.window_reduce_vectors && red_len >= 2;
      if (short_ok)
        for (int x : cone_nodes(rn.in[0])) {
          const OpK k = g.nodes[x].k;
          if (x != rn.in[0] && mat[x]) continue;
          if (is_index_op(k) && k != OpK::Window && k != OpK::BroadcastInDim && k != OpK::Pad) short_ok = false;
        }
      const bool long_enough = esz == 2 ? short_ok : red_len >= 16;
      if (inn.ty.dims[kept.back()] % v == 0 && nout / v >= 64 && long_enough) VEC = v;
    }
    // A kept minor dimension that one vector covers (the few rows of a skinny matrix product, written as a reduction
    // over k of x[b][k] * w[k][n] with the result as [n][b]): a thread then takes RB consecutive values of the
    // next kept dimension as well, an RB x VEC block of the result.  What varies along that dimension only (w) is then
    // read RB elements at a time, one 16-byte load instead of four 4-byte ones, and what does not (x) once for the block.
    int RB = 1, wnode = -1;
    Emitter emr(g, [&](int x) { return mat[x]; });
    std::string wbody, wval;
    if (opt.reduce_row_blocks && VEC > 1 && esz == 4 && kept.size() >= 2 && red.size() == 1 && inn.ty.dims[kept.back()] == VEC &&
        inn.ty.dims[kept[kept.size() - 2]] % 4 == 0 && red_len >= 256 && nout / VEC / 4 >= 256 && !mat[rn.in[0]] && inn.k == OpK::Binary && inn.op == "multiply") {
      for (int side = 0; side < 2; ++side)
        if (em.minor_uniform(inn.in[side]) && !em.minor_uniform(inn.in[1 - side]) && g.nodes[inn.in[side]].ty.dims == inn.ty.dims) wnode = inn.in[side];
      if (wnode >= 0) {
        // the kernel's text again, in two parts: the operand that the block shares (for eight reduction steps ahead of
        // the arithmetic, so that eight 16-byte loads are in flight), then the rest with that operand's value in scope
        RB = 4;
        emr.excess_precision = opt.excess_precision;
        emr.idx64 = em.idx64;
        emr.set_root({}, {}, false);
        emr.indent = 8;
        emr.push_scope();
        wval = emr.emit(wnode, ix);
        wbody = emr.take_code();
        emr.pop_scope();
        emr.bound[wnode] = "wq_";
        emr.indent = 10;
        val = emr.emit(rn.in[0], ix);
        body = emr.take_code();
        emr.indent = 2;
        initv = emr.emit(rn.in[1], Index{});
        ibody = emr.take_code();
      }
    }
    Emitter& eu = RB > 1 ? emr : em;     // the emitter whose inputs the kernel takes
    const int64_t nthr = nout / VEC / RB;
    int64_t split = 1;
    if (!red.empty() && nout > 0 && nthr <= 32 * 1024 && red_len >= 64) {
      const int64_t ds = inn.ty.dims[red[ks]];
      // (threads of a block carry many times the bytes in flight: a quarter of the threads suffices, and the partials stay small; twice the threads, or sixteen steps per block, measured slower)
      split = std::min<int64_t>({ds, ((RB > 1 ? 128 : 512) * 1024 + nthr - 1) / nthr, 1024, std::max<int64_t>(1, red_len / 16)});
    }
    const bool two_pass = split >= 2;
    const int64_t chunk = two_pass ? (inn.ty.dims[red[ks]] + split - 1) / split : 0;
    if (two_pass) split = (inn.ty.dims[red[ks]] + chunk - 1) / chunk;
    std::ostringstream o;
    o << "// reduce (generic" << (two_pass ? ", reduced dimension cut into " + std::to_string(split) + " chunks" : std::string()) << "): " << describe(rn.in[0])
      << " over dims -> " << rn.ty.str() << "\n";
    o << signature(kname, eu.inputs, {{two_pass ? ACC : std::string(info(dt).stype), two_pass ? "partial" : "out0"}}) << " {\n";
    if (VEC > 1) o << "  const " << it << " oid = ((" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x) * " << VEC * RB << ";\n";
    else o << "  const " << it << " oid = (" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x;\n";
    o << "  if (oid >= " << nout << ") return;\n";
    o << "  " << it << " rr = oid;\n";
    for (int k = (int)kept.size() - 1; k >= 0; --k) {
      o << "  const " << it << " o" << k << ((VEC > 1 && k == (int)kept.size() - 1) || (RB > 1 && k == (int)kept.size() - 2) ? "b" : "") << " = rr % " << inn.ty.dims[kept[k]] << ";\n";
      o << "  rr /= " << inn.ty.dims[kept[k]] << ";\n";
    }
    if (VEC > 1) {
      o << "  " << ACC << " accv[" << VEC * RB << "];\n#pragma unroll\n  for (int l = 0; l < " << VEC * RB << "; ++l) accv[l] = " << red_identity(rn.red, dt) << ";\n";
    } else {
      o << "  " << ACC << " acc = " << red_identity(rn.red, dt) << ";\n";
    }
    if (RB > 1) {
      // one reduced dimension: blocks of eight steps, the shared operand's values of a block first
      const std::string wct = info(g.nodes[wnode].ty.dt).ctype;
      const std::string ok2 = "o" + std::to_string(kept.size() - 2), ok1 = "o" + std::to_string(kept.size() - 1);
      if (two_pass) {
        o << "  const " << it << " r0_end = rx_min<" << it << ">(((" << it << ")blockIdx.y + 1) * " << chunk << ", " << inn.ty.dims[red[0]] << ");\n";
        o << "  " << it << " r0s = (" << it << ")blockIdx.y * " << chunk << ";\n";
      } else {
        o << "  const " << it << " r0_end = " << inn.ty.dims[red[0]] << ";\n  " << it << " r0s = 0;\n";
      }
      auto steps = [&](int U) {
        o << "    " << wct << " wq[" << U * RB << "];\n";
        o << "#pragma unroll\n    for (int u = 0; u < " << U << "; ++u) {\n      const " << it << " r0 = r0s + u;\n";
        o << "#pragma unroll\n      for (int j = 0; j < " << RB << "; ++j) {\n        const " << it << " " << ok2 << " = " << ok2 << "b + j, " << ok1 << " = " << ok1 << "b;\n";
        o << wbody << "        wq[u * " << RB << " + j] = " << wval << ";\n      }\n    }\n";
        o << "#pragma unroll\n    for (int u = 0; u < " << U << "; ++u) {\n      const " << it << " r0 = r0s + u;\n";
        o << "#pragma unroll\n      for (int j = 0; j < " << RB << "; ++j) {\n        const " << it << " " << ok2 << " = " << ok2 << "b + j;\n        const " << wct << " wq_ = wq[u * " << RB << " + j];\n";
        o << "#pragma unroll\n        for (int l = 0; l < " << VEC << "; ++l) {\n          const " << it << " " << ok1 << " = " << ok1 << "b + l;\n";
        o << body;
        const std::string slot = "accv[j * " + std::to_string(VEC) + " + l]";
        o << "          " << slot << " = " << red_apply(rn.red, dt, slot, "(" + ACC + ")" + val) << ";\n        }\n      }\n    }\n";
      };
      o << "  for (; r0s + 8 <= r0_end; r0s += 8) {\n";
      steps(8);
      o << "  }\n  for (; r0s < r0_end; ++r0s) {\n";
      steps(1);
      o << "  }\n";
    }
    for (size_t k = 0; k < red.size() && RB == 1; ++k) {
      const std::string pad(2 + 2 * k, ' ');
      const std::string unroll = VEC > 1 && k + 1 == red.size() ? "#pragma unroll 8\n" : "";
      if (two_pass && k == ks) {
        o << pad << "const " << it << " r" << k << "_end = rx_min<" << it << ">(((" << it << ")blockIdx.y + 1) * " << chunk << ", " << inn.ty.dims[red[k]] << ");\n";
        o << unroll << pad << "for (" << it << " r" << k << " = (" << it << ")blockIdx.y * " << chunk << "; r" << k << " < r" << k << "_end; ++r" << k << ") {\n";
      } else {
        o << unroll << pad << "for (" << it << " r" << k << " = 0; r" << k << " < " << inn.ty.dims[red[k]] << "; ++r" << k << ") {\n";
      }
    }
    if (RB > 1) {
    } else if (VEC > 1) {
      const std::string pad(2 + 2 * red.size(), ' ');
      o << "#pragma unroll\n" << pad << "for (int l = 0; l < " << VEC << "; ++l) {\n";
      o << pad << "  const " << it << " o" << kept.size() - 1 << " = o" << kept.size() - 1 << "b + l;\n";
      o << body;
      o << pad << "  accv[l] = " << red_apply(rn.red, dt, "accv[l]", "(" + ACC + ")" + val) << ";\n";
      o << pad << "}\n";
    } else {
      o << body;
      o << std::string(4 + 2 * red.size(), ' ') << "acc = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + val) << ";\n";
    }
    for (int k = (int)red.size() - 1; k >= 0 && RB == 1; --k) o << std::string(2 + 2 * k, ' ') << "}\n";
    std::string rv = is_narrow_float(dt) ? Emitter::round_narrow(dt, "r") : std::string("(") + info(dt).ctype + ")r";
    std::vector<int> fin_inputs;
    int comb_lanes = 1;      // wavefronts of the combine kernel that share an output
    if (!two_pass) {
      o << ibody;
      if (VEC > 1) {
        o << "#pragma unroll\n  for (int l = 0; l < " << VEC * RB << "; ++l) {\n";
        o << "    const " << ACC << " r = " << red_apply(rn.red, dt, "accv[l]", "(" + ACC + ")" + initv) << ";\n";
        o << "    out0[oid + l] = " << Emitter::store_conv(dt, rv) << ";\n  }\n}\n\n";
      } else {
        o << "  const " << ACC << " r = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + initv) << ";\n";
        o << "  out0[oid] = " << Emitter::store_conv(dt, rv) << ";\n}\n\n";
      }
    } else {
      if (VEC > 1) o << "#pragma unroll\n  for (int l = 0; l < " << VEC * RB << "; ++l) partial[(" << it << ")blockIdx.y * " << nout << " + oid + l] = accv[l];\n}\n\n";
      else o << "  partial[(" << it << ")blockIdx.y * " << nout << " + oid] = acc;\n}\n\n";
      // the init value may read buffers of its own: evaluate it with a fresh numbering
      Emitter e3(g, [&](int x) { return mat[x]; });
      e3.excess_precision = opt.excess_precision;
      e3.indent = 2;
      std::string initv2 = e3.emit(rn.in[1], Index{});
      std::string ibody2 = e3.take_code();
      fin_inputs = e3.inputs;
      o << "// reduce (generic): combine " << split << " partials per output, apply init -> " << rn.ty.str() << "\n";
      std::string sg = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void @K@_reduce_combine(const " + ACC + "* __restrict__ partial";
      for (size_t k = 0; k < fin_inputs.size(); ++k) sg += ", " + ptr_decl(info(g.nodes[fin_inputs[k]].ty.dt).stype, true, "in" + std::to_string(k));
      sg += ", " + ptr_decl(info(dt).stype, false, "out0") + ")";
      o << sg << " {\n";
      // Many partials per output: the wavefronts of a workgroup share 64 outputs, wavefront w adds partials w, w + W,
      // ... (loads of 64 consecutive outputs), and the first one adds the W sums in order -- a fixed order, and W
      // times the workgroups of one thread per output, whose loop of dependent loads ran on 32 compute units for
      // 8192 outputs (column sums of 8192^2: combine 7.8 -> 3 us).
      comb_lanes = split >= 16 ? kBlock / 64 : 1;
      if (comb_lanes > 1) {
        o << "  __shared__ " << ACC << " part[" << kBlock << "];\n";
        o << "  const int oid = (int)blockIdx.x * 64 + (threadIdx.x & 63), w = threadIdx.x >> 6;\n";
        o << "  " << ACC << " acc = " << red_identity(rn.red, dt) << ";\n";
        o << "  if (oid < " << nout << ")\n#pragma unroll 8\n    for (int s = w; s < " << split << "; s += " << comb_lanes << ") acc = "
          << red_apply(rn.red, dt, "acc", "partial[s * " + std::to_string(nout) + " + oid]") << ";\n";
        o << "  part[threadIdx.x] = acc;\n  __syncthreads();\n";
        o << "  if (w != 0 || oid >= " << nout << ") return;\n";
        o << "#pragma unroll\n  for (int i = 1; i < " << comb_lanes << "; ++i) acc = " << red_apply(rn.red, dt, "acc", "part[i * 64 + threadIdx.x]") << ";\n";
      } else {
        o << "  const int oid = (int)blockIdx.x * " << kBlock << " + threadIdx.x;\n";
        o << "  if (oid >= " << nout << ") return;\n";
        o << "  " << ACC << " acc = " << red_identity(rn.red, dt) << ";\n";
        o << "  for (int s = 0; s < " << split << "; ++s) acc = " << red_apply(rn.red, dt, "acc", "partial[s * " + std::to_string(nout) + " + oid]") << ";\n";
      }
      o << ibody2;
      o << "  const " << ACC << " r = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + initv2) << ";\n";
      o << "  out0[oid] = " << Emitter::store_conv(dt, rv) << ";\n}\n\n";
    }
    const std::string kb_final = finalize(o.str());
    Launch L;
    L.kernel = named(kname, kb_final);
    L.kind = "reduce_generic";
    L.grid[0] = (unsigned)((nthr + kBlock - 1) / kBlock);
    L.grid[1] = (unsigned)(two_pass ? split : 1);
    L.block[0] = kBlock;
    for (int i : eu.inputs) L.args.push_back(buffer_for(i));
    L.algo_bytes = algo_bytes(eu.inputs, {root});
    L.desc = describe(rn.in[0]) + " reduce";
    if (!two_pass) {
      L.args.push_back(buffer_for(root));
      plan.launches.push_back(L);
      return;
    }
    const int sc = scratch(split * nout * (dt == DT::F64 || info(dt).size == 8 ? 8 : 4));
    L.args.push_back(sc);
    plan.launches.push_back(L);
    Launch L2;
    L2.kernel = named("@K@_reduce_combine", kb_final);
    L2.kind = "reduce_final";
    L2.grid[0] = (unsigned)(comb_lanes > 1 ? (nout + 63) / 64 : (nout + kBlock - 1) / kBlock);
    L2.block[0] = kBlock;
    L2.args.push_back(sc);
    for (int i : fin_inputs) L2.args.push_back(buffer_for(i));
    L2.args.push_back(buffer_for(root));
    L2.desc = "combine partials";
    plan.launches.push_back(L2);
  }

  // ------------------------------------------------------------------ prefix scans
  // Inclusive prefix combine along one dimension (what cumsum / cumprod / cummax arrive as).  The
  // scanned dimension is cut into chunks; a first kernel reduces every chunk, the scan kernel
  // starts each chunk from the combination of the chunk totals before it.  Along the minor
  // dimension a workgroup scans a chunk in tiles of 1024 elements (4 per lane, wavefront scan,
  // wavefront totals through LDS); along any other dimension a thread walks its chunk and the
  // lanes lie along the minor dimension, so both forms read and write coalesced.
  void emit_scan(int root) {
    const Node& rn = g.nodes[root];
    const TType& ty = rn.ty;
    const DT dt = ty.dt;
    const int a = (int)rn.a0[0];
    const bool rev = rn.a1[0] != 0;
    const std::string ACC = acc_ctype(dt);
    const std::string OP = red_functor(rn.red);
    const std::string IDENT = red_identity(rn.red, dt);
    const int64_t n = ty.dims[a];
    int64_t outer = 1, inner = 1;
    for (int d = 0; d < a; ++d) outer *= ty.dims[d];
    for (int d = a + 1; d < ty.rank(); ++d) inner *= ty.dims[d];
    // short rows are walked by one thread each (a row is a few cache lines, all of them used)
    const bool rowwise = inner == 1 && n >= 256 && outer * ((n + 4095) / 4096) < ((int64_t)1 << 31);
    Emitter em(g, [&](int x) { return mat[x]; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(rn.in[0])) || ty.numel() >= ((int64_t)1 << 31);
    const std::string it = em.idx_t();
    // forward scans along the minor dimension whose rows are whole vectors read and write 16 bytes per lane
    const int vecw = (rowwise && !rev && a == ty.rank() - 1 && pick_vec(ty) > 1) ? pick_vec(ty) : 1;
    const int V = vecw > 1 ? vecw : 4;
    Index ix(ty.rank());
    std::vector<std::string> vars;
    for (int d = 0; d < ty.rank(); ++d) {
      ix[d].var = d == a ? std::string("j") : (d < a ? "o" : "q") + std::to_string(d);
      ix[d].hi = ty.dims[d] - 1;
      vars.push_back(ix[d].var);
    }
    if (vecw > 1) {
      em.set_root(ty.dims, vars, true);
      em.vec = vecw;
      em.direct_expr = vec_name;
    } else {
      em.set_root({}, {}, false);
    }
    em.indent = rowwise ? 8 : 4;
    const std::string val = em.emit(rn.in[0], ix);
    const std::string body = em.take_code();
    em.indent = 2;
    const std::string initv = em.emit(rn.in[1], Index{});
    const std::string ibody = em.take_code();
    const std::string ost = info(dt).stype;
    const std::string rv = is_narrow_float(dt) ? Emitter::round_narrow(dt, "r") : std::string("(") + info(dt).ctype + ")r";
    const std::string jexpr = rev ? std::to_string(n - 1) + " - p" : std::string("p");
    auto decompose = [&](std::ostringstream& o, const std::string& var, int d0, int d1) {
      o << "  " << it << " rr_" << var << " = " << var << ";\n";
      for (int d = d1 - 1; d >= d0; --d) {
        o << "  const " << it << " " << (d < a ? "o" : "q") << d << " = rr_" << var << " % " << ty.dims[d] << ";\n";
        o << "  rr_" << var << " /= " << ty.dims[d] << ";\n";
      }
      o << "  (void)rr_" << var << ";\n";
    };
    std::ostringstream o;
    Launch L1, L2;
    int64_t NC = 1, CH = n;
    if (rowwise) {
      const int TILE = kBlock * V;
      // preloads of the inputs that are read at the scan's own index, one vector per lane
      auto preload = [&](std::ostringstream& oo, const std::string& pad) {
        if (vecw == 1) return;
        oo << pad << "const " << it << " lin0 = row * " << n << " + pb;\n";
        for (auto& sd : em.direct_vecs) {
          const int slot = sd.first;
          const std::string vt = "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vecw) + ">";
          oo << pad << vt << " " << vec_name(slot, 0) << " = {};\n";
          oo << pad << "if (pb < pend) " << vec_name(slot, 0) << " = rx_load<" << vt << ">(in" << slot << " + lin0);\n";
        }
      };
      NC = std::max<int64_t>(1, std::min<int64_t>((n + 4 * TILE - 1) / (4 * TILE), std::max<int64_t>(1, 2048 / std::max<int64_t>(outer, 1))));
      CH = ((n + NC - 1) / NC + TILE - 1) / TILE * TILE;
      NC = (n + CH - 1) / CH;
      auto head = [&](const std::string& kname, bool with_tot, bool with_out) {
        std::string sg = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void " + kname + "(";
        bool first = true;
        for (size_t k = 0; k < em.inputs.size(); ++k) {
          sg += (first ? "" : ", ") + ptr_decl(info(g.nodes[em.inputs[k]].ty.dt).stype, true, "in" + std::to_string(k));
          first = false;
        }
        if (with_tot) { sg += (first ? "" : ", ") + ptr_decl(ACC, with_out, "tot"); first = false; }
        if (with_out) sg += (first ? "" : ", ") + ptr_decl(ost, false, "out0");
        return sg + ")";
      };
      auto prologue = [&](std::ostringstream& oo) {
        oo << "  const " << it << " c = (" << it << ")(blockIdx.x % " << NC << "u), row = (" << it << ")(blockIdx.x / " << NC << "u);\n";
        decompose(oo, "row", 0, a);
        for (int d = a + 1; d < ty.rank(); ++d) oo << "  const " << it << " q" << d << " = 0;\n";
        oo << "  const " << it << " pend = rx_min<" << it << ">((c + 1) * " << CH << ", " << n << ");\n";
      };
      // Long rows in one launch.  A workgroup owns a chunk of T tiles, keeps its values in registers, publishes the
      // chunk's total as flagged 64-bit words (rx_publish_partial: no fence), and builds its carry from what the
      // chunks before it published.  Totals exist per chunk and per group of 256 chunks (summed and published by the
      // group's last chunk).  A chunk's carry is the totals of the groups up to the last but one before its own, then
      // the chunks of the group before its own and of its own group up to itself: at most 511 chunk slots and one
      // slot per older group, all requested at once and combined in an order that depends on the chunk index alone,
      // so the result does not depend on timing.  A group's total is first needed by chunks that start 256 chunks
      // after the one that publishes it, so nobody waits for a sum of sums: with groups of 32 whose totals the next
      // group needs at once, a chunk waited 5.4 us on average, with this window 3.7 (2^26 f32, time stamps inside
      // the kernel).  Every workgroup waits only for lower-numbered ones, which the dispatcher
      // started no later (workgroups start in index order on each die: an assumption about the dispatcher).  Waits are
      // bounded: one that expires sets the device's fault word, the next call that waits for the device raises an
      // error instead of handing out the result, and from then on the host rebuilds every executable with such a kernel
      // in the two-launch form (also what RX_SINGLE_PASS_SCAN=0 selects), which never waits.  Nothing is cleared between runs: a flag is the row's epoch, a word that
      // the row's last chunk advances once its carry is complete -- by then every chunk of the row has published, so
      // has read the epoch (one counter of finished workgroups would cost 60 ns each: atomics on one address from
      // eight dies).  The data is read once and written once.
      {
        constexpr int GS = kBlock;
        // tiles per chunk: 2^26 f32 takes 121 / 99 / 97 us with 8 / 16 / 32 (few tiles: too many workgroups polling;
        // 32: 182 registers)
        const int T = getenv("RX_SCAN_T") ? std::max(1, std::min(32, atoi(getenv("RX_SCAN_T")))) : 16;
        const int64_t sCH = (int64_t)T * TILE;
        const int64_t sNC = (n + sCH - 1) / sCH;
        const int64_t sNG = (sNC + GS - 1) / GS, SL = sNC + sNG;
        const int NW = (ACC == "double" || info(dt).size == 8) ? 2 : 1;
        const int64_t slot_words = outer * SL * NW + outer;   // + one epoch word per row
        if (opt.single_pass_scan && sNC > 1 && sNC * outer < ((int64_t)1 << 30) && slot_words * 8 <= ((int64_t)64 << 20)) {
          auto slot_of = [&](const std::string& idx) { return "slots + (row * " + std::to_string(SL) + " + " + idx + ") * " + std::to_string(NW); };
          std::string sg = head("@K@_scan", false, false);
          sg.pop_back();
          sg += std::string(em.inputs.empty() ? "" : ", ") + "unsigned long long* __restrict__ slots, unsigned* __restrict__ fault, " + ptr_decl(ost, false, "out0") + ")";
          // polls before a wait gives up (about 0.1 s); RX_SCAN_SPIN_LIMIT exists so that a test can make a wait expire
          const int spin_limit = getenv("RX_SCAN_SPIN_LIMIT") ? std::max(0, atoi(getenv("RX_SCAN_SPIN_LIMIT"))) : (1 << 16);
          o << "// scan along the minor dimension of " << ty.str() << " (" << sNC << " chunks per row, one launch): " << describe(rn.in[0]) << "\n";
          o << sg << " {\n";
          o << "  __shared__ " << ACC << " lds[" << kBlock / 64 << "];\n  __shared__ " << ACC << " wsum[" << T * (kBlock / 64) << "];\n  __shared__ int anyw;\n";
          o << "  bool bad = false;   // a wait of this thread expired\n";
          o << "  const " << it << " c = (" << it << ")(blockIdx.x % " << sNC << "u), row = (" << it << ")(blockIdx.x / " << sNC << "u);\n";
          decompose(o, "row", 0, a);
          for (int d = a + 1; d < ty.rank(); ++d) o << "  const " << it << " q" << d << " = 0;\n";
          // rows that are a whole number of chunks need none of the guards below
          const bool whole = n % sCH == 0;
          const std::string in_chunk = whole ? "true" : "pb < pend", in_row = whole ? "true" : "p < pend";
          o << "  const " << it << " pend = rx_min<" << it << ">((c + 1) * " << sCH << ", " << n << ");\n  (void)pend;\n";
          o << ibody;
          o << "  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;\n";
          o << "  const rx_u32 epoch = (rx_u32)slots[" << outer * SL * NW << " + row] + 1u;\n";
          o << "  " << ACC << " v[" << T << "][" << V << "], pre[" << T << "];\n";
          // all loads of the chunk first (rows of whole vectors), so that a workgroup has its whole chunk in flight
          if (vecw > 1) {
            for (auto& sd : em.direct_vecs) {
              const int slot = sd.first;
              const std::string vt = "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vecw) + ">";
              o << "  " << vt << " " << vec_name(slot, 0) << "t[" << T << "];\n";
            }
            o << "#pragma unroll\n  for (int t = 0; t < " << T << "; ++t) {\n";
            o << "    const " << it << " pb = c * " << sCH << " + t * " << TILE << " + (" << it << ")threadIdx.x * " << V << ";\n";
            for (auto& sd : em.direct_vecs) {
              const int slot = sd.first;
              const std::string vt = "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vecw) + ">";
              o << "    " << vec_name(slot, 0) << "t[t] = " << vt << "{};\n";
              o << "    if (" << in_chunk << ") " << vec_name(slot, 0) << "t[t] = " << (opt.nt_loads ? "rx_load_nt" : "rx_load") << "<" << vt << ">(in" << slot << " + row * " << n << " + pb);\n";
            }
            o << "  }\n";
          }
          o << "#pragma unroll\n  for (int t = 0; t < " << T << "; ++t) {\n";
          o << "    const " << it << " pb = c * " << sCH << " + t * " << TILE << " + (" << it << ")threadIdx.x * " << V << ";\n";
          if (vecw > 1) {
            o << "    const " << it << " lin0 = row * " << n << " + pb;\n    (void)lin0;\n";
            for (auto& sd : em.direct_vecs) o << "    const auto& " << vec_name(sd.first, 0) << " = " << vec_name(sd.first, 0) << "t[t];\n";
          }
          o << "#pragma unroll\n    for (int l = 0; l < " << V << "; ++l) {\n      const " << it << " p = pb + l;\n      v[t][l] = " << IDENT << ";\n      if (" << in_row << ") {\n";
          o << "        const " << it << " j = " << jexpr << ";\n" << body;
          o << "        v[t][l] = (" << ACC << ")" << val << ";\n      }\n    }\n  }\n";
          // The chunk's total goes out before the scans inside the chunk, in an order of its own (values of a lane,
          // lanes, wavefronts): the chunks behind this one wait for it, and the scans are a microsecond of work
          // (2^26 f32: 99 -> 87 us in a standalone kernel, the wait for the carry 6.7 -> 3.6 us per chunk).
          o << "  {\n    " << ACC << " tot = " << IDENT << ";\n";
          o << "#pragma unroll\n    for (int t = 0; t < " << T << "; ++t) {\n      " << ACC << " s = v[t][0];\n";
          o << "#pragma unroll\n      for (int l = 1; l < " << V << "; ++l) s = " << red_apply(rn.red, dt, "s", "v[t][l]") << ";\n";
          o << "      tot = " << red_apply(rn.red, dt, "tot", "s") << ";\n    }\n";
          o << "    tot = rx_block_reduce<" << ACC << ", decltype(" << OP << "), " << kBlock / 64 << ">(tot, " << OP << ", lds);\n";
          o << "    if (threadIdx.x == 0) rx_publish_partial<" << ACC << ">(" << slot_of("c") << ", tot, epoch);\n  }\n";
          o << "#pragma unroll\n  for (int t = 0; t < " << T << "; ++t) {\n";
          o << "#pragma unroll\n    for (int l = 1; l < " << V << "; ++l) v[t][l] = " << red_apply(rn.red, dt, "v[t][l - 1]", "v[t][l]") << ";\n";
          o << "    const " << ACC << " incl = rx_wave_scan(v[t][" << V - 1 << "], " << OP << ");\n";
          o << "    if (lane == 63) wsum[t * " << kBlock / 64 << " + w] = incl;\n";
          o << "    pre[t] = rx_lane_from(incl, (rx_u32)(lane - 1) & 63u);\n  }\n";
          o << "  __syncthreads();\n";
          o << "  " << ACC << " run = " << IDENT << ";\n";
          o << "#pragma unroll\n  for (int t = 0; t < " << T << "; ++t) {\n";
          o << "    " << ACC << " pt = run;\n    " << ACC << " total = wsum[t * " << kBlock / 64 << "];\n";
          o << "#pragma unroll\n    for (int i = 0; i < " << kBlock / 64 << "; ++i) {\n      if (i < w) pt = " << red_apply(rn.red, dt, "pt", "wsum[t * " + std::to_string(kBlock / 64) + " + i]") << ";\n";
          o << "      if (i > 0) total = " << red_apply(rn.red, dt, "total", "wsum[t * " + std::to_string(kBlock / 64) + " + i]") << ";\n    }\n";
          o << "    if (lane > 0) pt = " << red_apply(rn.red, dt, "pt", "pre[t]") << ";\n";
          // pinned here: left to itself the compiler computes these after the waits below and keeps the wavefront
          // totals of every tile in registers until then (186 registers instead of 102, half the resident workgroups)
          o << "    pre[t] = pt;\n    rx_pin(pre[t]);\n";
          o << "    run = " << red_apply(rn.red, dt, "run", "total") << ";\n  }\n";
          // the last chunk of a group also publishes the group's total
          o << "  if (c % " << GS << " == " << GS - 1 << ") {\n";
          o << "    " << ACC << " part = rx_peek_partial<" << ACC << ">(" << slot_of("(c - " + std::to_string(GS - 1) + " + (" + it + ")threadIdx.x)") << ", epoch, " << spin_limit << ", fault, &bad);\n";
          o << "    part = rx_block_reduce<" << ACC << ", decltype(" << OP << "), " << kBlock / 64 << ">(part, " << OP << ", lds);\n";
          // a group total built from a slot that never arrived is not published: the chunks that need it expire in turn
          o << "    const bool gbad = rx_block_any(bad, &anyw);\n";
          o << "    if (threadIdx.x == 0 && !gbad) rx_publish_partial<" << ACC << ">(" << slot_of(std::to_string(sNC) + " + c / " + std::to_string(GS)) << ", part, epoch);\n";
          o << "  }\n";
          // carry
          o << "  " << ACC << " carry = (" << ACC << ")" << initv << ";\n";
          o << "  {\n    const " << it << " g = c / " << GS << ", ngr = g >= 2 ? g - 1 : 0, c0 = (g >= 1 ? g - 1 : 0) * " << GS << ";\n";
          o << "    " << ACC << " part = " << IDENT << ";\n";
          o << "    for (" << it << " k = threadIdx.x; k < ngr + (c - c0); k += " << kBlock << ") {\n";
          o << "      const " << it << " idx = k < ngr ? " << sNC << " + k : c0 + (k - ngr);\n";
          o << "      part = " << red_apply(rn.red, dt, "part", "rx_peek_partial<" + ACC + ">(" + slot_of("idx") + ", epoch, " + std::to_string(spin_limit) + ", fault, &bad)") << ";\n    }\n";
          o << "    part = rx_block_reduce<" << ACC << ", decltype(" << OP << "), " << kBlock / 64 << ">(part, " << OP << ", lds);\n";
          o << "    if (c != 0) carry = " << red_apply(rn.red, dt, "carry", "part") << ";\n  }\n";
          // the row's last chunk has, through its carry, heard from every chunk of the row: the next run's epoch.  Not
          // when one of its waits expired: a chunk that has not started yet would read the new epoch and publish under it
          // (the host rebuilds the executable without waits before it runs again, so the stale flags are never read)
          o << "  if (c == " << sNC - 1 << ") {\n    const bool rbad = rx_block_any(bad, &anyw);\n";
          o << "    if (threadIdx.x == 0 && !rbad) slots[" << outer * SL * NW << " + row] = (unsigned long long)(epoch == 0xffffffffu ? 0u : epoch);\n  }\n";
          // results
          o << "#pragma unroll\n  for (int t = 0; t < " << T << "; ++t) {\n";
          o << "    const " << it << " pb = c * " << sCH << " + t * " << TILE << " + (" << it << ")threadIdx.x * " << V << ";\n";
          o << "    const " << ACC << " pt = " << red_apply(rn.red, dt, "carry", "pre[t]") << ";\n";
          if (vecw > 1) {
            o << "    if (" << in_chunk << ") {\n      rx_vec<" << ost << ", " << V << "> res;\n";
            o << "#pragma unroll\n      for (int l = 0; l < " << V << "; ++l) {\n";
            o << "        const " << ACC << " r = " << red_apply(rn.red, dt, "pt", "v[t][l]") << ";\n";
            o << "        res.v[l] = " << Emitter::store_conv(dt, rv) << ";\n      }\n";
            o << "      *reinterpret_cast<rx_vec<" << ost << ", " << V << ">*>(out0 + row * " << n << " + pb) = res;\n    }\n";
          } else {
            o << "#pragma unroll\n    for (int l = 0; l < " << V << "; ++l) {\n      const " << it << " p = pb + l;\n      if (" << in_row << ") {\n";
            o << "        const " << ACC << " r = " << red_apply(rn.red, dt, "pt", "v[t][l]") << ";\n";
            o << "        out0[row * " << n << " + (" << jexpr << ")] = " << Emitter::store_conv(dt, rv) << ";\n      }\n    }\n";
          }
          o << "  }\n}\n\n";
          const std::string kb_single = finalize(o.str());
          BufferDesc cb;
          cb.kind = BufferDesc::Const;          // lives with the executable; zero when loaded
          cb.ty.dt = DT::U64;
          cb.ty.dims = {slot_words};
          cb.bytes = slot_words * 8;
          cb.data.assign((size_t)cb.bytes, 0);
          plan.buffers.push_back(cb);
          const int slots_buf = (int)plan.buffers.size() - 1;
          BufferDesc fb;
          fb.kind = BufferDesc::Fault;
          fb.ty.dt = DT::U32;
          fb.ty.dims = {1};
          fb.bytes = 4;
          plan.buffers.push_back(fb);
          const int fault_buf = (int)plan.buffers.size() - 1;
          Launch L;
          L.kernel = named("@K@_scan", kb_single);
          L.kind = "scan";
          L.grid[0] = (unsigned)(sNC * outer);
          L.block[0] = kBlock;
          for (int i : em.inputs) L.args.push_back(buffer_for(i));
          L.args.push_back(slots_buf);
          L.args.push_back(fault_buf);
          L.args.push_back(buffer_for(root));
          L.algo_bytes = algo_bytes(em.inputs, {root});
          L.desc = describe(rn.in[0]) + " scan";
          plan.launches.push_back(L);
          return;
        }
      }
      o << "// scan along the minor dimension of " << ty.str() << " (" << NC << " chunk" << (NC > 1 ? "s" : "") << " per row): " << describe(rn.in[0]) << "\n";
      if (NC > 1) {
        o << head("@K@_scan_totals", true, false) << " {\n";
        o << "  __shared__ " << ACC << " lds[" << kBlock / 64 << "];\n";
        prologue(o);
        if (vecw > 1) {
          // Rows of whole vectors: a vector that starts inside the chunk lies inside it.  Four tiles per
          // iteration, their loads issued together (one 16-byte load in flight per lane does not
          // cover the memory latency), each with its own accumulator.
          constexpr int U = 4;
          o << "  " << ACC << " accu[" << U << "];\n#pragma unroll\n  for (int u = 0; u < " << U << "; ++u) accu[u] = " << IDENT << ";\n";
          o << "  " << it << " pb = c * " << CH << " + (" << it << ")threadIdx.x * " << V << ";\n";
          auto one = [&](const std::string& pbexpr, int u, const std::string& pad) {
            // the generated expression names its preloaded vectors; give every tile of the group its own
            std::string b = body, vv = val;
            for (auto& sd : em.direct_vecs) {
              const std::string from = vec_name(sd.first, 0), to = from + "u" + std::to_string(u);
              for (std::string* t : {&b, &vv})
                for (size_t q = t->find(from + "."); q != std::string::npos; q = t->find(from + ".", q + to.size())) t->replace(q, from.size(), to);
            }
            o << pad << "{\n" << pad << "  const " << it << " pbu = " << pbexpr << ";\n";
            o << "#pragma unroll\n" << pad << "  for (int l = 0; l < " << V << "; ++l) {\n" << pad << "    const " << it << " j = pbu + l;\n" << b;
            o << pad << "    accu[" << u << "] = " << red_apply(rn.red, dt, "accu[" + std::to_string(u) + "]", "(" + ACC + ")" + vv) << ";\n" << pad << "  }\n" << pad << "}\n";
          };
          auto loads = [&](const std::string& pbexpr, int u, const std::string& pad) {
            for (auto& sd : em.direct_vecs) {
              const int slot = sd.first;
              const std::string vt = "rx_vec<" + std::string(info(g.nodes[em.inputs[slot]].ty.dt).stype) + ", " + std::to_string(vecw) + ">";
              o << pad << "const " << vt << " " << vec_name(slot, 0) << "u" << u << " = " << (opt.nt_loads ? "rx_load_nt" : "rx_load") << "<" << vt << ">(in" << slot << " + row * " << n << " + " << pbexpr << ");\n";
            }
          };
          o << "  for (; pb + " << (U - 1) * TILE << " < pend; pb += " << U * TILE << ") {\n";
          for (int u = 0; u < U; ++u) loads("pb + " + std::to_string(u * TILE), u, "    ");
          for (int u = 0; u < U; ++u) one("pb + " + std::to_string(u * TILE), u, "    ");
          o << "  }\n  for (; pb < pend; pb += " << TILE << ") {\n";
          loads("pb", 0, "    ");
          one("pb", 0, "    ");
          o << "  }\n  " << ACC << " acc = accu[0];\n#pragma unroll\n  for (int u = 1; u < " << U << "; ++u) acc = " << red_apply(rn.red, dt, "acc", "accu[u]") << ";\n";
        } else {
          o << "  " << ACC << " acc = " << IDENT << ";\n";
          o << "  for (" << it << " pb = c * " << CH << " + (" << it << ")threadIdx.x * " << V << "; pb < pend; pb += " << TILE << ") {\n";
          o << "#pragma unroll\n    for (int l = 0; l < " << V << "; ++l) {\n      const " << it << " p = pb + l;\n      if (p < pend) {\n";
          o << "        const " << it << " j = " << jexpr << ";\n" << body;
          o << "        acc = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + val) << ";\n      }\n    }\n  }\n";
        }
        o << "  acc = rx_block_reduce<" << ACC << ", decltype(" << OP << "), " << kBlock / 64 << ">(acc, " << OP << ", lds);\n";
        o << "  if (threadIdx.x == 0) tot[row * " << NC << " + c] = acc;\n}\n\n";
      }
      o << head("@K@_scan", NC > 1, true) << " {\n";
      o << "  __shared__ " << ACC << " lds[" << kBlock / 64 << "];\n  __shared__ " << ACC << " wsum[" << kBlock / 64 << "];\n";
      prologue(o);
      o << ibody;
      o << "  " << ACC << " carry = " << IDENT << ";\n";
      o << "  if (c == 0) carry = (" << ACC << ")" << initv << ";\n";
      if (NC > 1) {
        o << "  {\n    " << ACC << " part = " << IDENT << ";\n";
        o << "    for (" << it << " s = threadIdx.x; s < c; s += " << kBlock << ") part = " << red_apply(rn.red, dt, "part", "tot[row * " + std::to_string(NC) + " + s]") << ";\n";
        o << "    part = rx_block_reduce<" << ACC << ", decltype(" << OP << "), " << kBlock / 64 << ">(part, " << OP << ", lds);\n";
        o << "    if (c != 0) carry = " << red_apply(rn.red, dt, "(" + ACC + ")" + initv, "part") << ";\n  }\n";
      } else {
        o << "  (void)lds;\n";
      }
      o << "  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;\n";
      o << "  for (" << it << " tb = c * " << CH << "; tb < pend; tb += " << TILE << ") {\n";
      o << "    const " << it << " pb = tb + (" << it << ")threadIdx.x * " << V << ";\n";
      o << "    " << ACC << " v[" << V << "];\n";
      preload(o, "    ");
      o << "#pragma unroll\n    for (int l = 0; l < " << V << "; ++l) {\n      const " << it << " p = pb + l;\n      v[l] = " << IDENT << ";\n      if (p < pend) {\n";
      o << "        const " << it << " j = " << jexpr << ";\n" << body;
      o << "        v[l] = (" << ACC << ")" << val << ";\n      }\n    }\n";
      o << "#pragma unroll\n    for (int l = 1; l < " << V << "; ++l) v[l] = " << red_apply(rn.red, dt, "v[l - 1]", "v[l]") << ";\n";
      o << "    const " << ACC << " incl = rx_wave_scan(v[" << V - 1 << "], " << OP << ");\n";
      o << "    __syncthreads();\n    if (lane == 63) wsum[w] = incl;\n    __syncthreads();\n";
      o << "    " << ACC << " pre = carry;\n    " << ACC << " total = wsum[0];\n";
      o << "#pragma unroll\n    for (int i = 0; i < " << kBlock / 64 << "; ++i) {\n      if (i < w) pre = " << red_apply(rn.red, dt, "pre", "wsum[i]") << ";\n";
      o << "      if (i > 0) total = " << red_apply(rn.red, dt, "total", "wsum[i]") << ";\n    }\n";
      o << "    const " << ACC << " below = rx_lane_from(incl, (rx_u32)(lane - 1) & 63u);\n";
      o << "    if (lane > 0) pre = " << red_apply(rn.red, dt, "pre", "below") << ";\n";
      if (vecw > 1) {
        o << "    if (pb < pend) {\n      rx_vec<" << ost << ", " << V << "> res;\n";
        o << "#pragma unroll\n      for (int l = 0; l < " << V << "; ++l) {\n";
        o << "        const " << ACC << " r = " << red_apply(rn.red, dt, "pre", "v[l]") << ";\n";
        o << "        res.v[l] = " << Emitter::store_conv(dt, rv) << ";\n      }\n";
        o << "      *reinterpret_cast<rx_vec<" << ost << ", " << V << ">*>(out0 + lin0) = res;\n    }\n";
      } else {
        o << "#pragma unroll\n    for (int l = 0; l < " << V << "; ++l) {\n      const " << it << " p = pb + l;\n      if (p < pend) {\n";
        o << "        const " << ACC << " r = " << red_apply(rn.red, dt, "pre", "v[l]") << ";\n";
        o << "        out0[row * " << n << " + (" << jexpr << ")] = " << Emitter::store_conv(dt, rv) << ";\n      }\n    }\n";
      }
      o << "    carry = " << red_apply(rn.red, dt, "carry", "total") << ";\n  }\n}\n\n";
      L1.grid[0] = L2.grid[0] = (unsigned)(NC * outer);
    } else {
      const int64_t lines = outer * inner;
      NC = std::max<int64_t>(1, std::min<int64_t>(65536 / std::max<int64_t>(lines, 1), n / 16));
      CH = (n + NC - 1) / NC;
      NC = (n + CH - 1) / CH;
      auto head = [&](const std::string& kname, bool with_tot, bool with_out) {
        std::string sg = "extern \"C\" __global__ __launch_bounds__(" + std::to_string(kBlock) + ") void " + kname + "(";
        bool first = true;
        for (size_t k = 0; k < em.inputs.size(); ++k) {
          sg += (first ? "" : ", ") + ptr_decl(info(g.nodes[em.inputs[k]].ty.dt).stype, true, "in" + std::to_string(k));
          first = false;
        }
        if (with_tot) { sg += (first ? "" : ", ") + ptr_decl(ACC, with_out, "tot"); first = false; }
        if (with_out) sg += (first ? "" : ", ") + ptr_decl(ost, false, "out0");
        return sg + ")";
      };
      // thread id -> (outer index, chunk, inner index); the inner index is the fastest
      auto prologue = [&](std::ostringstream& oo) {
        oo << "  const " << it << " tid = (" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x;\n";
        oo << "  if (tid >= " << lines * NC << ") return;\n";
        oo << "  const " << it << " qi = tid % " << inner << ";\n";
        oo << "  const " << it << " c = (tid / " << inner << ") % " << NC << ";\n";
        oo << "  const " << it << " oi = tid / " << inner * NC << ";\n";
        decompose(oo, "qi", a + 1, ty.rank());
        decompose(oo, "oi", 0, a);
        oo << "  const " << it << " pend = rx_min<" << it << ">((c + 1) * " << CH << ", " << n << ");\n";
      };
      o << "// scan along dimension " << a << " of " << ty.str() << " (" << NC << " chunk" << (NC > 1 ? "s" : "") << " per line): " << describe(rn.in[0]) << "\n";
      if (NC > 1) {
        o << head("@K@_scan_totals", true, false) << " {\n";
        prologue(o);
        o << "  " << ACC << " acc = " << IDENT << ";\n";
        o << "  for (" << it << " p = c * " << CH << "; p < pend; ++p) {\n";
        o << "    const " << it << " j = " << jexpr << ";\n" << body;
        o << "    acc = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + val) << ";\n  }\n";
        o << "  tot[(oi * " << NC << " + c) * " << inner << " + qi] = acc;\n}\n\n";
      }
      o << head("@K@_scan", NC > 1, true) << " {\n";
      prologue(o);
      o << ibody;
      o << "  " << ACC << " acc = (" << ACC << ")" << initv << ";\n";
      if (NC > 1)
        o << "  for (" << it << " s = 0; s < c; ++s) acc = " << red_apply(rn.red, dt, "acc", "tot[(oi * " + std::to_string(NC) + " + s) * " + std::to_string(inner) + " + qi]") << ";\n";
      o << "  for (" << it << " p = c * " << CH << "; p < pend; ++p) {\n";
      o << "    const " << it << " j = " << jexpr << ";\n" << body;
      o << "    acc = " << red_apply(rn.red, dt, "acc", "(" + ACC + ")" + val) << ";\n";
      o << "    const " << ACC << " r = acc;\n";
      o << "    out0[(oi * " << n << " + j) * " << inner << " + qi] = " << Emitter::store_conv(dt, rv) << ";\n  }\n}\n\n";
      L1.grid[0] = L2.grid[0] = (unsigned)((lines * NC + kBlock - 1) / kBlock);
    }
    const std::string kb_final = finalize(o.str());
    int sc = -1;
    if (NC > 1) {
      sc = scratch(outer * inner * NC * (int64_t)(ACC == "double" || info(dt).size == 8 ? 8 : 4));
      L1.kernel = named("@K@_scan_totals", kb_final);
      L1.kind = "scan_totals";
      L1.block[0] = kBlock;
      for (int i : em.inputs) L1.args.push_back(buffer_for(i));
      L1.args.push_back(sc);
      L1.algo_bytes = algo_bytes(em.inputs, {});
      L1.desc = describe(rn.in[0]) + " chunk totals";
      plan.launches.push_back(L1);
    }
    L2.kernel = named("@K@_scan", kb_final);
    L2.kind = "scan";
    L2.block[0] = kBlock;
    for (int i : em.inputs) L2.args.push_back(buffer_for(i));
    if (NC > 1) L2.args.push_back(sc);
    L2.args.push_back(buffer_for(root));
    L2.algo_bytes = algo_bytes(em.inputs, {root});
    L2.desc = describe(rn.in[0]) + " scan";
    plan.launches.push_back(L2);
  }

  // ------------------------------------------------------------------ row groups
  // `root` is either a Reduce over the trailing dims (plain row reduction) or an
  // elementwise node of shape [rows.., cols] whose cone contains row reductions `phases`.
  void emit_row(int root, const std::vector<int>& phases) {
    const Node& rn = g.nodes[root];
    const bool root_is_reduce = rn.k == OpK::Reduce;
    const TType& full = root_is_reduce ? g.nodes[rn.in[0]].ty : rn.ty;
    const int n = full.rank();
    int nkeep;
    if (root_is_reduce) nkeep = red_shape(rn).nkeep;
    else nkeep = red_shape(g.nodes[phases[0]]).nkeep;
    int64_t rows = 1, cols = 1;
    for (int d = 0; d < n; ++d) (d < nkeep ? rows : cols) *= full.dims[d];
    int vec = pick_vec(full);
    while (vec > 1 && cols % vec) vec >>= 1;
    // lanes cooperating on one row: a workgroup for long rows, a wavefront for medium ones, an
    // aligned group of 2..32 lanes for short ones (several rows per wavefront)
    int L = cols / vec >= 512 ? 256 : 64;
    if (cols / vec <= 32) {
      L = 1;
      while (L < cols / vec) L <<= 1;
    }
    const int rows_per_block = kBlock / L;
    const int64_t iters = (cols / vec + L - 1) / L;
    const bool cache = iters <= 8;
    const std::string kname = "@K@_row";

    std::set<int> phase_set(phases.begin(), phases.end());
    Emitter em(g, [&](int x) { return mat[x] && x != root && !phase_set.count(x); });
    em.excess_precision = opt.excess_precision;
    std::vector<int> touched = cone_nodes(root);
    for (int p : phases) { auto c = cone_nodes(p); touched.insert(touched.end(), c.begin(), c.end()); }
    em.idx64 = needs64(touched);
    const std::string it = em.idx_t();
    std::vector<std::string> vars;
    for (int d = 0; d < n; ++d) vars.push_back("i" + std::to_string(d));
    em.set_root(full.dims, vars, true);
    em.vec = vec;
    em.direct_expr = [&](int slot, int64_t) { return cache ? "c" + std::to_string(slot) + "[itv]" : "d" + std::to_string(slot); };
    Index ix = root_index(full.dims);

    struct PhaseCode { int node; std::string body, val; };
    std::vector<PhaseCode> pcs;
    std::vector<int> order = phases;
    std::sort(order.begin(), order.end());
    em.indent = 6;
    for (int p : order) {
      PhaseCode pc;
      pc.node = p;
      em.push_scope();
      pc.val = em.emit(g.nodes[p].in[0], ix);
      pc.body = em.take_code();
      em.pop_scope();
      em.bound[p] = "r" + std::to_string(p);
      pcs.push_back(pc);
    }
    std::string fbody, fval;
    if (!root_is_reduce) {
      em.push_scope();
      fval = em.emit(root, ix);
      fbody = em.take_code();
      em.pop_scope();
    }
    // init values of the reductions (scalars)
    em.indent = 2;
    std::map<int, std::string> inits;
    for (int p : order) inits[p] = em.emit(g.nodes[p].in[1], Index{});
    std::string init_code = em.take_code();

    std::ostringstream o;
    std::vector<std::pair<std::string, std::string>> outs;
    if (root_is_reduce) outs.push_back({info(rn.ty.dt).stype, "out0"});
    else outs.push_back({info(rn.ty.dt).stype, "out0"});
    o << "// row group (" << rows << " rows x " << cols << "): " << describe(root, phases) << "\n";
    o << signature(kname, em.inputs, outs) << " {\n";
    o << "  const int lane = threadIdx.x % " << L << ";\n";
    o << "  const " << it << " row = (" << it << ")blockIdx.x * " << rows_per_block << " + threadIdx.x / " << L << ";\n";
    if (L <= 64) o << "  if (row >= " << rows << ") return;\n";  // whole groups of lanes leave together
    o << init_code;
    // decode row -> leading index vars
    {
      o << "  " << it << " rr = row;\n";
      for (int d = nkeep - 1; d >= 0; --d) {
        o << "  const " << it << " i" << d << " = rr % " << full.dims[d] << ";\n";
        o << "  rr /= " << full.dims[d] << ";\n";
      }
    }
    o << "  const " << it << " rowbase = row * " << cols << (em.idx64 ? "LL" : "") << ";\n";
    if (L == 256) o << "  __shared__ double lds_raw[" << kBlock / 64 << "];\n";
    // column loop header: declares trailing index vars for vector `itv`
    auto loop_open = [&](std::ostringstream& s) {
      s << "#pragma unroll\n  for (int itv = 0; itv < " << iters << "; ++itv) {\n";
      s << "    const " << it << " cv = (" << it << ")(itv * " << L << " + lane) * " << vec << ";\n";
      s << "    if (cv < " << cols << ") {\n";
      s << "      const " << it << " lin0 = rowbase + cv;\n";
    };
    auto decode_cols = [&](std::ostringstream& s) {
      // column offset c = cv + l -> trailing dims
      if (n - nkeep == 1) {
        s << "        const " << it << " i" << n - 1 << " = cv + l;\n";
      } else {
        s << "        " << it << " cc = cv + l;\n";
        for (int d = n - 1; d > nkeep; --d) {
          s << "        const " << it << " i" << d << " = cc % " << full.dims[d] << ";\n";
          s << "        cc /= " << full.dims[d] << ";\n";
        }
        s << "        const " << it << " i" << nkeep << " = cc;\n";
      }
    };
    // preload of direct inputs
    auto preload = [&](std::ostringstream& s, bool into_cache) {
      for (auto& sd : em.direct_vecs) {
        const int slot = sd.first;
        const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
        if (into_cache)
          s << "      c" << slot << "[itv] = *reinterpret_cast<const rx_vec<" << st << ", " << vec << ">*>(in" << slot << " + lin0);\n";
        else
          s << "      const rx_vec<" << st << ", " << vec << "> d" << slot << " = *reinterpret_cast<const rx_vec<" << st << ", " << vec << ">*>(in" << slot
            << " + lin0);\n";
      }
    };
    if (cache) {
      for (auto& sd : em.direct_vecs) {
        const int slot = sd.first;
        const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
        o << "  rx_vec<" << st << ", " << vec << "> c" << slot << "[" << iters << "];\n";
      }
      if (!em.direct_vecs.empty()) {
        loop_open(o);
        preload(o, true);
        o << "    }\n  }\n";
      }
    }
    for (auto& pc : pcs) {
      const Node& p = g.nodes[pc.node];
      const DT dt = p.ty.dt;
      const std::string ACC = acc_ctype(dt);
      o << "  " << ACC << " a" << pc.node << " = " << red_identity(p.red, dt) << ";\n";
      loop_open(o);
      if (!cache) preload(o, false);
      o << "#pragma unroll\n      for (int l = 0; l < " << vec << "; ++l) {\n";
      decode_cols(o);
      o << pc.body;
      o << "        a" << pc.node << " = " << red_apply(p.red, dt, "a" + std::to_string(pc.node), "(" + ACC + ")" + pc.val) << ";\n";
      o << "      }\n    }\n  }\n";
      if (L == 64)
        o << "  a" << pc.node << " = rx_wave_reduce(a" << pc.node << ", " << red_functor(p.red) << ");\n";
      else if (L < 64)
        o << "  a" << pc.node << " = rx_group_reduce<" << L << ">(a" << pc.node << ", " << red_functor(p.red) << ");\n";
      else
        o << "  a" << pc.node << " = rx_block_reduce<" << ACC << ", decltype(" << red_functor(p.red) << "), " << kBlock / 64 << ">(a" << pc.node << ", "
          << red_functor(p.red) << ", reinterpret_cast<" << ACC << "*>(lds_raw));\n";
      std::string comb = red_apply(p.red, dt, "a" + std::to_string(pc.node), "(" + ACC + ")" + inits[pc.node]);
      // a reduction consumed inside the kernel stays in f32 under excess precision
      const bool rnd = is_narrow_float(dt) && !(opt.excess_precision && !root_is_reduce);
      std::string rv = rnd ? Emitter::round_narrow(dt, comb) : std::string("(") + info(dt).ctype + ")(" + comb + ")";
      o << "  const " << info(dt).ctype << " r" << pc.node << " = " << rv << ";\n";
    }
    if (root_is_reduce) {
      o << "  if (lane == 0) out0[row] = " << Emitter::store_conv(rn.ty.dt, "r" + std::to_string(root)) << ";\n";
    } else {
      const std::string ost = info(rn.ty.dt).stype;
      loop_open(o);
      if (!cache) preload(o, false);
      o << "      rx_vec<" << ost << ", " << vec << "> res;\n";
      o << "#pragma unroll\n      for (int l = 0; l < " << vec << "; ++l) {\n";
      decode_cols(o);
      o << fbody;
      o << "        res.v[l] = " << em.store_value(rn.ty.dt, fval) << ";\n      }\n";
      o << "      *reinterpret_cast<rx_vec<" << ost << ", " << vec << ">*>(out0 + lin0) = res;\n";
      o << "    }\n  }\n";
    }
    o << "}\n\n";
    const std::string kb_final = finalize(o.str());

    Launch Lc;
    Lc.kernel = named(kname, kb_final);
    Lc.kind = "row";
    Lc.grid[0] = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
    Lc.block[0] = kBlock;
    for (int i : em.inputs) Lc.args.push_back(buffer_for(i));
    Lc.args.push_back(buffer_for(root));
    Lc.algo_bytes = algo_bytes(em.inputs, {root});
    Lc.desc = describe(root, phases);
    plan.launches.push_back(Lc);
    (void)L;
  }

  // Row reductions that can run inside the kernel of `root` (see header comment).
  // All calls come after the analysis has settled, so the answers are kept; the reductions of the
  // module are listed once (a time loop unrolls into thousands of roots and no reduction at all).
  std::map<int, std::vector<int>> row_phase_cache;
  std::vector<int> row_reduces;
  bool row_reduces_listed = false;
  std::vector<int> row_phases(int root) {
    auto hit = row_phase_cache.find(root);
    if (hit != row_phase_cache.end()) return hit->second;
    return row_phase_cache[root] = row_phases_uncached(root);
  }
  std::vector<int> row_phases_uncached(int root) {
    const Node& rn = g.nodes[root];
    std::vector<int> phases;
    if (!opt.row_fusion || rn.ty.rank() < 2) return phases;
    if (!row_reduces_listed) {
      row_reduces_listed = true;
      for (int x = 0; x < (int)g.nodes.size(); ++x)
        if (live[x] && g.nodes[x].k == OpK::Reduce && std::find(g.results.begin(), g.results.end(), x) == g.results.end()) row_reduces.push_back(x);
    }
    std::set<int> S{root};
    bool changed = true;
    while (changed) {
      changed = false;
      for (int x : row_reduces) {
        if (S.count(x)) continue;
        const Node& r = g.nodes[x];
        const TType& in = g.nodes[r.in[0]].ty;
        if (in.dims != rn.ty.dims) continue;
        RedShape rs = red_shape(r);
        if (!rs.trailing || rs.nkeep == 0 || rs.nkeep == in.rank()) continue;
        if (!phases.empty() && red_shape(g.nodes[phases[0]]).nkeep != rs.nkeep) continue;
        if (ctx[x].empty()) continue;
        bool ok = true;
        for (auto& c : ctx[x]) {
          if (!S.count(c.first)) { ok = false; break; }
          // path must be: (elementwise)* broadcast_in_dim(dims = 0..nkeep-1) (elementwise on the kept shape)*
          const std::string& sig = c.second;
          if (sig.size() < 2 || sig[0] != '/' || sig.find('/', 1) != std::string::npos) { ok = false; break; }
          int bid = std::stoi(sig.substr(1, sig.find(':') - 1));
          const Node& b = g.nodes[bid];
          if (b.k != OpK::BroadcastInDim || b.ty.dims != rn.ty.dims || (int)b.a0.size() != rs.nkeep) { ok = false; break; }
          for (int k = 0; k < rs.nkeep; ++k) ok = ok && b.a0[k] == k;
          if (!ok) break;
        }
        if (!ok) continue;
        S.insert(x);
        phases.push_back(x);
        changed = true;
      }
    }
    return phases;
  }

  // ------------------------------------------------------------------ dot groups
  struct DotForm {
    bool ok = false;        // matrix (optionally batched) form the GEMM skeletons understand
    int64_t batch = 1, M = 1, N = 1, K = 1;
    bool a_k_contig = false;  // lhs stored [.., M, K] (true) or [.., K, M]
    bool b_k_contig = false;  // rhs stored [.., N, K] (true) or [.., K, N]
  };
  DotForm dot_form(const Node& d) const {
    DotForm f;
    const TType &l = g.nodes[d.in[0]].ty, &r = g.nodes[d.in[1]].ty;
    if (d.a2.size() != 1) return f;
    if (d.a0.size() > 1) return f;
    const int nb = (int)d.a0.size();
    if (l.rank() != 2 + nb || r.rank() != 2 + nb) return f;
    if (nb == 1 && (d.a0[0] != 0 || d.a1[0] != 0)) return f;
    const int lc = (int)d.a2[0], rc = (int)d.a3[0];
    f.batch = nb ? l.dims[0] : 1;
    f.K = l.dims[lc];
    f.a_k_contig = lc == nb + 1;
    f.b_k_contig = rc == nb + 1;
    f.M = l.dims[f.a_k_contig ? nb : nb + 1];
    f.N = r.dims[f.b_k_contig ? nb : nb + 1];
    f.ok = true;
    return f;
  }

  // Emit the dot group rooted at `root`; `dot` is the DotGeneral node inside it
  // (root == dot when there is no epilogue).
  void emit_dot(int root, int dot) {
    const Node& d = g.nodes[dot];
    const Node& rn = g.nodes[root];
    const TType &lt = g.nodes[d.in[0]].ty, &rt = g.nodes[d.in[1]].ty;
    DotForm f = dot_form(d);
    const std::string kbase = "@K@";
    const int n = rn.ty.rank();

    // Epilogue: the cone from the root down to the dot accumulator, evaluated on NV
    // consecutive elements of the minor output dimension (vector loads of same-shaped
    // operands such as C in alpha*A*B + beta*C, one vector store).
    const bool fuse_a = fused_operands.count({dot, 0}) != 0, fuse_b = fused_operands.count({dot, 1}) != 0;
    GemmChoice gc;
    const int ksplit = d.a4.empty() ? 1 : (int)d.a4[0];
    if (opt.mfma && f.ok && n >= 2) gc = choose_gemm(lt.dt, rt.dt, d.ty.dt, f.batch, f.M, f.N, f.K, f.a_k_contig, f.b_k_contig, fuse_a || fuse_b, ksplit);
    if ((fuse_a || fuse_b) && !gc.ok) throw Error("internal: a fused dot_general operand without a GEMM skeleton");
    if (ksplit > 1 && (!gc.ok || gc.split != ksplit || root != dot)) throw Error("internal: a dot_general cut along K without the skeleton that slices K");

    Emitter em(g, [&](int x) { return mat[x] && x != root; });
    em.excess_precision = opt.excess_precision;
    em.idx64 = needs64(cone_nodes(root)) || lt.numel() >= ((int64_t)1 << 31) || rt.numel() >= ((int64_t)1 << 31);
    const std::string it = em.idx_t();
    std::vector<std::string> vars;
    for (int k = 0; k < n; ++k) vars.push_back("i" + std::to_string(k));
    em.set_root(rn.ty.dims, vars, n > 0);
    em.vec = 4;  // only unshifted vectors are used here; the width is the template parameter NV
    em.direct_expr = vec_name;
    em.indent = 6;
    const std::string DCT = info(d.ty.dt).ctype;
    // The product's only consumer adds a vector along the result's columns (a bias): the streaming skeletons take it as
    // the accumulators' first values (rx_epi_has_init), and the epilogue starts behind the addition.  Only where narrow
    // results keep their float32 values inside a kernel anyway (the sum is then rounded once either way).
    int init_add = -1, init_vec = -1;
    if (opt.epilogue_init && opt.excess_precision && root != dot && gc.ok && (gc.skeleton == "rx_gemm_body_pp" || gc.skeleton == "rx_gemm_body_s") && d.a0.empty() &&
        n == 2 && is_float(d.ty.dt) && d.ty.dt != DT::F64) {
      int users = 0, add = -1;
      for (int x : cone_nodes(root))
        for (int i : g.nodes[x].in)
          if (i == dot) { ++users; add = x; }
      if (users == 1 && g.nodes[add].k == OpK::Binary && g.nodes[add].op == "add" && g.nodes[add].ty.dims == d.ty.dims && g.nodes[add].ty.dt == d.ty.dt) {
        const Node& an = g.nodes[add];
        const int other = an.in[0] == dot ? an.in[1] : an.in[0];
        const Node& bn = g.nodes[other];
        if (other != dot && bn.k == OpK::BroadcastInDim && !mat[other] && bn.a0.size() == 1 && bn.a0[0] == n - 1 && mat[bn.in[0]] && g.nodes[bn.in[0]].ty.rank() == 1 &&
            g.nodes[bn.in[0]].ty.dims[0] == d.ty.dims[n - 1] && g.nodes[bn.in[0]].ty.dt == d.ty.dt) {
          init_add = add;
          init_vec = bn.in[0];
        }
      }
    }
    if (init_add >= 0) em.bound[init_add] = "accv";
    em.bound[dot] = "accv";
    std::string val = root == dot ? std::string("accv") : em.emit(root, root_index(rn.ty.dims));
    std::string ebody = em.take_code();
    const int init_slot = init_vec >= 0 ? em.slot_of(init_vec) : -1;
    const std::string ACC = is_float(d.ty.dt) ? (d.ty.dt == DT::F64 ? "double" : "float") : info(d.ty.dt).ctype;

    std::ostringstream o;
    // operand functors: element (row, column) of the operand as it would be stored, evaluated from the fused cone
    GemmOperandFn fn_a, fn_b;
    std::vector<int> in_a, in_b;
    auto make_operand_fn = [&](int side, GemmOperandFn& fn, std::vector<int>& inputs) {
      const int x = d.in[side];
      const TType& xt = g.nodes[x].ty;
      Emitter e(g, [&](int y) { return mat[y] != 0; });
      e.excess_precision = opt.excess_precision;
      e.idx64 = needs64(cone_nodes(x));
      e.set_root({}, {}, false);
      e.indent = 4;
      const std::string eit = e.idx_t();
      const int nbd = (int)d.a0.size();
      Index ix(xt.rank());
      for (int k = 0; k < xt.rank(); ++k) {
        ix[k].var = k < nbd ? "ob" : (k == nbd ? "r" : "c");
        ix[k].hi = xt.dims[k] - 1;
      }
      const std::string v = e.emit(x, ix);
      const std::string code = e.take_code();
      inputs = e.inputs;
      const std::string tag = side == 0 ? "opa" : "opb";
      const std::string E = info(xt.dt).stype;
      o << "// dot operand " << (side == 0 ? "A" : "B") << " computed on the fly: " << describe(x) << "\n";
      o << "struct " << kbase << "_" << tag << " {\n  static constexpr bool none = false;\n";
      for (size_t k = 0; k < inputs.size(); ++k) o << "  const " << info(g.nodes[inputs[k]].ty.dt).stype << "* __restrict__ in" << k << ";\n";
      o << "  __device__ __forceinline__ " << E << " operator()(long long ob_, int r_, int c_) const {\n";
      o << "    const " << eit << " ob = (" << eit << ")ob_, r = (" << eit << ")r_, c = (" << eit << ")c_;\n    (void)ob;\n";
      o << code;
      o << "    return " << e.store_value(xt.dt, v) << ";\n  }\n";
      // The same for a whole 16-byte vector of consecutive columns starting at a multiple of the vector width: the
      // index arithmetic that does not depend on the lane (the splitting of row and column numbers into the operand's
      // own coordinates) is written once per lane in the text but on the same expressions, so it is computed once.
      const int VE = 16 / (int)info(xt.dt).size;
      const int64_t minor = xt.dims[xt.rank() - 1];
      if (VE > 1 && minor % VE == 0 && xt.rank() == nbd + 2) {
        Emitter ev(g, [&](int y) { return mat[y] != 0; });
        ev.excess_precision = opt.excess_precision;
        ev.idx64 = e.idx64;
        ev.set_root({}, {}, false);
        ev.indent = 4;
        ev.inputs = e.inputs;
        std::vector<std::string> vals;
        for (int l = 0; l < VE; ++l) {
          Index il = ix;
          il[xt.rank() - 1].off = l;
          il[xt.rank() - 1].align = VE;
          il[xt.rank() - 1].hi = xt.dims[xt.rank() - 1] - 1;
          vals.push_back(ev.store_value(xt.dt, ev.emit(x, il)));
        }
        if (ev.inputs == e.inputs) {
          o << "  static constexpr int vec_width = " << VE << ";\n";
          o << "  __device__ __forceinline__ void vec(long long ob_, int r_, int c_, " << E << "* out) const {\n";
          o << "    const " << eit << " ob = (" << eit << ")ob_, r = (" << eit << ")r_, c = (" << eit << ")c_;\n    (void)ob;\n";
          o << ev.take_code();
          for (int l = 0; l < VE; ++l) o << "    out[" << l << "] = " << vals[l] << ";\n";
          o << "  }\n";
        } else {
          o << "  static constexpr int vec_width = 0;\n";
        }
      } else {
        o << "  static constexpr int vec_width = 0;\n";
      }
      o << "};\n\n";
      fn.type = kbase + "_" + tag;
      fn.ctor = fn.type + " " + (side == 0 ? "la" : "lb") + "{";
      for (size_t k = 0; k < inputs.size(); ++k) {
        const std::string pn = (side == 0 ? "fa" : "fb") + std::to_string(k);
        fn.params += ", const " + std::string(info(g.nodes[inputs[k]].ty.dt).stype) + "* __restrict__ " + pn;
        fn.ctor += (k ? ", " : "") + pn;
      }
      fn.ctor += "};";
    };
    if (fuse_a) make_operand_fn(0, fn_a, in_a);
    if (fuse_b) make_operand_fn(1, fn_b, in_b);
    o << "// dot epilogue: " << describe(root) << "\n";
    o << "struct " << kbase << "_epi {\n";
    for (size_t k = 0; k < em.inputs.size(); ++k)
      o << "  const " << info(g.nodes[em.inputs[k]].ty.dt).stype << "* __restrict__ in" << k << ";\n";
    const std::string ost = info(rn.ty.dt).stype;
    o << "  " << ost << "* __restrict__ out0;\n";
    if (init_slot >= 0) {
      o << "  static constexpr bool has_init = true;\n";
      o << "  template <int NV>\n  __device__ __forceinline__ void init(float (&v)[NV], int n) const {\n";
      o << "#pragma unroll\n    for (int l = 0; l < NV; ++l) v[l] = (float)" << em.load_conv(d.ty.dt, "in" + std::to_string(init_slot) + "[rx_min<int>(n + l, " + std::to_string(d.ty.dims[n - 1] - 1) + ")]") << ";\n";
      o << "  }\n";
    }
    o << "  template <int NV>\n  __device__ __forceinline__ void operator()(const " << ACC << " (&acc)[NV]";
    for (int k = 0; k < n; ++k) o << ", " << it << " i" << k << (k == n - 1 ? "b" : "");
    o << ") const {\n";
    {
      Index rix = root_index(rn.ty.dims);
      if (n > 0) rix[n - 1].var = "i" + std::to_string(n - 1) + "b";
      o << "    const " << it << " lin0 = " << (n ? em.linear(rix, rn.ty.dims) : std::string("0")) << ";\n";
    }
    for (auto& sd : em.direct_vecs) {
      const int slot = sd.first;
      const std::string st = info(g.nodes[em.inputs[slot]].ty.dt).stype;
      o << "    const rx_vec<" << st << ", NV> d" << slot << " = *reinterpret_cast<const rx_vec<" << st << ", NV>*>(in" << slot << " + lin0);\n";
    }
    o << "    rx_vec<" << ost << ", NV> res;\n";
    o << "#pragma unroll\n    for (int l = 0; l < NV; ++l) {\n";
    if (n > 0) o << "      const " << it << " i" << n - 1 << " = i" << n - 1 << "b + l;\n";
    {
      std::string accv = (is_narrow_float(d.ty.dt) && !(opt.excess_precision && root != dot)) ? Emitter::round_narrow(d.ty.dt, "acc[l]") : std::string("(") + DCT + ")acc[l]";
      o << "      const " << DCT << " accv = " << accv << ";\n";
    }
    o << ebody;
    o << "      res.v[l] = " << em.store_value(rn.ty.dt, val) << ";\n    }\n";
    o << "    *reinterpret_cast<rx_vec<" << ost << ", NV>*>(out0 + lin0) = res;\n";
    o << "  }\n};\n\n";

    std::vector<int> epi_inputs = em.inputs;
    Launch L;
    {
      double kprod = 1;
      for (auto c : d.a2) kprod *= (double)lt.dims[c];
      L.flops = 2.0 * (double)d.ty.numel() * kprod / (double)(d.a4.empty() ? 1 : d.a4[0]);
    }
    std::vector<int> all_in;
    if (fuse_a) all_in.insert(all_in.end(), in_a.begin(), in_a.end()); else all_in.push_back(d.in[0]);
    if (fuse_b) all_in.insert(all_in.end(), in_b.begin(), in_b.end()); else all_in.push_back(d.in[1]);
    for (int i : epi_inputs) if (std::find(all_in.begin(), all_in.end(), i) == all_in.end()) all_in.push_back(i);
    L.algo_bytes = algo_bytes(all_in, {root});
    L.desc = describe(root);

    auto epi_ctor = [&]() {
      std::string s = kbase + "_epi epi{";
      for (size_t k = 0; k < epi_inputs.size(); ++k) s += "in" + std::to_string(k) + ", ";
      return s + "out0};";
    };
    auto epi_params = [&]() {
      std::string s;
      for (size_t k = 0; k < epi_inputs.size(); ++k) s += ", const " + std::string(info(g.nodes[epi_inputs[k]].ty.dt).stype) + "* __restrict__ in" + std::to_string(k);
      return s + ", " + ost + "* __restrict__ out0";
    };

    if (gc.ok) {
      o << gemm_instance(gc, kbase, epi_params(), epi_ctor(), d.a0.size() == 1, fn_a, fn_b);
      L.kernel = kbase + "_gemm";
      L.kind = gc.kind;
      L.grid[0] = gc.grid[0]; L.grid[1] = gc.grid[1]; L.grid[2] = gc.grid[2];
      L.block[0] = gc.block;
      L.lds_bytes = gc.lds_bytes;
    } else {
      // scalar contraction: one thread per output element; any dims, any element type
      const int64_t nout = d.ty.numel();
      o << "// dot_general (scalar loop) " << lt.str() << " x " << rt.str() << "\n";
      o << "extern \"C\" __global__ __launch_bounds__(" << kBlock << ") void " << kbase << "_dot(const " << info(lt.dt).stype << "* __restrict__ A, const "
        << info(rt.dt).stype << "* __restrict__ B" << epi_params() << ") {\n";
      o << "  const " << it << " oid = (" << it << ")blockIdx.x * " << kBlock << " + threadIdx.x;\n";
      o << "  if (oid >= " << nout << ") return;\n";
      std::vector<int> lfree, rfree;
      auto isin = [](const std::vector<int64_t>& v, int x) { return std::find(v.begin(), v.end(), (int64_t)x) != v.end(); };
      for (int k = 0; k < lt.rank(); ++k) if (!isin(d.a0, k) && !isin(d.a2, k)) lfree.push_back(k);
      for (int k = 0; k < rt.rank(); ++k) if (!isin(d.a1, k) && !isin(d.a3, k)) rfree.push_back(k);
      o << "  " << it << " rr = oid;\n";
      for (int k = d.ty.rank() - 1; k >= 0; --k) {
        o << "  const " << it << " i" << k << " = rr % " << d.ty.dims[k] << ";\n";
        o << "  rr /= " << d.ty.dims[k] << ";\n";
      }
      std::vector<std::string> li(lt.rank()), ri(rt.rank());
      int od = 0;
      for (size_t k = 0; k < d.a0.size(); ++k, ++od) { li[d.a0[k]] = "i" + std::to_string(od); ri[d.a1[k]] = "i" + std::to_string(od); }
      for (int k : lfree) li[k] = "i" + std::to_string(od++);
      for (int k : rfree) ri[k] = "i" + std::to_string(od++);
      for (size_t k = 0; k < d.a2.size(); ++k) { li[d.a2[k]] = "k" + std::to_string(k); ri[d.a3[k]] = "k" + std::to_string(k); }
      auto lin = [&](const std::vector<std::string>& ixs, const std::vector<int64_t>& dims) {
        std::string s2 = "0";
        int64_t stride = 1;
        for (int k = (int)dims.size() - 1; k >= 0; --k) {
          s2 += " + (" + it + ")" + ixs[k] + " * " + std::to_string(stride);
          stride *= dims[k];
        }
        return s2;
      };
      o << "  " << ACC << " acc[1] = {0};\n";
      for (size_t k = 0; k < d.a2.size(); ++k)
        o << "  for (" << it << " k" << k << " = 0; k" << k << " < " << lt.dims[d.a2[k]] << "; ++k" << k << ")\n";
      Emitter tmp(g, [](int) { return true; });
      o << "    acc[0] += (" << ACC << ")" << tmp.load_conv(lt.dt, "A[" + lin(li, lt.dims) + "]") << " * (" << ACC << ")"
        << tmp.load_conv(rt.dt, "B[" + lin(ri, rt.dims) + "]") << ";\n";
      o << "  " << epi_ctor() << "\n";
      o << "  epi(acc";
      for (int k = 0; k < n; ++k) o << ", i" << k;
      o << ");\n}\n\n";
      L.kernel = kbase + "_dot";
      L.kind = "dot_scalar";
      L.grid[0] = (unsigned)((nout + kBlock - 1) / kBlock);
      L.block[0] = kBlock;
    }
    const std::string kb_final = finalize(o.str());
    L.kernel = named(L.kernel, kb_final);
    if (!fuse_a) L.args.push_back(buffer_for(d.in[0]));
    if (!fuse_b) L.args.push_back(buffer_for(d.in[1]));
    for (int i : in_a) L.args.push_back(buffer_for(i));
    for (int i : in_b) L.args.push_back(buffer_for(i));
    for (int i : epi_inputs) L.args.push_back(buffer_for(i));
    L.args.push_back(buffer_for(root));
    plan.launches.push_back(L);
  }

  // ------------------------------------------------------------------ driver
  void run() {
    const bool timing = getenv("RX_PLAN_TIMING") != nullptr;
    auto t_prev = std::chrono::steady_clock::now();
    auto lap = [&](const char* what) {
      if (!timing) return;
      auto t = std::chrono::steady_clock::now();
      fprintf(stderr, "[plan] %s: %.3f s\n", what, std::chrono::duration<double>(t - t_prev).count());
      t_prev = t;
    };
    canonicalize();
    lap("canonicalize");
    decide_fused_operands();
    lap("decide_fused_operands");
    const int N = (int)g.nodes.size();
    // Decisions about a node depend on which of its producers own buffers; sweep until stable.
    prev_mat.assign(N, 0);
    for (int sweep = 0; sweep < 6; ++sweep) {
      analyze();
      if (mat == prev_mat) break;
      prev_mat = mat;
    }
    lap("analysis sweeps");
    buf_of.assign(N, -1);
    plan.aliasing_output = g.aliasing_output;
    for (int p : g.params) { plan.param_types.push_back(g.nodes[p].ty); buffer_for(p); }

    // dot epilogues: an elementwise root that consumes a dot result at the identity index
    epilogue_of.clear();
    for (int x = 0; x < N && opt.product_epilogues; ++x) {
      if (!live[x] || (g.nodes[x].k != OpK::DotGeneral && g.nodes[x].k != OpK::Conv)) continue;
      if (std::find(g.results.begin(), g.results.end(), x) != g.results.end()) continue;
      if (ctx[x].size() != 1) continue;
      const Ctx& c = *ctx[x].begin();
      if (!c.second.empty()) continue;
      const Node& r = g.nodes[c.first];
      if (r.k == OpK::Reduce || r.k == OpK::Scan || r.k == OpK::Scatter || r.k == OpK::Conv || r.k == OpK::DotGeneral) continue;
      if (r.ty.dims != g.nodes[x].ty.dims) continue;
      // the root must not be the anchor of a row group (its reductions need the full row)
      if (!row_phases(c.first).empty()) continue;
      // a root takes one product into its kernel; a second one feeding the same root (A*B' + B*A') runs
      // on its own and is read back as an input
      bool taken = false;
      for (auto& kv : epilogue_of) taken = taken || kv.second == c.first;
      if (taken) continue;
      epilogue_of[x] = c.first;
    }
    std::set<int> absorbed_roots;
    for (auto& kv : epilogue_of) absorbed_roots.insert(kv.second);
    std::set<int> fused_reduces;

    // A reshape that must own a buffer and reads a value that owns one is the same bytes in the same
    // (row-major) order: it shares that buffer and costs no launch.  A result may share only a
    // temporary of this module that nothing else returns.
    {
      std::vector<char> is_result(N, 0);
      for (int r : g.results) is_result[r] = 1;
      std::set<int> returned_bases;
      for (int x = 0; x < N; ++x) {
        if (!live[x] || !mat[x]) continue;
        const Node& n = g.nodes[x];
        if (n.k != OpK::Reshape || absorbed_roots.count(x)) continue;
        int base = n.in[0];
        if (!mat[base]) continue;
        while (reshape_alias.count(base)) base = reshape_alias[base];
        if (is_result[x]) {
          const Node& bn = g.nodes[base];
          if (bn.k == OpK::Param || bn.k == OpK::Constant || is_result[base] || returned_bases.count(base)) continue;
          returned_bases.insert(base);
        }
        reshape_alias[x] = base;
      }
    }

    lap("epilogues and aliases");
    // kernels in topological order of their roots
    std::vector<std::pair<int, std::function<void()>>> jobs;
    for (int x = 0; x < N; ++x) {
      if (!live[x] || !mat[x]) continue;
      const Node& n = g.nodes[x];
      if (n.k == OpK::Param || (n.k == OpK::Constant && !n.splat)) continue;
      if (n.k == OpK::DotGeneral) {
        auto e = epilogue_of.find(x);
        if (e != epilogue_of.end()) continue;  // emitted with its root
        jobs.push_back({x, [this, x] { emit_dot(x, x); }});
        continue;
      }
      if (absorbed_roots.count(x)) {
        int dot = -1;
        for (auto& kv : epilogue_of) if (kv.second == x) dot = kv.first;
        if (g.nodes[dot].k == OpK::Conv) jobs.push_back({x, [this, x, dot] { emit_conv(x, dot); }});
        else jobs.push_back({x, [this, x, dot] { emit_dot(x, dot); }});
        continue;
      }
      if (n.k == OpK::Scan) {
        jobs.push_back({x, [this, x] { emit_scan(x); }});
        continue;
      }
      if (n.k == OpK::Scatter) {
        jobs.push_back({x, [this, x] { emit_scatter(x); }});
        continue;
      }
      if (n.k == OpK::Conv) {
        if (epilogue_of.count(x)) continue;  // emitted with its root
        jobs.push_back({x, [this, x] { emit_conv(x, x); }});
        continue;
      }
      if (reshape_alias.count(x)) continue;
      if (n.k == OpK::Reduce) {
        jobs.push_back({x, [this, x, &fused_reduces] {
          if (fused_reduces.count(x)) return;
          const Node& r = g.nodes[x];
          RedShape rs = red_shape(r);
          if (g.nodes[r.in[0]].ty.numel() == 0 || r.ty.numel() == 0) { emit_reduce_generic(x); return; }
          if (rs.nkeep == 0) { emit_reduce_full(x); return; }
          if (rs.trailing && rs.cols >= 64) { emit_row(x, {x}); return; }
          emit_reduce_generic(x);
        }});
        continue;
      }
      jobs.push_back({x, [this, x, &fused_reduces] {
        std::vector<int> ph = row_phases(x);
        if (!ph.empty()) {
          for (int p : ph) fused_reduces.insert(p);
          emit_row(x, ph);
        } else emit_map(x);
      }});
    }
    // Two consecutive stencil steps share a kernel when the first step has no other reader.
    if (opt.stencil_fuse_steps) {
      std::vector<char> is_result(N, 0);
      for (int r : g.results) is_result[r] = 1;
      auto plain_map_root = [&](int x) {
        const Node& n = g.nodes[x];
        if (!live[x] || !mat[x]) return false;
        if (n.k == OpK::Param || n.k == OpK::Constant || n.k == OpK::Reduce || n.k == OpK::Scan || n.k == OpK::Scatter || n.k == OpK::Conv || n.k == OpK::DotGeneral) return false;
        if (reshape_alias.count(x)) return false;
        if (absorbed_roots.count(x) || !row_phases(x).empty()) return false;
        return true;
      };
      for (int x = 0; x < N; ++x) {
        if (!plain_map_root(x)) continue;
        StencilProbe sp;
        if (!probe_stencil(x, &sp) || sp.staged.size() != 1) continue;
        const int s = sp.staged[0];
        if (!plain_map_root(s) || is_result[s] || lds_only.count(s) || fuse_prev.count(s)) continue;
        bool only = !ctx[s].empty();
        for (auto& c : ctx[s]) only = only && c.first == x;
        if (!only) continue;
        StencilProbe sq;
        if (!probe_stencil(s, &sq) || sq.staged.size() != 1) continue;
        fuse_prev[x] = s;
        lds_only.insert(s);
      }
    }
    // Runs of update steps over small arrays share chain kernels.
    if (opt.chain_steps == 0 || opt.chain_steps >= 2) {
      std::vector<char> is_result(N, 0);
      for (int r : g.results) is_result[r] = 1;
      size_t i = 0;
      while (i < jobs.size()) {
        std::vector<int> steps;
        std::vector<ChainProbe> probes;
        std::set<int> group;
        std::map<int, int> field_of;
        std::vector<int> cur;
        for (size_t j = i; j < jobs.size() && (steps.empty() || steps.size() < (size_t)chain_cap(g.nodes[steps[0]].ty.rank())); ++j) {
          const int x = jobs[j].first;
          if (absorbed_roots.count(x) || reshape_alias.count(x) || !row_phases(x).empty()) break;
          ChainProbe q;
          if (!probe_chain_step(x, &q)) break;
          if (!steps.empty() && !(g.nodes[x].ty == g.nodes[steps[0]].ty)) break;
          bool ok = true;
          // what a step reads is either outside the kernel or the latest version of a field
          for (auto& kv : q.reads) ok = ok && (!group.count(kv.first) || cur[field_of[kv.first]] == kv.first);
          for (int y : q.others) ok = ok && !group.count(y);
          // a version superseded inside the kernel exists nowhere else
          if (ok && group.count(q.base)) ok = !is_result[q.base] && read_only_by(q.base, group, x);
          if (!ok) break;
          for (auto& kv : q.reads)
            if (!field_of.count(kv.first)) { field_of[kv.first] = (int)cur.size(); cur.push_back(kv.first); }
          const int fw = field_of[q.base];
          field_of[x] = fw;
          cur[fw] = x;
          group.insert(x);
          steps.push_back(x);
          probes.push_back(q);
        }
        if (getenv("RX_CHAIN_DEBUG")) fprintf(stderr, "[chain] job %zu (node %d, %s): run of %zu steps\n", i, jobs[i].first, g.nodes[jobs[i].first].ty.str().c_str(), steps.size());
        if (steps.size() < 2) { ++i; continue; }
        chain_at[steps[0]] = steps;
        auto plain0 = jobs[i].second;
        jobs[i].second = [this, steps, probes, plain0] {
          size_t at = 0;
          while (steps.size() - at >= 2) {
            const size_t used = emit_chain(std::vector<int>(steps.begin() + at, steps.end()), std::vector<ChainProbe>(probes.begin() + at, probes.end()));
            if (!used) break;
            for (size_t q = 0; q < used; ++q) chain_member.insert(steps[at + q]);
            at += used;
          }
          if (!chain_member.count(steps[0])) plain0();
        };
        for (size_t q = 1; q < steps.size(); ++q) {
          auto plain = jobs[i + q].second;
          const int x = steps[q];
          jobs[i + q].second = [this, x, plain] { if (!chain_member.count(x)) plain(); };
        }
        i += steps.size();
      }
    }
    // row groups claim their reductions before those would be emitted on their own
    for (auto& j : jobs) {
      const Node& n = g.nodes[j.first];
      if (n.k != OpK::Reduce && n.k != OpK::Scan && n.k != OpK::Scatter && n.k != OpK::Conv && n.k != OpK::DotGeneral && !absorbed_roots.count(j.first))
        for (int p : row_phases(j.first)) { fused_reduces.insert(p); row_anchor[p] = j.first; }
    }
    lap("job list, chains");
    for (auto& j : jobs) j.second();
    lap("emit");

    for (int r : g.results) {
      plan.result_types.push_back(g.nodes[r].ty);
      int b = buffer_for(r);
      plan.buffers[b].is_result = true;
      plan.result_buffers.push_back(b);
    }
    merge_parameter_maps();
    // liveness over the launch list
    for (size_t li = 0; li < plan.launches.size(); ++li) {
      auto& L = plan.launches[li];
      for (int b : L.args) {
        auto& B = plan.buffers[b];
        if (B.first_def < 0) B.first_def = (int)li;
        B.last_use = (int)li;
      }
    }
    plan.source = "#include \"rx_preamble.h\"\n#include \"rx_gemm_kernels.h\"\n\n" + src.str();
  }
};

}  // namespace

std::string Plan::report() const {
  std::ostringstream o;
  o << "buffers: " << buffers.size() << ", launches: " << launches.size() << "\n";
  for (size_t i = 0; i < launches.size(); ++i) {
    auto& L = launches[i];
    o << "  [" << i << "] " << L.kernel << " kind=" << L.kind << " grid=" << L.grid[0] << "x" << L.grid[1] << "x" << L.grid[2] << " block=" << L.block[0]
      << " lds=" << L.lds_bytes << " algo_bytes=" << (long long)L.algo_bytes << " flops=" << (long long)L.flops << " :: " << L.desc << "\n";
  }
  o << "module costs: flops=" << (long long)hlo_flops << " transcendentals=" << (long long)hlo_transcendentals << " bytes_accessed=" << (long long)hlo_bytes_accessed
    << " output_bytes=" << (long long)hlo_output_bytes << "\n";
  return o.str();
}

// Operation counts of the module as written, in the conventions of XLA's HloCostAnalysis: a product counts 2 M N K,
// every other arithmetic op one operation per result element (a reduction one per reduced element), transcendental ops
// are counted apart, and every op reads its operands and writes its result once.
static void count_hlo_costs(const Graph& g, Plan* plan) {
  const size_t N = g.nodes.size();
  std::vector<char> live(N, 0);
  std::vector<int> stack(g.results.begin(), g.results.end());
  while (!stack.empty()) {
    const int x = stack.back();
    stack.pop_back();
    if (live[x]) continue;
    live[x] = 1;
    for (int i : g.nodes[x].in) stack.push_back(i);
  }
  static const char* const kTrans[] = {"exponential", "exponential_minus_one", "log", "log_plus_one", "logistic", "tanh", "sine", "cosine", "tan",
                                       "rsqrt", "sqrt", "cbrt", "erf", "power", "atan2"};
  double flops = 0, trans = 0, bytes = 0;
  for (size_t x = 0; x < N; ++x) {
    if (!live[x]) continue;
    const Node& n = g.nodes[x];
    const double numel = (double)n.ty.numel();
    bool is_trans = n.k == OpK::Gelu;
    for (const char* t : kTrans) is_trans = is_trans || n.op == t;
    switch (n.k) {
      case OpK::Param: case OpK::Constant: case OpK::Iota: break;
      case OpK::DotGeneral: {
        double kk = 1;
        for (int64_t d : n.a2) kk *= (double)g.nodes[n.in[0]].ty.dims[d];
        flops += 2.0 * numel * kk;
        break;
      }
      case OpK::Conv: {
        const TType& wt = g.nodes[n.in[1]].ty;
        flops += 2.0 * numel * (double)(wt.rank() == 2 ? wt.dims[1] : wt.dims[1] * wt.dims[2] * wt.dims[3]);
        break;
      }
      case OpK::Reduce: case OpK::Scan: flops += (double)g.nodes[n.in[0]].ty.numel(); break;
      case OpK::Unary: case OpK::Binary: case OpK::Gelu:
        if (is_trans) trans += numel; else flops += numel;
        break;
      case OpK::Compare: case OpK::Select: case OpK::Clamp: case OpK::Scatter: flops += numel; break;
      default: break;   // data movement
    }
    if (n.k != OpK::Param && n.k != OpK::Constant) {
      bytes += (double)n.ty.bytes();
      for (int i : n.in) bytes += (double)g.nodes[i].ty.bytes();
    }
  }
  plan->hlo_flops = flops;
  plan->hlo_transcendentals = trans;
  plan->hlo_bytes_accessed = bytes;
  for (size_t k = 0; k < 2 && k < g.params.size(); ++k) plan->hlo_operand_bytes[k] = (double)g.nodes[g.params[k]].ty.bytes();
  for (int r : g.results) plan->hlo_output_bytes += (double)g.nodes[r].ty.bytes();
}

Plan make_plan(const Graph& g, const PlanOptions& opt) {
  try {
    Planner p(g, opt);
    p.run();
    count_hlo_costs(g, &p.plan);
    return std::move(p.plan);
  } catch (const ChainNotAbsorbed&) {
    PlanOptions plain = opt;
    plain.chain_convs = false;
    return make_plan(g, plain);
  }
}

}  // namespace rx
