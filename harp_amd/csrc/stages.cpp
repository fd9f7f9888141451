// Canonical stages of the elementwise / reduce schedules, how kernels are grouped into them, and
// the helpers that describe a kernel's output layout and fold a gather into its reader.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <mutex>
#include <set>
#include <sstream>

#include "codegen_parts.hpp"

namespace eh {

// ---------------------------------------------------------------------------------------------
// canonical stages and grouping
// ---------------------------------------------------------------------------------------------





NodePtr rename(const NodePtr& n, const std::map<std::string, NodePtr>& m) {
  if (n->op == Op::Var) {
    auto it = m.find(n->name);
    return it == m.end() ? n : it->second;
  }
  bool changed = false;
  std::vector<NodePtr> args;
  args.reserve(n->args.size());
  for (const auto& a : n->args) {
    NodePtr r = rename(a, m);
    changed = changed || r != a;
    args.push_back(std::move(r));
  }
  if (!changed) return n;
  auto c = std::make_shared<Node>(*n);
  c->args = std::move(args);
  return c;
}

// Canonical form of a kernel: `nrows` of its non-trivial loops are rows, then (for Wide) one
// column loop; a reduce kernel's column is its reduce loop.
bool canonicalise(const NestKernel& k, StageKind kind, std::vector<int64_t>* rows, int64_t* C, Stage* out) {
  std::vector<Loop> live;
  std::map<std::string, NodePtr> m;
  for (const auto& l : k.loops) {
    if (l.extent == 0) return false;
    if (l.extent == 1) m[l.var] = make_i64(0);
    else live.push_back(l);
  }
  rows->clear();
  size_t nrow = live.size();
  if (kind == StageKind::Wide) {
    if (live.empty()) {
      *C = 1;
    } else {
      nrow = live.size() - 1;
      *C = live.back().extent;
      m[live.back().var] = make_var("c");
    }
  } else if (kind == StageKind::Reduce) {
    if (k.rloop.extent == 0) return false;
    *C = k.rloop.extent;
    m[k.rloop.var] = k.rloop.extent == 1 ? make_i64(0) : make_var("c");
  }
  for (size_t i = 0; i < nrow; ++i) {
    rows->push_back(live[i].extent);
    m[live[i].var] = make_var("r" + std::to_string(i));
  }
  out->kind = kind;
  out->kname = k.name;
  out->value = rename(k.value, m);
  out->rk = k.rkind;
  out->identity = k.identity;
  out->acc_dtype = k.acc_dtype;
  out->out_buf = k.out_buf;
  out->out_dtype = k.out_dtype;
  auto oa = affine_of(*rename(k.out_index, m));
  if (!oa) return false;
  out->out_aff = *oa;
  return true;
}

// A reduce kernel is a row program candidate when its reduce loop walks memory contiguously
// for at least one operand (otherwise lanes along the loop would not coalesce).
bool reduce_is_rowwise(const NestKernel& k) {
  std::vector<LoadRef> loads;
  collect_loads(*k.value, loads);
  bool any_unit = false, any_dep = false;
  // the operand with the largest footprint decides when operands disagree (a vector times a
  // matrix: the vector is contiguous along the reduce axis, the matrix along the outputs)
  int64_t widest = 0;
  bool widest_unit = false;
  for (const auto& lr : loads) {
    auto a = affine_of(*lr.load->args[1]);
    if (!a) continue;
    int64_t c = a->of(k.rloop.var);
    if (c != 0) any_dep = true;
    if (c == 1 || c == -1) any_unit = true;
    if (c == 0) continue;
    int64_t foot = k.rloop.extent;
    for (const auto& l : k.loops)
      if (a->of(l.var) != 0) foot *= l.extent;
    const bool unit = c == 1 || c == -1;
    if (foot > widest || (foot == widest && unit)) { widest = foot; widest_unit = unit; }
  }
  if (!any_dep) return true;
  return any_unit && widest_unit;
}

// Loads of buffers produced inside the group must hit exactly the element the producer wrote.
bool aligned_with_group(const Group& g, const Stage& s) {
  std::vector<LoadRef> loads;
  collect_loads(*s.value, loads);
  for (const auto& lr : loads) {
    const Stage* p = g.producer(lr.load->args[0]->name);
    if (!p) continue;
    auto a = affine_of(*lr.load->args[1]);
    if (!a || !(*a == p->out_aff)) return false;
    if (s.kind == StageKind::Scalar && p->kind == StageKind::Wide) return false;
  }
  return true;
}


Canon canon_as(const NestKernel& k, StageKind kind) {
  Canon c;
  c.ok = canonicalise(k, kind, &c.rows, &c.C, &c.stage);
  return c;
}


// Row-major strides of a kernel's loops when its output index is exactly the dense linear index
// of those loops (coefficient of each live loop = product of the inner extents, no offset).
std::optional<std::vector<int64_t>> dense_strides(const NestKernel& k, int64_t* numel) {
  if (!k.out_aff || k.out_aff->c != 0) return std::nullopt;
  int64_t stride = 1;
  std::vector<int64_t> strides(k.loops.size(), 0);
  for (size_t i = k.loops.size(); i-- > 0;) {
    const Loop& l = k.loops[i];
    if (l.extent <= 0) return std::nullopt;
    strides[i] = stride;
    if (l.extent > 1 && k.out_aff->of(l.var) != stride) return std::nullopt;
    stride *= l.extent;
  }
  for (const auto& kv : k.out_aff->coef) {
    bool live = false;
    for (const auto& l : k.loops) live = live || l.var == kv.first;     // a loop that runs once adds nothing
    if (kv.second != 0 && !live) return std::nullopt;
  }
  *numel = stride;
  return strides;
}

std::string gather_fn_name(const std::string& buf) { return "eh_win_" + buf; }

// The arguments of gather g's function for the element at `index` of its dense output: one
// per loop of g, the digit (index / stride) % extent.  `index` is affine over the caller's
// loops, so most digits come out as one of those loops (or a constant after unrolling)
// without a division: terms whose coefficient is a multiple of stride * extent vanish,
// terms below the stride cannot carry when together they stay below it.
std::string gather_call(const NestKernel& g, const std::string& src, const Node& index, const std::vector<Loop>& caller,
                        const std::string& idx_type) {
  ExprRenderer plain;
  const std::string whole = "((" + idx_type + ")(" + plain.expr(index) + "))";
  auto a = affine_of(index);
  std::string args;
  // the index as a mixed-radix number over the caller's loops: coefficients ascending, each
  // above everything the smaller terms can add up to
  struct Term { int64_t c, ext; std::string var; };
  std::vector<Term> terms;
  bool nested = a.has_value() && a->c == 0;
  if (nested) {
    for (const auto& kv : a->coef) {
      if (kv.second == 0) continue;
      int64_t ext = 0;
      for (const auto& l : caller)
        if (l.var == kv.first) ext = l.extent;
      if (kv.second < 0 || ext <= 0) { nested = false; break; }
      if (ext > 1) terms.push_back({kv.second, ext, kv.first});
    }
    std::sort(terms.begin(), terms.end(), [](const Term& x, const Term& y) { return x.c < y.c; });
    int64_t reach = 0;
    for (const auto& t : terms) {
      if (t.c <= reach) { nested = false; break; }
      reach += t.c * (t.ext - 1);
    }
  }
  int64_t stride = 1;
  std::vector<std::string> digits(g.loops.size());
  for (size_t q = g.loops.size(); q-- > 0;) {
    const int64_t e = g.loops[q].extent;
    std::string d;
    if (e == 1) {
      d = "0";
    } else {
      bool symbolic = nested;
      int64_t dmax = 0;
      std::string sum;
      auto add = [&](const std::string& t, int64_t tmax) {
        sum += (sum.empty() ? "" : " + ") + t;
        dmax += tmax;
      };
      if (symbolic)
        for (const auto& t : terms) {
          if (t.c % (stride * e) == 0) continue;                       // vanishes modulo the extent
          if (t.c >= stride) {
            if (t.c % stride) { symbolic = false; break; }
            const int64_t m = t.c / stride;
            add(m == 1 ? t.var : t.var + " * " + std::to_string(m), m * (t.ext - 1));
          } else if (t.c * (t.ext - 1) >= stride) {                      // reaches into this digit from below
            if (stride % t.c) { symbolic = false; break; }
            const int64_t dv = stride / t.c;
            add("(" + t.var + " / " + std::to_string(dv) + ")", (t.ext - 1) / dv);
          }
        }
      if (symbolic) d = sum.empty() ? "0" : dmax < e ? "(" + sum + ")" : "((" + sum + ") % " + std::to_string(e) + ")";
      else d = "((" + whole + " / " + std::to_string(stride) + ") % " + std::to_string(e) + ")";
    }
    digits[q] = d;
    stride *= e;
  }
  for (const auto& d : digits) args += ", " + d;
  return gather_fn_name(g.out_buf) + "(" + src + args + ")";
}

// Gather g as a device function of its own loop variables; `inner`, when given, is the gather
// whose output g reads: that load becomes a call of inner's function.
std::string gather_fn_text(const NestKernel& g, const std::string& src, const NestKernel* inner, const std::string& idx_type) {
  std::ostringstream os;
  os << "// the element of what kernel " << g.name << " would have written, by its loop variables\n";
  os << "__device__ __forceinline__ float " << gather_fn_name(g.out_buf) << "(const float* __restrict__ " << src;
  for (const auto& l : g.loops) os << ", const " << idx_type << " " << l.var;
  os << ") {\n";
  ExprRenderer er;
  if (inner)
    er.load_hook = [&](const Node& ld, std::string* out) {
      if (ld.args[0]->op != Op::Var || ld.args[0]->name != inner->out_buf) return false;
      *out = gather_call(*inner, src, *ld.args[1], g.loops, idx_type);
      return true;
    };
  os << "  return (float)(" << er.expr(*g.value) << ");\n}\n";
  return os.str();
}

// An elementwise kernel as a function of the linear index of its (dense, row-major) output, for
// contractions that evaluate it in their tile loader.  Only kernels reading one f32 buffer.
std::optional<FoldedOperand> make_fold(const NestKernel& k, const std::map<std::string, size_t>& elems, bool computing) {
  if (k.rkind != ReduceKind::None || k.out_dtype.ty != Ty::F32 || !k.out_aff || k.out_aff->c != 0) return std::nullopt;
  int64_t stride = 1, numel = 1;
  std::vector<int64_t> strides(k.loops.size(), 0);
  size_t used = 0;
  for (size_t i = k.loops.size(); i-- > 0;) {
    const Loop& l = k.loops[i];
    if (l.extent <= 0) return std::nullopt;
    strides[i] = stride;
    if (l.extent > 1) {
      if (k.out_aff->of(l.var) != stride) return std::nullopt;
      ++used;
    }
    stride *= l.extent;
    numel *= l.extent;
  }
  for (const auto& kv : k.out_aff->coef) {
    bool live = false;
    for (const auto& l : k.loops) live = live || l.var == kv.first;     // a loop that runs once adds nothing
    if (kv.second != 0 && !live) return std::nullopt;
  }
  (void)used;
  std::vector<LoadRef> loads;
  collect_loads(*k.value, loads);
  if (loads.empty()) return std::nullopt;
  const std::string src = loads[0].load->args[0]->name;
  for (const auto& lr : loads) {
    if (lr.load->args[0]->op != Op::Var || lr.load->args[0]->name != src) return std::nullopt;
    if (lr.load->dtype.ty != Ty::F32 || lr.load->count != 1) return std::nullopt;
  }
  if (src == k.out_buf) return std::nullopt;
  // pure gathers only (a load, possibly under an index-only guard with a constant default):
  // anything that computes is cheaper done once than once per tile that reads it
  if (!computing) {
    const Node* v = k.value.get();
    if (v->op == Op::Select && v->args[2]->op == Op::Const) {
      std::vector<LoadRef> in_cond;
      collect_loads(*v->args[0], in_cond);
      if (!in_cond.empty()) return std::nullopt;
      v = v->args[1].get();
    }
    if (v->op != Op::Load) return std::nullopt;
  }
  auto it = elems.find(src);
  const bool small = it != elems.end() && it->second < (size_t{1} << 30) && numel < (int64_t{1} << 30);
  FoldedOperand f;
  f.src = src;
  f.kernel = k.name;
  f.small = small;
  f.src_bytes = it == elems.end() ? 0.0 : 4.0 * static_cast<double>(it->second);
  for (size_t i = 0; i < k.loops.size(); ++i) f.loops.push_back({k.loops[i].var, k.loops[i].extent, strides[i]});
  ExprRenderer er;
  std::map<std::string, size_t> ranged;
  if (g_ranged_loads && !g_guard_branches && small && it->second * 4 < (size_t{1} << 31)) {
    f.ranged_bytes = it->second * 4;
    ranged[src] = f.ranged_bytes;
    er.ranged = &ranged;
  }
  f.expr = er.expr(*k.value);
  f.value = k.value;
  if (auto a = affine_of(*loads[0].load->args[1])) {
    for (size_t i = 0; i < k.loops.size(); ++i)
      if (k.loops[i].extent > 1) f.src_stride[strides[i]] = a->of(k.loops[i].var);
    f.plain = k.value->op == Op::Load && loads.size() == 1;
    f.src_off = a->c;
  }
  return f;
}

// C of contraction `g` is dense; consumer `sk` (dense output) reads it at `read` (affine over
// sk's loops), a bijection between the two index spaces.  Returns g's output index rewritten
// so that each element lands at the consumer's own linear index, or nullopt when the consumer's
// loops do not regroup into g's loops.
std::optional<Affine> relayout(const NestKernel& g, const NestKernel& sk, const Affine& read) {
  if (read.c != 0 || !g.out_aff || !sk.out_aff) return std::nullopt;
  struct CV { int64_t read, out, extent; };
  std::vector<CV> cv;
  int64_t reach = 0;
  for (const auto& l : sk.loops) {
    if (l.extent <= 1) continue;
    int64_t r = read.of(l.var);
    if (r <= 0) return std::nullopt;
    cv.push_back({r, sk.out_aff->of(l.var), l.extent});
    reach += r * (l.extent - 1);
  }
  for (const auto& kv : read.coef) {
    bool live = false;
    for (const auto& l : sk.loops) live = live || l.var == kv.first;    // a loop that runs once adds nothing
    if (kv.second != 0 && !live) return std::nullopt;
  }
  std::sort(cv.begin(), cv.end(), [](const CV& a, const CV& b) { return a.read > b.read; });
  struct GV { std::string var; int64_t stride, extent; };
  std::vector<GV> gv;
  int64_t total = 1;
  for (const auto& l : g.loops) {
    if (l.extent <= 1) continue;
    gv.push_back({l.var, g.out_aff->of(l.var), l.extent});
    total *= l.extent;
  }
  if (reach != total - 1) return std::nullopt;
  std::sort(gv.begin(), gv.end(), [](const GV& a, const GV& b) { return a.stride > b.stride; });
  Affine out;
  size_t ci = 0;
  for (const auto& v : gv) {
    // consumer loops that together walk this loop of the contraction: same span of C, and
    // walking as one axis in the consumer's output too
    int64_t covered = 1;
    size_t first = ci;
    while (ci < cv.size() && covered < v.extent) {
      covered *= cv[ci].extent;
      ++ci;
    }
    if (covered != v.extent || ci == first) return std::nullopt;
    if (cv[ci - 1].read != v.stride) return std::nullopt;
    for (size_t q = first; q + 1 < ci; ++q)
      if (cv[q].read != cv[q + 1].read * cv[q + 1].extent || cv[q].out != cv[q + 1].out * cv[q + 1].extent)
        return std::nullopt;
    out.coef[v.var] = cv[ci - 1].out;
  }
  if (ci != cv.size()) return std::nullopt;
  return out;
}

}  // namespace eh
