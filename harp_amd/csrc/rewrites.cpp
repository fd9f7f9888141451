// Program-level rewrites: passes over the lowered kernels before any schedule is chosen.
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
// few, very long reduce lines: split over workgroups before planning
// ---------------------------------------------------------------------------------------------


NodePtr make_range(const std::string& var, int64_t extent, NodePtr body) {
  auto r = make(Op::Range, {make_i64(0), make_i64(1), make_i64(extent), std::move(body)});
  r->name = var;
  r->parallel = "sequential";
  return r;
}

NodePtr make_combine(ReduceKind k, const NodePtr& acc, const NodePtr& v) {
  switch (k) {
    case ReduceKind::Sum: return make(Op::Add, {acc, v});
    case ReduceKind::Prod: return make(Op::Mul, {acc, v});
    case ReduceKind::Max: return make(Op::Max, {acc, v});
    default: return make(Op::Select, {make(Op::Lt, {acc, v}), acc, v});     // min, as node.rs:63-77 writes it
  }
}

NodePtr make_kernel(const std::string& name, std::vector<Param> params, NodePtr body) {
  auto k = std::make_shared<Node>(Op::Kernel);
  k->name = name;
  k->params = std::move(params);
  k->args = {std::move(body)};
  for (int i = 0; i < 3; ++i) {
    k->grid.push_back(make_i64(1));
    k->tg.push_back(make_i64(1));
  }
  return k;
}

// acc = identity; for var in [0, extent): acc = combine(acc, value); out[index] = acc
static NodePtr make_reduce_block(const NestKernel& nk, const std::string& var, int64_t extent, const NodePtr& value,
                          const std::string& out_buf, const NodePtr& out_index) {
  auto acc = make_var("acc");
  auto init = make(Op::Assign, {nk.identity});
  init->name = "acc";
  auto step = make(Op::Assign, {make_combine(nk.rkind, acc, value)});
  step->name = "acc";
  auto store = make(Op::Store, {make_var(out_buf), out_index, acc});
  auto blk = make(Op::Block, {init, make_range(var, extent, step), store});
  blk->decls.push_back({"acc", nk.acc_dtype});
  return blk;
}


// A reduce whose lines are few and very long (a total over a whole tensor, a softmax over two
// rows of millions) would occupy a handful of workgroups.  Rewritten as two reduces -- every
// line cut into `chunks` pieces, then the pieces of a line combined -- both take the ordinary
// row schedule, the first with lines * chunks rows.  The combine order changes (reduction
// tolerance for sums and products, exact for max and min).
std::optional<RowSplit> split_long_rows(const NestKernel& nk) {
  if (nk.rkind == ReduceKind::None || !nk.out_aff) return std::nullopt;
  int64_t lines = 1;
  for (const auto& l : nk.loops) lines *= l.extent;
  const int64_t K = nk.rloop.extent;
  {
    // measured on MI355X: a workgroup streams its line at about 92 GB/s whatever the number of
    // lines (up to one per CU); the two launches cost about 5.5 us plus the traffic
    const double whole_us = 1.5 + double(K) * 4.0 / 92e3;
    const double cut_us = 5.5 + double(lines) * double(K) * 4.0 / 10e6;
    if (lines > 128 || K < (int64_t{1} << 17) || whole_us <= 1.2 * cut_us) return std::nullopt;
  }
  std::vector<LoadRef> loads;
  collect_loads(*nk.value, loads);
  bool unit = false;
  for (const auto& lr : loads) {
    auto a = affine_of(*lr.load->args[1]);
    if (!a || lr.load->args[0]->op != Op::Var) return std::nullopt;
    const int64_t c = a->of(nk.rloop.var);
    if (c != 0 && c != 1) return std::nullopt;
    unit = unit || c == 1;
  }
  if (!unit) return std::nullopt;
  int64_t chunks = 0;
  for (int64_t align : {4, 1}) {           // chunks that start on a 16-byte boundary first
    for (int64_t s = 4096 / lines; s >= 8 && !chunks; --s)
      if (K % (s * align) == 0 && K / s >= 4096) chunks = s;
  }
  if (!chunks) return std::nullopt;
  const int64_t CH = K / chunks;
  RowSplit rs;
  rs.scratch.name = "eh_rowpart_" + nk.name;
  rs.scratch.dtype = nk.acc_dtype;
  rs.scratch.shape = {lines * chunks};
  rs.scratch.role = "temp";
  // position of a line among the lines (row-major over the outer loops)
  NodePtr line = make_i64(0);
  for (const auto& l : nk.loops) line = make(Op::Add, {make(Op::Mul, {line, make_i64(l.extent)}), make_var(l.var)});
  const std::string sv = "eh_chunk", kv = "eh_k";
  auto part_index = make(Op::Add, {make(Op::Mul, {line, make_i64(chunks)}), make_var(sv)});
  DType pt;
  pt.ty = Ty::Ptr;
  pt.inner = std::make_shared<DType>(nk.acc_dtype);
  {
    // value with the reduce variable replaced by chunk * CH + k
    NodePtr pos = make(Op::Add, {make(Op::Mul, {make_var(sv), make_i64(CH)}), make_var(kv)});
    NodePtr value = rename(nk.value, {{nk.rloop.var, pos}});
    NodePtr body = make_range(sv, chunks, make_reduce_block(nk, kv, CH, value, rs.scratch.name, part_index));
    for (size_t i = nk.loops.size(); i-- > 0;) body = make_range(nk.loops[i].var, nk.loops[i].extent, body);
    std::vector<Param> params;
    for (const auto& p : nk.params)
      if (!p.mut_) params.push_back(p);
    Param sp;
    sp.name = rs.scratch.name;
    sp.dtype = pt;
    sp.mut_ = true;
    params.push_back(sp);
    rs.part = make_kernel(nk.name + "_rows", params, body);
  }
  {
    auto ld = make(Op::Load, {make_var(rs.scratch.name), part_index});
    ld->dtype = nk.acc_dtype;
    NodePtr body = make_reduce_block(nk, sv, chunks, ld, nk.out_buf, nk.out_index);
    for (size_t i = nk.loops.size(); i-- > 0;) body = make_range(nk.loops[i].var, nk.loops[i].extent, body);
    std::vector<Param> params;
    Param sp;
    sp.name = rs.scratch.name;
    sp.dtype = pt;
    params.push_back(sp);
    for (const auto& p : nk.params)
      if (p.mut_) params.push_back(p);
    rs.final_ = make_kernel(nk.name, params, body);
  }
  return rs;
}


// ---------------------------------------------------------------------------------------------
// a value an earlier kernel already stored is read back instead of being computed again
// ---------------------------------------------------------------------------------------------

// Structural equality of `s` (over S's loop variables) and `r` (over R's) under a one-to-one
// renaming of loop variables, which is built up in `map` as the trees are walked.
static bool same_under_renaming(const Node& s, const Node& r, const std::set<std::string>& s_vars, const std::set<std::string>& r_vars,
                         std::map<std::string, std::string>* map) {
  if (s.op != r.op || s.args.size() != r.args.size()) return false;
  if (s.op == Op::Var) {
    const bool sv = s_vars.count(s.name) != 0, rv = r_vars.count(r.name) != 0;
    if (sv != rv) return false;
    if (!sv) return s.name == r.name;
    auto it = map->find(s.name);
    if (it != map->end()) return it->second == r.name;
    for (const auto& kv : *map)
      if (kv.second == r.name) return false;
    (*map)[s.name] = r.name;
    return true;
  }
  if (s.op == Op::Const) return s.dtype.ty == r.dtype.ty && s.ival == r.ival && std::memcmp(&s.fval, &r.fval, sizeof s.fval) == 0;
  if (s.name != r.name || s.count != r.count) return false;
  if ((s.op == Op::Cast || s.op == Op::Load) && s.dtype.ty != r.dtype.ty) return false;
  for (size_t i = 0; i < s.args.size(); ++i) {
    if (!s.args[i] || !r.args[i]) return false;
    if (!same_under_renaming(*s.args[i], *r.args[i], s_vars, r_vars, map)) return false;
  }
  return true;
}

static size_t count_loads(const Node& n) {
  size_t c = n.op == Op::Load ? 1 : 0;
  for (const auto& a : n.args)
    if (a) c += count_loads(*a);
  return c;
}

// R with every subexpression that equals what S stored (same loop extents under the renaming)
// replaced by a load of S's output; null when there is none.  Only expressions of two loads or
// more are taken: the point is to read one buffer instead of several.
static NodePtr reuse_stored_value(const NestKernel& S, const NestKernel& R) {
  if (S.rkind != ReduceKind::None || !S.out_aff || S.out_buf == R.out_buf) return nullptr;
  if (count_loads(*S.value) < 2 || infer_ty(*S.value, nullptr) != S.out_dtype.ty) return nullptr;
  std::set<std::string> s_vars, r_vars;
  std::map<std::string, int64_t> s_ext, r_ext;
  for (const auto& l : S.loops) { s_vars.insert(l.var); s_ext[l.var] = l.extent; }
  for (const auto& l : R.loops) { r_vars.insert(l.var); r_ext[l.var] = l.extent; }
  if (R.rkind != ReduceKind::None) { r_vars.insert(R.rloop.var); r_ext[R.rloop.var] = R.rloop.extent; }
  for (const auto& pp : R.params)
    if (pp.name == S.out_buf && pp.mut_) return nullptr;
  bool changed = false;
  std::function<NodePtr(const NodePtr&)> walk = [&](const NodePtr& n) -> NodePtr {
    std::map<std::string, std::string> m;
    if (same_under_renaming(*S.value, *n, s_vars, r_vars, &m)) {
      bool ok = true;
      std::map<std::string, NodePtr> ren;
      for (const auto& l : S.loops) {
        auto it = m.find(l.var);
        if (it == m.end()) { ok = ok && (l.extent == 1 || S.out_aff->of(l.var) == 0); ren[l.var] = make_i64(0); continue; }
        ok = ok && r_ext[it->second] == l.extent;
        ren[l.var] = make_var(it->second);
      }
      if (ok) {
        auto ld = make(Op::Load, {make_var(S.out_buf), rename(S.out_index, ren)});
        ld->dtype = S.out_dtype;
        changed = true;
        return ld;
      }
    }
    bool ch = false;
    std::vector<NodePtr> args;
    args.reserve(n->args.size());
    for (const auto& a : n->args) {
      NodePtr x = a ? walk(a) : a;
      ch = ch || x != a;
      args.push_back(std::move(x));
    }
    if (!ch) return n;
    auto c = std::make_shared<Node>(*n);
    c->args = std::move(args);
    return c;
  };
  NodePtr value = walk(R.value);
  if (!changed) return nullptr;
  NodePtr body = R.rkind == ReduceKind::None ? make(Op::Store, {make_var(R.out_buf), R.out_index, value})
                                             : make_reduce_block(R, R.rloop.var, R.rloop.extent, value, R.out_buf, R.out_index);
  for (size_t i = R.loops.size(); i-- > 0;) body = make_range(R.loops[i].var, R.loops[i].extent, body);
  // parameters: what the new value still reads, then S's output, then R's outputs
  std::vector<LoadRef> lds;
  collect_loads(*value, lds);
  std::set<std::string> read;
  for (const auto& lr : lds)
    if (lr.load->args[0]->op == Op::Var) read.insert(lr.load->args[0]->name);
  std::vector<Param> params;
  bool have_s = false;
  for (const auto& pp : R.params) {
    if (pp.dtype.is_ptr() && !pp.mut_ && !read.count(pp.name)) continue;
    if (pp.mut_ && !have_s) {
      bool listed = false;
      for (const auto& q : params) listed = listed || q.name == S.out_buf;
      if (!listed) {
        Param sp;
        sp.name = S.out_buf;
        sp.dtype.ty = Ty::Ptr;
        sp.dtype.inner = std::make_shared<DType>(S.out_dtype);
        params.push_back(sp);
      }
      have_s = true;
    }
    params.push_back(pp);
  }
  return make_kernel(R.name, params, body);
}

// ---------------------------------------------------------------------------------------------
// elementwise producers read through another index space: evaluated where they are read
// ---------------------------------------------------------------------------------------------


static bool pure_gather(const NestKernel& k) {
  const Node* v = k.value.get();
  if (v->op == Op::Select && v->args[2]->op == Op::Const) v = v->args[1].get();
  return v->op == Op::Load;
}

static NodePtr replace_loads(const NodePtr& n, const std::string& buf, const NodePtr& with) {
  if (n->op == Op::Load && n->args[0]->op == Op::Var && n->args[0]->name == buf) return with;
  bool changed = false;
  std::vector<NodePtr> args;
  args.reserve(n->args.size());
  for (const auto& a : n->args) {
    NodePtr r = a ? replace_loads(a, buf, with) : a;
    changed = changed || r != a;
    args.push_back(std::move(r));
  }
  if (!changed) return n;
  auto c = std::make_shared<Node>(*n);
  c->args = std::move(args);
  return c;
}

static std::optional<Inlined> inline_producer(const NestKernel& P, const NestKernel& C, bool same_space = false) {
  if (P.rkind != ReduceKind::None || C.rkind != ReduceKind::None) return std::nullopt;
  // a pure gather stays one: contractions and window reductions fold gathers (and chains of them)
  // into their loaders in their own way, which a gather that computes would be lost to
  if (pure_gather(C) || !C.out_aff) return std::nullopt;
  int64_t numel = 0;
  auto strides = dense_strides(P, &numel);
  if (!strides) return std::nullopt;
  // every load of the temp in C, all through the same affine index without offset
  std::vector<LoadRef> loads;
  collect_loads(*C.value, loads);
  std::optional<Affine> idx;
  for (const auto& lr : loads) {
    if (lr.load->args[0]->op != Op::Var) return std::nullopt;
    if (lr.load->args[0]->name != P.out_buf) {
      for (const auto& pp : P.params)               // C must not write what P reads
        if (pp.name == C.out_buf) return std::nullopt;
      continue;
    }
    if (lr.load->count != 1) return std::nullopt;
    auto a = affine_of(*lr.load->args[1]);
    if (!a || a->c != 0) return std::nullopt;
    if (idx && !(*idx == *a)) return std::nullopt;
    idx = a;
  }
  if (!idx) return std::nullopt;
  // the new C: (split) loops, P's value (cast to the temp's element type) where the temp was read
  auto build = [&](const std::map<std::string, NodePtr>& p_map, const std::map<std::string, NodePtr>& c_map,
                   const std::map<std::string, std::vector<Loop>>& c_split) {
    NodePtr pv = rename(P.value, p_map);
    if (!(P.out_dtype.ty == Ty::F32 && infer_ty(*P.value, nullptr) == Ty::F32)) {
      auto cast = make(Op::Cast, {pv});
      cast->dtype = P.out_dtype;
      pv = cast;
    }
    NodePtr value = replace_loads(rename(C.value, c_map), P.out_buf, pv);
    NodePtr body = make(Op::Store, {make_var(C.out_buf), rename(C.out_index, c_map), value});
    for (size_t i = C.loops.size(); i-- > 0;) {
      auto it = c_split.find(C.loops[i].var);
      if (it == c_split.end()) {
        body = make_range(C.loops[i].var, C.loops[i].extent, body);
      } else {
        for (size_t j = it->second.size(); j-- > 0;) body = make_range(it->second[j].var, it->second[j].extent, body);
      }
    }
    std::vector<Param> params;
    std::set<std::string> have;
    for (const auto& pp : C.params)
      if (pp.name != P.out_buf && have.insert(pp.name).second) params.push_back(pp);
    // P's operands go in front of C's output (immutable parameters first, as kernels list them)
    std::vector<Param> ins;
    for (const auto& pp : P.params)
      if (pp.dtype.is_ptr() && !pp.mut_ && have.insert(pp.name).second) ins.push_back(pp);
    size_t first_mut = 0;
    while (first_mut < params.size() && !params[first_mut].mut_) ++first_mut;
    params.insert(params.begin() + static_cast<long>(first_mut), ins.begin(), ins.end());
    Inlined r;
    r.kernel = make_kernel(C.name, params, body);
    return r;
  };
  {
    // the same index space already: the ordinary fusion takes neighbours; a reader far away
    // (`same_space`) evaluates P at its own loop variables
    bool same = P.loops.size() == C.loops.size();
    for (size_t i = 0; same && i < P.loops.size(); ++i)
      same = P.loops[i].extent == C.loops[i].extent && idx->of(C.loops[i].var) == (*strides)[i] * (P.loops[i].extent > 1 ? 1 : 0);
    if (same) {
      if (!same_space) return std::nullopt;
      std::map<std::string, NodePtr> p_map;
      for (size_t i = 0; i < P.loops.size(); ++i) p_map[P.loops[i].var] = make_var(C.loops[i].var);
      return build(p_map, {}, {});
    }
    if (same_space) return std::nullopt;
  }
  // C's terms of the index, ascending; each must rise above what the smaller ones reach
  struct Term { std::string var; int64_t c, ext; };
  std::vector<Term> terms;
  for (const auto& l : C.loops) {
    const int64_t c = idx->of(l.var);
    if (c < 0) return std::nullopt;
    if (c > 0 && l.extent > 1) terms.push_back({l.var, c, l.extent});
  }
  for (const auto& kv : idx->coef) {
    bool known = kv.second == 0;
    for (const auto& l : C.loops) known = known || l.var == kv.first;
    if (!known) return std::nullopt;
  }
  std::sort(terms.begin(), terms.end(), [](const Term& a, const Term& b) { return a.c < b.c; });
  int64_t reach = 0;
  for (const auto& t : terms) {
    if (t.c <= reach) return std::nullopt;
    reach += t.c * (t.ext - 1);
  }
  if (reach >= numel) return std::nullopt;
  // cut every term at P's loop boundaries that fall inside it
  struct Sub { std::string var; int64_t c, ext; };
  std::vector<Sub> subs;
  std::map<std::string, NodePtr> c_map;               // C's split variables as sums of their parts
  std::map<std::string, std::vector<Loop>> c_split;
  for (const auto& t : terms) {
    std::vector<int64_t> cuts;                         // factors of the extent, ascending
    for (size_t q = 0; q < P.loops.size(); ++q) {
      const int64_t b = (*strides)[q];
      if (P.loops[q].extent <= 1 || b <= t.c || b >= t.c * t.ext) continue;
      if (b % t.c || (t.c * t.ext) % b) return std::nullopt;
      cuts.push_back(b / t.c);
    }
    std::sort(cuts.begin(), cuts.end());
    cuts.erase(std::unique(cuts.begin(), cuts.end()), cuts.end());
    for (size_t i = 0; i + 1 < cuts.size(); ++i)
      if (cuts[i + 1] % cuts[i]) return std::nullopt;
    if (cuts.empty()) {
      subs.push_back({t.var, t.c, t.ext});
      continue;
    }
    if (t.ext % cuts.back()) return std::nullopt;
    NodePtr sum;
    std::vector<Loop> parts;                           // outermost first
    int64_t below = 1;
    cuts.push_back(t.ext);
    for (size_t i = 0; i < cuts.size(); ++i) {
      const std::string name = t.var + "_p" + std::to_string(i);
      const int64_t ext = cuts[i] / below;
      subs.push_back({name, t.c * below, ext});
      NodePtr part = below == 1 ? make_var(name) : make(Op::Mul, {make_var(name), make_i64(below)});
      sum = sum ? make(Op::Add, {part, sum}) : part;
      parts.insert(parts.begin(), Loop{name, ext});
      below = cuts[i];
    }
    c_map[t.var] = sum;
    c_split[t.var] = parts;
  }
  // every loop variable of P as the sum of the parts that lie inside its digit
  std::map<std::string, NodePtr> p_map;
  for (size_t q = 0; q < P.loops.size(); ++q) {
    const int64_t s = (*strides)[q], e = P.loops[q].extent;
    NodePtr sum;
    int64_t top = 0;
    if (e > 1)
      for (const auto& sb : subs) {
        if (sb.c * sb.ext <= s || sb.c >= s * e) continue;      // entirely below or above this digit
        if (sb.c < s || sb.c % s || sb.c * sb.ext > s * e) return std::nullopt;
        const int64_t m = sb.c / s;
        NodePtr part = m == 1 ? make_var(sb.var) : make(Op::Mul, {make_var(sb.var), make_i64(m)});
        sum = sum ? make(Op::Add, {sum, part}) : part;
        top += m * (sb.ext - 1);
      }
    if (top > e - 1) return std::nullopt;
    p_map[P.loops[q].var] = sum ? sum : make_i64(0);
  }
  return build(p_map, c_map, c_split);
}


// ---------------------------------------------------------------------------------------------
// a contraction's temp stored the other way round when its reader walks it column by column
// ---------------------------------------------------------------------------------------------

// A contraction writes a dense temp T[m][n] (n contiguous) and the one elementwise kernel that
// reads it walks m with its innermost loop (the input gradient of a convolution: the columns
// written by `dY x W`, summed window by window along the image's x): every lane then reads from
// another row, N elements apart.  A temp's layout is nobody else's business, so both sides are
// rewritten to T[n][m]: the contraction computes the transposed product (same work, stores still
// along its tile's contiguous axis) and the reader's innermost loop becomes unit stride.
static NodePtr affine_expr(const Affine& a) {
  NodePtr e;
  for (const auto& kv : a.coef) {
    if (kv.second == 0) continue;
    NodePtr t = kv.second == 1 ? make_var(kv.first) : make(Op::Mul, {make_var(kv.first), make_i64(kv.second)});
    e = e ? make(Op::Add, {e, t}) : t;
  }
  if (a.c != 0 || !e) e = e ? make(Op::Add, {e, make_i64(a.c)}) : make_i64(a.c);
  return e;
}

// idx = m*N + n with 0 <= n < N for every value of the loops  ->  n*M + m; nullopt when the
// split cannot be read off the coefficients
static std::optional<Affine> transposed_index(const Affine& a, const std::vector<Loop>& loops, const Loop* rloop, int64_t M, int64_t N) {
  Affine r;
  const int64_t lo_c = ((a.c % N) + N) % N;
  int64_t lo_max = lo_c;
  r.c = lo_c * M + (a.c - lo_c) / N;
  for (const auto& kv : a.coef) {
    if (kv.second == 0) continue;
    int64_t ext = 0;
    for (const auto& l : loops)
      if (l.var == kv.first) ext = l.extent;
    if (rloop && rloop->var == kv.first) ext = rloop->extent;
    if (ext <= 0 || kv.second < 0) return std::nullopt;
    if (kv.second % N == 0) {
      r.coef[kv.first] = kv.second / N;
    } else {
      if (kv.second >= N) return std::nullopt;
      lo_max += kv.second * (ext - 1);
      r.coef[kv.first] = kv.second * M;
    }
  }
  if (lo_max >= N) return std::nullopt;
  return r;
}

static NodePtr reindex_loads(const NodePtr& n, const std::string& buf, const std::function<NodePtr(const Node&)>& new_index) {
  if (n->op == Op::Load && n->args[0]->op == Op::Var && n->args[0]->name == buf) {
    auto c = std::make_shared<Node>(*n);
    c->args[1] = new_index(*n->args[1]);
    return c;
  }
  bool changed = false;
  std::vector<NodePtr> args;
  args.reserve(n->args.size());
  for (const auto& a : n->args) {
    NodePtr r = a ? reindex_loads(a, buf, new_index) : a;
    changed = changed || r != a;
    args.push_back(std::move(r));
  }
  if (!changed) return n;
  auto c = std::make_shared<Node>(*n);
  c->args = std::move(args);
  return c;
}

// The contraction K with its output stored transposed; M and N are set to T's extents.
static NodePtr transpose_producer(const NestKernel& K, const GenOptions& opt, int64_t* Mo, int64_t* No) {
  if (K.rkind != ReduceKind::Sum || !K.out_aff || !opt.gemm) return nullptr;
  auto sh = match_gemm(K);
  if (!sh || sh->batch != 1 || !gemm_output_dense(*sh) || sh->c_buf != K.out_buf) return nullptr;
  const int64_t M = sh->M, N = sh->N;
  if (M * N < (int64_t{1} << 20) || N < 8) return nullptr;
  auto kout = transposed_index(*K.out_aff, K.loops, nullptr, M, N);
  if (!kout) return nullptr;
  NodePtr body = make_reduce_block(K, K.rloop.var, K.rloop.extent, K.value, K.out_buf, affine_expr(*kout));
  for (size_t i = K.loops.size(); i-- > 0;) body = make_range(K.loops[i].var, K.loops[i].extent, body);
  *Mo = M;
  *No = N;
  return make_kernel(K.name, K.params, body);
}

// Reader E of T[M][N] rewritten for T[N][M]; null when E does not walk T's rows with its
// innermost loop in every load, or an index does not split.
static NodePtr transpose_reader(const NestKernel& E, const std::string& T, int64_t M, int64_t N) {
  if (E.rkind != ReduceKind::None) return nullptr;
  std::vector<LoadRef> loads;
  collect_loads(*E.value, loads);
  // the reader's innermost live loop must walk rows of T in every load of it
  const Loop* inner = nullptr;
  for (const auto& l : E.loops)
    if (l.extent > 1) inner = &l;
  if (!inner) return nullptr;
  size_t sites = 0;
  for (const auto& lr : loads) {
    if (lr.load->args[0]->op != Op::Var || lr.load->args[0]->name != T) continue;
    if (lr.load->count != 1) return nullptr;
    auto a = affine_of(*lr.load->args[1]);
    if (!a || a->of(inner->var) != N) return nullptr;
    if (!transposed_index(*a, E.loops, nullptr, M, N)) return nullptr;
    ++sites;
  }
  if (!sites) return nullptr;
  NodePtr value = reindex_loads(E.value, T, [&](const Node& idx) {
    return affine_expr(*transposed_index(*affine_of(idx), E.loops, nullptr, M, N));
  });
  NodePtr body = make(Op::Store, {make_var(E.out_buf), E.out_index, value});
  for (size_t i = E.loops.size(); i-- > 0;) body = make_range(E.loops[i].var, E.loops[i].extent, body);
  return make_kernel(E.name, E.params, body);
}


// The program-level rewrites in front of planning (option `reindex`): whole-buffer copies dropped,
// stored values read back, elementwise producers evaluated in readers that walk another index
// space, contraction temps stored the way their readers walk them.  `kernels` is the program's
// kernel list in execution order (entries are replaced or removed), `rewritten` owns the new
// kernels, `plan->elided` collects the temps that disappear.
void rewrite_for_readers(const Node& program, const GenOptions& opt, std::vector<const Node*>* kernels,
                         std::vector<NodePtr>* rewritten, ProgramPlan* plan) {
  auto is_temp = [&](const std::string& name) {
    for (const auto& b : plan->buffers)
      if (b.name == name) return b.role == "temp";
    return false;
  };
  auto writers_of = [&](const std::string& name) {
    size_t n = 0;
    for (const Node* k : *kernels)
      for (const auto& pp : k->params) n += pp.dtype.is_ptr() && pp.mut_ && pp.name == name;
    return n;
  };
  auto rename_buffer = [&](const NodePtr& k, const std::string& from, const std::string& to) {
    NodePtr body = rename(k->args[0], {{from, make_var(to)}});
    std::vector<Param> params;
    bool have = false;
    for (const auto& pp : k->params) have = have || pp.name == to;
    for (auto pp : k->params) {
      if (pp.name == from) {
        if (have) continue;
        pp.name = to;
      }
      params.push_back(pp);
    }
    auto c = std::make_shared<Node>(*k);
    c->params = std::move(params);
    c->args = {body};
    return c;
  };
  // phase 0 drops whole-buffer copies; then values that an earlier kernel already stored are
  // read back where a later kernel computes them again; phase 1 evaluates producers in readers
  for (int phase = 0; phase < 2; ++phase) {
    if (phase == 1) {
      for (size_t si = 0; si < kernels->size(); ++si) {
        auto ns = extract_nest(*(*kernels)[si]);
        if (!ns || ns->rkind != ReduceKind::None || writers_of(ns->out_buf) != 1) continue;
        for (size_t ri = si + 1; ri < kernels->size(); ++ri) {
          auto nr = extract_nest(*(*kernels)[ri]);
          if (!nr) continue;
          NodePtr nk = reuse_stored_value(*ns, *nr);
          if (!nk) continue;
          rewritten->push_back(nk);
          (*kernels)[ri] = nk.get();
        }
      }
    }
    for (bool again = true; again;) {
      again = false;
      for (size_t p = 0; p < kernels->size() && !again; ++p) {
        auto np = extract_nest(*(*kernels)[p]);
        if (!np || np->rkind != ReduceKind::None || !is_temp(np->out_buf) || writers_of(np->out_buf) != 1) continue;
        std::vector<size_t> rd;
        bool early = false;
        for (size_t c = 0; c < kernels->size(); ++c)
          for (const auto& pp : (*kernels)[c]->params)
            if (pp.dtype.is_ptr() && !pp.mut_ && pp.name == np->out_buf) {
              rd.push_back(c);
              early = early || c <= p;
            }
        if (rd.empty() || early) continue;
        // a copy of a whole buffer, element for element: its readers read the original
        if (np->value->op == Op::Load && np->value->args[0]->op == Op::Var && np->value->count == 1 && np->out_aff) {
          const std::string& src = np->value->args[0]->name;
          auto a = affine_of(*np->value->args[1]);
          int64_t numel = 0;
          bool same_type = false;
          for (const auto& pp : np->params) same_type = same_type || (pp.name == src && pp.dtype.is_ptr() && pp.dtype.elem().ty == np->out_dtype.ty);
          if (a && *a == *np->out_aff && dense_strides(*np, &numel) && same_type && src != np->out_buf && writers_of(src) <= 1) {
            bool src_written_later = false;
            for (size_t m = p + 1; m < kernels->size(); ++m)
              for (const auto& pm : (*kernels)[m]->params) src_written_later = src_written_later || (pm.dtype.is_ptr() && pm.mut_ && pm.name == src);
            if (!src_written_later) {
              for (size_t c : rd) {
                NodePtr owner;
                for (const auto& f : program.args)
                  if (f.get() == (*kernels)[c]) owner = f;
                for (const auto& f : *rewritten)
                  if (f.get() == (*kernels)[c]) owner = f;
                if (!owner) throw Error("internal: kernel without owner");
                NodePtr nk = rename_buffer(owner, np->out_buf, src);
                rewritten->push_back(nk);
                (*kernels)[c] = nk.get();
              }
              plan->elided.insert(np->out_buf);
              kernels->erase(kernels->begin() + static_cast<long>(p));
              again = true;
              continue;
            }
          }
        }
        if (phase == 0 || rd.size() > 3) continue;
        {
          // what reads a reduction's result element for element stays with it: it is that
          // reduction's epilogue, and evaluated elsewhere it would keep the raw result alive for a
          // reader far away
          int64_t p_numel = 1;
          for (const auto& l : np->loops) p_numel *= l.extent;
          bool after_reduce = false;
          for (const auto& pp : (*kernels)[p]->params) {
            if (!pp.dtype.is_ptr() || pp.mut_) continue;
            for (size_t w = 0; w < p; ++w) {
              bool writes = false;
              for (const auto& pw : (*kernels)[w]->params) writes = writes || (pw.dtype.is_ptr() && pw.mut_ && pw.name == pp.name);
              if (!writes) continue;
              auto nw = extract_nest(*(*kernels)[w]);
              int64_t w_numel = 1;
              if (nw)
                for (const auto& l : nw->loops) w_numel *= l.extent;
              after_reduce = after_reduce || !nw || (nw->rkind != ReduceKind::None && w_numel == p_numel);
            }
          }
          if (after_reduce) continue;
        }
        {
          std::vector<LoadRef> pl;
          collect_loads(*np->value, pl);
          std::set<std::string> srcs;
          for (const auto& lr : pl)
            if (lr.load->args[0]->op == Op::Var) srcs.insert(lr.load->args[0]->name);
          if (rd.size() > 1 && srcs.size() > 6) continue;    // evaluated once per reader: keep it cheap
        }
        size_t left = rd.size();
        for (size_t reader : rd) {
          // nothing between the two may write what P reads
          bool clobbered = false;
          for (size_t m = p + 1; m <= reader; ++m)
            for (const auto& pm : (*kernels)[m]->params)
              if (pm.dtype.is_ptr() && pm.mut_)
                for (const auto& pp : (*kernels)[p]->params) clobbered = clobbered || (pp.name == pm.name && !pp.mut_);
          if (clobbered) continue;
          auto nc = extract_nest(*(*kernels)[reader]);
          if (!nc) continue;
          auto in = inline_producer(*np, *nc);
          // A reader over the same index space that the ordinary fusion cannot reach (a reduce
          // or a contraction lies between the two: the backward pass reading what the forward
          // pass saved) evaluates a cheap producer again instead of reading its stored result,
          // when what the producer reads is kept in memory for later readers anyway: one store
          // and one load of the whole tensor less, the same operations on the same values.
          if (!in && opt.rematerialize && reader > p + 1) {
            bool barrier = false;
            for (size_t m = p + 1; m < reader && !barrier; ++m) {
              auto nm = extract_nest(*(*kernels)[m]);
              barrier = !nm || nm->rkind != ReduceKind::None;
            }
            std::function<size_t(const Node&)> size_of = [&](const Node& n) {
              size_t c = 1;
              for (const auto& a : n.args)
                if (a && n.op != Op::Load) c += size_of(*a);
              return c;
            };
            std::vector<LoadRef> pl;
            collect_loads(*np->value, pl);
            bool kept = barrier && pl.size() <= 2 && size_of(*np->value) <= 8;
            for (const auto& lr : pl) {
              if (!kept) break;
              if (lr.load->args[0]->op != Op::Var) { kept = false; break; }
              const std::string& b = lr.load->args[0]->name;
              if (!is_temp(b)) continue;
              bool later = false;          // read by this reader already, or by a kernel after it
              for (size_t q = reader; q < kernels->size() && !later; ++q)
                for (const auto& pq : (*kernels)[q]->params) later = later || (pq.dtype.is_ptr() && !pq.mut_ && pq.name == b);
              kept = later;
            }
            if (kept) in = inline_producer(*np, *nc, true);
          }
          if (!in) continue;
          rewritten->push_back(in->kernel);
          (*kernels)[reader] = in->kernel.get();
          --left;
          again = true;
        }
        if (left == 0) {
          plan->elided.insert(np->out_buf);
          kernels->erase(kernels->begin() + static_cast<long>(p));
        }
      }
    }
  }
  // temps between a contraction and an elementwise reader that walks them column by column
  for (size_t p = 0; p < kernels->size(); ++p) {
    auto nk = extract_nest(*(*kernels)[p]);
    if (!nk || nk->rkind != ReduceKind::Sum) continue;
    bool temp = false;
    for (const auto& b : plan->buffers) temp = temp || (b.name == nk->out_buf && b.role == "temp");
    if (!temp) continue;
    std::vector<size_t> rd;
    size_t nwriters = 0;
    bool early = false;
    for (size_t c = 0; c < kernels->size(); ++c)
      for (const auto& pp : (*kernels)[c]->params)
        if (pp.dtype.is_ptr() && pp.name == nk->out_buf) {
          if (pp.mut_) ++nwriters;
          else { rd.push_back(c); early = early || c <= p; }
        }
    if (rd.empty() || nwriters != 1 || early) continue;
    {
      // one reader that reads every element once, unguarded, is a plain permutation: the
      // contraction's epilogue writes that reader's result in place instead
      size_t sites = 0;
      bool guarded = false;
      for (size_t c : rd) {
        auto ne = extract_nest(*(*kernels)[c]);
        if (!ne) continue;
        std::vector<LoadRef> lds;
        collect_loads(*ne->value, lds);
        for (const auto& lr : lds)
          if (lr.load->args[0]->op == Op::Var && lr.load->args[0]->name == nk->out_buf) {
            ++sites;
            guarded = guarded || lr.guarded;
          }
      }
      if (sites < 2 && !guarded) continue;
    }
    int64_t M = 0, N = 0;
    NodePtr prod = transpose_producer(*nk, opt, &M, &N);
    if (!prod) continue;
    std::vector<NodePtr> readers_new;
    for (size_t c : rd) {
      auto ne = extract_nest(*(*kernels)[c]);
      NodePtr r = ne ? transpose_reader(*ne, nk->out_buf, M, N) : nullptr;
      if (!r) break;
      readers_new.push_back(r);
    }
    if (readers_new.size() != rd.size()) continue;
    rewritten->push_back(prod);
    (*kernels)[p] = prod.get();
    for (size_t i = 0; i < rd.size(); ++i) {
      rewritten->push_back(readers_new[i]);
      (*kernels)[rd[i]] = readers_new[i].get();
    }
  }
}


// ---------------------------------------------------------------------------------------------
// passes of plan_program over the kernels in canonical form
// ---------------------------------------------------------------------------------------------

// An elementwise kernel separated from the kernel that produces what it reads by small
// kernels it has nothing to do with (the roots of a step are lowered one after another, so
// the loss's bookkeeping of a few thousand elements can land inside another root's chain)
// moves up behind its producer, where the producer's fused launch can take it.  Past a large
// kernel it stays: computed early, its result would have to be kept in memory instead.
void move_elementwise_behind_producers(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (!plan.buffers.empty() && opt.fuse && opt.reindex) {
    auto outs_of = [](const Node* k) {
      std::set<std::string> o;
      for (const auto& p : k->params)
        if (p.dtype.is_ptr() && p.mut_) o.insert(p.name);
      return o;
    };
    auto small = [&](const Node* k) {
      for (const auto& p : k->params) {
        if (!p.dtype.is_ptr() || !p.mut_) continue;
        bool known = false;
        for (const auto& b : plan.buffers)
          if (b.name == p.name) { known = true; if (b.numel() > (size_t{1} << 16)) return false; }
        if (!known) return false;
      }
      return true;
    };
    for (size_t c = 2; c < kernels.size(); ++c) {
      const Node* kc = kernels[c];
      if (kc->name.rfind("E_", 0) != 0) continue;
      std::set<std::string> c_in, c_all;
      for (const auto& p : kc->params)
        if (p.dtype.is_ptr()) { c_all.insert(p.name); if (!p.mut_) c_in.insert(p.name); }
      const auto co = outs_of(kc);
      size_t pos = c;
      bool found = false;
      while (pos > 0) {
        const Node* kb = kernels[pos - 1];
        bool produces = false, clash = false;
        for (const auto& p : kb->params) {
          if (!p.dtype.is_ptr()) continue;
          produces = produces || (p.mut_ && c_in.count(p.name));
          clash = clash || co.count(p.name) || (p.mut_ && c_all.count(p.name) && !c_in.count(p.name));
        }
        if (produces) { found = true; break; }
        if (clash || !small(kb)) break;
        --pos;
      }
      if (!found || pos == c) continue;
      kernels.erase(kernels.begin() + static_cast<long>(c));
      kernels.insert(kernels.begin() + static_cast<long>(pos), kc);
    }
  }
}

// A contraction per batch element whose results the next kernel sums over the batch (the
// weight gradient of a convolution: per-image products, then a sum over images) is one
// contraction with the batch folded into k, when both operands walk (batch, k) as one axis.
// The summing kernel disappears, and so does the per-batch result buffer.
void merge_batch_sums_into_contractions(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (opt.gemm && opt.gemm_merge_batch && have_table) {
    for (size_t i = 0; i + 1 < kernels.size(); ++i) {
      if (!nests[i] || !nests[i + 1]) continue;
      const NestKernel& g0 = *nests[i];
      const NestKernel& r2 = *nests[i + 1];
      if (g0.rkind != ReduceKind::Sum || r2.rkind != ReduceKind::Sum || !gemm_shaped(g0, opt)) continue;
      auto gs = match_gemm(g0);
      if (!gs || gs->batch <= 1 || gs->a_b != gs->K * gs->a_k || gs->b_b != gs->K * gs->b_k) continue;
      if (role_of(g0.out_buf) != "temp" || readers[g0.out_buf] != std::vector<size_t>{i + 1}) continue;
      if (!r2.identity || r2.identity->fval != 0.0 || r2.acc_dtype.ty != Ty::F32 || r2.out_dtype.ty != Ty::F32) continue;
      const Node& v = *r2.value;
      if (v.op != Op::Load || v.args[0]->op != Op::Var || v.args[0]->name != g0.out_buf || v.count != 1) continue;
      auto ra = affine_of(*v.args[1]);
      if (!ra || !r2.out_aff || !g0.out_aff || ra->c != g0.out_aff->c) continue;
      // the batch loop of g0: the one both operands move with
      std::string bvar;
      {
        const Node& gv = *g0.value;
        auto aa = affine_of(*gv.args[0]->args[1]);
        auto ab = affine_of(*gv.args[1]->args[1]);
        if (!aa || !ab) continue;
        int nb = 0;
        for (const auto& l : g0.loops)
          if (l.extent > 1 && aa->of(l.var) != 0 && ab->of(l.var) != 0) { bvar = l.var; ++nb; }
        if (nb != 1) continue;
      }
      // r2 must sum exactly that axis and keep the others: match loops by their stride in C
      if (r2.rloop.extent != gs->batch || ra->of(r2.rloop.var) != g0.out_aff->of(bvar)) continue;
      std::map<std::string, NodePtr> to_g0;     // r2's loop variables in terms of g0's
      bool ok = true;
      size_t matched = 0;
      for (const auto& l2 : r2.loops) {
        if (l2.extent <= 1) { to_g0[l2.var] = make_i64(0); continue; }
        const Loop* hit = nullptr;
        for (const auto& l0 : g0.loops)
          if (l0.var != bvar && l0.extent == l2.extent && g0.out_aff->of(l0.var) == ra->of(l2.var)) hit = &l0;
        if (!hit) { ok = false; break; }
        to_g0[l2.var] = make_var(hit->var);
        ++matched;
      }
      size_t live0 = 0;
      for (const auto& l0 : g0.loops) live0 += (l0.extent > 1 && l0.var != bvar);
      if (!ok || matched != live0) continue;
      NestKernel m = g0;
      m.value = rename(g0.value, {{bvar, make_i64(0)}});
      m.rloop.extent = g0.rloop.extent * gs->batch;
      for (auto& l : m.loops)
        if (l.var == bvar) l.extent = 1;
      m.out_buf = r2.out_buf;
      m.out_dtype = r2.out_dtype;
      m.out_index = rename(rename(r2.out_index, {{r2.rloop.var, make_i64(0)}}), to_g0);
      m.out_aff = affine_of(*m.out_index);
      for (const auto& p : r2.params)
        if (p.mut_) {
          for (auto& q : m.params)
            if (q.mut_) q = p;
        }
      if (!m.out_aff || !gemm_shaped(m, opt)) continue;
      plan.elided.insert(g0.out_buf);      // (g0 refers to nests[i]: use it before the assignment)
      absorbed_name[i] = r2.name;
      absorbed.insert(i + 1);
      nests[i] = m;
    }
  }
}

// A sum over one axis whose result the next kernel only sums over a neighbouring axis (a bias
// gradient as the reference lowers it: over the image's columns, then its rows, then the
// batch) is one sum over both when every operand walks the two axes as one: the second kernel
// and the buffer between them disappear, and what was two short strided passes is one pass
// along memory.  (The order of the additions changes, as it does in every parallel reduce.)
void merge_sums_over_neighbouring_axes(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (opt.fuse && opt.reindex && have_table) {
    for (size_t i = 0; i + 1 < kernels.size(); ++i) {
      if (!nests[i] || !nests[i + 1] || absorbed.count(i) || absorbed.count(i + 1)) continue;
      const NestKernel& r1 = *nests[i];
      const NestKernel& r2 = *nests[i + 1];
      if (r1.rkind != ReduceKind::Sum || r2.rkind != ReduceKind::Sum || !r1.out_aff || !r2.out_aff) continue;
      if (r1.acc_dtype.ty != Ty::F32 || r1.out_dtype.ty != Ty::F32 || r2.acc_dtype.ty != Ty::F32 || r2.out_dtype.ty != Ty::F32) continue;
      if (!r1.identity || r1.identity->fval != 0.0 || !r2.identity || r2.identity->fval != 0.0) continue;
      if (opt.gemm && (gemm_shaped(r1, opt) || gemm_shaped(r2, opt))) continue;
      if (role_of(r1.out_buf) != "temp" || readers[r1.out_buf] != std::vector<size_t>{i + 1}) continue;
      if (r1.out_buf.rfind("eh_", 0) == 0) continue;       // pieces of lines the planner itself cut: they stay two reduces
      const Node& v2 = *r2.value;
      if (v2.op != Op::Load || v2.count != 1 || v2.args[0]->op != Op::Var || v2.args[0]->name != r1.out_buf) continue;
      auto ra = affine_of(*v2.args[1]);
      if (!ra || ra->c != r1.out_aff->c) continue;
      // r2's loops (and its reduce loop) against r1's output loops, matched by their stride in the buffer between
      std::map<std::string, NodePtr> to_r1;       // r2's loop variables in terms of r1's
      const Loop* outer = nullptr;                // the loop of r1 that r2 sums over
      bool ok = true;
      size_t matched = 0;
      auto match = [&](const Loop& l2) -> const Loop* {
        const Loop* hit = nullptr;
        for (const auto& l1 : r1.loops)
          if (l1.extent > 1 && l1.extent == l2.extent && r1.out_aff->of(l1.var) == ra->of(l2.var)) hit = &l1;
        return hit;
      };
      for (const auto& l2 : r2.loops) {
        if (l2.extent <= 1) { to_r1[l2.var] = make_i64(0); continue; }
        const Loop* hit = match(l2);
        if (!hit) { ok = false; break; }
        to_r1[l2.var] = make_var(hit->var);
        ++matched;
      }
      if (!ok || r2.rloop.extent < 2) continue;
      outer = match(r2.rloop);
      size_t live1 = 0;
      for (const auto& l1 : r1.loops) live1 += l1.extent > 1;
      if (!outer || matched + 1 != live1) continue;
      // every load of r1 must walk (outer, r1's reduce loop) as one axis, unguarded
      std::vector<LoadRef> loads;
      collect_loads(*r1.value, loads);
      for (const auto& lr : loads) {
        auto a = affine_of(*lr.load->args[1]);
        ok = ok && a && !lr.guarded && a->of(outer->var) == r1.rloop.extent * a->of(r1.rloop.var);
      }
      // (not into few long lines: one workgroup per line needs many lines to fill the chip)
      int64_t lines = 1;
      for (const auto& l2 : r2.loops) lines *= l2.extent;
      if (!ok || loads.empty() || r1.rloop.extent * outer->extent > 8192 || lines < 1024) continue;
      // the two loop variables may appear in load indices only (not as values: an iota, a mask by position)
      std::function<bool(const Node&)> as_value = [&](const Node& n) {
        if (n.op == Op::Load) return false;
        if ((n.op == Op::Var || n.op == Op::Wildcard) && (n.name == outer->var || n.name == r1.rloop.var)) return true;
        for (const auto& a : n.args)
          if (a && as_value(*a)) return true;
        return false;
      };
      if (as_value(*r1.value)) continue;
      NestKernel m = r1;
      m.value = rename(r1.value, {{outer->var, make_i64(0)}});
      m.rloop.extent = r1.rloop.extent * outer->extent;
      for (auto& l : m.loops)
        if (l.var == outer->var) l.extent = 1;
      m.out_buf = r2.out_buf;
      m.out_dtype = r2.out_dtype;
      m.out_index = rename(rename(r2.out_index, {{r2.rloop.var, make_i64(0)}}), to_r1);
      m.out_aff = affine_of(*m.out_index);
      for (const auto& p : r2.params)
        if (p.mut_) {
          for (auto& q : m.params)
            if (q.mut_) q = p;
        }
      if (!m.out_aff) continue;
      plan.elided.insert(r1.out_buf);
      absorbed_name[i] = r2.name;
      absorbed.insert(i + 1);
      nests[i] = m;
    }
  }
}

// gather / copy kernels read only by contractions are evaluated inside those contractions'
// tile loaders (implicit GEMM): no launch, no buffer
void fold_gathers_into_contractions(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (opt.gemm && opt.gemm_fold && have_table) {
    for (size_t p = 0; p < kernels.size(); ++p) {
      if (!nests[p] || nests[p]->rkind != ReduceKind::None) continue;
      const NestKernel& pk = *nests[p];
      if (role_of(pk.out_buf) != "temp") continue;
      auto rd = readers.find(pk.out_buf);
      if (rd == readers.end() || rd->second.empty()) continue;
      bool ok = true;
      for (size_t r : rd->second) {
        if (r <= p || !nests[r] || !gemm_shaped(*nests[r], opt)) { ok = false; break; }
        auto g = match_gemm(*nests[r]);
        if (!g || (g->a_buf == pk.out_buf) == (g->b_buf == pk.out_buf)) { ok = false; break; }
      }
      if (!ok) continue;
      auto f = make_fold(pk, elems);
      if (!f || folded.count(f->src)) continue;
      // The gather's own source may be a buffer another pure gather wrote for it alone (a
      // convolution as the reference lowers it applies the unfold view twice): that gather
      // becomes a device function the first one calls, and its buffer goes too.
      for (size_t q = 0; q < p && opt.window; ++q) {
        if (!nests[q] || nests[q]->out_buf != f->src || nests[q]->rkind != ReduceKind::None) continue;
        if (folded_kernels.count(q) || absorbed.count(q) || role_of(f->src) != "temp") break;
        if (readers[f->src] != std::vector<size_t>{p}) break;
        auto fi = make_fold(*nests[q], elems);
        auto in_elems = elems.find(f->src);
        if (!fi || folded.count(fi->src) || in_elems == elems.end()) break;
        std::vector<LoadRef> pl;
        collect_loads(*pk.value, pl);
        bool ok = true;
        for (const auto& lr : pl) {
          auto a = affine_of(*lr.load->args[1]);
          if (!a) { ok = false; break; }
          if (!lr.guarded && max_abs_index(*a, pk.loops, nullptr) >= static_cast<int64_t>(in_elems->second)) ok = false;
        }
        if (!ok) break;
        const NestKernel& inner = *nests[q];
        f->small = f->small && fi->small;
        const std::string IT = f->small ? "int" : "long long";
        f->prelude = gather_fn_text(inner, fi->src, nullptr, IT);
        ExprRenderer er;
        er.load_hook = [&](const Node& ld, std::string* out) {
          if (ld.args[0]->op != Op::Var || ld.args[0]->name != inner.out_buf) return false;
          *out = gather_call(inner, fi->src, *ld.args[1], pk.loops, IT);
          return true;
        };
        f->expr = er.expr(*pk.value);
        f->kernel = inner.name + ", then " + pk.name;
        f->src = fi->src;
        f->src_bytes = fi->src_bytes;
        f->src_stride.clear();
        f->plain = false;
        f->ranged_bytes = 0;              // (the expression now calls the inner gather's function)
        f->value = nullptr;
        folded_kernels.insert(q);
        plan.elided.insert(inner.out_buf);
        break;
      }
      folded[pk.out_buf] = *f;
      folded_kernels.insert(p);
      plan.elided.insert(pk.out_buf);
    }
  }
}

// A short reduce over windows that pure gather kernels laid out for it (max-pool, avg-pool:
// unfold, copy, reduce over the window axis) reads the source through the gathers' index
// maps instead: the window buffers are never written.
void read_windows_through_their_gathers(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (opt.fuse && opt.window && have_table) {
    std::map<std::string, size_t> writer;
    for (size_t q = 0; q < kernels.size(); ++q)
      if (nests[q] && !folded_kernels.count(q) && !absorbed.count(q)) writer[nests[q]->out_buf] = q;
    // a gather that reads `buf` stays inside it, and walks it almost contiguously as the
    // innermost loop outside the window advances
    auto gather_ok = [&](const NestKernel& g, int64_t K) {
      if (!make_fold(g, elems)) return false;
      std::vector<LoadRef> loads;
      collect_loads(*g.value, loads);
      int64_t tail = 1;
      size_t t = g.loops.size();
      while (t > 0 && tail < K) tail *= g.loops[--t].extent;
      if (tail != K || t == 0) return false;
      while (t > 0 && g.loops[t - 1].extent == 1) --t;
      if (t == 0) return false;
      const auto src_elems = elems.find(loads[0].load->args[0]->name);
      for (const auto& lr : loads) {
        auto a = affine_of(*lr.load->args[1]);
        if (!a || std::llabs(a->of(g.loops[t - 1].var)) > 8) return false;
        if (!lr.guarded && (src_elems == elems.end() ||
                            max_abs_index(*a, g.loops, nullptr) >= static_cast<int64_t>(src_elems->second)))
          return false;
      }
      return true;
    };
    for (size_t r = 0; r < kernels.size(); ++r) {
      if (!nests[r] || folded_kernels.count(r) || absorbed.count(r)) continue;
      const NestKernel& rk = *nests[r];
      if (rk.rkind == ReduceKind::None || !rk.out_aff || rk.rloop.extent > 64 || rk.rloop.extent < 2) continue;
      if (rk.acc_dtype.ty != Ty::F32 || rk.out_dtype.ty != Ty::F32 || gemm_shaped(rk, opt)) continue;
      std::vector<LoadRef> loads;
      collect_loads(*rk.value, loads);
      std::string T;
      bool ok = !loads.empty();
      for (const auto& lr : loads) {
        if (lr.load->args[0]->op != Op::Var || lr.load->count != 1) { ok = false; break; }
        const std::string& b = lr.load->args[0]->name;
        auto w = writer.find(b);
        if (role_of(b) != "temp" || w == writer.end() || w->second >= r) continue;
        if (!T.empty() && T != b) { ok = false; break; }
        T = b;
      }
      if (!ok || T.empty() || readers[T] != std::vector<size_t>{r}) continue;
      const auto t_elems = elems.find(T);
      for (const auto& lr : loads) {
        if (lr.load->args[0]->name != T) continue;
        auto a = affine_of(*lr.load->args[1]);
        if (!a || a->of(rk.rloop.var) != 1 || t_elems == elems.end() ||
            max_abs_index(*a, rk.loops, &rk.rloop) >= static_cast<int64_t>(t_elems->second))
          ok = false;
      }
      if (!ok) continue;
      std::vector<size_t> chain;
      std::string buf = T;
      while (chain.size() < 3) {
        auto w = writer.find(buf);
        if (w == writer.end() || role_of(buf) != "temp") break;
        const size_t q = w->second;
        if (nests[q]->rkind != ReduceKind::None || !gather_ok(*nests[q], rk.rloop.extent)) break;
        if (!chain.empty() && readers[buf] != std::vector<size_t>{chain.back()}) break;
        chain.push_back(q);
        std::vector<LoadRef> gl;
        collect_loads(*nests[q]->value, gl);
        buf = gl[0].load->args[0]->name;
      }
      if (chain.empty()) continue;
      // The source itself may be a cheap elementwise function of a buffer that stays in memory
      // anyway (the activation max(z, 0) of a pre-activation z that the backward pass reads): the
      // windows then read z and apply the function, and the activation is never stored.
      if (opt.rematerialize && chain.size() < 3) {
        auto w = writer.find(buf);
        if (w != writer.end() && role_of(buf) == "temp" && readers[buf] == std::vector<size_t>{chain.back()}) {
          const size_t q = w->second;
          const NestKernel& e = *nests[q];
          std::function<size_t(const Node&)> size_of = [&](const Node& n) {
            size_t c = 1;
            for (const auto& a : n.args)
              if (a && n.op != Op::Load) c += size_of(*a);
            return c;
          };
          std::vector<LoadRef> el;
          if (e.rkind == ReduceKind::None && e.value) collect_loads(*e.value, el);
          bool ok_e = !el.empty() && el.size() <= 2 && size_of(*e.value) <= 8 && e.out_aff && make_fold(e, elems, true).has_value();
          std::string z;
          for (const auto& lr : el) {
            if (!ok_e) break;
            auto a = affine_of(*lr.load->args[1]);
            ok_e = a && *a == *e.out_aff && !lr.guarded && lr.load->args[0]->op == Op::Var;    // element for element
            if (ok_e) z = lr.load->args[0]->name;
          }
          if (ok_e) {
            // z is kept: an input or output of the program, or a temp that a kernel behind r reads
            bool kept = role_of(z) != "temp";
            for (size_t c : readers[z]) kept = kept || c > r;
            // ... and nothing between its writer and r overwrites it
            for (size_t m = q + 1; m <= r && kept; ++m)
              if (nests[m] && nests[m]->out_buf == z && !folded_kernels.count(m) && !absorbed.count(m)) kept = false;
            if (kept) {
              chain.push_back(q);
              buf = z;
            }
          }
        }
      }
      windows[r] = chain;
      for (size_t q : chain) {
        folded_kernels.insert(q);
        writer.erase(nests[q]->out_buf);
        plan.elided.insert(nests[q]->out_buf);
      }
    }
  }
}

// A contraction whose result only a run of kernels adding up shifted reads of it sees (the
// input gradient of a convolution) is one window contraction with those kernels.
void join_shifted_sums_with_their_contraction(Planning& st) {
  [[maybe_unused]] const GenOptions& opt = st.opt;
  [[maybe_unused]] ProgramPlan& plan = st.plan;
  [[maybe_unused]] auto& kernels = st.kernels;
  [[maybe_unused]] auto& elems = st.elems;
  [[maybe_unused]] const bool have_table = st.have_table;
  [[maybe_unused]] auto& readers = st.readers;
  [[maybe_unused]] auto& nests = st.nests;
  [[maybe_unused]] auto& absorbed = st.absorbed;
  [[maybe_unused]] auto& absorbed_name = st.absorbed_name;
  [[maybe_unused]] auto& folded = st.folded;
  [[maybe_unused]] auto& folded_kernels = st.folded_kernels;
  [[maybe_unused]] auto& windows = st.windows;
  [[maybe_unused]] auto& scattered = st.scattered;
  [[maybe_unused]] auto& partly_written = st.partly_written;
  [[maybe_unused]] auto role_of = [&](const std::string& name) { return st.role_of(name); };
  if (opt.gemm && opt.gemm_window && opt.fuse && opt.reindex && have_table && opt.gemm_bm == 0 && opt.gemm_split_k <= 1) {
    ProgramView pv;
    pv.nests = &nests;
    pv.readers = &readers;
    pv.elems = &elems;
    pv.role_of = role_of;
    pv.folded_gather = [&](const std::string& buf) -> const NestKernel* {
      for (size_t q : folded_kernels)
        if (nests[q] && nests[q]->out_buf == buf) return &*nests[q];
      return nullptr;
    };
    pv.taken = [&](size_t q) {
      if (folded_kernels.count(q) || absorbed.count(q) || windows.count(q)) return true;
      for (const auto& w : windows)
        if (std::find(w.second.begin(), w.second.end(), q) != w.second.end()) return true;
      return false;
    };
    for (size_t q = 0; q + 1 < kernels.size(); ++q) {
      if (!nests[q] || absorbed_name.count(q) || !gemm_shaped(*nests[q], opt)) continue;
      const Node& v = *nests[q]->value;
      bool plain = v.op == Op::Mul;
      for (size_t o = 0; plain && o < 2; ++o)
        plain = v.args[o]->op == Op::Load && v.args[o]->args[0]->op == Op::Var &&
                (!folded.count(v.args[o]->args[0]->name) || folded.at(v.args[o]->args[0]->name).prelude.empty());
      if (!plain) continue;
      auto sw = try_emit_scattered_window(q, pv, options_for_launch(opt, *kernels[q]));
      if (!sw) continue;
      for (size_t c = q + 1; c < sw->next; ++c) absorbed.insert(c);
      for (const auto& b : sw->elided) plan.elided.insert(b);
      if (sw->partial) partly_written.insert(nests[sw->next - 1]->name);
      scattered[q] = std::move(*sw);
    }
  }
}

}  // namespace eh
