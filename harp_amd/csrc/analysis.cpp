#include "analysis.hpp"

#include <algorithm>
#include <cstdlib>

namespace eh {

namespace {

bool int_const(const Node& n, int64_t* v) {
  if (n.op != Op::Const || n.dtype.is_float()) return false;
  *v = n.ival;
  return true;
}

}  // namespace

std::optional<Affine> affine_of(const Node& n) {
  switch (n.op) {
    case Op::Const: {
      int64_t v;
      if (!int_const(n, &v)) return std::nullopt;
      Affine a;
      a.c = v;
      return a;
    }
    case Op::Var: {
      Affine a;
      a.coef[n.name] = 1;
      return a;
    }
    case Op::Add: {
      auto l = affine_of(*n.args[0]);
      auto r = affine_of(*n.args[1]);
      if (!l || !r) return std::nullopt;
      l->c = add_ck(l->c, r->c);
      for (auto& kv : r->coef) {
        l->coef[kv.first] = add_ck(l->coef[kv.first], kv.second);
        if (l->coef[kv.first] == 0) l->coef.erase(kv.first);
      }
      return l;
    }
    case Op::Mul: {
      auto l = affine_of(*n.args[0]);
      auto r = affine_of(*n.args[1]);
      if (!l || !r) return std::nullopt;
      if (!l->coef.empty() && !r->coef.empty()) return std::nullopt;
      const Affine& k = l->coef.empty() ? *l : *r;   // the constant side
      Affine v = l->coef.empty() ? *r : *l;
      v.c = mul_ck(v.c, k.c);
      for (auto it = v.coef.begin(); it != v.coef.end();) {
        it->second = mul_ck(it->second, k.c);
        it = it->second == 0 ? v.coef.erase(it) : std::next(it);
      }
      return v;
    }
    default:
      return std::nullopt;
  }
}

void collect_loads(const Node& e, std::vector<LoadRef>& out, bool guarded) {
  if (e.op == Op::Load) {
    out.push_back({&e, guarded});
    // an index may itself hold loads (gather); those are evaluated first
    collect_loads(*e.args[1], out, guarded);
    return;
  }
  if (e.op == Op::Select) {
    collect_loads(*e.args[0], out, guarded);
    collect_loads(*e.args[1], out, true);
    collect_loads(*e.args[2], out, true);
    return;
  }
  for (const auto& a : e.args) collect_loads(*a, out, guarded);
}

int64_t max_abs_index(const Affine& a, const std::vector<Loop>& loops, const Loop* rloop) {
  int64_t hi = a.c > 0 ? a.c : 0, lo = a.c < 0 ? a.c : 0;
  auto add = [&](const Loop& l) {
    int64_t k = mul_ck(a.of(l.var), l.extent > 0 ? l.extent - 1 : 0);
    if (k > 0) hi = add_ck(hi, k); else lo = add_ck(lo, k);
  };
  for (const auto& l : loops) add(l);
  if (rloop) add(*rloop);
  return hi > -lo ? hi : -lo;
}

namespace {

// Range with start 0, step 1 and a constant stop.
bool simple_range(const Node& n, Loop* out) {
  if (n.op != Op::Range || n.args.size() != 4) return false;
  int64_t start, step, stop;
  if (!int_const(*n.args[0], &start) || !int_const(*n.args[1], &step) || !int_const(*n.args[2], &stop))
    return false;
  if (start != 0 || step != 1 || stop < 0) return false;
  if (!n.parallel.empty() && n.parallel != "sequential") return false;
  out->var = n.name;
  out->extent = stop;
  return true;
}

bool is_var(const Node& n, const std::string& name) { return n.op == Op::Var && n.name == name; }

bool mentions_var(const Node& n, const std::string& name) {
  if (is_var(n, name)) return true;
  for (const auto& a : n.args)
    if (mentions_var(*a, name)) return true;
  return false;
}

// acc = combine(acc, value): which reduction, and what is combined in.
}  // namespace

bool match_combine(const Node& e, const std::string& acc, ReduceKind* kind, NodePtr* value) {
  auto binary = [&](ReduceKind k) {
    if (is_var(*e.args[0], acc) && !mentions_var(*e.args[1], acc)) {
      *kind = k;
      *value = e.args[1];
      return true;
    }
    if (k != ReduceKind::None && is_var(*e.args[1], acc) && !mentions_var(*e.args[0], acc)) {
      *kind = k;
      *value = e.args[0];
      return true;
    }
    return false;
  };
  switch (e.op) {
    case Op::Add: return binary(ReduceKind::Sum);
    case Op::Mul: return binary(ReduceKind::Prod);
    case Op::Max: return binary(ReduceKind::Max);
    case Op::Fma:
      // fma(a, b, acc) is the rewritten form of acc + a*b
      if (is_var(*e.args[2], acc) && !mentions_var(*e.args[0], acc) && !mentions_var(*e.args[1], acc)) {
        *kind = ReduceKind::Sum;
        *value = make(Op::Mul, {e.args[0], e.args[1]});
        return true;
      }
      return false;
    case Op::Select: {
      // select(acc < v, acc, v)
      const Node& c = *e.args[0];
      if (c.op == Op::Lt && is_var(*c.args[0], acc) && is_var(*e.args[1], acc) &&
          !mentions_var(*e.args[2], acc) && to_text(*c.args[1]) == to_text(*e.args[2])) {
        *kind = ReduceKind::Min;
        *value = e.args[2];
        return true;
      }
      return false;
    }
    default:
      return false;
  }
}

namespace {

bool buffer_param(const std::vector<Param>& ps, const std::string& name, DType* elem) {
  for (const auto& p : ps)
    if (p.name == name && p.dtype.is_ptr()) {
      if (elem) *elem = p.dtype.elem();
      return true;
    }
  return false;
}

// All loads must address kernel pointer parameters directly.
bool loads_ok(const Node& e, const std::vector<Param>& ps) {
  if (e.op == Op::Load) {
    if (e.count != 1 || e.args[0]->op != Op::Var || !buffer_param(ps, e.args[0]->name, nullptr)) return false;
  }
  switch (e.op) {
    case Op::Store: case Op::Assign: case Op::AtomicAdd: case Op::AtomicMax: case Op::Block: case Op::Range:
    case Op::If: case Op::Barrier: case Op::Rand: case Op::Call: case Op::Return: case Op::SharedAlloc:
    case Op::SharedLoad: case Op::SharedStore: case Op::Allocate: case Op::Deallocate: case Op::WmmaMatmul:
    case Op::Wildcard:
      return false;
    default:
      break;
  }
  for (const auto& a : e.args)
    if (!loads_ok(*a, ps)) return false;
  return true;
}

}  // namespace

std::optional<NestKernel> extract_nest(const Node& kernel) {
  if (kernel.op != Op::Kernel || kernel.args.size() != 1) return std::nullopt;
  for (const auto& p : kernel.params)
    if (p.kind != VarKind::Normal || (!p.dtype.is_ptr())) return std::nullopt;  // already parallelised / shape vars
  NestKernel k;
  k.name = kernel.name;
  k.params = kernel.params;
  const Node* cur = kernel.args[0].get();
  // a Block holding a single statement and no declarations is transparent
  auto unwrap = [](const Node* n) {
    while (n->op == Op::Block && n->decls.empty() && n->args.size() == 1) n = n->args[0].get();
    return n;
  };
  cur = unwrap(cur);
  Loop l;
  while (simple_range(*cur, &l)) {
    for (const auto& e : k.loops)
      if (e.var == l.var) return std::nullopt;
    k.loops.push_back(l);
    cur = unwrap(cur->args[3].get());
  }
  const Node* store = nullptr;
  if (cur->op == Op::Store) {
    store = cur;
    k.value = cur->args[2];
  } else if (cur->op == Op::Block && cur->args.size() == 3 && cur->decls.size() == 1) {
    const std::string& acc = cur->decls[0].first;
    const Node& init = *cur->args[0];
    const Node* red = unwrap(cur->args[1].get());
    const Node& post = *cur->args[2];
    if (init.op != Op::Assign || init.name != acc || init.args[0]->op != Op::Const) return std::nullopt;
    if (!simple_range(*red, &k.rloop)) return std::nullopt;
    const Node* body = unwrap(red->args[3].get());
    if (body->op != Op::Assign || body->name != acc) return std::nullopt;
    if (!match_combine(*body->args[0], acc, &k.rkind, &k.value)) return std::nullopt;
    if (post.op != Op::Store || !is_var(*post.args[2], acc)) return std::nullopt;
    for (const auto& e : k.loops)
      if (e.var == k.rloop.var) return std::nullopt;
    k.identity = init.args[0];
    k.acc_dtype = cur->decls[0].second;
    store = &post;
  } else {
    return std::nullopt;
  }
  if (store->args[0]->op != Op::Var) return std::nullopt;
  k.out_buf = store->args[0]->name;
  if (!buffer_param(k.params, k.out_buf, &k.out_dtype)) return std::nullopt;
  for (const auto& p : k.params)
    if (p.name == k.out_buf && !p.mut_) return std::nullopt;
  k.out_index = store->args[1];
  k.out_aff = affine_of(*k.out_index);
  if (!k.out_aff) return std::nullopt;     // scattered stores are left to the statement renderer
  if (k.rkind != ReduceKind::None && k.out_aff->of(k.rloop.var) != 0) return std::nullopt;
  if (!loads_ok(*k.value, k.params)) return std::nullopt;
  // the output must not also be read
  std::vector<LoadRef> loads;
  collect_loads(*k.value, loads);
  for (const auto& lr : loads)
    if (lr.load->args[0]->name == k.out_buf) return std::nullopt;
  // every variable used must be a loop variable
  std::vector<const Node*> stack = {k.value.get(), k.out_index.get()};
  while (!stack.empty()) {
    const Node* n = stack.back();
    stack.pop_back();
    if (n->op == Op::Var) {
      bool known = (k.rkind != ReduceKind::None && n->name == k.rloop.var) ||
                   buffer_param(k.params, n->name, nullptr);
      for (const auto& e : k.loops) known = known || e.var == n->name;
      if (!known) return std::nullopt;
    }
    for (const auto& a : n->args) stack.push_back(a.get());
  }
  return k;
}

namespace {

// Sizes are caller-supplied.  Everything the planner later multiplies -- loop extents, strides,
// footprints, largest reachable indices -- is bounded here once (with checked arithmetic), so
// that the products it forms stay far inside 64 bits: a loop runs at most 2^33 times, a nest at
// most 2^48, a constant is at most 2^46 in magnitude, and no index expression can reach beyond
// 2^46 elements.  Larger programs are refused, not wrapped.
constexpr int64_t kMaxExtent = int64_t{1} << 33, kMaxNest = int64_t{1} << 48, kMaxIndex = int64_t{1} << 46;

void validate_node(const Node& n, std::vector<Loop>& loops, int64_t nest) {
  auto too_big = [](const std::string& what) {
    throw Error(what + " is beyond the sizes this backend plans for: not supported");
  };
  if (n.op == Op::Const && !n.dtype.is_float() && (n.ival > kMaxIndex || n.ival < -kMaxIndex)) too_big("an integer constant");
  if (n.op == Op::Range && n.args.size() == 4) {
    for (int i = 0; i < 3; ++i) validate_node(*n.args[i], loops, nest);
    int64_t extent = 1;
    const Node &s = *n.args[0], &st = *n.args[1], &e = *n.args[2];
    if (s.op == Op::Const && st.op == Op::Const && e.op == Op::Const && !s.dtype.is_float() && !e.dtype.is_float() &&
        !st.dtype.is_float() && st.ival >= 1)
      extent = e.ival > s.ival ? (e.ival - s.ival + st.ival - 1) / st.ival : 0;
    if (extent > kMaxExtent) too_big("the extent of loop '" + n.name + "'");
    const int64_t inner = mul_ck(nest, std::max<int64_t>(extent, 1));
    if (inner > kMaxNest) too_big("the iteration count of the nest around loop '" + n.name + "'");
    loops.push_back({n.name, extent});
    validate_node(*n.args[3], loops, inner);
    loops.pop_back();
    return;
  }
  const bool indexed = (n.op == Op::Load || n.op == Op::Store || n.op == Op::AtomicAdd || n.op == Op::AtomicMax) &&
                       n.args.size() >= 2;
  if (indexed)
    if (auto a = affine_of(*n.args[1]))
      if (max_abs_index(*a, loops, nullptr) > kMaxIndex) too_big("an index of buffer access in a kernel");
  for (const auto& c : n.args) validate_node(*c, loops, nest);
}

}  // namespace

void validate_sizes(const Node& n) {
  for (const auto& b : n.buffers) {
    int64_t numel = 1;
    for (auto d : b.shape) {
      if (d < 0) throw Error("buffer '" + b.name + "' has a negative dimension");
      numel = mul_ck(numel, std::max<int64_t>(d, 1));
      if (numel > kMaxIndex) throw Error("buffer '" + b.name + "' is beyond the sizes this backend plans for: not supported");
    }
  }
  std::vector<Loop> loops;
  validate_node(n, loops, 1);
}

}  // namespace eh
