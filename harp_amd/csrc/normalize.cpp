#include "normalize.hpp"

#include <algorithm>
#include <cstring>
#include <limits>
#include <optional>
#include <set>

#include "analysis.hpp"

namespace eh {

NodePtr substitute_vars(const NodePtr& n, const std::map<std::string, NodePtr>& m) {
  if (n->op == Op::Var) {
    auto it = m.find(n->name);
    return it == m.end() ? n : it->second;
  }
  bool changed = false;
  std::vector<NodePtr> args;
  args.reserve(n->args.size());
  for (const auto& a : n->args) {
    NodePtr r = substitute_vars(a, m);
    changed = changed || r != a;
    args.push_back(std::move(r));
  }
  if (!changed) return n;
  auto c = std::make_shared<Node>(*n);
  c->args = std::move(args);
  return c;
}

namespace {

bool int_const(const Node& n, int64_t* v) {
  if (n.op != Op::Const || n.dtype.is_float()) return false;
  *v = n.ival;
  return true;
}

bool int_type(const DType& d) {
  switch (d.ty) {
    case Ty::I8: case Ty::I16: case Ty::I32: case Ty::I64: case Ty::U8: case Ty::U16: case Ty::U32: case Ty::U64:
    case Ty::Int:
      return true;
    default:
      return false;
  }
}

NodePtr with_args(const Node& n, std::vector<NodePtr> args) {
  auto c = std::make_shared<Node>(n);
  c->args = std::move(args);
  return c;
}

NodePtr int_like(const Node& like, int64_t v) {
  auto c = std::make_shared<Node>(Op::Const);
  c->dtype = like.dtype;
  c->ival = v;
  return c;
}

bool mentions(const Node& n, const std::string& var) {
  if ((n.op == Op::Var || n.op == Op::Assign) && n.name == var) return true;
  for (const auto& a : n.args)
    if (mentions(*a, var)) return true;
  return false;
}

bool assigns(const Node& n, const std::string& var) {
  if ((n.op == Op::Assign || n.op == Op::Range) && n.name == var) return true;
  for (const auto& a : n.args)
    if (assigns(*a, var)) return true;
  return false;
}

// c + sum(coef * var), variables in name order
NodePtr affine_to_node(const Affine& a) {
  NodePtr sum;
  for (const auto& kv : a.coef) {
    if (kv.second == 0) continue;
    NodePtr t = kv.second == 1 ? make_var(kv.first) : make(Op::Mul, {make_var(kv.first), make_i64(kv.second)});
    sum = sum ? make(Op::Add, {sum, t}) : t;
  }
  if (!sum) return make_i64(a.c);
  return a.c == 0 ? sum : make(Op::Add, {sum, make_i64(a.c)});
}

// Shifts by a constant back to multiplications (the reference only ever produces left shifts,
// from `x * 2^n`), and integer constant subtrees folded.
NodePtr fold_expr(const NodePtr& n) {
  if (n->args.empty()) return n;
  bool changed = false;
  std::vector<NodePtr> args;
  args.reserve(n->args.size());
  for (const auto& a : n->args) {
    NodePtr r = fold_expr(a);
    changed = changed || r != a;
    args.push_back(std::move(r));
  }
  NodePtr cur = changed ? with_args(*n, args) : n;
  int64_t a = 0, b = 0;
  if (cur->op == Op::Shl && cur->args.size() == 2 && int_const(*cur->args[1], &b) && b >= 0 && b < 62) {
    if (int_const(*cur->args[0], &a)) return int_like(*cur->args[0], mul_ck(a, int64_t{1} << b));
    return make(Op::Mul, {cur->args[0], int_like(*cur->args[1], int64_t{1} << b)});
  }
  if (cur->args.size() == 2 && int_const(*cur->args[0], &a) && int_const(*cur->args[1], &b)) {
    switch (cur->op) {
      case Op::Add: return int_like(*cur->args[0], add_ck(a, b));
      case Op::Mul: return int_like(*cur->args[0], mul_ck(a, b));
      case Op::Max: return int_like(*cur->args[0], std::max(a, b));
      case Op::Idiv: if (b != 0 && b != -1) return int_like(*cur->args[0], a / b); break;
      case Op::Rem: if (b != 0 && b != -1) return int_like(*cur->args[0], a % b); break;
      default: break;
    }
  }
  return cur;
}

bool is_empty_stmt(const Node& n) {
  if (n.op == Op::Block) return n.args.empty();
  if (n.op == Op::Range) {
    int64_t s, e;
    return int_const(*n.args[0], &s) && int_const(*n.args[2], &e) && s >= e;
  }
  return false;
}

NodePtr make_block(std::vector<NodePtr> stmts, std::vector<std::pair<std::string, DType>> decls) {
  if (decls.empty() && stmts.size() == 1) return stmts[0];
  auto b = std::make_shared<Node>(Op::Block);
  b->args = std::move(stmts);
  b->decls = std::move(decls);
  return b;
}

NodePtr make_loop(const Node& like, const std::string& var, NodePtr start, NodePtr step, NodePtr stop, NodePtr body) {
  auto r = std::make_shared<Node>(Op::Range);
  r->name = var;
  r->parallel = like.parallel;
  r->args = {std::move(start), std::move(step), std::move(stop), std::move(body)};
  return r;
}

struct Normalizer {
  std::set<std::string> int_vars;     // loop variables and integer block variables of the kernel
  std::set<std::string> rolled;       // loop variables made by rolling repeated statements back into a loop
  int fresh = 0;

  void collect_int_vars(const Node& n) {
    if (n.op == Op::Range) int_vars.insert(n.name);
    for (const auto& d : n.decls)
      if (int_type(d.second)) int_vars.insert(d.first);
    for (const auto& p : n.params)
      if (p.kind != VarKind::Normal || int_type(p.dtype)) int_vars.insert(p.name);
    for (const auto& a : n.args) collect_int_vars(*a);
  }

  // affine over integer variables only
  std::optional<Affine> int_affine(const Node& e) const {
    auto a = affine_of(e);
    if (!a) return std::nullopt;
    for (const auto& kv : a->coef)
      if (!int_vars.count(kv.first)) return std::nullopt;
    return a;
  }

  // ---- rolling a block of repeated statements back into a loop ------------------------------

  // One template for `copies` (the same statement or expression in each repetition) over the new
  // loop variable `u`, or null.  Integer positions are compared by their affine forms, so that a
  // copy the reference's simplifier rewrote (`0 * 1024 + j` to `j`) still matches its siblings.
  NodePtr unify(const std::vector<NodePtr>& copies, const std::string& u, bool int_pos) const {
    const Node& f = *copies[0];
    bool same = true;
    for (size_t t = 1; t < copies.size() && same; ++t) same = copies[t] == copies[0];
    if (same) return copies[0];
    if (int_pos) {
      std::vector<Affine> affs;
      for (const auto& c : copies) {
        auto a = int_affine(*c);
        if (!a) break;
        affs.push_back(*a);
      }
      if (affs.size() == copies.size()) {
        const int64_t d = affs[1].c - affs[0].c;
        for (size_t t = 0; t < affs.size(); ++t)
          if (affs[t].coef != affs[0].coef || affs[t].c != affs[0].c + d * static_cast<int64_t>(t)) return nullptr;
        bool identical = d == 0;
        for (size_t t = 1; t < copies.size() && identical; ++t) identical = shape_of(*copies[t]) == shape_of(f);
        if (identical) return copies[0];               // same form as well as same value: keep the text
        Affine r = affs[0];
        if (d != 0) r.coef[u] += d;
        return affine_to_node(r);
      }
    }
    for (const auto& c : copies) {
      if (c->op != f.op || c->name != f.name || !(c->dtype == f.dtype) || c->count != f.count ||
          c->parallel != f.parallel || c->args.size() != f.args.size() || c->decls.size() != f.decls.size())
        return nullptr;
      for (size_t i = 0; i < f.decls.size(); ++i)
        if (c->decls[i].first != f.decls[i].first || !(c->decls[i].second == f.decls[i].second)) return nullptr;
    }
    if (f.op == Op::Const) {
      if (f.dtype.is_float()) {
        for (const auto& c : copies)
          if (std::memcmp(&c->fval, &f.fval, sizeof f.fval) != 0) return nullptr;
        return copies[0];
      }
      const int64_t d = copies[1]->ival - f.ival;
      for (size_t t = 0; t < copies.size(); ++t)
        if (copies[t]->ival != f.ival + d * static_cast<int64_t>(t)) return nullptr;
      if (d == 0) return copies[0];
      return make(Op::Add, {copies[0], make(Op::Mul, {make_var(u), int_like(f, d)})});
    }
    if (f.args.empty()) return copies[0];                 // a variable (names compared above), a barrier
    std::vector<NodePtr> args;
    bool changed = false;
    for (size_t i = 0; i < f.args.size(); ++i) {
      std::vector<NodePtr> sub;
      for (const auto& c : copies) sub.push_back(c->args[i]);
      bool pos = int_pos;
      switch (f.op) {
        case Op::Load: case Op::Store: case Op::AtomicAdd: case Op::AtomicMax: case Op::SharedLoad: case Op::SharedStore:
          pos = i == 1;
          break;
        case Op::Assign: pos = int_vars.count(f.name) > 0; break;
        case Op::Range: pos = i < 3; break;
        case Op::Block: case Op::If: case Op::Select: pos = false; break;
        case Op::Lt: pos = true; break;                    // guards compare indices
        default: break;
      }
      NodePtr r = unify(sub, u, pos);
      if (!r) return nullptr;
      changed = changed || r != f.args[i];
      args.push_back(std::move(r));
    }
    return changed ? with_args(f, std::move(args)) : copies[0];
  }

  // The form of a statement with its integer literals blanked: repetitions of an unrolled loop
  // share it.
  uint64_t shape_of(const Node& n) const {
    uint64_t h = 1469598103934665603ull;
    auto mix = [&](uint64_t v) {
      h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
    };
    mix(static_cast<uint64_t>(n.op));
    for (unsigned char c : n.name) mix(c);
    mix(static_cast<uint64_t>(n.dtype.ty));
    mix(static_cast<uint64_t>(n.count));
    mix(n.args.size());
    mix(n.decls.size());
    if (n.op == Op::Const && n.dtype.is_float()) {
      uint64_t bits;
      std::memcpy(&bits, &n.fval, sizeof bits);
      mix(bits);
    }
    for (size_t i = 0; i < n.args.size(); ++i) {
      // an integer position counts by its affine coefficients, not by its spelling: the
      // reference's simplifier rewrites one repetition (`o + 0` to `o`) and not its siblings
      bool pos = false;
      switch (n.op) {
        case Op::Load: case Op::Store: case Op::AtomicAdd: case Op::AtomicMax: case Op::SharedLoad: case Op::SharedStore:
          pos = i == 1;
          break;
        case Op::Assign: pos = int_vars.count(n.name) > 0; break;
        case Op::Range: pos = i < 3; break;
        default: break;
      }
      std::optional<Affine> a;
      if (pos) a = int_affine(*n.args[i]);
      if (a) {
        mix(0xaff1e);
        for (const auto& kv : a->coef) {
          if (kv.second == 0) continue;
          for (unsigned char c : kv.first) mix(c);
          mix(static_cast<uint64_t>(kv.second));
        }
      } else {
        mix(shape_of(*n.args[i]));
      }
    }
    return h;
  }

  // A block whose statements are k >= 2 repetitions of p statements that differ only by integers
  // in arithmetic progression (what full unrolling leaves, src/opt/ast/transforms.rs:238-361)
  // becomes `for u in 0..k { the p statements over u }`.  Variables the block declares move into
  // the loop body, which is sound when every repetition assigns them before it reads them.
  // `n` with the loops named in `m` (and every use of their variables) renamed
  static NodePtr rename_loops(const NodePtr& n, const std::map<std::string, std::string>& m) {
    if (n->op == Op::Var) {
      auto it = m.find(n->name);
      return it == m.end() ? n : make_var(it->second);
    }
    bool changed = false;
    std::vector<NodePtr> args;
    args.reserve(n->args.size());
    for (const auto& a : n->args) {
      NodePtr r = rename_loops(a, m);
      changed = changed || r != a;
      args.push_back(std::move(r));
    }
    auto it = n->op == Op::Range ? m.find(n->name) : m.end();
    if (!changed && it == m.end()) return n;
    auto c = std::make_shared<Node>(*n);
    c->args = std::move(args);
    if (it != m.end()) c->name = it->second;
    return c;
  }
  void rolled_loops_in(const Node& n, std::vector<std::string>* out) const {
    if (n.op == Op::Range && rolled.count(n.name)) out->push_back(n.name);
    for (const auto& a : n.args) rolled_loops_in(*a, out);
  }

  NodePtr reroll(const std::vector<NodePtr>& stmts, const std::vector<std::pair<std::string, DType>>& decls) {
    const size_t n = stmts.size();
    // the smallest period of the statements' forms (failure function over their hashes); a
    // nest of unrolled loops repeats at multiples of it
    std::vector<uint64_t> sig(n);
    for (size_t j = 0; j < n; ++j) sig[j] = shape_of(*stmts[j]);
    std::vector<size_t> fail(n, 0);
    for (size_t j = 1, k = 0; j < n; ++j) {
      while (k > 0 && sig[j] != sig[k]) k = fail[k - 1];
      if (sig[j] == sig[k]) ++k;
      fail[j] = k;
    }
    const size_t p0 = n - fail[n - 1];
    if (n % p0 != 0 || p0 == n) return nullptr;
    for (size_t p = p0; p * 2 <= n; p += p0) {
      if (n % p) continue;
      const size_t k = n / p;
      bool decls_ok = true;
      for (const auto& d : decls) {
        for (size_t j = 0; j < p; ++j) {
          const Node& s = *stmts[j];
          if (!mentions(s, d.first)) continue;
          decls_ok = decls_ok && s.op == Op::Assign && s.name == d.first && !mentions(*s.args[0], d.first);
          break;
        }
      }
      if (!decls_ok) continue;
      const std::string u = "eh_u" + std::to_string(fresh);
      std::vector<NodePtr> body;
      for (size_t j = 0; j < p; ++j) {
        std::vector<NodePtr> copies;
        for (size_t t = 0; t < k; ++t) copies.push_back(stmts[t * p + j]);
        NodePtr tpl = unify(copies, u, false);
        if (!tpl) break;
        body.push_back(std::move(tpl));
      }
      if (body.size() != p) continue;
      ++fresh;
      int_vars.insert(u);
      rolled.insert(u);
      Node like(Op::Range);
      like.parallel = "sequential";
      return loop(make_loop(like, u, make_i64(0), make_i64(1), make_i64(static_cast<int64_t>(k)), block(body, decls)));
    }
    return nullptr;
  }

  // ---- an interchanged strip-mined pair -----------------------------------------------------------

  // `n` with the pair (u, r) replaced by one variable w = u + T * r, or null: every integer
  // position (an index, a bound, a compared value) that mentions u or r must be affine with
  // coefficient(r) == T * coefficient(u); u and r may appear nowhere else.  With `canon` set and no
  // pair given (u empty) the integer positions are only rewritten into their canonical affine
  // text, so that two bodies that differ in spelling compare equal.
  NodePtr repair(const NodePtr& n, const std::string& u, const std::string& r, int64_t T, const std::string& w, bool pos,
                 bool* ok) const {
    if (pos) {
      auto a = int_affine(*n);
      if (a) {
        Affine out = *a;
        if (!u.empty()) {
          const int64_t cu = a->of(u), cr = a->of(r);
          if (cr != cu * T) {
            *ok = false;
            return n;
          }
          out.coef.erase(u);
          out.coef.erase(r);
          if (cu != 0) out.coef[w] += cu;
        }
        return affine_to_node(out);
      }
    }
    if (n->op == Op::Var && !u.empty() && (n->name == u || n->name == r)) {
      *ok = false;
      return n;
    }
    if (n->args.empty()) return n;
    std::vector<NodePtr> args;
    bool changed = false;
    for (size_t i = 0; i < n->args.size(); ++i) {
      bool p = false;
      switch (n->op) {
        case Op::Load: case Op::Store: case Op::AtomicAdd: case Op::AtomicMax: case Op::SharedLoad: case Op::SharedStore:
          p = i == 1;
          break;
        case Op::Assign: p = int_vars.count(n->name) > 0; break;
        case Op::Range: p = i < 3; break;
        case Op::Lt: p = true; break;
        default: break;
      }
      NodePtr x = repair(n->args[i], u, r, T, w, p, ok);
      changed = changed || x != n->args[i];
      args.push_back(std::move(x));
    }
    return changed ? with_args(*n, std::move(args)) : n;
  }

  std::string canonical_text(const NodePtr& n) const {
    bool ok = true;
    return to_text(*repair(n, "", "", 0, "", false, &ok));
  }

  // The one statement of a loop body, single-statement blocks without declarations unwrapped.
  static const Node* sole_statement(const Node* b) {
    while (b->op == Op::Block && b->decls.empty() && b->args.size() == 1) b = b->args[0].get();
    return b;
  }

  // ---- loops ----------------------------------------------------------------------------------

  // `decls` without `var`; false when it is not declared there
  static bool drop_decl(std::vector<std::pair<std::string, DType>>* decls, const std::string& var) {
    for (auto it = decls->begin(); it != decls->end(); ++it)
      if (it->first == var) {
        decls->erase(it);
        return true;
      }
    return false;
  }

  // The loop after every rewrite that applies to it (its body is already normal).
  NodePtr loop(NodePtr r) {
    for (;;) {
      int64_t s = 0, step = 0, e = 0;
      const bool consts = int_const(*r->args[0], &s) && int_const(*r->args[1], &step) && int_const(*r->args[2], &e);
      const NodePtr& body = r->args[3];
      if (!consts || step < 1) return r;
      // strip-mined pair: for o in s..e step T { for i in 0..T { v = o + i; rest } } -> for v in s..e { rest }
      // (tile_loop, src/opt/ast/transforms.rs:393-500), or with a guard: for o in 0..G { for i in 0..T {
      // v = o * T + i; if (v < E) { rest } } } -> for v in 0..E { rest } (tile_loop_with_guard, :520-630)
      if (body->op == Op::Range) {
        const Node& in = *body;
        int64_t is = 0, istep = 0, T = 0;
        const Node& ib = *in.args[3];
        if (int_const(*in.args[0], &is) && int_const(*in.args[1], &istep) && int_const(*in.args[2], &T) && is == 0 &&
            istep == 1 && T >= 1 && ib.op == Op::Block && ib.args.size() >= 2 && ib.args[0]->op == Op::Assign) {
          const std::string v = ib.args[0]->name;         // a copy: `r` is replaced below, and its body with it
          auto a = int_affine(*ib.args[0]->args[0]);
          auto decls = ib.decls;
          bool clean = a && a->c == 0 && a->coef.size() == 2 && a->of(in.name) == 1 && drop_decl(&decls, v);
          for (size_t q = 1; q < ib.args.size() && clean; ++q)
            clean = !mentions(*ib.args[q], r->name) && !mentions(*ib.args[q], in.name) && !assigns(*ib.args[q], v);
          if (clean && a->of(r->name) == 1 && step == T && (e - s) % T == 0) {
            std::vector<NodePtr> rest(ib.args.begin() + 1, ib.args.end());
            r = make_loop(*r, v, r->args[0], make_i64(1), r->args[2], block(rest, decls));
            int_vars.insert(v);
            continue;
          }
          if (clean && a->of(r->name) == T && step == 1 && s == 0 && T >= 2) {
            const Node& g = *ib.args[1];
            int64_t E = 0;
            if (ib.args.size() == 2 && g.op == Op::If && g.args.size() == 2 && g.args[0]->op == Op::Lt &&
                g.args[0]->args[0]->op == Op::Var && g.args[0]->args[0]->name == v &&
                int_const(*g.args[0]->args[1], &E) && E <= e * T && E > (e - 1) * T) {
              r = make_loop(*r, v, make_i64(0), make_i64(1), make_i64(E), block({g.args[1]}, decls));
              int_vars.insert(v);
              continue;
            }
            bool guarded = false;
            for (size_t q = 1; q < ib.args.size(); ++q) guarded = guarded || ib.args[q]->op == Op::If;
            if (!guarded) {
              std::vector<NodePtr> rest(ib.args.begin() + 1, ib.args.end());
              r = make_loop(*r, v, make_i64(0), make_i64(1), make_i64(e * T), block(rest, decls));
              int_vars.insert(v);
              continue;
            }
          }
        }
      }
      // a strip-mined pair whose loops were interchanged and the tile loop unrolled and rolled back
      // (u is a loop `reroll` made; two loops the lowerer wrote over a dense tensor have the same
      // index form and stay two): for u in 0..T { for q in 0..n { body(u + T*q) } } -> for w in 0..T*n { body(w) }.  The body
      // is one store (iterations independent) or one accumulation by a commutative, associative
      // operator, whose order every schedule here is free to choose; w ascending is the order the
      // lowerer wrote.
      if (s == 0 && step == 1 && e >= 2 && rolled.count(r->name) && sole_statement(body.get())->op == Op::Range) {
        const Node& in = *sole_statement(body.get());
        int64_t is = 0, istep = 0, n_in = 0;
        const Node* st = sole_statement(in.args[3].get());
        bool shape_ok = int_const(*in.args[0], &is) && int_const(*in.args[1], &istep) && int_const(*in.args[2], &n_in) &&
                        is == 0 && istep == 1 && n_in >= 2;
        if (shape_ok) {
          ReduceKind kind = ReduceKind::None;
          NodePtr value;
          shape_ok = st->op == Op::Store ||
                     (st->op == Op::Assign && !int_vars.count(st->name) && match_combine(*st->args[0], st->name, &kind, &value));
        }
        if (shape_ok) {
          const std::string w = "eh_w" + std::to_string(fresh);
          bool ok = true;
          int_vars.insert(w);
          NodePtr nb = repair(in.args[3], r->name, in.name, e, w, false, &ok);
          if (ok && mentions(*nb, w)) {
            ++fresh;
            r = make_loop(*r, w, make_i64(0), make_i64(1), make_i64(mul_ck(e, n_in)), nb);
            continue;
          }
          int_vars.erase(w);
        }
      }
      // renamed loop variable: for q in s..e { v = q + d; rest } -> for v in s+d..e+d { rest }
      // (the remainder loop of tile_loop; a rolled-back unrolled loop)
      if (body->op == Op::Block && body->args.size() >= 2 && body->args[0]->op == Op::Assign && step == 1) {
        const Node& b = *body;
        const std::string v = b.args[0]->name;
        auto a = int_affine(*b.args[0]->args[0]);
        auto decls = b.decls;
        bool clean = a && a->coef.size() == 1 && a->of(r->name) == 1 && drop_decl(&decls, v);
        for (size_t q = 1; q < b.args.size() && clean; ++q)
          clean = !mentions(*b.args[q], r->name) && !assigns(*b.args[q], v);
        if (clean) {
          std::vector<NodePtr> rest(b.args.begin() + 1, b.args.end());
          r = make_loop(*r, v, make_i64(s + a->c), make_i64(1), make_i64(e + a->c), block(rest, decls));
          int_vars.insert(v);
          continue;
        }
      }
      return r;
    }
  }

  // ---- blocks ---------------------------------------------------------------------------------

  NodePtr block(std::vector<NodePtr> stmts, std::vector<std::pair<std::string, DType>> decls) {
    stmts.erase(std::remove_if(stmts.begin(), stmts.end(), [](const NodePtr& s) { return is_empty_stmt(*s); }),
                stmts.end());
    // Loops that an inner roll made carry fresh names, one per repetition of an enclosing unrolled
    // loop (or of a loop and its remainder): each statement's are renamed by their order in it, so
    // that the repetitions compare equal below.
    if (stmts.size() >= 2) {
      const int id = fresh++;
      for (auto& st : stmts) {
        std::vector<std::string> inner;
        rolled_loops_in(*st, &inner);
        if (inner.empty()) continue;
        std::map<std::string, std::string> m;
        for (size_t k = 0; k < inner.size(); ++k) {
          const std::string to = "eh_c" + std::to_string(id) + "_" + std::to_string(k);
          if (!m.emplace(inner[k], to).second) { m.clear(); break; }     // (a name bound twice in one statement: left alone)
          int_vars.insert(to);
          rolled.insert(to);
        }
        if (!m.empty()) st = rename_loops(st, m);
      }
    }
    // neighbouring loops with the same body over adjoining ranges are one loop; so are two whose
    // ranges adjoin once the second one's variable is shifted (a remainder loop that was moved to
    // start at 0, its offset now inside its body): bodies are compared with their integer
    // positions in canonical affine form
    for (size_t j = 0; j + 1 < stmts.size();) {
      const Node &x = *stmts[j], &y = *stmts[j + 1];
      int64_t xs, xt, xe, ys, yt, ye;
      bool join = x.op == Op::Range && y.op == Op::Range && int_const(*x.args[0], &xs) && int_const(*x.args[1], &xt) &&
                  int_const(*x.args[2], &xe) && int_const(*y.args[0], &ys) && int_const(*y.args[1], &yt) &&
                  int_const(*y.args[2], &ye) && xt == 1 && yt == 1 && xe > xs && ye > ys && x.parallel == y.parallel &&
                  (y.name == x.name || !mentions(*y.args[3], x.name)) && !assigns(*y.args[3], y.name) &&
                  !assigns(*x.args[3], x.name);
      if (join) {
        const int64_t shift = ys - xe;
        if (shift == 0) {
          NodePtr yb = y.name == x.name ? y.args[3] : substitute_vars(y.args[3], {{y.name, make_var(x.name)}});
          join = to_text(*yb) == to_text(*x.args[3]) || canonical_text(yb) == canonical_text(x.args[3]);
        } else {
          NodePtr yb = substitute_vars(y.args[3], {{y.name, make(Op::Add, {make_var(x.name), make_i64(shift)})}});
          join = int_vars.count(x.name) > 0 && canonical_text(yb) == canonical_text(x.args[3]);
        }
      }
      if (!join) {
        ++j;
        continue;
      }
      stmts[j] = make_loop(x, x.name, x.args[0], x.args[1], make_i64(xe + (ye - ys)), x.args[3]);
      stmts.erase(stmts.begin() + static_cast<long>(j) + 1);
    }
    if (stmts.size() >= 2)
      if (NodePtr rolled = reroll(stmts, decls)) return rolled;
    return make_block(std::move(stmts), std::move(decls));
  }

  NodePtr stmt(const NodePtr& n) {
    switch (n->op) {
      case Op::Block: {
        std::vector<NodePtr> stmts;
        for (const auto& a : n->args) stmts.push_back(stmt(a));
        return block(std::move(stmts), n->decls);
      }
      case Op::Range:
        return loop(make_loop(*n, n->name, fold_expr(n->args[0]), fold_expr(n->args[1]), fold_expr(n->args[2]),
                              stmt(n->args[3])));
      case Op::If: {
        std::vector<NodePtr> args = {fold_expr(n->args[0])};
        for (size_t i = 1; i < n->args.size(); ++i) args.push_back(stmt(n->args[i]));
        return with_args(*n, std::move(args));
      }
      default:
        return fold_expr(n);
    }
  }

  // `for v in [0, e) { if (v < c) S }` is `for v in [0, min(e, c)) S`: what is left of a guarded
  // tiling once its tile loops were unrolled and rolled back into one loop over the padded extent.
  NodePtr unguard(const NodePtr& loop) const {
    int64_t s = 0, step = 0, e = 0, c = 0;
    if (loop->op != Op::Range || !int_const(*loop->args[0], &s) || !int_const(*loop->args[1], &step) ||
        !int_const(*loop->args[2], &e) || s != 0 || step != 1)
      return loop;
    const Node* body = loop->args[3].get();
    while (body->op == Op::Block && body->args.size() == 1 && body->decls.empty()) body = body->args[0].get();
    if (body->op != Op::If || body->args.size() != 2) return loop;
    const Node& cond = *body->args[0];
    if (cond.op != Op::Lt || cond.args[0]->op != Op::Var || cond.args[0]->name != loop->name || !int_const(*cond.args[1], &c)) return loop;
    if (assigns(*body->args[1], loop->name)) return loop;
    return make_loop(*loop, loop->name, make_i64(0), make_i64(1), make_i64(std::max<int64_t>(0, std::min(e, c))), body->args[1]);
  }

  // ---- second pass: what the first left behind ------------------------------------------------

  // Integer block variables assigned once from an affine expression are substituted into the
  // statements that follow (a strip-mined pair whose loops were interchanged apart keeps its
  // `v = o + i`), and every loop with constant bounds starts at 0 and steps by 1.
  NodePtr settle(const NodePtr& n) {
    switch (n->op) {
      case Op::Block: {
        std::vector<NodePtr> stmts = n->args;
        auto decls = n->decls;
        for (size_t j = 0; j < stmts.size();) {
          const Node& s = *stmts[j];
          bool sub = s.op == Op::Assign && int_vars.count(s.name) > 0 && int_affine(*s.args[0]).has_value() &&
                     !mentions(*s.args[0], s.name);
          if (sub) {
            bool declared = false;
            for (const auto& d : decls) declared = declared || d.first == s.name;
            sub = declared;
            for (size_t q = 0; q < stmts.size() && sub; ++q)
              sub = q == j || !assigns(*stmts[q], s.name);
            for (size_t q = 0; q < j && sub; ++q) sub = !mentions(*stmts[q], s.name);
          }
          if (!sub) {
            ++j;
            continue;
          }
          const std::string v = s.name;
          const NodePtr e = s.args[0];
          for (size_t q = j + 1; q < stmts.size(); ++q) stmts[q] = substitute_vars(stmts[q], {{v, e}});
          stmts.erase(stmts.begin() + static_cast<long>(j));
          drop_decl(&decls, v);
        }
        for (auto& s : stmts) s = settle(s);
        return make_block(std::move(stmts), std::move(decls));
      }
      case Op::Range: {
        int64_t s = 0, step = 0, e = 0;
        NodePtr body = n->args[3];
        if (int_const(*n->args[0], &s) && int_const(*n->args[1], &step) && int_const(*n->args[2], &e) && step >= 1 &&
            (s != 0 || step != 1) && !assigns(*body, n->name)) {
          const int64_t count = e > s ? (e - s + step - 1) / step : 0;
          Affine a;
          a.c = s;
          a.coef[n->name] = step;
          body = substitute_vars(body, {{n->name, affine_to_node(a)}});
          return unguard(make_loop(*n, n->name, make_i64(0), make_i64(1), make_i64(count), settle(body)));
        }
        return unguard(make_loop(*n, n->name, n->args[0], n->args[1], n->args[2], settle(body)));
      }
      case Op::If: {
        std::vector<NodePtr> args = {n->args[0]};
        for (size_t i = 1; i < n->args.size(); ++i) args.push_back(settle(n->args[i]));
        return with_args(*n, std::move(args));
      }
      default:
        return n;
    }
  }
};

}  // namespace

NodePtr normalize_kernel(const NodePtr& kernel) {
  if (kernel->op != Op::Kernel || kernel->args.size() != 1) return kernel;
  Normalizer nz;
  nz.collect_int_vars(*kernel);
  NodePtr body = nz.stmt(kernel->args[0]);
  body = nz.settle(body);
  body = nz.stmt(body);                       // substitutions may have exposed foldable integers
  if (to_text(*body) == to_text(*kernel->args[0])) return kernel;
  return [&] {
    auto k = std::make_shared<Node>(*kernel);
    k->args = {body};
    return k;
  }();
}

namespace {

// [lo, hi] of an integer expression over variables with known ranges; false when the expression
// is not affine or names a variable without a range
bool int_range(const Node& e, const std::map<std::string, std::pair<int64_t, int64_t>>& env, int64_t* lo, int64_t* hi) {
  auto a = affine_of(e);
  if (!a) return false;
  int64_t l = a->c, h = a->c;
  for (const auto& kv : a->coef) {
    if (kv.second == 0) continue;
    auto it = env.find(kv.first);
    if (it == env.end()) return false;
    const int64_t x = mul_ck(kv.second, it->second.first), y = mul_ck(kv.second, it->second.second);
    l = add_ck(l, std::min(x, y));
    h = add_ck(h, std::max(x, y));
  }
  *lo = l;
  *hi = h;
  return true;
}

double serial_iterations_in(const Node& n, std::map<std::string, std::pair<int64_t, int64_t>>* env) {
  switch (n.op) {
    case Op::Range: {
      // bounds that move with the enclosing loops are bounded over those loops' ranges: the
      // earliest start, the latest stop
      int64_t step = 0, slo = 0, shi = 0, elo = 0, ehi = 0;
      if (!int_const(*n.args[1], &step) || step < 1 || !int_range(*n.args[0], *env, &slo, &shi) ||
          !int_range(*n.args[2], *env, &elo, &ehi))
        return std::numeric_limits<double>::infinity();
      (void)shi;
      (void)elo;
      const double trips = ehi > slo ? static_cast<double>((ehi - slo + step - 1) / step) : 0.0;
      if (trips == 0.0) return 0.0;
      auto saved = env->find(n.name) == env->end() ? std::optional<std::pair<int64_t, int64_t>>() : (*env)[n.name];
      (*env)[n.name] = {slo, ehi - 1};
      const double inner = serial_iterations_in(*n.args[3], env);
      if (saved) (*env)[n.name] = *saved;
      else env->erase(n.name);
      return trips * std::max(1.0, inner);
    }
    case Op::Block: case Op::Kernel: {
      double sum = 0;
      for (const auto& a : n.args) sum += serial_iterations_in(*a, env);
      return sum;
    }
    case Op::If: {
      double m = 0;
      for (size_t i = 1; i < n.args.size(); ++i) m = std::max(m, serial_iterations_in(*n.args[i], env));
      return m;
    }
    default:
      return 0;
  }
}

}  // namespace

double serial_iterations(const Node& n) {
  std::map<std::string, std::pair<int64_t, int64_t>> env;
  return serial_iterations_in(n, &env);
}

}  // namespace eh
