// Structural analysis of lowered kernels: recognises the loop nests the reference's lowerer
// emits (src/lowerer/loop_gen.rs:51-233) and turns index expressions into affine forms, so a
// schedule can be chosen instead of replaying the sequential loops.
#pragma once

#include <map>
#include <optional>
#include <string>
#include <vector>

#include "ast.hpp"

namespace eh {

// Index arithmetic on caller-supplied constants: an overflow is an error, never wrapped.
inline int64_t mul_ck(int64_t a, int64_t b) {
  int64_t r;
  if (__builtin_mul_overflow(a, b, &r)) throw Error("integer overflow in index arithmetic: sizes of this magnitude are not supported");
  return r;
}
inline int64_t add_ck(int64_t a, int64_t b) {
  int64_t r;
  if (__builtin_add_overflow(a, b, &r)) throw Error("integer overflow in index arithmetic: sizes of this magnitude are not supported");
  return r;
}

// value = c + sum(coef[var] * var)
struct Affine {
  int64_t c = 0;
  std::map<std::string, int64_t> coef;
  int64_t of(const std::string& v) const {
    auto it = coef.find(v);
    return it == coef.end() ? 0 : it->second;
  }
  bool operator==(const Affine& o) const { return c == o.c && coef == o.coef; }
};

// Integer affine form of an index expression over loop variables; nullopt when the
// expression is not affine (Rem/Idiv, loads, float literals ...).
std::optional<Affine> affine_of(const Node& n);

struct Loop {
  std::string var;
  int64_t extent = 0;
};

enum class ReduceKind { None, Sum, Max, Min, Prod };

// One lowered kernel in canonical form.
//   elementwise / copy:  for loops...: out[out_index] = value
//   reduce:              for loops...: acc = identity; for rloop: acc = combine(acc, value);
//                        out[out_index] = acc
struct NestKernel {
  std::string name;
  std::vector<Param> params;
  std::vector<Loop> loops;       // enclosing loops, outermost first (without the reduce loop)
  ReduceKind rkind = ReduceKind::None;
  Loop rloop;                    // valid when rkind != None
  NodePtr identity;              // Const node, valid when rkind != None
  DType acc_dtype;
  NodePtr value;                 // element expression (holds Load nodes)
  std::string out_buf;
  NodePtr out_index;
  std::optional<Affine> out_aff;
  DType out_dtype;               // element type of the output buffer
};

// Recognises the canonical forms above; nullopt for anything else (scatter, scan, hand-tiled
// or already parallelised kernels), which are rendered statement by statement instead.
std::optional<NestKernel> extract_nest(const Node& kernel);

// `e` as `combine(acc, value)` for one of the reference's reduce / scan operators
// (src/graph/node.rs:63-77): sum, product, max, select-min, or the fused multiply-add form.
bool match_combine(const Node& e, const std::string& acc, ReduceKind* kind, NodePtr* value);

// Every Load in an expression, in evaluation order, with whether it sits under a Select branch.
struct LoadRef {
  const Node* load;
  bool guarded;
};
void collect_loads(const Node& expr, std::vector<LoadRef>& out, bool guarded = false);

// Refuses (eh::Error) a program, kernel or statement whose sizes are beyond what the planner's
// integer arithmetic is laid out for; see the bounds in analysis.cpp.  Everything that takes
// caller-supplied ASTs calls this first.
void validate_sizes(const Node& n);

// Largest absolute element index an affine form can reach over the given loops.
int64_t max_abs_index(const Affine& a, const std::vector<Loop>& loops, const Loop* rloop);

}  // namespace eh
