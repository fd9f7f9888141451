// What the parts of the generator share among themselves (not part of the library's interface):
//   codegen.cpp   expressions, statements, kernels replayed as written
//   stages.cpp    canonical stages and groups, output layouts, folded gathers
//   rewrites.cpp  passes over the lowered kernels before schedules are chosen
//   plan.cpp      plan_program
//   emitters.cpp  source text of the elementwise / reduce schedules
//   launches.cpp  passes over the planned launches (written flags, merging, lanes)
#pragma once

#include <functional>
#include <map>
#include <optional>
#include <set>
#include <string>
#include <vector>

#include "analysis.hpp"
#include "codegen.hpp"
#include "gemm.hpp"
#include "normalize.hpp"
#include "window.hpp"

namespace eh {

// ---- codegen.cpp ------------------------------------------------------------------------------
extern thread_local bool g_guard_branches;      // guarded loads as branches (option guard_branches)
extern thread_local bool g_ranged_loads;        // guarded loads through a buffer resource (option ranged_loads)
std::string ctype(const DType& d);
std::string literal(const Node& n);
Ty infer_ty(const Node& n, const std::map<std::string, Ty>* vars = nullptr);
const char* infix(Op op);
bool holds_load(const Node& n);
std::string hdr(const GenOptions&);

using LoadHook = std::function<bool(const Node& load, std::string* out)>;

struct ExprRenderer {
  LoadHook load_hook;
  const std::map<std::string, Ty>* var_types = nullptr;
  // Conditions of the selects around the expression being rendered.  A load under a select
  // (padding, window edges: `inside ? x[i] : 0`) is not left to a branch: a load in a branch is
  // waited for at the branch's end, so the guarded loads of a work-item would go to memory one
  // after the other, a full latency each.  Both arms are evaluated, the load with its index
  // clamped to element 0 where the condition does not hold (every buffer has one), and the
  // select picks: the loads are independent and in flight together.
  // A load that a hook renders (a value kept in a register, a call of another gather) cannot
  // have its index clamped here: a select that holds one keeps its branch.
  mutable std::vector<std::string> guards;
  mutable bool hooked_under_guard = false;
  mutable int plain_selects = 0;
  // Buffers (name -> bytes, below 2^31) read through a buffer resource `eh_rs_<name>` instead
  // of a pointer: the hardware checks the byte offset against the resource's size and an
  // out-of-range load returns zero.  A guarded fp32 load is then one load whose offset is out
  // of range where the guard fails, and `guard ? load : 0` needs no select; the address is a
  // 32-bit offset, not a 64-bit pointer sum.
  // Only guarded loads take this form (an unguarded load keeps its pointer, so that an index that
  // runs out of its buffer is not quietly turned into a zero), and only under guards that test
  // indices: an offset that waits for another load's value (a mask read from memory) would put the
  // two loads one after the other.
  const std::map<std::string, size_t>* ranged = nullptr;
  mutable int value_guards = 0;         // selects around the current node whose condition holds a load
  bool is_ranged(const Node& n, bool guarded) const {
    return ranged && n.op == Op::Load && n.count == 1 && n.dtype.ty == Ty::F32 && n.args[0]->op == Op::Var &&
           ranged->count(n.args[0]->name) && guarded && value_guards == 0;
  }

  std::string math1(const char* f32, const char* f64, const Node& n) const {
    bool dbl = infer_ty(*n.args[0], var_types) == Ty::F64;
    return std::string(dbl ? f64 : f32) + "(" + expr(*n.args[0]) + ")";
  }

  std::string expr(const Node& n) const {
    // a conjunction of pure conditions is evaluated without short-circuit branches (the compiler
    // otherwise keeps the branches and sinks guarded loads back into them)
    if (n.op == Op::And && !holds_load(n)) return "((bool)" + expr(*n.args[0]) + " & (bool)" + expr(*n.args[1]) + ")";
    if (const char* s = infix(n.op)) return "(" + expr(*n.args[0]) + " " + s + " " + expr(*n.args[1]) + ")";
    switch (n.op) {
      case Op::Const: return literal(n);
      case Op::Var: case Op::Wildcard: return n.name;
      case Op::Max: {
        Ty t = infer_ty(n, var_types);
        std::string a = expr(*n.args[0]), b = expr(*n.args[1]);
        if (t == Ty::F32 || t == Ty::F16 || t == Ty::BF16) return "fmaxf(" + a + ", " + b + ")";
        if (t == Ty::F64) return "fmax(" + a + ", " + b + ")";
        return "((" + a + ") > (" + b + ") ? (" + a + ") : (" + b + "))";
      }
      case Op::Recip:
        return infer_ty(*n.args[0], var_types) == Ty::F64 ? "(1.0 / " + expr(*n.args[0]) + ")"
                                                         : "(1.0f / " + expr(*n.args[0]) + ")";
      case Op::Sqrt: return math1("sqrtf", "sqrt", n);
      case Op::Log2: return math1("log2f", "log2", n);
      case Op::Exp2: return math1("exp2f", "exp2", n);
      case Op::Sin: return math1("sinf", "sin", n);
      case Op::Floor: return math1("floorf", "floor", n);
      case Op::Not: return "(!" + expr(*n.args[0]) + ")";
      case Op::BitNot: return "(~" + expr(*n.args[0]) + ")";
      case Op::Cast: return "(" + ctype(n.dtype) + ")(" + expr(*n.args[0]) + ")";
      case Op::Fma: {
        // The reference renders `fma(a, b, c)` whatever the operands' type
        // (src/backend/renderer.rs:107-109), which in C on float operands is the double-precision
        // function on promoted values, its result converted back on use: product exact, one
        // rounding to double, one to float.  Rendered as exactly that, so that an elementwise
        // kernel in this form stays bit-identical to the C backend's (fmaf rounds once and
        // differs where the double result sits on a float tie).
        const Ty t = infer_ty(n, var_types);
        if (t == Ty::F64) return "fma(" + expr(*n.args[0]) + ", " + expr(*n.args[1]) + ", " + expr(*n.args[2]) + ")";
        return "(" + ctype(DType{t, nullptr, 0}) + ")fma((double)(" + expr(*n.args[0]) + "), (double)(" + expr(*n.args[1]) + "), (double)(" +
               expr(*n.args[2]) + "))";
      }
      case Op::Select: {
        if (g_guard_branches || plain_selects > 0 || (!holds_load(*n.args[1]) && !holds_load(*n.args[2])))
          return "(" + expr(*n.args[0]) + " ? " + expr(*n.args[1]) + " : " + expr(*n.args[2]) + ")";
        const std::string c = expr(*n.args[0]);
        struct ValueGuard {
          int& n;
          bool on;
          ValueGuard(int& c, bool o) : n(c), on(o) { n += on; }
          ~ValueGuard() { n -= on; }
        } value_guard(value_guards, holds_load(*n.args[0]));
        // `inside ? x[i] : 0` through a buffer resource: the load alone
        if (is_ranged(*n.args[1], true) && n.args[2]->op == Op::Const && n.args[2]->dtype.ty == Ty::F32 && n.args[2]->fval == 0.0 &&
            !std::signbit(n.args[2]->fval)) {
          guards.push_back("(bool)" + c);
          const std::string a = expr(*n.args[1]);
          guards.pop_back();
          return a;
        }
        const bool outer_hooked = hooked_under_guard;
        hooked_under_guard = false;
        guards.push_back("(bool)" + c);
        const std::string a = expr(*n.args[1]);
        guards.back() = "(!" + c + ")";
        const std::string b = expr(*n.args[2]);
        guards.pop_back();
        const bool hooked = hooked_under_guard;
        hooked_under_guard = outer_hooked || hooked;
        if (hooked) {
          ++plain_selects;
          const std::vector<std::string> saved = std::move(guards);
          guards.clear();
          const std::string r = "(" + c + " ? " + expr(*n.args[1]) + " : " + expr(*n.args[2]) + ")";
          guards = saved;
          --plain_selects;
          return r;
        }
        return "({ const auto eh_sa = " + a + "; const auto eh_sb = " + b + "; " + c + " ? eh_sa : eh_sb; })";
      }
      case Op::Load: {
        std::string s;
        if (!is_ranged(n, !guards.empty()) && load_hook && load_hook(n, &s)) {
          if (!guards.empty()) hooked_under_guard = true;
          return s;
        }
        if (is_ranged(n, !guards.empty())) {
          const std::string off = "((unsigned)(" + expr(*n.args[1]) + ") << 2)";
          if (guards.empty()) return "eh_ranged_load(eh_rs_" + n.args[0]->name + ", " + off + ")";
          std::string g = guards[0];
          for (size_t i = 1; i < guards.size(); ++i) g += " & " + guards[i];
          return "eh_ranged_load(eh_rs_" + n.args[0]->name + ", (" + g + ") ? " + off + " : 0x80000000u)";
        }
        if (n.count == 1 && !guards.empty()) {
          std::string g = guards[0];
          for (size_t i = 1; i < guards.size(); ++i) g += " & " + guards[i];
          return expr(*n.args[0]) + "[(" + g + ") ? " + expr(*n.args[1]) + " : 0]";
        }
        if (n.count == 1) return expr(*n.args[0]) + "[" + expr(*n.args[1]) + "]";
        return "*reinterpret_cast<const " + ctype(n.dtype) + "*>(&" + expr(*n.args[0]) + "[" + expr(*n.args[1]) + "])";
      }
      case Op::SharedLoad: return expr(*n.args[0]) + "[" + expr(*n.args[1]) + "]";
      case Op::Rand:
        // the C backend renders libc's rand() (src/backend/renderer.rs:313): host state, no
        // device counterpart, and no graph operation produces the node
        throw Error("the Rand node (libc rand() in the C backend) has no device implementation");
      case Op::Call: {
        std::string s = n.name + "(";
        for (size_t i = 0; i < n.args.size(); ++i) s += (i ? ", " : "") + expr(*n.args[i]);
        return s + ")";
      }
      case Op::AtomicAdd:
        return "atomicAdd(&" + expr(*n.args[0]) + "[" + expr(*n.args[1]) + "], " + expr(*n.args[2]) + ")";
      case Op::AtomicMax:
        if (n.dtype.ty == Ty::F32)
          return "eh_atomic_max_f32(&" + expr(*n.args[0]) + "[" + expr(*n.args[1]) + "], " + expr(*n.args[2]) + ")";
        return "atomicMax(&" + expr(*n.args[0]) + "[" + expr(*n.args[1]) + "], " + expr(*n.args[2]) + ")";
      default:
        throw Error(std::string("cannot render '") + op_name(n.op) + "' as an expression");
    }
  }
};

// ---- stages.cpp -------------------------------------------------------------------------------
enum class StageKind { Wide, Reduce, Scalar };

struct Stage {
  StageKind kind = StageKind::Wide;
  std::string kname;
  NodePtr value;             // over canonical variables r0.. and c
  ReduceKind rk = ReduceKind::None;
  NodePtr identity;
  DType acc_dtype;
  std::string out_buf;
  Affine out_aff;
  DType out_dtype;
  bool store = true;
};

struct Group {
  std::vector<int64_t> rows;   // extents of the row loops (all > 1)
  int64_t C = 1;               // extent of the column loop
  std::vector<Stage> stages;
  bool has_reduce() const {
    for (const auto& s : stages)
      if (s.kind == StageKind::Reduce) return true;
    return false;
  }
  int64_t R() const {
    int64_t r = 1;
    for (auto e : rows) r *= e;
    return r;
  }
  const Stage* producer(const std::string& buf) const {
    for (const auto& s : stages)
      if (s.out_buf == buf) return &s;
    return nullptr;
  }
};

struct Canon {
  bool ok = false;
  Stage stage;
  std::vector<int64_t> rows;
  int64_t C = 1;
};

NodePtr rename(const NodePtr& n, const std::map<std::string, NodePtr>& m);
bool canonicalise(const NestKernel& k, StageKind kind, std::vector<int64_t>* rows, int64_t* C, Stage* out);
bool reduce_is_rowwise(const NestKernel& k);
bool aligned_with_group(const Group& g, const Stage& s);
Canon canon_as(const NestKernel& k, StageKind kind);
std::optional<std::vector<int64_t>> dense_strides(const NestKernel& k, int64_t* numel);
std::string gather_fn_name(const std::string& buf);
std::string gather_call(const NestKernel& g, const std::string& src, const Node& index, const std::vector<Loop>& caller,
                        const std::string& idx_type);
std::string gather_fn_text(const NestKernel& g, const std::string& src, const NestKernel* inner, const std::string& idx_type);
// (`computing`: any expression of that one buffer, not only a load under an index-only guard)
std::optional<FoldedOperand> make_fold(const NestKernel& k, const std::map<std::string, size_t>& elems, bool computing = false);
std::optional<Affine> relayout(const NestKernel& g, const NestKernel& sk, const Affine& read);

// ---- rewrites.cpp -----------------------------------------------------------------------------
struct RowSplit {
  NodePtr part, final_;      // the two kernels that replace the original
  BufferInfo scratch;        // [lines * chunks] partial results
};

// Kernel P computes a temp elementwise, and one other elementwise kernel C is all that reads it --
// but through other loops: a permutation made contiguous, windows put back into an image, a
// reshape that regroups axes.  The ordinary fusion needs both kernels to walk the same index
// space.  Here C's loops are split where P's loop boundaries cut them, so that every loop
// variable of P becomes a sum of C's (sub-)loop variables, and P's expression takes the place of
// the load: P, its launch and the temp disappear, and C reads P's operands directly.  Only
// exact digit correspondences are taken (no division or remainder is ever introduced); C must
// compute something itself (a pure gather is left alone: contractions and window reductions
// fold those into their loaders in their own way).
struct Inlined {
  NodePtr kernel;            // replaces C
};

NodePtr make_range(const std::string& var, int64_t extent, NodePtr body);
NodePtr make_combine(ReduceKind k, const NodePtr& acc, const NodePtr& v);
NodePtr make_kernel(const std::string& name, std::vector<Param> params, NodePtr body);
std::optional<RowSplit> split_long_rows(const NestKernel& nk);
void rewrite_for_readers(const Node& program, const GenOptions& opt, std::vector<const Node*>* kernels, std::vector<NodePtr>* rewritten,
                         ProgramPlan* plan);

// What plan_program has found out so far; the passes below read and extend it.
struct Planning {
  explicit Planning(const GenOptions& o) : opt(o) {}
  const GenOptions& opt;
  ProgramPlan plan;
  std::vector<const Node*> kernels;          // in execution order (rewritten ones included)
  std::vector<NodePtr> rewritten;            // owns the kernels that replace given ones
  std::map<std::string, size_t> elems;       // elements per buffer
  bool have_table = false;                   // the program came with a buffer table
  std::map<std::string, std::vector<size_t>> readers;      // kernels (indices) that read a buffer
  std::vector<std::optional<NestKernel>> nests;            // kernels in canonical form, where they have one
  std::set<size_t> absorbed;                 // kernels that became part of an earlier one
  std::map<size_t, std::string> absorbed_name;
  FoldMap folded;                            // gathers evaluated inside the contractions that read them
  std::set<size_t> folded_kernels;
  std::map<size_t, std::vector<size_t>> windows;           // reduce kernel -> its gathers, nearest first
  std::map<size_t, ScatteredWindow> scattered;             // contraction -> the launch that covers it and its shifted sums
  std::set<std::string> partly_written;      // kernels whose output is written only where it is read
  std::string role_of(const std::string& name) const {
    for (const auto& b : plan.buffers)
      if (b.name == name) return b.role;
    throw Error("kernel parameter '" + name + "' is missing from the program's buffer table");
  }
};
// The passes, in the order plan_program runs them (one function each; tests/test_host_cpu.py holds
// a plan test per pass).
void move_elementwise_behind_producers(Planning& st);
void merge_batch_sums_into_contractions(Planning& st);
void merge_sums_over_neighbouring_axes(Planning& st);
void fold_gathers_into_contractions(Planning& st);
void read_windows_through_their_gathers(Planning& st);
void join_shifted_sums_with_their_contraction(Planning& st);

// ---- emitters.cpp -----------------------------------------------------------------------------
std::string combine_text(ReduceKind k, const DType& t, const std::string& acc, const std::string& v);
LaunchSpec emit_group(const Group& g, const GenOptions& opt, const std::map<std::string, size_t>& buf_elems);
void emit_serial_reduce(const NestKernel& k, const GenOptions& opt, ProgramPlan* plan, const EpilogueSpec* epi = nullptr);
LaunchSpec emit_window_reduce(const NestKernel& r, const std::vector<const NestKernel*>& chain, const GenOptions& opt,
                              const std::map<std::string, size_t>& elems);
bool window_reduce_tail(const NestKernel& r, const std::vector<const NestKernel*>& chain,
                        const std::map<std::string, size_t>& elems, EpilogueSpec* epi);

// ---- launches.cpp -----------------------------------------------------------------------------
void mark_written(ProgramPlan* plan, const std::vector<const Node*>& kernels);
void issue_independent_launches_together(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt);
void assign_lanes(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt);
LaunchSpec merge_launches(const std::vector<LaunchSpec>& parts, const GenOptions& opt);

}  // namespace eh
