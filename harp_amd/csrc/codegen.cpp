#include "codegen.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <mutex>
#include <set>
#include <cstdio>
#include <sstream>

#include "gemm.hpp"
#include "window.hpp"
#include "normalize.hpp"

namespace eh {

// ---------------------------------------------------------------------------------------------
// preamble shared by every generated translation unit
// ---------------------------------------------------------------------------------------------

const std::string& preamble() {
  static const std::string s = R"EHP(
// wave64 helpers for gfx950
template <typename T> using EhV4 = T __attribute__((ext_vector_type(4)));
template <bool NT, typename T> __device__ __forceinline__ EhV4<T> eh_load4(const T* p) {
  if (NT) return __builtin_nontemporal_load(reinterpret_cast<const EhV4<T>*>(p));
  return *reinterpret_cast<const EhV4<T>*>(p);
}
template <bool NT, typename T> __device__ __forceinline__ void eh_store4(T* p, EhV4<T> v) {
  if (NT) __builtin_nontemporal_store(v, reinterpret_cast<EhV4<T>*>(p));
  else *reinterpret_cast<EhV4<T>*>(p) = v;
}

struct EhSum  { template <class T> __device__ __forceinline__ static T f(T a, T b) { return a + b; } };
struct EhProd { template <class T> __device__ __forceinline__ static T f(T a, T b) { return a * b; } };
struct EhMax {
  __device__ __forceinline__ static float f(float a, float b) { return fmaxf(a, b); }
  __device__ __forceinline__ static double f(double a, double b) { return fmax(a, b); }
  template <class T> __device__ __forceinline__ static T f(T a, T b) { return a > b ? a : b; }
};
struct EhMin { template <class T> __device__ __forceinline__ static T f(T a, T b) { return a < b ? a : b; } };

template <int CTRL> __device__ __forceinline__ float eh_dpp(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}

// Combines W adjacent lanes (W a power of two, at most 64); every lane of a group ends with
// the group's result.  fp32: DPP quad permutes and row mirrors inside a row of 16 lanes,
// ds_swizzle across rows, readlane across the two halves of the wave.
template <class Op, int W> __device__ __forceinline__ float eh_lanes_reduce(float v) {
  if (W >= 2) v = Op::f(v, eh_dpp<0xB1>(v));    // quad_perm [1,0,3,2]
  if (W >= 4) v = Op::f(v, eh_dpp<0x4E>(v));    // quad_perm [2,3,0,1]
  if (W >= 8) v = Op::f(v, eh_dpp<0x141>(v));   // row_half_mirror
  if (W >= 16) v = Op::f(v, eh_dpp<0x140>(v));  // row_mirror
  if (W >= 32) v = Op::f(v, __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F)));
  if (W >= 64) {
    float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    v = Op::f(lo, hi);
  }
  return v;
}
template <class Op, int W, class T> __device__ __forceinline__ T eh_lanes_reduce(T v) {
#pragma unroll
  for (int m = 1; m < W; m <<= 1) v = Op::f(v, __shfl_xor(v, m, 64));
  return v;
}

// Reduction over the T threads that share a row.  T <= 64: lanes only.  T > 64: per-wave partials
// staged through LDS (`lds`: this row's T/64 slots, one slot array per reduction, one barrier).
template <class Op, int T, class V> __device__ __forceinline__ V eh_row_reduce(V v, V* lds, int lr) {
  if (T <= 64) return eh_lanes_reduce<Op, T>(v);
  v = eh_lanes_reduce<Op, 64>(v);
  constexpr int NW = T / 64 > 0 ? T / 64 : 1;
  if ((lr & 63) == 0) lds[lr >> 6] = v;
  __syncthreads();
  V r = lds[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) r = Op::f(r, lds[w]);
  return r;
}
)EHP";
  return s;
}

std::string kernel_header() {
  return "// generated for gfx950 by eclat backend-hip\n#ifndef __HIPCC_RTC__\n#include <hip/hip_runtime.h>\n#endif\n" + preamble();
}

// ---------------------------------------------------------------------------------------------
// types and literals
// ---------------------------------------------------------------------------------------------

namespace {

std::string ctype(const DType& d) {
  switch (d.ty) {
    case Ty::Void: return "void";
    case Ty::Bool: case Ty::U8: return "unsigned char";
    case Ty::I8: return "signed char";
    case Ty::I16: return "short";
    case Ty::I32: return "int";
    case Ty::I64: case Ty::Int: return "long long";
    case Ty::U16: return "unsigned short";
    case Ty::U32: return "unsigned int";
    case Ty::U64: return "unsigned long long";
    case Ty::F16: return "_Float16";
    case Ty::BF16: return "__bf16";
    case Ty::F32: return "float";
    case Ty::F64: return "double";
    case Ty::Ptr: return ctype(*d.inner) + "*";
    default: throw Error("no HIP type for dtype " + d.name());
  }
}

std::string literal(const Node& n) {
  char buf[64];
  switch (n.dtype.ty) {
    case Ty::F32: case Ty::F16: case Ty::BF16: {
      std::string cast = n.dtype.ty == Ty::F32 ? "" : "(" + ctype(n.dtype) + ")";
      if (std::isnan(n.fval)) return cast + "__builtin_nanf(\"\")";
      if (std::isinf(n.fval)) return cast + (n.fval > 0 ? "__builtin_inff()" : "(-__builtin_inff())");
      float f = static_cast<float>(n.fval);
      if (f == std::floor(f) && std::fabs(f) < 1e6f) snprintf(buf, sizeof buf, "%.1ff", f);
      else snprintf(buf, sizeof buf, "%af", f);           // hex float: exact
      return cast + buf;
    }
    case Ty::F64:
      if (std::isnan(n.fval)) return "__builtin_nan(\"\")";
      if (std::isinf(n.fval)) return n.fval > 0 ? "__builtin_inf()" : "(-__builtin_inf())";
      snprintf(buf, sizeof buf, "%a", n.fval);
      return buf;
    case Ty::Bool: return n.ival ? "1" : "0";
    case Ty::U8: case Ty::U16: case Ty::U32:
      return std::to_string(static_cast<unsigned long long>(n.ival)) + "u";
    case Ty::U64:
      return std::to_string(static_cast<unsigned long long>(n.ival)) + "ull";
    case Ty::I64: case Ty::Int:
      if (n.ival == INT64_MIN) return "(-9223372036854775807ll - 1)";
      if (n.ival > INT32_MAX || n.ival < INT32_MIN) return std::to_string(n.ival) + "ll";
      return std::to_string(n.ival);
    case Ty::I32:
      if (n.ival == INT32_MIN) return "(-2147483647 - 1)";
      return std::to_string(n.ival);
    default:
      return std::to_string(n.ival);
  }
}

// Result type of an expression, as far as rendering needs it.
Ty infer_ty(const Node& n, const std::map<std::string, Ty>* vars = nullptr) {
  switch (n.op) {
    case Op::Const: return n.dtype.ty;
    case Op::Load: case Op::SharedLoad: case Op::Cast: return n.dtype.ty;
    case Op::Lt: case Op::And: case Op::Not: return Ty::Bool;
    case Op::Recip: case Op::Sqrt: case Op::Log2: case Op::Exp2: case Op::Sin: case Op::Floor: {
      Ty t = infer_ty(*n.args[0], vars);
      return t == Ty::F64 ? Ty::F64 : Ty::F32;
    }
    case Op::Select: return infer_ty(*n.args[1], vars);
    case Op::Fma: return infer_ty(*n.args[0], vars);
    case Op::Var:
      if (vars) {
        auto it = vars->find(n.name);
        if (it != vars->end()) return it->second;
      }
      return Ty::I64;
    case Op::Rand: return Ty::F32;
    case Op::AtomicAdd: case Op::AtomicMax: return n.dtype.ty;
    default:
      if (n.args.empty()) return Ty::Unknown;
      {
        Ty a = infer_ty(*n.args[0], vars);
        if (n.args.size() > 1) {
          Ty b = infer_ty(*n.args[1], vars);
          auto rank = [](Ty t) { return t == Ty::F64 ? 4 : t == Ty::F32 ? 3 : (t == Ty::F16 || t == Ty::BF16) ? 2 : 1; };
          return rank(b) > rank(a) ? b : a;
        }
        return a;
      }
  }
}

const char* infix(Op op) {
  switch (op) {
    case Op::Add: return "+";
    case Op::Mul: return "*";
    case Op::Rem: return "%";
    case Op::Idiv: return "/";
    case Op::Lt: return "<";
    case Op::And: return "&&";
    case Op::BitAnd: return "&";
    case Op::BitOr: return "|";
    case Op::BitXor: return "^";
    case Op::Shl: return "<<";
    case Op::Shr: return ">>";
    default: return nullptr;
  }
}

using LoadHook = std::function<bool(const Node& load, std::string* out)>;

bool holds_load(const Node& n) {
  if (n.op == Op::Load) return true;
  for (const auto& a : n.args)
    if (a && holds_load(*a)) return true;
  return false;
}

// set by plan_program for the plan it is making (GenOptions::guard_branches)
thread_local bool g_guard_branches = false;
thread_local bool g_ranged_loads = true;

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
  // With a load hook installed (a schedule that renders plain loads itself) only guarded loads
  // take this form, and only under guards that test indices: an offset that waits for another
  // load's value (a mask read from memory) would put the two loads one after the other.
  const std::map<std::string, size_t>* ranged = nullptr;
  mutable int value_guards = 0;         // selects around the current node whose condition holds a load
  bool is_ranged(const Node& n, bool guarded) const {
    return ranged && n.op == Op::Load && n.count == 1 && n.dtype.ty == Ty::F32 && n.args[0]->op == Op::Var &&
           ranged->count(n.args[0]->name) && (!load_hook || (guarded && value_guards == 0));
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
        return "(" + ctype(DType{t}) + ")fma((double)(" + expr(*n.args[0]) + "), (double)(" + expr(*n.args[1]) + "), (double)(" +
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

std::string hdr(const GenOptions&) { return kernel_header(); }

// ---------------------------------------------------------------------------------------------
// statement-by-statement rendering (kernels no schedule recognises)
// ---------------------------------------------------------------------------------------------

struct StmtRenderer {
  ExprRenderer er;
  int level = 1;
  std::string ind() const { return std::string(static_cast<size_t>(level) * 2, ' '); }

  std::string stmt(const Node& n) {
    switch (n.op) {
      case Op::Store:
        return ind() + er.expr(*n.args[0]) + "[" + er.expr(*n.args[1]) + "] = " + er.expr(*n.args[2]) + ";\n";
      case Op::Assign:
        return ind() + n.name + " = " + er.expr(*n.args[0]) + ";\n";
      case Op::Block: {
        std::string s;
        for (const auto& d : n.decls) s += ind() + ctype(d.second) + " " + d.first + ";\n";
        for (const auto& a : n.args) s += stmt(*a);
        return s;
      }
      case Op::Range: {
        std::string s = ind() + "for (long long " + n.name + " = " + er.expr(*n.args[0]) + "; " + n.name + " < " +
                        er.expr(*n.args[2]) + "; " + n.name + " += " + er.expr(*n.args[1]) + ") {\n";
        ++level;
        s += stmt(*n.args[3]);
        --level;
        return s + ind() + "}\n";
      }
      case Op::If: {
        std::string s = ind() + "if (" + er.expr(*n.args[0]) + ") {\n";
        ++level;
        s += stmt(*n.args[1]);
        --level;
        s += ind() + "}";
        if (n.args.size() > 2) {
          s += " else {\n";
          ++level;
          s += stmt(*n.args[2]);
          --level;
          s += ind() + "}";
        }
        return s + "\n";
      }
      case Op::Barrier: return ind() + "__syncthreads();\n";
      case Op::Return: return ind() + "return " + er.expr(*n.args[0]) + ";\n";
      case Op::SharedAlloc:
        return ind() + "__shared__ " + ctype(n.dtype) + " " + n.name + "[" + er.expr(*n.args[0]) + "];\n";
      case Op::SharedStore:
        return ind() + er.expr(*n.args[0]) + "[" + er.expr(*n.args[1]) + "] = " + er.expr(*n.args[2]) + ";\n";
      case Op::WmmaMatmul:
        throw Error("WmmaMatmul (f16 16x16x16 tiles) is not part of the fp32 path of this backend");
      default:
        return ind() + er.expr(n) + ";\n";
    }
  }
};

// Value of a dispatch-size expression, evaluated as the reference's pipeline does
// (`evaluate_ast_expr`, src/backend/pipeline.rs:505-553): constants, +, *, integer division and
// remainder (a zero divisor gives 1 and 0), max.  Shape variables are not supported on this
// path, so a variable or any other node is an error rather than the reference's silent 1.
int64_t dispatch_value(const Node& n) {
  switch (n.op) {
    case Op::Const: return n.dtype.is_float() ? static_cast<int64_t>(n.fval) : n.ival;
    case Op::Add: return dispatch_value(*n.args[0]) + dispatch_value(*n.args[1]);
    case Op::Mul: return dispatch_value(*n.args[0]) * dispatch_value(*n.args[1]);
    case Op::Idiv: {
      const int64_t d = dispatch_value(*n.args[1]);
      return d != 0 ? dispatch_value(*n.args[0]) / d : 1;
    }
    case Op::Rem: {
      const int64_t d = dispatch_value(*n.args[1]);
      return d != 0 ? dispatch_value(*n.args[0]) % d : 0;
    }
    case Op::Max: return std::max(dispatch_value(*n.args[0]), dispatch_value(*n.args[1]));
    default:
      throw Error(std::string("dispatch size uses '") + op_name(n.op) + "', which cannot be evaluated at compile time");
  }
}

const char* kAtomicMaxF32 = R"EHA(
__device__ inline float eh_atomic_max_f32(float* addr, float v) {
  unsigned int* a = reinterpret_cast<unsigned int*>(addr);
  unsigned int old = *a, assumed;
  do {
    assumed = old;
    if (__uint_as_float(assumed) >= v) break;
    old = atomicCAS(a, assumed, __float_as_uint(v));
  } while (assumed != old);
  return __uint_as_float(old);
}
)EHA";

}  // namespace

std::string render_expr_text(const Node& e) {
  ExprRenderer er;
  return er.expr(e);
}

namespace {
// A kernel (or one of its loop nests) that is about to run in a single work-item: fine for the
// few statements of a short scan, hopeless for millions of iterations.  Refused rather than
// launched, unless the caller asked for it.
void refuse_long_serial(const std::string& kernel, const Node& body, const GenOptions& opt) {
  const double limit = 131072;
  const double n = serial_iterations(body);
  if (n <= limit || opt.allow_serial) return;
  throw Error("kernel '" + kernel + "' has a form no schedule of this backend recognises and would run its " +
              std::to_string(static_cast<long long>(n)) +
              " loop iterations in one work-item: not supported (compile with allow_serial=1 to run it anyway)");
}
}  // namespace

// local[i] = the largest divisor of global[i] that is at most preferred[i]
// (`compute_compatible_local_size`, src/backend/pipeline.rs:475-489); then, while the workgroup
// exceeds `max_work_group`, its largest dimension steps down to the next smaller divisor of that
// dimension's global size (pipeline.rs:176-192).
void fit_local_size(const uint64_t global[3], const uint64_t preferred[3], uint64_t max_work_group, uint64_t local[3]) {
  for (int i = 0; i < 3; ++i) {
    uint64_t l = 1;
    if (global[i] != 0) {
      l = std::min(preferred[i], global[i]);
      while (l > 1 && global[i] % l != 0) --l;
      if (l < 1) l = 1;
    }
    local[i] = l;
  }
  while (local[0] * local[1] * local[2] > max_work_group) {
    const int m = (local[0] >= local[1] && local[0] >= local[2]) ? 0 : (local[1] >= local[2] ? 1 : 2);
    uint64_t v = local[m] - 1;
    while (v > 1 && global[m] % v != 0) --v;
    local[m] = std::max<uint64_t>(v, 1);
  }
}

LaunchSpec render_kernel_as_written(const Node& k, const GenOptions& opt) {
  if (k.op != Op::Kernel) throw Error("expected a kernel node");
  LaunchSpec ls;
  ls.entry = k.name;
  ls.kernels = {k.name};
  ls.schedule = "as-written";
  std::ostringstream os;
  os << hdr(opt) << kAtomicMaxF32;
  os << "extern \"C\" __global__ void " << k.name << "(";
  bool first = true;
  std::string decls;
  static const char* dim[] = {"x", "y", "z"};
  for (const auto& p : k.params) {
    if (p.kind == VarKind::Normal) {
      if (!p.dtype.is_ptr())
        throw Error("kernel '" + k.name + "' takes the shape variable '" + p.name +
                    "'; only static shapes are supported on this path");
      os << (first ? "" : ", ") << (p.mut_ ? "" : "const ") << ctype(p.dtype.elem()) << "* __restrict__ " << p.name;
      first = false;
      ls.arg_bufs.push_back(p.name);
    } else {
      const char* src = p.kind == VarKind::GroupId ? "blockIdx" : p.kind == VarKind::LocalId ? "threadIdx"
                        : p.kind == VarKind::GroupSize ? "blockDim" : "gridDim";
      if (p.axis < 0 || p.axis > 2) throw Error("bad axis on parameter " + p.name);
      decls += "  const long long " + p.name + " = " + src + "." + dim[p.axis] +
               (p.kind == VarKind::GridSize ? std::string(" * blockDim.") + dim[p.axis] : std::string()) + ";\n";
    }
  }
  os << ") {\n" << decls;
  StmtRenderer sr;
  os << sr.stmt(*k.args[0]) << "}\n";
  ls.source = os.str();
  {
    // global size = grid x thread group (the AST's grid counts workgroups), local size = the
    // thread group fitted to the device as Pipeline::compile_ast does (src/backend/pipeline.rs:
    // 160-192), launched as global / local workgroups
    uint64_t global[3], preferred[3], local[3];
    for (int i = 0; i < 3; ++i) {
      int64_t g = k.grid.size() == 3 ? dispatch_value(*k.grid[i]) : 1;
      int64_t t = k.tg.size() == 3 ? dispatch_value(*k.tg[i]) : 1;
      if (g < 1 || t < 1 || g > (int64_t{1} << 31) || t > (int64_t{1} << 31) || g * t > (int64_t{1} << 40))
        throw Error("kernel '" + k.name + "' has an unusable dispatch size");
      global[i] = static_cast<uint64_t>(g * t);
      preferred[i] = static_cast<uint64_t>(t);
    }
    fit_local_size(global, preferred, 1024, local);
    for (int i = 0; i < 3; ++i) {
      if (global[i] / local[i] > 0x7fffffffull) throw Error("kernel '" + k.name + "' has an unusable dispatch size");
      ls.block[i] = static_cast<unsigned>(local[i]);
      ls.grid[i] = static_cast<unsigned>(global[i] / local[i]);
    }
  }
  if (1ull * ls.grid[0] * ls.grid[1] * ls.grid[2] * ls.block[0] * ls.block[1] * ls.block[2] == 1)
    refuse_long_serial(k.name, *k.args[0], opt);
  return ls;
}

// ---------------------------------------------------------------------------------------------
// outer-parallel rendering of kernels no schedule recognises (scan, scatter-add, ...)
// ---------------------------------------------------------------------------------------------

namespace {

struct WriteRef {
  std::string buf;
  const Node* index;
  bool atomic;      // AtomicAdd / AtomicMax: safe from any number of work-items at once
};

// A prefix scan along one line, as `LoopGenerator::generate_scan` writes it
// (src/lowerer/lower.rs:691-735): acc = identity; for the inner loops { acc = combine(acc,
// value); out[index] = acc }.
struct ScanLine {
  std::string acc;
  DType acc_dtype;
  NodePtr identity, value, out_ptr, out_index;
  ReduceKind kind = ReduceKind::None;
  std::vector<Loop> loops;     // the scanned loops, outermost first
  int64_t length = 1;
};

std::optional<ScanLine> match_scan_line(const Node& n) {
  if (n.op != Op::Block || n.decls.size() != 1 || n.args.size() != 2) return std::nullopt;
  ScanLine sl;
  sl.acc = n.decls[0].first;
  sl.acc_dtype = n.decls[0].second;
  const Node& init = *n.args[0];
  if (init.op != Op::Assign || init.name != sl.acc || init.args[0]->op != Op::Const) return std::nullopt;
  sl.identity = init.args[0];
  const Node* cur = n.args[1].get();
  while (cur->op == Op::Range && cur->args[0]->op == Op::Const && cur->args[0]->ival == 0 &&
         cur->args[1]->op == Op::Const && cur->args[1]->ival == 1 && cur->args[2]->op == Op::Const &&
         cur->args[2]->ival >= 1) {
    sl.loops.push_back({cur->name, cur->args[2]->ival});
    sl.length *= cur->args[2]->ival;
    const Node* b = cur->args[3].get();
    while (b->op == Op::Block && b->decls.empty() && b->args.size() == 1) b = b->args[0].get();
    cur = b;
  }
  if (sl.loops.empty() || cur->op != Op::Block || !cur->decls.empty() || cur->args.size() != 2) return std::nullopt;
  const Node& step = *cur->args[0];
  const Node& store = *cur->args[1];
  if (step.op != Op::Assign || step.name != sl.acc) return std::nullopt;
  if (!match_combine(*step.args[0], sl.acc, &sl.kind, &sl.value)) return std::nullopt;
  if (sl.kind != ReduceKind::Sum && sl.kind != ReduceKind::Prod && sl.kind != ReduceKind::Max) return std::nullopt;
  if (store.op != Op::Store || store.args[2]->op != Op::Var || store.args[2]->name != sl.acc) return std::nullopt;
  sl.out_ptr = store.args[0];
  sl.out_index = store.args[1];
  return sl;
}

std::string combine_text(ReduceKind k, const DType& t, const std::string& acc, const std::string& v);

void collect_writes(const Node& n, std::vector<WriteRef>& writes, std::set<std::string>& read_bufs,
                    std::map<std::string, int64_t>& inner_extents, bool* ok) {
  if (n.op == Op::Store || n.op == Op::AtomicAdd || n.op == Op::AtomicMax) {
    if (n.args[0]->op != Op::Var) *ok = false;
    else writes.push_back({n.args[0]->name, n.args[1].get(), n.op != Op::Store});
  }
  if (n.op == Op::Load) {
    if (n.args[0]->op == Op::Var) read_bufs.insert(n.args[0]->name);
    else *ok = false;
  }
  if (n.op == Op::Range) {
    if (n.args[0]->op != Op::Const || n.args[1]->op != Op::Const || n.args[2]->op != Op::Const) *ok = false;
    else inner_extents[n.name] = n.args[2]->ival - n.args[0]->ival;
  }
  if (n.op == Op::Barrier || n.op == Op::SharedAlloc || n.op == Op::SharedStore || n.op == Op::WmmaMatmul ||
      n.op == Op::Return)
    *ok = false;
  for (const auto& a : n.args) collect_writes(*a, writes, read_bufs, inner_extents, ok);
}

// True when distinct value tuples of `vars` (each 0 <= v < extent) give distinct indices:
// sorted by |coefficient|, every coefficient exceeds the reach of all smaller ones.
bool injective(const Affine& a, const std::vector<Loop>& vars) {
  std::vector<std::pair<int64_t, int64_t>> ce;   // (|coef|, extent)
  for (const auto& v : vars) {
    if (v.extent <= 1) continue;
    int64_t c = std::llabs(a.of(v.var));
    if (c == 0) return false;
    ce.push_back({c, v.extent});
  }
  std::sort(ce.begin(), ce.end());
  int64_t reach = 0;
  for (const auto& p : ce) {
    if (p.first <= reach) return false;
    reach += p.first * (p.second - 1);
  }
  return true;
}

}  // namespace

namespace {

bool stores_anything(const Node& n) {
  if (n.op == Op::Store || n.op == Op::AtomicAdd || n.op == Op::AtomicMax) return true;
  for (const auto& a : n.args)
    if (stores_anything(*a)) return true;
  return false;
}

// A loop of at least 64 iterations that only accumulates (assigns, stores nothing): the inner loop of
// a reduction, as opposed to a scan's, which stores every step.
bool has_accumulating_loop(const Node& n) {
  if (n.op == Op::Range) {
    int64_t s = 0, e = 0;
    const bool counted = n.args[0]->op == Op::Const && n.args[2]->op == Op::Const;
    if (counted) {
      s = n.args[0]->ival;
      e = n.args[2]->ival;
    }
    if ((!counted || e - s >= 64) && !stores_anything(*n.args[3])) {
      bool assigns_something = false;
      std::vector<const Node*> todo = {n.args[3].get()};
      while (!todo.empty() && !assigns_something) {
        const Node* x = todo.back();
        todo.pop_back();
        assigns_something = x->op == Op::Assign;
        for (const auto& a : x->args) todo.push_back(a.get());
      }
      if (assigns_something) return true;
    }
  }
  for (const auto& a : n.args)
    if (has_accumulating_loop(*a)) return true;
  return false;
}

void warn_once_degraded(const std::string& kernel) {
  static std::mutex mu;
  static std::set<std::string> seen;
  std::lock_guard<std::mutex> lock(mu);
  if (seen.size() > 256 || !seen.insert(kernel).second) return;
  std::fprintf(stderr, "eclat-hip: kernel '%s' has a loop structure no schedule recognises as written and runs one "
               "work-item per outer iteration (plan marked 'degraded')\n", kernel.c_str());
}

}  // namespace

// Kernels outside the canonical forms arrive as sequential loop nests for one work-item
// (src/lowerer/lower.rs:580-735: prefix scans, zero-fill + scatter-add).  Each top-level nest
// becomes its own launch, in order; the outer loops of a nest are spread over work-items when
// their iterations cannot touch the same output element (every write index is affine and
// injective in the loop variables, nothing written is read), each work-item then runs what is
// left of the nest exactly as written, so sums keep the reference's order.  Writes the AST
// marks atomic (the scatter-add of overlapping windows) may collide: the device's atomics
// make that safe, and only the order of the additions is left open.  A nest that does not
// qualify runs as written in one work-item.  Empty result: the kernel has a form this
// does not cover (shape variables, hand-placed group/local ids, shared memory).
std::vector<LaunchSpec> render_kernel_outer_parallel(const Node& k, const GenOptions& opt,
                                                     std::vector<BufferInfo>* extra_buffers) {
  std::vector<LaunchSpec> out;
  if (k.op != Op::Kernel) return out;
  for (const auto& p : k.params)
    if (p.kind != VarKind::Normal || !p.dtype.is_ptr()) return {};
  for (int i = 0; i < 3; ++i) {
    if (k.grid.size() == 3 && dispatch_value(*k.grid[i]) != 1) return {};
    if (k.tg.size() == 3 && dispatch_value(*k.tg[i]) != 1) return {};
  }
  const Node& body = *k.args[0];
  std::vector<const Node*> tops;
  // a scan lowered with one accumulator for the whole tensor (axis 0) is a single line
  bool whole_scan = false;
  if (body.op == Op::Block && !body.decls.empty()) {
    auto sl = match_scan_line(body);
    whole_scan = sl && sl->length >= 512;        // a short one stays as written
  }
  if (whole_scan) {
    tops.push_back(&body);
  } else if (body.op == Op::Block) {
    if (!body.decls.empty()) return {};
    for (const auto& a : body.args) tops.push_back(a.get());
  } else {
    tops.push_back(&body);
  }
  if (tops.empty()) return {};
  // buffers written anywhere in the kernel must not be read by a nest that is spread out
  std::set<std::string> written_anywhere;
  {
    std::vector<WriteRef> w;
    std::set<std::string> r;
    std::map<std::string, int64_t> e;
    bool ok = true;
    collect_writes(body, w, r, e, &ok);
    if (!ok) return {};
    for (const auto& x : w) written_anywhere.insert(x.buf);
  }
  std::string sig;
  std::vector<std::string> arg_bufs;
  for (const auto& p : k.params) {
    sig += (sig.empty() ? "" : ", ") + std::string(p.mut_ ? "" : "const ") + ctype(p.dtype.elem()) + "* __restrict__ " + p.name;
    arg_bufs.push_back(p.name);
  }
  bool any_parallel = false;
  for (size_t t = 0; t < tops.size(); ++t) {
    if (tops[t]->op != Op::Range && !whole_scan) return {};
    // the perfect nest at the top of this statement
    std::vector<Loop> loops;
    const Node* cur = tops[t];
    while (cur->op == Op::Range && cur->args[0]->op == Op::Const && cur->args[0]->ival == 0 &&
           cur->args[1]->op == Op::Const && cur->args[1]->ival == 1 && cur->args[2]->op == Op::Const &&
           cur->args[2]->ival >= 1) {
      loops.push_back({cur->name, cur->args[2]->ival});
      const Node* b = cur->args[3].get();
      if (b->op == Op::Block && b->decls.empty() && b->args.size() == 1) b = b->args[0].get();
      cur = b;
      if (cur->op != Op::Range) break;
    }
    const Node* inner = cur;
    if (loops.empty() && !whole_scan) return {};
    if (inner->op == Op::Range) {
      // the walk stopped at a loop it cannot spread (non-constant bounds): keep it inside
    }
    std::vector<WriteRef> writes;
    std::set<std::string> reads;
    std::map<std::string, int64_t> inner_extents;
    bool ok = true;
    collect_writes(*inner, writes, reads, inner_extents, &ok);
    if (!ok) return {};
    bool spread = !writes.empty();
    bool colliding = false;
    for (const auto& r : reads) spread = spread && !written_anywhere.count(r);
    for (const auto& w : writes) {
      auto a = affine_of(*w.index);
      if (!a) {
        if (w.atomic) { colliding = true; continue; }
        spread = false;
        break;
      }
      std::vector<Loop> vars = loops;
      for (const auto& kv : a->coef)
        if (kv.second != 0) {
          bool is_outer = false;
          for (const auto& l : loops) is_outer = is_outer || l.var == kv.first;
          if (is_outer) continue;
          auto ie = inner_extents.find(kv.first);
          if (ie == inner_extents.end()) { spread = false; break; }
          vars.push_back({kv.first, ie->second});
        }
      if (!spread) break;
      if (!injective(*a, vars)) {
        if (w.atomic) colliding = true;
        else { spread = false; break; }
      }
    }
    LaunchSpec ls;
    ls.entry = k.name + "_n" + std::to_string(t);
    ls.kernels = {k.name};
    ls.arg_bufs = arg_bufs;
    std::ostringstream os;
    os << hdr(opt) << kAtomicMaxF32;
    StmtRenderer sr;
    // A long scanned line gets a workgroup instead of a work-item: tiles of 256 x 4 elements,
    // each thread scans its four, the wave and then the workgroup scan the thread totals, and
    // the tile's total is carried into the next tile.  The combine order differs from the
    // sequential one (exact for max, the reduction tolerance for sums and products).
    std::optional<ScanLine> scan = spread ? match_scan_line(*inner) : std::nullopt;
    if (scan && scan->length >= 512) {
      int64_t lines = 1;
      for (const auto& l : loops) lines *= l.extent;
      if (lines >= (int64_t{1} << 31)) return {};
      const std::string T = ctype(scan->acc_dtype);
      const std::string ident = literal(*scan->identity);
      ExprRenderer er;
      auto comb = [&](const std::string& a, const std::string& b) { return combine_text(scan->kind, scan->acc_dtype, a, b); };
      // 128-bit accesses when the line is one loop walked with unit stride by every load and by
      // the store, everything 16-byte aligned, four-byte elements
      bool vec = scan->loops.size() == 1 && scan->length % 4 == 0 && scan->acc_dtype.itemsize() == 4;
      const std::string sv = scan->loops[0].var;
      std::vector<LoadRef> sloads;
      collect_loads(*scan->value, sloads);
      auto unit_aligned = [&](const Node& index) {
        auto a = affine_of(index);
        if (!a || a->of(sv) != 1 || a->c % 4) return false;
        for (const auto& kv : a->coef)
          if (kv.first != sv && kv.second % 4) return false;
        return true;
      };
      for (const auto& lr : sloads)
        vec = vec && !lr.guarded && lr.load->count == 1 && lr.load->dtype.itemsize() == 4 &&
              lr.load->args[0]->op == Op::Var && unit_aligned(*lr.load->args[1]);
      vec = vec && scan->out_ptr->op == Op::Var && unit_aligned(*scan->out_index);
      // A few long lines (a scan over axis 0 is lowered as one line over the whole tensor)
      // would occupy a few workgroups, each bound by the tile-to-tile dependency: cut every line into chunks of whole
      // tiles, total each chunk in a first launch, and let the workgroup that scans a chunk
      // start from the combined totals of the chunks ahead of it.
      int64_t chunks = 1, chunk_len = scan->length;
      if (extra_buffers && lines <= 256 && scan->length >= (int64_t{1} << 14)) {
        const int64_t want = 2048 / lines;
        chunk_len = std::max<int64_t>(4096, ((scan->length + want - 1) / want + 1023) / 1024 * 1024);
        chunks = (scan->length + chunk_len - 1) / chunk_len;
      }
      const std::string scratch = "eh_scanpart_" + k.name + "_n" + std::to_string(t);
      // the four values of this thread in the tile at eh_t0, each combined with the ones before
      // it in the thread: eh_v[3] is the thread's total
      auto emit_tile_values = [&](std::ostringstream& os) {
        os << "    " << T << " eh_v[4];\n";
        if (vec) {
          os << "    const long long eh_tb = eh_t0 + threadIdx.x * 4;\n    const bool eh_in = eh_tb < " << scan->length << "ll;\n";
          os << "    {\n      const long long " << sv << " = eh_in ? eh_tb : 0;\n";
          std::vector<std::string> seen;
          for (const auto& lr : sloads) {
            const std::string key = to_text(*lr.load);
            if (std::find(seen.begin(), seen.end(), key) != seen.end()) continue;
            os << "      const EhV4<" << ctype(lr.load->dtype) << "> eh_ld" << seen.size() << " = eh_load4<false>("
               << lr.load->args[0]->name << " + " << er.expr(*lr.load->args[1]) << ");\n";
            seen.push_back(key);
          }
          ExprRenderer ev;
          ev.load_hook = [&](const Node& ld, std::string* out) {
            const std::string key = to_text(ld);
            for (size_t q = 0; q < seen.size(); ++q)
              if (seen[q] == key) { *out = "eh_ld" + std::to_string(q) + "[eh_e]"; return true; }
            return false;
          };
          os << "#pragma unroll\n      for (int eh_e = 0; eh_e < 4; ++eh_e) {\n";
          os << "        eh_v[eh_e] = eh_in ? (" << T << ")(" << ev.expr(*scan->value) << ") : " << ident << ";\n";
          os << "        if (eh_e) eh_v[eh_e] = " << comb("eh_v[eh_e - 1]", "eh_v[eh_e]") << ";\n      }\n    }\n";
        } else {
          os << "#pragma unroll\n    for (int eh_e = 0; eh_e < 4; ++eh_e) {\n";
          os << "      const long long eh_t = eh_t0 + threadIdx.x * 4 + eh_e;\n";
          os << "      eh_v[eh_e] = " << ident << ";\n";
          os << "      if (eh_t < " << scan->length << "ll) {\n        long long eh_q = eh_t;\n";
          for (size_t i = scan->loops.size(); i-- > 0;) {
            os << "        const long long " << scan->loops[i].var << " = eh_q % " << scan->loops[i].extent << ";\n";
            if (i) os << "        eh_q /= " << scan->loops[i].extent << ";\n";
          }
          os << "        eh_v[eh_e] = (" << T << ")(" << er.expr(*scan->value) << ");\n      }\n";
          os << "      if (eh_e) eh_v[eh_e] = " << comb("eh_v[eh_e - 1]", "eh_v[eh_e]") << ";\n    }\n";
        }
      };
      // entry, line variables, lane ids; with chunks also eh_chunk and the tile range of the chunk
      auto emit_head = [&](std::ostringstream& os, const std::string& entry, const std::string& params) {
        os << "extern \"C\" __global__ void __launch_bounds__(256) " << entry << "(" << params << ") {\n";
        if (chunks > 1) {
          os << "  const long long eh_chunk = blockIdx.x % " << chunks << ", eh_line = blockIdx.x / " << chunks << ";\n";
          os << "  long long eh_r = eh_line;\n";
          os << "  const long long eh_first = eh_chunk * " << chunk_len << "ll;\n";
          os << "  const long long eh_last = eh_first + " << chunk_len << "ll < " << scan->length << "ll ? eh_first + "
             << chunk_len << "ll : " << scan->length << "ll;\n";
        } else {
          os << "  long long eh_r = blockIdx.x;\n";
          os << "  const long long eh_first = 0, eh_last = " << scan->length << "ll;\n";
        }
        for (size_t i = loops.size(); i-- > 0;) {
          os << "  const long long " << loops[i].var << " = eh_r % " << loops[i].extent << ";\n";
          if (i) os << "  eh_r /= " << loops[i].extent << ";\n";
        }
        os << "  __shared__ " << T << " eh_wave_total[4];\n";
        os << "  const int eh_lane = threadIdx.x & 63, eh_wave = threadIdx.x >> 6;\n";
      };
      // eh_p of every thread combined over the workgroup into `dst` (same value in every thread)
      auto emit_block_combine = [&](std::ostringstream& os, const std::string& dst) {
        os << "#pragma unroll\n  for (int eh_d = 32; eh_d > 0; eh_d >>= 1) eh_p = " << comb("eh_p", "__shfl_xor(eh_p, eh_d, 64)") << ";\n";
        os << "  if (eh_lane == 0) eh_wave_total[eh_wave] = eh_p;\n  __syncthreads();\n";
        os << "  for (int eh_w = 0; eh_w < 4; ++eh_w) " << dst << " = " << comb(dst, "eh_wave_total[eh_w]") << ";\n";
        os << "  __syncthreads();\n";
      };
      if (chunks > 1) {
        // first launch: the total of every chunk
        LaunchSpec lt;
        lt.entry = ls.entry + "_tot";
        lt.kernels = {k.name};
        std::string tsig;
        for (const auto& p : k.params) {
          if (p.mut_) continue;
          tsig += (tsig.empty() ? "" : ", ") + std::string("const ") + ctype(p.dtype.elem()) + "* __restrict__ " + p.name;
          lt.arg_bufs.push_back(p.name);
        }
        tsig += (tsig.empty() ? "" : ", ") + T + "* __restrict__ " + scratch;
        lt.arg_bufs.push_back(scratch);
        std::ostringstream ot;
        ot << hdr(opt);
        emit_head(ot, lt.entry, tsig);
        ot << "  " << T << " eh_p = " << ident << ";\n";
        ot << "  for (long long eh_t0 = eh_first; eh_t0 < eh_last; eh_t0 += 1024) {\n";
        emit_tile_values(ot);
        ot << "    eh_p = " << comb("eh_p", "eh_v[3]") << ";\n  }\n";
        ot << "  " << T << " eh_total = " << ident << ";\n";
        emit_block_combine(ot, "eh_total");
        ot << "  if (threadIdx.x == 0) " << scratch << "[blockIdx.x] = eh_total;\n}\n";
        lt.source = ot.str();
        lt.grid[0] = static_cast<unsigned>(lines * chunks);
        lt.block[0] = 256;
        lt.schedule = "scan-row-totals(lines=" + std::to_string(lines) + ",chunks=" + std::to_string(chunks) + ")";
        out.push_back(std::move(lt));
        BufferInfo sb;
        sb.name = scratch;
        sb.dtype = scan->acc_dtype;
        sb.shape = {lines * chunks};
        sb.role = "temp";
        extra_buffers->push_back(sb);
        ls.arg_bufs.push_back(scratch);
      }
      emit_head(os, ls.entry, chunks > 1 ? sig + ", const " + T + "* __restrict__ " + scratch : sig);
      os << "  " << T << " eh_carry = " << ident << ";\n";
      if (chunks > 1) {
        // everything ahead of this chunk in its line
        os << "  {\n  " << T << " eh_p = " << ident << ";\n";
        os << "  for (long long eh_q = threadIdx.x; eh_q < eh_chunk; eh_q += 256) eh_p = "
           << comb("eh_p", scratch + "[eh_line * " + std::to_string(chunks) + " + eh_q]") << ";\n";
        emit_block_combine(os, "eh_carry");
        os << "  }\n";
      }
      os << "  for (long long eh_t0 = eh_first; eh_t0 < eh_last; eh_t0 += 1024) {\n";
      emit_tile_values(os);
      // inclusive scan of the thread totals across the wave, then across the four waves
      os << "    " << T << " eh_inc = eh_v[3];\n";
      os << "#pragma unroll\n    for (int eh_d = 1; eh_d < 64; eh_d <<= 1) {\n";
      os << "      const " << T << " eh_o = __shfl_up(eh_inc, eh_d, 64);\n";
      os << "      if (eh_lane >= eh_d) eh_inc = " << comb("eh_o", "eh_inc") << ";\n    }\n";
      os << "    if (eh_lane == 63) eh_wave_total[eh_wave] = eh_inc;\n    __syncthreads();\n";
      os << "    " << T << " eh_before = eh_carry;            // everything ahead of this thread's four\n";
      os << "    for (int eh_w = 0; eh_w < eh_wave; ++eh_w) eh_before = " << comb("eh_before", "eh_wave_total[eh_w]") << ";\n";
      os << "    const " << T << " eh_prev = __shfl_up(eh_inc, 1, 64);\n";
      os << "    if (eh_lane) eh_before = " << comb("eh_before", "eh_prev") << ";\n";
      os << "    " << T << " eh_all = eh_carry;\n";
      os << "    for (int eh_w = 0; eh_w < 4; ++eh_w) eh_all = " << comb("eh_all", "eh_wave_total[eh_w]") << ";\n";
      os << "    eh_carry = eh_all;\n";
      if (vec) {
        os << "    if (eh_in) {\n      const long long " << sv << " = eh_tb;\n      EhV4<" << T << "> eh_out;\n";
        os << "#pragma unroll\n      for (int eh_e = 0; eh_e < 4; ++eh_e) eh_out[eh_e] = " << comb("eh_before", "eh_v[eh_e]") << ";\n";
        os << "      eh_store4<false>(" << scan->out_ptr->name << " + " << er.expr(*scan->out_index) << ", eh_out);\n    }\n";
      } else {
        os << "#pragma unroll\n    for (int eh_e = 0; eh_e < 4; ++eh_e) {\n";
        os << "      const long long eh_t = eh_t0 + threadIdx.x * 4 + eh_e;\n";
        os << "      if (eh_t < " << scan->length << "ll) {\n        long long eh_q = eh_t;\n";
        for (size_t i = scan->loops.size(); i-- > 0;) {
          os << "        const long long " << scan->loops[i].var << " = eh_q % " << scan->loops[i].extent << ";\n";
          if (i) os << "        eh_q /= " << scan->loops[i].extent << ";\n";
        }
        os << "        " << er.expr(*scan->out_ptr) << "[" << er.expr(*scan->out_index) << "] = " << comb("eh_before", "eh_v[eh_e]") << ";\n      }\n    }\n";
      }
      os << "    __syncthreads();\n  }\n}\n";
      ls.grid[0] = static_cast<unsigned>(lines * chunks);
      ls.block[0] = 256;
      ls.schedule = "scan-row(lines=" + std::to_string(lines) + ",length=" + std::to_string(scan->length) +
                    (chunks > 1 ? ",chunks=" + std::to_string(chunks) : "") + ")";
      any_parallel = true;
    } else if (spread) {
      int64_t total = 1;
      for (const auto& l : loops) total *= l.extent;
      if (total >= (int64_t{1} << 40)) return {};
      os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "(" << sig << ") {\n";
      os << "  long long eh_r = (long long)blockIdx.x * 256 + threadIdx.x;\n  if (eh_r >= " << total << "ll) return;\n";
      for (size_t i = loops.size(); i-- > 0;) {
        os << "  const long long " << loops[i].var << " = eh_r % " << loops[i].extent << ";\n";
        if (i) os << "  eh_r /= " << loops[i].extent << ";\n";
      }
      os << sr.stmt(*inner) << "}\n";
      ls.grid[0] = static_cast<unsigned>((total + 255) / 256);
      ls.block[0] = 256;
      // A large nest that ends up here was not recognised for what it is (the optimiser's rewrites
      // were not undone): few work-items each walking a long stretch, or a reduction that stores
      // after its accumulating loop (a sum, a contraction that missed the matrix cores) run one
      // output per work-item.  Correct, slow, and said so in the plan.
      const double per_item = std::max(1.0, serial_iterations(*inner));
      const bool big = per_item * static_cast<double>(total) >= 1048576.0;
      const bool degraded = big && (total < 16384 || has_accumulating_loop(*inner));
      if (degraded) warn_once_degraded(k.name);
      ls.schedule = "outer-parallel(work-items=" + std::to_string(total) + (colliding ? ",atomics" : "") +
                    (degraded ? ",degraded)" : ")");
      any_parallel = true;
    } else {
      refuse_long_serial(k.name, *tops[t], opt);
      os << "extern \"C\" __global__ void " << ls.entry << "(" << sig << ") {\n" << sr.stmt(*tops[t]) << "}\n";
      ls.schedule = "as-written";
    }
    ls.source = os.str();
    out.push_back(std::move(ls));
  }
  if (!any_parallel) return {};
  return out;
}

// ---------------------------------------------------------------------------------------------
// canonical stages and grouping
// ---------------------------------------------------------------------------------------------

namespace {

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

struct Canon {
  bool ok = false;
  Stage stage;
  std::vector<int64_t> rows;
  int64_t C = 1;
};

Canon canon_as(const NestKernel& k, StageKind kind) {
  Canon c;
  c.ok = canonicalise(k, kind, &c.rows, &c.C, &c.stage);
  return c;
}

}  // namespace

// The emitters live below; declared here so plan_program reads top-down.
namespace {
LaunchSpec emit_group(const Group& g, const GenOptions& opt, const std::map<std::string, size_t>& buf_elems);
void emit_serial_reduce(const NestKernel& k, const GenOptions& opt, ProgramPlan* plan, const EpilogueSpec* epi = nullptr);
bool serial_reduce_is_one_launch(const NestKernel& k, const GenOptions& opt);
LaunchSpec merge_launches(const std::vector<LaunchSpec>& parts, const GenOptions& opt);
LaunchSpec emit_window_reduce(const NestKernel& r, const std::vector<const NestKernel*>& chain, const GenOptions& opt,
                              const std::map<std::string, size_t>& elems);
}  // namespace

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
std::optional<FoldedOperand> make_fold(const NestKernel& k, const std::map<std::string, size_t>& elems) {
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
  {
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

// ---------------------------------------------------------------------------------------------
// few, very long reduce lines: split over workgroups before planning
// ---------------------------------------------------------------------------------------------

namespace {

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
NodePtr make_reduce_block(const NestKernel& nk, const std::string& var, int64_t extent, const NodePtr& value,
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

struct RowSplit {
  NodePtr part, final_;      // the two kernels that replace the original
  BufferInfo scratch;        // [lines * chunks] partial results
};

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
bool same_under_renaming(const Node& s, const Node& r, const std::set<std::string>& s_vars, const std::set<std::string>& r_vars,
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

size_t count_loads(const Node& n) {
  size_t c = n.op == Op::Load ? 1 : 0;
  for (const auto& a : n.args)
    if (a) c += count_loads(*a);
  return c;
}

// R with every subexpression that equals what S stored (same loop extents under the renaming)
// replaced by a load of S's output; null when there is none.  Only expressions of two loads or
// more are taken: the point is to read one buffer instead of several.
NodePtr reuse_stored_value(const NestKernel& S, const NestKernel& R) {
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

bool pure_gather(const NestKernel& k) {
  const Node* v = k.value.get();
  if (v->op == Op::Select && v->args[2]->op == Op::Const) v = v->args[1].get();
  return v->op == Op::Load;
}

NodePtr replace_loads(const NodePtr& n, const std::string& buf, const NodePtr& with) {
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

std::optional<Inlined> inline_producer(const NestKernel& P, const NestKernel& C, bool same_space = false) {
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
NodePtr affine_expr(const Affine& a) {
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
std::optional<Affine> transposed_index(const Affine& a, const std::vector<Loop>& loops, const Loop* rloop, int64_t M, int64_t N) {
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

NodePtr reindex_loads(const NodePtr& n, const std::string& buf, const std::function<NodePtr(const Node&)>& new_index) {
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
NodePtr transpose_producer(const NestKernel& K, const GenOptions& opt, int64_t* Mo, int64_t* No) {
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
NodePtr transpose_reader(const NestKernel& E, const std::string& T, int64_t M, int64_t N) {
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

}  // namespace


// Which buffers each launch writes, and which launches may run beside each other.
//
// A program's launches are planned in an order that is valid one after the other.  Many of them
// do not depend on each other, though: in a training step the gradient of every parameter and
// its update hang off the chain that carries the gradient back through the layers, and most of
// them are small launches that cost their few microseconds of launch latency whatever they
// compute.  Launches are therefore given lanes: lane 0 (the device's stream) takes the chain of
// dependent launches with the largest estimated duration, the others go to side lanes that run
// concurrently; a launch waits for the launches on other lanes whose buffers it reads or
// overwrites (`waits`), and the executor joins the lanes at the end of the program.  The results
// do not depend on the lanes: every launch still sees exactly the inputs it would have seen.
// Which of its buffers each launch writes: the outputs of the lowered kernels it covers; a scratch
// buffer the plan added is written by the first launch that binds it and read by the later ones.
void mark_written(ProgramPlan* plan, const std::vector<const Node*>& kernels) {
  auto& L = plan->launches;
  std::map<std::string, const Node*> by_name;
  for (const Node* k : kernels) by_name[k->name] = k;
  // written: outputs of the lowered kernels a launch covers; a scratch buffer the plan added is
  // written by the first launch that binds it and read by the later ones
  std::set<std::string> scratch_seen;
  for (auto& ls : L) {
    std::set<std::string> outs;
    bool known = !ls.kernels.empty();
    for (const auto& kn : ls.kernels) {
      auto it = by_name.find(kn);
      if (it == by_name.end()) { known = false; continue; }
      for (const auto& p : it->second->params)
        if (p.dtype.is_ptr() && p.mut_) outs.insert(p.name);
    }
    // a launch whose kernels cannot be looked up is taken to write everything it binds
    ls.arg_written.assign(ls.arg_bufs.size(), known ? 0 : 1);
    for (size_t a = 0; a < ls.arg_bufs.size() && known; ++a) {
      const std::string& b = ls.arg_bufs[a];
      bool declared = false;
      for (const Node* k : kernels)
        for (const auto& p : k->params) declared = declared || p.name == b;
      if (outs.count(b)) ls.arg_written[a] = 1;
      else if (!declared && scratch_seen.insert(b).second) ls.arg_written[a] = 1;
    }
  }
}

// Launches of the elementwise / reduce schedules that do not depend on each other are issued as one
// launch (merge_launches).  A launch that could be merged is held until a launch that depends on it
// (reads what it writes, writes what it reads or writes) comes up; launches that depend on nothing
// held pass it by, which only changes the order among independent launches.  What is held at
// that point goes out together, grouped by workgroup size.
void issue_independent_launches_together(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt) {
  if (!(opt.fuse && opt.reindex && opt.merge_launches) || plan->launches.size() < 3) return;
  mark_written(plan, kernels);
  const std::string head = kernel_header();
  auto mergeable = [&](const LaunchSpec& ls) {
    if (ls.grid[1] != 1 || ls.grid[2] != 1 || ls.block[1] != 1 || ls.block[2] != 1 || ls.block[0] % 64 || ls.lds_bytes) return false;
    if (ls.source.rfind(head, 0) != 0 || ls.schedule.rfind("together(", 0) == 0 || ls.kernels.empty()) return false;
    const std::string open = "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(ls.block[0]) + ") " + ls.entry + "(";
    const size_t at = ls.source.find(open);
    return at != std::string::npos && ls.source.find("__global__", at + open.size()) == std::string::npos &&
           ls.source.find("blockIdx.y") == std::string::npos && ls.source.find("blockDim") == std::string::npos;
  };
  auto conflict = [](const LaunchSpec& a, const LaunchSpec& b) {
    for (size_t i = 0; i < a.arg_bufs.size(); ++i)
      for (size_t j = 0; j < b.arg_bufs.size(); ++j)
        if (a.arg_bufs[i] == b.arg_bufs[j] && (a.arg_written[i] || b.arg_written[j])) return true;
    return false;
  };
  std::vector<LaunchSpec> in = std::move(plan->launches), out, held;
  std::vector<char> taken(in.size(), 0);       // pulled forward into an earlier launch
  // The held launches of every workgroup size that has one in the way of `trigger` (all of them
  // at the end) go out as one launch per size.  Each takes along what further down the list could
  // run here just as well: launches of its size that depend on nothing between here and there
  // (the final launches of a training step, which nothing reads, were put at the end of the list).
  auto flush = [&](size_t next, const LaunchSpec* trigger) {
    std::map<unsigned, std::vector<LaunchSpec>> by_block;
    std::vector<LaunchSpec> stay;
    std::set<unsigned> go;
    for (const auto& h : held)
      if (!trigger || conflict(*trigger, h)) go.insert(h.block[0]);
    for (auto& h : held) {
      if (go.count(h.block[0])) by_block[h.block[0]].push_back(std::move(h));
      else stay.push_back(std::move(h));
    }
    held = std::move(stay);
    for (auto& kv : by_block) {
      for (size_t q = next; q < in.size(); ++q) {
        if (taken[q] || in[q].block[0] != kv.first || !mergeable(in[q])) continue;
        bool free_to_move = true;
        for (size_t p = next; p < q && free_to_move; ++p) free_to_move = taken[p] || !conflict(in[q], in[p]);
        for (const auto& h : held) free_to_move = free_to_move && !conflict(in[q], h);
        for (const auto& g : by_block)
          for (const auto& m : g.second) free_to_move = free_to_move && !conflict(in[q], m);
        if (!free_to_move) continue;
        kv.second.push_back(std::move(in[q]));
        taken[q] = 1;
      }
      if (kv.second.size() >= 2) out.push_back(merge_launches(kv.second, opt));
      else out.push_back(std::move(kv.second.front()));
    }
  };
  for (size_t q = 0; q < in.size(); ++q) {
    if (taken[q]) continue;
    LaunchSpec& ls = in[q];
    bool dep = false;
    for (const auto& h : held) dep = dep || conflict(ls, h);
    if (dep) flush(q, &ls);
    if (mergeable(ls)) held.push_back(std::move(ls));
    else out.push_back(std::move(ls));
    taken[q] = 1;
  }
  flush(in.size(), nullptr);
  plan->launches = std::move(out);
}

void assign_lanes(ProgramPlan* plan, const std::vector<const Node*>& kernels, const GenOptions& opt) {
  auto& L = plan->launches;
  const size_t n = L.size();
  mark_written(plan, kernels);
  plan->lanes = 1;
  for (auto& ls : L) { ls.lane = 0; ls.waits.clear(); }
  if (opt.lanes < 2 || n < 8) return;
  // dependences: read after write, write after write, write after read
  std::vector<std::vector<int>> deps(n);
  for (size_t j = 0; j < n; ++j)
    for (size_t i = 0; i < j; ++i) {
      bool dep = false;
      for (size_t a = 0; a < L[i].arg_bufs.size() && !dep; ++a)
        for (size_t b = 0; b < L[j].arg_bufs.size() && !dep; ++b)
          dep = L[i].arg_bufs[a] == L[j].arg_bufs[b] && (L[i].arg_written[a] || L[j].arg_written[b]);
      if (dep) deps[j].push_back(static_cast<int>(i));
    }
  // estimated microseconds: a launch floor plus traffic at half the memory rate or the matrix
  // cores at a third of theirs
  std::vector<double> est(n), path(n);
  std::vector<int> prev(n, -1);
  for (size_t j = 0; j < n; ++j) {
    est[j] = 4.0 + std::max(L[j].algo_bytes / 4.0e6, L[j].flops / 5.0e7);
    path[j] = est[j];
    for (int i : deps[j])
      if (path[static_cast<size_t>(i)] + est[j] > path[j]) {
        path[j] = path[static_cast<size_t>(i)] + est[j];
        prev[j] = i;
      }
  }
  size_t end = 0;
  for (size_t j = 0; j < n; ++j)
    if (path[j] > path[end]) end = j;
  std::vector<char> on_main(n, 0);
  for (int j = static_cast<int>(end); j >= 0; j = prev[static_cast<size_t>(j)]) on_main[static_cast<size_t>(j)] = 1;
  // a launch that fills the chip for long gains nothing from company and slows down in it
  if (opt.lane_us > 0)
    for (size_t j = 0; j < n; ++j)
      if (est[j] > opt.lane_us) on_main[j] = 1;
  // lane 0 never waits for a side lane: whatever a launch of lane 0 depends on is on lane 0 too
  for (size_t j = n; j-- > 0;)
    if (on_main[j])
      for (int i : deps[j]) on_main[static_cast<size_t>(i)] = 1;
  double side_us = 0;
  for (size_t j = 0; j < n; ++j)
    if (!on_main[j]) side_us += est[j];
  if (side_us < 24.0) return;                       // not worth a fork and a join
  const int lanes = std::min(opt.lanes, 4);
  // bottom level: what still has to run behind a launch, the launch included
  std::vector<double> tail(n);
  for (size_t j = n; j-- > 0;) {
    tail[j] = std::max(tail[j], est[j]);
    for (int i : deps[j]) tail[static_cast<size_t>(i)] = std::max(tail[static_cast<size_t>(i)], est[static_cast<size_t>(i)] + tail[j]);
  }
  // List scheduling: of the launches whose producers are placed, the one that can start first
  // goes next (the longer tail on a tie); chain launches on lane 0, the others on the side lane
  // that is free first.  The order of placement is the order of issue: a lane runs in order, so
  // a side lane must be handed its launches in the order in which their inputs become ready.
  std::vector<double> lane_free(static_cast<size_t>(lanes), 0.0), finish(n, 0.0);
  std::vector<char> placed(n, 0);
  std::vector<int> lane_of(n, 0);
  std::vector<size_t> order;
  while (order.size() < n) {
    int best = -1, best_lane = 0;
    double best_start = 0;
    for (size_t j = 0; j < n; ++j) {
      if (placed[j]) continue;
      bool ok = true;
      double ready = 0;
      int dep_lane = -1;
      for (int i : deps[j]) {
        ok = ok && placed[static_cast<size_t>(i)];
        if (finish[static_cast<size_t>(i)] >= ready) {
          ready = finish[static_cast<size_t>(i)];
          dep_lane = lane_of[static_cast<size_t>(i)];
        }
      }
      if (!ok) continue;
      int lane = 0;
      if (!on_main[j]) {
        lane = 1;
        for (int t = 2; t < lanes; ++t)
          if (lane_free[static_cast<size_t>(t)] < lane_free[static_cast<size_t>(lane)]) lane = t;
        // behind its last producer when that costs nothing: no wait across lanes then
        if (dep_lane > 0 && lane_free[static_cast<size_t>(dep_lane)] <= std::max(ready, lane_free[static_cast<size_t>(lane)])) lane = dep_lane;
      }
      const double start = std::max(ready, lane_free[static_cast<size_t>(lane)]);
      if (best < 0 || start < best_start - 1e-9 || (start < best_start + 1e-9 && tail[j] > tail[static_cast<size_t>(best)])) {
        best = static_cast<int>(j);
        best_lane = lane;
        best_start = start;
      }
    }
    const size_t j = static_cast<size_t>(best);
    placed[j] = 1;
    lane_of[j] = best_lane;
    finish[j] = best_start + est[j];
    lane_free[static_cast<size_t>(best_lane)] = finish[j];
    order.push_back(j);
  }
  std::vector<int> position(n);
  for (size_t q = 0; q < n; ++q) position[order[q]] = static_cast<int>(q);
  std::vector<LaunchSpec> sorted;
  sorted.reserve(n);
  for (size_t q = 0; q < n; ++q) {
    sorted.push_back(std::move(L[order[q]]));
    sorted.back().lane = lane_of[order[q]];
    plan->lanes = std::max(plan->lanes, sorted.back().lane + 1);
  }
  // a lane runs its launches in order, so waiting for one launch of a lane covers that lane's
  // earlier launches too
  std::vector<std::vector<int>> waited(static_cast<size_t>(lanes), std::vector<int>(static_cast<size_t>(lanes), -1));
  for (size_t q = 0; q < n; ++q) {
    const size_t lj = static_cast<size_t>(sorted[q].lane);
    std::vector<int> latest(static_cast<size_t>(lanes), -1);
    for (int i : deps[order[q]]) {
      const int pi = position[static_cast<size_t>(i)];
      const size_t li = static_cast<size_t>(sorted[static_cast<size_t>(pi)].lane);
      if (li != lj) latest[li] = std::max(latest[li], pi);
    }
    for (size_t t = 0; t < latest.size(); ++t)
      if (latest[t] > waited[lj][t]) {
        sorted[q].waits.push_back(latest[t]);
        waited[lj][t] = latest[t];
      }
  }
  L = std::move(sorted);
}

ProgramPlan plan_program(const Node& program, const GenOptions& opt) {
  if (program.op != Op::Program) throw Error("expected a program node");
  g_guard_branches = opt.guard_branches;
  g_ranged_loads = opt.ranged_loads;
  validate_sizes(program);
  ProgramPlan plan;
  std::vector<const Node*> kernels;
  for (const auto& f : program.args) {
    if (f->op == Op::Kernel) kernels.push_back(f.get());
    else if (f->op == Op::Function) throw Error("helper functions in a program are not supported by this backend");
  }
  if (kernels.empty()) throw Error("program holds no kernel");
  std::vector<NodePtr> rewritten;          // owns the kernels that replace given ones
  // what the reference's AST optimiser did to the lowered loop nests is undone first
  if (opt.normalize)
    for (size_t q = 0; q < kernels.size(); ++q)
      for (const auto& f : program.args)
        if (f.get() == kernels[q]) {
          NodePtr nk = normalize_kernel(f);
          if (nk != f) {
            rewritten.push_back(nk);
            kernels[q] = nk.get();
          }
        }

  // buffer table: given, or synthesised from the kernels' pointer parameters
  plan.buffers = program.buffers;
  if (!plan.buffers.empty() && opt.fuse) {
    std::vector<const Node*> out;
    for (const Node* k : kernels) {
      auto nk = extract_nest(*k);
      auto rs = nk ? split_long_rows(*nk) : std::nullopt;
      if (!rs) { out.push_back(k); continue; }
      rewritten.push_back(rs->part);
      rewritten.push_back(rs->final_);
      out.push_back(rs->part.get());
      out.push_back(rs->final_.get());
      plan.buffers.push_back(rs->scratch);
    }
    kernels = out;
  }
  if (!plan.buffers.empty() && opt.fuse && opt.reindex) rewrite_for_readers(program, opt, &kernels, &rewritten, &plan);
  if (!plan.buffers.empty() && opt.fuse && opt.reindex) {
    // An elementwise kernel separated from the kernel that produces what it reads by small
    // kernels it has nothing to do with (the roots of a step are lowered one after another, so
    // the loss's bookkeeping of a few thousand elements can land inside another root's chain)
    // moves up behind its producer, where the producer's fused launch can take it.  Past a large
    // kernel it stays: computed early, its result would have to be kept in memory instead.
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
  std::map<std::string, size_t> elems;
  bool have_table = !plan.buffers.empty();
  if (have_table) {
    for (const auto& b : plan.buffers) elems[b.name] = b.numel();
  } else {
    std::set<std::string> seen;
    for (const Node* k : kernels)
      for (const auto& p : k->params)
        if (p.dtype.is_ptr() && seen.insert(p.name).second) {
          BufferInfo bi;
          bi.name = p.name;
          bi.dtype = p.dtype.elem();
          bi.role = p.mut_ ? "output" : "input";
          bi.shape_known = false;
          plan.buffers.push_back(bi);
        } else if (p.dtype.is_ptr() && p.mut_) {
          for (auto& b : plan.buffers)
            if (b.name == p.name) b.role = "output";
        }
  }
  auto role_of = [&](const std::string& name) -> std::string {
    for (const auto& b : plan.buffers)
      if (b.name == name) return b.role;
    throw Error("kernel parameter '" + name + "' is missing from the program's buffer table");
  };
  for (const Node* k : kernels)
    for (const auto& p : k->params)
      if (p.dtype.is_ptr()) role_of(p.name);

  // consumers per buffer (kernel indices)
  std::map<std::string, std::vector<size_t>> readers;
  for (size_t i = 0; i < kernels.size(); ++i)
    for (const auto& p : kernels[i]->params)
      if (p.dtype.is_ptr() && !p.mut_) readers[p.name].push_back(i);

  // inputs the executor itself fills with a constant (role ones / zeros): reads of them are
  // folded into literals wherever a kernel is recognised, so they cost no memory traffic
  std::map<std::string, double> consts;
  for (const auto& b : plan.buffers) {
    if (b.role == "ones") consts[b.name] = 1.0;
    if (b.role == "zeros") consts[b.name] = 0.0;
  }
  std::function<NodePtr(const NodePtr&)> fold = [&](const NodePtr& n) -> NodePtr {
    if (n->op == Op::Load && n->args[0]->op == Op::Var && consts.count(n->args[0]->name) && n->count == 1) {
      auto c = std::make_shared<Node>(Op::Const);
      c->dtype = n->dtype;
      c->fval = consts.at(n->args[0]->name);
      c->ival = static_cast<int64_t>(c->fval);
      return c;
    }
    bool changed = false;
    std::vector<NodePtr> args;
    for (const auto& a : n->args) {
      NodePtr r = fold(a);
      changed = changed || r != a;
      args.push_back(std::move(r));
    }
    if (!changed) return n;
    auto c = std::make_shared<Node>(*n);
    c->args = std::move(args);
    return c;
  };

  std::vector<std::optional<NestKernel>> nests;
  for (const Node* k : kernels) {
    nests.push_back(extract_nest(*k));
    if (nests.back() && nests.back()->rkind == ReduceKind::None) {
      // An elementwise nest has no loop-carried dependence, so its loops may run in any order:
      // walk the output in address order (largest stride outermost).  A kernel lowered through
      // a transposing view otherwise strides through memory with its innermost loop, and it
      // would not share an index space with the kernel that produced its operand.
      NestKernel& nk = *nests.back();
      const Affine& oa = *nk.out_aff;
      bool all_used = true;
      for (const auto& l : nk.loops) all_used = all_used && (l.extent == 1 || oa.of(l.var) != 0);
      if (all_used) {
        std::vector<Loop> wide;                       // loops of extent 1 keep their places
        for (const auto& l : nk.loops)
          if (l.extent > 1) wide.push_back(l);
        std::stable_sort(wide.begin(), wide.end(), [&](const Loop& a, const Loop& b) {
          return std::llabs(oa.of(a.var)) > std::llabs(oa.of(b.var));
        });
        size_t w = 0;
        for (auto& l : nk.loops)
          if (l.extent > 1) l = wide[w++];
      }
    }
    if (nests.back() && !consts.empty()) {
      NestKernel& nk = *nests.back();
      nk.value = fold(nk.value);
      std::vector<LoadRef> loads;
      collect_loads(*nk.value, loads);
      std::set<std::string> used;
      for (const auto& lr : loads) used.insert(lr.load->args[0]->name);
      std::vector<Param> kept;
      for (const auto& p : nk.params)
        if (p.mut_ || used.count(p.name) || !consts.count(p.name)) kept.push_back(p);
      nk.params = kept;
    }
  }

  // A contraction per batch element whose results the next kernel sums over the batch (the
  // weight gradient of a convolution: per-image products, then a sum over images) is one
  // contraction with the batch folded into k, when both operands walk (batch, k) as one axis.
  // The summing kernel disappears, and so does the per-batch result buffer.
  std::set<size_t> absorbed;
  std::map<size_t, std::string> absorbed_name;
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

  // A sum over one axis whose result the next kernel only sums over a neighbouring axis (a bias
  // gradient as the reference lowers it: over the image's columns, then its rows, then the
  // batch) is one sum over both when every operand walks the two axes as one: the second kernel
  // and the buffer between them disappear, and what was two short strided passes is one pass
  // along memory.  (The order of the additions changes, as it does in every parallel reduce.)
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

  // gather / copy kernels read only by contractions are evaluated inside those contractions'
  // tile loaders (implicit GEMM): no launch, no buffer
  FoldMap folded;
  std::set<size_t> folded_kernels;
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

  // A short reduce over windows that pure gather kernels laid out for it (max-pool, avg-pool:
  // unfold, copy, reduce over the window axis) reads the source through the gathers' index
  // maps instead: the window buffers are never written.
  std::map<size_t, std::vector<size_t>> windows;     // reduce kernel -> its gathers, nearest first
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
      windows[r] = chain;
      for (size_t q : chain) {
        folded_kernels.insert(q);
        writer.erase(nests[q]->out_buf);
        plan.elided.insert(nests[q]->out_buf);
      }
    }
  }

  // A contraction whose result only a run of kernels adding up shifted reads of it sees (the
  // input gradient of a convolution) is one window contraction with those kernels.
  std::map<size_t, ScatteredWindow> scattered;
  std::set<std::string> partly_written;      // kernels whose output is written only where it is read
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
      auto sw = try_emit_scattered_window(q, pv, opt);
      if (!sw) continue;
      for (size_t c = q + 1; c < sw->next; ++c) absorbed.insert(c);
      for (const auto& b : sw->elided) plan.elided.insert(b);
      if (sw->partial) partly_written.insert(nests[sw->next - 1]->name);
      scattered[q] = std::move(*sw);
    }
  }

  // Elementwise kernels that follow kernel i (a reduce with a dense output of `total` elements)
  // over the same dense index space and feed on its result: the function that applies them to
  // one element while it is still in a register.  `k0r`: k0 with its output laid out as a
  // consumer that reads it through a permutation wants it, when that applies and is allowed.
  auto build_epilogue = [&](size_t i, const NestKernel& k0, int64_t total, bool allow_relayout, NestKernel& k0r,
                            EpilogueSpec& epi, size_t& after) -> bool {
    bool have_epi = false;
    const bool small = total < (int64_t{1} << 30);
    std::map<std::string, DType> avail;          // values held in registers: C and stage outputs
    avail[k0.out_buf] = k0.out_dtype;
    bool c_relaid = false;
    size_t relaid_pos = 0;                       // position in `taken` of the stage that reads through a permutation
    Affine relaid_read;                          // ... and the index it reads at, over its own loops
    std::set<std::string> old_space;             // values produced before that stage
    std::set<size_t> independent;                // taken stages that read no value of the chain
    std::vector<size_t> taken;
    size_t j = i + 1;
    for (; j < kernels.size(); ++j) {
      if (absorbed.count(j)) continue;
      if (!nests[j] || folded_kernels.count(j) || nests[j]->rkind != ReduceKind::None) break;
      const NestKernel& sk = *nests[j];
      int64_t numel = 0;
      auto strides = dense_strides(sk, &numel);
      if (!strides || numel != total || avail.count(sk.out_buf)) break;
      std::vector<LoadRef> loads;
      collect_loads(*sk.value, loads);
      bool feeds = false, ok = true;
      std::optional<Affine> permuted;            // the one index all values of the chain are read at, if not the aligned one
      for (const auto& lr : loads) {
        if (lr.load->args[0]->op != Op::Var || lr.load->count != 1) { ok = false; break; }
        const std::string& b = lr.load->args[0]->name;
        if (!avail.count(b)) continue;
        auto a = affine_of(*lr.load->args[1]);
        if (!a) { ok = false; break; }
        const bool aligned = *a == *sk.out_aff;
        if (c_relaid && (old_space.count(b) || !aligned)) { ok = false; break; }
        if (!aligned) {
          if (feeds && !permuted) { ok = false; break; }          // the stage reads the chain both ways
          if (permuted && !(*permuted == *a)) { ok = false; break; }
          permuted = *a;
        } else if (permuted) {
          ok = false;
          break;
        }
        feeds = true;
      }
      if (!ok) break;
      // a stage over the same index space that reads nothing of the chain (the square of a
      // saved activation, say) rides along when a later stage combines it with the chain
      if (!feeds) independent.insert(j);
      if (permuted) {
        // A consumer may read the chain's values through a permutation (a transposed weight
        // gradient and its update, NHWC -> NCHW after a convolution).  If nothing computed so
        // far is needed outside the chain, the contraction can put each element where this
        // consumer wants it: C takes the consumer's index space, the stages before it are
        // evaluated at the element's original position, and the read becomes the aligned one.
        bool sole = true;
        for (const auto& kv : avail) {
          sole = sole && role_of(kv.first) == "temp";
          for (size_t r : readers[kv.first]) sole = sole && r > i && r <= j;
        }
        auto na = sole && allow_relayout ? relayout(k0, sk, *permuted) : std::nullopt;
        if (!na) break;
        k0r.out_aff = *na;
        if (!gemm_shaped(k0r, opt)) { k0r.out_aff = k0.out_aff; break; }
        c_relaid = true;
        relaid_pos = taken.size();
        relaid_read = *permuted;
        for (const auto& kv : avail) old_space.insert(kv.first);
      }
      avail[sk.out_buf] = sk.out_dtype;
      taken.push_back(j);
    }
    while (!taken.empty() && independent.count(taken.back())) {
      avail.erase(nests[taken.back()]->out_buf);      // nothing after it uses the chain: leave it out
      independent.erase(taken.back());
      taken.pop_back();
    }
    if (!taken.empty()) {
      after = taken.back() + 1;
      auto needed = [&](const std::string& buf) {
        if (role_of(buf) != "temp") return true;
        for (size_t r : readers[buf])
          if (r <= i || r >= after) return true;
        return false;
      };
      std::ostringstream fn, body;
      // the same function in two parts, for schedules that finish many elements per work-item in a
      // row: everything read from memory first (eh_epilogue_load), the arithmetic and the stores
      // after (eh_epilogue_apply); only when no read sits under a guard
      std::ostringstream load_body, apply_body;
      std::vector<std::string> slot_types;
      bool split_ok = true;
      // ... and for four elements in a row (eh_e a multiple of four): what does not move inside the
      // four is read once, what is read at the element itself as one vector, stores as vectors
      std::ostringstream quad_load, quad_apply;
      std::vector<std::string> quad_slots;         // declarations of EhEpiLoads4's members
      int quad_regs = 0;
      bool quad_ok = !(c_relaid && relaid_pos > 0);
      std::vector<std::string> ext_order;
      std::map<std::string, std::pair<std::string, size_t>> ext;   // name -> (declaration, min bytes)
      epi.store_c = needed(k0.out_buf);
      if (!epi.store_c) plan.elided.insert(k0.out_buf);
      const std::string IT = small ? "int" : "long long";
      const std::string UT = small ? "unsigned" : "unsigned long long";
      body << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n";
      load_body << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n";
      body << "  const " << ctype(k0.out_dtype) << " eh_v_" << k0.out_buf << " = eh_acc;\n";
      if (epi.store_c) body << "  " << k0.out_buf << "[eh_e] = eh_acc;\n";
      apply_body << body.str();
      quad_load << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n";
      quad_apply << "  const " << IT << " eh_l = (" << IT << ")eh_e;\n  (void)eh_l;\n  " << ctype(k0.out_dtype) << " eh_v_" << k0.out_buf
                 << "[4] = {eh_acc[0], eh_acc[1], eh_acc[2], eh_acc[3]};\n";
      if (epi.store_c)
        quad_apply << "  *reinterpret_cast<EhQ<float>*>(" << k0.out_buf << " + eh_e) = EhQ<float>{eh_acc[0], eh_acc[1], eh_acc[2], eh_acc[3]};\n";
      auto decode_to = [&](std::ostringstream& to, const NestKernel& sk, const std::string& from) {
        int64_t numel = 0;
        auto strides = *dense_strides(sk, &numel);
        for (size_t li = 0; li < sk.loops.size(); ++li) {
          const Loop& l = sk.loops[li];
          if (l.extent == 1) to << "    const " << IT << " " << l.var << " = 0;\n";
          else to << "    const " << IT << " " << l.var << " = (" << IT << ")(((" << UT << ")" << from << " / " << strides[li] << "u) % "
                  << l.extent << "u);\n";    // (never negative: the unsigned division is the cheaper one)
        }
      };
      auto decode = [&](const NestKernel& sk, const std::string& from) { decode_to(body, sk, from); };
      if (c_relaid && relaid_pos > 0) {
        // where this element sat before C took the later consumer's layout: the stages
        // ahead of that consumer index their other operands with it
        if (epi.store_c) throw Error("internal: relaid contraction '" + k0.name + "' must not store C");
        split_ok = false;
        body << "  " << IT << " eh_lo;\n  {\n";
        decode(*nests[taken[relaid_pos]], "eh_l");
        body << "    eh_lo = ";
        bool first_term = true;
        for (const auto& kv : relaid_read.coef) {
          if (kv.second == 0) continue;
          body << (first_term ? "" : " + ") << kv.first << " * " << kv.second;
          first_term = false;
        }
        if (first_term) body << "0";
        body << ";\n  }\n";
      }
      for (size_t ti = 0; ti < taken.size(); ++ti) {
        const size_t j2 = taken[ti];
        const NestKernel& sk = *nests[j2];
        epi.kernels.push_back(sk.name);
        body << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << ";\n  {\n";
        decode(sk, (c_relaid && ti < relaid_pos) ? "eh_lo" : "eh_l");
        ExprRenderer er;
        er.load_hook = [&](const Node& ld, std::string* out) {
          const std::string& b = ld.args[0]->name;
          if (!avail.count(b)) return false;
          *out = "eh_v_" + b;
          return true;
        };
        std::vector<LoadRef> loads;
        collect_loads(*sk.value, loads);
        for (const auto& lr : loads) {
          const std::string& b = lr.load->args[0]->name;
          if (avail.count(b) || ext.count(b)) {
            if (ext.count(b) && !lr.guarded) {
              if (auto a = affine_of(*lr.load->args[1]))
                ext[b].second = std::max(ext[b].second, static_cast<size_t>(max_abs_index(*a, sk.loops, nullptr) + 1) *
                                                             lr.load->dtype.itemsize());
            }
            continue;
          }
          size_t mb = 0;
          if (!lr.guarded)
            if (auto a = affine_of(*lr.load->args[1]))
              mb = static_cast<size_t>(max_abs_index(*a, sk.loops, nullptr) + 1) * lr.load->dtype.itemsize();
          DType et = lr.load->dtype;
          for (const auto& pp : sk.params)
            if (pp.name == b) et = pp.dtype.elem();
          ext[b] = {"const " + ctype(et) + "* __restrict__ " + b, mb};
          ext_order.push_back(b);
          epi.bytes += static_cast<double>(elems.count(b) ? elems.at(b) : 0) * et.itemsize();
        }
        body << "    eh_v_" << sk.out_buf << " = (" << ctype(sk.out_dtype) << ")(" << er.expr(*sk.value) << ");\n";
        {
          // the two-part form of this stage
          std::set<const Node*> guarded;
          for (const auto& lr : loads)
            if (lr.guarded) guarded.insert(lr.load);
          apply_body << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << ";\n  {\n";
          decode_to(apply_body, sk, "eh_l");
          load_body << "  {\n";
          decode_to(load_body, sk, "eh_l");
          ExprRenderer er2;
          er2.load_hook = [&](const Node& ld, std::string* out) {
            const std::string& lb = ld.args[0]->name;
            if (avail.count(lb)) {
              *out = "eh_v_" + lb;
              return true;
            }
            if (guarded.count(&ld)) split_ok = false;
            ExprRenderer plain;
            const std::string slot = "eh_p.v" + std::to_string(slot_types.size());
            load_body << "    " << slot << " = " << plain.expr(ld) << ";\n";
            slot_types.push_back(ctype(ld.dtype));
            *out = slot;
            return true;
          };
          apply_body << "    eh_v_" << sk.out_buf << " = (" << ctype(sk.out_dtype) << ")(" << er2.expr(*sk.value) << ");\n";
          load_body << "  }\n";
          if (needed(sk.out_buf)) apply_body << "    " << sk.out_buf << "[eh_e] = eh_v_" << sk.out_buf << ";\n";
          apply_body << "  }\n";
        }
        if (quad_ok) {
          int64_t numel4 = 0;
          const auto strides4 = *dense_strides(sk, &numel4);
          std::set<std::string> still, vars;      // loops that keep their value over four aligned elements; all loops
          for (size_t li = 0; li < sk.loops.size(); ++li) {
            vars.insert(sk.loops[li].var);
            if (sk.loops[li].extent == 1 || strides4[li] % 4 == 0) still.insert(sk.loops[li].var);
          }
          std::function<bool(const Node&)> as_value = [&](const Node& n) {
            if (n.op == Op::Load) return false;
            if ((n.op == Op::Var || n.op == Op::Wildcard) && vars.count(n.name)) return true;
            for (const auto& a : n.args)
              if (a && as_value(*a)) return true;
            return false;
          };
          if (as_value(*sk.value) || (needed(sk.out_buf) && sk.out_dtype.itemsize() != 4)) quad_ok = false;
          quad_load << "  {\n";
          decode_to(quad_load, sk, "eh_l");
          quad_apply << "  " << ctype(sk.out_dtype) << " eh_v_" << sk.out_buf << "[4];\n  {\n";
          std::map<const Node*, std::string> slot_of;
          for (int c = 0; c < 4 && quad_ok; ++c) {
            ExprRenderer er4;
            er4.load_hook = [&](const Node& ld, std::string* out) {
              const std::string& lb = ld.args[0]->name;
              const std::string comp = "[" + std::to_string(c) + "]";
              if (avail.count(lb)) {
                *out = "eh_v_" + lb + comp;
                return true;
              }
              auto known = slot_of.find(&ld);
              if (known == slot_of.end()) {
                auto a = affine_of(*ld.args[1]);
                bool uniform = a.has_value();
                if (a)
                  for (const auto& kv : a->coef) uniform = uniform && (kv.second == 0 || still.count(kv.first));
                const bool at_element = a && sk.out_aff && *a == *sk.out_aff && ld.dtype.itemsize() == 4;
                for (const auto& lr : loads)
                  if (lr.load == &ld && lr.guarded) uniform = false;
                const std::string name = "eh_p.s" + std::to_string(quad_slots.size());
                if (uniform) {
                  ExprRenderer plain;
                  quad_load << "    " << name << " = " << plain.expr(ld) << ";\n";
                  quad_slots.push_back(ctype(ld.dtype) + " s" + std::to_string(quad_slots.size()));
                  quad_regs += 1;
                  known = slot_of.emplace(&ld, name).first;
                } else if (at_element) {
                  quad_load << "    " << name << " = *reinterpret_cast<const EhQ<" << ctype(ld.dtype) << ">*>(" << lb << " + eh_e);\n";
                  quad_slots.push_back("EhQ<" + ctype(ld.dtype) + "> s" + std::to_string(quad_slots.size()));
                  quad_regs += 4;
                  known = slot_of.emplace(&ld, name + "[]").first;
                } else {
                  quad_ok = false;
                  *out = "0";
                  return true;
                }
              }
              const std::string& sl = known->second;
              *out = sl.size() > 2 && sl.compare(sl.size() - 2, 2, "[]") == 0 ? sl.substr(0, sl.size() - 2) + comp : sl;
              return true;
            };
            quad_apply << "    eh_v_" << sk.out_buf << "[" << c << "] = (" << ctype(sk.out_dtype) << ")(" << er4.expr(*sk.value) << ");\n";
          }
          quad_load << "  }\n";
          if (needed(sk.out_buf))
            quad_apply << "    *reinterpret_cast<EhQ<" << ctype(sk.out_dtype) << ">*>(" << sk.out_buf << " + eh_e) = EhQ<" << ctype(sk.out_dtype)
                       << ">{eh_v_" << sk.out_buf << "[0], eh_v_" << sk.out_buf << "[1], eh_v_" << sk.out_buf << "[2], eh_v_" << sk.out_buf
                       << "[3]};\n";
          quad_apply << "  }\n";
        }
        if (needed(sk.out_buf)) {
          body << "    " << sk.out_buf << "[eh_e] = eh_v_" << sk.out_buf << ";\n";
          ext[sk.out_buf] = {ctype(sk.out_dtype) + "* __restrict__ " + sk.out_buf,
                             static_cast<size_t>(total) * sk.out_dtype.itemsize()};
          ext_order.push_back(sk.out_buf);
          epi.bytes += static_cast<double>(total) * sk.out_dtype.itemsize();
        } else {
          plan.elided.insert(sk.out_buf);
        }
        body << "  }\n";
      }
      for (const auto& b : ext_order) {
        epi.params += ", " + ext[b].first;
        epi.args += ", " + b;
        epi.bufs.push_back(b);
        epi.min_bytes.push_back(ext[b].second);
      }
      fn << "// what kernels";
      for (const auto& n : epi.kernels) fn << " " << n;
      fn << " do to element eh_e of " << k0.out_buf << "\n";
      fn << "__device__ __forceinline__ void eh_epilogue(long long eh_e, float eh_acc"
         << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params
         << ") {\n" << body.str() << "}\n";
      epi.function = fn.str();
      if (split_ok && !slot_types.empty() && slot_types.size() <= 8) {
        std::ostringstream sp;
        sp << "// the same in two parts: what it reads from memory, then the rest\nstruct EhEpiLoads {\n";
        for (size_t q = 0; q < slot_types.size(); ++q) sp << "  " << slot_types[q] << " v" << q << ";\n";
        sp << "};\n__device__ __forceinline__ void eh_epilogue_load(long long eh_e, EhEpiLoads& eh_p" << epi.params << ") {\n"
           << load_body.str() << "}\n";
        sp << "__device__ __forceinline__ void eh_epilogue_apply(long long eh_e, float eh_acc, const EhEpiLoads& eh_p"
           << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params << ") {\n"
           << apply_body.str() << "}\n";
        epi.split_functions = sp.str();
        epi.n_loads = static_cast<int>(slot_types.size());
      }
      if (quad_ok && total % 4 == 0 && quad_regs <= 24) {
        std::ostringstream qd;
        qd << "// the same for four elements in a row (eh_e a multiple of four), reads first\n"
              "template <typename T> using EhQ = T __attribute__((ext_vector_type(4)));\nstruct EhEpiLoads4 {\n";
        for (const auto& d : quad_slots) qd << "  " << d << ";\n";
        qd << "};\n__device__ __forceinline__ void eh_epilogue_load4(long long eh_e, EhEpiLoads4& eh_p" << epi.params << ") {\n"
           << quad_load.str() << "}\n";
        qd << "__device__ __forceinline__ void eh_epilogue_apply4(long long eh_e, const float (&eh_acc)[4], const EhEpiLoads4& eh_p"
           << (epi.store_c ? ", " + ctype(k0.out_dtype) + "* __restrict__ " + k0.out_buf : std::string()) << epi.params << ") {\n"
           << quad_apply.str() << "}\n";
        epi.quad_functions = qd.str();
        epi.quad_regs = quad_regs;
      }
      have_epi = true;
    }
    return have_epi;
  };

  std::vector<LaunchSpec> held_back;       // independent final reductions, issued together at the end
  // The launch just planned for kernels [i, next) (the last of them, when there are two) can run
  // whenever its inputs are ready if nothing later reads what it writes or writes what it reads
  // (a parameter's update at the end of its gradient's chain): it is taken out of the sequence.
  auto hold_back_if_sink = [&](size_t i, size_t next) {
    if (!(opt.fuse && opt.reindex && opt.merge_launches && have_table) || plan.launches.empty()) return;
    const LaunchSpec& ls = plan.launches.back();
    if (ls.grid[1] != 1 || ls.grid[2] != 1 || ls.lds_bytes || ls.block[0] % 64 || ls.source.rfind(kernel_header(), 0) != 0) return;
    std::set<std::string> written;
    for (size_t q = i; q < next; ++q)
      if (nests[q]) written.insert(nests[q]->out_buf);
      else return;
    bool sink = true;
    for (const auto& b : written)
      for (size_t r : readers[b]) sink = sink && r < next;
    for (size_t m = next; m < kernels.size() && sink; ++m)
      for (const auto& pm : kernels[m]->params)
        if (pm.dtype.is_ptr() && pm.mut_)
          sink = sink && std::find(ls.arg_bufs.begin(), ls.arg_bufs.end(), pm.name) == ls.arg_bufs.end();
    if (!sink) return;
    held_back.push_back(plan.launches.back());
    plan.launches.pop_back();
  };
  size_t i = 0;
  while (i < kernels.size()) {
    if (folded_kernels.count(i) || absorbed.count(i)) {
      ++i;
      continue;
    }
    if (auto sw = scattered.find(i); sw != scattered.end()) {
      for (auto& ls : sw->second.launches) plan.launches.push_back(std::move(ls));
      i = sw->second.next;
      continue;
    }
    if (auto w = windows.find(i); w != windows.end()) {
      std::vector<const NestKernel*> chain;
      for (size_t q : w->second) chain.push_back(&*nests[q]);
      plan.launches.push_back(emit_window_reduce(*nests[i], chain, opt, elems));
      ++i;
      continue;
    }
    if (!nests[i]) {
      auto spread = render_kernel_outer_parallel(*kernels[i], opt, have_table && opt.fuse ? &plan.buffers : nullptr);
      if (spread.empty()) plan.launches.push_back(render_kernel_as_written(*kernels[i], opt));
      else for (auto& ls : spread) plan.launches.push_back(std::move(ls));
      ++i;
      continue;
    }
    const NestKernel& k0 = *nests[i];
    // contraction (matmul-shaped reduce) -> MFMA schedule
    if (k0.rkind == ReduceKind::Sum && opt.gemm) {
      // elementwise kernels that follow over the same dense index space and feed on the
      // result become the contraction's epilogue
      EpilogueSpec epi;
      size_t after = i + 1;
      bool have_epi = false;
      NestKernel k0r = k0;          // k0 with C laid out as its consumer wants it, when that applies
      if (opt.gemm_epilogue && opt.fuse && have_table && gemm_shaped(k0, opt)) {
        auto gs = match_gemm(k0);
        if (gs && gemm_output_dense(*gs)) {
          have_epi = build_epilogue(i, k0, gs->batch * gs->M * gs->N, true, k0r, epi, after);
        }
      }
      auto gl = try_emit_gemm(have_epi ? k0r : k0, opt, &plan.buffers, &folded, have_epi ? &epi : nullptr);
      if (!gl.empty()) {
        if (absorbed_name.count(i)) gl.back().kernels.push_back(absorbed_name[i]);
        // K was split and the next kernel only sums the (dense) result over the batch axis: it
        // sums the partial tiles of all chunks and all batch elements in one go (chunks lie
        // above the batch in the scratch buffer, so the two walk as one axis), and the launch
        // that would add the chunks up goes
        if (gl.size() == 2 && !have_epi && !absorbed_name.count(i) && opt.fuse && opt.reindex && have_table) {
          size_t j = i + 1;
          while (j < kernels.size() && (absorbed.count(j) || folded_kernels.count(j))) ++j;
          auto gs = match_gemm(k0);
          const std::string& scratch = gl[0].arg_bufs.back();
          if (j < kernels.size() && nests[j] && gs && gs->batch > 1 && gemm_output_dense(*gs) &&
              gl[0].grid[1] > 1 && scratch.rfind("eh_part_", 0) == 0) {
            NestKernel& r2 = *nests[j];
            const Node& v2 = *r2.value;
            auto ra = v2.op == Op::Load && v2.count == 1 && v2.args[0]->op == Op::Var && v2.args[0]->name == k0.out_buf
                          ? affine_of(*v2.args[1]) : std::nullopt;
            const int64_t tile = gs->M * gs->N;
            bool ok = r2.rkind == ReduceKind::Sum && ra && ra->c == 0 && r2.acc_dtype.ty == Ty::F32 &&
                      r2.rloop.extent == gs->batch && ra->of(r2.rloop.var) == tile && role_of(k0.out_buf) == "temp" &&
                      readers[k0.out_buf] == std::vector<size_t>{j} && !(opt.gemm && gemm_shaped(r2, opt));
            // the other loops of r2 stay inside one tile
            int64_t reach = 0;
            if (ok)
              for (const auto& l : r2.loops) {
                if (l.extent <= 1) continue;
                ok = ok && ra->of(l.var) > 0;
                reach += ra->of(l.var) * (l.extent - 1);
              }
            if (ok && reach < tile) {
              const int64_t S = gl[0].grid[1];
              std::map<std::string, NodePtr> to_scratch{{k0.out_buf, make_var(scratch)}};
              r2.value = rename(r2.value, to_scratch);
              r2.rloop.extent *= S;
              for (auto& pp : r2.params)
                if (pp.name == k0.out_buf) pp.name = scratch;
              plan.elided.insert(k0.out_buf);
              gl.pop_back();
            }
          }
        }
        const bool two = gl.size() == 2;
        for (auto& ls : gl) plan.launches.push_back(std::move(ls));
        if (two && !absorbed_name.count(i)) hold_back_if_sink(i, have_epi ? after : i + 1);   // the launch that sums the chunks (and updates the weight)
        i = have_epi ? after : i + 1;
        continue;
      }
      if (have_epi) throw Error("internal: contraction '" + k0.name + "' matched but could not be emitted");
    }
    if (k0.rkind != ReduceKind::None && !reduce_is_rowwise(k0)) {
      // elementwise kernels over the reduce's (dense) output that feed on it ride along: a
      // parameter's update in the launch that finishes its gradient's sum
      EpilogueSpec epi;
      size_t after = i + 1;
      NestKernel k0r = k0;
      int64_t numel = 0;
      bool have_epi = false;
      if (opt.gemm_epilogue && opt.fuse && have_table && k0.acc_dtype.ty == Ty::F32 && k0.out_dtype.ty == Ty::F32 &&
          dense_strides(k0, &numel))
        have_epi = build_epilogue(i, k0, numel, false, k0r, epi, after);
      emit_serial_reduce(k0, opt, &plan, have_epi ? &epi : nullptr);
      // A one-launch reduce at the end of its chain (nothing later reads what it writes or
      // writes what it reads: a parameter's update) can run whenever its inputs are ready:
      // it is held back and issued together with the others of its kind as one launch.
      hold_back_if_sink(i, have_epi ? after : i + 1);
      i = have_epi ? after : i + 1;
      continue;
    }
    // start a group with kernel i and extend it while the next kernels fit
    Group g;
    size_t first = i;
    {
      Canon c = canon_as(k0, k0.rkind == ReduceKind::None ? StageKind::Wide : StageKind::Reduce);
      if (!c.ok) {
        plan.launches.push_back(render_kernel_as_written(*kernels[i], opt));
        ++i;
        continue;
      }
      g.rows = c.rows;
      g.C = c.C;
      g.stages.push_back(c.stage);
    }
    ++i;
    // kernel k as the group's next stage, if it fits
    auto stage_for = [&](const NestKernel& k) {
      Canon pick;
      if (k.rkind == ReduceKind::Sum && opt.gemm && gemm_shaped(k, opt)) return pick;
      if (k.rkind != ReduceKind::None) {
        if (!reduce_is_rowwise(k)) return pick;
        Canon c = canon_as(k, StageKind::Reduce);
        if (c.ok && c.rows == g.rows && c.C == g.C) pick = c;
      } else {
        Canon w = canon_as(k, StageKind::Wide);
        if (w.ok && w.rows == g.rows && w.C == g.C) pick = w;
        else {
          Canon s = canon_as(k, StageKind::Scalar);
          if (s.ok && s.rows == g.rows && g.has_reduce()) pick = s;
        }
      }
      // a buffer may be written once per group
      if (pick.ok && (!aligned_with_group(g, pick.stage) || g.producer(pick.stage.out_buf))) pick.ok = false;
      return pick;
    };
    while (opt.fuse && i < kernels.size() && nests[i] && !folded_kernels.count(i)) {
      if (absorbed.count(i)) {
        ++i;
        continue;
      }
      Canon pick = stage_for(*nests[i]);
      if (!pick.ok) break;
      g.stages.push_back(pick.stage);
      ++i;
    }
    // Kernels further down that carry on with this group's rows on a few thousand elements (the
    // bookkeeping of a loss, lowered behind the kernels of another root) join it when nothing in
    // between has a hand in what they read or write: one launch less on the way, and no large
    // value has to be kept for them.
    if (opt.fuse && opt.reindex && opt.merge_launches && have_table && g.has_reduce()) {
      auto tiny = [&](const Node* k) {
        for (const auto& p : k->params) {
          if (!p.dtype.is_ptr()) continue;
          auto e = elems.find(p.name);
          if (e == elems.end() || e->second > (size_t{1} << 12)) return false;
        }
        return true;
      };
      for (size_t j = i; j < kernels.size() && j < i + 200; ++j) {
        if (absorbed.count(j) || folded_kernels.count(j) || windows.count(j) || scattered.count(j) || absorbed_name.count(j)) continue;
        if (!nests[j] || !tiny(kernels[j])) continue;
        bool feeds = false;
        for (const auto& p : kernels[j]->params)
          feeds = feeds || (p.dtype.is_ptr() && !p.mut_ && g.producer(p.name));
        if (!feeds) continue;
        bool free_to_move = true;
        for (size_t m = i; m < j && free_to_move; ++m) {
          if (absorbed.count(m)) continue;              // (already part of an earlier launch, this group's included)
          for (const auto& pm : kernels[m]->params)
            for (const auto& pj : kernels[j]->params)
              if (pm.dtype.is_ptr() && pj.dtype.is_ptr() && pm.name == pj.name && (pm.mut_ || pj.mut_)) free_to_move = false;
        }
        if (!free_to_move) continue;
        Canon pick = stage_for(*nests[j]);
        if (!pick.ok) continue;
        g.stages.push_back(pick.stage);
        absorbed.insert(j);
      }
    }
    // which stage outputs must reach memory
    for (size_t s = 0; s < g.stages.size(); ++s) {
      Stage& st = g.stages[s];
      bool needed = role_of(st.out_buf) != "temp";
      for (size_t r : readers[st.out_buf])
        if (r < first || r >= i) needed = true;
      st.store = needed;
      if (!needed) plan.elided.insert(st.out_buf);
    }
    plan.launches.push_back(emit_group(g, opt, elems));
  }
  // what was held back goes to the end one by one: the pass that issues independent launches together
  // (below) merges it with whatever else is still waiting there, by workgroup size (a part's surplus
  // work-items leave at once, but they are launched all the same)
  for (auto& ls : held_back) plan.launches.push_back(std::move(ls));
  // constant inputs no launch binds any more need not exist
  for (const auto& c : consts) {
    bool bound = false;
    for (const auto& ls : plan.launches)
      for (const auto& a : ls.arg_bufs) bound = bound || a == c.first;
    if (!bound) plan.elided.insert(c.first);
  }
  // a launch that covers a kernel which took another one in covers that one too
  // (before launches are merged: the covered kernels decide which buffers a launch writes)
  for (auto& ls : plan.launches) {
    const std::vector<std::string> covered = ls.kernels;
    for (const auto& kn : covered)
      for (const auto& an : absorbed_name)
        if (nests[an.first] && nests[an.first]->name == kn &&
            std::find(ls.kernels.begin(), ls.kernels.end(), an.second) == ls.kernels.end())
          ls.kernels.push_back(an.second);
  }
  issue_independent_launches_together(&plan, kernels, opt);
  // A lowered kernel whose output index is the dense index of its loops writes every element of
  // its output; the launch that stores it overwrites a buffer of exactly that size, whatever it
  // held (the executor need not have zero-filled it first).
  {
    std::map<std::string, std::pair<std::string, size_t>> dense_out;     // kernel -> (buffer, bytes)
    for (const auto& nk : nests) {
      int64_t numel = 0;
      if (nk && !partly_written.count(nk->name) && dense_strides(*nk, &numel))
        dense_out[nk->name] = {nk->out_buf, static_cast<size_t>(numel) * nk->out_dtype.itemsize()};
    }
    for (auto& ls : plan.launches) {
      ls.arg_full_bytes.assign(ls.arg_bufs.size(), 0);
      for (const auto& kn : ls.kernels) {
        auto it = dense_out.find(kn);
        if (it == dense_out.end()) continue;
        for (size_t a = 0; a < ls.arg_bufs.size(); ++a)
          if (ls.arg_bufs[a] == it->second.first) ls.arg_full_bytes[a] = it->second.second;
      }
    }
  }
  assign_lanes(&plan, kernels, opt);
  return plan;
}

// ---------------------------------------------------------------------------------------------
// emitters
// ---------------------------------------------------------------------------------------------

namespace {

const char* op_struct(ReduceKind k) {
  switch (k) {
    case ReduceKind::Sum: return "EhSum";
    case ReduceKind::Max: return "EhMax";
    case ReduceKind::Min: return "EhMin";
    case ReduceKind::Prod: return "EhProd";
    default: return "?";
  }
}

std::string combine_text(ReduceKind k, const DType& t, const std::string& acc, const std::string& v) {
  switch (k) {
    case ReduceKind::Sum: return "(" + acc + " + " + v + ")";
    case ReduceKind::Prod: return "(" + acc + " * " + v + ")";
    case ReduceKind::Max:
      if (t.ty == Ty::F32) return "fmaxf(" + acc + ", " + v + ")";
      if (t.ty == Ty::F64) return "fmax(" + acc + ", " + v + ")";
      return "(" + acc + " > " + v + " ? " + acc + " : " + v + ")";
    case ReduceKind::Min: return "(" + acc + " < " + v + " ? " + acc + " : " + v + ")";
    default: return acc;
  }
}

bool pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
int64_t pow2_ceil(int64_t v) {
  int64_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

// One distinct external access: buffer + affine index over canonical vars.
struct ExtLoad {
  std::string buf;
  Affine aff;
  DType dtype;
  int id = 0;
  bool cached = false;   // held in registers for the whole row
};

// Index arithmetic is done in 32-bit `int` while every index, every loop counter and the
// grid-stride increments added to them (a grid's worth of work-items times the vector width)
// stay well below 2^31; from 2^30 reachable elements on, kernels use 64-bit indices.
constexpr int64_t kIndex32Limit = int64_t{1} << 30;

struct GroupEmitter {
  const Group& g;
  const GenOptions& opt;
  std::vector<ExtLoad> ext;          // distinct affine external loads eligible for caching/vectorising
  std::vector<std::string> in_bufs;  // external buffers read, parameter order
  std::map<std::string, DType> in_dtype;
  bool idx64 = false;
  int V = 1;
  std::map<std::string, int64_t> need;   // elements each bound buffer must hold (max index + 1)
  // lets a schedule serve some external loads from somewhere else (an LDS tile)
  std::function<bool(const std::string& buf, const Affine& index, std::string* text)> load_override;
  // fp32 inputs whose guarded loads go through a buffer resource (name -> bytes); see ExprRenderer::ranged
  std::map<std::string, size_t> ranged;

  GroupEmitter(const Group& grp, const GenOptions& o) : g(grp), opt(o) {}

  std::string sname(const std::string& buf) const { return "s_" + buf; }

  int find_ext(const std::string& buf, const Affine& a) const {
    for (const auto& e : ext)
      if (e.buf == buf && e.aff == a) return e.id;
    return -1;
  }

  // Collect external loads (recursing through nothing: stage values only reference buffers).
  void scan() {
    int64_t reach = 0;
    std::vector<Loop> loops;
    for (size_t i = 0; i < g.rows.size(); ++i) loops.push_back({"r" + std::to_string(i), g.rows[i]});
    Loop cl{"c", g.C};
    for (const auto& st : g.stages) {
      std::vector<LoadRef> loads;
      collect_loads(*st.value, loads);
      for (const auto& lr : loads) {
        const std::string& b = lr.load->args[0]->name;
        if (g.producer(b) && g.producer(b) != &st) {
          // only earlier stages can be producers; a later stage writing a buffer read here is external
          bool earlier = false;
          for (const auto& p : g.stages) {
            if (&p == &st) break;
            if (p.out_buf == b) earlier = true;
          }
          if (earlier) continue;
        }
        if (std::find(in_bufs.begin(), in_bufs.end(), b) == in_bufs.end()) {
          in_bufs.push_back(b);
          in_dtype[b] = lr.load->dtype;
        }
        auto a = affine_of(*lr.load->args[1]);
        if (!a) { idx64 = true; continue; }     // opaque index: stay in 64-bit to be safe
        const int64_t top = max_abs_index(*a, loads_loops(loops), &cl);
        reach = std::max(reach, top);
        // a load under a Select only happens where its bounds condition holds
        if (!lr.guarded) need[b] = std::max(need[b], top + 1);
        if (!lr.guarded && a->of("c") == 1 && find_ext(b, *a) < 0) {
          ExtLoad e;
          e.buf = b;
          e.aff = *a;
          e.dtype = lr.load->dtype;
          e.id = static_cast<int>(ext.size());
          ext.push_back(e);
        }
      }
      if (st.store) {
        const int64_t top = max_abs_index(st.out_aff, loops, &cl);
        reach = std::max(reach, top);
        need[st.out_buf] = std::max(need[st.out_buf], top + 1);
      }
    }
    if (reach >= kIndex32Limit || g.R() * g.C >= kIndex32Limit) idx64 = true;
  }
  static const std::vector<Loop>& loads_loops(const std::vector<Loop>& l) { return l; }

  // every vectorised access of `width` elements starts on a multiple of the width
  bool aligned(const Affine& a, int width) const {
    if (a.c % width) return false;
    for (const auto& kv : a.coef)
      if (kv.first != "c" && kv.second % width) return false;
    return true;
  }
  bool vector_ok(int width) const {
    if (!opt.vectorize || g.C % width) return false;
    for (const auto& e : ext)
      if (!aligned(e.aff, width) || e.dtype.itemsize() != 4) return false;
    for (const auto& st : g.stages)
      if (st.kind == StageKind::Wide && st.store &&
          (st.out_aff.of("c") != 1 || !aligned(st.out_aff, width) || st.out_dtype.itemsize() != 4))
        return false;
    return true;
  }

  void choose_vector() { V = vector_ok(4) ? 4 : 1; }
  // the flat schedule also takes pairs (a pooling window two wide: 64-bit accesses, one index
  // decode and one read of everything that does not move along the pair per two elements)
  void choose_vector_flat() {
    if (V == 1 && vector_ok(2)) V = 2;
  }

  std::string affine_text(const Affine& a, const std::string& cvar) const {
    std::string s;
    auto term = [&](const std::string& t) { s += s.empty() ? t : " + " + t; };
    for (const auto& kv : a.coef) {
      std::string v = kv.first == "c" ? cvar : kv.first;
      if (kv.second == 1) term(v);
      else term(v + " * " + std::to_string(kv.second) + (idx64 ? "ll" : ""));
    }
    if (a.c != 0 || s.empty()) term(std::to_string(a.c));
    return "(" + s + ")";
  }

  // Value of a stage for the element whose column variable is `c` (declared in scope).
  // `ld` maps a cached/vectorised external load id to the text that yields its value.
  std::string value_text(const Stage& st, const std::function<std::string(int)>& ld) const {
    ExprRenderer er;
    if (!ranged.empty()) er.ranged = &ranged;
    er.load_hook = [&](const Node& load, std::string* out) {
      const std::string& b = load.args[0]->name;
      const Stage* p = nullptr;
      for (const auto& q : g.stages) {
        if (&q == &st) break;
        if (q.out_buf == b) p = &q;
      }
      if (p) {
        if (p->kind == StageKind::Wide) {
          *out = "((" + ctype(p->out_dtype) + ")(" + value_text(*p, ld) + "))";
        } else {
          *out = sname(b);
        }
        return true;
      }
      auto a = affine_of(*load.args[1]);
      if (a) {
        if (load_override && load_override(b, *a, out)) return true;
        int id = find_ext(b, *a);
        if (id >= 0) {
          std::string t = ld(id);
          if (!t.empty()) { *out = t; return true; }
        }
        *out = b + "[" + affine_text(*a, "c") + "]";
        return true;
      }
      return false;   // opaque index: rendered from the tree with canonical variable names
    };
    return er.expr(*st.value);
  }

  std::string params_text(std::vector<std::string>* order) const {
    std::string s;
    for (const auto& b : in_bufs) {
      bool also_out = false;
      for (const auto& st : g.stages) also_out = also_out || (st.store && st.out_buf == b);
      if (also_out) throw Error("buffer '" + b + "' is both read as an input and written in one fused launch");
      s += (s.empty() ? "" : ", ") + std::string("const ") + ctype(in_dtype.at(b)) + "* __restrict__ " + b;
      order->push_back(b);
    }
    for (const auto& st : g.stages)
      if (st.store) {
        s += (s.empty() ? "" : ", ") + ctype(st.out_dtype) + "* __restrict__ " + st.out_buf;
        order->push_back(st.out_buf);
      }
    return s;
  }

  std::string row_decode(const std::string& rowvar) const {
    // row -> r0..rn-1 (row-major over the row loops)
    std::string s;
    if (g.rows.empty()) return s;
    if (g.rows.size() == 1) return "  const idx_t r0 = " + rowvar + ";\n";
    // (never negative: lets the compiler take the cheaper unsigned forms of the divisions)
    s += "  idx_t eh_rem = " + rowvar + ";\n  __builtin_assume(eh_rem >= 0);\n";
    for (size_t i = g.rows.size(); i-- > 0;) {
      if (i == 0) s += "  const idx_t r0 = eh_rem;\n";
      else {
        s += "  const idx_t r" + std::to_string(i) + " = eh_rem % " + std::to_string(g.rows[i]) + ";\n";
        s += "  eh_rem /= " + std::to_string(g.rows[i]) + ";\n";
      }
    }
    return s;
  }

  // Streaming (non-temporal) hints.  By default only stores of outputs too large to be
  // re-read from cache by a following kernel are streamed.
  bool nt_stores() const {
    if (opt.nontemporal >= 0) return opt.nontemporal >= 1;
    int64_t bytes = 0;
    for (const auto& st : g.stages)
      if (st.store && st.kind == StageKind::Wide) bytes += g.R() * g.C * static_cast<int64_t>(st.out_dtype.itemsize());
    return bytes >= (int64_t{32} << 20);
  }
  bool nt_loads() const { return opt.nontemporal >= 2; }

  void fill_min_bytes(LaunchSpec* ls) const {
    for (const auto& b : ls->arg_bufs) {
      size_t item = 4;
      auto it = in_dtype.find(b);
      if (it != in_dtype.end()) item = it->second.itemsize();
      for (const auto& st : g.stages)
        if (st.store && st.out_buf == b) item = st.out_dtype.itemsize();
      auto n = need.find(b);
      ls->arg_min_bytes.push_back(n == need.end() ? 0 : static_cast<size_t>(n->second) * item);
    }
  }

  double algo_bytes(const std::map<std::string, size_t>& elems) const {
    double b = 0;
    for (const auto& n : in_bufs) {
      auto it = elems.find(n);
      double cnt = it != elems.end() ? static_cast<double>(it->second) : static_cast<double>(g.R() * g.C);
      b += cnt * static_cast<double>(in_dtype.at(n).itemsize());
    }
    for (const auto& st : g.stages)
      if (st.store)
        b += static_cast<double>(st.kind == StageKind::Wide ? g.R() * g.C : g.R()) *
             static_cast<double>(st.out_dtype.itemsize());
    return b;
  }

  // ---- flat: no reductions; a grid-stride loop over 4-element vectors --------------------
  LaunchSpec emit_flat(const std::map<std::string, size_t>& elems) {
    LaunchSpec ls;
    const int64_t N = g.R() * g.C;
    const int64_t NVEC = N / V;
    const int block = opt.flat_block;
    int64_t want = (NVEC + static_cast<int64_t>(block) * opt.flat_iters - 1) / (static_cast<int64_t>(block) * opt.flat_iters);
    int64_t blocks = std::max<int64_t>(1, std::min<int64_t>(want, 1 << 20));
    const char* nt = nt_loads() ? "true" : "false";
    const char* nts = nt_stores() ? "true" : "false";
    ls.entry = "ehk_" + g.stages.front().kname;
    ls.schedule = "flat(V=" + std::to_string(V) + ",block=" + std::to_string(block) + (nt_stores() ? ",nt-store" : "") +
                  (nt_loads() ? ",nt-load" : "") + ")";
    ls.grid[0] = static_cast<unsigned>(blocks);
    ls.block[0] = static_cast<unsigned>(block);
    std::ostringstream os;
    os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
    if (V == 2)
      os << "template <typename T> using EhV2 = T __attribute__((ext_vector_type(2)));\n"
            "template <bool NT, typename T> __device__ __forceinline__ EhV2<T> eh_load2(const T* p) {\n"
            "  if (NT) return __builtin_nontemporal_load(reinterpret_cast<const EhV2<T>*>(p));\n"
            "  return *reinterpret_cast<const EhV2<T>*>(p);\n}\n"
            "template <bool NT, typename T> __device__ __forceinline__ void eh_store2(T* p, EhV2<T> v) {\n"
            "  if (NT) __builtin_nontemporal_store(v, reinterpret_cast<EhV2<T>*>(p));\n"
            "  else *reinterpret_cast<EhV2<T>*>(p) = v;\n}\n";
    // guarded reads of an input whose size the buffer table fixes: one load each, out of range
    // (and so zero) where the guard fails
    bool any_guarded = false;
    for_each_external_load([&](const LoadRef& lr) { any_guarded = any_guarded || lr.guarded; });
    if (any_guarded && g_ranged_loads && !g_guard_branches && !idx64)
      for (const auto& b : in_bufs) {
        auto it = elems.find(b);
        if (it != elems.end() && in_dtype.at(b).ty == Ty::F32 && it->second * 4 < (size_t{1} << 31)) ranged[b] = it->second * 4;
      }
    if (!ranged.empty())
      os << "__device__ __forceinline__ float eh_ranged_load(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {\n"
            "  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, 0));\n}\n";
    os << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << ls.entry << "("
       << params_text(&ls.arg_bufs) << ") {\n";
    for (const auto& rb : ranged)
      os << "  const __amdgpu_buffer_rsrc_t eh_rs_" << rb.first << " = __builtin_amdgcn_make_buffer_rsrc((void*)" << rb.first
         << ", 0, " << rb.second << ", 0x00020000);\n";
    os << "  const idx_t eh_nvec = " << NVEC << ";\n";
    os << "  const idx_t eh_stride = (idx_t)gridDim.x * " << block << ";\n";
    os << "  for (idx_t eh_g = (idx_t)blockIdx.x * " << block << " + threadIdx.x; eh_g < eh_nvec; eh_g += eh_stride) {\n";
    os << "  const idx_t eh_p = eh_g * " << V << ";\n";
    if (!g.rows.empty()) {
      os << "  __builtin_assume(eh_p >= 0);\n  const idx_t eh_row = eh_p / " << g.C << ";\n  const idx_t c0 = eh_p % " << g.C << ";\n";
      os << row_decode("eh_row");
    } else {
      os << "  const idx_t c0 = eh_p;\n";
    }
    // vector loads
    auto ld = [&](int id) -> std::string {
      return V > 1 ? "ld" + std::to_string(id) + "[v]" : std::string();
    };
    if (V == 4)
      for (const auto& e : ext)
        os << "  const EhV4<" << ctype(e.dtype) << "> ld" << e.id << " = eh_load4<" << nt << ">(" << e.buf << " + "
           << affine_text(e.aff, "c0") << ");\n";
    if (V == 2)
      for (const auto& e : ext)
        os << "  const EhV2<" << ctype(e.dtype) << "> ld" << e.id << " = eh_load2<" << nt << ">(" << e.buf << " + "
           << affine_text(e.aff, "c0") << ");\n";
    for (const auto& st : g.stages) {
      if (!st.store) continue;
      std::string T = ctype(st.out_dtype);
      if (V > 1) {
        os << "  { EhV" << V << "<" << T << "> eh_o;\n#pragma unroll\n  for (int v = 0; v < " << V << "; ++v) { const idx_t c = c0 + v; eh_o[v] = ("
           << T << ")(" << value_text(st, ld) << "); }\n";
        os << "  eh_store" << V << "<" << nts << ">(" << st.out_buf << " + " << affine_text(st.out_aff, "c0") << ", eh_o); }\n";
      } else {
        os << "  { const idx_t c = c0; " << st.out_buf << "[" << affine_text(st.out_aff, "c") << "] = (" << T << ")("
           << value_text(st, ld) << "); }\n";
      }
    }
    os << "  }\n}\n";
    ls.source = os.str();
    ls.algo_bytes = algo_bytes(elems);
    fill_min_bytes(&ls);
    for (const auto& st : g.stages) ls.kernels.push_back(st.kname);
    return ls;
  }

  // ---- transposing copies: a 64 x 64 tile through LDS ---------------------------------------
  // Elementwise groups in which some operand is contiguous along a row loop while the output is
  // contiguous along the column loop (permute + contiguous, NCHW <-> NHWC, x^T + y).  Read
  // as written, such an operand is fetched with a stride between neighbouring work-items.
  struct TransposedLoad { std::string buf; Affine aff; DType dtype; };

  // every external load of the group, with whether a Select guards it
  template <class F> void for_each_external_load(F&& f) const {
    for (const auto& st : g.stages) {
      std::vector<LoadRef> loads;
      collect_loads(*st.value, loads);
      for (const auto& lr : loads) {
        const std::string& b = lr.load->args[0]->name;
        bool earlier = false;
        for (const auto& p : g.stages) {
          if (&p == &st) break;
          if (p.out_buf == b) earlier = true;
        }
        if (!earlier) f(lr);
      }
    }
  }

  // Which loops the tile spans.  `row_run`: adjacent row loops (outermost first) that every
  // strided operand walks as one contiguous axis; `col_run`: row loops that, followed by the
  // column loop, every store walks as one contiguous axis.  Empty row_run: not this form.
  struct TransposePlan {
    std::vector<size_t> row_run, col_run;
    int64_t Rt = 1, Ct = 1;
  };

  TransposePlan transposed_axes(std::vector<TransposedLoad>* tl) const {
    TransposePlan none;
    if (g.has_reduce() || g.rows.empty() || g.R() * g.C < (1 << 16)) return none;
    for (const auto& st : g.stages)
      if (st.store && st.out_aff.of("c") != 1) return none;
    auto rv = [](size_t i) { return "r" + std::to_string(i); };
    int inner = -1;
    bool ok = true;
    for_each_external_load([&](const LoadRef& lr) {
      auto a = affine_of(*lr.load->args[1]);
      if (!a || lr.load->count != 1) { ok = false; return; }
      if (a->of("c") == 1 || a->of("c") == 0) return;       // aligned with the output, or a broadcast
      if (lr.guarded || std::llabs(a->of("c")) < 8) { ok = false; return; }
      int t = -1;
      for (size_t i = 0; i < g.rows.size(); ++i)
        if (a->of(rv(i)) == 1) t = static_cast<int>(i);
      if (t < 0 || (inner >= 0 && inner != t)) { ok = false; return; }
      inner = t;
      for (const auto& e : *tl)
        if (e.buf == lr.load->args[0]->name && e.aff == *a) return;
      tl->push_back({lr.load->args[0]->name, *a, lr.load->dtype});
    });
    if (!ok || inner < 0 || tl->empty() || tl->size() > 4) return none;
    TransposePlan tp;
    // the column side: c, then the innermost row loops while every store keeps walking on
    tp.Ct = g.C;
    for (size_t i = g.rows.size(); i-- > 0;) {
      if (static_cast<int>(i) == inner) break;
      bool chains = true;
      for (const auto& st : g.stages)
        if (st.store) chains = chains && st.out_aff.of(rv(i)) == tp.Ct;
      if (!chains) break;
      tp.col_run.insert(tp.col_run.begin(), i);
      tp.Ct *= g.rows[i];
    }
    // the row side: the operands' unit-stride loop, then the loops outside it while every
    // strided operand keeps walking on
    tp.row_run = {static_cast<size_t>(inner)};
    tp.Rt = g.rows[static_cast<size_t>(inner)];
    for (size_t i = static_cast<size_t>(inner); i-- > 0;) {
      bool chains = true;
      for (const auto& e : *tl) chains = chains && e.aff.of(rv(i)) == tp.Rt;
      if (!chains) break;
      tp.row_run.insert(tp.row_run.begin(), i);
      tp.Rt *= g.rows[i];
    }
    if (tp.Rt < 32 || tp.Ct < 32) return none;
    return tp;
  }

  LaunchSpec emit_transposed(const std::map<std::string, size_t>& elems, const TransposePlan& tp,
                             const std::vector<TransposedLoad>& tl) {
    LaunchSpec ls;
    const int64_t nrt = (tp.Rt + 63) / 64, nct = (tp.Ct + 63) / 64;
    std::vector<bool> in_tile(g.rows.size(), false);
    for (size_t i : tp.row_run) in_tile[i] = true;
    for (size_t i : tp.col_run) in_tile[i] = true;
    int64_t others = 1;
    for (size_t i = 0; i < g.rows.size(); ++i)
      if (!in_tile[i]) others *= g.rows[i];
    const int64_t blocks = nrt * nct * others;
    if (blocks >= (int64_t{1} << 31)) throw Error("too many tiles for one launch");
    ls.entry = "ehk_" + g.stages.front().kname;
    ls.schedule = "transpose(tile=64x64,rows=" + std::to_string(tp.Rt) + ",cols=" + std::to_string(tp.Ct) +
                  ",operands=" + std::to_string(tl.size()) + ")";
    ls.grid[0] = static_cast<unsigned>(blocks);
    ls.block[0] = 256;
    std::ostringstream os;
    os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
    os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "(" << params_text(&ls.arg_bufs) << ") {\n";
    for (size_t k = 0; k < tl.size(); ++k)
      os << "  __shared__ " << ctype(tl[k].dtype) << " eh_tile" << k << "[64][65];\n";
    os << "  const int eh_tx = threadIdx.x & 63, eh_ty = threadIdx.x >> 6;\n";
    os << "  idx_t eh_b = blockIdx.x;\n";
    os << "  const idx_t eh_c0 = (eh_b % " << nct << ") * 64;\n  eh_b /= " << nct << ";\n";
    os << "  const idx_t eh_r0 = (eh_b % " << nrt << ") * 64;\n  eh_b /= " << nrt << ";\n";
    for (size_t i = g.rows.size(); i-- > 0;) {
      if (in_tile[i]) continue;
      os << "  const idx_t r" << i << " = eh_b % " << g.rows[i] << ";\n  eh_b /= " << g.rows[i] << ";\n";
    }
    // position along the merged row axis -> its loops; along the merged column axis -> its loops and c
    auto decode_rows = [&](const std::string& m, const std::string& ind) {
      std::string t = ind + "idx_t eh_q = " + m + ";\n";
      for (size_t q = tp.row_run.size(); q-- > 0;) {
        const size_t i = tp.row_run[q];
        if (q == 0) t += ind + "const idx_t r" + std::to_string(i) + " = eh_q;\n";
        else {
          t += ind + "const idx_t r" + std::to_string(i) + " = eh_q % " + std::to_string(g.rows[i]) + ";\n";
          t += ind + "eh_q /= " + std::to_string(g.rows[i]) + ";\n";
        }
      }
      return t;
    };
    auto decode_cols = [&](const std::string& m, const std::string& ind) {
      std::string t = ind + "idx_t eh_p = " + m + ";\n";
      if (tp.col_run.empty()) return t + ind + "const idx_t c = eh_p;\n";
      t += ind + "const idx_t c = eh_p % " + std::to_string(g.C) + ";\n" + ind + "eh_p /= " + std::to_string(g.C) + ";\n";
      for (size_t q = tp.col_run.size(); q-- > 0;) {
        const size_t i = tp.col_run[q];
        if (q == 0) t += ind + "const idx_t r" + std::to_string(i) + " = eh_p;\n";
        else {
          t += ind + "const idx_t r" + std::to_string(i) + " = eh_p % " + std::to_string(g.rows[i]) + ";\n";
          t += ind + "eh_p /= " + std::to_string(g.rows[i]) + ";\n";
        }
      }
      return t;
    };
    // phase 1: neighbouring work-items walk the operands' contiguous axis
    os << "  if (eh_r0 + eh_tx < " << tp.Rt << ") {\n" << decode_rows("eh_r0 + eh_tx", "    ");
    os << "#pragma unroll 4\n    for (int eh_cc = eh_ty; eh_cc < 64; eh_cc += 4) {\n";
    os << "      if (eh_c0 + eh_cc < " << tp.Ct << ") {\n" << decode_cols("eh_c0 + eh_cc", "        ");
    for (size_t k = 0; k < tl.size(); ++k)
      os << "        eh_tile" << k << "[eh_cc][eh_tx] = " << tl[k].buf << "[" << affine_text(tl[k].aff, "c") << "];\n";
    os << "      }\n    }\n  }\n  __syncthreads();\n";
    // phase 2: neighbouring work-items walk the output's contiguous axis
    load_override = [&](const std::string& buf, const Affine& a, std::string* text) {
      for (size_t k = 0; k < tl.size(); ++k)
        if (tl[k].buf == buf && tl[k].aff == a) {
          *text = "eh_tile" + std::to_string(k) + "[eh_tx][eh_rr]";
          return true;
        }
      return false;
    };
    auto none = [](int) { return std::string(); };
    os << "  if (eh_c0 + eh_tx < " << tp.Ct << ") {\n" << decode_cols("eh_c0 + eh_tx", "    ");
    os << "#pragma unroll 4\n    for (int eh_rr = eh_ty; eh_rr < 64; eh_rr += 4) {\n";
    os << "      if (eh_r0 + eh_rr < " << tp.Rt << ") {\n" << decode_rows("eh_r0 + eh_rr", "        ");
    for (const auto& st : g.stages) {
      if (!st.store) continue;
      os << "        " << st.out_buf << "[" << affine_text(st.out_aff, "c") << "] = (" << ctype(st.out_dtype) << ")("
         << value_text(st, none) << ");\n";
    }
    os << "      }\n    }\n  }\n}\n";
    load_override = nullptr;
    ls.source = os.str();
    ls.algo_bytes = algo_bytes(elems);
    fill_min_bytes(&ls);
    for (const auto& st : g.stages) ls.kernels.push_back(st.kname);
    return ls;
  }

  // ---- row program: T threads per row, DPP/LDS reductions ---------------------------------
  LaunchSpec emit_rows(const std::map<std::string, size_t>& elems) {
    LaunchSpec ls;
    const int64_t R = g.R(), C = g.C;
    int64_t T = opt.row_threads > 0 ? opt.row_threads : pow2_ceil((C + opt.row_elems - 1) / opt.row_elems);
    T = std::max<int64_t>(1, std::min<int64_t>(T, 1024));
    if (!pow2(T)) T = pow2_ceil(T);
    // two waves per row would pay for an LDS exchange and a barrier; one wave with twice the
    // elements per lane is faster for rows this short
    if (opt.row_threads == 0 && T == 128) T = 64;
    while (T * V > pow2_ceil(C) && T > 1) T >>= 1;          // no more threads than vectors in a row
    const int64_t per_iter = T * V;
    const int64_t NV = (C + per_iter - 1) / per_iter;
    const bool reg = NV * V <= 64;                           // whole row of a thread fits registers
    const bool tail = (C % per_iter) != 0;
    const int64_t block = T >= 256 ? T : 256;
    const int64_t RPB = block / T;
    const int64_t blocks = (R + RPB - 1) / RPB;
    if (blocks >= (int64_t{1} << 31)) throw Error("too many rows for one launch");
    int nred = 0;
    for (const auto& st : g.stages) nred += st.kind == StageKind::Reduce;
    const char* nt = nt_loads() ? "true" : "false";
    const char* nts = nt_stores() ? "true" : "false";
    ls.entry = "ehk_" + g.stages.front().kname;
    ls.schedule = "row(T=" + std::to_string(T) + ",V=" + std::to_string(V) + ",NV=" + std::to_string(NV) +
                  (reg ? ",reg" : ",stream") + ",rows/block=" + std::to_string(RPB) + (nt_stores() ? ",nt-store" : "") +
                  (nt_loads() ? ",nt-load" : "") + ")";
    ls.grid[0] = static_cast<unsigned>(blocks);
    ls.block[0] = static_cast<unsigned>(block);
    for (auto& e : ext) e.cached = reg;

    std::ostringstream os;
    os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
    os << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << ls.entry << "("
       << params_text(&ls.arg_bufs) << ") {\n";
    os << "  constexpr int T = " << T << ", V = " << V << ", NV = " << NV << ";\n";
    os << "  constexpr idx_t C = " << C << ", R = " << R << ";\n";
    os << "  const int lr = threadIdx.x % T;\n";
    os << "  idx_t eh_row = (idx_t)blockIdx.x * " << RPB << " + threadIdx.x / T;\n";
    os << "  const bool eh_row_ok = eh_row < R;\n  if (!eh_row_ok) eh_row = R - 1;\n";
    os << row_decode("eh_row");
    if (T > 64 && nred > 0) {
      // LDS slots typed per reduction
      int r = 0;
      for (const auto& st : g.stages)
        if (st.kind == StageKind::Reduce)
          os << "  __shared__ " << ctype(st.acc_dtype) << " eh_red" << r++ << "[" << RPB * (T / 64) << "];\n";
    }
    const std::string iter_open = std::string(reg ? "#pragma unroll\n" : "") +
                                  "  for (int k = 0; k < NV; ++k) {\n    const idx_t c0 = (idx_t)(k * T + lr) * V;\n";
    const std::string guard_open = tail ? "    if (c0 < C) {\n" : "    {\n";
    // preload the row slices every stage shares
    if (reg) {
      for (const auto& e : ext) os << "  " << ctype(e.dtype) << " xc" << e.id << "[NV * V];\n";
      if (!ext.empty()) {
        os << iter_open << guard_open;
        for (const auto& e : ext) {
          if (V == 4) {
            os << "      const EhV4<" << ctype(e.dtype) << "> t" << e.id << " = eh_load4<" << nt << ">(" << e.buf << " + "
               << affine_text(e.aff, "c0") << ");\n";
            os << "#pragma unroll\n      for (int v = 0; v < 4; ++v) xc" << e.id << "[k * 4 + v] = t" << e.id << "[v];\n";
          } else {
            os << "      xc" << e.id << "[k] = " << e.buf << "[" << affine_text(e.aff, "c0") << "];\n";
          }
        }
        os << "    }\n  }\n";
      }
    }
    auto ld = [&](int id) -> std::string {
      if (reg) return "xc" + std::to_string(id) + "[k * V + v]";
      return std::string();
    };
    int red_i = 0;
    for (const auto& st : g.stages) {
      const std::string T_out = ctype(st.out_dtype);
      os << "  // " << st.kname << "\n";
      if (st.kind == StageKind::Reduce) {
        const std::string TA = ctype(st.acc_dtype);
        const std::string acc = "acc" + std::to_string(red_i);
        os << "  " << TA << " " << acc << " = " << literal(*st.identity) << ";\n";
        os << iter_open << guard_open;
        os << "#pragma unroll\n      for (int v = 0; v < V; ++v) { const idx_t c = c0 + v; " << acc << " = "
           << combine_text(st.rk, st.acc_dtype, acc, "(" + TA + ")(" + value_text(st, ld) + ")") << "; }\n";
        os << "    }\n  }\n";
        os << "  const " << TA << " " << sname(st.out_buf) << " = eh_row_reduce<" << op_struct(st.rk) << ", T>(" << acc
           << ", "
           << (T > 64 ? "eh_red" + std::to_string(red_i) + " + (threadIdx.x / T) * (T / 64)" : std::string("(" + TA + "*)nullptr"))
           << ", lr);\n";
        if (st.store)
          os << "  if (lr == 0 && eh_row_ok) " << st.out_buf << "[" << affine_text(st.out_aff, "0") << "] = ("
             << T_out << ")" << sname(st.out_buf) << ";\n";
        ++red_i;
      } else if (st.kind == StageKind::Scalar) {
        // per-row value; loads of wide operands cannot occur here
        auto none = [](int) { return std::string(); };
        os << "  const " << T_out << " " << sname(st.out_buf) << " = (" << T_out << ")(" << value_text(st, none) << ");\n";
        if (st.store)
          os << "  if (lr == 0 && eh_row_ok) " << st.out_buf << "[" << affine_text(st.out_aff, "0") << "] = "
             << sname(st.out_buf) << ";\n";
      } else if (st.store) {
        os << iter_open << guard_open;
        if (V == 4) {
          os << "      EhV4<" << T_out << "> eh_o;\n#pragma unroll\n      for (int v = 0; v < 4; ++v) { const idx_t c = c0 + v; eh_o[v] = ("
             << T_out << ")(" << value_text(st, ld) << "); }\n";
          os << "      if (eh_row_ok) eh_store4<" << nts << ">(" << st.out_buf << " + " << affine_text(st.out_aff, "c0")
             << ", eh_o);\n";
        } else {
          os << "      const int v = 0; const idx_t c = c0; const " << T_out << " eh_o = (" << T_out << ")(" << value_text(st, ld)
             << ");\n      if (eh_row_ok) " << st.out_buf << "[" << affine_text(st.out_aff, "c") << "] = eh_o;\n";
        }
        os << "    }\n  }\n";
      }
    }
    os << "}\n";
    ls.source = os.str();
    ls.algo_bytes = algo_bytes(elems);
    fill_min_bytes(&ls);
    for (const auto& st : g.stages) ls.kernels.push_back(st.kname);
    return ls;
  }
};

LaunchSpec emit_group(const Group& g, const GenOptions& opt, const std::map<std::string, size_t>& elems) {
  GroupEmitter ge(g, opt);
  ge.scan();
  ge.choose_vector();
  bool any_store = false;
  for (const auto& st : g.stages) any_store = any_store || st.store;
  if (!any_store) throw Error("fused group starting at '" + g.stages.front().kname + "' produces nothing");
  if (!g.has_reduce()) {
    std::vector<GroupEmitter::TransposedLoad> tl;
    GroupEmitter::TransposePlan tp;
    if (opt.transpose) tp = ge.transposed_axes(&tl);
    if (!tp.row_run.empty()) return ge.emit_transposed(elems, tp, tl);
    ge.choose_vector_flat();
    return ge.emit_flat(elems);
  }
  return ge.emit_rows(elems);
}

// Reductions over a non-contiguous axis that are not contractions.  One thread per output
// element, adjacent threads on adjacent outputs (so loads along the fastest output axis
// coalesce), the reduce loop serial inside the thread.  When there are few outputs and a long
// reduce axis the axis is split over gridDim.y: each workgroup (64 outputs x 4 row phases)
// reduces one chunk into a scratch buffer [chunks][outputs] and a second launch combines the
// chunks -- deterministic, no atomics.
struct SerialReduce {
  const NestKernel& k;
  const GenOptions& opt;
  std::vector<Loop> live;
  std::map<std::string, NodePtr> zero;
  int64_t N = 1;
  bool idx64 = false;
  // elementwise kernels applied to each result before it is stored (the update that follows a
  // gradient's sum), or null
  const EpilogueSpec* epi = nullptr;

  SerialReduce(const NestKernel& kk, const GenOptions& o, const EpilogueSpec* e = nullptr) : k(kk), opt(o), epi(e) {
    for (const auto& l : k.loops) {
      if (l.extent == 0) throw Error("kernel '" + k.name + "' has an empty loop");
      if (l.extent == 1) zero[l.var] = make_i64(0);
      else live.push_back(l);
    }
    if (k.rloop.extent == 0) throw Error("kernel '" + k.name + "' reduces over an empty axis");
    for (const auto& l : live) N *= l.extent;
    std::vector<LoadRef> loads;
    collect_loads(*k.value, loads);
    int64_t reach = max_abs_index(*k.out_aff, k.loops, &k.rloop);
    for (const auto& lr : loads) {
      auto a = affine_of(*lr.load->args[1]);
      if (!a) { idx64 = true; break; }
      reach = std::max(reach, max_abs_index(*a, k.loops, &k.rloop));
    }
    if (reach >= kIndex32Limit || N >= kIndex32Limit) idx64 = true;
  }

  std::string params(LaunchSpec* ls, bool with_out, const std::string& extra) const {
    std::string t;
    for (const auto& p : k.params) {
      if (p.mut_ && (!with_out || (epi && !epi->store_c))) continue;
      t += (t.empty() ? "" : ", ") + std::string(p.mut_ ? "" : "const ") + ctype(p.dtype.elem()) + "* __restrict__ " + p.name;
      ls->arg_bufs.push_back(p.name);
    }
    if (!extra.empty()) t += (t.empty() ? "" : ", ") + extra;
    if (with_out && epi) t += epi->params;        // (bound by finish_epilogue, after the reduce's own buffers)
    return t;
  }

  // the statement that puts result `value` of the current output where it belongs
  std::string store(const std::string& value, const std::string& indent) const {
    NodePtr oi = rename(k.out_index, {{k.rloop.var, make_i64(0)}});
    ExprRenderer er;
    if (!epi) return indent + k.out_buf + "[" + er.expr(*oi) + "] = (" + ctype(k.out_dtype) + ")" + value + ";\n";
    return indent + "eh_epilogue((long long)(" + er.expr(*oi) + "), (float)" + value + (epi->store_c ? ", " + k.out_buf : std::string()) +
           epi->args + ");\n";
  }
  // the launch that stores the results also binds what the epilogue reads and writes
  void finish_epilogue(LaunchSpec* ls) const {
    if (!epi) return;
    for (size_t i = 0; i < epi->bufs.size(); ++i) {
      ls->arg_bufs.push_back(epi->bufs[i]);
      ls->arg_min_bytes.push_back(epi->min_bytes[i]);
    }
    for (const auto& n : epi->kernels) ls->kernels.push_back(n);
    ls->schedule.insert(ls->schedule.size() - 1, ",epilogue=" + std::to_string(epi->kernels.size()));
    ls->algo_bytes += epi->bytes;
  }
  std::string epilogue_function() const { return epi ? epi->function : std::string(); }

  std::string decode(const std::string& ovar) const {
    std::string t = "  idx_t eh_rem = " + ovar + ";\n  __builtin_assume(eh_rem >= 0);\n";
    for (size_t i = live.size(); i-- > 0;) {
      t += "  const idx_t " + live[i].var + " = eh_rem % " + std::to_string(live[i].extent) + ";\n";
      if (i) t += "  eh_rem /= " + std::to_string(live[i].extent) + ";\n";
    }
    for (const auto& z : zero) t += "  const idx_t " + z.first + " = 0;\n";
    return t;
  }

  void min_bytes(LaunchSpec* ls) const {
    std::map<std::string, int64_t> need;
    std::vector<LoadRef> loads;
    collect_loads(*k.value, loads);
    std::set<std::string> opaque;          // buffers some load reaches through a non-affine index
    for (const auto& lr : loads) {
      auto a = affine_of(*lr.load->args[1]);
      if (!a) { opaque.insert(lr.load->args[0]->name); continue; }
      if (lr.guarded) continue;
      auto& n = need[lr.load->args[0]->name];
      n = std::max(n, max_abs_index(*a, k.loops, &k.rloop) + 1);
    }
    need[k.out_buf] = max_abs_index(*k.out_aff, k.loops, nullptr) + 1;
    for (const auto& b : ls->arg_bufs) {
      size_t item = 4;
      bool is_out = false;
      for (const auto& p : k.params)
        if (p.name == b) { item = p.dtype.elem().itemsize(); is_out = p.mut_; }
      auto it = need.find(b);
      ls->arg_min_bytes.push_back(it == need.end() || (opaque.count(b) && !is_out) ? 0 : static_cast<size_t>(it->second) * item);
    }
  }

  LaunchSpec single() const {
    LaunchSpec ls;
    const int block = 256;
    const int64_t blocks = (N + block - 1) / block;
    if (blocks >= (int64_t{1} << 31)) throw Error("too many outputs for one launch");
    ls.entry = "ehk_" + k.name;
    ls.kernels = {k.name};
    ls.schedule = "serial-reduce(block=256)";
    ls.grid[0] = static_cast<unsigned>(blocks);
    ls.block[0] = block;
    std::ostringstream os;
    os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n" << epilogue_function();
    os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "(" << params(&ls, true, "") << ") {\n";
    os << "  const idx_t eh_o = (idx_t)blockIdx.x * 256 + threadIdx.x;\n  if (eh_o >= " << N << ") return;\n";
    os << decode("eh_o");
    ExprRenderer er;
    const std::string TA = ctype(k.acc_dtype);
    os << "  " << TA << " acc = " << literal(*k.identity) << ";\n";
    os << "  for (idx_t " << k.rloop.var << " = 0; " << k.rloop.var << " < " << k.rloop.extent << "; ++" << k.rloop.var << ") {\n";
    os << "    acc = " << combine_text(k.rkind, k.acc_dtype, "acc", "(" + TA + ")(" + er.expr(*k.value) + ")") << ";\n  }\n";
    os << store("acc", "  ") << "}\n";
    ls.source = os.str();
    min_bytes(&ls);
    finish_epilogue(&ls);
    return ls;
  }

  // (two launches pay only where there is enough to read: a megabyte goes through one)
  bool wants_split() const { return k.rloop.extent >= 512 && N <= (1 << 18) && N * k.rloop.extent >= (int64_t{1} << 21); }
  bool wants_columns() const { return k.rloop.extent >= 32 && N <= (1 << 16); }

  // One launch; a workgroup owns 64 outputs and RG threads share each output's reduction
  // (interleaved rows, partials combined through LDS in a fixed order).  For reductions too
  // short to split over workgroups but long enough that one thread per output would spend
  // its time waiting on dependent loads.
  LaunchSpec columns() const {
    const int64_t K = k.rloop.extent;
    const int RG = K >= 128 ? 16 : 4;
    const int block = 64 * RG;
    LaunchSpec ls;
    ls.entry = "ehk_" + k.name;
    ls.kernels = {k.name};
    ls.schedule = "column-reduce(block=" + std::to_string(block) + ",threads/output=" + std::to_string(RG) + ")";
    ls.grid[0] = static_cast<unsigned>((N + 63) / 64);
    ls.block[0] = static_cast<unsigned>(block);
    const std::string TA = ctype(k.acc_dtype);
    ExprRenderer er;
    std::ostringstream os;
    os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n" << epilogue_function();
    os << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << ls.entry << "(" << params(&ls, true, "")
       << ") {\n";
    os << "  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;\n";
    os << "  const idx_t eh_oo = (idx_t)blockIdx.x * 64 + tx;\n  const bool eh_ok = eh_oo < " << N << ";\n";
    os << "  const idx_t eh_o = eh_ok ? eh_oo : " << N - 1 << ";\n";
    os << decode("eh_o");
    os << "  " << TA << " acc = " << literal(*k.identity) << ";\n";
    os << "#pragma unroll 4\n";
    os << "  for (idx_t " << k.rloop.var << " = ty; " << k.rloop.var << " < " << K << "; " << k.rloop.var << " += " << RG
       << ") {\n";
    os << "    acc = " << combine_text(k.rkind, k.acc_dtype, "acc", "(" + TA + ")(" + er.expr(*k.value) + ")") << ";\n  }\n";
    os << "  __shared__ " << TA << " eh_sm[" << RG << "][64];\n  eh_sm[ty][tx] = acc;\n  __syncthreads();\n";
    os << "  if (ty == 0 && eh_ok) {\n    " << TA << " r = eh_sm[0][tx];\n";
    os << "    for (int q = 1; q < " << RG << "; ++q) r = " << combine_text(k.rkind, k.acc_dtype, "r", "eh_sm[q][tx]") << ";\n";
    os << store("r", "    ") << "  }\n}\n";
    ls.source = os.str();
    min_bytes(&ls);
    finish_epilogue(&ls);
    return ls;
  }

  // Two launches and one scratch buffer (appended to `buffers`).
  std::vector<LaunchSpec> split(std::vector<BufferInfo>* buffers) const {
    const int64_t K = k.rloop.extent;
    const int64_t cols = (N + 63) / 64;
    int64_t S = std::max<int64_t>(1, std::min<int64_t>((2048 + cols - 1) / cols, K / 128));
    const int64_t CH = (K + S - 1) / S;
    S = (K + CH - 1) / CH;
    const std::string TA = ctype(k.acc_dtype);
    const std::string scratch = "eh_part_" + k.name;
    BufferInfo sb;
    sb.name = scratch;
    sb.dtype = k.acc_dtype;
    sb.shape = {S, N};
    sb.role = "temp";
    buffers->push_back(sb);
    ExprRenderer er;
    std::vector<LaunchSpec> out(2);
    {
      LaunchSpec& ls = out[0];
      ls.entry = "ehk_" + k.name + "_part";
      ls.kernels = {k.name};
      ls.schedule = "split-reduce(chunks=" + std::to_string(S) + ",rows/chunk=" + std::to_string(CH) + ")";
      ls.grid[0] = static_cast<unsigned>(cols);
      ls.grid[1] = static_cast<unsigned>(S);
      ls.block[0] = 256;
      std::ostringstream os;
      os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
      os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "("
         << params(&ls, false, TA + "* __restrict__ " + scratch) << ") {\n";
      ls.arg_bufs.push_back(scratch);
      os << "  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;\n";
      os << "  const idx_t eh_oo = (idx_t)blockIdx.x * 64 + tx;\n  const bool eh_ok = eh_oo < " << N << ";\n";
      os << "  const idx_t eh_o = eh_ok ? eh_oo : " << N - 1 << ";\n";
      os << decode("eh_o");
      os << "  const idx_t eh_r0 = (idx_t)blockIdx.y * " << CH << ";\n";
      os << "  const idx_t eh_r1 = eh_r0 + " << CH << " < " << K << " ? eh_r0 + " << CH << " : " << K << ";\n";
      os << "  " << TA << " acc = " << literal(*k.identity) << ";\n";
      os << "#pragma unroll 8\n";
      os << "  for (idx_t " << k.rloop.var << " = eh_r0 + ty; " << k.rloop.var << " < eh_r1; " << k.rloop.var << " += 4) {\n";
      os << "    acc = " << combine_text(k.rkind, k.acc_dtype, "acc", "(" + TA + ")(" + er.expr(*k.value) + ")") << ";\n  }\n";
      os << "  __shared__ " << TA << " eh_sm[4][64];\n  eh_sm[ty][tx] = acc;\n  __syncthreads();\n";
      os << "  if (ty == 0 && eh_ok) {\n    " << TA << " r = eh_sm[0][tx];\n";
      for (int q = 1; q < 4; ++q)
        os << "    r = " << combine_text(k.rkind, k.acc_dtype, "r", "eh_sm[" + std::to_string(q) + "][tx]") << ";\n";
      os << "    " << scratch << "[(idx_t)blockIdx.y * " << N << " + eh_oo] = r;\n  }\n}\n";
      ls.source = os.str();
      min_bytes(&ls);
      ls.arg_min_bytes.back() = static_cast<size_t>(S * N) * k.acc_dtype.itemsize();
    }
    {
      LaunchSpec& ls = out[1];
      ls.entry = "ehk_" + k.name;
      ls.kernels = {k.name};
      ls.schedule = "split-reduce-final(chunks=" + std::to_string(S) + ")";
      ls.grid[0] = static_cast<unsigned>((N + 255) / 256);
      ls.block[0] = 256;
      std::ostringstream os;
      os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n" << epilogue_function();
      const bool with_out = !(epi && !epi->store_c);
      os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "(const " << TA << "* __restrict__ "
         << scratch << (with_out ? ", " + ctype(k.out_dtype) + "* __restrict__ " + k.out_buf : std::string())
         << (epi ? epi->params : std::string()) << ") {\n";
      ls.arg_bufs = {scratch};
      if (with_out) ls.arg_bufs.push_back(k.out_buf);
      os << "  const idx_t eh_o = (idx_t)blockIdx.x * 256 + threadIdx.x;\n  if (eh_o >= " << N << ") return;\n";
      os << decode("eh_o");
      os << "  " << TA << " acc = " << literal(*k.identity) << ";\n";
      os << "  for (idx_t s = 0; s < " << S << "; ++s) acc = "
         << combine_text(k.rkind, k.acc_dtype, "acc", scratch + "[s * " + std::to_string(N) + " + eh_o]") << ";\n";
      os << store("acc", "  ") << "}\n";
      ls.source = os.str();
      ls.arg_min_bytes = {static_cast<size_t>(S * N) * k.acc_dtype.itemsize()};
      if (with_out)
        ls.arg_min_bytes.push_back(static_cast<size_t>(max_abs_index(*k.out_aff, k.loops, nullptr) + 1) * k.out_dtype.itemsize());
      finish_epilogue(&ls);
    }
    return out;
  }
};

// One work-item per output of a short reduce `r`; `chain` are the pure gathers between the
// source and r's operand, nearest first (chain[0] wrote what r reads).  Each gather becomes a
// device function of the element's position in its dense output: the loop variables are
// decoded from the position and the gather's own expression is evaluated, with its load of
// the previous gather's output turned into a call of that gather's function.
LaunchSpec emit_window_reduce(const NestKernel& r, const std::vector<const NestKernel*>& chain, const GenOptions& opt,
                              const std::map<std::string, size_t>& elems) {
  LaunchSpec ls;
  ls.entry = "ehk_" + r.name;
  ls.kernels = {};
  for (size_t j = chain.size(); j-- > 0;) ls.kernels.push_back(chain[j]->name);
  ls.kernels.push_back(r.name);
  int64_t N = 1;
  std::vector<Loop> live;
  for (const auto& l : r.loops) {
    N *= l.extent;
    if (l.extent > 1) live.push_back(l);
  }
  if ((N + 255) / 256 >= (int64_t{1} << 31)) throw Error("too many outputs for one launch");
  std::vector<LoadRef> deep;
  collect_loads(*chain.back()->value, deep);
  const std::string src = deep[0].load->args[0]->name;
  bool idx64 = N >= kIndex32Limit;
  auto big = [&](const std::string& b) {
    auto it = elems.find(b);
    return it == elems.end() || it->second >= static_cast<size_t>(kIndex32Limit);
  };
  idx64 = idx64 || big(src) || big(r.out_buf);
  for (const auto* g : chain) idx64 = idx64 || big(g->out_buf);
  std::vector<LoadRef> rloads;
  collect_loads(*r.value, rloads);
  for (const auto& lr : rloads) idx64 = idx64 || big(lr.load->args[0]->name);
  std::ostringstream os;
  os << hdr(opt) << "typedef " << (idx64 ? "long long" : "int") << " idx_t;\n";
  for (size_t j = chain.size(); j-- > 0;)
    os << gather_fn_text(*chain[j], src, j + 1 < chain.size() ? chain[j + 1] : nullptr, "idx_t");
  // parameters: r's own, with the window buffer replaced by the source
  const std::string T = chain[0]->out_buf;
  std::string sig;
  bool src_listed = false;
  for (const auto& p : r.params) {
    std::string name = p.name;
    if (name == T) name = src;
    if (name == src) {
      if (src_listed) continue;
      src_listed = true;
    }
    sig += (sig.empty() ? "" : ", ") + std::string(p.mut_ ? "" : "const ") + ctype(p.dtype.elem()) + "* __restrict__ " + name;
    ls.arg_bufs.push_back(name);
  }
  os << "extern \"C\" __global__ void __launch_bounds__(256) " << ls.entry << "(" << sig << ") {\n";
  os << "  const idx_t eh_o = (idx_t)blockIdx.x * 256 + threadIdx.x;\n  if (eh_o >= " << N << ") return;\n";
  os << "  idx_t eh_rem = eh_o;\n  __builtin_assume(eh_rem >= 0);\n";
  for (size_t q = live.size(); q-- > 0;) {
    os << "  const idx_t " << live[q].var << " = eh_rem % " << live[q].extent << ";\n";
    if (q) os << "  eh_rem /= " << live[q].extent << ";\n";
  }
  for (const auto& l : r.loops)
    if (l.extent == 1) os << "  const idx_t " << l.var << " = 0;\n";
  ExprRenderer er;
  std::vector<Loop> rvars = r.loops;
  rvars.push_back(r.rloop);
  er.load_hook = [&](const Node& ld, std::string* out) {
    if (ld.args[0]->op != Op::Var || ld.args[0]->name != T) return false;
    *out = gather_call(*chain[0], src, *ld.args[1], rvars, "idx_t");
    return true;
  };
  os << "  float acc = " << literal(*r.identity) << ";\n#pragma unroll\n";
  os << "  for (idx_t " << r.rloop.var << " = 0; " << r.rloop.var << " < " << r.rloop.extent << "; ++" << r.rloop.var << ") {\n";
  os << "    acc = " << combine_text(r.rkind, r.acc_dtype, "acc", "(float)(" + er.expr(*r.value) + ")") << ";\n  }\n";
  NodePtr oi = rename(r.out_index, {{r.rloop.var, make_i64(0)}});
  ExprRenderer eo;
  os << "  " << r.out_buf << "[" << eo.expr(*oi) << "] = acc;\n}\n";
  ls.source = os.str();
  ls.grid[0] = static_cast<unsigned>((N + 255) / 256);
  ls.block[0] = 256;
  ls.schedule = "window-reduce(window=" + std::to_string(r.rloop.extent) + ",gathers=" + std::to_string(chain.size()) + ")";
  // smallest buffers: the source as the innermost gather reads it (unguarded loads), r's other
  // operands and its output as r indexes them
  std::map<std::string, int64_t> need;
  for (const auto& lr : deep) {
    auto a = affine_of(*lr.load->args[1]);
    if (!a || lr.guarded) continue;
    auto& n = need[src];
    n = std::max(n, max_abs_index(*a, chain.back()->loops, nullptr) + 1);
  }
  for (const auto& lr : rloads) {
    const std::string& b = lr.load->args[0]->name;
    auto a = affine_of(*lr.load->args[1]);
    if (b == T || !a || lr.guarded) continue;
    auto& n = need[b];
    n = std::max(n, max_abs_index(*a, r.loops, &r.rloop) + 1);
  }
  need[r.out_buf] = max_abs_index(*r.out_aff, r.loops, nullptr) + 1;
  std::set<std::string> counted;
  for (const auto& b : ls.arg_bufs) {
    auto it = need.find(b);
    ls.arg_min_bytes.push_back(it == need.end() ? 0 : static_cast<size_t>(it->second) * 4);
    auto e = elems.find(b);
    if (e != elems.end() && counted.insert(b).second) ls.algo_bytes += 4.0 * static_cast<double>(e->second);
  }
  return ls;
}

void emit_serial_reduce(const NestKernel& k, const GenOptions& opt, ProgramPlan* plan, const EpilogueSpec* epi) {
  SerialReduce sr(k, opt, epi);
  if (sr.wants_split()) {
    for (auto& ls : sr.split(&plan->buffers)) plan->launches.push_back(std::move(ls));
  } else if (sr.wants_columns()) {
    plan->launches.push_back(sr.columns());
  } else {
    plan->launches.push_back(sr.single());
  }
}

bool serial_reduce_is_one_launch(const NestKernel& k, const GenOptions& opt) { return !SerialReduce(k, opt).wants_split(); }

// Several launches of the serial-reduce family that do not depend on each other, as one launch:
// each becomes a device function in a namespace of its own (its index type, its epilogue), and
// the merged kernel hands every workgroup to the part whose range of workgroup numbers it falls
// into.  Every dependent launch costs about four microseconds whatever it computes, so the
// updates of a training step's parameters, each a few workgroups, are worth taking together.
LaunchSpec merge_launches(const std::vector<LaunchSpec>& parts, const GenOptions& opt) {
  LaunchSpec out;
  const std::string head = hdr(opt);
  unsigned block = 0;
  for (const auto& p : parts) block = std::max(block, p.block[0]);
  out.entry = parts.front().entry + "_and_" + std::to_string(parts.size() - 1);
  std::ostringstream os, sig, body;
  os << head;
  unsigned first = 0;
  for (size_t i = 0; i < parts.size(); ++i) {
    const LaunchSpec& p = parts[i];
    if (p.source.rfind(head, 0) != 0 || p.grid[1] != 1 || p.grid[2] != 1 || p.block[1] != 1 || p.block[2] != 1 || p.block[0] % 64 || p.lds_bytes)
      throw Error("internal: launch '" + p.entry + "' cannot be merged");
    std::string text = p.source.substr(head.size());
    const std::string open = "extern \"C\" __global__ void __launch_bounds__(" + std::to_string(p.block[0]) + ") " + p.entry + "(";
    const size_t at = text.find(open);
    const size_t close = at == std::string::npos ? at : text.find(") {\n", at);
    if (close == std::string::npos) throw Error("internal: launch '" + p.entry + "' has no entry point to merge");
    const std::string params = text.substr(at + open.size(), close - at - open.size());
    text.replace(at, open.size(), "__device__ __forceinline__ void eh_run(const unsigned eh_bx, ");
    for (size_t q = text.find("blockIdx.x"); q != std::string::npos; q = text.find("blockIdx.x", q)) text.replace(q, 10, "eh_bx");
    const std::string own_grid = std::to_string(p.grid[0]) + "u";
    for (size_t q = text.find("gridDim.x"); q != std::string::npos; q = text.find("gridDim.x", q)) text.replace(q, 9, own_grid);
    const std::string ns = "eh_part" + std::to_string(i);
    os << "namespace " << ns << " {\n" << text << "}  // namespace " << ns << "\n";
    // the part's parameters, renamed, in the merged signature; the same names in the call
    std::string call;
    size_t from = 0, n = 0;
    while (from < params.size()) {
      size_t comma = params.find(", ", from);
      if (comma == std::string::npos) comma = params.size();
      const std::string one = params.substr(from, comma - from);
      const size_t sp = one.rfind(' ');
      const std::string name = "p" + std::to_string(i) + "_" + one.substr(sp + 1);
      sig << (sig.tellp() > 0 ? ", " : "") << one.substr(0, sp + 1) << name;
      call += ", " + name;
      from = comma + 2;
      ++n;
    }
    if (n != p.arg_bufs.size()) throw Error("internal: launch '" + p.entry + "' lists " + std::to_string(p.arg_bufs.size()) + " buffers for " + std::to_string(n) + " parameters");
    body << "  if (blockIdx.x < " << first + p.grid[0] << "u) {\n    if (threadIdx.x < " << p.block[0] << "u) " << ns << "::eh_run(blockIdx.x - "
         << first << "u" << call << ");\n    return;\n  }\n";
    first += p.grid[0];
    for (size_t a = 0; a < p.arg_bufs.size(); ++a) {
      out.arg_bufs.push_back(p.arg_bufs[a]);
      out.arg_min_bytes.push_back(a < p.arg_min_bytes.size() ? p.arg_min_bytes[a] : 0);
    }
    for (const auto& kn : p.kernels) out.kernels.push_back(kn);
    out.algo_bytes += p.algo_bytes;
    out.flops += p.flops;
    out.schedule += (i ? " + " : "together(") + p.schedule;
  }
  out.schedule += ")";
  os << "extern \"C\" __global__ void __launch_bounds__(" << block << ") " << out.entry << "(" << sig.str() << ") {\n" << body.str() << "}\n";
  out.source = os.str();
  out.grid[0] = first;
  out.block[0] = block;
  return out;
}

}  // namespace

}  // namespace eh
