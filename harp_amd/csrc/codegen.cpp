// Rendering of expressions and statements, and the two schedules that replay a kernel as it is
// written: one work-item, or the outer loops of each nest over work-items.
#include "codegen.hpp"

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
Ty infer_ty(const Node& n, const std::map<std::string, Ty>* vars) {
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


bool holds_load(const Node& n) {
  if (n.op == Op::Load) return true;
  for (const auto& a : n.args)
    if (a && holds_load(*a)) return true;
  return false;
}

// set by plan_program for the plan it is making (GenOptions::guard_branches)
thread_local bool g_guard_branches = false;
thread_local bool g_ranged_loads = true;


std::string hdr(const GenOptions&) { return kernel_header(); }

// ---------------------------------------------------------------------------------------------
// statement-by-statement rendering (kernels no schedule recognises)
// ---------------------------------------------------------------------------------------------

namespace {
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
        for (const auto& a : n.args) {
          // A block with declarations inside a block gets braces: the reference prints it without
          // (src/backend/renderer.rs:604-624), and an unrolled loop around a reduction -- the same
          // block with its accumulator several times over -- is then a redefinition in C.
          if (a->op == Op::Block && !a->decls.empty()) {
            s += ind() + "{\n";
            ++level;
            s += stmt(*a);
            --level;
            s += ind() + "}\n";
          } else {
            s += stmt(*a);
          }
        }
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
}  // namespace

// Value of a dispatch-size expression, evaluated as the reference's pipeline does
// (`evaluate_ast_expr`, src/backend/pipeline.rs:505-553): constants, +, *, integer division and
// remainder (a zero divisor gives 1 and 0), max.  Shape variables are not supported on this
// path, so a variable or any other node is an error rather than the reference's silent 1.
static int64_t dispatch_value(const Node& n) {
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

static const char* const kAtomicMaxF32 = R"EHA(
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


std::string render_expr_text(const Node& e) {
  ExprRenderer er;
  return er.expr(e);
}

// A kernel (or one of its loop nests) that is about to run in a single work-item: fine for the
// few statements of a short scan, hopeless for millions of iterations.  Refused rather than
// launched, unless the caller asked for it.
static void refuse_long_serial(const std::string& kernel, const Node& body, const GenOptions& opt) {
  const double limit = 131072;
  const double n = serial_iterations(body);
  if (n <= limit || opt.allow_serial) return;
  throw Error("kernel '" + kernel + "' has a form no schedule of this backend recognises and would run its " +
              std::to_string(static_cast<long long>(n)) +
              " loop iterations in one work-item: not supported (compile with allow_serial=1 to run it anyway)");
}

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
}  // namespace

// A prefix scan along one line, as `LoopGenerator::generate_scan` writes it
// (src/lowerer/lower.rs:691-735): acc = identity; for the inner loops { acc = combine(acc,
// value); out[index] = acc }.
namespace {
struct ScanLine {
  std::string acc;
  DType acc_dtype;
  NodePtr identity, value, out_ptr, out_index;
  ReduceKind kind = ReduceKind::None;
  std::vector<Loop> loops;     // the scanned loops, outermost first
  int64_t length = 1;
};
}  // namespace

static std::optional<ScanLine> match_scan_line(const Node& n) {
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


static void collect_writes(const Node& n, std::vector<WriteRef>& writes, std::set<std::string>& read_bufs,
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
static bool injective(const Affine& a, const std::vector<Loop>& vars) {
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



static bool stores_anything(const Node& n) {
  if (n.op == Op::Store || n.op == Op::AtomicAdd || n.op == Op::AtomicMax) return true;
  for (const auto& a : n.args)
    if (stores_anything(*a)) return true;
  return false;
}

// A loop of at least 64 iterations that only accumulates (assigns, stores nothing): the inner loop of
// a reduction, as opposed to a scan's, which stores every step.
static bool has_accumulating_loop(const Node& n) {
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

static void warn_once_degraded(const std::string& kernel) {
  static std::mutex mu;
  static std::set<std::string> seen;
  std::lock_guard<std::mutex> lock(mu);
  if (seen.size() > 256 || !seen.insert(kernel).second) return;
  std::fprintf(stderr, "eclat-hip: kernel '%s' has a loop structure no schedule recognises as written and runs one "
               "work-item per outer iteration (plan marked 'degraded')\n", kernel.c_str());
}


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
// options
// ---------------------------------------------------------------------------------------------

unsigned long long fnv1a(const std::string& text) {
  unsigned long long h = 1469598103934665603ull;
  for (unsigned char c : text) {
    h ^= c;
    h *= 1099511628211ull;
  }
  return h;
}

// (the kernel's own name and the names of its buffers count for nothing: the same lowered kernel
// gets other names in another program)
unsigned long long launch_tune_key(const Node& kernel) {
  std::string text = to_text(kernel);
  auto rename_all = [&](const std::string& from, const std::string& to) {
    const std::string q = "\"" + from + "\"";
    for (size_t at = text.find(q); at != std::string::npos; at = text.find(q, at + to.size() + 2)) text.replace(at, q.size(), "\"" + to + "\"");
  };
  if (!kernel.name.empty()) rename_all(kernel.name, "k");
  size_t n = 0;
  for (const auto& p : kernel.params)
    if (p.dtype.is_ptr()) rename_all(p.name, "b" + std::to_string(n++));
  return fnv1a(text);
}

void apply_options(GenOptions* out, const std::string& text) {
  GenOptions& o = *out;
  std::stringstream ss(text);
  std::string item;
  while (std::getline(ss, item, ',')) {
    if (item.empty()) continue;
    if (item[0] == '@') {
      // "@<16 hex digits>:<name>=<value>": for the launch with that key only
      const size_t colon = item.find(':');
      if (colon != 17 || item.find('=', colon) == std::string::npos) throw Error("option '" + item + "' is not @<key>:name=value");
      unsigned long long key = 0;
      try {
        key = std::stoull(item.substr(1, 16), nullptr, 16);
      } catch (const std::logic_error&) {
        throw Error("option '" + item + "': the key is not 16 hex digits");
      }
      GenOptions probe;                                  // (checked now, applied when the launch is planned)
      apply_options(&probe, item.substr(colon + 1));
      std::string& s = o.launch_options[key];
      s += (s.empty() ? "" : ",") + item.substr(colon + 1);
      continue;
    }
    size_t eq = item.find('=');
    if (eq == std::string::npos) throw Error("option '" + item + "' is not key=value");
    std::string k = item.substr(0, eq), v = item.substr(eq + 1);
    auto as_int = [&]() {
      try {
        return std::stoi(v);
      } catch (const std::logic_error&) {
        throw Error("option '" + k + "' needs an integer, got '" + v + "'");
      }
    };
    if (k == "arch") o.arch = v;
    else if (k == "fuse") o.fuse = as_int() != 0;
    else if (k == "vectorize") o.vectorize = as_int() != 0;
    else if (k == "transpose") o.transpose = as_int() != 0;
    else if (k == "window") o.window = as_int() != 0;
    else if (k == "row_threads") o.row_threads = as_int();
    else if (k == "row_elems") o.row_elems = std::max(1, as_int());
    else if (k == "flat_block") o.flat_block = as_int();
    else if (k == "flat_iters") o.flat_iters = std::max(1, as_int());
    else if (k == "gemm") o.gemm = as_int() != 0;
    else if (k == "gemm_bm") o.gemm_bm = as_int();
    else if (k == "gemm_bn") o.gemm_bn = as_int();
    else if (k == "gemm_bk") o.gemm_bk = as_int();
    else if (k == "gemm_wm") o.gemm_wm = as_int();
    else if (k == "gemm_wn") o.gemm_wn = as_int();
    else if (k == "gemm_split_k") o.gemm_split_k = as_int();
    else if (k == "gemm_setprio") o.gemm_setprio = as_int();
    else if (k == "gemm_waves") o.gemm_waves = as_int();
    else if (k == "gemm_fold") o.gemm_fold = as_int() != 0;
    else if (k == "gemm_window") o.gemm_window = as_int() != 0;
    else if (k == "window_passes") o.window_passes = std::max(0, std::min(4, as_int()));
    else if (k == "gemm_merge_batch") o.gemm_merge_batch = as_int() != 0;
    else if (k == "gemm_dma") o.gemm_dma = std::max(0, std::min(3, as_int()));
    else if (k == "gemm_mix") o.gemm_mix = as_int() != 0;
    else if (k == "gemm_transpose") o.gemm_transpose = as_int() != 0;
    else if (k == "gemm_prefetch") o.gemm_prefetch = std::max(0, as_int());
    else if (k == "reindex") o.reindex = as_int() != 0;
    else if (k == "guard_branches") o.guard_branches = as_int() != 0;
    else if (k == "ranged_loads") o.ranged_loads = as_int() != 0;
    else if (k == "rematerialize") o.rematerialize = as_int() != 0;
    else if (k == "merge_launches") o.merge_launches = as_int() != 0;
    else if (k == "merge_templates") o.merge_templates = as_int() != 0;
    else if (k == "gemm_tail") o.gemm_tail = as_int() != 0;
    else if (k == "lanes") o.lanes = std::max(1, as_int());
    else if (k == "lane_us") o.lane_us = std::max(0, as_int());
    else if (k == "gemm_epilogue") o.gemm_epilogue = as_int() != 0;
    else if (k == "nontemporal") o.nontemporal = as_int();
    else if (k == "normalize") o.normalize = as_int() != 0;
    else if (k == "allow_serial") o.allow_serial = as_int() != 0;
    else throw Error("unknown option '" + k + "'");
  }
  if (o.flat_block < 64 || o.flat_block > 1024 || (o.flat_block & (o.flat_block - 1)))
    throw Error("flat_block must be a power of two in [64, 1024]");
  if (o.row_threads < 0 || o.row_threads > 1024 || (o.row_threads & (o.row_threads - 1)))
    throw Error("row_threads must be 0 or a power of two up to 1024");
}

GenOptions parse_options(const char* text) {
  GenOptions o;
  if (const char* env = std::getenv("ECLAT_HIP_ARCH")) o.arch = env;
  if (text) apply_options(&o, text);
  return o;
}

GenOptions options_for_launch(const GenOptions& opt, const Node& anchor) {
  if (opt.launch_options.empty()) return opt;
  auto it = opt.launch_options.find(launch_tune_key(anchor));
  if (it == opt.launch_options.end()) return opt;
  GenOptions o = opt;
  apply_options(&o, it->second);
  return o;
}


}  // namespace eh
