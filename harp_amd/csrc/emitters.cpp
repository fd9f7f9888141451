// Source text of the elementwise / reduce schedules.
#include <cctype>
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
// emitters
// ---------------------------------------------------------------------------------------------


static const char* op_struct(ReduceKind k) {
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

static bool pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
static int64_t pow2_ceil(int64_t v) {
  int64_t p = 1;
  while (p < v) p <<= 1;
  return p;
}

// One distinct external access: buffer + affine index over canonical vars.
namespace {
struct ExtLoad {
  std::string buf;
  Affine aff;
  DType dtype;
  int id = 0;
  bool cached = false;   // held in registers for the whole row
};
}  // namespace

// Index arithmetic is done in 32-bit `int` while every index, every loop counter and the
// grid-stride increments added to them (a grid's worth of work-items times the vector width)
// stay well below 2^31; from 2^30 reachable elements on, kernels use 64-bit indices.
constexpr int64_t kIndex32Limit = int64_t{1} << 30;

namespace {
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
    // (only those reads: an unguarded read keeps its pointer, so that an index that runs out of
    // its buffer is not quietly turned into a zero)
    std::set<std::string> guarded_bufs;
    for_each_external_load([&](const LoadRef& lr) {
      if (lr.guarded && lr.load->args[0]->op == Op::Var) guarded_bufs.insert(lr.load->args[0]->name);
    });
    if (!guarded_bufs.empty() && g_ranged_loads && !g_guard_branches && !idx64)
      for (const auto& b : in_bufs) {
        auto it = elems.find(b);
        if (guarded_bufs.count(b) && it != elems.end() && in_dtype.at(b).ty == Ty::F32 && it->second * 4 < (size_t{1} << 31))
          ranged[b] = it->second * 4;
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
}  // namespace

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
namespace {
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
      // what the epilogue reads as well comes in once, with the epilogue's parameters
      if (!p.mut_ && with_out && epi && std::find(epi->bufs.begin(), epi->bufs.end(), p.name) != epi->bufs.end()) continue;
      t += (t.empty() ? "" : ", ") + std::string(p.mut_ ? "" : "const ") + ctype(p.dtype.elem()) + "* __restrict__ " + p.name;
      ls->arg_bufs.push_back(p.name);
    }
    if (!extra.empty()) t += (t.empty() ? "" : ", ") + extra;
    // (bound by finish_epilogue, after the reduce's own buffers; the text starts with ", ")
    if (with_out && epi) t += t.empty() && epi->params.size() > 2 ? epi->params.substr(2) : epi->params;
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
}  // namespace

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

// The same reduce as a function of an output's position, for the launch that produces its source
// to call once a workgroup has stored what that output reads (EpilogueSpec's tail).  Only the
// plain case: r reads nothing but the window buffer, no gather of the chain is guarded, and the
// source is a buffer the epilogue stores.  False when it does not apply.
bool window_reduce_tail(const NestKernel& r, const std::vector<const NestKernel*>& chain,
                        const std::map<std::string, size_t>& elems, EpilogueSpec* epi) {
  if (chain.empty() || !r.out_aff || r.acc_dtype.ty != Ty::F32 || r.out_dtype.ty != Ty::F32) return false;
  std::vector<LoadRef> deep;
  collect_loads(*chain.back()->value, deep);
  if (deep.empty() || deep[0].load->args[0]->op != Op::Var) return false;
  const std::string src = deep[0].load->args[0]->name;
  if (std::find(epi->bufs.begin(), epi->bufs.end(), src) == epi->bufs.end()) return false;
  const std::string T = chain[0]->out_buf;
  std::vector<LoadRef> rloads;
  collect_loads(*r.value, rloads);
  for (const auto& lr : rloads)
    if (lr.load->args[0]->op != Op::Var || lr.load->args[0]->name != T || lr.guarded || !affine_of(*lr.load->args[1])) return false;
  for (const auto* g : chain) {
    std::vector<LoadRef> gl;
    collect_loads(*g->value, gl);
    for (const auto& lr : gl)
      if (lr.guarded || lr.load->args[0]->op != Op::Var || !affine_of(*lr.load->args[1]) || !g->out_aff) return false;
  }
  int64_t N = 1;
  std::vector<Loop> live;
  for (const auto& l : r.loops) {
    N *= l.extent;
    if (l.extent > 1) live.push_back(l);
  }
  auto big = [&](const std::string& b) {
    auto it = elems.find(b);
    return it == elems.end() || it->second >= static_cast<size_t>(kIndex32Limit);
  };
  if (N >= kIndex32Limit || big(src) || big(r.out_buf)) return false;
  for (const auto* g : chain)
    if (big(g->out_buf)) return false;
  // dense output in the order of r's loops: a workgroup's share is a run of positions
  {
    int64_t stride = 1;
    for (size_t i = r.loops.size(); i-- > 0;) {
      if (r.loops[i].extent > 1 && r.out_aff->of(r.loops[i].var) != stride) return false;
      stride *= r.loops[i].extent;
    }
    if (r.out_aff->c != 0 || r.out_aff->of(r.rloop.var) != 0) return false;
  }
  std::ostringstream os;
  os << "// the reduce " << r.name << " over windows of " << src << ", by the position of its output\nnamespace eh_tail_ns {\ntypedef int idx_t;\n";
  for (size_t j = chain.size(); j-- > 0;)
    os << gather_fn_text(*chain[j], src, j + 1 < chain.size() ? chain[j + 1] : nullptr, "idx_t");
  std::string sig;
  epi->tail_params.clear();
  epi->tail_args.clear();
  epi->tail_bufs.clear();
  epi->tail_min_bytes.clear();
  bool src_listed = false;
  for (const auto& p : r.params) {
    std::string name = p.name;
    if (name == T) name = src;
    if (name == src) {
      if (src_listed) continue;
      src_listed = true;
    }
    if (name != src && name != r.out_buf) return false;
    const std::string decl = std::string(p.mut_ ? "" : "const ") + ctype(p.dtype.elem()) + "* __restrict__ " + name;
    sig += ", " + decl;
    epi->tail_args += ", " + (name == src ? std::string("eh_tail_lds") : name);
    if (name != src) {
      if (std::find(epi->bufs.begin(), epi->bufs.end(), name) != epi->bufs.end()) return false;
      epi->tail_params += ", " + decl;
      epi->tail_bufs.push_back(name);
      epi->tail_min_bytes.push_back(static_cast<size_t>(N) * 4);
    }
  }
  if (!src_listed || epi->tail_bufs.size() != 1) return false;
  // output eh_l of group eh_g.  Where a group is one step of the outermost loop, only the inner
  // loops are decoded, from the small number (the workgroup has its SIMDs to itself: every
  // integer division of the decode is time nothing else hides).
  os << "__device__ __forceinline__ void eh_tail(const idx_t eh_g, const idx_t eh_l" << sig << ") {\n";
  os << "  const idx_t eh_o = eh_g * EH_TAIL_PER_GROUP + eh_l;\n";
  int64_t inner = 1;
  for (size_t q = 1; q < live.size(); ++q) inner *= live[q].extent;
  if (!live.empty()) {
    os << "#if EH_TAIL_PER_GROUP == " << inner << "\n  unsigned eh_rem = (unsigned)eh_l;\n";
    for (size_t q = live.size(); q-- > 1;) {
      os << "  const idx_t " << live[q].var << " = (idx_t)(eh_rem % " << live[q].extent << "u);\n";
      if (q > 1) os << "  eh_rem /= " << live[q].extent << "u;\n";
    }
    os << "  const idx_t " << live[0].var << " = eh_g;\n#else\n";
  }
  os << "  unsigned eh_rem = (unsigned)eh_o;\n";
  for (size_t q = live.size(); q-- > 0;) {
    os << "  const idx_t " << live[q].var << " = (idx_t)(eh_rem % " << live[q].extent << "u);\n";
    if (q) os << "  eh_rem /= " << live[q].extent << "u;\n";
  }
  if (!live.empty()) os << "#endif\n";
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
  os << "  " << r.out_buf << "[eh_o] = acc;\n}\n}  // namespace eh_tail_ns\n";
  epi->tail_function = os.str();
  // The launch keeps its workgroup's share of the source in LDS (eh_tail_lds, element e of the
  // source at e - EH_TAIL_BASE): the tail reads it there, and wherever the epilogue stores the
  // source it stores into LDS as well.
  {
    std::string& t = epi->tail_function;
    const std::string from = src + "[", to = src + "[-(idx_t)EH_TAIL_BASE + ";
    size_t n_loads = 0;
    for (size_t q = t.find(from); q != std::string::npos; q = t.find(from, q + to.size())) {
      if (q > 0 && (std::isalnum(static_cast<unsigned char>(t[q - 1])) || t[q - 1] == '_')) continue;
      t.replace(q, from.size(), to);
      ++n_loads;
    }
    if (n_loads == 0) return false;
    size_t n_stores = 0;
    auto twin = [&](std::string* text) {
      const std::string scalar = "    " + src + "[eh_e] = eh_v_" + src + ";\n";
      for (size_t q = text->find(scalar); q != std::string::npos; q = text->find(scalar, q)) {
        const std::string add = scalar + "#ifdef EH_TAIL\n    eh_tail_lds[eh_e - EH_TAIL_BASE] = eh_v_" + src + ";\n#endif\n";
        text->replace(q, scalar.size(), add);
        q += add.size();
        ++n_stores;
      }
      const std::string quad = "    *reinterpret_cast<EhQ<float>*>(" + src + " + eh_e) = ";
      for (size_t q = text->find(quad); q != std::string::npos; q = text->find(quad, q)) {
        const size_t end = text->find(";\n", q);
        if (end == std::string::npos) break;
        const std::string value = text->substr(q + quad.size(), end - q - quad.size());
        const std::string add = "#ifdef EH_TAIL\n    *reinterpret_cast<EhQ<float>*>(eh_tail_lds + (eh_e - EH_TAIL_BASE)) = " + value + ";\n#endif\n";
        text->insert(end + 2, add);
        q = end + 2 + add.size();
        ++n_stores;
      }
    };
    twin(&epi->function);
    twin(&epi->split_functions);
    twin(&epi->quad_functions);
    if (n_stores == 0) return false;
  }
  epi->tail_source = src;
  epi->tail_outputs = N;
  epi->tail_bytes = 4.0 * static_cast<double>(N);
  epi->tail_tag = "window-reduce(window=" + std::to_string(r.rloop.extent) + ",gathers=" + std::to_string(chain.size()) + ")";
  epi->tail_kernels.clear();
  for (size_t j = chain.size(); j-- > 0;) epi->tail_kernels.push_back(chain[j]->name);
  epi->tail_kernels.push_back(r.name);
  // which elements of the source an output reads: the chain's index maps, evaluated on the host
  const NestKernel rk = r;
  std::vector<NestKernel> gs;
  for (const auto* g : chain) gs.push_back(*g);
  epi->tail_reads = [rk, gs, T](int64_t o, std::vector<int64_t>* out) {
    std::map<std::string, int64_t> val;
    int64_t rem = o;
    for (size_t q = rk.loops.size(); q-- > 0;) {
      val[rk.loops[q].var] = rem % rk.loops[q].extent;
      rem /= rk.loops[q].extent;
    }
    auto eval = [](const Affine& a, const std::map<std::string, int64_t>& v) {
      int64_t x = a.c;
      for (const auto& kv : a.coef) {
        auto it = v.find(kv.first);
        x += kv.second * (it == v.end() ? 0 : it->second);
      }
      return x;
    };
    std::vector<LoadRef> rl;
    collect_loads(*rk.value, rl);
    for (int64_t j = 0; j < rk.rloop.extent; ++j) {
      val[rk.rloop.var] = j;
      std::vector<int64_t> at;                       // positions in the current buffer
      for (const auto& lr : rl) at.push_back(eval(*affine_of(*lr.load->args[1]), val));
      for (const auto& g : gs) {
        std::vector<LoadRef> gl;
        collect_loads(*g.value, gl);
        std::vector<int64_t> next;
        for (int64_t pos : at) {
          std::map<std::string, int64_t> gv;         // g's loops from a position in its dense output
          int64_t pr = pos;
          for (size_t q = g.loops.size(); q-- > 0;) {
            gv[g.loops[q].var] = pr % g.loops[q].extent;
            pr /= g.loops[q].extent;
          }
          for (const auto& lr : gl) next.push_back(eval(*affine_of(*lr.load->args[1]), gv));
        }
        at = std::move(next);
      }
      out->insert(out->end(), at.begin(), at.end());
    }
  };
  return true;
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


// Several launches of the serial-reduce family that do not depend on each other, as one launch:
// each becomes a device function in a namespace of its own (its index type, its epilogue), and
// the merged kernel hands every workgroup to the part whose range of workgroup numbers it falls
// into.  Every dependent launch costs about four microseconds whatever it computes, so the
// updates of a training step's parameters, each a few workgroups, are worth taking together.
}  // namespace eh
