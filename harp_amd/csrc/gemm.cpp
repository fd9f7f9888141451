#include "gemm.hpp"

#include <sstream>

namespace eh {

namespace {

// The kernel text is kept in kernels/gemm_f32_mfma.hip and wrapped into a raw string literal
// by the build.
const char* kGemmSource =
#include "kernels/gemm_f32_mfma.hip.inc"
    ;

struct Tile {
  int bm, bn, bk, wm, wn;
};

// Largest first.  Each uses 256 threads (four waves).
const Tile kTiles[] = {{128, 128, 16, 64, 64}, {64, 64, 16, 32, 32}};

bool pick_tile(const GemmShape& s, const GenOptions& opt, Tile* out) {
  auto fits = [&](const Tile& t) {
    if (s.M % t.bm || s.N % t.bn || s.K % t.bk) return false;
    if (t.bm % t.wm || t.bn % t.wn || t.wm % 32 || t.wn % 32) return false;
    int nt = (t.bm / t.wm) * (t.bn / t.wn) * 64;
    if (nt > 1024 || (t.bm * t.bk) % (4 * nt) || (t.bn * t.bk) % (4 * nt)) return false;
    size_t lds = 2ull * static_cast<size_t>(t.bk) * (t.bm + 4 + t.bn + 4) * 4;
    return lds <= 160 * 1024;
  };
  if (opt.gemm_bm > 0) {
    Tile t{opt.gemm_bm, opt.gemm_bn, opt.gemm_bk, opt.gemm_wm, opt.gemm_wn};
    if (fits(t)) { *out = t; return true; }
    return false;
  }
  for (const auto& t : kTiles)
    if (fits(t)) {
      // prefer the small tile when the big one cannot fill the chip
      if (t.bm == 128 && (s.M / 128) * (s.N / 128) * s.batch < 256 && fits(kTiles[1])) continue;
      *out = t;
      return true;
    }
  return false;
}

// 128-bit global loads need every row start on a 4-float boundary.
bool vector_ok(const GemmShape& s) {
  bool a_k = s.a_k == 1, a_m = s.a_m == 1;
  bool b_n = s.b_n == 1, b_k = s.b_k == 1;
  if (!(a_k || a_m) || !(b_n || b_k)) return false;
  int64_t lda = a_k ? s.a_m : s.a_k, ldb = b_n ? s.b_k : s.b_n;
  if (lda % 4 || ldb % 4 || s.a_off % 4 || s.b_off % 4 || s.a_b % 4 || s.b_b % 4) return false;
  return s.c_n == 1;
}

}  // namespace

std::optional<GemmShape> match_gemm(const NestKernel& k) {
  if (k.rkind != ReduceKind::Sum || !k.identity || k.identity->fval != 0.0) return std::nullopt;
  if (k.acc_dtype.ty != Ty::F32 || k.out_dtype.ty != Ty::F32) return std::nullopt;
  const Node& v = *k.value;
  if (v.op != Op::Mul || v.args[0]->op != Op::Load || v.args[1]->op != Op::Load) return std::nullopt;
  const Node* la = v.args[0].get();
  const Node* lb = v.args[1].get();
  if (la->dtype.ty != Ty::F32 || lb->dtype.ty != Ty::F32) return std::nullopt;
  auto aa = affine_of(*la->args[1]);
  auto ab = affine_of(*lb->args[1]);
  if (!aa || !ab || !k.out_aff) return std::nullopt;
  const std::string& kv = k.rloop.var;
  if (aa->of(kv) <= 0 || ab->of(kv) <= 0 || k.rloop.extent < 2) return std::nullopt;
  std::string mvar, nvar, bvar;
  int64_t M = 0, N = 0, batch = 1;
  for (const auto& l : k.loops) {
    if (l.extent == 1) continue;
    bool in_a = aa->of(l.var) != 0, in_b = ab->of(l.var) != 0;
    if (in_a && !in_b) {
      if (!mvar.empty()) return std::nullopt;
      mvar = l.var;
      M = l.extent;
    } else if (in_b && !in_a) {
      if (!nvar.empty()) return std::nullopt;
      nvar = l.var;
      N = l.extent;
    } else if (in_a && in_b) {
      if (!bvar.empty()) return std::nullopt;
      bvar = l.var;
      batch = l.extent;
    } else {
      return std::nullopt;
    }
  }
  if (mvar.empty() || nvar.empty()) return std::nullopt;
  // operands may come in either order; make `A` the one indexed by the output's row variable
  GemmShape s;
  s.M = M; s.N = N; s.K = k.rloop.extent; s.batch = batch;
  s.a_buf = la->args[0]->name; s.b_buf = lb->args[0]->name; s.c_buf = k.out_buf;
  s.a_m = aa->of(mvar); s.a_k = aa->of(kv); s.a_off = aa->c;
  s.b_n = ab->of(nvar); s.b_k = ab->of(kv); s.b_off = ab->c;
  s.c_m = k.out_aff->of(mvar); s.c_n = k.out_aff->of(nvar); s.c_off = k.out_aff->c;
  if (!bvar.empty()) {
    s.a_b = aa->of(bvar); s.b_b = ab->of(bvar); s.c_b = k.out_aff->of(bvar);
  }
  if (s.a_m <= 0 || s.b_n <= 0 || s.c_m <= 0 || s.c_n <= 0) return std::nullopt;
  if (s.c_n != 1 && s.c_m == 1) {
    // C is column-major: compute C^T = B^T A^T instead, which is row-major
    GemmShape t = s;
    t.M = s.N; t.N = s.M;
    t.a_buf = s.b_buf; t.b_buf = s.a_buf;
    t.a_m = s.b_n; t.a_k = s.b_k; t.a_off = s.b_off; t.a_b = s.b_b;
    t.b_n = s.a_m; t.b_k = s.a_k; t.b_off = s.a_off; t.b_b = s.a_b;
    t.c_m = s.c_n; t.c_n = s.c_m;
    return t;
  }
  return s;
}

bool gemm_shaped(const NestKernel& k, const GenOptions& opt) {
  auto s = match_gemm(k);
  Tile t;
  return s && vector_ok(*s) && pick_tile(*s, opt, &t);
}

std::optional<LaunchSpec> try_emit_gemm(const NestKernel& k, const GenOptions& opt) {
  auto s = match_gemm(k);
  Tile t;
  if (!s || !vector_ok(*s) || !pick_tile(*s, opt, &t)) return std::nullopt;
  const bool a_kc = s->a_k == 1, b_nc = s->b_n == 1;
  LaunchSpec ls;
  ls.entry = "ehk_" + k.name;
  ls.kernels = {k.name};
  const int nt = (t.bm / t.wm) * (t.bn / t.wn) * 64;
  std::ostringstream os;
  os << "// generated for gfx950 by eclat backend-hip: MFMA contraction\n";
  os << "#define EH_ENTRY " << ls.entry << "\n";
  os << "#define EH_M " << s->M << "\n#define EH_N " << s->N << "\n#define EH_K " << s->K << "\n#define EH_BATCH "
     << s->batch << "\n";
  os << "#define EH_BM " << t.bm << "\n#define EH_BN " << t.bn << "\n#define EH_BK " << t.bk << "\n#define EH_WM "
     << t.wm << "\n#define EH_WN " << t.wn << "\n";
  os << "#define EH_A_KCONTIG " << (a_kc ? 1 : 0) << "\n#define EH_B_NCONTIG " << (b_nc ? 1 : 0) << "\n";
  os << "#define EH_LDA " << (a_kc ? s->a_m : s->a_k) << "LL\n#define EH_LDB " << (b_nc ? s->b_k : s->b_n)
     << "LL\n#define EH_LDC " << s->c_m << "LL\n";
  os << "#define EH_A_OFF " << s->a_off << "LL\n#define EH_B_OFF " << s->b_off << "LL\n#define EH_C_OFF " << s->c_off
     << "LL\n";
  os << "#define EH_A_BS " << s->a_b << "LL\n#define EH_B_BS " << s->b_b << "LL\n#define EH_C_BS " << s->c_b << "LL\n";
  os << "#define EH_GROUP_M 8\n";
  os << kGemmSource;
  ls.source = os.str();
  ls.schedule = "mfma32x32x2(tile=" + std::to_string(t.bm) + "x" + std::to_string(t.bn) + "x" + std::to_string(t.bk) +
                ",wave=" + std::to_string(t.wm) + "x" + std::to_string(t.wn) + (a_kc ? ",A:k" : ",A:m") +
                (b_nc ? ",B:n" : ",B:k") + ")";
  ls.grid[0] = static_cast<unsigned>((s->M / t.bm) * (s->N / t.bn));
  ls.grid[2] = static_cast<unsigned>(s->batch);
  ls.block[0] = static_cast<unsigned>(nt);
  ls.arg_bufs = {s->a_buf, s->b_buf, s->c_buf};
  ls.arg_min_bytes = {
      4 * static_cast<size_t>(s->a_off + (s->M - 1) * s->a_m + (s->K - 1) * s->a_k + (s->batch - 1) * s->a_b + 1),
      4 * static_cast<size_t>(s->b_off + (s->K - 1) * s->b_k + (s->N - 1) * s->b_n + (s->batch - 1) * s->b_b + 1),
      4 * static_cast<size_t>(s->c_off + (s->M - 1) * s->c_m + (s->N - 1) * s->c_n + (s->batch - 1) * s->c_b + 1)};
  ls.flops = 2.0 * static_cast<double>(s->M) * static_cast<double>(s->N) * static_cast<double>(s->K) *
             static_cast<double>(s->batch);
  ls.algo_bytes = 4.0 * static_cast<double>(s->batch) *
                  (static_cast<double>(s->M) * s->K + static_cast<double>(s->K) * s->N + static_cast<double>(s->M) * s->N);
  return ls;
}

}  // namespace eh
