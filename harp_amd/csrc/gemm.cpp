#include "gemm.hpp"
#include "window.hpp"

#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdlib>
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

// Candidate tiles: {bm, bn, bk, wm, wn}, workgroups one CU holds at once (registers and LDS),
// sustained TFLOP/s with the chip full (measured on 4096^3), and the share of a full CU's
// rate that a single resident workgroup reaches.
struct Candidate {
  Tile tile;
  int wgs_per_cu;
  double rate, alone;
  double step_us;   // time one k-step of a workgroup takes when nothing hides its load latency
};
const Candidate kCandidates[] = {
    {{256, 256, 16, 64, 64}, 1, 133.0, 1.0, 1.2},    // 16 waves
    {{128, 128, 16, 64, 64}, 4, 124.0, 0.4, 1.0},    // 4 waves
    {{64, 64, 16, 32, 32}, 8, 105.0, 0.25, 0.8},     // 4 waves
    // narrow tiles for contractions with few rows or columns (a convolution's 32 channels, a
    // 3x3 filter's nine taps, ten classes), where a 64-wide tile multiplies mostly padding
    // (measured on the CNN step: 32x64 takes the first convolution, 32 channels by 784 pixels,
    // from 23 to 16 us; 64x32, 128x32x32 and 32x32x16 tiles were tried as well and lost to 64x64 wherever
    // they were chosen)
    {{32, 64, 16, 32, 32}, 12, 80.0, 0.12, 0.8},     // 2 waves
    // one wave: only for results that fit one MFMA tile (the first convolution's weight gradient,
    // 32 channels by 9 taps per image: 19.5 -> 14.9 us, the second wave multiplied only padding)
    {{32, 32, 16, 32, 32}, 16, 50.0, 0.06, 0.8},
};

bool tile_valid(const Tile& t) {
  if (t.bm <= 0 || t.bn <= 0 || t.bk <= 0 || t.wm <= 0 || t.wn <= 0) return false;
  if (t.bm % t.wm || t.bn % t.wn || t.wm % 32 || t.wn % 32 || t.bk % 16) return false;
  int nt = (t.bm / t.wm) * (t.bn / t.wn) * 64;
  if (nt > 1024 || (t.bm * t.bk) % (4 * nt) || (t.bn * t.bk) % (4 * nt)) return false;
  size_t lds = 2ull * static_cast<size_t>(t.bk) * (t.bm + 4 + t.bn + 4) * 4;
  return lds <= 160 * 1024;
}

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

struct Choice {
  Tile tile;
  int split_k = 1;
};

// Estimated microseconds for one tile shape and K split: whole rounds of resident
// workgroups at the tile's sustained rate, a last partial round no faster than a lone
// workgroup allows, plus writing and re-reading the partial tiles when K is split.
double estimate_us(const GemmShape& s, const Candidate& c, int split) {
  const double cus = 256.0;
  const int64_t wgs = ceil_div(s.M, c.tile.bm) * ceil_div(s.N, c.tile.bn) * s.batch * split;
  const int64_t ksteps = ceil_div(ceil_div(s.K, c.tile.bk), split);
  const double wg_flops = 2.0 * c.tile.bm * c.tile.bn * static_cast<double>(ksteps) * c.tile.bk;
  const double slots = cus * c.wgs_per_cu;
  // with at most four k-steps a workgroup is all fill and drain: the small tiles then run at
  // the same rate, and the one that pads less wins (the second convolution's input gradient,
  // 288 rows and K = 64: 27.1 us with 64x64 tiles, 24.8 us with 32x64)
  const double rate = (ksteps <= 4 && c.tile.bm * c.tile.bn <= 64 * 64) ? 105.0 : c.rate;
  const double round_us = slots * wg_flops / (rate * 1e6);
  const int64_t full = wgs / static_cast<int64_t>(slots);
  const int64_t rest = wgs - full * static_cast<int64_t>(slots);
  double us = static_cast<double>(full) * round_us;
  if (rest > 0) {
    double per_cu = static_cast<double>(ceil_div(rest, static_cast<int64_t>(cus))) / c.wgs_per_cu;
    us += round_us * std::max(per_cu, c.alone / c.wgs_per_cu * 1.0);
  }
  // a workgroup cannot finish faster than its k-steps' dependent load latencies allow
  // (measured: 49 steps of a lone 64x64 workgroup take 40 us)
  const double rounds = std::ceil(static_cast<double>(wgs) / slots);
  us = std::max(us, rounds * static_cast<double>(ksteps) * c.step_us);
  us += 2.0;   // prologue, epilogue, launch
  if (split > 1) us += 3.0 + (split + 1.0) * 4.0 * static_cast<double>(s.batch * s.M * s.N) / 4e6;
  return us;
}

// Tile and K split for a contraction.
bool choose(const GemmShape& s, const GenOptions& opt, Choice* out, bool computed_operand = false) {
  if (s.K < 8 || s.M < 2 || s.N < 2) return false;
  // the batch rides on blockIdx.z (at most 65535 workgroups); the tiles of one batch on blockIdx.x.
  // Beyond either the contraction is left to the other reduce schedules.
  if (s.batch > 65535 || ceil_div(s.M, 32) * ceil_div(s.N, 32) >= (int64_t{1} << 31)) return false;
  Choice best;
  if (opt.gemm_bm > 0) {
    best.tile = Tile{opt.gemm_bm, opt.gemm_bn, opt.gemm_bk, opt.gemm_wm, opt.gemm_wn};
    if (!tile_valid(best.tile)) return false;
    int64_t ksteps = ceil_div(s.K, best.tile.bk);
    if (opt.gemm_split_k > 1) best.split_k = static_cast<int>(std::min<int64_t>(opt.gemm_split_k, ksteps));
    *out = best;
    return true;
  }
  double best_us = 0;
  bool have = false;
  for (const auto& c : kCandidates) {
    // an operand evaluated in the tile loader (index decode, guards) slows every k-step of a
    // workgroup down; many small workgroups hide that, a few large ones do not (measured: a
    // 3x3 convolution over [32,128,28,28], 64x64 tiles 142 us, 128x128 295 us, 256x256 380 us)
    if (computed_operand && c.tile.bm * c.tile.bn > 64 * 64) continue;
    if (c.tile.bm * c.tile.bn == 32 * 32 && (s.M > 32 || s.N > 32)) continue;
    const int64_t ksteps = ceil_div(s.K, c.tile.bk);
    for (int split : {1, 2, 4, 8, 16, 32, 64, 128, 256}) {
      if (split > 1 && (opt.gemm_split_k == 0 || opt.gemm_split_k == 1)) break;
      if (opt.gemm_split_k > 1 && split != 1) break;
      // a split of the planner's own keeps at least eight k-steps per chunk -- two where the
      // whole result is at most four small tiles, K is split anyway and the k-steps' dependent
      // loads are all there is to wait for (a 128 x 10 weight gradient over a batch of 256: 7.9 us in two chunks, 4 us in
      // eight) -- and a requested one two
      const bool few = s.M * s.N * s.batch <= 4 * 64 * 64 && ksteps >= 16;
      const int64_t least = opt.gemm_split_k > 1 || few ? 2 : 8;
      int sp = opt.gemm_split_k > 1
                   ? static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(opt.gemm_split_k, ksteps / 2)))
                   : split;
      if (sp > 1 && ksteps / sp < least) break;
      double us = estimate_us(s, c, sp);
      if (!have || us < best_us) {
        have = true;
        best_us = us;
        best.tile = c.tile;
        best.split_k = sp;
      }
    }
  }
  *out = best;
  return have;
}

// Whether an operand can be read with aligned 128-bit loads along its unit-stride axis.
bool vec_ok(int64_t unit_extent, int64_t s_unit, int64_t s_other, int64_t off, int64_t bs) {
  return s_unit == 1 && unit_extent % 4 == 0 && s_other % 4 == 0 && off % 4 == 0 && bs % 4 == 0;
}

struct VarUse {
  std::string var;
  int64_t extent;
};

// Merges neighbouring loop variables (outer, inner) that every given affine index walks as
// one longer axis: stride(outer) == extent(inner) * stride(inner).
void collapse(std::vector<VarUse>* vars, const std::vector<Affine*>& affs) {
  for (size_t i = 0; i + 1 < vars->size();) {
    const VarUse &o = (*vars)[i], &in = (*vars)[i + 1];
    bool ok = true;
    for (const Affine* a : affs) ok = ok && a->of(o.var) == in.extent * a->of(in.var);
    if (!ok) {
      ++i;
      continue;
    }
    // the merged axis keeps the inner variable's name and stride
    for (Affine* a : affs) a->coef.erase(o.var);
    (*vars)[i + 1].extent *= o.extent;
    vars->erase(vars->begin() + static_cast<long>(i));
  }
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
  Affine ac = *k.out_aff;
  const std::string& kv = k.rloop.var;
  if (aa->of(kv) <= 0 || ab->of(kv) <= 0 || k.rloop.extent < 2) return std::nullopt;
  // output loops by which operands they index: A only -> rows, B only -> columns, both -> batch
  std::vector<VarUse> mv, nv, bv;
  for (const auto& l : k.loops) {
    if (l.extent == 1) continue;
    bool in_a = aa->of(l.var) != 0, in_b = ab->of(l.var) != 0;
    if (ac.of(l.var) <= 0) return std::nullopt;
    if (in_a && aa->of(l.var) < 0) return std::nullopt;
    if (in_b && ab->of(l.var) < 0) return std::nullopt;
    if (in_a && !in_b) mv.push_back({l.var, l.extent});
    else if (in_b && !in_a) nv.push_back({l.var, l.extent});
    else if (in_a && in_b) bv.push_back({l.var, l.extent});
    else return std::nullopt;
  }
  collapse(&mv, {&*aa, &ac});
  collapse(&nv, {&*ab, &ac});
  collapse(&bv, {&*aa, &*ab, &ac});
  GemmShape s;
  // Two row (column) axes left: where the operand walks them as one axis and the inner extent
  // would leave every image's last tile ragged (196 pixels an image), they are one axis and only
  // C's address keeps the two extents (tiles run across images, none is padded per image) ...
  auto merge_for = [&](std::vector<VarUse>* v, Affine* op, int64_t* split, int64_t* outer_stride) {
    if (!bv.empty() || v->size() != 2) return false;
    const VarUse o = (*v)[0], in = (*v)[1];
    if (in.extent % 64 == 0 || op->of(o.var) != in.extent * op->of(in.var)) return false;
    *split = in.extent;
    *outer_stride = ac.of(o.var);
    op->coef.erase(o.var);
    (*v)[1].extent *= o.extent;
    v->erase(v->begin());
    return true;
  };
  if (merge_for(&mv, &*aa, &s.c_msplit, &s.c_m2) || merge_for(&nv, &*ab, &s.c_nsplit, &s.c_n2)) {
    // one axis now
  } else if (bv.empty() && mv.size() == 2) {
    // ... otherwise the outer one rides on the batch axis: the other operand simply does not
    // move with it
    bv.push_back(mv[0]);
    mv.erase(mv.begin());
  } else if (bv.empty() && nv.size() == 2) {
    bv.push_back(nv[0]);
    nv.erase(nv.begin());
  }
  if (mv.size() != 1 || nv.size() != 1 || bv.size() > 1) return std::nullopt;
  const std::string &mvar = mv[0].var, &nvar = nv[0].var;
  s.M = mv[0].extent; s.N = nv[0].extent; s.K = k.rloop.extent;
  s.a_buf = la->args[0]->name; s.b_buf = lb->args[0]->name; s.c_buf = k.out_buf;
  s.a_m = aa->of(mvar); s.a_k = aa->of(kv); s.a_off = aa->c;
  s.b_n = ab->of(nvar); s.b_k = ab->of(kv); s.b_off = ab->c;
  s.c_m = ac.of(mvar); s.c_n = ac.of(nvar); s.c_off = ac.c;
  if (!bv.empty()) {
    s.batch = bv[0].extent;
    s.a_b = aa->of(bv[0].var); s.b_b = ab->of(bv[0].var); s.c_b = ac.of(bv[0].var);
  }
  if (s.a_off < 0 || s.b_off < 0 || s.c_off < 0) return std::nullopt;
  if (s.c_n != 1 && s.c_m == 1) {
    // C is column-major: compute C^T = B^T A^T instead, which is row-major
    GemmShape t = s;
    t.M = s.N; t.N = s.M;
    t.a_buf = s.b_buf; t.b_buf = s.a_buf;
    t.a_m = s.b_n; t.a_k = s.b_k; t.a_off = s.b_off; t.a_b = s.b_b;
    t.b_n = s.a_m; t.b_k = s.a_k; t.b_off = s.a_off; t.b_b = s.a_b;
    t.c_m = s.c_n; t.c_n = s.c_m;
    t.c_msplit = s.c_nsplit; t.c_m2 = s.c_n2; t.c_nsplit = s.c_msplit; t.c_n2 = s.c_m2;
    return t;
  }
  return s;
}

bool gemm_output_dense(const GemmShape& s) {
  return s.c_off == 0 && s.c_n == 1 && s.c_m == s.N && (s.batch == 1 || s.c_b == s.M * s.N) && !s.c_msplit && !s.c_nsplit;
}

bool gemm_shaped(const NestKernel& k, const GenOptions& opt) {
  auto s = match_gemm(k);
  Choice c;
  return s && choose(*s, opt, &c);
}

namespace {

// A computed operand whose producer only copies through a view (one unguarded load at an affine
// index) is, where the contraction's axes line up with the producer's loops, an ordinary strided
// operand in the producer's source: offset and strides of (batch, row, k) there, so that it is
// read with the plain (possibly 128-bit) loads instead of an element function.  Each axis must
// cover exactly a run of the producer's loops (no carry into other digits), the runs must not
// overlap, the offset must not reach into them, and along each axis the source address must be
// linear (checked over the whole axis).
// offset of the last row of an axis of `rows` rows (stride sr, or two nested extents)
int64_t row_reach(int64_t rows, int64_t sr, int64_t split, int64_t sr2) {
  if (!split) return (rows - 1) * sr;
  return (rows / split - 1) * sr2 + (split - 1) * sr;
}

struct PlainOperand {
  int64_t off, bs, sr, sk;
  int64_t rsplit = 0, sr2 = 0;      // the row axis in two nested extents: rows per inner extent, outer stride
};
std::optional<PlainOperand> plain_operand(const FoldedOperand& f, int64_t off, int64_t bs, int64_t sr, int64_t sk, int64_t batch,
                                          int64_t rows, int64_t kext) {
  if (!f.plain) return std::nullopt;
  auto address = [&](int64_t i) {
    int64_t a = f.src_off;
    for (const auto& l : f.loops) {
      if (l.extent <= 1) continue;
      auto it = f.src_stride.find(l.stride);
      a += ((i / l.stride) % l.extent) * (it == f.src_stride.end() ? 0 : it->second);
    }
    return a;
  };
  struct Axis { int64_t s, e, sigma; };
  Axis axes[3] = {{bs, batch, 0}, {sr, rows, 0}, {sk, kext, 0}};
  int64_t rsplit = 0, sr2 = 0;
  std::vector<std::pair<int64_t, int64_t>> spans;      // [s, s*e) of every moving axis
  for (auto& ax : axes) {
    if (ax.e <= 1) continue;
    if (ax.s <= 0) return std::nullopt;
    int64_t lo = 0, prod = 1;
    for (const auto& l : f.loops) {
      if (l.extent <= 1 || l.stride < ax.s || l.stride >= ax.s * ax.e) continue;
      if (l.stride * l.extent > ax.s * ax.e) return std::nullopt;
      lo = lo == 0 ? l.stride : std::min(lo, l.stride);
      prod *= l.extent;
    }
    if (lo != ax.s || prod != ax.e) return std::nullopt;
    if ((off / ax.s) % ax.e != 0) return std::nullopt;
    for (const auto& sp : spans)
      if (ax.s < sp.second && sp.first < ax.s * ax.e) return std::nullopt;
    spans.push_back({ax.s, ax.s * ax.e});
    ax.sigma = address(off + ax.s) - address(off);
    int64_t first_bad = 0;
    for (int64_t j = 0; j < ax.e && !first_bad; ++j)
      if (address(off + j * ax.s) - address(off) != j * ax.sigma) first_bad = j;
    if (!first_bad) continue;
    // the row axis may run over two nested extents (pixels inside images): linear inside, one
    // more stride between them
    if (&ax != &axes[1] || ax.e % first_bad) return std::nullopt;
    rsplit = first_bad;
    sr2 = address(off + rsplit * ax.s) - address(off);
    for (int64_t j = 0; j < ax.e; ++j)
      if (address(off + j * ax.s) - address(off) != (j / rsplit) * sr2 + (j % rsplit) * ax.sigma) return std::nullopt;
  }
  PlainOperand p{address(off), axes[0].sigma, axes[1].sigma, axes[2].sigma, rsplit, sr2};
  if (p.off < 0 || p.sr < 0 || p.sk < 0 || p.bs < 0 || p.sr2 < 0) return std::nullopt;
  return p;
}

}  // namespace

std::vector<LaunchSpec> try_emit_gemm(const NestKernel& k, const GenOptions& opt, std::vector<BufferInfo>* buffers,
                                      const FoldMap* folded, const EpilogueSpec* epilogue) {
  auto s = match_gemm(k);
  Choice ch;
  if (!s) return {};
  const FoldedOperand* fa = nullptr;
  const FoldedOperand* fb = nullptr;
  if (folded) {
    auto ia = folded->find(s->a_buf), ib = folded->find(s->b_buf);
    if (ia != folded->end()) fa = &ia->second;
    if (ib != folded->end()) fb = &ib->second;
  }
  std::string plain_tag;
  if (fa)
    if (auto p = plain_operand(*fa, s->a_off, s->a_b, s->a_m, s->a_k, s->batch, s->M, s->K)) {
      s->a_buf = fa->src; s->a_off = p->off; s->a_b = p->bs; s->a_m = p->sr; s->a_k = p->sk;
      s->a_msplit = p->rsplit; s->a_m2 = p->sr2;
      fa = nullptr;
      plain_tag += ",A:source";
    }
  if (fb)
    if (auto p = plain_operand(*fb, s->b_off, s->b_b, s->b_n, s->b_k, s->batch, s->N, s->K)) {
      s->b_buf = fb->src; s->b_off = p->off; s->b_b = p->bs; s->b_n = p->sr; s->b_k = p->sk;
      s->b_nsplit = p->rsplit; s->b_n2 = p->sr2;
      fb = nullptr;
      plain_tag += ",B:source";
    }
  if (opt.gemm_window && (fa != nullptr) != (fb != nullptr) && opt.gemm_bm == 0 && opt.gemm_split_k <= 1) {
    auto w = try_emit_window_gemm(k, *s, fa, fb, opt, epilogue);
    if (!w.empty()) return w;
  }
  if (!choose(*s, opt, &ch, fa || fb)) return {};
  const Tile& t = ch.tile;
  // each thread fetches four elements along the operand's faster axis
  bool a_kc = s->a_k <= s->a_m, b_nc = s->b_n <= s->b_k;
  // a computed operand is walked along whichever of its axes is contiguous in the memory its
  // producer reads (rows when both are or neither is known)
  auto along_k = [](const FoldedOperand& f, int64_t s_row, int64_t s_k) {
    auto ir = f.src_stride.find(s_row), ik = f.src_stride.find(s_k);
    int64_t r = ir == f.src_stride.end() ? 0 : std::llabs(ir->second);
    int64_t kk = ik == f.src_stride.end() ? 0 : std::llabs(ik->second);
    return kk != 0 && (r == 0 || kk < r);
  };
  if (fa) a_kc = along_k(*fa, s->a_m, s->a_k);
  if (fb) b_nc = !along_k(*fb, s->b_n, s->b_k);
  // (a split row axis: vectors along the rows must not straddle two inner extents)
  const bool a_split_ok = !s->a_msplit || (s->a_m2 % 4 == 0 && (a_kc || s->a_msplit % 4 == 0));
  const bool b_split_ok = !s->b_nsplit || (s->b_n2 % 4 == 0 && (!b_nc || s->b_nsplit % 4 == 0));
  const bool a_vec = !fa && a_split_ok && (a_kc ? vec_ok(s->K, s->a_k, s->a_m, s->a_off, s->a_b) : vec_ok(s->M, s->a_m, s->a_k, s->a_off, s->a_b));
  const bool b_vec = !fb && b_split_ok && (b_nc ? vec_ok(s->N, s->b_n, s->b_k, s->b_off, s->b_b) : vec_ok(s->K, s->b_k, s->b_n, s->b_off, s->b_b));
  const int S = ch.split_k;
  std::vector<LaunchSpec> out(S > 1 ? 2 : 1);
  LaunchSpec& ls = out[0];
  ls.entry = "ehk_" + k.name + (S > 1 ? "_part" : "");
  ls.kernels = {k.name};
  const int nt = (t.bm / t.wm) * (t.bn / t.wn) * 64;
  const std::string scratch = "eh_part_" + k.name;
  std::ostringstream os;
  std::string dma_tag;
  os << "// generated for gfx950 by eclat backend-hip: MFMA contraction\n";
  os << "#define EH_ENTRY " << ls.entry << "\n";
  os << "#define EH_M " << s->M << "\n#define EH_N " << s->N << "\n#define EH_K " << s->K << "\n#define EH_BATCH "
     << s->batch << "\n";
  os << "#define EH_BM " << t.bm << "\n#define EH_BN " << t.bn << "\n#define EH_BK " << t.bk << "\n#define EH_WM "
     << t.wm << "\n#define EH_WN " << t.wn << "\n";
  os << "#define EH_A_KCONTIG " << (a_kc ? 1 : 0) << "\n#define EH_B_NCONTIG " << (b_nc ? 1 : 0) << "\n";
  os << "#define EH_A_VEC " << (a_vec ? 1 : 0) << "\n#define EH_B_VEC " << (b_vec ? 1 : 0) << "\n";
  {
    // direct-to-LDS loads: row-contiguous operand, 128-bit loads, no guards needed on its tile
    const bool k_exact = s->K % t.bk == 0 && ((s->K / t.bk) % ch.split_k) == 0;
    const bool a_dma = (opt.gemm_dma == 1 || opt.gemm_dma == 3) && !a_kc && a_vec && k_exact && s->M % t.bm == 0 && !s->a_msplit;
    const bool b_dma = (opt.gemm_dma == 1 || opt.gemm_dma == 2) && b_nc && b_vec && k_exact && s->N % t.bn == 0 && !s->b_nsplit;
    os << "#define EH_A_DMA " << (a_dma ? 1 : 0) << "\n#define EH_B_DMA " << (b_dma ? 1 : 0) << "\n";
    dma_tag = std::string(a_dma ? ",A>lds" : "") + (b_dma ? ",B>lds" : "");
  }
  os << "#define EH_A_SM " << s->a_m << "LL\n#define EH_A_SK " << s->a_k << "LL\n";
  os << "#define EH_B_SK " << s->b_k << "LL\n#define EH_B_SN " << s->b_n << "LL\n";
  os << "#define EH_C_SM " << s->c_m << "LL\n#define EH_C_SN " << s->c_n << "LL\n";
  os << "#define EH_A_OFF " << s->a_off << "LL\n#define EH_B_OFF " << s->b_off << "LL\n#define EH_C_OFF " << s->c_off
     << "LL\n";
  os << "#define EH_A_BS " << s->a_b << "LL\n#define EH_B_BS " << s->b_b << "LL\n#define EH_C_BS " << s->c_b << "LL\n";
  os << "#define EH_A_MSPLIT " << s->a_msplit << "LL\n#define EH_A_SM2 " << s->a_m2 << "LL\n";
  os << "#define EH_B_NSPLIT " << s->b_nsplit << "LL\n#define EH_B_SN2 " << s->b_n2 << "LL\n";
  os << "#define EH_C_MSPLIT " << s->c_msplit << "LL\n#define EH_C_SM2 " << s->c_m2 << "LL\n";
  os << "#define EH_C_NSPLIT " << s->c_nsplit << "LL\n#define EH_C_SN2 " << s->c_n2 << "LL\n";
  os << "#define EH_SPLITK " << S << "\n";
  os << "#define EH_GROUP_M 8\n";
  // A computed operand's element (row r, k) sits at off + bz*bs + r*sr + k*sk of the producer's
  // output.  Split that index at Q (a boundary between the producer's loops): when the row part
  // only moves the quotient and the k part only the remainder (mode 1), or the other way round
  // (mode 2), the part that belongs to the row is the same for every k step, and the compiler
  // hoists its decode out of the k loop; no division by Q is needed either.
  auto emit_fold = [&](const FoldedOperand* f, const char* X, const char* /*fn*/, int64_t off, int64_t bs, int64_t sr,
                       int64_t sk, int64_t rows, int64_t kext) {
    if (!f) return;
    int64_t total = 1;
    for (const auto& l : f->loops) total *= l.extent;
    auto boundary = [&](int64_t q) {
      for (const auto& l : f->loops)
        if (l.stride == q) return true;
      return q == total;
    };
    int mode = 0;
    int64_t Q = total;
    if (sr > 0 && boundary(sr) && off % sr == 0 && bs % sr == 0 && kext * sk <= sr) {
      mode = 1;
      Q = sr;
    } else if (sk > 0 && boundary(sk) && off % sk == 0 && bs % sk == 0 && rows * sr <= sk) {
      mode = 2;
      Q = sk;
    }
    const std::string IT = f->small ? "int" : "long long";
    os << "#define EH_" << X << "_FOLD 1\n#define EH_" << X << "_FOLD_MODE " << mode << "\n#define EH_" << X << "_FOLD_Q " << Q
       << "LL\n";
    if (f->ranged_bytes)
      os << "#ifndef EH_RANGED_LOAD\n#define EH_RANGED_LOAD 1\n// one fp32 at a byte offset into a buffer resource; zero beyond the resource's size\n"
            "__device__ __forceinline__ float eh_ranged_load(__amdgpu_buffer_rsrc_t r, unsigned byte_offset) {\n"
            "  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, byte_offset, 0, 0));\n}\n#endif\n";
    os << f->prelude;
    // The element at index eh_U * Q + eh_I of what the producer would have written: its loop
    // variables above Q are decoded from eh_U, those below from eh_I, each by a function of its
    // own, so that the caller decodes the half that belongs to the row once and the half that
    // belongs to k once per k.
    const std::string P = std::string("eh_") + static_cast<char>(std::tolower(X[0]));
    std::ostringstream up, lo, dup, dlo, use;
    for (const auto& l : f->loops) {
      if (l.extent == 1) {
        use << "  const " << IT << " " << l.name << " = 0;\n";
      } else if (l.stride >= Q) {
        up << "  " << IT << " " << l.name << ";\n";
        dup << "  r." << l.name << " = (" << IT << ")((eh_U / " << l.stride / Q << "u) % " << l.extent << "u);\n";
        use << "  const " << IT << " " << l.name << " = eh_u." << l.name << ";\n";
      } else {
        lo << "  " << IT << " " << l.name << ";\n";
        dlo << "  r." << l.name << " = (" << IT << ")((eh_I / " << l.stride << "u) % " << l.extent << "u);\n";
        use << "  const " << IT << " " << l.name << " = eh_l." << l.name << ";\n";
      }
      // the guards of a padded gather repeat what the loops' extents already say: let the compiler drop those
      if (l.extent > 1) use << "  __builtin_assume(" << l.name << " >= 0 && " << l.name << " < " << l.extent << ");\n";
    }
    os << "// element (eh_U * " << Q << " + eh_I) of what kernel " << f->kernel << " would have written\n";
    os << "struct " << P << "_upper {\n" << up.str() << "};\nstruct " << P << "_lower {\n" << lo.str() << "};\n";
    // (indices are never negative: unsigned division by a constant is the cheaper one)
    const std::string UT = f->small ? "unsigned" : "unsigned long long";
    os << "__device__ __forceinline__ " << P << "_upper " << P << "_dec_upper(long long eh_U64) {\n  const " << UT << " eh_U = ("
       << UT << ")eh_U64;\n  (void)eh_U;\n  " << P << "_upper r;\n" << dup.str() << "  return r;\n}\n";
    os << "__device__ __forceinline__ " << P << "_lower " << P << "_dec_lower(long long eh_I64) {\n  const " << UT << " eh_I = ("
       << UT << ")eh_I64;\n  (void)eh_I;\n  " << P << "_lower r;\n" << dlo.str() << "  return r;\n}\n";
    os << "__device__ __forceinline__ float " << P << "_val(const float* __restrict__ " << f->src << ", const " << P
       << "_upper& eh_u, const " << P << "_lower& eh_l) {\n  (void)eh_u;\n  (void)eh_l;\n" << use.str();
    if (f->ranged_bytes)
      os << "  const __amdgpu_buffer_rsrc_t eh_rs_" << f->src << " = __builtin_amdgcn_make_buffer_rsrc((void*)" << f->src << ", 0, "
         << f->ranged_bytes << ", 0x00020000);\n";
    os << "  return (float)(" << f->expr << ");\n}\n";
  };
  const bool epi_here = epilogue && S == 1;     // with K split the epilogue runs in the summing launch
  if (epi_here) {
    os << "#define EH_EPILOGUE 1\n#define EH_EPI_PARAMS " << epilogue->params << "\n#define EH_EPI_ARGS " << epilogue->args
       << "\n";
    if (!epilogue->store_c) os << "#define EH_NO_C 1\n";
    os << epilogue->function;
  }
  emit_fold(fa, "A", "eh_a_elem", s->a_off, s->a_b, s->a_m, s->a_k, s->M, s->K);
  emit_fold(fb, "B", "eh_b_elem", s->b_off, s->b_b, s->b_n, s->b_k, s->N, s->K);
  {
    // register budget: 512 lanes' registers per SIMD shared by the resident waves; a wave needs
    // its accumulators (wm*wn/64) plus about 56 for operands, staging and addresses
    int waves = 8;
    while (waves > 1 && 512 / waves < t.wm * t.wn / 64 + 56) waves /= 2;
    if (opt.gemm_waves > 0) waves = opt.gemm_waves;
    os << "#define EH_WAVES_PER_SIMD " << std::min(8, waves) << "\n";
  }
  os << "#define EH_SETPRIO " << std::max(0, std::min(3, opt.gemm_setprio)) << "\n";
  os << "#define EH_MIX " << (opt.gemm_mix ? 1 : 0) << "\n";
  {
    // small tiles multiply for a fraction of a load's latency: their loads leave three steps ahead
    int pf = opt.gemm_prefetch > 0 ? opt.gemm_prefetch : (t.bm * t.bn <= 64 * 64 ? 3 : 1);
    if (pf > 1 && pf % 2 == 0) ++pf;            // stages = prefetch + 1 must be even
    os << "#define EH_PREFETCH " << pf << "\n";
  }
  os << "#define EH_TRANSPOSE " << (opt.gemm_transpose ? 1 : 0) << "\n";
  os << "#define EH_LOAD_BRANCH " << (opt.guard_branches ? 1 : 0) << "\n";
  os << kGemmSource;
  ls.source = os.str();
  ls.part_params = std::string("const float* __restrict__ A, const float* __restrict__ B") +
                   (epi_here && !epilogue->store_c ? "" : ", float* __restrict__ C") + (epi_here ? epilogue->params : "");
  const bool ragged = s->M % t.bm || s->N % t.bn || s->K % t.bk;
  ls.schedule = "mfma32x32x2(tile=" + std::to_string(t.bm) + "x" + std::to_string(t.bn) + "x" + std::to_string(t.bk) +
                ",wave=" + std::to_string(t.wm) + "x" + std::to_string(t.wn) + (a_kc ? ",A:k" : ",A:m") +
                (fa ? "/folded" : a_vec ? "" : "/scalar") + (b_nc ? ",B:n" : ",B:k") +
                (fb ? "/folded" : b_vec ? "" : "/scalar") +
                plain_tag + dma_tag + (s->c_msplit || s->c_nsplit ? ",C:split" : "") + (ragged ? ",edges" : "") + (S > 1 ? ",split-k=" + std::to_string(S) : "") +
                (epi_here ? ",epilogue=" + std::to_string(epilogue->kernels.size()) : "") + ")";
  ls.grid[0] = static_cast<unsigned>(ceil_div(s->M, t.bm) * ceil_div(s->N, t.bn));
  ls.grid[1] = static_cast<unsigned>(S);
  ls.grid[2] = static_cast<unsigned>(s->batch);
  ls.block[0] = static_cast<unsigned>(nt);
  const size_t c_elems =
      static_cast<size_t>(s->c_off + row_reach(s->M, s->c_m, s->c_msplit, s->c_m2) + row_reach(s->N, s->c_n, s->c_nsplit, s->c_n2) +
                          (s->batch - 1) * s->c_b + 1);
  const size_t part_elems = static_cast<size_t>(S) * static_cast<size_t>(s->batch * s->M * s->N);
  ls.arg_bufs = {fa ? fa->src : s->a_buf, fb ? fb->src : s->b_buf};
  // a folded operand binds the producer's source, whose size the buffer table already fixes
  ls.arg_min_bytes = {
      fa ? 0 : 4 * static_cast<size_t>(s->a_off + row_reach(s->M, s->a_m, s->a_msplit, s->a_m2) + (s->K - 1) * s->a_k + (s->batch - 1) * s->a_b + 1),
      fb ? 0 : 4 * static_cast<size_t>(s->b_off + (s->K - 1) * s->b_k + row_reach(s->N, s->b_n, s->b_nsplit, s->b_n2) + (s->batch - 1) * s->b_b + 1)};
  if (!(epi_here && !epilogue->store_c)) {
    ls.arg_bufs.push_back(S > 1 ? scratch : s->c_buf);
    ls.arg_min_bytes.push_back(4 * (S > 1 ? part_elems : c_elems));
  }
  if (epi_here) {
    for (size_t i = 0; i < epilogue->bufs.size(); ++i) {
      ls.arg_bufs.push_back(epilogue->bufs[i]);
      ls.arg_min_bytes.push_back(epilogue->min_bytes[i]);
    }
    for (const auto& n : epilogue->kernels) ls.kernels.push_back(n);
  }
  ls.flops = 2.0 * static_cast<double>(s->M) * static_cast<double>(s->N) * static_cast<double>(s->K) *
             static_cast<double>(s->batch);
  {
    // an operand the batch does not move (stride 0) is read once, not once per batch
    const double nb = static_cast<double>(s->batch);
    double a_bytes = 4.0 * static_cast<double>(s->M) * s->K * (s->a_b == 0 ? 1.0 : nb);
    double b_bytes = 4.0 * static_cast<double>(s->K) * s->N * (s->b_b == 0 ? 1.0 : nb);
    if (fa && fa->src_bytes > 0) a_bytes = fa->src_bytes;
    if (fb && fb->src_bytes > 0) b_bytes = fb->src_bytes;
    const double c_bytes = 4.0 * nb * static_cast<double>(s->M) * s->N;
    ls.algo_bytes = a_bytes + b_bytes + (epilogue && !epilogue->store_c ? 0.0 : c_bytes) + (epilogue ? epilogue->bytes : 0.0);
  }
  if (S > 1) {
    BufferInfo sb;
    sb.name = scratch;
    sb.dtype = k.out_dtype;
    sb.shape = {S, s->batch, s->M, s->N};
    sb.role = "temp";
    buffers->push_back(sb);
    // second launch: C[b,m,n] = sum over splits, in split order (deterministic)
    LaunchSpec& fin = out[1];
    fin.entry = "ehk_" + k.name;
    fin.kernels = {k.name};
    fin.schedule = "split-k-final(chunks=" + std::to_string(S) + ")";
    const int64_t total = s->batch * s->M * s->N;
    fin.grid[0] = static_cast<unsigned>(ceil_div(total, 256));
    fin.block[0] = 256;
    const bool fin_c = !(epilogue && !epilogue->store_c);
    fin.arg_bufs = {scratch};
    fin.arg_min_bytes = {4 * part_elems};
    if (fin_c) {
      fin.arg_bufs.push_back(s->c_buf);
      fin.arg_min_bytes.push_back(4 * c_elems);
    }
    std::ostringstream fs;
    fs << kernel_header() << "// sum of split-K partial tiles\n";
    if (epilogue) {
      fs << epilogue->function;
      for (size_t i = 0; i < epilogue->bufs.size(); ++i) {
        fin.arg_bufs.push_back(epilogue->bufs[i]);
        fin.arg_min_bytes.push_back(epilogue->min_bytes[i]);
      }
      for (const auto& n : epilogue->kernels) fin.kernels.push_back(n);
      fin.schedule = "split-k-final(chunks=" + std::to_string(S) + ",epilogue=" + std::to_string(epilogue->kernels.size()) + ")";
    }
    fs << "extern \"C\" __global__ void __launch_bounds__(256) " << fin.entry << "(const float* __restrict__ P"
       << (fin_c ? ", float* __restrict__ C" : "") << (epilogue ? epilogue->params : std::string()) << ") {\n";
    fs << "  const long long o = (long long)blockIdx.x * 256 + threadIdx.x;\n  if (o >= " << total << "LL) return;\n";
    fs << "  float acc = 0.0f;\n  for (int s = 0; s < " << S << "; ++s) acc += P[(long long)s * " << total << "LL + o];\n";
    fs << "  const long long n = o % " << s->N << "LL, m = (o / " << s->N << "LL) % " << s->M << "LL, b = o / "
       << (s->M * s->N) << "LL;\n";
    auto axis = [](const char* v, int64_t stride, int64_t split, int64_t outer) {
      std::ostringstream a;
      if (split) a << "(" << v << " / " << split << "LL) * " << outer << "LL + (" << v << " % " << split << "LL) * " << stride << "LL";
      else a << v << " * " << stride << "LL";
      return a.str();
    };
    fs << "  const long long e = " << s->c_off << "LL + b * " << s->c_b << "LL + " << axis("m", s->c_m, s->c_msplit, s->c_m2) << " + "
       << axis("n", s->c_n, s->c_nsplit, s->c_n2) << ";\n";
    if (epilogue) {
      // the epilogue takes the address of the element in C's layout
      fs << "  eh_epilogue(e, acc" << (epilogue->store_c ? ", C" : "") << epilogue->args << ");\n}\n";
    } else {
      fs << "  C[e] = acc;\n}\n";
    }
    fin.source = fs.str();
  }
  return out;
}

}  // namespace eh
