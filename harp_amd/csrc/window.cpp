#include "window.hpp"

#include <algorithm>
#include <cstdlib>
#include <map>
#include <set>
#include <sstream>

namespace eh {

namespace {

// The kernel text is kept in kernels/window_f32_mfma.hip and wrapped into a raw string literal
// by the build.
const char* kWindowSource =
#include "kernels/window_f32_mfma.hip.inc"
    ;

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

enum Side { kBatch = 0, kRow = 1, kK = 2 };

// One loop of the folded gather: which axis of the contraction it belongs to, its unit there
// (the index along that axis moves by `unit` per step of the loop), its stride in the source.
struct WLoop {
  std::string name;
  int64_t extent = 1, ostride = 0, sstride = 0, unit = 0;
  Side side = kRow;
  int axis = -1;          // patch axis (loops inside the workgroup), or -1
  bool in_wg = false;
};

// One coordinate of the patch: a source axis walked by one loop, or by the sum of a row loop and
// a window loop (same stride in the source).
struct PAxis {
  int64_t sstride = 0, extent = 1, lds = 0;
  int64_t lo = 0, hi = 0;     // coordinates in [lo, hi) exist in the source; the rest is padding
};

// e >= bound (ge) or e < bound, e an affine form over the gather's loops without constant term
struct Atom {
  Affine e;
  bool ge = false;
  int64_t bound = 0;
};

bool collect_atoms(const Node& c, std::vector<Atom>* out) {
  if (c.op == Op::And || c.op == Op::BitAnd) return collect_atoms(*c.args[0], out) && collect_atoms(*c.args[1], out);
  const Node* lt = &c;
  bool neg = false;
  if (c.op == Op::Not && c.args[0]->op == Op::Lt) {
    lt = c.args[0].get();
    neg = true;
  }
  if (lt->op != Op::Lt) return false;
  auto l = affine_of(*lt->args[0]);
  auto r = affine_of(*lt->args[1]);
  if (!l || !r) return false;
  // l < r  <=>  (l - r without constants) < r.c - l.c
  Atom a;
  a.e = *l;
  for (const auto& kv : r->coef) a.e.coef[kv.first] -= kv.second;
  a.bound = r->c - l->c;
  a.e.c = 0;
  a.ge = neg;
  for (auto it = a.e.coef.begin(); it != a.e.coef.end();)
    it = it->second == 0 ? a.e.coef.erase(it) : std::next(it);
  out->push_back(a);
  return true;
}

struct Layout {
  int waves_m = 1, waves_n = 1, mb = 1, nb = 1;
};

}  // namespace

std::vector<LaunchSpec> try_emit_window_gemm(const NestKernel& k, const GemmShape& s_in, const FoldedOperand* fa,
                                             const FoldedOperand* fb, const GenOptions& opt, const EpilogueSpec* epilogue) {
  if ((fa != nullptr) == (fb != nullptr)) return {};
  // the folded operand takes the column side: C^T = F^T A^T when it came as A
  GemmShape s = s_in;
  const FoldedOperand* f = fb;
  if (fa) {
    f = fa;
    s.M = s_in.N; s.N = s_in.M;
    s.a_buf = s_in.b_buf; s.b_buf = s_in.a_buf;
    s.a_m = s_in.b_n; s.a_k = s_in.b_k; s.a_off = s_in.b_off; s.a_b = s_in.b_b;
    s.a_msplit = s_in.b_nsplit; s.a_m2 = s_in.b_n2;
    s.b_n = s_in.a_m; s.b_k = s_in.a_k; s.b_off = s_in.a_off; s.b_b = s_in.a_b;
    s.b_nsplit = s_in.a_msplit; s.b_n2 = s_in.a_m2;
    s.c_m = s_in.c_n; s.c_n = s_in.c_m;
    s.c_msplit = s_in.c_nsplit; s.c_m2 = s_in.c_n2; s.c_nsplit = s_in.c_msplit; s.c_n2 = s_in.c_m2;
  }
  if (!f->value || f->ranged_bytes == 0 || !f->small || !f->prelude.empty()) return {};
  if (s.b_off != 0 || s.b_nsplit != 0 || s.K < 4 || s.M < 2 || s.N < 2 || s.batch > 65535) return {};
  if (s.a_off < 0 || s.a_k <= 0 || s.a_m < 0) return {};

  // ---- the gather: load index and guard ----------------------------------------------------
  const Node* v = f->value.get();
  std::vector<Atom> atoms;
  if (v->op == Op::Select) {
    if (v->args[2]->op != Op::Const || v->args[2]->fval != 0.0 || !collect_atoms(*v->args[0], &atoms)) return {};
    v = v->args[1].get();
  }
  if (v->op != Op::Load || v->args[0]->op != Op::Var || v->args[0]->name != f->src) return {};
  auto idx = affine_of(*v->args[1]);
  if (!idx) return {};

  // ---- loops by contraction axis -------------------------------------------------------------
  std::vector<WLoop> loops;
  struct AxisRange { int64_t s, e; Side side; };
  const AxisRange ranges[3] = {{s.b_b, s.batch, kBatch}, {s.b_n, s.N, kRow}, {s.b_k, s.K, kK}};
  int64_t covered[3] = {1, 1, 1}, lowest[3] = {0, 0, 0};
  for (const auto& l : f->loops) {
    if (l.extent <= 1) {
      if (idx->of(l.name) != 0 && l.extent < 1) return {};
      continue;
    }
    WLoop w;
    w.name = l.name;
    w.extent = l.extent;
    w.ostride = l.stride;
    w.sstride = idx->of(l.name);
    if (w.sstride <= 0) return {};
    bool placed = false;
    for (const auto& r : ranges) {
      if (r.e <= 1 || r.s <= 0) continue;
      if (l.stride < r.s || l.stride >= r.s * r.e) continue;
      if (l.stride * l.extent > r.s * r.e || l.stride % r.s != 0) return {};
      w.side = r.side;
      w.unit = l.stride / r.s;
      covered[r.side] *= l.extent;
      lowest[r.side] = lowest[r.side] == 0 ? l.stride : std::min(lowest[r.side], l.stride);
      placed = true;
      break;
    }
    if (!placed) return {};
    loops.push_back(w);
  }
  for (const auto& r : ranges) {
    if (r.e <= 1) continue;
    if (covered[r.side] != r.e || lowest[r.side] != r.s) return {};
  }
  // every variable of the index is one of these loops
  for (const auto& kv : idx->coef) {
    if (kv.second == 0) continue;
    bool known = false;
    for (const auto& l : f->loops) known = known || l.name == kv.first;
    if (!known) return {};
  }
  auto find_loop = [&](const std::string& name) -> WLoop* {
    for (auto& w : loops)
      if (w.name == name) return &w;
    return nullptr;
  };

  // ---- patch axes: loops grouped by their stride in the source ----------------------------------
  // outermost first within each side
  std::sort(loops.begin(), loops.end(), [](const WLoop& a, const WLoop& b) {
    return a.side != b.side ? a.side < b.side : a.ostride > b.ostride;
  });
  std::map<int64_t, std::vector<size_t>> by_stride;
  for (size_t i = 0; i < loops.size(); ++i) by_stride[loops[i].sstride].push_back(i);
  std::set<size_t> paired_rows;
  for (const auto& kv : by_stride) {
    const auto& g = kv.second;
    if (g.size() == 1) continue;
    if (g.size() != 2) return {};
    const WLoop &x = loops[g[0]], &y = loops[g[1]];
    if (!((x.side == kRow && y.side == kK) || (x.side == kK && y.side == kRow))) return {};
    paired_rows.insert(x.side == kRow ? g[0] : g[1]);
  }
  if (paired_rows.empty()) return {};      // no window: a plain strided operand, handled elsewhere

  // rows inside a workgroup: from some row loop inward, at least from the outermost window row loop
  std::vector<size_t> row_loops, k_loops, batch_loops;
  for (size_t i = 0; i < loops.size(); ++i)
    (loops[i].side == kRow ? row_loops : loops[i].side == kK ? k_loops : batch_loops).push_back(i);
  size_t first_needed = row_loops.size();
  for (size_t q = 0; q < row_loops.size(); ++q)
    if (paired_rows.count(row_loops[q])) {
      first_needed = q;
      break;
    }

  // ---- sub-k digit and the steps of the multiply loop ---------------------------------------------
  // the four k of a step run along a k loop whose extent is a multiple of four when there is one
  int sub = -1;
  for (size_t q = 0; q < k_loops.size(); ++q)
    if (loops[k_loops[q]].extent % 4 == 0 && (sub < 0 || loops[k_loops[q]].sstride > loops[k_loops[static_cast<size_t>(sub)]].sstride))
      sub = static_cast<int>(q);
  const int64_t kdelta = sub >= 0 ? loops[k_loops[static_cast<size_t>(sub)]].unit : 1;
  const int64_t ksteps = sub >= 0 ? s.K / 4 : ceil_div(s.K, 4);
  if (ksteps > 512) return {};
  std::vector<int64_t> k0(static_cast<size_t>(ksteps));
  if (sub >= 0) {
    // every combination of the other k digits, times the blocks of four of the sub digit
    std::vector<int64_t> digit(k_loops.size(), 0);
    for (int64_t st = 0; st < ksteps; ++st) {
      int64_t kk = 0;
      for (size_t q = 0; q < k_loops.size(); ++q)
        kk += digit[q] * loops[k_loops[q]].unit * (static_cast<int>(q) == sub ? 4 : 1);
      k0[static_cast<size_t>(st)] = kk;
      for (size_t q = k_loops.size(); q-- > 0;) {
        const int64_t lim = static_cast<int>(q) == sub ? loops[k_loops[q]].extent / 4 : loops[k_loops[q]].extent;
        if (++digit[q] < lim) break;
        digit[q] = 0;
      }
    }
  } else {
    for (int64_t st = 0; st < ksteps; ++st) k0[static_cast<size_t>(st)] = 4 * st;
  }

  // ---- choose how many row loops a workgroup takes, and the wave layout -----------------------------
  const int64_t mblk_all = ceil_div(s.M, 16);
  Layout lay;
  size_t first_in = row_loops.size();
  std::vector<PAxis> axes;
  int64_t NG = 0, patch_elems = 0;
  // Candidates from the largest group (fewest workgroups) to the smallest: the first that still
  // gives the chip a workgroup per CU is taken, else the one with the most workgroups.
  bool enough = false;
  for (size_t start = 0; start <= first_needed && !enough; ++start) {
    for (auto& w : loops) {
      w.in_wg = w.side == kK;
      w.axis = -1;
    }
    int64_t ng = 1;
    for (size_t q = start; q < row_loops.size(); ++q) {
      loops[row_loops[q]].in_wg = true;
      ng *= loops[row_loops[q]].extent;
    }
    if (ng > 4096) continue;
    // axes by source stride, largest first
    std::vector<PAxis> ax;
    bool ok = true;
    for (auto it = by_stride.rbegin(); it != by_stride.rend() && ok; ++it) {
      PAxis a;
      a.sstride = it->first;
      int64_t ext = 1;
      bool any = false;
      for (size_t i : it->second) {
        if (!loops[i].in_wg) {
          if (it->second.size() == 2) ok = false;     // a window pair split between workgroups
          continue;
        }
        ext += loops[i].extent - 1;
        any = true;
      }
      if (!any) continue;
      a.extent = ext;
      a.lo = 0;
      a.hi = ext;
      for (size_t i : it->second)
        if (loops[i].in_wg) loops[i].axis = static_cast<int>(ax.size());
      ax.push_back(a);
    }
    if (!ok || ax.empty()) continue;
    int64_t elems = 1;
    for (const auto& a : ax) elems *= a.extent;
    if (elems > 24576) continue;                       // 96 KiB of LDS at most
    // wave layout: M-blocks over the waves first, the N-blocks of the group over what is left
    Layout l;
    l.waves_m = mblk_all >= 4 ? 4 : mblk_all >= 2 ? 2 : 1;
    l.waves_n = 4 / l.waves_m;
    const int64_t nblk = ceil_div(ng, 16);
    if (nblk < l.waves_n) l.waves_n = static_cast<int>(std::max<int64_t>(1, nblk));
    l.mb = static_cast<int>(ceil_div(mblk_all, l.waves_m));
    l.nb = static_cast<int>(ceil_div(nblk, l.waves_n));
    // registers of a lane: accumulators, operand slots, row bases (a few patterns at most)
    const int64_t regs = 4LL * l.mb * l.nb + 2LL * (l.mb + l.nb) + 4LL * l.nb;
    if (regs > 400 || l.nb > 64) continue;
    // LDS: the patch and A's rows (K floats and a pad each)
    if ((elems + 64 + static_cast<int64_t>(l.waves_m) * l.mb * 16 * (ceil_div(s.K, 4) * 4 + 64)) * 4 > 150 * 1024) continue;
    first_in = start;
    lay = l;
    axes = ax;
    NG = ng;
    patch_elems = elems;
    enough = (s.N / ng) * s.batch >= 256;
  }
  if (first_in == row_loops.size() || NG < 4) return {};
  // restore the choice (the loop above leaves the last candidate's marks when it broke out early)
  for (auto& w : loops) {
    w.in_wg = w.side == kK;
    w.axis = -1;
  }
  for (size_t q = first_in; q < row_loops.size(); ++q) loops[row_loops[q]].in_wg = true;
  {
    size_t ai = 0;
    for (auto it = by_stride.rbegin(); it != by_stride.rend(); ++it) {
      bool any = false;
      for (size_t i : it->second) any = any || loops[i].in_wg;
      if (!any) continue;
      for (size_t i : it->second)
        if (loops[i].in_wg) loops[i].axis = static_cast<int>(ai);
      ++ai;
    }
  }

  // ---- guards: each atom bounds one patch coordinate (or repeats a loop's own extent) ------------
  for (const auto& a : atoms) {
    std::vector<WLoop*> vars;
    for (const auto& kv : a.e.coef) {
      WLoop* w = find_loop(kv.first);
      if (!w) {
        // a loop that runs once: contributes nothing
        bool once = false;
        for (const auto& l : f->loops) once = once || (l.name == kv.first && l.extent <= 1);
        if (!once) return {};
        continue;
      }
      if (kv.second != 1) return {};
      vars.push_back(w);
    }
    if (vars.empty()) {
      // a constant condition: must hold
      if (a.ge ? !(0 >= a.bound) : !(0 < a.bound)) return {};
      continue;
    }
    if (vars.size() == 1 && !vars[0]->in_wg) {
      // a loop outside the workgroup: only the trivial bound on its own extent is accepted
      if (a.ge ? a.bound > 0 : a.bound < vars[0]->extent) return {};
      continue;
    }
    if (vars.size() > 2) return {};
    if (vars.size() == 2 && (vars[0]->axis < 0 || vars[0]->axis != vars[1]->axis)) return {};
    if (vars[0]->axis < 0) return {};
    PAxis& ax = axes[static_cast<size_t>(vars[0]->axis)];
    // a bound on one loop of a pair axis alone cannot be expressed on the pair's coordinate
    int members = 0;
    for (const auto& w : loops) members += w.axis == vars[0]->axis ? 1 : 0;
    if (static_cast<int>(vars.size()) != members) {
      if (a.ge ? a.bound > 0 : a.bound < vars[0]->extent) return {};
      continue;
    }
    if (a.ge) ax.lo = std::max(ax.lo, a.bound);
    else ax.hi = std::min(ax.hi, a.bound);
  }
  for (const auto& a : axes)
    if (a.lo >= a.hi) return {};

  // ---- LDS layout of the patch: dense, outermost axis padded against bank conflicts ----------------
  auto set_strides = [&](int64_t pad) {
    int64_t st = 1;
    for (size_t i = axes.size(); i-- > 0;) {
      axes[i].lds = st + (i == 0 && axes.size() > 1 ? pad : 0);
      st = axes[i].lds * axes[i].extent;
    }
  };
  auto k_lds = [&](int64_t kk) {
    int64_t o = 0;
    for (size_t q : k_loops) {
      const WLoop& w = loops[q];
      o += ((kk / w.unit) % w.extent) * axes[static_cast<size_t>(w.axis)].lds;
    }
    return o;
  };
  auto row_lds = [&](int64_t n) {
    int64_t o = 0;
    for (size_t q = first_in; q < row_loops.size(); ++q) {
      const WLoop& w = loops[row_loops[q]];
      const int64_t unit_in = w.unit / loops[row_loops.back()].unit;    // unit relative to the group's first row
      o += ((n / unit_in) % w.extent) * axes[static_cast<size_t>(w.axis)].lds;
    }
    return o;
  };
  // the rows of a group are NG consecutive rows of the contraction: the innermost row loop has unit 1
  if (loops[row_loops.back()].unit != 1) return {};
  auto conflict_cost = [&]() {
    int64_t cost = 0;
    const int64_t steps = std::min<int64_t>(ksteps, 12);
    const int64_t blocks = std::min<int64_t>(ceil_div(NG, 16), 8);
    for (int64_t st = 0; st < steps; ++st)
      for (int64_t nb = 0; nb < blocks; ++nb) {
        int64_t addr[64];
        for (int lane = 0; lane < 64; ++lane) {
          const int64_t n = std::min<int64_t>(nb * 16 + lane % 16, NG - 1);
          const int64_t kk = std::min<int64_t>(k0[static_cast<size_t>(st)] + (lane / 16) * kdelta, s.K - 1);
          addr[lane] = row_lds(n) + k_lds(kk);
        }
        for (int banks : {32, 64}) {
          const int group = banks;                          // lanes served together
          for (int g0 = 0; g0 < 64; g0 += group) {
            std::map<int64_t, std::set<int64_t>> per_bank;
            for (int lane = g0; lane < g0 + group; ++lane) per_bank[addr[lane] % banks].insert(addr[lane]);
            size_t worst = 1;
            for (const auto& kv : per_bank) worst = std::max(worst, kv.second.size());
            cost += static_cast<int64_t>(worst) - 1;
          }
        }
      }
    return cost;
  };
  {
    int64_t best_pad = 0, best_cost = -1;
    for (int64_t pad = 0; pad < 64; ++pad) {
      set_strides(pad);
      const int64_t c = conflict_cost();
      if (best_cost < 0 || c < best_cost) {
        best_cost = c;
        best_pad = pad;
      }
      if (c == 0) break;
    }
    set_strides(best_pad);
  }
  int64_t patch_floats = 1;
  for (const auto& a : axes) patch_floats += (a.extent - 1) * a.lds;
  if (patch_floats * 4 > 120 * 1024) return {};

  // ---- step tables ---------------------------------------------------------------------------------
  std::vector<std::vector<int64_t>> patterns;
  std::vector<int64_t> koff(static_cast<size_t>(ksteps)), kpat(static_cast<size_t>(ksteps));
  for (int64_t st = 0; st < ksteps; ++st) {
    const int64_t base = k_lds(std::min<int64_t>(k0[static_cast<size_t>(st)], s.K - 1));
    std::vector<int64_t> p(4);
    for (int j = 0; j < 4; ++j) p[static_cast<size_t>(j)] = k_lds(std::min<int64_t>(k0[static_cast<size_t>(st)] + j * kdelta, s.K - 1)) - base;
    size_t id = 0;
    while (id < patterns.size() && patterns[id] != p) ++id;
    if (id == patterns.size()) patterns.push_back(p);
    koff[static_cast<size_t>(st)] = base;
    kpat[static_cast<size_t>(st)] = static_cast<int64_t>(id);
  }
  if (patterns.size() > 16 || static_cast<int64_t>(patterns.size()) * lay.nb > 160) return {};

  // ---- A's rows in LDS: row stride padded so that the sixteen rows and four sub-k of a read spread over the banks
  const int64_t kpad = ceil_div(s.K, 4) * 4;
  const bool a_vec = s.a_k == 1 && s.K % 4 == 0 && s.a_m % 4 == 0 && s.a_off % 4 == 0 && s.a_b % 4 == 0 &&
                     (!s.a_msplit || s.a_m2 % 4 == 0);
  int64_t a_lds = kpad;
  {
    int64_t best = -1;
    for (int64_t pad = 0; pad < 64; pad += a_vec ? 4 : 1) {
      const int64_t ks = kpad + pad;
      int64_t cost = 0;
      for (int banks : {32, 64})
        for (int g0 = 0; g0 < 64; g0 += banks) {
          std::map<int64_t, std::set<int64_t>> per_bank;
          for (int lane = g0; lane < g0 + banks; ++lane) {
            const int64_t addr = (lane % 16) * ks + (lane / 16) * kdelta;
            per_bank[addr % banks].insert(addr);
          }
          size_t worst = 1;
          for (const auto& kv : per_bank) worst = std::max(worst, kv.second.size());
          cost += static_cast<int64_t>(worst) - 1;
        }
      if (best < 0 || cost < best) {
        best = cost;
        a_lds = ks;
      }
      if (cost == 0) break;
    }
  }
  const int64_t mrows = static_cast<int64_t>(lay.waves_m) * lay.mb * 16;
  if ((patch_floats + mrows * a_lds) * 4 > 158 * 1024) return {};
  // the per-lane base (row + pattern offset) plus a step's offset stays inside the patch by construction

  // ---- groups: the row loops outside the workgroup, and the batch loops -----------------------------
  int64_t groups = 1;
  for (size_t q = 0; q < first_in; ++q) groups *= loops[row_loops[q]].extent;
  if (groups * NG != s.N || groups > 0x7fffffffLL) return {};

  // ---- source ---------------------------------------------------------------------------------------
  std::ostringstream os;
  LaunchSpec ls;
  ls.entry = "ehk_" + k.name;
  ls.kernels = {k.name};
  os << "// generated for gfx950 by eclat backend-hip: MFMA contraction with a window operand staged in LDS\n";
  os << "#define EW_ENTRY " << ls.entry << "\n";
  os << "#define EW_M " << s.M << "\n#define EW_MW " << s.M << "\n#define EW_NG " << NG << "\n#define EW_GROUPS " << groups
     << "\n#define EW_K " << s.K << "\n";
  os << "#define EW_WAVES_M " << lay.waves_m << "\n#define EW_WAVES_N " << lay.waves_n << "\n#define EW_MB " << lay.mb
     << "\n#define EW_NB " << lay.nb << "\n";
  os << "#define EW_KSTEPS " << ksteps << "\n#define EW_NPAT " << patterns.size() << "\n#define EW_KDELTA " << kdelta << "\n";
  os << "#define EW_PATCH_FLOATS " << patch_floats << "\n#define EW_PATCH_ELEMS " << patch_elems << "\n";
  os << "#define EW_A_OFF " << s.a_off << "LL\n#define EW_A_BS " << s.a_b << "LL\n#define EW_A_SM " << s.a_m
     << "LL\n#define EW_A_SK " << s.a_k << "LL\n#define EW_A_MSPLIT " << s.a_msplit << "LL\n#define EW_A_SM2 " << s.a_m2 << "LL\n";
  os << "#define EH_C_OFF " << s.c_off << "LL\n#define EH_C_BS " << s.c_b << "LL\n#define EH_C_SM " << s.c_m
     << "LL\n#define EH_C_SN " << s.c_n << "LL\n";
  os << "#define EH_C_MSPLIT " << s.c_msplit << "LL\n#define EH_C_SM2 " << s.c_m2 << "LL\n#define EH_C_NSPLIT " << s.c_nsplit
     << "LL\n#define EH_C_SN2 " << s.c_n2 << "LL\n";
  os << "#define EW_A_VEC " << (a_vec ? 1 : 0) << "\n#define EW_KPAD " << kpad << "\n#define EW_A_LDS " << a_lds << "\n";
  os << "#define EW_SRC_BYTES " << f->ranged_bytes << "u\n";
  os << "#define EW_MIX " << (opt.gemm_mix ? 1 : 0) << "\n";
  if (epilogue) {
    os << "#define EH_EPILOGUE 1\n#define EH_EPI_PARAMS " << epilogue->params << "\n#define EH_EPI_ARGS " << epilogue->args << "\n";
    if (!epilogue->store_c) os << "#define EH_NO_C 1\n";
    os << epilogue->function;
  }
  auto table = [&](const char* name, const std::vector<int64_t>& vals) {
    os << "constexpr int " << name << "[" << vals.size() << "] = {";
    for (size_t i = 0; i < vals.size(); ++i) os << (i ? ", " : "") << vals[i];
    os << "};\n";
  };
  os << "// step s multiplies k = ew_k0[s] + j * EW_KDELTA (j = 0..3); in the patch those sit at\n"
        "// ew_koff[s] + ew_pat[ew_kpat[s]][j] beyond the row's base\n";
  os << "namespace {\n";
  table("ew_k0", k0);
  table("ew_koff", koff);
  table("ew_kpat", kpat);
  os << "}\n";
  // sub-step j of a step with pattern p: offset by arithmetic on the bits of j over literals
  os << "__device__ __forceinline__ int ew_pat_lane(int p, int j) {\n  const int b0 = j & 1, b1 = j >> 1;\n  (void)b0; (void)b1;\n";
  for (size_t p = 0; p < patterns.size(); ++p) {
    const auto& o = patterns[p];
    os << "  if (p == " << p << ") return " << o[0] << " + b0 * " << (o[1] - o[0]) << " + b1 * " << (o[2] - o[0]) << " + (b0 & b1) * "
       << (o[3] - o[2] - o[1] + o[0]) << ";\n";
  }
  os << "  return 0;\n}\n";
  // row n of the group -> LDS offset
  os << "// what the rows of kernel " << f->kernel << " read of " << f->src << ", as a patch in LDS: axes";
  for (const auto& a : axes) os << " [" << a.extent << " x stride " << a.sstride << ", valid " << a.lo << ".." << a.hi << ", lds " << a.lds << "]";
  os << "\n__device__ __forceinline__ int ew_row_lds(int n) {\n  const unsigned u = (unsigned)n;\n  (void)u;\n  return 0";
  for (size_t q = first_in; q < row_loops.size(); ++q) {
    const WLoop& w = loops[row_loops[q]];
    os << " + (int)((u / " << w.unit << "u) % " << w.extent << "u) * " << axes[static_cast<size_t>(w.axis)].lds;
  }
  os << ";\n}\n";
  // patch element e of group g, batch bz -> LDS offset, byte offset in the source (out of range where padding)
  os << "__device__ __forceinline__ void ew_patch_elem(int e, long long g, long long bz, int* lds, unsigned* src_byte) {\n";
  os << "  const unsigned u = (unsigned)e, ug = (unsigned)g, ub = (unsigned)bz;\n  (void)u; (void)ug; (void)ub;\n";
  {
    int64_t radix = 1;
    std::vector<std::string> decl(axes.size());
    for (size_t i = axes.size(); i-- > 0;) {
      std::ostringstream d;
      d << "  const int p" << i << " = (int)((u / " << radix << "u) % " << axes[i].extent << "u);\n";
      decl[i] = d.str();
      radix *= axes[i].extent;
    }
    for (const auto& d : decl) os << d;
  }
  os << "  *lds = 0";
  for (size_t i = 0; i < axes.size(); ++i) os << " + p" << i << " * " << axes[i].lds;
  os << ";\n  const bool ok = true";
  for (size_t i = 0; i < axes.size(); ++i) {
    if (axes[i].lo > 0) os << " & (p" << i << " >= " << axes[i].lo << ")";
    if (axes[i].hi < axes[i].extent) os << " & (p" << i << " < " << axes[i].hi << ")";
  }
  os << ";\n  long long src = " << idx->c << "LL";
  for (size_t i = 0; i < axes.size(); ++i) os << " + (long long)p" << i << " * " << axes[i].sstride << "LL";
  {
    // digits of the group over the row loops outside the workgroup, of the batch over the batch loops
    int64_t radix = 1;
    for (size_t q = first_in; q-- > 0;) {
      const WLoop& w = loops[row_loops[q]];
      os << " + (long long)((ug / " << radix << "u) % " << w.extent << "u) * " << w.sstride << "LL";
      radix *= w.extent;
    }
    for (size_t q : batch_loops) {
      const WLoop& w = loops[q];
      os << " + (long long)((ub / " << w.unit << "u) % " << w.extent << "u) * " << w.sstride << "LL";
    }
  }
  os << ";\n  *src_byte = ok ? (unsigned)(src << 2) : 0x80000000u;\n}\n";
  os << kWindowSource;
  ls.source = os.str();
  ls.schedule = "mfma16x16x4(window,group=" + std::to_string(NG) + ",M=" + std::to_string(s.M) + ",K=" + std::to_string(s.K) +
                ",waves=" + std::to_string(lay.waves_m) + "x" + std::to_string(lay.waves_n) + ",blocks=" + std::to_string(lay.mb) +
                "x" + std::to_string(lay.nb) + ",steps=" + std::to_string(ksteps) + ",patterns=" + std::to_string(patterns.size()) +
                ",lds=" + std::to_string((patch_floats + mrows * a_lds) * 4) + "B" + (fa ? ",C^T" : "") +
                (epilogue ? ",epilogue=" + std::to_string(epilogue->kernels.size()) : "") + ")";
  ls.grid[0] = static_cast<unsigned>(groups);
  ls.grid[1] = 1;
  ls.grid[2] = static_cast<unsigned>(s.batch);
  ls.block[0] = static_cast<unsigned>(lay.waves_m * lay.waves_n * 64);
  auto reach = [](int64_t rows, int64_t sr, int64_t split, int64_t sr2) {
    if (!split) return (rows - 1) * sr;
    return (rows / split - 1) * sr2 + (split - 1) * sr;
  };
  const size_t c_elems = static_cast<size_t>(s.c_off + reach(s.M, s.c_m, s.c_msplit, s.c_m2) + reach(s.N, s.c_n, s.c_nsplit, s.c_n2) +
                                             (s.batch - 1) * s.c_b + 1);
  ls.arg_bufs = {s.a_buf, f->src};
  ls.arg_min_bytes = {4 * static_cast<size_t>(s.a_off + reach(s.M, s.a_m, s.a_msplit, s.a_m2) + (s.K - 1) * s.a_k + (s.batch - 1) * s.a_b + 1), 0};
  if (!(epilogue && !epilogue->store_c)) {
    ls.arg_bufs.push_back(s.c_buf);
    ls.arg_min_bytes.push_back(4 * c_elems);
  }
  if (epilogue) {
    for (size_t i = 0; i < epilogue->bufs.size(); ++i) {
      ls.arg_bufs.push_back(epilogue->bufs[i]);
      ls.arg_min_bytes.push_back(epilogue->min_bytes[i]);
    }
    for (const auto& n : epilogue->kernels) ls.kernels.push_back(n);
  }
  ls.flops = 2.0 * static_cast<double>(s.M) * static_cast<double>(s.N) * static_cast<double>(s.K) * static_cast<double>(s.batch);
  {
    const double nb = static_cast<double>(s.batch);
    const double a_bytes = 4.0 * static_cast<double>(s.M) * s.K * (s.a_b == 0 ? 1.0 : nb);
    const double f_bytes = f->src_bytes > 0 ? f->src_bytes : 4.0 * static_cast<double>(s.K) * s.N * nb;
    const double c_bytes = 4.0 * nb * static_cast<double>(s.M) * s.N;
    ls.algo_bytes = a_bytes + f_bytes + (epilogue && !epilogue->store_c ? 0.0 : c_bytes) + (epilogue ? epilogue->bytes : 0.0);
  }
  return {ls};
}

}  // namespace eh
