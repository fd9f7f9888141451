#include "window.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <functional>
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

// why a problem was turned down, for whoever sets EH_WINDOW_DEBUG
#define BAIL(n)                                                                                   \
  do {                                                                                            \
    if (std::getenv("EH_WINDOW_DEBUG")) std::fprintf(stderr, "window schedule: %s declined at check %d\n", p.entry.c_str(), n); \
    return {};                                                                                    \
  } while (0)

// A loop with what the emitter derives for it.
struct L {
  WLoop w;
  int64_t unit = 1;       // weight in its side's flat index
  int axis = -1;          // patch axis (loops inside the workgroup that move F's source), or -1
  bool in_wg = false;
};

// One coordinate of the patch: a source axis walked by one loop, or by a row loop and a window
// loop together (same stride in the source, either sign: the coordinate is the sum of the digits
// of the loops with a positive stride and of extent - 1 - digit of those with a negative one).
struct PAxis {
  int64_t sstride = 0, extent = 1, lds = 0, shift = 0;
  int64_t lo = 0, hi = 0;     // coordinates in [lo, hi) exist in the source; the rest is padding
};

struct Layout {
  int waves_m = 1, waves_n = 1, mb = 1, nb = 1;
};

// worst number of distinct addresses falling into one LDS bank, minus one, summed over the two
// halves of a wave for 32 banks and over the wave for 64
int64_t bank_cost(const int64_t (&addr)[64]) {
  int64_t cost = 0;
  for (int banks : {32, 64})
    for (int g0 = 0; g0 < 64; g0 += banks) {
      std::map<int64_t, std::set<int64_t>> per_bank;
      for (int lane = g0; lane < g0 + banks; ++lane) per_bank[((addr[lane] % banks) + banks) % banks].insert(addr[lane]);
      size_t worst = 1;
      for (const auto& kv : per_bank) worst = std::max(worst, kv.second.size());
      cost += static_cast<int64_t>(worst) - 1;
    }
  return cost;
}

// text: sum over `ls` of ((<var> / unit) % extent) * stride(l), as long long
std::string digits_sum(const std::vector<const L*>& ls, const std::string& var, const std::function<int64_t(const L&)>& stride) {
  std::ostringstream os;
  os << "0LL";
  for (const L* l : ls) {
    if (stride(*l) == 0) continue;
    os << " + (long long)((" << var << " / " << l->unit << "u) % " << l->w.extent << "u) * " << stride(*l) << "LL";
  }
  return os.str();
}

}  // namespace

std::vector<LaunchSpec> emit_window(const WindowProblem& p, const GenOptions& opt, const EpilogueSpec* epilogue) {
  // ---- loops by side, units ---------------------------------------------------------------------
  std::vector<L> loops;
  for (const auto& w : p.loops) {
    if (w.extent < 1) BAIL(1);
    if (w.extent == 1) continue;
    L l;
    l.w = w;
    loops.push_back(l);
  }
  auto side_loops = [&](WSide s) {
    std::vector<size_t> v;
    for (size_t i = 0; i < loops.size(); ++i)
      if (loops[i].w.side == s) v.push_back(i);
    return v;
  };
  const std::vector<size_t> row_loops = side_loops(WSide::Row), k_loops = side_loops(WSide::K), m_loops = side_loops(WSide::M),
                            batch_loops = side_loops(WSide::Batch);
  auto set_units = [&](const std::vector<size_t>& v) {
    int64_t u = 1;
    for (size_t q = v.size(); q-- > 0;) {
      loops[v[q]].unit = u;
      u *= loops[v[q]].w.extent;
    }
    return u;
  };
  const int64_t N = set_units(row_loops), K = set_units(k_loops), M = set_units(m_loops), batch = set_units(batch_loops);
  if (K < 4 || M < 2 || N < 2 || batch > 65535 || M > (1 << 20) || K > (1 << 20)) BAIL(2);
  for (const auto& l : loops) {
    if ((l.w.side == WSide::Row || l.w.side == WSide::K) && l.w.f == 0) BAIL(3);
    if (l.w.side == WSide::M && l.w.f != 0) BAIL(4);
    if (l.w.side == WSide::Row && l.w.a != 0) BAIL(5);
    if (l.w.side == WSide::K && l.w.c != 0) BAIL(6);
    if (l.w.a < 0 || l.w.c < 0) BAIL(7);
    if (l.w.side == WSide::Batch && l.w.f < 0) BAIL(8);
  }
  if (p.f_bytes == 0 || p.f_bytes >= (size_t{1} << 31)) BAIL(9);
  auto find_loop = [&](const std::string& name) -> L* {
    for (auto& l : loops)
      if (l.w.name == name) return &l;
    return nullptr;
  };

  // ---- patch axes: row and k loops grouped by the magnitude of their stride in the source ---------
  std::map<int64_t, std::vector<size_t>> by_stride;
  for (size_t i = 0; i < loops.size(); ++i)
    if (loops[i].w.side == WSide::Row || loops[i].w.side == WSide::K) by_stride[std::llabs(loops[i].w.f)].push_back(i);
  std::set<size_t> paired_rows;
  for (const auto& kv : by_stride) {
    const auto& g = kv.second;
    if (g.size() == 1) continue;
    if (g.size() != 2) BAIL(10);
    const L &x = loops[g[0]], &y = loops[g[1]];
    if (x.w.side == y.w.side) BAIL(11);
    paired_rows.insert(x.w.side == WSide::Row ? g[0] : g[1]);
  }
  if (paired_rows.empty()) BAIL(12);      // no window: a plain strided operand, handled elsewhere
  // rows inside a workgroup: from some row loop inward, at least from the outermost window row loop
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
    if (loops[k_loops[q]].w.extent % 4 == 0 &&
        (sub < 0 || std::llabs(loops[k_loops[q]].w.f) > std::llabs(loops[k_loops[static_cast<size_t>(sub)]].w.f)))
      sub = static_cast<int>(q);
  const int64_t kdelta = sub >= 0 ? loops[k_loops[static_cast<size_t>(sub)]].unit : 1;
  const int64_t ksteps = sub >= 0 ? K / 4 : ceil_div(K, 4);
  if (ksteps > 512) BAIL(13);
  std::vector<int64_t> k0(static_cast<size_t>(ksteps));
  if (sub >= 0) {
    // every combination of the other k digits, times the blocks of four of the sub digit
    std::vector<int64_t> digit(k_loops.size(), 0);
    for (int64_t st = 0; st < ksteps; ++st) {
      int64_t kk = 0;
      for (size_t q = 0; q < k_loops.size(); ++q) kk += digit[q] * loops[k_loops[q]].unit * (static_cast<int>(q) == sub ? 4 : 1);
      k0[static_cast<size_t>(st)] = kk;
      for (size_t q = k_loops.size(); q-- > 0;) {
        const int64_t lim = static_cast<int>(q) == sub ? loops[k_loops[q]].w.extent / 4 : loops[k_loops[q]].w.extent;
        if (++digit[q] < lim) break;
        digit[q] = 0;
      }
    }
  } else {
    for (int64_t st = 0; st < ksteps; ++st) k0[static_cast<size_t>(st)] = 4 * st;
  }
  const int64_t kpad = ceil_div(K, 4) * 4;

  // ---- choose how many row loops a workgroup takes, and the wave layout -----------------------------
  const int64_t mblk_all = ceil_div(M, 16);
  Layout lay;
  size_t first_in = row_loops.size();
  int64_t NG = 0;
  auto mark = [&](size_t start, std::vector<PAxis>* ax_out) {
    for (auto& l : loops) {
      l.in_wg = l.w.side == WSide::K;
      l.axis = -1;
    }
    for (size_t q = start; q < row_loops.size(); ++q) loops[row_loops[q]].in_wg = true;
    // axes by source stride, largest first
    std::vector<PAxis> ax;
    for (auto it = by_stride.rbegin(); it != by_stride.rend(); ++it) {
      PAxis a;
      a.sstride = it->first;
      int64_t ext = 1, shift = 0;
      bool any = false;
      for (size_t i : it->second) {
        if (!loops[i].in_wg) {
          if (it->second.size() == 2) return false;     // a window pair split between workgroups
          continue;
        }
        ext += loops[i].w.extent - 1;
        if (loops[i].w.f < 0) shift += loops[i].w.extent - 1;
        any = true;
      }
      if (!any) continue;
      a.extent = ext;
      a.shift = shift;
      a.lo = 0;
      a.hi = ext;
      for (size_t i : it->second)
        if (loops[i].in_wg) loops[i].axis = static_cast<int>(ax.size());
      ax.push_back(a);
    }
    *ax_out = ax;
    return !ax.empty();
  };
  // Candidates from the largest group (fewest workgroups) to the smallest: the first that still
  // gives the chip a workgroup per CU is taken, else the one with the most workgroups.
  bool enough = false;
  for (size_t start = 0; start <= first_needed && !enough; ++start) {
    int64_t ng = 1;
    for (size_t q = start; q < row_loops.size(); ++q) ng *= loops[row_loops[q]].w.extent;
    if (ng > 4096) continue;
    std::vector<PAxis> ax;
    if (!mark(start, &ax)) continue;
    int64_t elems = 1;
    for (const auto& a : ax) elems *= a.extent;
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
    if ((elems + 64 + static_cast<int64_t>(l.waves_m) * l.mb * 16 * (kpad + 4)) * 4 > 160 * 1024) continue;
    first_in = start;
    lay = l;
    NG = ng;
    enough = (N / ng) * batch >= 256;
  }
  if (first_in == row_loops.size() || NG < 4) BAIL(14);
  std::vector<PAxis> axes;
  if (!mark(first_in, &axes)) BAIL(15);
  int64_t patch_elems = 1;
  for (const auto& a : axes) patch_elems *= a.extent;
  const int64_t groups = N / NG;
  if (groups > 0x7fffffffLL) BAIL(16);
  // (a handful of workgroups for a large product leaves most of the chip idle: the tiled schedule then)
  if (groups * batch < 16 && static_cast<double>(M) * static_cast<double>(N) * static_cast<double>(K) * static_cast<double>(batch) > 3.0e7) BAIL(28);

  // ---- guards: each bounds one patch coordinate (or repeats a loop's own extent) -------------------
  for (const auto& g : p.guards) {
    std::vector<std::pair<L*, int64_t>> vars;
    for (const auto& t : g.terms) {
      if (t.second == 0) continue;
      L* l = find_loop(t.first);
      if (!l) {
        bool once = false;      // a loop that runs once contributes nothing
        for (const auto& w : p.loops) once = once || (w.name == t.first && w.extent == 1);
        if (!once) BAIL(17);
        continue;
      }
      vars.push_back({l, t.second});
    }
    if (vars.empty()) {
      if (g.ge ? !(0 >= g.bound) : !(0 < g.bound)) BAIL(18);     // a constant condition must hold
      continue;
    }
    auto trivial = [&]() {
      // one loop with coefficient +-1: true for every value of the loop?
      if (vars.size() != 1 || std::llabs(vars[0].second) != 1) return false;
      const int64_t e = vars[0].first->w.extent;
      if (vars[0].second == 1) return g.ge ? g.bound <= 0 : g.bound >= e;
      return g.ge ? g.bound <= -(e - 1) : g.bound >= 1;
    };
    const int ax_id = vars[0].first->axis;
    bool same_axis = ax_id >= 0;
    for (const auto& v : vars) same_axis = same_axis && v.first->axis == ax_id;
    int members = 0;
    for (const auto& l : loops) members += (ax_id >= 0 && l.axis == ax_id) ? 1 : 0;
    if (!same_axis || static_cast<int>(vars.size()) != members) {
      if (!trivial()) BAIL(19);
      continue;
    }
    // coefficients: the signs of the loops' strides, all of them or all negated
    int sigma = 0;
    for (const auto& v : vars) {
      if (std::llabs(v.second) != 1) BAIL(20);
      const int sg = static_cast<int>(v.second) * (v.first->w.f > 0 ? 1 : -1);
      if (sigma != 0 && sg != sigma) BAIL(21);
      sigma = sg;
    }
    PAxis& ax = axes[static_cast<size_t>(ax_id)];
    // sum(sign * digit) = coordinate - shift
    if (sigma > 0) {
      if (g.ge) ax.lo = std::max(ax.lo, g.bound + ax.shift);
      else ax.hi = std::min(ax.hi, g.bound + ax.shift);
    } else {
      if (g.ge) ax.hi = std::min(ax.hi, ax.shift - g.bound + 1);      // -(x) >= b  <=>  x <= -b
      else ax.lo = std::max(ax.lo, ax.shift - g.bound + 1);           // -(x) < b   <=>  x > -b
    }
  }
  for (const auto& a : axes)
    if (a.lo >= a.hi) BAIL(22);

  // ---- A's rows in LDS: [m][k], row stride padded so that the sixteen rows and four sub-k of a read spread over the banks
  // A is fetched in the order of its memory: the loops that index it sorted by their stride there
  std::vector<const L*> a_order;
  for (size_t q : m_loops) a_order.push_back(&loops[q]);
  for (size_t q : k_loops) a_order.push_back(&loops[q]);
  for (const L* l : a_order)
    if (l->w.a <= 0) BAIL(25);
  std::stable_sort(a_order.begin(), a_order.end(), [](const L* x, const L* y) { return x->w.a > y->w.a; });
  const L* a_fast = a_order.back();
  bool a_vec = a_fast->w.side == WSide::K && a_fast->w.a == 1 && a_fast->unit == 1 && a_fast->w.extent % 4 == 0 && p.a_c0 % 4 == 0;
  for (const auto& l : loops)
    if (&l != a_fast && l.w.a % 4 != 0) a_vec = false;
  // ... or all of k as one run (every k loop's stride in A is its weight in k): four k at once whatever the loops' extents
  bool a_flat = !a_vec && K % 4 == 0 && p.a_c0 % 4 == 0;
  for (const auto& l : loops) {
    if (l.w.side == WSide::K) a_flat = a_flat && l.w.a == l.unit;
    else a_flat = a_flat && l.w.a % 4 == 0;
  }
  if (a_flat) {
    a_vec = true;
    std::vector<const L*> ms;
    for (const L* l : a_order)
      if (l->w.side == WSide::M) ms.push_back(l);
    a_order = ms;
  }
  int64_t a_lds = kpad;
  {
    int64_t best = -1;
    for (int64_t pad = 0; pad < 64; pad += a_vec ? 4 : 1) {
      int64_t addr[64];
      for (int lane = 0; lane < 64; ++lane) addr[lane] = (lane % 16) * (kpad + pad) + (lane / 16) * kdelta;
      const int64_t cost = bank_cost(addr);
      if (best < 0 || cost < best) {
        best = cost;
        a_lds = kpad + pad;
      }
      if (cost == 0) break;
    }
  }
  const int64_t mrows = static_cast<int64_t>(lay.waves_m) * lay.mb * 16;

  // ---- LDS layout of the patch: dense, one axis' stride padded against bank conflicts ------------------
  auto set_strides = [&](size_t pad_axis, int64_t pad) {
    int64_t st = 1;
    for (size_t i = axes.size(); i-- > 0;) {
      axes[i].lds = st + (i == pad_axis && i + 1 < axes.size() ? pad : 0);
      st = axes[i].lds * axes[i].extent;
    }
  };
  auto floats_now = [&]() {
    int64_t f = 1;
    for (const auto& a : axes) f += (a.extent - 1) * a.lds;
    return f;
  };
  // a loop's share of the patch offset for digit d
  auto lds_of = [&](const L& l, int64_t d) {
    const int64_t st = axes[static_cast<size_t>(l.axis)].lds;
    return (l.w.f > 0 ? d : l.w.extent - 1 - d) * st;
  };
  auto k_lds = [&](int64_t kk) {
    int64_t o = 0;
    for (size_t q : k_loops) o += lds_of(loops[q], (kk / loops[q].unit) % loops[q].w.extent);
    return o;
  };
  auto row_lds = [&](int64_t n) {
    int64_t o = 0;
    for (size_t q = first_in; q < row_loops.size(); ++q)
      o += lds_of(loops[row_loops[q]], (n / loops[row_loops[q]].unit) % loops[row_loops[q]].w.extent);
    return o;
  };
  {
    int64_t best_pad = 0, best_cost = -1, best_floats = 0;
    size_t best_axis = 0;
    for (size_t pa = 0; pa + 1 < std::max<size_t>(axes.size(), 2); ++pa)
      for (int64_t pad = 0; pad < 64; ++pad) {
        set_strides(pa, pad);
        const int64_t fl = floats_now();
        if ((fl + mrows * a_lds) * 4 > 160 * 1024) break;
        int64_t c = 0;
        const int64_t steps = std::min<int64_t>(ksteps, 12);
        const int64_t blocks = std::min<int64_t>(ceil_div(NG, 16), 8);
        for (int64_t st = 0; st < steps; ++st)
          for (int64_t nb = 0; nb < blocks; ++nb) {
            int64_t addr[64];
            for (int lane = 0; lane < 64; ++lane) {
              const int64_t n = std::min<int64_t>(nb * 16 + lane % 16, NG - 1);
              const int64_t kk = std::min<int64_t>(k0[static_cast<size_t>(st)] + (lane / 16) * kdelta, K - 1);
              addr[lane] = row_lds(n) + k_lds(kk);
            }
            c += bank_cost(addr);
          }
        if (best_cost < 0 || c < best_cost || (c == best_cost && fl < best_floats)) {
          best_cost = c;
          best_pad = pad;
          best_axis = pa;
          best_floats = fl;
        }
        if (c == 0) break;
      }
    if (best_cost < 0) BAIL(26);
    set_strides(best_axis, best_pad);
  }
  int64_t patch_floats = 1;
  for (const auto& a : axes) patch_floats += (a.extent - 1) * a.lds;

  // ---- step tables ---------------------------------------------------------------------------------
  std::vector<std::vector<int64_t>> patterns;
  std::vector<int64_t> koff(static_cast<size_t>(ksteps)), kpat(static_cast<size_t>(ksteps));
  int64_t min_rel = 0;
  for (int64_t st = 0; st < ksteps; ++st) {
    const int64_t base = k_lds(std::min<int64_t>(k0[static_cast<size_t>(st)], K - 1));
    std::vector<int64_t> pt(4);
    for (int j = 0; j < 4; ++j) {
      pt[static_cast<size_t>(j)] = k_lds(std::min<int64_t>(k0[static_cast<size_t>(st)] + j * kdelta, K - 1)) - base;
      min_rel = std::min(min_rel, pt[static_cast<size_t>(j)]);
    }
    size_t id = 0;
    while (id < patterns.size() && patterns[id] != pt) ++id;
    if (id == patterns.size()) patterns.push_back(pt);
    koff[static_cast<size_t>(st)] = base;
    kpat[static_cast<size_t>(st)] = static_cast<int64_t>(id);
  }
  if (patterns.size() > 16 || static_cast<int64_t>(patterns.size()) * lay.nb > 160) BAIL(23);
  // (a step's offset is an immediate of the read and must not be negative: what a pattern reaches
  // back is moved from the steps' offsets into the lanes' bases)
  if (min_rel < 0) {
    for (auto& pt : patterns)
      for (auto& o : pt) o -= min_rel;
    for (auto& o : koff) o += min_rel;
    for (const auto& o : koff)
      if (o < 0) BAIL(24);
  }

  const bool a_zero = mrows != M || kpad != K;            // padding rows / columns of A's tile must read as zero
  const int64_t a_elems = a_vec ? M * K / 4 : M * K;

  // ---- four rows in a row of the group next to each other in C, on a 16-byte boundary? ------------------
  // (then the product is computed transposed: a lane ends up with four consecutive rows of F for
  // one row of A, and stores them as one vector)
  bool c_quad = NG % 4 == 0 && p.c_c0 % 4 == 0 && !(epilogue && epilogue->quad_functions.empty());
  {
    auto c_of_n = [&](int64_t n) {
      int64_t o = 0;
      for (size_t q = first_in; q < row_loops.size(); ++q) o += ((n / loops[row_loops[q]].unit) % loops[row_loops[q]].w.extent) * loops[row_loops[q]].w.c;
      return o;
    };
    for (int64_t n = 0; n + 3 < NG && c_quad; n += 4)
      for (int64_t q = 0; q < 4; ++q) c_quad = c_quad && c_of_n(n) % 4 == 0 && c_of_n(n + q) == c_of_n(n) + q;
    for (size_t q = 0; q < first_in; ++q) c_quad = c_quad && loops[row_loops[q]].w.c % 4 == 0;
    for (size_t q : m_loops) c_quad = c_quad && loops[q].w.c % 4 == 0;
    for (size_t q : batch_loops) c_quad = c_quad && loops[q].w.c % 4 == 0;
  }

  // ---- passes over k: at least six blocks each, so that a step's reads still hide behind its MFMAs -------
  int passes = opt.window_passes > 0 ? opt.window_passes : static_cast<int>(std::min<int64_t>(4, std::max<int64_t>(1, int64_t{lay.nb} * lay.mb / 6)));
  passes = std::max(1, std::min(passes, lay.nb));
  while (passes > 1 && (lay.nb + passes - 1) / passes * (passes - 1) >= lay.nb) --passes;

  // ---- source ---------------------------------------------------------------------------------------
  std::ostringstream os;
  LaunchSpec ls;
  ls.entry = p.entry;
  ls.kernels = p.kernels;
  os << "// generated for gfx950 by eclat backend-hip: MFMA contraction with a window operand staged in LDS\n";
  os << "#define EW_ENTRY " << ls.entry << "\n";
  os << "#define EW_M " << M << "\n#define EW_NG " << NG << "\n#define EW_GROUPS " << groups << "\n#define EW_K " << K << "\n";
  os << "#define EW_WAVES_M " << lay.waves_m << "\n#define EW_WAVES_N " << lay.waves_n << "\n#define EW_MB " << lay.mb
     << "\n#define EW_NB " << lay.nb << "\n";
  os << "#define EW_KSTEPS " << ksteps << "\n#define EW_NPAT " << patterns.size() << "\n#define EW_KDELTA " << kdelta << "\n";
  os << "#define EW_PATCH_FLOATS " << patch_floats << "\n#define EW_PATCH_ELEMS " << patch_elems << "\n";
  os << "#define EW_A_VEC " << (a_vec ? 1 : 0) << "\n#define EW_A_ELEMS " << a_elems << "\n#define EW_A_ZERO " << (a_zero ? 1 : 0)
     << "\n#define EW_KPAD " << kpad << "\n#define EW_A_LDS " << a_lds << "\n";
  os << "#define EW_SRC_BYTES " << p.f_bytes << "u\n";
  os << "#define EW_MIX " << (opt.gemm_mix ? 1 : 0) << "\n#define EW_C_VEC " << (c_quad ? 4 : 1) << "\n#define EW_PASSES " << passes << "\n";
  // The epilogue's tail (a pooling reduce over what this launch stores): taken when the outputs
  // split evenly over the groups, group g's outputs read nothing outside the block of the stored
  // buffer that workgroup g writes -- checked on the first two groups and the last by walking
  // every address either side touches -- and that block fits into LDS beside the tiles: the
  // epilogue then stores its results there as well, and the tail reads them back from LDS behind
  // a barrier that does not wait for the stores to memory.
  bool tail = false;
  int64_t tail_per_group = 0, tail_block = 0, tail_lo = 0;
  if (epilogue && !epilogue->tail_function.empty() && epilogue->tail_reads && batch == 1 && groups > 0 &&
      epilogue->tail_outputs % groups == 0 && !epilogue->store_c) {
    tail_per_group = epilogue->tail_outputs / groups;
    tail_block = M * NG;
    auto digit_sum = [&](const std::vector<size_t>& which, int64_t v) {
      int64_t o = 0;
      for (size_t q : which) o += ((v / loops[q].unit) % loops[q].w.extent) * loops[q].w.c;
      return o;
    };
    tail = tail_block <= (int64_t{1} << 16) && tail_block % 4 == 0 &&
           (patch_floats + mrows * a_lds + tail_block) * 4 + 64 <= 160 * 1024;
    std::set<int64_t> gs = {0, std::min<int64_t>(1, groups - 1), groups - 1};
    for (int64_t g : gs) {
      if (!tail) break;
      int64_t lo = INT64_MAX, hi = INT64_MIN;
      for (int64_t m = 0; m < M; ++m) {
        const int64_t cm = digit_sum(m_loops, m);
        for (int64_t n = g * NG; n < (g + 1) * NG; ++n) {
          const int64_t at = p.c_c0 + cm + digit_sum(row_loops, n);
          lo = std::min(lo, at);
          hi = std::max(hi, at);
        }
      }
      if (g == 0) tail_lo = lo;
      // a closed block, every element written, group g's right behind group g - 1's
      tail = hi - lo + 1 == tail_block && lo == tail_lo + g * tail_block && tail_lo % 4 == 0;
      std::vector<int64_t> reads;
      for (int64_t o = g * tail_per_group; o < (g + 1) * tail_per_group && tail; ++o) {
        reads.clear();
        epilogue->tail_reads(o, &reads);
        for (int64_t at : reads) tail = tail && at >= lo && at <= hi;
      }
    }
  }
  if (tail) {
    os << "#define EH_TAIL 1\n#define EH_TAIL_PER_GROUP " << tail_per_group << "\n#define EH_TAIL_BLOCK " << tail_block
       << "\n#define EH_TAIL_BASE ((long long)blockIdx.x * " << tail_block << "LL + " << tail_lo << "LL)\n"
       << "#define EH_TAIL_PARAMS " << epilogue->tail_params << "\n#define EH_TAIL_ARGS " << epilogue->tail_args << "\n"
       << "// the workgroup's share of " << epilogue->tail_source << ", kept for the tail\n"
       << "__shared__ __attribute__((aligned(16))) float eh_tail_lds[EH_TAIL_BLOCK];\n";
  }
  if (epilogue) {
    os << "#define EH_EPILOGUE 1\n#define EH_EPI_PARAMS " << epilogue->params << "\n#define EH_EPI_ARGS " << epilogue->args << "\n";
    if (!epilogue->store_c) os << "#define EH_NO_C 1\n";
    os << epilogue->function;
    if (!epilogue->split_functions.empty()) os << "#define EH_EPILOGUE_SPLIT " << epilogue->n_loads << "\n" << epilogue->split_functions;
    if (c_quad) os << "#define EH_EPILOGUE_QUAD " << std::max(1, epilogue->quad_regs) << "\n" << epilogue->quad_functions;
    if (tail) os << epilogue->tail_function;
  }
  auto table = [&](const char* name, const std::vector<int64_t>& vals) {
    os << "constexpr int " << name << "[" << vals.size() << "] = {";
    for (size_t i = 0; i < vals.size(); ++i) os << (i ? ", " : "") << vals[i];
    os << "};\n";
  };
  os << "// step s multiplies k = ew_k0[s] + j * EW_KDELTA (j = 0..3); in the patch those sit at\n"
        "// ew_koff[s] + ew_pat_lane(ew_kpat[s], j) beyond the row's base\n";
  os << "namespace {\n";
  table("ew_k0", k0);
  table("ew_koff", koff);
  table("ew_kpat", kpat);
  os << "}\n";
  // sub-step j of a step with pattern p: offset by arithmetic on the bits of j over literals
  os << "__device__ __forceinline__ int ew_pat_lane(int p, int j) {\n  const int b0 = j & 1, b1 = j >> 1;\n  (void)b0; (void)b1;\n";
  for (size_t q = 0; q < patterns.size(); ++q) {
    const auto& o = patterns[q];
    os << "  if (p == " << q << ") return " << o[0] << " + b0 * " << (o[1] - o[0]) << " + b1 * " << (o[2] - o[0]) << " + (b0 & b1) * "
       << (o[3] - o[2] - o[1] + o[0]) << ";\n";
  }
  os << "  return 0;\n}\n";
  // row n of the group -> LDS offset
  os << "// " << p.what << ": what a group of " << NG << " rows reads of " << p.f_buf << ", as a patch in LDS: axes";
  for (const auto& a : axes) os << " [" << a.extent << " x stride " << a.sstride << ", valid " << a.lo << ".." << a.hi << ", lds " << a.lds << "]";
  os << "\n__device__ __forceinline__ int ew_row_lds(int n) {\n  const unsigned u = (unsigned)n;\n  (void)u;\n  return 0";
  for (size_t q = first_in; q < row_loops.size(); ++q) {
    const L& l = loops[row_loops[q]];
    const int64_t st = axes[static_cast<size_t>(l.axis)].lds;
    if (l.w.f > 0) os << " + (int)((u / " << l.unit << "u) % " << l.w.extent << "u) * " << st;
    else os << " + (" << (l.w.extent - 1) << " - (int)((u / " << l.unit << "u) % " << l.w.extent << "u)) * " << st;
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
  os << ";\n  long long src = " << p.f_c0 << "LL";
  for (size_t i = 0; i < axes.size(); ++i) os << " + (long long)(p" << i << " - " << axes[i].shift << ") * " << axes[i].sstride << "LL";
  {
    // digits of the group over the row loops outside the workgroup, of the batch over the batch loops
    int64_t radix = 1;
    for (size_t q = first_in; q-- > 0;) {
      const L& l = loops[row_loops[q]];
      if (l.w.f < 0) BAIL(27);
      os << " + (long long)((ug / " << radix << "u) % " << l.w.extent << "u) * " << l.w.f << "LL";
      radix *= l.w.extent;
    }
    for (size_t q : batch_loops)
      os << " + (long long)((ub / " << loops[q].unit << "u) % " << loops[q].w.extent << "u) * " << loops[q].w.f << "LL";
  }
  os << ";\n  *src_byte = ok ? (unsigned)(src << 2) : 0x80000000u;\n}\n";
  // A: element e (in the order of A's memory; four along k at once where they can be read as one vector)
  {
    os << "// element (m, k) of A for e = 0.." << a_elems << ", walked in the order of A's memory: its offset there and in the tile\n";
    os << "__device__ __forceinline__ void ew_a_elem(int e, long long bz, int* lds, long long* off) {\n";
    os << "  const unsigned u = (unsigned)e, ub = (unsigned)bz;\n  (void)u; (void)ub;\n  long long o = " << p.a_c0 << "LL;\n  int m = 0, k = 0;\n";
    int64_t radix = 1;
    if (a_flat) {
      os << "  {\n    const int d = (int)(u % " << K / 4 << "u) * 4;\n    o += d;\n    k += d;\n  }\n";
      radix = K / 4;
    }
    for (size_t i = a_order.size(); i-- > 0;) {
      const L* l = a_order[i];
      const bool quad = a_vec && !a_flat && l == a_fast;
      const int64_t ext = quad ? l->w.extent / 4 : l->w.extent;
      os << "  {\n    const int d = (int)((u / " << radix << "u) % " << ext << "u)" << (quad ? " * 4" : "") << ";\n";
      os << "    o += (long long)d * " << l->w.a << "LL;\n";
      os << "    " << (l->w.side == WSide::M ? "m" : "k") << " += d * " << l->unit << ";\n  }\n";
      radix *= ext;
    }
    for (size_t q : batch_loops)
      if (loops[q].w.a) os << "  o += (long long)((ub / " << loops[q].unit << "u) % " << loops[q].w.extent << "u) * " << loops[q].w.a << "LL;\n";
    os << "  *lds = m * " << a_lds << " + k;\n  *off = o;\n}\n";
  }
  // C: offsets of row m, of row n of F (over all groups), of batch bz
  {
    std::vector<const L*> ms, ns, bs;
    for (size_t q : m_loops) ms.push_back(&loops[q]);
    for (size_t q : row_loops) ns.push_back(&loops[q]);
    for (size_t q : batch_loops) bs.push_back(&loops[q]);
    auto cs = [](const L& l) { return l.w.c; };
    os << "__device__ __forceinline__ long long ew_c_m(int m) {\n  const unsigned u = (unsigned)m;\n  (void)u;\n  return "
       << digits_sum(ms, "u", cs) << ";\n}\n";
    os << "__device__ __forceinline__ long long ew_c_n(long long n) {\n  const unsigned u = (unsigned)n;\n  (void)u;\n  return "
       << digits_sum(ns, "u", cs) << ";\n}\n";
    os << "__device__ __forceinline__ long long ew_c_b(long long bz) {\n  const unsigned u = (unsigned)bz;\n  (void)u;\n  return " << p.c_c0
       << "LL + " << digits_sum(bs, "u", cs) << ";\n}\n";
  }
  os << kWindowSource;
  ls.source = os.str();
  ls.part_params = std::string("const float* __restrict__ A, const float* __restrict__ F") +
                   (epilogue && !epilogue->store_c ? "" : ", float* __restrict__ C") + (epilogue ? epilogue->params : "") +
                   (tail ? epilogue->tail_params : "");
  ls.schedule = "mfma16x16x4(window,group=" + std::to_string(NG) + ",M=" + std::to_string(M) + ",K=" + std::to_string(K) +
                ",waves=" + std::to_string(lay.waves_m) + "x" + std::to_string(lay.waves_n) + ",blocks=" + std::to_string(lay.mb) +
                "x" + std::to_string(lay.nb) + ",steps=" + std::to_string(ksteps) + ",patterns=" + std::to_string(patterns.size()) +
                ",lds=" + std::to_string((patch_floats + mrows * a_lds + (tail ? tail_block : 0)) * 4) + "B" + (c_quad ? ",C:x4" : "") + (passes > 1 ? ",passes=" + std::to_string(passes) : std::string()) + p.tag +
                (epilogue ? ",epilogue=" + std::to_string(epilogue->kernels.size()) : "") + (tail ? ",tail=" + epilogue->tail_tag : "") + ")";
  ls.grid[0] = static_cast<unsigned>(groups);
  ls.grid[1] = 1;
  ls.grid[2] = static_cast<unsigned>(batch);
  ls.block[0] = 256;
  // smallest buffers: the furthest element each address can reach
  auto reach = [&](int64_t c0, int64_t WLoop::*stride) {
    int64_t r = c0;
    for (const auto& l : loops) r += (l.w.extent - 1) * std::max<int64_t>(0, l.w.*stride);
    return static_cast<size_t>(r + 1);
  };
  ls.arg_bufs = {p.a_buf, p.f_buf};
  ls.arg_min_bytes = {4 * reach(p.a_c0, &WLoop::a), 0};
  if (!(epilogue && !epilogue->store_c)) {
    ls.arg_bufs.push_back(p.c_buf);
    ls.arg_min_bytes.push_back(4 * reach(p.c_c0, &WLoop::c));
  }
  if (epilogue) {
    for (size_t i = 0; i < epilogue->bufs.size(); ++i) {
      ls.arg_bufs.push_back(epilogue->bufs[i]);
      ls.arg_min_bytes.push_back(epilogue->min_bytes[i]);
    }
    for (const auto& n : epilogue->kernels) ls.kernels.push_back(n);
    if (tail) {
      for (size_t i = 0; i < epilogue->tail_bufs.size(); ++i) {
        ls.arg_bufs.push_back(epilogue->tail_bufs[i]);
        ls.arg_min_bytes.push_back(epilogue->tail_min_bytes[i]);
      }
      for (const auto& n : epilogue->tail_kernels) ls.kernels.push_back(n);
    }
  }
  ls.flops = 2.0 * static_cast<double>(M) * static_cast<double>(N) * static_cast<double>(K) * static_cast<double>(batch);
  {
    bool a_moves = false;
    for (size_t q : batch_loops) a_moves = a_moves || loops[q].w.a != 0;
    const double nb = static_cast<double>(batch);
    const double a_bytes = 4.0 * static_cast<double>(M) * K * (a_moves ? nb : 1.0);
    const double f_bytes = p.f_algo_bytes > 0 ? p.f_algo_bytes : 4.0 * static_cast<double>(K) * N * nb;
    const double c_bytes = 4.0 * nb * static_cast<double>(M) * N;
    ls.algo_bytes = a_bytes + f_bytes + (epilogue && !epilogue->store_c ? 0.0 : c_bytes) + (epilogue ? epilogue->bytes : 0.0) +
                    (tail ? epilogue->tail_bytes : 0.0);
  }
  return {ls};
}

// ---------------------------------------------------------------------------------------------------
// from a matched contraction and its folded operand
// ---------------------------------------------------------------------------------------------------

namespace {

// e >= bound or e < bound over loop names, from one comparison of the gather's guard
bool collect_guards(const Node& c, std::vector<WGuard>* out) {
  if (c.op == Op::And || c.op == Op::BitAnd) return collect_guards(*c.args[0], out) && collect_guards(*c.args[1], out);
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
  Affine e = *l;
  for (const auto& kv : r->coef) e.coef[kv.first] -= kv.second;
  WGuard g;
  g.bound = r->c - l->c;
  g.ge = neg;
  for (const auto& kv : e.coef)
    if (kv.second != 0) g.terms.push_back({kv.first, kv.second});
  out->push_back(g);
  return true;
}

// stride of a loop (weight `unit` in an axis' flat index v) when v sits at
// split ? (v / split) * s2 + (v % split) * s1 : v * s1; false when the loop straddles the split
bool axis_stride(int64_t unit, int64_t extent, int64_t s1, int64_t split, int64_t s2, int64_t* out) {
  if (!split) {
    *out = unit * s1;
    return true;
  }
  if (unit >= split) {
    if (unit % split) return false;
    *out = (unit / split) * s2;
    return true;
  }
  if (unit * extent > split) return false;
  *out = unit * s1;
  return true;
}

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
  if (s.b_off != 0 || s.b_nsplit != 0 || s.a_off < 0 || s.a_k <= 0 || s.a_m <= 0 || s.c_off < 0) return {};

  WindowProblem p;
  p.entry = "ehk_" + k.name;
  p.kernels = {k.name};
  p.what = "rows of kernel " + f->kernel;
  p.a_buf = s.a_buf;
  p.f_buf = f->src;
  p.c_buf = s.c_buf;
  p.f_bytes = f->ranged_bytes;
  p.f_algo_bytes = f->src_bytes;
  p.a_c0 = s.a_off;
  p.c_c0 = s.c_off;
  p.tag = fa ? ",C^T" : "";

  // the gather: load index and guard
  const Node* v = f->value.get();
  if (v->op == Op::Select) {
    if (v->args[2]->op != Op::Const || v->args[2]->fval != 0.0 || !collect_guards(*v->args[0], &p.guards)) return {};
    v = v->args[1].get();
  }
  if (v->op != Op::Load || v->args[0]->op != Op::Var || v->args[0]->name != f->src) return {};
  auto idx = affine_of(*v->args[1]);
  if (!idx) return {};
  p.f_c0 = idx->c;
  for (const auto& kv : idx->coef) {
    if (kv.second == 0) continue;
    bool known = false;
    for (const auto& l : f->loops) known = known || l.name == kv.first;
    if (!known) return {};
  }

  // the gather's loops by the axis of the contraction their stride in its output falls into
  struct AxisRange { int64_t s, e; WSide side; };
  const AxisRange ranges[3] = {{s.b_b, s.batch, WSide::Batch}, {s.b_n, s.N, WSide::Row}, {s.b_k, s.K, WSide::K}};
  std::map<WSide, int64_t> covered, lowest;
  std::vector<std::pair<int64_t, WLoop>> placed;      // by stride in the gather's output, for ordering
  for (const auto& l : f->loops) {
    if (l.extent <= 1) {
      WLoop once;               // a loop that runs once: known by name (guards may mention it), otherwise ignored
      once.name = l.name;
      once.extent = 1;
      p.loops.push_back(once);
      continue;
    }
    WLoop w;
    w.name = l.name;
    w.extent = l.extent;
    w.f = idx->of(l.name);
    bool ok = false;
    for (const auto& r : ranges) {
      if (r.e <= 1 || r.s <= 0) continue;
      if (l.stride < r.s || l.stride >= r.s * r.e) continue;
      if (l.stride * l.extent > r.s * r.e || l.stride % r.s != 0) return {};
      w.side = r.side;
      const int64_t unit = l.stride / r.s;
      if (r.side == WSide::K) w.a = unit * s.a_k;
      if (r.side == WSide::Batch) {
        w.a = unit * s.a_b;
        w.c = unit * s.c_b;
      }
      if (r.side == WSide::Row && !axis_stride(unit, l.extent, s.c_n, s.c_nsplit, s.c_n2, &w.c)) return {};
      covered[r.side] = (covered.count(r.side) ? covered[r.side] : 1) * l.extent;
      lowest[r.side] = lowest.count(r.side) ? std::min(lowest[r.side], l.stride) : l.stride;
      ok = true;
      break;
    }
    if (!ok) return {};
    placed.push_back({l.stride, w});
  }
  for (const auto& r : ranges) {
    if (r.e <= 1) continue;
    if (covered[r.side] != r.e || lowest[r.side] != r.s) return {};
  }
  std::stable_sort(placed.begin(), placed.end(), [](const auto& x, const auto& y) { return x.first > y.first; });
  for (const auto& pl : placed) p.loops.push_back(pl.second);
  // A's and C's rows
  if (s.a_msplit) {
    if (s.M % s.a_msplit || (s.c_msplit && s.c_msplit != s.a_msplit)) return {};
    WLoop o, in;
    o.name = "eh_m_outer"; o.side = WSide::M; o.extent = s.M / s.a_msplit; o.a = s.a_m2;
    in.name = "eh_m_inner"; in.side = WSide::M; in.extent = s.a_msplit; in.a = s.a_m;
    if (!axis_stride(s.a_msplit, o.extent, s.c_m, s.c_msplit, s.c_m2, &o.c) || !axis_stride(1, in.extent, s.c_m, s.c_msplit, s.c_m2, &in.c))
      return {};
    p.loops.push_back(o);
    p.loops.push_back(in);
  } else if (s.c_msplit) {
    if (s.M % s.c_msplit) return {};
    WLoop o, in;
    o.name = "eh_m_outer"; o.side = WSide::M; o.extent = s.M / s.c_msplit; o.a = s.a_m * s.c_msplit; o.c = s.c_m2;
    in.name = "eh_m_inner"; in.side = WSide::M; in.extent = s.c_msplit; in.a = s.a_m; in.c = s.c_m;
    p.loops.push_back(o);
    p.loops.push_back(in);
  } else {
    WLoop m;
    m.name = "eh_m"; m.side = WSide::M; m.extent = s.M; m.a = s.a_m; m.c = s.c_m;
    p.loops.push_back(m);
  }
  return emit_window(p, opt, epilogue);
}

// ---------------------------------------------------------------------------------------------------
// from a kernel written as a window contraction
// ---------------------------------------------------------------------------------------------------

std::optional<WindowProblem> match_window_kernel(const Node& kernel, const std::map<std::string, size_t>& buffer_elems) {
  if (kernel.op != Op::Kernel || kernel.args.size() != 1) return std::nullopt;
  for (const auto& pr : kernel.params)
    if (pr.kind != VarKind::Normal || !pr.dtype.is_ptr()) return std::nullopt;
  struct Lp { std::string var; int64_t extent; };
  auto range_of = [](const Node& n, Lp* out) {
    if (n.op != Op::Range || n.args[0]->op != Op::Const || n.args[0]->ival != 0 || n.args[1]->op != Op::Const ||
        n.args[1]->ival != 1 || n.args[2]->op != Op::Const || n.args[2]->ival < 1)
      return false;
    *out = {n.name, n.args[2]->ival};
    return true;
  };
  auto unwrap = [](const Node* b) {
    while (b->op == Op::Block && b->decls.empty() && b->args.size() == 1) b = b->args[0].get();
    return b;
  };
  std::vector<Lp> outer, red;
  const Node* cur = unwrap(kernel.args[0].get());
  Lp lp;
  while (range_of(*cur, &lp)) {
    outer.push_back(lp);
    cur = unwrap(cur->args[3].get());
  }
  // block (decls acc): acc = 0; <reduce loops>; store
  if (cur->op != Op::Block || cur->decls.size() != 1 || cur->args.size() != 3) return std::nullopt;
  const std::string acc = cur->decls[0].first;
  if (cur->decls[0].second.ty != Ty::F32) return std::nullopt;
  const Node &init = *cur->args[0], &store = *cur->args[2];
  if (init.op != Op::Assign || init.name != acc || init.args[0]->op != Op::Const || init.args[0]->fval != 0.0) return std::nullopt;
  if (store.op != Op::Store || store.args[0]->op != Op::Var || store.args[2]->op != Op::Var || store.args[2]->name != acc)
    return std::nullopt;
  const Node* r = unwrap(cur->args[1].get());
  while (range_of(*r, &lp)) {
    red.push_back(lp);
    r = unwrap(r->args[3].get());
  }
  if (red.size() < 2 || r->op != Op::Assign || r->name != acc) return std::nullopt;      // (a single reduce loop is a NestKernel)
  ReduceKind kind = ReduceKind::None;
  NodePtr value;
  if (!match_combine(*r->args[0], acc, &kind, &value) || kind != ReduceKind::Sum || value->op != Op::Mul) return std::nullopt;
  WindowProblem p;
  const Node *fx = value->args[0].get(), *ax = value->args[1].get();
  auto gathered = [&](const Node* x, std::vector<WGuard>* gs) -> const Node* {
    if (x->op == Op::Select) {
      if (x->args[2]->op != Op::Const || x->args[2]->fval != 0.0 || !collect_guards(*x->args[0], gs)) return nullptr;
      x = x->args[1].get();
    }
    return x->op == Op::Load && x->args[0]->op == Op::Var && x->dtype.ty == Ty::F32 && x->count == 1 ? x : nullptr;
  };
  if (fx->op != Op::Select && ax->op == Op::Select) std::swap(fx, ax);
  const Node* fl = gathered(fx, &p.guards);
  std::vector<WGuard> none;
  const Node* al = gathered(ax, &none);
  if (!fl || !al || !none.empty() || ax->op == Op::Select) return std::nullopt;
  auto fi = affine_of(*fl->args[1]), ai = affine_of(*al->args[1]), ci = affine_of(*store.args[1]);
  if (!fi || !ai || !ci) return std::nullopt;
  p.f_buf = fl->args[0]->name;
  p.a_buf = al->args[0]->name;
  p.c_buf = store.args[0]->name;
  if (p.f_buf == p.c_buf || p.a_buf == p.c_buf) return std::nullopt;
  p.f_c0 = fi->c;
  p.a_c0 = ai->c;
  p.c_c0 = ci->c;
  if (p.a_c0 < 0 || p.c_c0 < 0) return std::nullopt;
  std::set<std::string> names;
  for (const auto& l : outer) {
    WLoop w;
    w.name = l.var;
    w.extent = l.extent;
    w.f = fi->of(l.var);
    w.a = ai->of(l.var);
    w.c = ci->of(l.var);
    if (w.extent > 1 && w.c <= 0) return std::nullopt;
    w.side = w.f != 0 && w.a != 0 ? WSide::Batch : w.f != 0 ? WSide::Row : WSide::M;
    if (w.extent > 1 && w.f == 0 && w.a == 0) return std::nullopt;
    p.loops.push_back(w);
    names.insert(l.var);
  }
  for (const auto& l : red) {
    WLoop w;
    w.name = l.var;
    w.extent = l.extent;
    w.f = fi->of(l.var);
    w.a = ai->of(l.var);
    w.side = WSide::K;
    if (ci->of(l.var) != 0) return std::nullopt;
    if (w.extent > 1 && (w.f == 0 || w.a <= 0)) return std::nullopt;
    p.loops.push_back(w);
    names.insert(l.var);
  }
  for (const Affine* a : {&*fi, &*ai, &*ci})
    for (const auto& kv : a->coef)
      if (kv.second != 0 && !names.count(kv.first)) return std::nullopt;
  auto it = buffer_elems.find(p.f_buf);
  if (it == buffer_elems.end() || it->second * 4 >= (size_t{1} << 31)) return std::nullopt;
  p.f_bytes = it->second * 4;
  p.f_algo_bytes = static_cast<double>(p.f_bytes);
  p.entry = "ehk_" + kernel.name;
  p.kernels = {kernel.name};
  p.what = "the guarded operand of kernel " + kernel.name;
  return p;
}

// ---------------------------------------------------------------------------------------------------
// from a contraction and the kernels that add up shifted reads of its result
// ---------------------------------------------------------------------------------------------------

namespace {

void add_terms(const NodePtr& e, std::vector<NodePtr>* out) {
  if (e->op == Op::Add) {
    add_terms(e->args[0], out);
    add_terms(e->args[1], out);
  } else {
    out->push_back(e);
  }
}

int64_t pos_mod(int64_t a, int64_t m) { return ((a % m) + m) % m; }

struct Tap {                      // one shifted read of the contraction's result
  Affine index;                   // where, over the adding kernels' loops
  std::vector<WGuard> guards;     // when
  Affine op[2];                   // the addresses of the contraction's two operands this stands for
};

// a loop that runs once is at zero: its terms go
void drop_single(Affine* a, const std::vector<Loop>& loops) {
  for (const auto& l : loops)
    if (l.extent <= 1) a->coef.erase(l.var);
}

// loops of extent > 1 by their stride in `a`, largest first; false unless the strides are positive
// and no loop reaches into the next one's stride (a digit per loop)
bool digit_loops(const std::vector<Loop>& loops, const Affine& a, std::vector<std::pair<int64_t, Loop>>* out) {
  out->clear();
  for (const auto& l : loops) {
    if (l.extent <= 1) continue;
    if (a.of(l.var) <= 0) return false;
    out->push_back({a.of(l.var), l});
  }
  std::stable_sort(out->begin(), out->end(), [](const auto& x, const auto& y) { return x.first > y.first; });
  for (size_t j = 0; j + 1 < out->size(); ++j)
    if ((*out)[j].first < (*out)[j + 1].first * (*out)[j + 1].second.extent) return false;
  return true;
}

// `idx` (over `loops`, wherever `guards` hold) as one affine value per loop of the producer:
// producer.out_aff evaluated at those values is idx, and every value stays inside its loop.
bool producer_digits(const Affine& idx, const std::vector<WGuard>& guards, const std::vector<Loop>& loops, const NestKernel& prod,
                     std::map<std::string, Affine>* digits) {
  // what the guards leave of each loop's range
  std::map<std::string, std::pair<int64_t, int64_t>> range;
  for (const auto& l : loops) range[l.var] = {0, l.extent - 1};
  for (const auto& g : guards) {
    if (g.terms.size() != 1 || std::llabs(g.terms[0].second) != 1 || !range.count(g.terms[0].first)) continue;
    auto& r = range[g.terms[0].first];
    if (g.terms[0].second == 1) {
      if (g.ge) r.first = std::max(r.first, g.bound);
      else r.second = std::min(r.second, g.bound - 1);
    } else {
      if (g.ge) r.second = std::min(r.second, -g.bound);
      else r.first = std::max(r.first, -g.bound + 1);
    }
  }
  for (const auto& kv : range)
    if (kv.second.first > kv.second.second) return false;
  std::vector<std::pair<int64_t, Loop>> pl;
  if (!digit_loops(prod.loops, *prod.out_aff, &pl) || pl.empty()) return false;
  std::vector<Affine> e(pl.size());
  for (const auto& kv : idx.coef) {
    if (kv.second == 0) continue;
    if (!range.count(kv.first)) return false;
    size_t j = 0;
    while (j < pl.size() && pl[j].first > std::llabs(kv.second)) ++j;
    if (j == pl.size() || kv.second % pl[j].first) return false;
    e[j].coef[kv.first] = kv.second / pl[j].first;
  }
  int64_t rest = idx.c - prod.out_aff->c;
  for (size_t j = pl.size(); j-- > 0;) {
    int64_t vlo = 0, vhi = 0;
    for (const auto& kv : e[j].coef) {
      const auto& r = range[kv.first];
      vlo += kv.second > 0 ? kv.second * r.first : kv.second * r.second;
      vhi += kv.second > 0 ? kv.second * r.second : kv.second * r.first;
    }
    const int64_t s = pl[j].first, ext = pl[j].second.extent;
    if (rest % s) return false;
    int64_t d = rest / s;
    if (j > 0) {
      if (pl[j - 1].first % s) return false;
      const int64_t ratio = pl[j - 1].first / s;
      // d is fixed modulo the ratio to the next stride; the one value that keeps the digit in its loop
      d = -vlo + pos_mod(d + vlo, ratio);      // the smallest such value that keeps the digit from going negative
    }
    if (vlo + d < 0 || vhi + d > ext - 1) return false;
    e[j].c = d;
    rest -= d * s;
  }
  if (rest != 0) return false;
  digits->clear();
  for (size_t j = 0; j < pl.size(); ++j) (*digits)[pl[j].second.var] = e[j];
  for (const auto& l : prod.loops)
    if (l.extent <= 1) (*digits)[l.var] = Affine{};
  return true;
}

// `op` (over the producer's loops and its reduce loop) with the producer's loops replaced by `digits`
// (its reduce loop, `kvar`, is called `kname` in the result: the names of the two nests may clash)
bool substitute(const Affine& op, const std::map<std::string, Affine>& digits, const std::string& kvar, const std::string& kname,
                Affine* out) {
  Affine r;
  r.c = op.c;
  for (const auto& kv : op.coef) {
    if (kv.second == 0) continue;
    if (kv.first == kvar) {
      r.coef[kname] += kv.second;
      continue;
    }
    auto d = digits.find(kv.first);
    if (d == digits.end()) return false;
    r.c += kv.second * d->second.c;
    for (const auto& dv : d->second.coef) r.coef[dv.first] += kv.second * dv.second;
  }
  for (auto it = r.coef.begin(); it != r.coef.end();) it = it->second == 0 ? r.coef.erase(it) : std::next(it);
  *out = r;
  return true;
}

// the part of each loop's range that the loads of `buf` in `reader` reach (digits of the loops'
// strides in `out`); false when that cannot be told
bool read_box(const NestKernel& reader, const std::string& buf, const std::vector<std::pair<int64_t, Loop>>& dl, int64_t out_c,
              std::map<std::string, std::pair<int64_t, int64_t>>* box) {
  std::vector<LoadRef> loads;
  collect_loads(*reader.value, loads);
  std::map<std::string, int64_t> extent;
  for (const auto& l : reader.loops) extent[l.var] = l.extent;
  if (reader.rkind != ReduceKind::None) extent[reader.rloop.var] = reader.rloop.extent;
  for (const auto& lr : loads) {
    if (lr.load->args[0]->op != Op::Var) return false;
    if (lr.load->args[0]->name != buf) continue;
    if (lr.load->count != 1) return false;
    auto a = affine_of(*lr.load->args[1]);
    if (!a) return false;
    std::vector<int64_t> lo(dl.size(), 0), span(dl.size(), 0);
    int64_t rest = a->c - out_c;
    if (rest < 0) return false;
    for (size_t j = 0; j < dl.size(); ++j) {
      lo[j] = rest / dl[j].first;
      rest -= lo[j] * dl[j].first;
    }
    if (rest != 0) return false;
    for (const auto& kv : a->coef) {
      if (kv.second == 0) continue;
      auto ex = extent.find(kv.first);
      if (ex == extent.end() || kv.second < 0) return false;
      size_t j = 0;
      while (j < dl.size() && dl[j].first > kv.second) ++j;
      if (j == dl.size() || kv.second % dl[j].first) return false;
      span[j] += (kv.second / dl[j].first) * (ex->second - 1);
    }
    for (size_t j = 0; j < dl.size(); ++j) {
      if (lo[j] + span[j] > dl[j].second.extent - 1) return false;
      auto it = box->find(dl[j].second.var);
      if (it == box->end()) (*box)[dl[j].second.var] = {lo[j], lo[j] + span[j]};
      else it->second = {std::min(it->second.first, lo[j]), std::max(it->second.second, lo[j] + span[j])};
    }
  }
  return true;
}

}  // namespace

// why a candidate was turned down, for whoever sets EH_WINDOW_DEBUG
#define SW_DECLINE(n)                                                                             \
  do {                                                                                            \
    if (std::getenv("EH_WINDOW_DEBUG")) std::fprintf(stderr, "shifted-sum window: %s declined at check %d\n", nests[i]->name.c_str(), n); \
    return std::nullopt;                                                                          \
  } while (0)

std::optional<ScatteredWindow> try_emit_scattered_window(size_t i, const ProgramView& pv, const GenOptions& opt) {
  const auto& nests = *pv.nests;
  if (i >= nests.size() || !nests[i] || pv.taken(i)) return std::nullopt;
  const NestKernel& P = *nests[i];
  if (P.rkind != ReduceKind::Sum || !P.identity || P.identity->fval != 0.0 || P.acc_dtype.ty != Ty::F32 || P.out_dtype.ty != Ty::F32 ||
      !P.out_aff || P.rloop.extent < 4 || pv.role_of(P.out_buf) != "temp")
    SW_DECLINE(2);
  const Node& pvl = *P.value;
  if (pvl.op != Op::Mul) SW_DECLINE(3);
  Affine pop[2];
  std::string pbuf[2];
  for (int o = 0; o < 2; ++o) {
    const Node& ld = *pvl.args[static_cast<size_t>(o)];
    if (ld.op != Op::Load || ld.args[0]->op != Op::Var || ld.count != 1 || ld.dtype.ty != Ty::F32) SW_DECLINE(4);
    auto a = affine_of(*ld.args[1]);
    if (!a) SW_DECLINE(5);
    pop[o] = *a;
    drop_single(&pop[o], P.loops);
    pbuf[o] = ld.args[0]->name;
  }
  auto rd = pv.readers->find(P.out_buf);
  if (rd == pv.readers->end() || rd->second.empty()) SW_DECLINE(6);
  const size_t n = rd->second.size();
  for (size_t q = 0; q < n; ++q)
    if (rd->second[q] != i + 1 + q) SW_DECLINE(7);
  // an operand that is itself a gather evaluated in place (a permuting copy folded into the
  // contraction) is read at its source
  const NestKernel* gat[2] = {nullptr, nullptr};
  Affine gsrc[2];
  for (int o = 0; o < 2; ++o) {
    gat[o] = pv.folded_gather(pbuf[o]);
    if (!gat[o]) continue;
    const Node& gv = *gat[o]->value;
    if (gat[o]->rkind != ReduceKind::None || !gat[o]->out_aff || gv.op != Op::Load || gv.args[0]->op != Op::Var || gv.count != 1 ||
        gv.dtype.ty != Ty::F32)
      SW_DECLINE(100);
    auto gi = affine_of(*gv.args[1]);
    if (!gi) SW_DECLINE(101);
    gsrc[o] = *gi;
    drop_single(&gsrc[o], gat[o]->loops);
    pbuf[o] = gv.args[0]->name;
  }
  if (i + n >= nests.size()) SW_DECLINE(8);

  // ---- the adding kernels and their shifted reads --------------------------------------------------
  std::vector<Tap> taps;
  const NestKernel* first = nullptr;
  ScatteredWindow out;
  out.elided.push_back(P.out_buf);
  for (size_t q = 0; q < n; ++q) {
    const size_t ci = i + 1 + q;
    if (!nests[ci] || pv.taken(ci)) SW_DECLINE(9);
    const NestKernel& C = *nests[ci];
    if (C.rkind != ReduceKind::None || !C.out_aff || C.out_dtype.ty != Ty::F32 || C.out_buf == pbuf[0] || C.out_buf == pbuf[1]) SW_DECLINE(10);
    if (!first) {
      first = &C;
    } else {
      if (C.loops.size() != first->loops.size() || !(*C.out_aff == *first->out_aff)) SW_DECLINE(11);
      for (size_t l = 0; l < C.loops.size(); ++l)
        if (C.loops[l].var != first->loops[l].var || C.loops[l].extent != first->loops[l].extent) SW_DECLINE(12);
    }
    if (q + 1 < n) {
      auto r = pv.readers->find(C.out_buf);
      if (pv.role_of(C.out_buf) != "temp" || r == pv.readers->end() || r->second != std::vector<size_t>{ci + 1}) SW_DECLINE(13);
      out.elided.push_back(C.out_buf);
    }
    std::vector<NodePtr> terms;
    add_terms(C.value, &terms);
    int running = 0;
    for (const auto& t : terms) {
      const Node* x = t.get();
      Tap tap;
      if (x->op == Op::Select) {
        if (x->args[2]->op != Op::Const || x->args[2]->fval != 0.0 || !collect_guards(*x->args[0], &tap.guards)) SW_DECLINE(14);
        x = x->args[1].get();
      }
      if (x->op != Op::Load || x->args[0]->op != Op::Var || x->count != 1 || x->dtype.ty != Ty::F32) SW_DECLINE(15);
      auto a = affine_of(*x->args[1]);
      if (!a) SW_DECLINE(16);
      if (q > 0 && x->args[0]->name == nests[ci - 1]->out_buf) {
        if (t->op == Op::Select || !(*a == *C.out_aff)) SW_DECLINE(17);
        ++running;
        continue;
      }
      if (x->args[0]->name != P.out_buf) SW_DECLINE(18);
      tap.index = *a;
      drop_single(&tap.index, C.loops);
      taps.push_back(tap);
    }
    if (running != (q > 0 ? 1 : 0)) SW_DECLINE(19);
  }
  const NestKernel& last = *nests[i + n];
  if (taps.size() < 2 || taps.size() > 64) SW_DECLINE(20);
  std::vector<std::pair<int64_t, Loop>> out_digits;
  if (!digit_loops(first->loops, *first->out_aff, &out_digits)) SW_DECLINE(21);

  // ---- each read as addresses of the contraction's operands ----------------------------------------
  const std::string kname = "eh_k";
  for (auto& t : taps) {
    std::map<std::string, Affine> digits;
    if (!producer_digits(t.index, t.guards, first->loops, P, &digits)) SW_DECLINE(22);
    std::vector<Loop> around = first->loops;
    around.push_back(Loop{kname, P.rloop.extent});
    for (int o = 0; o < 2; ++o) {
      if (gat[o]) {
        Affine at;
        std::map<std::string, Affine> gd;
        if (!substitute(pop[o], digits, P.rloop.var, kname, &at) || !producer_digits(at, t.guards, around, *gat[o], &gd) ||
            !substitute(gsrc[o], gd, "", "", &t.op[o]))
          SW_DECLINE(102);
        continue;
      }
      if (!substitute(pop[o], digits, P.rloop.var, kname, &t.op[o])) SW_DECLINE(23);
    }
  }
  for (const auto& t : taps)
    for (int o = 0; o < 2; ++o)
      if (t.op[o].coef != taps[0].op[o].coef) {
        if (std::getenv("EH_WINDOW_DEBUG")) {
          for (const auto& kv : t.op[o].coef) std::fprintf(stderr, " %s:%lld", kv.first.c_str(), (long long)kv.second);
          std::fprintf(stderr, " vs");
          for (const auto& kv : taps[0].op[o].coef) std::fprintf(stderr, " %s:%lld", kv.first.c_str(), (long long)kv.second);
          std::fprintf(stderr, "\n");
        }
        SW_DECLINE(24);
      }
  // the window operand is the one the guarded loops move
  std::map<std::string, int64_t> extent_of;
  for (const auto& l : first->loops) extent_of[l.var] = l.extent;
  auto always = [&](const WGuard& g) {
    if (g.terms.empty()) return g.ge ? 0 >= g.bound : 0 < g.bound;
    if (g.terms.size() != 1 || std::llabs(g.terms[0].second) != 1 || !extent_of.count(g.terms[0].first)) return false;
    const int64_t e = extent_of[g.terms[0].first];
    if (g.terms[0].second == 1) return g.ge ? g.bound <= 0 : g.bound >= e;
    return g.ge ? g.bound <= -(e - 1) : g.bound >= 1;
  };
  std::set<std::string> guard_vars;
  for (const auto& t : taps)
    for (const auto& g : t.guards)
      if (!always(g))
        for (const auto& tm : g.terms) guard_vars.insert(tm.first);
  if (guard_vars.empty()) SW_DECLINE(25);
  int fo = -1;
  for (int o = 0; o < 2; ++o) {
    bool all = true, none = true;
    for (const auto& v : guard_vars) {
      all = all && taps[0].op[o].of(v) != 0;
      none = none && taps[0].op[o].of(v) == 0;
    }
    if (all && fo < 0) fo = o;
    else if (!none) SW_DECLINE(26);
  }
  if (fo < 0) SW_DECLINE(27);
  const int ao = 1 - fo;
  for (const auto& v : guard_vars)
    if (taps[0].op[ao].of(v) != 0) SW_DECLINE(28);

  // ---- the shifts as one or two more reduce loops ----------------------------------------------------
  std::stable_sort(taps.begin(), taps.end(), [&](const Tap& x, const Tap& y) {
    return x.op[ao].c != y.op[ao].c ? x.op[ao].c < y.op[ao].c : x.op[fo].c < y.op[fo].c;
  });
  const int64_t nt = static_cast<int64_t>(taps.size());
  auto vec = [&](int64_t t) { return std::pair<int64_t, int64_t>{taps[static_cast<size_t>(t)].op[fo].c, taps[static_cast<size_t>(t)].op[ao].c}; };
  const auto v0 = vec(0);
  const std::pair<int64_t, int64_t> d2{vec(1).first - v0.first, vec(1).second - v0.second};
  int64_t n2 = 2;
  while (n2 < nt && vec(n2) == std::pair<int64_t, int64_t>{v0.first + n2 * d2.first, v0.second + n2 * d2.second}) ++n2;
  if (nt % n2) SW_DECLINE(29);
  const int64_t n1 = nt / n2;
  const std::pair<int64_t, int64_t> d1 = n1 > 1 ? std::pair<int64_t, int64_t>{vec(n2).first - v0.first, vec(n2).second - v0.second}
                                                 : std::pair<int64_t, int64_t>{0, 0};
  for (int64_t t = 0; t < nt; ++t)
    if (vec(t) != std::pair<int64_t, int64_t>{v0.first + (t / n2) * d1.first + (t % n2) * d2.first,
                                              v0.second + (t / n2) * d1.second + (t % n2) * d2.second})
      SW_DECLINE(30);
  if (d2.second <= 0 || d2.first == 0 || (n1 > 1 && (d1.second <= 0 || d1.first == 0))) SW_DECLINE(31);

  WindowProblem p;
  const char* tap_names[2] = {"eh_shift0", "eh_shift1"};
  // guards: one family per (terms, sense); a family's bounds move with the shift digits
  {
    std::map<std::pair<std::vector<std::pair<std::string, int64_t>>, bool>, std::vector<std::vector<int64_t>>> fam;
    for (int64_t t = 0; t < nt; ++t)
      for (const auto& g : taps[static_cast<size_t>(t)].guards) {
        auto terms = g.terms;
        std::sort(terms.begin(), terms.end());
        auto& f = fam[{terms, g.ge}];
        f.resize(static_cast<size_t>(nt));
        f[static_cast<size_t>(t)].push_back(g.bound);
      }
    for (const auto& kv : fam) {
      std::vector<int64_t> b(static_cast<size_t>(nt));
      bool everywhere = true;
      for (int64_t t = 0; t < nt; ++t) {
        const auto& v = kv.second[static_cast<size_t>(t)];
        if (v.empty()) { everywhere = false; break; }
        // several of one kind: the tightest
        b[static_cast<size_t>(t)] = kv.first.second ? *std::max_element(v.begin(), v.end()) : *std::min_element(v.begin(), v.end());
      }
      if (!everywhere) {
        // a condition some shifts lack must be one that always holds where it is stated
        WGuard g;
        g.terms = kv.first.first;
        g.ge = kv.first.second;
        for (int64_t t = 0; t < nt; ++t)
          for (int64_t bb : kv.second[static_cast<size_t>(t)]) {
            g.bound = bb;
            if (!always(g)) SW_DECLINE(32);
          }
        continue;
      }
      const int64_t b0 = b[0], s2 = b[1] - b[0], s1 = n1 > 1 ? b[static_cast<size_t>(n2)] - b[0] : 0;
      for (int64_t t = 0; t < nt; ++t)
        if (b[static_cast<size_t>(t)] != b0 + (t / n2) * s1 + (t % n2) * s2) SW_DECLINE(33);
      WGuard g;
      g.terms = kv.first.first;
      g.ge = kv.first.second;
      g.bound = b0;
      if (n1 > 1 && s1) g.terms.push_back({tap_names[0], -s1});
      if (s2) g.terms.push_back({tap_names[1], -s2});
      p.guards.push_back(g);
    }
  }

  // ---- the contraction over (k, shifts) ---------------------------------------------------------------
  const Affine &F = taps[0].op[fo], &A = taps[0].op[ao];
  for (const auto& l : first->loops) {
    WLoop w;
    w.name = l.var;
    w.extent = l.extent;
    w.f = F.of(l.var);
    w.a = A.of(l.var);
    w.c = first->out_aff->of(l.var);
    w.side = w.f != 0 && w.a != 0 ? WSide::Batch : w.f != 0 ? WSide::Row : WSide::M;
    if (w.extent > 1 && w.f == 0 && w.a == 0) SW_DECLINE(34);
    p.loops.push_back(w);
  }
  {
    WLoop k;
    k.name = kname;
    k.extent = P.rloop.extent;
    k.side = WSide::K;
    k.f = F.of(kname);
    k.a = A.of(kname);
    if (k.f == 0 || k.a <= 0) SW_DECLINE(35);
    p.loops.push_back(k);
    WLoop s1, s2;
    s1.name = tap_names[0]; s1.extent = n1; s1.side = WSide::K; s1.f = d1.first; s1.a = d1.second;
    s2.name = tap_names[1]; s2.extent = n2; s2.side = WSide::K; s2.f = d2.first; s2.a = d2.second;
    if (n1 > 1) p.loops.push_back(s1);
    p.loops.push_back(s2);
  }
  p.f_c0 = F.c;
  p.a_c0 = A.c;
  p.c_c0 = first->out_aff->c;
  p.f_buf = pbuf[fo];
  p.a_buf = pbuf[ao];
  p.c_buf = last.out_buf;
  if (p.a_c0 < 0 || p.c_c0 < 0 || p.f_buf == p.c_buf || p.a_buf == p.c_buf) SW_DECLINE(36);

  // ---- only what is read of the result ---------------------------------------------------------------
  if (pv.role_of(last.out_buf) == "temp") {
    auto r = pv.readers->find(last.out_buf);
    std::map<std::string, std::pair<int64_t, int64_t>> box;
    bool known = r != pv.readers->end() && !r->second.empty();
    if (known)
      for (size_t q : r->second) known = known && q > i + n && nests[q] && read_box(*nests[q], last.out_buf, out_digits, first->out_aff->c, &box);
    if (known)
      for (auto& w : p.loops) {
        auto b = box.find(w.name);
        if (b == box.end() || w.side == WSide::K) continue;
        const int64_t lo = b->second.first, cnt = b->second.second - b->second.first + 1;
        if (cnt == w.extent) continue;
        out.partial = true;
        w.extent = cnt;
        p.f_c0 += lo * w.f;
        p.a_c0 += lo * w.a;
        p.c_c0 += lo * w.c;
        for (auto& g : p.guards)
          for (const auto& tm : g.terms)
            if (tm.first == w.name) g.bound -= tm.second * lo;
      }
  }
  auto fe = pv.elems->find(p.f_buf);
  if (fe == pv.elems->end() || fe->second * 4 >= (size_t{1} << 31)) SW_DECLINE(37);
  p.f_bytes = fe->second * 4;
  p.f_algo_bytes = static_cast<double>(p.f_bytes);
  p.entry = "ehk_" + P.name;
  p.kernels = {P.name};
  for (size_t q = 0; q < n; ++q) p.kernels.push_back(nests[i + 1 + q]->name);
  p.what = "shifted reads of the product of kernel " + P.name + ", summed by " + std::to_string(n) + " kernels";
  p.tag = ",shifts=" + std::to_string(nt);
  out.launches = emit_window(p, opt, nullptr);
  if (out.launches.empty()) SW_DECLINE(38);
  out.next = i + 1 + n;
  return out;
}

}  // namespace eh
