// FP32 contraction C[m,n] = sum_k A[m,k] * F[n,k] on CDNA4 matrix cores (gfx950) where F is not
// in memory: it is a sliding-window gather (im2col of a padded image: pad -> unfold -> permute ->
// contiguous) that the generator folded into this kernel.  Evaluated per element in a tile loader,
// such an operand costs index arithmetic, a guard and a global load for every (row, k) pair, nine
// times per pixel of a 3x3 window, all of it vector instructions that a SIMD cannot issue while its
// matrix pipe runs.  Here the source region a group of rows reads (one image: every channel, the
// pixels with their zero border) is staged in LDS once, as a dense "patch" whose coordinates are
// the sums row digit + window digit, padding materialised as zeros.  Element (n, k) of F then sits at
//     patch[row_lds(n) + k_lds(k)]
// with row_lds depending on the lane's row only and k_lds on k only, so the multiply loop is
// nothing but ds_read_b32 at a per-lane base plus a compile-time offset, and MFMAs: no guards, no
// address arithmetic, each source element fetched from memory once per workgroup.
//
// One workgroup = one group of EW_NG rows of F (the rows that share a patch) x all rows of A x
// all of K.  A wave owns EW_MB x EW_NB accumulators of v_mfma_f32_16x16x4_f32 (16 rows of A by 16
// rows of F by 4 k).  A's rows are staged in LDS too, with coalesced loads (a lane needs
// A[i][k0(s) + j * delta] at step s: read straight from memory that is one cache line per lane
// and instruction, measured 8 of 31 us on a 3x3 convolution of 32 -> 64 channels), and come back
// one ds_read_b32 per step at "row base + k0(s)".  The four k of a step differ by a per-lane LDS
// offset that is constant along the loop except where the step straddles a digit boundary of k
// (a row of pixels ending): the generator lists the distinct offset patterns (EW_NPAT of them) and
// every lane keeps one base address per N-block and pattern.  The sum over k does not care in
// which order k is walked, so the generator lets the four k of a step differ along a digit of k
// whose extent is a multiple of four when there is one (the channels of a convolution: step s
// takes channels 4c..4c+3 of one tap, EW_KDELTA apart in k), which leaves a single pattern.
//
// The generator defines the EW_* / EH_* macros and the tables; the defaults below describe a 3x3
// convolution of 32 channels over 14x14 images so that the file compiles on its own.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

#ifndef EW_ENTRY
#define EW_ENTRY ehk_window_default
#define EW_M 64            // rows of A
#define EW_NG 196          // rows of F per group
#define EW_GROUPS 256      // groups per batch element
#define EW_K 288
#define EW_WAVES_M 4
#define EW_WAVES_N 1
#define EW_MB 1
#define EW_NB 13
#define EW_KSTEPS 72
#define EW_NPAT 1
#define EW_KDELTA 9         // k of sub-step j of step s: ew_k0[s] + j * EW_KDELTA
#define EW_PATCH_FLOATS 8688
#define EW_PATCH_ELEMS 8192
#define EW_A_VEC 1         // A is read with 128-bit loads along k
#define EW_A_ELEMS 4608    // elements (vectors of four with EW_A_VEC) of A to fetch
#define EW_A_ZERO 0        // A's tile has padding rows or columns, which must read as zero
#define EW_KPAD 288        // K rounded up to a multiple of four
#define EW_A_LDS 292       // floats between rows of A in LDS
#define EW_SRC_BYTES 6422528u
namespace {
struct EwTables {
  int k0[EW_KSTEPS], koff[EW_KSTEPS], kpat[EW_KSTEPS];
  constexpr EwTables() : k0{}, koff{}, kpat{} {
    for (int cs = 0; cs < 8; ++cs)
      for (int t = 0; t < 9; ++t) {
        k0[cs * 9 + t] = 36 * cs + t;                              // channels 4cs..4cs+3, tap t
        koff[cs * 9 + t] = 4 * cs * 272 + (t / 3) * 16 + t % 3;
        kpat[cs * 9 + t] = 0;
      }
  }
};
constexpr EwTables ew_tab{};
constexpr const int (&ew_k0)[EW_KSTEPS] = ew_tab.k0;
constexpr const int (&ew_koff)[EW_KSTEPS] = ew_tab.koff;
constexpr const int (&ew_kpat)[EW_KSTEPS] = ew_tab.kpat;
}
// LDS offset of sub-step j of a step with pattern p, beyond the step's offset: arithmetic on the
// two bits of j over literals (a table indexed by the lane would be a load from memory)
__device__ __forceinline__ int ew_pat_lane(int p, int j) {
  (void)p;
  return 272 * j;
}
// LDS offset of row n of the group; patch element e of group g: where it goes, where it comes from
__device__ __forceinline__ int ew_row_lds(int n) { return (n / 14) * 16 + n % 14; }
__device__ __forceinline__ void ew_patch_elem(int e, long long g, long long bz, int* lds, unsigned* src_byte) {
  (void)bz;
  const int c = e / 256, y = (e / 16) % 16, x = e % 16;
  *lds = c * 272 + y * 16 + x;
  const bool ok = (y >= 1) & (y < 15) & (x >= 1) & (x < 15);
  *src_byte = ok ? (unsigned)((g * 6272 + c * 196 + (y - 1) * 14 + (x - 1)) << 2) : 0x80000000u;
}
// element e of A in the order of its memory (here: vector e of four along k): offset in memory, offset in the tile
__device__ __forceinline__ void ew_a_elem(int e, long long bz, int* lds, long long* off) {
  (void)bz;
  const int m = e / 72, k = (e % 72) * 4;
  *lds = m * EW_A_LDS + k;
  *off = (long long)m * 288 + k;
}
// offsets in C of row m, of row n of F (counted over all groups), of batch element bz
__device__ __forceinline__ long long ew_c_m(int m) { return (long long)m * 196; }
__device__ __forceinline__ long long ew_c_n(long long n) { return (n / 196) * 12544 + n % 196; }
__device__ __forceinline__ long long ew_c_b(long long bz) { (void)bz; return 0; }
#endif

#ifndef EH_EPILOGUE
#define EH_EPI_PARAMS
#define EH_EPI_ARGS
#endif
// EH_TAIL: a short reduce over windows of a buffer the epilogue stores (the pooling behind a
// convolution).  Group g's EH_TAIL_PER_GROUP outputs read only what workgroup g stores, which the
// epilogue also keeps in LDS (eh_tail_lds): the workgroup computes those outputs itself at the
// end, eh_tail_ns::eh_tail(output, buffers...).  Not with EH_PART (the block is found by blockIdx).
#ifndef EH_TAIL
#define EH_TAIL_PARAMS
#endif
#ifdef EH_NO_C
#define EH_C_PARAM
#define EH_C_ARG
#else
#define EH_C_PARAM , float* __restrict__ C
#define EH_C_ARG , C
#endif
#ifndef EW_MIX
#define EW_MIX 1           // LDS reads of step s+1 issued one by one between the MFMAs of step s
#endif
#ifndef EW_PASSES
#define EW_PASSES 1        // passes over k, each for a share of a wave's N-blocks
#endif
#ifndef EW_C_VEC
#define EW_C_VEC 1         // 4: four rows of F in a row are neighbours in C (16-byte aligned): blocks computed transposed, 128-bit stores
#endif

typedef float ew_f4v __attribute__((ext_vector_type(4)));

namespace {
// Four waves whatever the layout: waves beyond EW_WAVES_M * EW_WAVES_N only help to fetch.
constexpr int EW_NT = 256;
static_assert(EW_WAVES_M * EW_WAVES_N <= 4, "at most four multiplying waves");
static_assert(EW_PASSES >= 1 && EW_PASSES <= 4 && (EW_NB + EW_PASSES - 1) / EW_PASSES * (EW_PASSES - 1) < EW_NB, "every pass has blocks");
template <int V> struct EwInt { static constexpr int value = V; };
}  // namespace

// EH_PART: this kernel is one of several issued as one launch.  It is then a function of its
// share of the launch's linear workgroup ids (its own grid is EH_PART_GX groups x batch) and of the
// launch's one block of LDS, which the parts use in turn; eh_lds_floats says how much it needs.
#ifdef EH_PART
constexpr int eh_lds_floats = ((EW_PATCH_FLOATS + 3) & ~3) + EW_WAVES_M * EW_MB * 16 * EW_A_LDS;
__device__ __forceinline__ void eh_run(const unsigned eh_bx, float* const eh_lds, const float* __restrict__ A, const float* __restrict__ F EH_C_PARAM EH_EPI_PARAMS EH_TAIL_PARAMS) {
  constexpr int MROWS = EW_WAVES_M * EW_MB * 16;
  float* const patch = eh_lds;
  float* const As = eh_lds + ((EW_PATCH_FLOATS + 3) & ~3);
  const long long g = eh_bx % EH_PART_GX, bz = eh_bx / EH_PART_GX;
#else
extern "C" __global__ void __launch_bounds__(EW_NT)
EW_ENTRY(const float* __restrict__ A, const float* __restrict__ F EH_C_PARAM EH_EPI_PARAMS EH_TAIL_PARAMS) {
  constexpr int MROWS = EW_WAVES_M * EW_MB * 16;        // rows of A a workgroup multiplies (padding rows are zero)
  __shared__ __attribute__((aligned(16))) float patch[EW_PATCH_FLOATS];
  __shared__ __attribute__((aligned(16))) float As[MROWS * EW_A_LDS];
  const long long g = blockIdx.x, bz = blockIdx.z;
#endif
  const int tid = threadIdx.x;
  const int lane = tid & 63, wid = tid >> 6;
  const int wm = wid % EW_WAVES_M, wn = wid / EW_WAVES_M;
  const int l16 = lane & 15, j4 = lane >> 4;

  // A into LDS, fetched in the order of its memory (128-bit loads where rows allow); rows beyond M
  // and k beyond K of the tile are zero.  Every load of a chunk is issued before the first value is
  // stored: a workgroup is alone on its CU for most of its life, so nothing else would hide one
  // load's latency behind another's.
  {
#if EW_A_ZERO
    for (int e = tid; e < MROWS * EW_A_LDS; e += EW_NT) As[e] = 0.0f;
    __syncthreads();
#endif
    constexpr int PER = (EW_A_ELEMS + EW_NT - 1) / EW_NT;
    constexpr int CH = PER < 24 ? PER : 24;
    for (int c0 = 0; c0 < PER; c0 += CH) {
#if EW_A_VEC
      ew_f4v v[CH];
#else
      float v[CH];
#endif
      int at[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        long long off = 0;
        ew_a_elem(e < EW_A_ELEMS ? e : 0, bz, &at[u], &off);
#if EW_A_VEC
        v[u] = *reinterpret_cast<const ew_f4v*>(A + off);
#else
        v[u] = A[off];
#endif
      }
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        if ((c0 + u) * EW_NT + tid < EW_A_ELEMS) {
#if EW_A_VEC
          *reinterpret_cast<ew_f4v*>(&As[at[u]]) = v[u];
#else
          As[at[u]] = v[u];
#endif
        }
      }
    }
  }

  // the patch: every element of the source region this group's rows read, once; zeros where the
  // window leaves the image (a byte offset beyond the resource reads as zero)
  {
    const __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc((void*)F, 0, EW_SRC_BYTES, 0x00020000);
    constexpr int PER = (EW_PATCH_ELEMS + EW_NT - 1) / EW_NT;      // elements per work-item
    constexpr int CH = PER < 32 ? PER : 32;
    for (int c0 = 0; c0 < PER; c0 += CH) {
      float v[CH];
      int at[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        unsigned src = 0x80000000u;
        at[u] = 0;
        if (e < EW_PATCH_ELEMS) ew_patch_elem(e, g, bz, &at[u], &src);
        v[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rs, src, 0, 0));
      }
#pragma unroll
      for (int u = 0; u < CH; ++u)
        if ((c0 + u) * EW_NT + tid < EW_PATCH_ELEMS) patch[at[u]] = v[u];
    }
  }
  __syncthreads();
  if (wid >= EW_WAVES_M * EW_WAVES_N) return;      // (no barrier follows)

  // per-lane LDS bases: the lane's row of A in each M-block plus its sub-k; the lane's row of F in
  // each N-block plus its sub-k offset under each pattern.  N-blocks are dealt to the waves in
  // turn (block nb * WAVES_N + wn), so that only a wave's last block can reach past the group.
  int abase[EW_MB];
#pragma unroll
  for (int mb = 0; mb < EW_MB; ++mb) abase[mb] = ((wm * EW_MB + mb) * 16 + l16) * EW_A_LDS + j4 * EW_KDELTA;
  int base[EW_NB][EW_NPAT];
#pragma unroll
  for (int nb = 0; nb < EW_NB; ++nb) {
    int n = (nb * EW_WAVES_N + wn) * 16 + l16;
    n = n < EW_NG ? n : EW_NG - 1;
    const int r = ew_row_lds(n);
#pragma unroll
    for (int p = 0; p < EW_NPAT; ++p)
      base[nb][p] = r + ew_pat_lane(p, j4);
  }

  // The N-blocks of a wave are multiplied in EW_PASSES passes over k, each finished (epilogue,
  // stores) before the next starts: a store only has to be issued, so the memory traffic of one
  // pass's results drains while the matrix pipe works on the next pass, and only the last pass's
  // stores are waited for at the end of the kernel.
  constexpr bool M_EDGE = MROWS != EW_M;
  const long long c_base = ew_c_b(bz);
  constexpr int NBP = (EW_NB + EW_PASSES - 1) / EW_PASSES;
  auto pass = [&](auto tag) __attribute__((always_inline)) {
    constexpr int NB0 = decltype(tag)::value * NBP;
    constexpr int CNT = EW_NB - NB0 < NBP ? EW_NB - NB0 : NBP;
    static_assert(CNT >= 1, "a pass without blocks");
    ew_f4v acc[EW_MB][CNT];
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < CNT; ++nb) acc[mb][nb] = ew_f4v{0.0f, 0.0f, 0.0f, 0.0f};

    // step s multiplies with the operands fetched during step s - 1
    float a[2][EW_MB], b[2][CNT];
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb) a[0][mb] = As[abase[mb] + ew_k0[0]];
#pragma unroll
    for (int nb = 0; nb < CNT; ++nb) b[0][nb] = patch[base[NB0 + nb][ew_kpat[0]] + ew_koff[0]];
#pragma unroll
    for (int s = 0; s < EW_KSTEPS; ++s) {
      if (s + 1 < EW_KSTEPS) {
#pragma unroll
        for (int mb = 0; mb < EW_MB; ++mb) a[(s + 1) & 1][mb] = As[abase[mb] + ew_k0[s + 1]];
#pragma unroll
        for (int nb = 0; nb < CNT; ++nb) b[(s + 1) & 1][nb] = patch[base[NB0 + nb][ew_kpat[s + 1]] + ew_koff[s + 1]];
      }
#pragma unroll
      for (int nb = 0; nb < CNT; ++nb)
#pragma unroll
        for (int mb = 0; mb < EW_MB; ++mb)
#if EW_C_VEC == 4
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(b[s & 1][nb], a[s & 1][mb], acc[mb][nb], 0, 0, 0);     // C^T block
#else
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s & 1][mb], b[s & 1][nb], acc[mb][nb], 0, 0, 0);
#endif
#if EW_MIX
      // (one LDS read after every MFMA; the reads of A's values ride with the first ones)
#pragma unroll
      for (int q = 0; q < EW_MB; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
#pragma unroll
      for (int q = EW_MB; q < CNT * EW_MB; ++q) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      }
#endif
      __builtin_amdgcn_sched_barrier(0);
    }

#if EW_C_VEC == 4
    // The blocks were computed transposed: accumulator register v of lane l holds row l % 16 of the
    // M-block, column 4 * (l / 16) + v of the N-block -- four rows of F in a row, next to each other
    // in C and on a 16-byte boundary (the generator checked).  A lane finishes them together: what
    // the epilogue reads is requested for a run of blocks before the run's first store goes out
    // (loads and stores leave through one queue, in order: a load behind a store waits for it).
#if defined(EH_EPILOGUE)
    constexpr int RUN = 48 / EH_EPILOGUE_QUAD < 1 ? 1 : 48 / EH_EPILOGUE_QUAD;
#else
    constexpr int RUN = 16;
#endif
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
      for (int nb0 = 0; nb0 < CNT; nb0 += RUN) {
        long long at[RUN];
        bool in[RUN];
#if defined(EH_EPILOGUE)
        EhEpiLoads4 got[RUN];
#endif
#pragma unroll
        for (int nb = nb0; nb < nb0 + RUN && nb < CNT; ++nb) {
          const int m = (wm * EW_MB + mb) * 16 + l16;
          const int n0 = ((NB0 + nb) * EW_WAVES_N + wn) * 16 + 4 * j4;
          in[nb - nb0] = (!M_EDGE || m < EW_M) && ((NB0 + nb + 1) * EW_WAVES_N * 16 <= EW_NG || n0 < EW_NG);
          at[nb - nb0] = c_base + ew_c_m(m < EW_M ? m : 0) + ew_c_n(g * EW_NG + (n0 < EW_NG ? n0 : 0));
#if defined(EH_EPILOGUE)
          if (in[nb - nb0]) eh_epilogue_load4(at[nb - nb0], got[nb - nb0] EH_EPI_ARGS);
#endif
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = nb0; nb < nb0 + RUN && nb < CNT; ++nb)
          if (in[nb - nb0]) {
#if defined(EH_EPILOGUE)
            const float four[4] = {acc[mb][nb][0], acc[mb][nb][1], acc[mb][nb][2], acc[mb][nb][3]};
            eh_epilogue_apply4(at[nb - nb0], four, got[nb - nb0] EH_C_ARG EH_EPI_ARGS);
#else
            *reinterpret_cast<ew_f4v*>(C + at[nb - nb0]) = acc[mb][nb];
#endif
          }
        __builtin_amdgcn_sched_barrier(0);
      }
#else
    // Accumulator register v of lane l holds row 4 * (l / 16) + v of the M-block, column l % 16 of the
    // N-block.  Blocks that lie inside the group whole are finished without a test per element, in one
    // run of straight-line code: whatever the epilogue loads (a bias, a saved activation) is then
    // requested for all of them before the first store goes out, where a branch around every element
    // would make each element's load wait for the stores of the one before (one queue for both).
    auto finish = [&](const int mb, const int nb, const int v, const bool test) {
      const int m = (wm * EW_MB + mb) * 16 + 4 * j4 + v;
      const int n = ((NB0 + nb) * EW_WAVES_N + wn) * 16 + l16;
      if (test && !(m < EW_M && n < EW_NG)) return;
      const long long e = c_base + ew_c_m(m) + ew_c_n(g * EW_NG + n);
#if defined(EH_EPILOGUE)
      eh_epilogue(e, acc[mb][nb][v] EH_C_ARG EH_EPI_ARGS);
#else
      C[e] = acc[mb][nb][v];
#endif
    };
#if defined(EH_EPILOGUE_SPLIT)
    // in runs of blocks: everything the epilogue reads for a run is requested before the run's first store
    constexpr int RUN = EH_EPILOGUE_SPLIT <= 1 ? 12 : EH_EPILOGUE_SPLIT <= 2 ? 6 : EH_EPILOGUE_SPLIT <= 4 ? 3 : 1;
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
      for (int nb0 = 0; nb0 < CNT; nb0 += RUN) {
        EhEpiLoads got[RUN][4];
        long long at[RUN][4];
#pragma unroll
        for (int nb = nb0; nb < nb0 + RUN && nb < CNT; ++nb)
          if (!M_EDGE && (NB0 + nb + 1) * EW_WAVES_N * 16 <= EW_NG) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
              const int m = (wm * EW_MB + mb) * 16 + 4 * j4 + v;
              const int n = ((NB0 + nb) * EW_WAVES_N + wn) * 16 + l16;
              at[nb - nb0][v] = c_base + ew_c_m(m) + ew_c_n(g * EW_NG + n);
              eh_epilogue_load(at[nb - nb0][v], got[nb - nb0][v] EH_EPI_ARGS);
            }
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb = nb0; nb < nb0 + RUN && nb < CNT; ++nb)
          if (!M_EDGE && (NB0 + nb + 1) * EW_WAVES_N * 16 <= EW_NG) {
#pragma unroll
            for (int v = 0; v < 4; ++v) eh_epilogue_apply(at[nb - nb0][v], acc[mb][nb][v], got[nb - nb0][v] EH_C_ARG EH_EPI_ARGS);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
#else
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < CNT; ++nb)
        if (!M_EDGE && (NB0 + nb + 1) * EW_WAVES_N * 16 <= EW_NG) {
#pragma unroll
          for (int v = 0; v < 4; ++v) finish(mb, nb, v, false);
        }
#endif
#pragma unroll
    for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
      for (int nb = 0; nb < CNT; ++nb)
        if (M_EDGE || (NB0 + nb + 1) * EW_WAVES_N * 16 > EW_NG) {
#pragma unroll
          for (int v = 0; v < 4; ++v) finish(mb, nb, v, true);
        }
#endif
  };
  pass(EwInt<0>{});
#if EW_PASSES > 1
  pass(EwInt<1>{});
#endif
#if EW_PASSES > 2
  pass(EwInt<2>{});
#endif
#if EW_PASSES > 3
  pass(EwInt<3>{});
#endif
#ifdef EH_TAIL
  // The epilogue has put this workgroup's results into eh_tail_lds as well.  The barrier waits for
  // those LDS stores only, not for the stores to memory; the waves that only fetched have left,
  // the multiplying waves share the outputs.  Unrolled: a work-item's outputs are independent.
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  constexpr int EW_TT = EW_WAVES_M * EW_WAVES_N * 64;
  constexpr int EW_TAIL_FULL = EH_TAIL_PER_GROUP / EW_TT;
#pragma unroll 8
  for (int q = 0; q < EW_TAIL_FULL; ++q) eh_tail_ns::eh_tail((int)g, tid + q * EW_TT EH_TAIL_ARGS);
  if (EW_TAIL_FULL * EW_TT + tid < EH_TAIL_PER_GROUP) eh_tail_ns::eh_tail((int)g, EW_TAIL_FULL * EW_TT + tid EH_TAIL_ARGS);
#endif
}
