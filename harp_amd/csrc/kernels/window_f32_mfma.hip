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
// One workgroup = one group of EW_NG rows of F (the rows that share a patch) x EW_MW rows of A x
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
#define EW_MW 64           // rows of A per workgroup (EW_M split over blockIdx.y)
#define EW_NG 196          // rows of F per group
#define EW_GROUPS 256      // groups per batch element
#define EW_K 288
#define EW_WAVES_M 4
#define EW_WAVES_N 1
#define EW_MB 1
#define EW_NB 13
#define EW_KSTEPS 72
#define EW_NPAT 1
#define EW_PATCH_FLOATS 8688
#define EW_PATCH_ELEMS 8192
#define EW_A_OFF 0LL
#define EW_A_BS 0LL
#define EW_A_SM 288LL
#define EW_A_SK 1LL
#define EW_A_MSPLIT 0LL
#define EW_A_SM2 0LL
#define EW_A_VEC 1         // A is read with 128-bit loads along k
#define EW_KPAD 288        // K rounded up to a multiple of four
#define EW_A_LDS 292       // floats between rows of A in LDS
#define EH_C_OFF 0LL
#define EH_C_BS 0LL
#define EH_C_SM 196LL
#define EH_C_SN 1LL
#define EH_C_MSPLIT 0LL
#define EH_C_SM2 0LL
#define EH_C_NSPLIT 196LL
#define EH_C_SN2 12544LL
#define EW_SRC_BYTES 6422528u
#define EW_KDELTA 9         // k of sub-step j of step s: ew_k0[s] + j * EW_KDELTA
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
#endif

#ifndef EH_EPILOGUE
#define EH_EPI_PARAMS
#define EH_EPI_ARGS
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

typedef float ew_f4v __attribute__((ext_vector_type(4)));

namespace {
constexpr int EW_NT = EW_WAVES_M * EW_WAVES_N * 64;

// offset of position v along an axis of stride S, or of SPLIT positions of stride S inside extents S2 apart
template <long long SPLIT, long long S, long long S2>
__device__ __forceinline__ long long ew_axis_offset(long long v) {
  constexpr long long D = SPLIT > 0 ? SPLIT : 1;
  return SPLIT > 0 ? (v / D) * S2 + (v % D) * S : v * S;
}
}  // namespace

extern "C" __global__ void __launch_bounds__(EW_NT)
EW_ENTRY(const float* __restrict__ A, const float* __restrict__ F EH_C_PARAM EH_EPI_PARAMS) {
  constexpr int MROWS = EW_WAVES_M * EW_MB * 16;        // rows of A a workgroup multiplies (padding rows are zero)
  __shared__ __attribute__((aligned(16))) float patch[EW_PATCH_FLOATS];
  __shared__ __attribute__((aligned(16))) float As[MROWS * EW_A_LDS];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wid = tid >> 6;
  const int wm = wid % EW_WAVES_M, wn = wid / EW_WAVES_M;
  const int l16 = lane & 15, j4 = lane >> 4;
  const long long g = blockIdx.x, bz = blockIdx.z;
  const int m_wg = blockIdx.y * EW_MW;

  // A's rows of this workgroup into LDS, read along whichever of its axes is contiguous in memory
  // (128-bit loads where rows allow); k beyond K and rows beyond M are zero.  Every load of a chunk is
  // issued before the first value is stored: a workgroup is alone on its CU for most of its life, so
  // nothing else would hide one load's latency behind another's.
  {
    const float* a0 = A + EW_A_OFF + bz * EW_A_BS;
#if EW_A_VEC
    constexpr int KQ = EW_KPAD / 4;
    constexpr int PER = (MROWS * KQ + EW_NT - 1) / EW_NT;
    constexpr int CH = PER < 24 ? PER : 24;
    for (int c0 = 0; c0 < PER; c0 += CH) {
      ew_f4v v[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        const int m = e / KQ, kq = e % KQ;
        const bool ok = e < MROWS * KQ && m_wg + m < EW_M && m < EW_MW && kq * 4 < EW_K;
        const long long mo = ew_axis_offset<EW_A_MSPLIT, EW_A_SM, EW_A_SM2>(ok ? m_wg + m : 0);
        const ew_f4v x = *reinterpret_cast<const ew_f4v*>(a0 + mo + (ok ? kq * 4 : 0));
        v[u] = ok ? x : ew_f4v{0.0f, 0.0f, 0.0f, 0.0f};
      }
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        if (e < MROWS * KQ) *reinterpret_cast<ew_f4v*>(&As[(e / KQ) * EW_A_LDS + (e % KQ) * 4]) = v[u];
      }
    }
#else
    constexpr int PER = (MROWS * EW_KPAD + EW_NT - 1) / EW_NT;
    constexpr int CH = PER < 32 ? PER : 32;
    for (int c0 = 0; c0 < PER; c0 += CH) {
      float v[CH];
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        // consecutive work-items along the axis with the smaller stride
        const int m = EW_A_SK <= EW_A_SM ? e / EW_KPAD : e % MROWS;
        const int k = EW_A_SK <= EW_A_SM ? e % EW_KPAD : e / MROWS;
        const bool ok = e < MROWS * EW_KPAD && m_wg + m < EW_M && m < EW_MW && k < EW_K;
        const long long mo = ew_axis_offset<EW_A_MSPLIT, EW_A_SM, EW_A_SM2>(ok ? m_wg + m : 0);
        const float x = a0[mo + (ok ? (long long)k * EW_A_SK : 0LL)];
        v[u] = ok ? x : 0.0f;
      }
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const int e = (c0 + u) * EW_NT + tid;
        const int m = EW_A_SK <= EW_A_SM ? e / EW_KPAD : e % MROWS;
        const int k = EW_A_SK <= EW_A_SM ? e % EW_KPAD : e / MROWS;
        if (e < MROWS * EW_KPAD) As[m * EW_A_LDS + k] = v[u];
      }
    }
#endif
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

  ew_f4v acc[EW_MB][EW_NB];
#pragma unroll
  for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < EW_NB; ++nb) acc[mb][nb] = ew_f4v{0.0f, 0.0f, 0.0f, 0.0f};

  // step s multiplies with the operands fetched during step s - 1
  float a[2][EW_MB], b[2][EW_NB];
#pragma unroll
  for (int mb = 0; mb < EW_MB; ++mb) a[0][mb] = As[abase[mb] + ew_k0[0]];
#pragma unroll
  for (int nb = 0; nb < EW_NB; ++nb) b[0][nb] = patch[base[nb][ew_kpat[0]] + ew_koff[0]];
#pragma unroll
  for (int s = 0; s < EW_KSTEPS; ++s) {
    if (s + 1 < EW_KSTEPS) {
#pragma unroll
      for (int mb = 0; mb < EW_MB; ++mb) a[(s + 1) & 1][mb] = As[abase[mb] + ew_k0[s + 1]];
#pragma unroll
      for (int nb = 0; nb < EW_NB; ++nb) b[(s + 1) & 1][nb] = patch[base[nb][ew_kpat[s + 1]] + ew_koff[s + 1]];
    }
#pragma unroll
    for (int nb = 0; nb < EW_NB; ++nb)
#pragma unroll
      for (int mb = 0; mb < EW_MB; ++mb)
        acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s & 1][mb], b[s & 1][nb], acc[mb][nb], 0, 0, 0);
#if EW_MIX
    // (one LDS read after every MFMA; the reads of A's values ride with the first ones)
#pragma unroll
    for (int q = 0; q < EW_MB; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int q = EW_MB; q < EW_NB * EW_MB; ++q) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
#endif
    __builtin_amdgcn_sched_barrier(0);
  }

  // Accumulator register v of lane l holds row 4 * (l / 16) + v of the M-block, column l % 16 of the
  // N-block.  Blocks that lie inside the group whole are finished without a test per element, in one
  // run of straight-line code: whatever the epilogue loads (a bias, a saved activation) is then
  // requested for all of them before the first store goes out, where a branch around every element
  // would make each element's load wait for the stores of the one before (one queue for both).
  constexpr bool M_EDGE = EW_M % 16 != 0 || EW_MW % 16 != 0 || MROWS != EW_MW;
  auto finish = [&](const int mb, const int nb, const int v, const bool test) {
    const int m = m_wg + (wm * EW_MB + mb) * 16 + 4 * j4 + v;
    const int n = (nb * EW_WAVES_N + wn) * 16 + l16;
    if (test && !(m < EW_M && m < m_wg + EW_MW && n < EW_NG)) return;
    const long long crow = ew_axis_offset<EH_C_MSPLIT, EH_C_SM, EH_C_SM2>(m);
    const long long ccol = ew_axis_offset<EH_C_NSPLIT, EH_C_SN, EH_C_SN2>(g * EW_NG + n);
    const long long e = EH_C_OFF + bz * EH_C_BS + crow + ccol;
#if defined(EH_EPILOGUE)
    eh_epilogue(e, acc[mb][nb][v] EH_C_ARG EH_EPI_ARGS);
#else
    C[e] = acc[mb][nb][v];
#endif
  };
#pragma unroll
  for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < EW_NB; ++nb)
      if (!M_EDGE && (nb + 1) * EW_WAVES_N * 16 <= EW_NG) {
#pragma unroll
        for (int v = 0; v < 4; ++v) finish(mb, nb, v, false);
      }
#pragma unroll
  for (int mb = 0; mb < EW_MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < EW_NB; ++nb)
      if (M_EDGE || (nb + 1) * EW_WAVES_N * 16 > EW_NG) {
#pragma unroll
        for (int v = 0; v < 4; ++v) finish(mb, nb, v, true);
      }
}
