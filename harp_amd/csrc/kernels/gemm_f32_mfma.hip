// FP32 contraction C[m,n] = sum_k A[m,k] * B[k,n] on CDNA4 matrix cores (gfx950).
//
// One workgroup owns a BM x BN tile of C and walks K in steps of BK.  Each wave owns a WM x WN
// sub-tile as (WM/32) x (WN/32) accumulators of v_mfma_f32_32x32x2_f32.
//
// LDS holds each operand tile in the layout its global layout allows to be written with one
// 128-bit store per thread, so nothing is transposed on the way in:
//   * an operand whose contiguous axis is k is kept as [k/4][row][4]: a thread's four
//     consecutive k values of one row are one LDS element, and a lane later reads the four
//     with one ds_read_b128;
//   * an operand whose contiguous axis is the row (m for A, n for B) is kept as [k][row].
// The sum over k does not care which k value goes to which MFMA, so inside a block of eight
// k values MFMA e (e = 0..3) multiplies k = 8j+e on lanes 0-31 and k = 8j+4+e on lanes 32-63:
// that is what makes the four-k element usable as is.  Rows are padded by four floats
// (elements) so that stores and reads spread over the banks.
//
// Two LDS buffers; the global loads of tile t+1 are issued before tile t is multiplied, the
// LDS operands of k-block j+1 are fetched while block j is multiplied, and the last block of a
// tile step is multiplied after the next tile has been published (store, barrier) and its
// first operands requested.  Workgroup ids are remapped so that each XCD (ids congruent mod
// 8) works on a compact block of tiles and shares A/B panels through its own L2.
// An operand can also be computed instead of loaded: when a gather or copy kernel (im2col,
// a layout change, padding) would have produced it, the generator passes that kernel as a
// function of the element index and the tile loader calls it (implicit GEMM).
// Sizes need not be multiples of the tile (edge tiles load zeros and skip stores), operands
// that cannot be read as aligned 128-bit vectors are read element by element, and a long K
// with few output tiles can be split over blockIdx.y into partial sums.
//
// The generator defines the EH_* macros; the defaults below make the file compile on its own.
#ifndef __HIPCC_RTC__
#include <hip/hip_runtime.h>
#endif

#ifndef EH_ENTRY
#define EH_ENTRY ehk_gemm_default
#define EH_M 4096
#define EH_N 4096
#define EH_K 4096
#define EH_BATCH 1
#define EH_BM 128
#define EH_BN 128
#define EH_BK 16
#define EH_WM 64
#define EH_WN 64
#define EH_A_KCONTIG 1
#define EH_B_NCONTIG 1
#define EH_A_VEC 1
#define EH_B_VEC 1
#define EH_A_SM 4096LL
#define EH_A_SK 1LL
#define EH_B_SK 4096LL
#define EH_B_SN 1LL
#define EH_C_SM 4096LL
#define EH_C_SN 1LL
#define EH_A_OFF 0
#define EH_B_OFF 0
#define EH_C_OFF 0
#define EH_A_BS 0
#define EH_B_BS 0
#define EH_C_BS 0
#define EH_SPLITK 1
#define EH_GROUP_M 8
#endif
#ifndef EH_SETPRIO
#define EH_SETPRIO 0     // wave priority while multiplying
#endif
#ifndef EH_LOAD_BRANCH
#define EH_LOAD_BRANCH 0  // element-by-element tile loads: a branch around each out-of-range element (1) or a clamped index and a select (0)
#endif
// A row-contiguous operand read with 128-bit loads is kept in LDS in the k-contiguous layout too
// ([k/4][row][4], one ds_read_b128 per four MFMAs instead of four scalar reads): the four lanes of
// a quad load the same four rows at four consecutive k and exchange elements (a 4x4 transpose
// over the quad, DPP quad permutes) before the store.  Off by default: the exchange costs about
// thirty vector instructions per 128-bit load, issued through the same port as the MFMAs, which
// outweighs the cheaper reads (4096^3: 135 against 140 TFLOP/s); EH_TRANSPOSE 0 keeps [k][row].
#ifndef EH_TRANSPOSE
#define EH_TRANSPOSE 0
#endif
#ifndef EH_A_MSPLIT
#define EH_A_MSPLIT 0     // rows of A per inner extent when its row axis is split in memory (0: one stride)
#define EH_A_SM2 0
#endif
#ifndef EH_B_NSPLIT
#define EH_B_NSPLIT 0
#define EH_B_SN2 0
#endif
#ifndef EH_C_MSPLIT
#define EH_C_MSPLIT 0     // rows of C per inner extent when its row axis is split in memory; likewise its columns
#define EH_C_SM2 0
#define EH_C_NSPLIT 0
#define EH_C_SN2 0
#endif
#ifndef EH_PREFETCH
#define EH_PREFETCH 1     // how many tile steps ahead of their use the global loads are issued
#endif
#ifndef EH_MIX
#define EH_MIX 1         // LDS operand reads are issued one at a time between the MFMAs of the block before
#endif
// The operand reads of a k-block and the MFMAs of the block before it, as one scheduling region:
// with EH_MIX the reads go out one after every MFMA instead of all at once.  Sixteen waves that
// leave a barrier together and each issue all their reads first fill the LDS queue, and a wave
// whose read cannot issue cannot issue the MFMAs behind it either (in-order issue): the matrix
// cores then wait for the LDS to drain.  Spread out, a read is still more than half a block
// (hundreds of cycles) ahead of its first use.  0x008: MFMA, 0x100: LDS read.
#if EH_MIX
#define EH_MIX_REGION()                                         \
  _Pragma("unroll") for (int eh_g = 0; eh_g < 12; ++eh_g) {     \
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);          \
    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);          \
  }
#define EH_FETCH_FENCE()
#else
#define EH_MIX_REGION()
#define EH_FETCH_FENCE() __builtin_amdgcn_sched_barrier(0)
#endif

typedef float eh_f16v __attribute__((ext_vector_type(16)));
typedef float eh_f4v __attribute__((ext_vector_type(4)));

namespace {
constexpr int BM = EH_BM, BN = EH_BN, BK = EH_BK, WM = EH_WM, WN = EH_WN;
constexpr int NWM = BM / WM, NWN = BN / WN, NT = NWM * NWN * 64;
// A row-contiguous operand whose tile needs no guards goes from global memory straight into
// LDS (global_load_lds_dwordx4: lane i of a wave writes its 16 bytes at base + 16*i): work-item
// q's four elements are element q of the unpadded [k][row] tile, so a wave's 64 loads fill
// 1 KiB of consecutive LDS and neither registers nor ds_write are involved.  (For a
// k-contiguous operand the lanes would have to take one row each, 16 bytes per cache line:
// measured 7 % slower than staging it through registers.)
#ifndef EH_A_DMA
#define EH_A_DMA 0
#endif
#ifndef EH_B_DMA
#define EH_B_DMA 0
#endif
#ifdef EH_A_FOLD
#define EH_A_TR 0
#else
#define EH_A_TR (EH_TRANSPOSE && !EH_A_KCONTIG && EH_A_VEC && !EH_A_DMA)
#endif
#ifdef EH_B_FOLD
#define EH_B_TR 0
#else
#define EH_B_TR (EH_TRANSPOSE && EH_B_NCONTIG && EH_B_VEC && !EH_B_DMA)
#endif
constexpr int AS = BM + (EH_A_DMA ? 0 : 4), BS = BN + (EH_B_DMA ? 0 : 4);   // (padded) rows per k in LDS
constexpr int AV = BM * BK / 4 / NT, BV = BN * BK / 4 / NT;   // 4-element loads per thread per tile
constexpr int IB = WM / 32, JB = WN / 32;
constexpr int NBLK = BK / 8;                       // blocks of eight k values per tile step
constexpr long long M = EH_M, N = EH_N, K = EH_K;
constexpr int TM = (EH_M + BM - 1) / BM, TN = (EH_N + BN - 1) / BN, NTILES = TM * TN;
constexpr int KT_ALL = (EH_K + BK - 1) / BK;
constexpr int KT = (KT_ALL + EH_SPLITK - 1) / EH_SPLITK;      // k-steps per split
// Ragged sizes: rows/columns past the end are loaded as zero and never stored.
constexpr bool EDGE_M = EH_M % BM != 0, EDGE_N = EH_N % BN != 0;
constexpr bool EDGE_K = EH_K % BK != 0 || KT_ALL % EH_SPLITK != 0;
static_assert(BM * BK % (4 * NT) == 0 && BN * BK % (4 * NT) == 0 && AV >= 1 && BV >= 1, "tile does not split over the threads");
static_assert(WM % 32 == 0 && WN % 32 == 0 && BK % 16 == 0, "wave tile must be built from 32x32x2 MFMAs, k in pairs of blocks of eight");
// 128-bit loads need the four elements to be in range together
static_assert(!EH_A_VEC || (EH_A_KCONTIG ? EH_K % 4 == 0 : EH_M % 4 == 0), "A cannot be loaded as vectors");
static_assert(!EH_B_VEC || (EH_B_NCONTIG ? EH_N % 4 == 0 : EH_K % 4 == 0), "B cannot be loaded as vectors");

// How an operand's element (batch bz, row r, k) is obtained: from memory at
// off + bz*bs + r*sr + k*sk, or (EH_A_FOLD / EH_B_FOLD) by evaluating the elementwise kernel
// that would have produced that element, on that kernel's own source.  Either way in three
// steps, so that what depends on the row alone is worked out once per work-item, ahead of the
// k loop, and what depends on k alone once per k: row(bz, r) and kk(bz, k) decode their share of
// the element's index, val(p, row, kk) reads or evaluates the element.  For a computed operand
// the generator splits the producer's loop variables at Q: in mode 1 the row decides the
// variables above Q and k those below, in mode 2 the other way round; in mode 0 the index does
// not separate and val decodes all of it.
// RSPLIT > 0: the row axis runs over two nested extents of the memory it reads (images of RSPLIT
// pixels each, say): row r sits at (r / RSPLIT) * SR2 + (r % RSPLIT) * SR.  Rows are decoded
// once per work-item, so the division is off the k loop.
template <long long OFF, long long BS, long long SR, long long SK, long long RSPLIT, long long SR2>
struct EhFromMemory {
  typedef long long Row;
  typedef long long Kk;
  __device__ __forceinline__ static Row row(long long bz, long long r) {
    if (RSPLIT > 0) return OFF + bz * BS + (r / RSPLIT) * SR2 + (r % RSPLIT) * SR;
    return OFF + bz * BS + r * SR;
  }
  __device__ __forceinline__ static Kk kk(long long, long long k) { return k * SK; }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) { return p[r + k]; }
  __device__ __forceinline__ static long long mem(const Row& r) { return r; }     // a row's offset in memory (128-bit path)
};
#ifdef EH_A_FOLD
struct EhAElem {
  static constexpr long long Q = EH_A_FOLD_Q;
  template <class R> __device__ __forceinline__ static long long mem(const R&) { return 0; }   // never read as vectors
#if EH_A_FOLD_MODE == 1
  typedef eh_a_upper Row;
  typedef eh_a_lower Kk;
  __device__ __forceinline__ static Row row(long long bz, long long r) { return eh_a_dec_upper(EH_A_OFF / Q + bz * (EH_A_BS / Q) + r * (EH_A_SM / Q)); }
  __device__ __forceinline__ static Kk kk(long long, long long k) { return eh_a_dec_lower(k * EH_A_SK); }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) { return eh_a_val(p, r, k); }
#elif EH_A_FOLD_MODE == 2
  typedef eh_a_lower Row;
  typedef eh_a_upper Kk;
  __device__ __forceinline__ static Row row(long long, long long r) { return eh_a_dec_lower(r * EH_A_SM); }
  __device__ __forceinline__ static Kk kk(long long bz, long long k) { return eh_a_dec_upper(EH_A_OFF / Q + bz * (EH_A_BS / Q) + k * (EH_A_SK / Q)); }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) { return eh_a_val(p, k, r); }
#else
  typedef long long Row;
  typedef long long Kk;
  __device__ __forceinline__ static Row row(long long bz, long long r) { return EH_A_OFF + bz * EH_A_BS + r * EH_A_SM; }
  __device__ __forceinline__ static Kk kk(long long, long long k) { return k * EH_A_SK; }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) {
    return eh_a_val(p, eh_a_dec_upper(0), eh_a_dec_lower(r + k));
  }
#endif
};
#else
using EhAElem = EhFromMemory<EH_A_OFF, EH_A_BS, EH_A_SM, EH_A_SK, EH_A_MSPLIT, EH_A_SM2>;
#endif
#ifdef EH_B_FOLD
struct EhBElem {
  static constexpr long long Q = EH_B_FOLD_Q;
  template <class R> __device__ __forceinline__ static long long mem(const R&) { return 0; }   // never read as vectors
#if EH_B_FOLD_MODE == 1
  typedef eh_b_upper Row;
  typedef eh_b_lower Kk;
  __device__ __forceinline__ static Row row(long long bz, long long r) { return eh_b_dec_upper(EH_B_OFF / Q + bz * (EH_B_BS / Q) + r * (EH_B_SN / Q)); }
  __device__ __forceinline__ static Kk kk(long long, long long k) { return eh_b_dec_lower(k * EH_B_SK); }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) { return eh_b_val(p, r, k); }
#elif EH_B_FOLD_MODE == 2
  typedef eh_b_lower Row;
  typedef eh_b_upper Kk;
  __device__ __forceinline__ static Row row(long long, long long r) { return eh_b_dec_lower(r * EH_B_SN); }
  __device__ __forceinline__ static Kk kk(long long bz, long long k) { return eh_b_dec_upper(EH_B_OFF / Q + bz * (EH_B_BS / Q) + k * (EH_B_SK / Q)); }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) { return eh_b_val(p, k, r); }
#else
  typedef long long Row;
  typedef long long Kk;
  __device__ __forceinline__ static Row row(long long bz, long long r) { return EH_B_OFF + bz * EH_B_BS + r * EH_B_SN; }
  __device__ __forceinline__ static Kk kk(long long, long long k) { return k * EH_B_SK; }
  __device__ __forceinline__ static float val(const float* __restrict__ p, const Row& r, const Kk& k) {
    return eh_b_val(p, eh_b_dec_upper(0), eh_b_dec_lower(r + k));
  }
#endif
};
#else
using EhBElem = EhFromMemory<EH_B_OFF, EH_B_BS, EH_B_SN, EH_B_SK, EH_B_NSPLIT, EH_B_SN2>;
#endif

// The rows a work-item reads of an operand tile, decoded once: one row (the four elements run
// along k) or four neighbouring ones (the four run along the row axis).  Rows past the end
// decode row 0 and are marked.
template <class ELEM, bool ALONG_K>
struct EhRows {
  static constexpr int NR = ALONG_K ? 1 : 4;
  typename ELEM::Row row[NR];
  bool ok[NR];
  __device__ __forceinline__ void set(long long bz, long long r, long long R) {
#pragma unroll
    for (int e = 0; e < NR; ++e) {
      ok[e] = r + e < R;
      row[e] = ELEM::row(bz, ok[e] ? r + e : 0);
    }
  }
};

// Four elements of an operand starting at (r, k) and running along its fast axis; elements
// outside [0,R) x [0,kend) read as zero.  ALONG_K says which axis the four run along; `base`
// is the operand's offset plus the batch offset (used by the 128-bit path), `rows` the decoded
// rows (used by the element-by-element path).
template <class ELEM, bool VEC, bool ALONG_K, bool EDGE_R, long long SR, long long SK>
__device__ __forceinline__ eh_f4v eh_tile_load(const float* __restrict__ p, long long base, long long bz, long long r,
                                              long long k, long long R, long long kend, const EhRows<ELEM, ALONG_K>& rows) {
  eh_f4v v = {0.0f, 0.0f, 0.0f, 0.0f};
  if (VEC) {
    // (the first of the work-item's rows: four rows of one vector never straddle a split)
    const bool ok = (!EDGE_R || r < R) && (!EDGE_K || k < kend);
    if (ok) v = *reinterpret_cast<const eh_f4v*>(p + ELEM::mem(rows.row[0]) + k * SK);
  } else if (ALONG_K) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool ok = (!EDGE_R || rows.ok[0]) & (!EDGE_K || k + e < kend);     // (no test where the tiles have no edge)
#if EH_LOAD_BRANCH
      if (ok) v[e] = ELEM::val(p, rows.row[0], ELEM::kk(bz, k + e));
#else
      const float x = ELEM::val(p, rows.row[0], ELEM::kk(bz, ok ? k + e : 0));
      v[e] = ok ? x : 0.0f;
#endif
    }
  } else {
    const bool kok = !EDGE_K || k < kend;
    const typename ELEM::Kk kinfo = ELEM::kk(bz, kok ? k : 0);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool ok = (!EDGE_R || rows.ok[e]) & kok;
#if EH_LOAD_BRANCH
      if (ok) v[e] = ELEM::val(p, rows.row[e], kinfo);
#else
      const float x = ELEM::val(p, rows.row[e], kinfo);
      v[e] = ok ? x : 0.0f;
#endif
    }
  }
  return v;
}

// One operand tile in LDS (RS = padded number of rows).  KC: [k/4][row][4], else [k][row].
template <bool KC, int RS>
struct EhTile {
  // where a thread's four elements go: (row r, k0..k0+3) for KC, (k, rows r0..r0+3) otherwise
  __device__ __forceinline__ static void put(float* t, int r, int k, eh_f4v v) {
    if (KC) *reinterpret_cast<eh_f4v*>(&t[((k >> 2) * RS + r) * 4]) = v;
    else *reinterpret_cast<eh_f4v*>(&t[k * RS + r]) = v;
  }
  // the four operand values of one lane for k-block j: element e feeds MFMA e
  __device__ __forceinline__ static eh_f4v get(const float* t, int j, int kh, int r) {
    if (KC) return *reinterpret_cast<const eh_f4v*>(&t[((2 * j + kh) * RS + r) * 4]);
    eh_f4v v;
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = t[(8 * j + 4 * kh + e) * RS + r];
    return v;
  }
};
using ATile = EhTile<EH_A_KCONTIG != 0 || EH_A_TR, AS>;
using BTile = EhTile<EH_B_NCONTIG == 0 || EH_B_TR, BS>;

// 4x4 transpose over the four lanes of a quad: lane t (= lane & 3) passes row t and gets column t.
// Round s: lane j hands its element j^s to lane j^s, which files it as element j of its result.
template <int CTRL> __device__ __forceinline__ float eh_quad(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float eh_pick4(const eh_f4v& v, int i) {
  return i == 0 ? v[0] : i == 1 ? v[1] : i == 2 ? v[2] : v[3];
}
__device__ __forceinline__ void eh_file4(eh_f4v& v, int i, float x) {
  v[0] = i == 0 ? x : v[0];
  v[1] = i == 1 ? x : v[1];
  v[2] = i == 2 ? x : v[2];
  v[3] = i == 3 ? x : v[3];
}
__device__ __forceinline__ eh_f4v eh_quad_transpose(const eh_f4v& v, int t) {
  eh_f4v out = {0.0f, 0.0f, 0.0f, 0.0f};
  eh_file4(out, t, eh_pick4(v, t));
  eh_file4(out, t ^ 1, eh_quad<0xB1>(eh_pick4(v, t ^ 1)));   // quad_perm [1,0,3,2]
  eh_file4(out, t ^ 2, eh_quad<0x4E>(eh_pick4(v, t ^ 2)));   // quad_perm [2,3,0,1]
  eh_file4(out, t ^ 3, eh_quad<0x1B>(eh_pick4(v, t ^ 3)));   // quad_perm [3,2,1,0]
  return out;
}
}  // namespace

// Epilogue: elementwise kernels that follow the contraction over the same dense index space
// run on each element while it is in the accumulator; eh_epilogue stores what must reach memory
// (C itself only if something else still reads it: EH_NO_C drops the parameter).
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

// offset of position v along an axis of stride S, or of SPLIT positions of stride S inside extents S2 apart
template <long long SPLIT, long long S, long long S2>
__device__ __forceinline__ long long eh_axis_offset(long long v) {
  constexpr long long D = SPLIT > 0 ? SPLIT : 1;
  return SPLIT > 0 ? (v / D) * S2 + (v % D) * S : v * S;
}

#ifndef EH_WAVES_PER_SIMD
#define EH_WAVES_PER_SIMD 4   // register budget: 512 / this many VGPRs+AGPRs per lane
#endif

// EH_PART: this kernel is one of several issued as one launch.  It is then a function of its
// share of the launch's linear workgroup ids (its own grid is EH_PART_GX x EH_PART_GY x batch) and
// of the launch's one block of LDS, which the parts use in turn; eh_lds_floats says how much it needs.
#ifdef EH_PART
#define EH_BLOCK_X (eh_bx % EH_PART_GX)
#define EH_BLOCK_Y (eh_bx / EH_PART_GX % EH_PART_GY)
#define EH_BLOCK_Z (eh_bx / (EH_PART_GX * EH_PART_GY))
constexpr int eh_lds_floats = 2 * BK * (AS + BS);
__device__ __forceinline__ void eh_run(const unsigned eh_bx, float* const eh_lds, const float* __restrict__ A, const float* __restrict__ B EH_C_PARAM EH_EPI_PARAMS) {
  float* const As0 = eh_lds;
  float* const As1 = eh_lds + BK * AS;
  float* const Bs0 = eh_lds + 2 * BK * AS;
  float* const Bs1 = Bs0 + BK * BS;
#if !(EH_A_DMA || EH_B_DMA)
  float (*const As)[BK * AS] = reinterpret_cast<float (*)[BK * AS]>(As0);
  float (*const Bs)[BK * BS] = reinterpret_cast<float (*)[BK * BS]>(Bs0);
  (void)As1;
  (void)Bs1;
#endif
#else
#define EH_BLOCK_X blockIdx.x
#define EH_BLOCK_Y blockIdx.y
#define EH_BLOCK_Z blockIdx.z
extern "C" __global__ void __launch_bounds__(NT) __attribute__((amdgpu_waves_per_eu(EH_WAVES_PER_SIMD, EH_WAVES_PER_SIMD)))
EH_ENTRY(const float* __restrict__ A, const float* __restrict__ B EH_C_PARAM EH_EPI_PARAMS) {
  // two tiles per operand, as separate arrays: the compiler then knows that a direct-to-LDS
  // load into one does not touch what is being read from the other
#if EH_A_DMA || EH_B_DMA
  __shared__ __attribute__((aligned(16))) float As0[BK * AS];
  __shared__ __attribute__((aligned(16))) float As1[BK * AS];
  __shared__ __attribute__((aligned(16))) float Bs0[BK * BS];
  __shared__ __attribute__((aligned(16))) float Bs1[BK * BS];
#else
  __shared__ __attribute__((aligned(16))) float As[2][BK * AS];
  __shared__ __attribute__((aligned(16))) float Bs[2][BK * BS];
  float* const As0 = As[0];
  float* const Bs0 = Bs[0];
#endif
#endif

  const int tid = threadIdx.x;
  const int lane = tid & 63, wid = tid >> 6;
  const int wm = wid / NWN, wn = wid % NWN;
  const int l32 = lane & 31, kh = lane >> 5;

  // workgroup -> tile: compact per XCD, then grouped along M so neighbours share B panels
  int tile = EH_BLOCK_X;
  if (NTILES % 8 == 0) tile = (tile % 8) * (NTILES / 8) + tile / 8;
  constexpr int GM = EH_GROUP_M < TM ? EH_GROUP_M : TM;
  const int group = tile / (GM * TN);
  const int first_m = group * GM;
  const int gsz = (TM - first_m) < GM ? (TM - first_m) : GM;
  const int in_g = tile - group * GM * TN;
  const int tm = first_m + in_g % gsz;
  const int tn = in_g / gsz;
  const long long m0 = (long long)tm * BM, n0 = (long long)tn * BN;

  const long long bz = EH_BLOCK_Z;
  const long long a_base = EH_A_OFF + bz * EH_A_BS, b_base = EH_B_OFF + bz * EH_B_BS;
#if EH_SPLITK > 1
  // partial sums go to a dense [split][batch][M][N] scratch; a second launch adds them up
  const long long kbeg = (long long)EH_BLOCK_Y * KT * BK;
  const long long kend = (kbeg + (long long)KT * BK) < K ? (kbeg + (long long)KT * BK) : K;
  float* Cb = C + ((long long)EH_BLOCK_Y * EH_BATCH + bz) * (M * N);
  constexpr long long CSM = N, CSN = 1;
#elif defined(EH_EPILOGUE)
  const long long kbeg = 0, kend = K;
#else
  const long long kbeg = 0, kend = K;
  float* Cb = C + EH_C_OFF + bz * EH_C_BS;
#endif

  // Register stages of tiles on their way from global memory to LDS.  One stage: the tile of the
  // next step.  With EH_PREFETCH = P > 1 there are P + 1 stages and the loads run P steps ahead: a
  // small tile multiplies for a fraction of a load's latency, and with few workgroups on a CU
  // nothing else would fill the wait.
  constexpr int NSTAGE = (EH_PREFETCH > 1 && !(EH_A_DMA || EH_B_DMA)) ? EH_PREFETCH + 1 : 1;
  eh_f4v ra[NSTAGE][AV], rb[NSTAGE][BV];
  // the rows of each tile this work-item fetches, decoded once (they do not change with k)
  EhRows<EhAElem, EH_A_KCONTIG != 0> a_rows[AV];
  EhRows<EhBElem, EH_B_NCONTIG == 0> b_rows[BV];
#if !EH_A_DMA
#pragma unroll
  for (int i = 0; i < AV; ++i) {
    const int q = tid + i * NT;
    a_rows[i].set(bz, EH_A_KCONTIG ? m0 + q / (BK / 4) : EH_A_TR ? m0 + ((q >> 2) % (BM / 4)) * 4 : m0 + (q % (BM / 4)) * 4, M);
  }
#endif
#if !EH_B_DMA
#pragma unroll
  for (int i = 0; i < BV; ++i) {
    const int q = tid + i * NT;
    b_rows[i].set(bz, EH_B_TR ? n0 + ((q >> 2) % (BN / 4)) * 4 : EH_B_NCONTIG ? n0 + (q % (BN / 4)) * 4 : n0 + q / (BK / 4), N);
  }
#endif

  // thread q of the tile owns four elements: along k at (row q / (BK/4), k 4*(q % (BK/4))) for
  // a k-contiguous operand, along the row at (k q / (rows/4), row 4*(q % (rows/4))) otherwise
  auto to_lds = [&](const float* gp, float* tile, int q_wave) {
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)gp,
                                     (__attribute__((address_space(3))) void*)(tile + q_wave * 4), 16, 0, 0);
  };
  auto gload = [&](int kt, float* a_tile, float* b_tile, const int stage) {
    (void)a_tile;
    (void)b_tile;
    const long long k0 = kbeg + (long long)kt * BK;
#pragma unroll
    for (int i = 0; i < AV; ++i) {
      const int q = tid + i * NT;
#if EH_A_DMA
      const int k = q / (BM / 4), mq = q % (BM / 4);
      to_lds(A + a_base + (k0 + k) * EH_A_SK + (m0 + mq * 4) * EH_A_SM, a_tile, (tid & ~63) + i * NT);
#elif EH_A_KCONTIG
      const int m = q / (BK / 4), kq = q % (BK / 4);
      ra[stage][i] = eh_tile_load<EhAElem, EH_A_VEC, true, EDGE_M, EH_A_SM, EH_A_SK>(A, a_base, bz, m0 + m, k0 + kq * 4, M, kend, a_rows[i]);
#elif EH_A_TR
      // quad = four consecutive k of the same four rows
      const int k = ((q >> 2) / (BM / 4)) * 4 + (q & 3), mq = (q >> 2) % (BM / 4);
      ra[stage][i] = eh_tile_load<EhAElem, EH_A_VEC, false, EDGE_M, EH_A_SM, EH_A_SK>(A, a_base, bz, m0 + mq * 4, k0 + k, M, kend, a_rows[i]);
#else
      const int k = q / (BM / 4), mq = q % (BM / 4);
      ra[stage][i] = eh_tile_load<EhAElem, EH_A_VEC, false, EDGE_M, EH_A_SM, EH_A_SK>(A, a_base, bz, m0 + mq * 4, k0 + k, M, kend, a_rows[i]);
#endif
    }
#pragma unroll
    for (int i = 0; i < BV; ++i) {
      const int q = tid + i * NT;
#if EH_B_DMA
      const int k = q / (BN / 4), nq = q % (BN / 4);
      to_lds(B + b_base + (k0 + k) * EH_B_SK + (n0 + nq * 4) * EH_B_SN, b_tile, (tid & ~63) + i * NT);
#elif EH_B_TR
      const int k = ((q >> 2) / (BN / 4)) * 4 + (q & 3), nq = (q >> 2) % (BN / 4);
      rb[stage][i] = eh_tile_load<EhBElem, EH_B_VEC, false, EDGE_N, EH_B_SN, EH_B_SK>(B, b_base, bz, n0 + nq * 4, k0 + k, N, kend, b_rows[i]);
#elif EH_B_NCONTIG
      const int k = q / (BN / 4), nq = q % (BN / 4);
      rb[stage][i] = eh_tile_load<EhBElem, EH_B_VEC, false, EDGE_N, EH_B_SN, EH_B_SK>(B, b_base, bz, n0 + nq * 4, k0 + k, N, kend, b_rows[i]);
#else
      const int n = q / (BK / 4), kq = q % (BK / 4);
      rb[stage][i] = eh_tile_load<EhBElem, EH_B_VEC, true, EDGE_N, EH_B_SN, EH_B_SK>(B, b_base, bz, n0 + n, k0 + kq * 4, N, kend, b_rows[i]);
#endif
    }
  };

  auto sstore = [&](float* a_tile, float* b_tile, const int stage) {
    (void)a_tile;
    (void)b_tile;
#if !EH_A_DMA
#pragma unroll
    for (int i = 0; i < AV; ++i) {
      const int q = tid + i * NT;
#if EH_A_KCONTIG
      ATile::put(a_tile, q / (BK / 4), (q % (BK / 4)) * 4, ra[stage][i]);
#elif EH_A_TR
      ATile::put(a_tile, ((q >> 2) % (BM / 4)) * 4 + (q & 3), ((q >> 2) / (BM / 4)) * 4, eh_quad_transpose(ra[stage][i], q & 3));
#else
      ATile::put(a_tile, (q % (BM / 4)) * 4, q / (BM / 4), ra[stage][i]);
#endif
    }
#endif
#if !EH_B_DMA
#pragma unroll
    for (int i = 0; i < BV; ++i) {
      const int q = tid + i * NT;
#if EH_B_TR
      BTile::put(b_tile, ((q >> 2) % (BN / 4)) * 4 + (q & 3), ((q >> 2) / (BN / 4)) * 4, eh_quad_transpose(rb[stage][i], q & 3));
#elif EH_B_NCONTIG
      BTile::put(b_tile, (q % (BN / 4)) * 4, q / (BN / 4), rb[stage][i]);
#else
      BTile::put(b_tile, q / (BK / 4), (q % (BK / 4)) * 4, rb[stage][i]);
#endif
    }
#endif
#if EH_A_DMA || EH_B_DMA
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wave's direct-to-LDS loads have landed
#endif
  };

  eh_f16v acc[IB][JB];
#pragma unroll
  for (int i = 0; i < IB; ++i)
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  gload(0, As0, Bs0, 0);
  if (NSTAGE > 1) {
    // the tiles of the first steps leave together
#pragma unroll
    for (int t = 1; t < NSTAGE - 1; ++t)
      if (t < KT) gload(t, As0, Bs0, t);
  }
  sstore(As0, Bs0, 0);
  __syncthreads();

  // two register slots of operands: block j+1 is fetched while block j is multiplied
  eh_f4v a[2][IB], b[2][JB];
  auto fetch = [&](const float* a_tile, const float* b_tile, int j, int slot) {
#pragma unroll
    for (int i = 0; i < IB; ++i) a[slot][i] = ATile::get(a_tile, j, kh, wm * WM + i * 32 + l32);
#pragma unroll
    for (int jj = 0; jj < JB; ++jj) b[slot][jj] = BTile::get(b_tile, j, kh, wn * WN + jj * 32 + l32);
  };
  auto multiply = [&](int slot) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int i = 0; i < IB; ++i)
#pragma unroll
        for (int jj = 0; jj < JB; ++jj)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[slot][i][e], b[slot][jj][e], acc[i][jj], 0, 0, 0);
  };
  // one tile step: multiply the tile in (a_cur, b_cur) while the next one travels to (a_nxt, b_nxt)
  // (`more`: a next tile exists; a literal in the unrolled loop, uniform otherwise)
  // (`load_kt`, `load_stage`: the tile whose loads leave in this step and where they land;
  //  `store_stage`: where the next step's tile has landed)
  auto step = [&](int kt, float* a_cur, float* b_cur, float* a_nxt, float* b_nxt, const bool more, const bool load,
                  const int load_kt, const int load_stage, const int store_stage) {
    if (load) {
      gload(load_kt, a_nxt, b_nxt, load_stage);
      // keep the global loads up here: their latency is hidden by the whole multiply loop only
      // if they are issued before it (the compiler would otherwise sink them to their use)
      asm volatile("" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    }
#if EH_SETPRIO
    __builtin_amdgcn_s_setprio(EH_SETPRIO);
#endif
#pragma unroll
    for (int j = 0; j < NBLK - 1; ++j) {
      fetch(a_cur, b_cur, j + 1, (j + 1) & 1);
      EH_FETCH_FENCE();                    // (without EH_MIX) reads of the next block stay ahead of these MFMAs
      multiply(j & 1);
      EH_MIX_REGION();
      __builtin_amdgcn_sched_barrier(0);
    }
#if EH_SETPRIO
    __builtin_amdgcn_s_setprio(0);
#endif
    if (more) sstore(a_nxt, b_nxt, store_stage);
    __syncthreads();
    if (more) fetch(a_nxt, b_nxt, 0, NBLK & 1);
    EH_FETCH_FENCE();
    multiply((NBLK - 1) & 1);
    EH_MIX_REGION();
    __builtin_amdgcn_sched_barrier(0);
  };

  fetch(As0, Bs0, 0, 0);
#if !(EH_A_DMA || EH_B_DMA)
  if (NSTAGE == 1) {
    // one loop body, buffers chosen by the step's parity
    for (int kt = 0; kt < KT; ++kt) {
      const int buf = kt & 1;
      step(kt, As[buf], Bs[buf], As[buf ^ 1], Bs[buf ^ 1], kt + 1 < KT, kt + 1 < KT, kt + 1, 0, 0);
    }
  } else {
    // unrolled by the number of stages, so that every stage is a fixed set of registers
    constexpr int P = NSTAGE - 1;
    static_assert(NSTAGE == 1 || NSTAGE % 2 == 0, "an even number of stages keeps the LDS buffer's parity fixed per slot");
    for (int kt0 = 0; kt0 < KT; kt0 += NSTAGE) {
#pragma unroll
      for (int u = 0; u < NSTAGE; ++u) {
        const int kt = kt0 + u;
        if (kt < KT)
          step(kt, As[u & 1], Bs[u & 1], As[(u & 1) ^ 1], Bs[(u & 1) ^ 1], kt + 1 < KT, kt + P < KT, kt + P, (u + P) % NSTAGE,
               (u + 1) % NSTAGE);
      }
    }
  }
#else
  // unrolled by two so that each direct-to-LDS load names its destination array statically
  int kt = 0;
  for (; kt + 2 < KT; kt += 2) {
    step(kt, As0, Bs0, As1, Bs1, true, true, kt + 1, 0, 0);
    step(kt + 1, As1, Bs1, As0, Bs0, true, true, kt + 2, 0, 0);
  }
  if (kt + 2 == KT) {
    step(kt, As0, Bs0, As1, Bs1, true, true, kt + 1, 0, 0);
    step(kt + 1, As1, Bs1, As0, Bs0, false, false, 0, 0, 0);
  } else {
    step(kt, As0, Bs0, As1, Bs1, false, false, 0, 0, 0);
  }
#endif

  // accumulator register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
  for (int i = 0; i < IB; ++i)
#pragma unroll
    for (int j = 0; j < JB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const long long row = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * kh + (r % 4);
        const long long col = n0 + wn * WN + j * 32 + l32;
        if ((!EDGE_M || row < M) && (!EDGE_N || col < N)) {
#if EH_SPLITK > 1
          Cb[row * CSM + col * CSN] = acc[i][j][r];
#else
          // an axis of C may run over two nested extents (pixels inside images)
          const long long crow = eh_axis_offset<EH_C_MSPLIT, EH_C_SM, EH_C_SM2>(row);
          const long long ccol = eh_axis_offset<EH_C_NSPLIT, EH_C_SN, EH_C_SN2>(col);
#if defined(EH_EPILOGUE)
          eh_epilogue(EH_C_OFF + bz * EH_C_BS + crow + ccol, acc[i][j][r] EH_C_ARG EH_EPI_ARGS);
#else
          Cb[crow + ccol] = acc[i][j][r];
#endif
#endif
        }
      }
}
