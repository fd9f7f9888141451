// AST -> HIP C for gfx950 (CDNA4).  Takes the place the reference gives a backend's Renderer
// (src/backend/renderer.rs:20-35, 69-159; crates/backend-cuda/src/renderer.rs for the GPU
// shape of it), but chooses a wave64 schedule from the kernel's structure instead of
// replaying its loops: flat 128-bit elementwise, row programs with DPP + LDS reductions,
// per-output serial reductions, FP32 MFMA contractions.
#pragma once

#include <cstdint>

#include <map>
#include <set>
#include <string>
#include <vector>

#include "analysis.hpp"
#include "ast.hpp"

namespace eh {

struct GenOptions {
  std::string arch = "gfx950";
  bool fuse = true;          // merge compatible kernels of a Program into one launch
  bool vectorize = true;     // 128-bit accesses where alignment allows
  bool transpose = true;     // transposing elementwise groups go through 64x64 LDS tiles
  bool window = true;             // short reduces over gathered windows read the source directly
  int row_threads = 0;       // threads cooperating on one row; 0 = choose from the row length
  int row_elems = 8;         // target elements per thread per row when choosing row_threads
  int flat_block = 256;
  int flat_iters = 4;        // vectors handled by one thread of a flat kernel
  int gemm_bm = 0, gemm_bn = 0, gemm_bk = 0, gemm_wm = 0, gemm_wn = 0;  // 0 = defaults
  int gemm_setprio = 0;               // wave priority during the multiply loop
  int gemm_waves = 0;                 // waves per SIMD the register allocation aims at (0 = from the tile)
  int lanes = 1;                      // streams a program's launches may be spread over (1 = one after the other)
  int lane_us = 100;                  // launches estimated longer than this many microseconds stay on lane 0 (0: no limit)
  bool reindex = true;                // elementwise producers evaluated in a reader that walks another index space
  bool merge_launches = true;         // independent final reductions of a program (parameter updates) are issued as one launch
  bool gemm_tail = true;               // a pooling reduce over a convolution's stored result runs in the convolution's launch
  bool merge_templates = true;        // ... and independent small MFMA contractions (template kernels) as one launch among themselves
  bool rematerialize = true;          // a cheap elementwise temp is evaluated again by a far reader of the same index space instead of being stored for it
  bool ranged_loads = true;           // a folded gather reads its source through a buffer resource: a guarded load is one load at an out-of-range offset where the guard fails
  bool guard_branches = false;        // guarded loads (padding, edges) behind branches instead of clamped indices and selects
  bool gemm_transpose = false;        // row-contiguous operands transposed over lane quads into the k-contiguous LDS layout (measured slower)
  int gemm_prefetch = 0;              // tile steps the global loads run ahead (0: 3 for tiles up to 64x64, else 1)
  bool gemm_mix = true;               // LDS operand reads interleaved with the MFMAs of the block before
  int gemm_dma = 2;                   // global_load_lds for row-contiguous operand tiles: 0 never, 1 wherever possible, 2 B only, 3 A only
  bool gemm_merge_batch = false;      // per-batch contractions summed over the batch become one contraction
  bool gemm_epilogue = true;          // run elementwise consumers of a contraction on its accumulators
  bool gemm_fold = true;              // evaluate gather/copy producers inside the tile loader (implicit GEMM)
  bool gemm_window = true;            // a folded sliding-window gather is staged in LDS once per group of rows instead of evaluated per element
  int window_passes = 0;              // of that schedule: passes over k, each for a share of a wave's blocks, stored while the next multiplies (0: chosen by the number of blocks)
  // options for single launches, "name=value,..." by the launch's key (launch_tune_key of the first kernel it covers):
  // applied on top of the above while that launch is planned (option items "@<key>:name=value", lines of the tuned-options file)
  std::map<unsigned long long, std::string> launch_options;
  int gemm_split_k = -1;              // -1 = decide from the shape, 0/1 = never, n = n chunks
  bool gemm = true;          // use the MFMA contraction schedule when the shape allows
  int nontemporal = -1;      // streaming hint: -1 stores of large outputs, 0 none, 1 stores, 2 loads and stores
  bool normalize = true;     // undo the reference optimiser's rewrites (shifts, tiling, unrolling) before planning
  bool allow_serial = false; // let a kernel no schedule recognises run in one work-item however long its loops are
};

struct LaunchSpec {
  std::string entry;
  std::string source;        // complete translation unit for hiprtc
  std::string schedule;      // human-readable schedule tag, e.g. "row(T=256,V=4,reg)"
  unsigned grid[3] = {1, 1, 1};
  unsigned block[3] = {1, 1, 1};
  unsigned lds_bytes = 0;
  std::vector<std::string> arg_bufs;   // buffer name per kernel parameter, in order
  std::vector<size_t> arg_min_bytes;   // smallest buffer each parameter may bind (0 = unknown)
  std::vector<std::string> kernels;    // names of the lowered kernels this launch covers
  double algo_bytes = 0;               // bytes of each distinct external buffer touched once
  double flops = 0;
  // A launch built from a kernel template that can also be compiled as a part of a larger launch
  // (the template's EH_PART mode): the parameter list of its entry point as written there.
  std::string part_params;
  // Filled in by plan_program once all launches are known:
  std::vector<char> arg_written;       // per parameter: the launch writes that buffer
  std::vector<size_t> arg_full_bytes;  // per parameter: the launch writes every byte of a buffer of exactly this size (0: not known to)
  unsigned long long tune_key = 0;     // launch_tune_key of the first kernel covered: what per-launch options are filed under
  int lane = 0;                        // 0 = the device's stream, 1.. = side streams that run beside it
  std::vector<int> waits;              // launches on other lanes that must have finished first
};

struct ProgramPlan {
  std::vector<LaunchSpec> launches;
  std::vector<BufferInfo> buffers;     // table (possibly synthesised from kernel params)
  std::set<std::string> elided;        // temp buffers that never reach memory
  int lanes = 1;                       // lanes in use (1: every launch on the device's stream)
};

// Plans a whole Program (one or more kernels, executed in order).  When the program carries no
// buffer table every mutable pointer parameter is an output and nothing is elided.
ProgramPlan plan_program(const Node& program, const GenOptions& opt);

// Statement-by-statement rendering of one kernel, as written (one work-item unless the kernel
// already carries group/local id parameters).  Used for forms no schedule recognises.
LaunchSpec render_kernel_as_written(const Node& kernel, const GenOptions& opt);

// One launch per top-level loop nest of such a kernel, the outer loops of a nest spread over
// work-items where their iterations cannot collide; empty when the kernel's form is not covered.
// `extra_buffers`: where a schedule that needs a scratch buffer may declare it (the Program's
// buffer table); null when the caller has no table, and such schedules are then not used.
std::vector<LaunchSpec> render_kernel_outer_parallel(const Node& kernel, const GenOptions& opt,
                                                     std::vector<BufferInfo>* extra_buffers = nullptr);

// The local work size the reference derives from a kernel's dispatch hints
// (src/backend/pipeline.rs:160-192, 475-489): per dimension the largest divisor of the global
// size not above the preferred size, then shrunk until the workgroup fits `max_work_group`.
void fit_local_size(const uint64_t global[3], const uint64_t preferred[3], uint64_t max_work_group, uint64_t local[3]);

// "key=value,key=value" on top of *o (items "@<16 hex digits>:key=value" are filed for that launch).
void apply_options(GenOptions* o, const std::string& text);
GenOptions parse_options(const char* text);       // ... on top of the defaults (and ECLAT_HIP_ARCH)
// FNV-1a (64 bit); a launch's key: of the canonical text of the first lowered kernel it covers,
// the kernel's name and its buffers' names replaced by their positions.
unsigned long long fnv1a(const std::string& text);
unsigned long long launch_tune_key(const Node& kernel);
// `opt` with what is filed for the launch that starts at kernel `anchor`, if anything is.
GenOptions options_for_launch(const GenOptions& opt, const Node& anchor);

// Expression text in HIP C (math calls, literals); exposed for tests.
std::string render_expr_text(const Node& e);

// Shared preamble (vector type, cross-lane reductions).
const std::string& preamble();
// What every generated translation unit of the elementwise / reduce schedules starts with.
std::string kernel_header();

}  // namespace eh
