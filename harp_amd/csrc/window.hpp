// Contractions with a sliding-window operand (a convolution as the reference lowers it,
// crates/nn/src/functional/conv.rs:113-187: pad -> unfold -> permute -> contiguous, then
// broadcast-multiply and sum): the gather folded into the contraction is recognised for what it
// is -- row digits and window digits that add up to source coordinates, guarded where the window
// leaves the image -- and the source region a group of rows reads is staged in LDS once, so that
// the multiply loop reads its operand at "row base + k offset" without guards or index arithmetic
// (kernels/window_f32_mfma.hip).
#pragma once

#include <optional>
#include <string>
#include <utility>
#include <vector>

#include "codegen.hpp"
#include "gemm.hpp"

namespace eh {

// C[m, n] = sum_k A[m, k] * F[n, k], every index a mixed-radix number over loops:
//   M loops    index A and C,
//   row loops  index F and C (the rows of F; groups of them share a patch),
//   k loops    index A and F,
//   batch loops index all three.
// Within a side the loops are listed outermost first; that order defines the flat index.
enum class WSide { Batch, Row, K, M };
struct WLoop {
  std::string name;
  int64_t extent = 1;
  WSide side = WSide::Row;
  int64_t f = 0, a = 0, c = 0;      // strides in F's source (signed), in A, in C (elements)
};
// sum(coef * loop) >= bound (ge) or < bound: where F's source element exists; elsewhere F is 0
struct WGuard {
  std::vector<std::pair<std::string, int64_t>> terms;
  bool ge = false;
  int64_t bound = 0;
};
struct WindowProblem {
  std::string entry;                    // kernel symbol
  std::string what;                     // comment: what F stands for
  std::vector<std::string> kernels;     // lowered kernels the launch covers
  std::vector<WLoop> loops;
  std::vector<WGuard> guards;
  int64_t f_c0 = 0, a_c0 = 0, c_c0 = 0; // constant terms of the three addresses
  std::string a_buf, f_buf, c_buf;
  size_t f_bytes = 0;                   // size of F's source buffer (read through a buffer resource)
  double f_algo_bytes = 0;              // what reading F's source once costs
  std::string tag;                      // appended to the schedule string
};

// The launch, or empty when the problem does not fit one workgroup per group of rows (LDS,
// registers) or has no window structure.
std::vector<LaunchSpec> emit_window(const WindowProblem& p, const GenOptions& opt, const EpilogueSpec* epilogue);

// The launch for contraction `k` (shape `s`, exactly one of `fa` / `fb` given: the folded operand)
// when the folded gather has the window structure; empty otherwise (the caller then uses the
// tile-loader schedule).
std::vector<LaunchSpec> try_emit_window_gemm(const NestKernel& k, const GemmShape& s, const FoldedOperand* fa,
                                             const FoldedOperand* fb, const GenOptions& opt, const EpilogueSpec* epilogue);

// A kernel written as a window contraction outright: a perfect nest of output loops around
//   acc = 0; for k loops ...: acc = acc + select(guard, F[..], 0) * A[..]; out[..] = acc
// (either factor order, the guard optional), every index affine.  `f_bytes`: size of F's buffer.
std::optional<WindowProblem> match_window_kernel(const Node& kernel, const std::map<std::string, size_t>& buffer_elems);

}  // namespace eh
