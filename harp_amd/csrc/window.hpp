// Contractions with a sliding-window operand (a convolution as the reference lowers it,
// crates/nn/src/functional/conv.rs:113-187: pad -> unfold -> permute -> contiguous, then
// broadcast-multiply and sum): the gather folded into the contraction is recognised for what it
// is -- row digits and window digits that add up to source coordinates, guarded where the window
// leaves the image -- and the source region a group of rows reads is staged in LDS once, so that
// the multiply loop reads its operand at "row base + k offset" without guards or index arithmetic
// (kernels/window_f32_mfma.hip).
#pragma once

#include <functional>
#include <map>
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

// A contraction whose result is read only by a run of elementwise kernels that add shifted,
// guarded reads of it to a running sum (a transposed convolution as the reference lowers it --
// the input gradient of conv2d, crates/nn/src/functional/conv.rs:113-187 differentiated: a
// product with the weights, then fold as a sum of padded slices): the sum over the shifts joins
// the sum of the contraction,
//   S[rows] = sum over (k, shift) of [guard(rows, shift)] F[rows - shift, k] * A[k, shift, m],
// and the product's result and the partial sums never reach memory.  Elements of S no later kernel
// reads (a border that the next kernel slices away) are not computed.
struct ProgramView {
  const std::vector<std::optional<NestKernel>>* nests = nullptr;
  const std::map<std::string, std::vector<size_t>>* readers = nullptr;      // kernels (by index) reading a buffer
  const std::map<std::string, size_t>* elems = nullptr;                     // elements per buffer
  std::function<std::string(const std::string&)> role_of;
  std::function<const NestKernel*(const std::string&)> folded_gather;       // the gather evaluated in place of reading this buffer, or null
  std::function<bool(size_t)> taken;                                        // kernel already folded into another
};
struct ScatteredWindow {
  std::vector<LaunchSpec> launches;
  size_t next = 0;                      // first kernel after the run
  std::vector<std::string> elided;      // buffers that no longer exist
  bool partial = false;                 // the output is not written everywhere (only where it is read)
};
std::optional<ScatteredWindow> try_emit_scattered_window(size_t i, const ProgramView& pv, const GenOptions& opt);

}  // namespace eh
