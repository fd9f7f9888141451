// Contractions with a sliding-window operand (a convolution as the reference lowers it,
// crates/nn/src/functional/conv.rs:113-187: pad -> unfold -> permute -> contiguous, then
// broadcast-multiply and sum): the gather folded into the contraction is recognised for what it
// is -- row digits and window digits that add up to source coordinates, guarded where the window
// leaves the image -- and the source region a group of rows reads is staged in LDS once, so that
// the multiply loop reads its operand at "row base + k offset" without guards or index arithmetic
// (kernels/window_f32_mfma.hip).
#pragma once

#include <vector>

#include "codegen.hpp"
#include "gemm.hpp"

namespace eh {

// The launch for contraction `k` (shape `s`, exactly one of `fa` / `fb` given: the folded operand)
// when the folded gather has the window structure and the patch, the accumulators and A's values
// fit one workgroup; empty otherwise (the caller then uses the tile-loader schedule).
std::vector<LaunchSpec> try_emit_window_gemm(const NestKernel& k, const GemmShape& s, const FoldedOperand* fa,
                                             const FoldedOperand* fb, const GenOptions& opt, const EpilogueSpec* epilogue);

}  // namespace eh
