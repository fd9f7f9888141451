// FP32 MFMA schedule for contraction-shaped reduce kernels:
//   for i, j: acc = 0; for k: acc += A[i,k] * B[k,j]; C[i,j] = acc
// which is how the reference lowers matmul / linear layers for fp32
// (src/lowerer/lower.rs:525-571 on the expand-mul-sum graph of examples/matmul_demo.rs:43-60
// and crates/nn/src/functional/linear.rs:27-56; its own MatMul node only fires for f16,
// src/opt/graph/suggesters/matmul.rs:60-65).
#pragma once

#include <map>
#include <functional>
#include <optional>

#include "analysis.hpp"
#include "codegen.hpp"

namespace eh {

struct GemmShape {
  int64_t M = 0, N = 0, K = 0, batch = 1;
  std::string a_buf, b_buf, c_buf;
  int64_t a_m = 0, a_k = 0, a_b = 0, a_off = 0;   // element strides / offset of A
  int64_t b_k = 0, b_n = 0, b_b = 0, b_off = 0;
  int64_t c_m = 0, c_n = 0, c_b = 0, c_off = 0;
  // a row axis that runs over two nested extents of the memory it reads: rows per inner extent
  // (0: one stride) and the stride between inner extents
  int64_t a_msplit = 0, a_m2 = 0, b_nsplit = 0, b_n2 = 0;
  // the same for C: rows (columns) the operand walks as one axis while the output keeps them in
  // two nested extents (images x pixels written as NCHW)
  int64_t c_msplit = 0, c_m2 = 0, c_nsplit = 0, c_n2 = 0;
};

// An elementwise producer (im2col gather, layout copy, padding ...) whose dense output a
// contraction would read: the tile loader evaluates it per element instead, so the buffer is
// never written.  The contraction builds a device function from this: the producer's loop
// variables are decoded from the element's index in the producer's output (loops with a
// stride of at least Q from the quotient, the others from the remainder, Q chosen so that one
// of the two parts does not change along the contraction's k loop) and `expr` is returned.
struct FoldedOperand {
  std::string src;        // the one buffer the producer reads
  std::string kernel;     // the producer's name (for comments)
  std::string expr;       // C expression over the loop variables and `src`
  std::string prelude;    // device functions `expr` calls (a gather folded into this one), or empty
  struct LoopVar {
    std::string name;
    int64_t extent, stride;   // stride in the producer's dense output
  };
  std::vector<LoopVar> loops;   // outermost first
  bool small = true;            // 32-bit index arithmetic suffices
  double src_bytes = 0;         // 0 = unknown
  // loop stride in the producer's output -> that loop's stride in the source (only when the
  // source index is affine); tells which operand axis is contiguous in the memory actually read
  std::map<int64_t, int64_t> src_stride;
  bool plain = false;           // the producer is one unguarded load at an affine index (a copy through a view)
  int64_t src_off = 0;          // constant term of that index
  // nonzero: `expr` reads `src` through the buffer resource `eh_rs_<src>` over that many bytes
  // (the element function declares it); a byte offset beyond them reads as zero
  size_t ranged_bytes = 0;
  // the producer's element expression itself (a load, possibly under an index guard with a zero
  // default), for schedules that take the gather apart instead of calling it; null when the
  // expression calls another gather's function
  NodePtr value;
};
using FoldMap = std::map<std::string, FoldedOperand>;   // by the producer's output buffer

// Elementwise kernels that follow a contraction over the same dense index space, run on each
// output element while it is still in the accumulator (bias, activation, saved intermediates).
// `function` is the text of
//   __device__ void eh_epilogue(long long eh_e, float eh_acc <params>)
// which stores whatever has to reach memory, C itself included when `store_c`.
struct EpilogueSpec {
  std::string function;
  std::string params;                  // ", const float* __restrict__ buf3, float* __restrict__ buf9"
  std::string args;                    // ", buf3, buf9"
  std::vector<std::string> bufs;       // the extra parameters' buffers, in order
  std::vector<size_t> min_bytes;
  std::vector<std::string> kernels;    // names of the kernels taken in
  bool store_c = true;
  double bytes = 0;                    // algorithmic bytes of the extra parameters
  // The same function in two parts, when nothing it reads sits under a guard (else empty):
  //   struct EhEpiLoads; void eh_epilogue_load(long long eh_e, EhEpiLoads&, <params>);
  //   void eh_epilogue_apply(long long eh_e, float eh_acc, const EhEpiLoads&, [C,] <params>);
  // for schedules that finish many elements per work-item: all reads first, then the stores.
  std::string split_functions;
  int n_loads = 0;                     // values eh_epilogue_load fetches per element
  // ... and for four elements in a row, eh_e a multiple of four (else empty): reads that do not move
  // inside the four once, reads at the element itself and the stores as 128-bit vectors:
  //   struct EhEpiLoads4; void eh_epilogue_load4(long long eh_e, EhEpiLoads4&, <params>);
  //   void eh_epilogue_apply4(long long eh_e, const float (&eh_acc)[4], const EhEpiLoads4&, [C,] <params>);
  std::string quad_functions;
  int quad_regs = 0;                   // registers EhEpiLoads4 takes
  // A tail: a short reduce over windows of a buffer this epilogue stores (the pooling behind a
  // convolution), offered to schedules whose workgroup stores a closed share of that buffer -- the
  // workgroup then also computes the reduce's outputs that read its share, once its stores are
  // done.  Filled by window_reduce_tail; a schedule that takes it lists tail_kernels in its launch.
  //   namespace eh_tail_ns { void eh_tail(idx_t output, <tail's own parameters>); }
  std::string tail_function;
  std::string tail_params;             // parameters the launch does not have yet, ", float* __restrict__ buf41"
  std::string tail_args;               // ", buf31, buf41": every parameter of eh_tail, by buffer name
  std::string tail_source;             // the stored buffer it reads
  std::string tail_tag;                // for the schedule string
  std::vector<std::string> tail_bufs;  // buffers of tail_params, in order
  std::vector<size_t> tail_min_bytes;
  std::vector<std::string> tail_kernels;
  int64_t tail_outputs = 0;            // outputs of the reduce; a workgroup's share is a run of them
  double tail_bytes = 0;
  std::function<void(int64_t, std::vector<int64_t>*)> tail_reads;   // elements of tail_source that output o reads
};

// True when element (b, m, n) of C sits at (b*M + m)*N + n, the index an epilogue is written for.
bool gemm_output_dense(const GemmShape& s);

// Recognises the contraction and returns its strides; nullopt otherwise.
std::optional<GemmShape> match_gemm(const NestKernel& k);

// True when match_gemm succeeds and the contraction is large enough for the MFMA schedule.
bool gemm_shaped(const NestKernel& k, const GenOptions& opt);

// HIP source + dispatch for the kernel; empty when it is not a contraction the MFMA schedule
// covers (the caller then falls back to another schedule).  One launch, or two when K is
// split: partial tiles into a scratch buffer appended to `buffers`, then their sum.
std::vector<LaunchSpec> try_emit_gemm(const NestKernel& k, const GenOptions& opt, std::vector<BufferInfo>* buffers,
                                      const FoldMap* folded = nullptr, const EpilogueSpec* epilogue = nullptr);

}  // namespace eh
