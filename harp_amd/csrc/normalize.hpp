// Brings a kernel back to the loop nest the reference's lowerer wrote.
//
// Before a backend sees a kernel the reference's executor runs its AST optimiser over the whole
// program (src/backend/executor.rs:169-176, src/backend/compile.rs:246-265, suggesters at
// compile.rs:326-337): algebraic rewrites (src/opt/ast/rules/mod.rs:67-108; multiplications by a
// power of two become shifts, rules/bit_ops.rs:19-85; sums and products are re-associated to the
// right; integer constants are folded), loop tiling with a remainder loop or with a guard
// (src/opt/ast/transforms.rs:393-500, 520-630), full unrolling of loops of up to eight iterations
// (transforms.rs:238-361), loop interchange.  All of them keep the kernel's meaning and hide its
// structure.  The passes here undo them by rewrites that each preserve the meaning on their own
// (so whatever they do not recognise is simply left as it is): shifts back to multiplications,
// integer constants folded, blocks of statements that differ only by an integer in arithmetic
// progression rolled back into a loop, strip-mined loop pairs (`v = outer + inner`) and renamed
// remainder loops (`v = r`) turned back into loops over `v`, neighbouring loops over adjoining
// ranges with the same body joined, loops shifted to start at 0 with step 1.
#pragma once

#include <map>
#include <string>

#include "ast.hpp"

namespace eh {

// The kernel with the rewrites above undone where they are recognised; the same node when
// nothing applies.  Never changes what the kernel computes, nor the order of its floating-point
// operations.
NodePtr normalize_kernel(const NodePtr& kernel);

// `n` with every Var named in `m` replaced by the mapped node.
NodePtr substitute_vars(const NodePtr& n, const std::map<std::string, NodePtr>& m);

// Innermost-loop iterations of a statement, loops multiplied out and neighbours added: how much
// work one work-item does when it runs the statement as written.  A bound that moves with the
// enclosing loops counts by its extreme over their ranges (an upper bound on the trips); a loop
// whose bounds cannot be bounded that way (not affine in the loop variables, or over a variable
// assigned in the body) makes the result infinite.
double serial_iterations(const Node& stmt);

}  // namespace eh
