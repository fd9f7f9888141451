"""CPU oracle for the eclat kernel path -- TEST INFRASTRUCTURE ONLY.

This package restates, for a CPU, what the reference's `backend-c` does with a
lowered kernel AST: render it to C99 text (`c_renderer.py`, following
`src/backend/renderer.rs` and `crates/backend-c/src/renderer.rs`), compile it
with `gcc -O3 -ffast-math -shared -fPIC ... -lm`
(`crates/backend-c/src/compiler.rs:153-165`) and call the entry point with
`(inputs..., outputs...)` pointers over zero-initialised host buffers
(`crates/backend-c/src/kernel.rs:95-171`, `buffer.rs:84-93`).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import
it; the product (`harp_amd`) never does and never falls back to it.

What pins it (all without running the reference, whose Rust toolchain is not
available): the rendered-text assertions the reference's own tests hold
(`crates/backend-c/src/renderer.rs:262-296`, `src/backend/renderer.rs`
literal forms), the reference's known-answer vectors, kept as data in
`tests/golden/reference_known_answers.json` (add/mul/2-D add,
`crates/backend-c/src/lib.rs:181-246`; 10 000-element add,
`crates/backend-openmp/src/lib.rs:207-230`; 2x2 matmul,
`crates/backend-metal/src/compiler.rs:193-257`; the 4x3x2 matmul loop of
`examples/matmul_demo.rs`; fold-of-unfold sum, `crates/backend-c/src/lib.rs:298-340`;
three gradients, `crates/backend-metal/src/lib.rs:261-369`), and numpy evaluation
of the same graphs (closed forms, finite differences for the exact VJPs,
brute force over every index form).  Parity unpinned: the reference's two AST beam searches may rewrite
`acc + a*b` into `fma(a, b, acc)` or re-tile loops before rendering; the
oracle renders the AST as lowered, so reductions are compared within
tolerance, never bit-for-bit.
"""
