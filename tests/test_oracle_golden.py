"""The CPU oracle against the reference's own known answers and rendered-text
assertions (no GPU)."""

import numpy as np
import pytest

from conftest import realize_on


def test_rendered_expression_text(frontend):
    # crates/backend-c/src/renderer.rs:262-296
    from oracle.c_renderer import render_expr
    A = frontend.AstNode
    one, two, four = A.const_f32(1.0), A.const_f32(2.0), A.const_f32(4.0)
    assert render_expr(A.add(one, two).to_sexpr()) == "(1.0f + 2.0f)"
    assert render_expr(A.mul(one, two).to_sexpr()) == "(1.0f * 2.0f)"
    assert render_expr(A.unary("sqrt", four).to_sexpr()) == "sqrtf(4.0f)"
    assert render_expr(A.unary("sin", four).to_sexpr()) == "sinf(4.0f)"
    assert render_expr(A.unary("log2", four).to_sexpr()) == "log2f(4.0f)"
    assert render_expr(A.max(A.var("a"), A.var("b")).to_sexpr()) == "fmaxf(a, b)"
    # src/backend/renderer.rs:196-215
    assert render_expr(A.const_f32(0.0).to_sexpr()) == "0.0f"
    assert render_expr(A.const_f32(float("-inf")).to_sexpr()) == "(-INFINITY)"
    assert render_expr(A.const_f32(float("inf")).to_sexpr()) == "INFINITY"
    assert render_expr(A.recip(A.var("x")).to_sexpr()) == "(1.0f / x)"


def test_header_and_types(frontend):
    # crates/backend-c/src/renderer.rs:236-258
    from oracle.c_renderer import HEADER, render_dtype
    assert "#include <math.h>" in HEADER and "#include <stdlib.h>" in HEADER and "C99" in HEADER
    assert render_dtype("f32") == "float" and render_dtype("f64") == "double"
    assert render_dtype("i32") == "int" and render_dtype("i64") == "long long"
    assert render_dtype(["ptr", "f32", "global"]) == "float*"


def test_add_mul_known_answers(frontend):
    # crates/backend-c/src/lib.rs:183-245
    a = np.array([1, 2, 3, 4], dtype=np.float32)
    b = np.array([5, 6, 7, 8], dtype=np.float32)
    assert realize_on(frontend, "c", lambda x, y: x + y, [a, b]).tolist() == [6, 8, 10, 12]
    a2 = np.array([1, 2, 3, 4], dtype=np.float32)
    b2 = np.array([2, 3, 4, 5], dtype=np.float32)
    assert realize_on(frontend, "c", lambda x, y: x * y, [a2, b2]).tolist() == [2, 6, 12, 20]
    a3 = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    b3 = a3[::-1, ::-1].copy()
    assert realize_on(frontend, "c", lambda x, y: x + y, [a3, b3]).tolist() == [7.0] * 6


def test_large_add_openmp(frontend):
    # crates/backend-openmp/src/lib.rs:205-230: 10 000 elements, a[i]=i, b[i]=10000-i
    a = np.arange(10000, dtype=np.float32)
    b = (10000 - np.arange(10000)).astype(np.float32)
    out = realize_on(frontend, "openmp", lambda x, y: x + y, [a, b])
    assert np.allclose(out, 10000.0, atol=1e-3)


def test_matmul_2x2_known_answer(frontend):
    # crates/backend-metal/src/compiler.rs:240-257
    a = np.array([[1, 2], [3, 4]], dtype=np.float32)
    b = np.array([[5, 6], [7, 8]], dtype=np.float32)
    out = realize_on(frontend, "c", lambda x, y: frontend.nn.matmul(x, y), [a, b])
    assert out.tolist() == [19, 22, 43, 50]


def test_matmul_demo_shape(frontend):
    # examples/matmul_demo.rs:114-129, 166-178: 4x3 @ 3x2 against the plain triple loop
    a = (np.arange(12, dtype=np.float32) * 0.5 - 1).reshape(4, 3)
    b = (np.arange(6, dtype=np.float32) * 0.25 + 1).reshape(3, 2)
    out = realize_on(frontend, "c", lambda x, y: frontend.nn.matmul(x, y), [a, b]).reshape(4, 2)
    ref = np.zeros((4, 2), dtype=np.float32)
    for i in range(4):
        for j in range(2):
            s = np.float32(0)
            for k in range(3):
                s = np.float32(s + a[i, k] * b[k, j])
            ref[i, j] = s
    assert np.array_equal(out, ref)


def test_fold_of_unfold_preserves_sum(frontend):
    # crates/backend-c/src/lib.rs:299-340: 4x4, 2x2 windows, stride 2
    x = np.arange(1, 17, dtype=np.float32).reshape(4, 4)

    def build(t):
        u = t.unfold([0, 1], [2, 2], [2, 2], [1, 1])
        return u.fold([4, 4], [0, 1], [2, 2], [2, 2], [1, 1])
    out = realize_on(frontend, "c", build, [x])
    assert out.size == 16
    assert abs(float(out.sum()) - float(x.sum())) < 1e-5
    # The scatter kernel reads the unfolded buffer through the unfold view's own index
    # (src/lowerer/lower.rs:623-630), so the result is a permutation of x, not x itself;
    # the reference's test pins only the length and the sum.
    assert sorted(out.tolist()) == sorted(x.ravel().tolist())


def test_softmax_closed_forms(frontend):
    rng = np.random.default_rng(7)
    x = rng.normal(0, 2, (16, 33)).astype(np.float32)
    out = realize_on(frontend, "c", lambda t: frontend.nn.softmax(t, 1), [x]).reshape(16, 33)
    assert np.allclose(out.sum(1), 1.0, atol=1e-5)
    e = np.exp(x.astype(np.float64) - x.max(1, keepdims=True))
    assert np.allclose(out, e / e.sum(1, keepdims=True), rtol=1e-5, atol=1e-7)
    # the row maximum maps to 1 / sum
    am = x.argmax(1)
    assert np.allclose(out[np.arange(16), am], 1.0 / e.sum(1), rtol=1e-5)


def test_relu_sum_two_roundings(frontend):
    rng = np.random.default_rng(3)
    a, b, c = (rng.normal(0, 1, (8, 40)).astype(np.float32) for _ in range(3))
    out = realize_on(frontend, "c",
                     lambda x, y, z: frontend.nn.relu(x * y + z).sum(1), [a, b, c])
    prod = (a * b).astype(np.float32)              # rounded once
    ref = np.maximum((prod + c).astype(np.float32), 0).astype(np.float64).sum(1)
    assert np.all(out >= 0)
    assert np.allclose(out, ref, rtol=1e-5)


@pytest.mark.parametrize("fn,ref", [
    (lambda t: t.permute([1, 0]).contiguous(), lambda x: x.T.copy()),
    (lambda t: t.unsqueeze(0).expand(0, 3).contiguous(), lambda x: np.broadcast_to(x, (3,) + x.shape)),
    (lambda t: t.reshape([3, 8]).sum(1), lambda x: x.reshape(3, 8).sum(1)),
    (lambda t: t.pad([(1, 2), (0, 1)]).contiguous(), lambda x: np.pad(x, [(1, 2), (0, 1)])),
    (lambda t: t.max(0), lambda x: x.max(0)),
    (lambda t: t.cumsum(1), lambda x: np.cumsum(x, 1)),
])
def test_index_forms_brute_force(frontend, fn, ref):
    x = np.random.default_rng(11).normal(0, 1, (4, 6)).astype(np.float32)
    out = realize_on(frontend, "c", fn, [x])
    assert np.allclose(out, np.asarray(ref(x)).ravel(), rtol=1e-6, atol=1e-6)
