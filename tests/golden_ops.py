"""Graphs named by the fixtures in tests/golden/reference_known_answers.json, and the loader.
The fixtures hold the inputs and expected outputs of the reference's own tests for the kernel
path; the graphs here are how those tests build them with the tensor API."""

import json
import os

import numpy as np

FIXTURES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")


def load():
    with open(FIXTURES) as f:
        return json.load(f)


def array(spec, shape):
    if isinstance(spec, str):                       # generated inputs, as the reference's loops make them
        kind, n = spec.split(":")
        n = int(n)
        a = np.arange(n, dtype=np.float32)
        return (a if kind == "arange" else (n - np.arange(n)).astype(np.float32)).reshape(shape)
    return np.asarray(spec, dtype=np.float32).reshape(shape)


def graph(fe, op):
    return {
        "add": lambda x, y: x + y,
        "mul": lambda x, y: x * y,
        "matmul": lambda x, y: fe.nn.matmul(x, y),
        "unfold_fold_2x2": lambda t: t.unfold([0, 1], [2, 2], [2, 2], [1, 1]).fold([4, 4], [0, 1], [2, 2], [2, 2], [1, 1]),
        "sum_square": lambda t: (t * t).sum(0),
        "sum_product": lambda s, t: (s * t).sum(0),
        "sum_double": lambda t: (t + t).sum(0),
    }[op]


def expr(fe, name):
    A = fe.AstNode
    one, two, four = A.const_f32(1.0), A.const_f32(2.0), A.const_f32(4.0)
    return {"add_1_2": A.add(one, two), "mul_1_2": A.mul(one, two), "sqrt_4": A.unary("sqrt", four),
            "max_a_b": A.max(A.var("a"), A.var("b")), "zero": A.const_f32(0.0),
            "neg_inf": A.const_f32(float("-inf"))}[name]


def check_forward(case, out):
    exp = case["expected"]
    if isinstance(exp, str):
        assert np.allclose(out, float(exp.split(":")[1]), atol=case.get("atol", 0.0)), case["id"]
    else:
        assert out.tolist() == [float(v) for v in exp], case["id"]
