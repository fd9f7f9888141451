"""Cases for the functional mirrors of `crates/nn/src/functional/` beyond the benchmark
configurations: (graph over the front end, input arrays, float64 numpy value of the intended
mathematics).  The graphs pass `exact=True`, so the factors the reference's `scale` and `mean`
drop are applied; they are lowered in exact mode (unfold read as a view)."""

import numpy as np


def _sig(v):
    return 1.0 / (1.0 + np.exp(-v))


def _softmax(z):
    e = np.exp(z - z.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def cases(fe):
    nn = fe.nn
    rng = np.random.default_rng(77)
    f32 = np.float32
    x = rng.normal(0, 1, (37, 65)).astype(f32)
    w = rng.uniform(0, 0.5, x.shape).astype(f32)
    x64 = x.astype(np.float64)
    out = {
        "leaky_relu": (lambda t: nn.leaky_relu(t, 0.1, exact=True), [x], np.where(x64 >= 0, x64, 0.1 * x64)),
        "gelu": (lambda t: nn.gelu(t, exact=True), [x],
                 0.5 * x64 * (1 + np.tanh(0.7978845608 * (x64 + 0.044715 * x64 ** 3)))),
        "silu": (lambda t: nn.silu(t), [x], x64 * _sig(x64)),
        "elu": (lambda t: nn.elu(t, 1.3, exact=True), [x], np.where(x64 > 0, x64, 1.3 * (np.exp(x64) - 1))),
        "prelu": (lambda t, u: nn.prelu(t, u), [x, w], np.maximum(x64, 0) - w * np.maximum(-x64, 0)),
    }
    b, h, l, d = 2, 3, 40, 16
    q, k, v = (rng.normal(0, 1, (b, h, l, d)).astype(f32) for _ in range(3))
    mask = (rng.uniform(0, 1, (b, h, l, l)) > 0.3).astype(f32)
    mask[..., 0] = 1.0                                   # no fully masked row
    s = q.astype(np.float64) @ k.astype(np.float64).transpose(0, 1, 3, 2) / np.sqrt(d)
    out["attention"] = (lambda a, b_, c: nn.scaled_dot_product_attention(a, b_, c, exact=True), [q, k, v],
                        _softmax(s) @ v)
    out["attention_masked"] = (lambda a, b_, c, m: nn.scaled_dot_product_attention(a, b_, c, m, exact=True),
                               [q, k, v, mask], _softmax(np.where(mask >= 0.5, s, -1e9)) @ v)
    xi = rng.normal(0, 1, (3, 4, 50)).astype(f32)
    wi = rng.normal(0, 0.3, (6, 4, 5)).astype(f32)
    bi = rng.normal(0, 1, (6,)).astype(f32)
    xp = np.pad(xi.astype(np.float64), ((0, 0), (0, 0), (2, 2)))
    l_out = (50 + 4 - 5) // 2 + 1
    conv = np.zeros((3, 6, l_out))
    for j in range(l_out):
        conv[:, :, j] = np.einsum("nck,ock->no", xp[:, :, 2 * j:2 * j + 5], wi) + bi
    out["conv1d"] = (lambda a, b_, c: nn.conv1d(a, b_, c, stride=2, padding=2), [xi, wi, bi], conv)
    xa = rng.normal(0, 1, (2, 3, 12, 10)).astype(f32)
    out["avg_pool2d"] = (lambda a: nn.avg_pool2d(a, (2, 2), exact=True), [xa],
                         xa.astype(np.float64).reshape(2, 3, 6, 2, 5, 2).mean((3, 5)))
    return out
