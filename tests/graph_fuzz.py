"""Seeded random tensor graphs for differential testing (HIP backend against the C oracle).

Each graph is a short chain over one or two inputs drawn from the tensor API the benchmark
configurations use: elementwise arithmetic and math, broadcasts, views (permute, reshape, pad,
expand), reductions over any axis, row-wise normalisations and small contractions.  Values stay
in a range where every op is well conditioned (no division by ~0, no overflow), so the
tolerance classes of the parity tests apply.
"""

import numpy as np


def _unary(rng, fe, t):
    k = rng.integers(0, 7)
    if k == 0:
        return t.neg()
    if k == 1:
        return (t * t + fe.Tensor.ones_like(t)).sqrt()
    if k == 2:
        return (t * t + fe.Tensor.ones_like(t)).recip()
    if k == 3:
        return t.sin()
    if k == 4:
        return fe.nn.relu(t)
    if k == 5:
        return fe.nn.sigmoid(t)
    return t.maximum(t.neg())


def _binary(rng, a, b):
    k = rng.integers(0, 5)
    if k == 0:
        return a + b
    if k == 1:
        return a * b
    if k == 2:
        return a - b
    if k == 3:
        return a.maximum(b)
    return a.minimum(b)


SMALL_DIMS = (1, 2, 3, 5, 8, 13, 32, 64, 100)
LARGE_DIMS = (1, 4, 31, 128, 257, 1000, 2048)      # with at most two axes: up to 4 Mi elements


def build(seed: int, fe, dims=SMALL_DIMS, max_rank=3, kinds=(0, 8)):
    """Returns (input shapes, function of input tensors -> output tensor, description).
    `kinds` is the half-open range the final stage is drawn from: 0-7 are reductions, gathering
    copies, row normalisations, padding, contractions, broadcasts and reshapes; 8-11 prefix
    scans, selects on comparisons, sliding windows and batched contractions."""
    rng = np.random.default_rng(seed)
    nd = int(rng.integers(1, max_rank + 1))
    shape = [int(rng.choice(dims)) for _ in range(nd)]
    kind = int(rng.integers(kinds[0], kinds[1]))
    red = int(rng.integers(0, 3))                        # kind 0: sum, max or min
    has_y = bool(rng.integers(0, 2))
    has_w = kind == 4 and nd >= 2

    def fn(*ins):
        x = ins[0]
        y = ins[1] if has_y else None
        r = np.random.default_rng(seed + 1)
        t = x if y is None else _binary(r, x, y)       # every input is used
        for _ in range(int(r.integers(1, 4))):
            t = _unary(r, fe, t) if (y is None or r.integers(0, 2)) else _binary(r, t, y)
        if kind == 0:                                   # reduce over a random axis
            ax = int(r.integers(0, t.ndim()))
            t = [t.sum, t.max, t.min][red](ax)
        elif kind == 1 and t.ndim() >= 2:               # permute then elementwise (gathering copy)
            perm = list(r.permutation(t.ndim()))
            t = _unary(r, fe, t.permute([int(p) for p in perm]).contiguous())
        elif kind == 2:                                 # softmax / log-softmax over the last axis
            ax = t.ndim() - 1
            t = fe.nn.softmax(t, ax) if r.integers(0, 2) else fe.nn.log_softmax(t, ax)
        elif kind == 3:                                 # pad, then reduce over the last axis
            pads = [(int(r.integers(0, 3)), int(r.integers(0, 3))) for _ in range(t.ndim())]
            t = t.pad(pads).contiguous()
            t = t.sum(t.ndim() - 1)
        elif kind == 4 and t.ndim() >= 2:               # contraction with a second operand
            a = t.reshape([t.numel() // t.shape()[-1], t.shape()[-1]])
            w = ins[-1]
            t = fe.nn.linear(a, w)
            t = _unary(r, fe, t)
        elif kind == 5:                                 # broadcast against a row vector
            v = t.sum(0).unsqueeze(0) if t.ndim() >= 2 else t
            t = _binary(r, t, v.expand(0, t.shape()[0])) if t.ndim() >= 2 else _unary(r, fe, t)
        elif kind == 6:                                 # reduce, then elementwise on the result
            t = _unary(r, fe, t.sum(t.ndim() - 1))
        elif kind == 8:                                 # prefix scan over the last axis
            ax = t.ndim() - 1
            # nothing after it: a prefix sum's rounding depends on the order of its additions, and
            # a steep function of the result would turn that into a large relative difference
            t = [t.cumsum, t.cummax][int(r.integers(0, 2))](ax)
        elif kind == 9:                                 # select on a comparison
            other = _unary(r, fe, t)
            cond = [t.lt, t.ge, t.gt, t.le][int(r.integers(0, 4))](other)
            t = t.where_cond(cond, other * other)
        elif kind == 10:                                # sliding windows over the last axis, reduced
            n = t.shape()[-1]
            k = 2 if n >= 2 else 1
            stride = int(r.integers(1, 3))
            w = t.unfold([t.ndim() - 1], [k], [stride], [1]).contiguous()
            t = [w.max, w.sum][int(r.integers(0, 2))](w.ndim() - 1)
        elif kind == 11 and t.ndim() == 3:              # batched contraction over the last axis
            a = t.unsqueeze(2)                          # [B, M, 1, K]
            b = _unary(r, fe, t).unsqueeze(1)           # [B, 1, M, K]
            t = (a * b).sum(3)                          # [B, M, M]
        else:                                           # reshape to rows of a different length
            n = t.numel()
            cols = [c for c in (1, 2, 4, 5, 8, 10, 16, 25) if n % c == 0]
            c = int(r.choice(cols))
            t = _unary(r, fe, t.reshape([n // c, c])).sum(1)
        return t

    shapes = [tuple(shape)]
    if has_y:
        shapes.append(tuple(shape))
    if has_w:
        shapes.append((int(rng.choice([3, 10, 33, 64])), shape[-1]))
    what = f"kind {kind}" + (f" ({['sum', 'max', 'min'][red]})" if kind == 0 else "")
    return shapes, fn, f"seed {seed}: shape {shape}, {what}"


def build_cnn(seed: int, fe):
    """A random small convolutional classifier: conv (1x1, 2x2 or 3x3, optional padding and
    bias) + relu, optional 2x2 max-pool, flatten, linear, log-softmax.  Returns
    (input shapes, function -> [batch, classes] log-probabilities, description)."""
    rng = np.random.default_rng(seed)
    b, cin = int(rng.choice([1, 2, 5])), int(rng.choice([1, 3, 4]))
    h, w = int(rng.choice([6, 8, 12])), int(rng.choice([6, 9, 12]))
    cout, k = int(rng.choice([2, 5, 8, 33])), int(rng.choice([1, 2, 3]))
    pad = int(rng.integers(0, 2)) if k == 3 else 0
    use_bias = bool(rng.integers(0, 2))
    ho, wo = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    pool = bool(rng.integers(0, 2)) and ho % 2 == 0 and wo % 2 == 0
    hp, wp = (ho // 2, wo // 2) if pool else (ho, wo)
    feat, classes = cout * hp * wp, int(rng.choice([3, 10]))

    def fn(x, w1, w2, b2, *rest):
        y = fe.nn.relu(fe.nn.conv2d(x, w1, rest[0] if use_bias else None, padding=(pad, pad)))
        if pool:
            y = fe.nn.max_pool2d(y, (2, 2))
        y = y.contiguous().reshape([b, feat])
        return fe.nn.log_softmax(fe.nn.linear(y, w2, b2), 1)

    shapes = [(b, cin, h, w), (cout, cin, k, k), (classes, feat), (classes,)]
    if use_bias:
        shapes.append((cout,))
    desc = (f"seed {seed}: x {shapes[0]}, conv {cout}x{cin}x{k}x{k} pad {pad} bias {use_bias}, "
            f"pool {pool}, classes {classes}")
    return shapes, fn, desc
