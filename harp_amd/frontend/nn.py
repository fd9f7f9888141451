"""Functional neural-network ops built from tensor primitives.

Host-side mirror of the reference's `crates/nn/src/functional/`:
`activation.rs` (relu `:18-21`, sigmoid `:50-57`, tanh `:70-76`, softmax
`:148-160`, log_softmax `:174-187`), `linear.rs:27-56`, `loss.rs:32-65`.
The op trees are the reference's, including what follows from
`Tensor::scale` ignoring its factor (so `tanh(x)` evaluates `sigmoid(x) - 1`).
"""

from __future__ import annotations

from typing import Optional

from .tensor import Tensor


def relu(x: Tensor) -> Tensor:
    return x.maximum(Tensor.zeros_like(x))


def sigmoid(x: Tensor) -> Tensor:
    exp_neg = x.neg().exp()
    return (Tensor.ones_like(x) + exp_neg).recip()


def tanh(x: Tensor) -> Tensor:
    sig = sigmoid(x.scale(2.0))
    return sig.scale(2.0) - Tensor.ones_like(x)


def softmax(x: Tensor, axis: int) -> Tensor:
    max_b = x.max(axis).unsqueeze(axis)
    exp_shifted = (x - max_b).exp()
    sum_b = exp_shifted.sum(axis).unsqueeze(axis)
    return exp_shifted / sum_b


def log_softmax(x: Tensor, axis: int) -> Tensor:
    max_b = x.max(axis).unsqueeze(axis)
    shifted = x - max_b
    log_sum = shifted.exp().sum(axis).ln().unsqueeze(axis)
    return shifted - log_sum


def linear(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None) -> Tensor:
    """x [B,K], weight [O,K] -> [B,O] as unsqueeze * unsqueeze, sum over K."""
    a = x.unsqueeze(2)
    b = weight.permute([1, 0]).unsqueeze(0)
    y = (a * b).sum(1)
    if bias is not None:
        return y + bias.unsqueeze(0)
    return y


def matmul(a: Tensor, b: Tensor) -> Tensor:
    """a [M,K] @ b [K,N] built as in `examples/matmul_demo.rs:43-60`."""
    m, _k = a.shape()
    _, n = b.shape()
    ae = a.unsqueeze(2).expand(2, n)
    be = b.permute([1, 0]).unsqueeze(0).permute([0, 2, 1]).expand(0, m)
    return (ae * be).sum(1)
