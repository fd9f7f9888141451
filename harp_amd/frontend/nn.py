"""Functional neural-network ops built from tensor primitives.

Host-side mirror of the reference's `crates/nn/src/functional/`:
`activation.rs` (relu `:18-21`, sigmoid `:50-57`, tanh `:70-76`, softmax
`:148-160`, log_softmax `:174-187`), `linear.rs:27-56`, `conv.rs:113-187`,
`pool.rs:117-162`, `loss.rs:32-65`.
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


def conv2d(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None, stride=(1, 1),
           padding=(0, 0), dilation=(1, 1)) -> Tensor:
    """x [N,Cin,H,W], weight [Cout,Cin,kH,kW] -> [N,Cout,Hout,Wout]: pad, unfold, permute,
    contiguous im2col [N, Hout*Wout, Cin*kH*kW], broadcast multiply with the flattened
    weight, sum over the last axis, reshape + permute, bias (`conv.rs:113-187`)."""
    cout, cin, kh, kw = weight.shape()
    (sh, sw), (ph, pw), (dh, dw) = stride, padding, dilation
    n, _, h, w = x.shape()
    h_out = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    w_out = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    padded = x.pad([(0, 0), (0, 0), (ph, ph), (pw, pw)])
    unfolded = padded.unfold_2d((kh, kw), (sh, sw), (dh, dw))
    cols = unfolded.permute([0, 2, 3, 1, 4, 5]).contiguous().reshape([n, h_out * w_out, cin * kh * kw])
    weight_flat = weight.reshape([cout, cin * kh * kw])
    product = cols.unsqueeze(2) * weight_flat.unsqueeze(0).unsqueeze(0)
    out = product.sum(3).reshape([n, h_out, w_out, cout]).permute([0, 3, 1, 2])
    if bias is not None:
        return out + bias.unsqueeze(0).unsqueeze(2).unsqueeze(3)
    return out


def max_pool2d(x: Tensor, kernel_size, stride=None, padding=(0, 0), dilation=(1, 1)) -> Tensor:
    """[N,C,H,W] -> [N,C,Hout,Wout]: pad (only when asked), unfold, contiguous, merge the
    window axes, max over them (`pool.rs:117-162`)."""
    kh, kw = kernel_size
    sh, sw = stride if stride is not None else kernel_size
    (ph, pw), (dh, dw) = padding, dilation
    n, c, h, w = x.shape()
    h_out = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1
    w_out = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1
    padded = x.pad([(0, 0), (0, 0), (ph, ph), (pw, pw)]) if (ph > 0 or pw > 0) else x
    unfolded = padded.unfold_2d((kh, kw), (sh, sw), (dh, dw))
    return unfolded.contiguous().reshape([n, c, h_out, w_out, kh * kw]).max(4)


def cross_entropy_loss(logits: Tensor, one_hot: Tensor, exact: bool = False) -> Tensor:
    """-mean over the batch of the log-probability of the labelled class (`loss.rs:32-65`).
    The reference builds `one_hot` [N,C] on the host from u8 labels and feeds it as an
    input; here the caller passes that input.  The final `scale(-1/N)` is the reference's
    (which ignores its factor) unless `exact`."""
    n = logits.shape()[0]
    total = (one_hot * log_softmax(logits, 1)).sum(1).sum(0)
    return total.scale_exact(-1.0 / n) if exact else total.scale(-1.0 / n)
