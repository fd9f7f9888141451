"""Functional neural-network ops built from tensor primitives.

Host-side mirror of the reference's `crates/nn/src/functional/`:
`activation.rs` (relu `:18-21`, leaky_relu `:34-39`, sigmoid `:50-57`, tanh `:70-76`,
gelu `:88-99`, silu `:111-114`, elu `:127-135`, softmax `:148-160`, log_softmax `:174-187`,
prelu `:201-210`), `linear.rs:27-56`, `conv.rs:26-92,113-187`, `pool.rs:117-162,172-213`,
`attention.rs:22-96`, `loss.rs:32-65`.
The op trees are the reference's, including what follows from
`Tensor::scale` ignoring its factor (so `tanh(x)` evaluates `sigmoid(x) - 1`) and from
`Tensor::mean` being `sum`.  Functions whose meaning depends on such a factor take
`exact=True` to apply it (not in the reference).
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


def _scaled(x: Tensor, factor: float, exact: bool) -> Tensor:
    return x.scale_exact(factor) if exact else x.scale(factor)


def _tanh(x: Tensor, exact: bool) -> Tensor:
    if not exact:
        return tanh(x)
    return sigmoid(x.scale_exact(2.0)).scale_exact(2.0) - Tensor.ones_like(x)


def leaky_relu(x: Tensor, negative_slope: float = 0.01, exact: bool = False) -> Tensor:
    """x where x >= 0, else negative_slope * x."""
    cond = x.ge(Tensor.zeros_like(x))
    return x.where_cond(cond, _scaled(x, negative_slope, exact))


def gelu(x: Tensor, exact: bool = False) -> Tensor:
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))."""
    x_cubed = x.square() * x
    inner = _scaled(x, 1.0, exact) + _scaled(x_cubed, 0.044715, exact)
    t = _tanh(_scaled(inner, 0.7978845608, exact), exact)
    return _scaled(x * (Tensor.ones_like(x) + t), 0.5, exact)


def silu(x: Tensor) -> Tensor:
    return x * sigmoid(x)


def elu(x: Tensor, alpha: float = 1.0, exact: bool = False) -> Tensor:
    """x where x > 0, else alpha (exp(x) - 1)."""
    cond = x.gt(Tensor.zeros_like(x))
    neg_part = _scaled(x.exp() - Tensor.ones_like(x), alpha, exact)
    return x.where_cond(cond, neg_part)


def prelu(x: Tensor, weight: Tensor) -> Tensor:
    """relu(x) - weight * relu(-x); `weight` has the shape of `x`."""
    zeros = Tensor.zeros_like(x)
    return x.maximum(zeros) - weight * x.neg().maximum(zeros)


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


def conv1d(x: Tensor, weight: Tensor, bias: Optional[Tensor] = None, stride: int = 1,
           padding: int = 0, dilation: int = 1) -> Tensor:
    """x [N,Cin,L], weight [Cout,Cin,K] -> [N,Cout,Lout]; here the batch is merged into the
    rows of the im2col matrix [N*Lout, Cin*K] (`conv.rs:26-92`)."""
    cout, cin, k = weight.shape()
    n, _, l = x.shape()
    l_out = (l + 2 * padding - dilation * (k - 1) - 1) // stride + 1
    padded = x.pad([(0, 0), (0, 0), (padding, padding)])
    cols = padded.unfold_1d(k, stride, dilation).permute([0, 2, 1, 3]).contiguous().reshape([n * l_out, cin * k])
    product = cols.unsqueeze(1) * weight.reshape([cout, cin * k]).unsqueeze(0)
    out = product.sum(2).reshape([n, l_out, cout]).permute([0, 2, 1])
    if bias is not None:
        return out + bias.unsqueeze(0).unsqueeze(2)
    return out


def avg_pool2d(x: Tensor, kernel_size, stride=None, padding=(0, 0), exact: bool = False) -> Tensor:
    """As max_pool2d with `mean` over the window (`pool.rs:172-213`); the reference's `mean`
    is a sum, `exact` divides by the window size."""
    kh, kw = kernel_size
    sh, sw = stride if stride is not None else kernel_size
    ph, pw = padding
    n, c, h, w = x.shape()
    h_out, w_out = (h + 2 * ph - kh) // sh + 1, (w + 2 * pw - kw) // sw + 1
    padded = x.pad([(0, 0), (0, 0), (ph, ph), (pw, pw)]) if (ph > 0 or pw > 0) else x
    windows = padded.unfold_2d((kh, kw), (sh, sw), (1, 1)).contiguous().reshape([n, c, h_out, w_out, kh * kw])
    out = windows.mean(4)
    return out.scale_exact(1.0 / (kh * kw)) if exact else out


def batched_matmul_d4(a: Tensor, b: Tensor) -> Tensor:
    """[B,H,M,K] @ [B,H,K,N] -> [B,H,M,N] as unsqueeze, broadcast multiply, sum over K
    (`attention.rs:22-35`)."""
    return (a.unsqueeze(4) * b.unsqueeze(2)).sum(3)


def scaled_dot_product_attention(query: Tensor, key: Tensor, value: Tensor,
                                 attn_mask: Optional[Tensor] = None, exact: bool = False) -> Tensor:
    """softmax(Q K^T / sqrt(D) [masked]) V for [B,H,L,D] tensors (`attention.rs:57-96`);
    mask 1.0 = attend, 0.0 = masked.  The reference's two `scale` calls (1/sqrt(D) and the
    -1e9 fill) lose their factors; `exact` applies them."""
    d = query.shape()[3]
    scores = _scaled(batched_matmul_d4(query, key.permute([0, 1, 3, 2])), 1.0 / float(d) ** 0.5, exact)
    if attn_mask is not None:
        neg_inf = _scaled(Tensor.ones_like(scores), -1e9, exact)
        keep = attn_mask.ge(_scaled(Tensor.ones_like(attn_mask), 0.5, exact))
        scores = scores.where_cond(keep, neg_inf)
    return batched_matmul_d4(softmax(scores, 3), value)


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
