"""The benchmark configurations as front-end graphs with seeded synthetic inputs.

Used by the benchmark, the smoke check and the parity tests so that all three
run the same graphs on the same data.
"""

from __future__ import annotations

from typing import Callable, Dict, List, Tuple

import numpy as np

from .frontend import AstNode, Tensor, lower_graph, nn
from .frontend.executor import buffer_table
from .frontend.graph import collect_inputs
from .frontend.optimize import optimize_program


def config1_inputs(n: int = 1024, seed: int = 1234) -> List[np.ndarray]:
    rng = np.random.default_rng(seed)
    return [rng.normal(0, 1, (n, n)).astype(np.float32) for _ in range(3)]


def config1_graph(a: Tensor, b: Tensor, c: Tensor) -> Tensor:
    """s = sum(relu(a*b + c), -1): one fused graph (E, E, R in the reference)."""
    return nn.relu(a * b + c).sum(1)


def config2_inputs(rows: int = 4096, cols: int = 4096, seed: int = 1235) -> List[np.ndarray]:
    rng = np.random.default_rng(seed)
    return [rng.normal(0, 2, (rows, cols)).astype(np.float32)]


def config2_graph(x: Tensor) -> Tensor:
    """Row softmax: exp(x - max) / sum(exp(x - max)) (R, E, E, R, E in the reference)."""
    return nn.softmax(x, 1)


def config3_inputs(n: int = 4096, seed: int = 1236) -> List[np.ndarray]:
    rng = np.random.default_rng(seed)
    return [rng.uniform(-1, 1, (n, n)).astype(np.float32) for _ in range(2)]


def config3_graph(a: Tensor, b: Tensor) -> Tensor:
    """C = A @ B as expand-mul-sum (one R kernel in the reference)."""
    return nn.matmul(a, b)


CONFIGS: Dict[str, Tuple[Callable, Callable]] = {
    "config1_relu_sum": (config1_inputs, config1_graph),
    "config2_softmax": (config2_inputs, config2_graph),
    "config3_matmul": (config3_inputs, config3_graph),
}


def lower_with_table(shapes: List[Tuple[int, ...]], graph_fn: Callable):
    """Lowers `graph_fn` over fresh inputs of the given shapes.  Returns the
    Program AST carrying its buffer table, the input buffer names (in argument
    order) and the output buffer name."""
    tensors = [Tensor.input(list(s)) for s in shapes]
    y = graph_fn(*tensors)
    prog, lw, _ = lower_graph([y.graph])
    prog = optimize_program(prog)            # what the executor's optimisation stage hands on
    by_id = {id(n): lw.lookup_buffer_name(n) for n in collect_inputs([y.graph])}
    arg_names = [by_id[id(t.graph)] for t in tensors]
    produced = [p.name for k in prog.args for p in k.attrs["params"] if p.dtype.is_ptr() and p.mutable]
    numbered = [n for n in produced if n.startswith("buf") and n[3:].isdigit()]
    out = max(numbered, key=lambda s: int(s[3:]))
    all_inputs = list(by_id.values())
    const_inputs = {by_id[id(n)]: n.name for n in collect_inputs([y.graph])
                    if by_id[id(n)] not in arg_names}
    table = buffer_table(prog, lw, all_inputs, [out],
                         {k: ("zeros" if v == "zeros" else "ones") for k, v in const_inputs.items()})
    return AstNode.program(list(prog.args), buffers=table), arg_names, out, const_inputs, prog


# ---------------------------------------------------------------------------
# config 4: MLP training step (exact gradients; see harp_amd/frontend/config.py)
# ---------------------------------------------------------------------------

def tanh_exact(x: Tensor) -> Tensor:
    """tanh(x) = 2*sigmoid(2x) - 1 with the factors actually applied (the reference's
    `nn::tanh` loses them because `Tensor::scale` ignores its argument)."""
    sig = nn.sigmoid(x.scale_exact(2.0))
    return sig.scale_exact(2.0) - Tensor.ones_like(x)


def mlp_sizes(full: bool = True):
    return (8192, [1024, 4096, 4096, 1024]) if full else (64, [32, 64, 64, 32])


def config4_inputs(batch: int = 8192, dims=(1024, 4096, 4096, 1024), seed: int = 1237):
    """x ~ U(-pi, pi), target sin(x) (first/last width must match), W ~ U(+-1/sqrt(fan_in))."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-np.pi, np.pi, (batch, dims[0])).astype(np.float32)
    t = np.sin(x[:, :dims[-1]]).astype(np.float32)
    params = []
    for fan_in, fan_out in zip(dims[:-1], dims[1:]):
        k = 1.0 / np.sqrt(fan_in)
        params.append(rng.uniform(-k, k, (fan_out, fan_in)).astype(np.float32))
        params.append(rng.uniform(-k, k, (fan_out,)).astype(np.float32))
    return [x, t] + params


def config4_graph(x: Tensor, t: Tensor, *params: Tensor, lr: float = 1e-3):
    """One SGD step as a single graph: forward, mean-squared error, exact backward,
    p - lr*grad for every parameter.  Returns [new parameters..., loss]."""
    from .frontend import exact_mode
    with exact_mode():
        h = x
        n_layers = len(params) // 2
        for i in range(n_layers):
            h = nn.linear(h, params[2 * i], params[2 * i + 1])
            if i + 1 < n_layers:
                h = tanh_exact(h)
        d = h - t
        n = 1
        for s in d.shape():
            n *= s
        loss = (d * d).sum(1).sum(0).scale_exact(1.0 / n)
        loss.backward_with_params(list(params))
        new_params = [p - p.grad().scale_exact(lr) for p in params]
    return new_params + [loss]


# ---------------------------------------------------------------------------
# config 5: MNIST-shaped CNN, forward + backward (exact gradients)
# ---------------------------------------------------------------------------

def cnn_sizes(full: bool = True):
    """(batch, image side, conv1 channels, conv2 channels, hidden width, classes)."""
    return (256, 28, 32, 64, 128, 10) if full else (4, 8, 4, 8, 16, 10)


def config5_inputs(batch=256, side=28, c1=32, c2=64, hidden=128, classes=10, seed: int = 1238):
    """images ~ U(0,1) [batch,1,side,side]; one-hot of uniform labels; conv and fc parameters
    ~ U(+-1/sqrt(fan_in)).  Returns [x, one_hot, w1, b1, w2, b2, w3, b3, w4, b4]."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(0, 1, (batch, 1, side, side)).astype(np.float32)
    labels = rng.integers(0, classes, batch)
    one_hot = np.zeros((batch, classes), np.float32)
    one_hot[np.arange(batch), labels] = 1.0
    flat = c2 * (side // 4) ** 2
    params = []
    for shape, fan_in in (((c1, 1, 3, 3), 9), ((c2, c1, 3, 3), 9 * c1),
                          ((hidden, flat), flat), ((classes, hidden), hidden)):
        k = 1.0 / np.sqrt(fan_in)
        params.append(rng.uniform(-k, k, shape).astype(np.float32))
        params.append(rng.uniform(-k, k, (shape[0],)).astype(np.float32))
    return [x, one_hot] + params


def config5_graph(x: Tensor, one_hot: Tensor, *params: Tensor, lr: float = None):
    """conv3x3(pad 1)+relu+maxpool2 twice, fc+relu, fc, cross-entropy; exact backward.
    Returns [gradient of every parameter..., loss], or with a learning rate the whole SGD
    step [p - lr*gradient for every parameter..., loss]."""
    from .frontend import exact_mode
    w1, b1, w2, b2, w3, b3, w4, b4 = params
    with exact_mode():
        h = nn.max_pool2d(nn.relu(nn.conv2d(x, w1, b1, padding=(1, 1))), (2, 2))
        h = nn.max_pool2d(nn.relu(nn.conv2d(h, w2, b2, padding=(1, 1))), (2, 2))
        n = h.shape()[0]
        h = h.reshape([n, h.numel() // n])
        h = nn.relu(nn.linear(h, w3, b3))
        logits = nn.linear(h, w4, b4)
        loss = nn.cross_entropy_loss(logits, one_hot, exact=True)
        loss.backward_with_params(list(params))
        # a gradient may come out as a view (the weight's is a permute); roots must own buffers
        if lr is not None:
            return [p - p.grad().scale_exact(lr) for p in params] + [loss]
        grads = [p.grad().contiguous() for p in params]
    return grads + [loss]


def lower_multi(tensors_in, roots):
    """Lowers several roots into one Program with a buffer table.  Returns (program AST,
    input buffer names in the order of `tensors_in`, output buffer name per root, constant
    inputs {buffer name: "ones" | "zeros"})."""
    from .frontend import exact_mode
    from .frontend.executor import _root_buffer_name
    with exact_mode():
        prog, lw, opt_roots = lower_graph([r.graph for r in roots])
    prog = optimize_program(prog)
    all_inputs = collect_inputs([r.graph for r in roots])
    by_id = {id(n): lw.lookup_buffer_name(n) for n in all_inputs}
    arg_names = [by_id[id(t.graph)] for t in tensors_in]
    produced = [p.name for k in prog.args for p in k.attrs["params"] if p.dtype.is_ptr() and p.mutable]
    avail = list(by_id.values()) + produced
    outs = [_root_buffer_name(r.graph, lw, avail, o) for r, o in zip(roots, opt_roots)]
    consts = {by_id[id(n)]: n.name for n in all_inputs if by_id[id(n)] not in arg_names}
    table = buffer_table(prog, lw, list(by_id.values()), outs,
                         {k: ("zeros" if v == "zeros" else "ones") for k, v in consts.items()})
    return AstNode.program(list(prog.args), buffers=table), arg_names, outs, consts, prog
