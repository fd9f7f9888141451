"""The BASELINE configurations as front-end graphs with seeded synthetic inputs.

Used by the benchmark, the smoke check and the parity tests so that all three
run the same graphs on the same data.
"""

from __future__ import annotations

from typing import Callable, Dict, List, Tuple

import numpy as np

from .frontend import AstNode, Tensor, lower_graph, nn
from .frontend.executor import buffer_table
from .frontend.graph import collect_inputs


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
    by_id = {id(n): lw.lookup_buffer_name(n) for n in collect_inputs([y.graph])}
    arg_names = [by_id[id(t.graph)] for t in tensors]
    produced = [p.name for k in prog.args for p in k.attrs["params"] if p.dtype.is_ptr() and p.mutable]
    numbered = [n for n in produced if n.startswith("buf") and n[3:].isdigit()]
    out = max(numbered, key=lambda s: int(s[3:]))
    all_inputs = list(by_id.values())
    table = buffer_table(prog, lw, all_inputs, [out])
    const_inputs = {by_id[id(n)]: n.name for n in collect_inputs([y.graph])
                    if by_id[id(n)] not in arg_names}
    return AstNode.program(list(prog.args), buffers=table), arg_names, out, const_inputs, prog
