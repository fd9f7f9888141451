"""CPU baseline timing with the oracle's C kernels (test infrastructure; see the
package docstring).  Runs the reference's unfused kernel sequence for a graph --
one gcc-compiled kernel per lowered kernel, called in order over host buffers --
and times only the kernel calls, as `CKernel::execute` would be timed
(`crates/backend-c/src/kernel.rs:95-171`).
"""

from __future__ import annotations

import os
import time
from typing import Callable, Dict, List, Sequence

import numpy as np

from .c_backend import CBuffer, compile_program_text


def _shape_of(info) -> List[int]:
    return [int(e.evaluate()) for e in info[0]]


def prepare(graph_fn: Callable, arrays: Sequence[np.ndarray], openmp: bool = False):
    """Lowers the graph with the product's front end (the reference shares its
    lowerer between backends too) and compiles every kernel with gcc."""
    from harp_amd.frontend import AstNode, Tensor, lower_graph
    from harp_amd.frontend.graph import collect_inputs
    tensors = [Tensor.input(list(a.shape)) for a in arrays]
    y = graph_fn(*tensors)
    roots = [r.graph for r in y] if isinstance(y, (list, tuple)) else [y.graph]
    prog, lw, _ = lower_graph(roots)
    bufs: Dict[str, CBuffer] = {}
    by_id = {id(t.graph): a for t, a in zip(tensors, arrays)}
    for n in collect_inputs(roots):
        name = lw.lookup_buffer_name(n)
        b = CBuffer([int(e.evaluate()) for e in n.shape()], n.dtype.name)
        if id(n) in by_id:
            b.write_from_host(np.ascontiguousarray(by_id[id(n)]).tobytes())
        else:
            fill = {"ones": 1.0, "zeros": 0.0, "scalar": 1.0}[n.name]
            b.write_from_host(np.full(b.byte_len() // 4, fill, dtype=np.float32).tobytes())
        bufs[name] = b
    calls = []
    last = None
    for k in prog.args:
        kern = compile_program_text(AstNode.program([k]).to_sexpr(), openmp=openmp)
        ptrs = []
        for p in k.attrs["params"]:
            if not p.dtype.is_ptr():
                continue
            if p.name not in bufs:
                info = lw.get_buffer_info_by_name(p.name)
                bufs[p.name] = CBuffer(_shape_of(info), info[1].name)
            ptrs.append(bufs[p.name].ptr())
            if p.mutable:
                last = p.name
        calls.append((kern, ptrs))
    return calls, bufs, last


def run_once(calls) -> float:
    t0 = time.perf_counter()
    for kern, ptrs in calls:
        kern.call_raw(*ptrs)
    return time.perf_counter() - t0


def time_graph(graph_fn: Callable, arrays: Sequence[np.ndarray], min_seconds: float = 2.0,
               max_reps: int = 50, openmp: bool = False):
    """Median seconds per pass, number of passes, and the result buffer."""
    if openmp:
        os.environ.setdefault("OMP_WAIT_POLICY", "passive")
        os.environ.setdefault("GOMP_SPINCOUNT", "0")
    calls, bufs, last = prepare(graph_fn, arrays, openmp=openmp)
    run_once(calls)                                   # first touch of the output pages
    times = []
    t_total = 0.0
    while len(times) < 3 or (t_total < min_seconds and len(times) < max_reps):
        t = run_once(calls)
        times.append(t)
        t_total += t
    out = np.frombuffer(bufs[last].read_to_host(), dtype=np.float32).copy()
    return float(np.median(times)), len(times), out
