"""A graph compiled once and run many times.

The reference re-lowers and re-optimises the graph on every `realize` (`execute_graph`,
`src/backend/executor.rs:149-450`); its only reuse is the per-kernel cache behind
`compile_ast_with_cache`.  For a training step that is the same graph every iteration, all of
that host work can be paid once: `CompiledStep` builds the graph over placeholder inputs, lowers
it with its buffer table, compiles it as one Program for the GPU and then only binds buffers and
queues launches.  Outputs stay on the device, so they can be fed back as the next call's inputs
(updated parameters) without a host copy.

    step = CompiledStep(lambda x, t, *p: workloads.config4_graph(x, t, *p), shapes)
    outs = step(x_buf, t_buf, *param_bufs)         # [new parameters..., loss] as device buffers
    param_bufs = outs[:-1]
"""

from __future__ import annotations

from typing import Callable, List, Optional, Sequence, Union

import numpy as np

from . import backend as hb
from . import workloads as wl
from .frontend import Tensor

ArrayOrBuffer = Union[np.ndarray, "hb.HipBuffer"]


class CompiledStep:
    def __init__(self, graph_fn: Callable, input_shapes: Sequence[Sequence[int]], device: Optional[hb.HipDevice] = None,
                 options=None):
        """`graph_fn(*tensors)` returns one tensor or a list of tensors (the roots)."""
        self.device = device or hb.HipDevice(0)
        tensors = [Tensor.input(list(s)) for s in input_shapes]
        roots = graph_fn(*tensors)
        self._single = isinstance(roots, Tensor)
        roots = [roots] if self._single else list(roots)
        prog_ast, self.input_names, self.output_names, consts, plain = wl.lower_multi(tensors, roots)
        self.input_shapes = [tuple(int(d) for d in s) for s in input_shapes]
        self.output_shapes = [tuple(r.shape()) for r in roots]
        self.lowered_kernels = len(plain.args)
        self.program = hb.HipProgram(self.device, prog_ast, options)
        self._by_name = {b["name"]: b for b in self.program.buffers}
        # synthesised ones / zeros the plan did not fold away are filled once and kept
        self._constants = {}
        for name, kind in consts.items():
            b = self._by_name.get(name)
            if b is None or b["elided"]:
                continue
            buf = self.device.alloc(b["bytes"])
            if kind != "zeros":
                buf.write_array(np.ones(b["bytes"] // 4, np.float32))
            self._constants[name] = buf

    @property
    def launches(self) -> List[dict]:
        return self.program.launches

    def upload(self, array: np.ndarray) -> "hb.HipBuffer":
        a = np.ascontiguousarray(array, dtype=np.float32)
        buf = self.device.alloc(a.nbytes)
        buf.write_array(a)
        return buf

    def __call__(self, *inputs: ArrayOrBuffer, sync: bool = False):
        """Queues one run.  Inputs are device buffers (or arrays, uploaded first) in the order of
        `input_shapes`; returns the roots' buffers, freshly allocated, in the order `graph_fn`
        returned them.  Reading a result (`read_array`) waits for it; `sync=True` waits here."""
        if len(inputs) != len(self.input_names):
            raise ValueError(f"expected {len(self.input_names)} inputs, got {len(inputs)}")
        named = dict(self._constants)
        for name, shape, x in zip(self.input_names, self.input_shapes, inputs):
            if name not in self._by_name:               # an input the graph does not use
                continue
            buf = self.upload(x) if isinstance(x, np.ndarray) else x
            want = self._by_name[name]["bytes"]
            if buf.byte_len() != want:
                raise ValueError(f"input '{name}' of shape {shape} needs {want} bytes, got {buf.byte_len()}")
            named[name] = buf
        outs = []
        for name in self.output_names:
            if name in named and name not in self.input_names:      # the same root returned twice
                outs.append(named[name])
                continue
            buf = self.device.alloc(self._by_name[name]["bytes"])
            named[name] = buf
            outs.append(buf)
        self.program.run(self.program.bind(named), sync=sync)
        return outs[0] if self._single else outs
