"""`execute_graph`: lower a graph and run its kernels on the default device.

Host-side mirror of the reference's `src/backend/executor.rs:149-450`:
lower (+ graph fusion), the AST optimisation stage at ECLAT_OPT_LEVEL (default 3,
`:169-176`; `optimize.py` says what of it is mirrored), then per kernel split the pointer parameters into
immutable inputs / mutable outputs (`:257-270`), look inputs up by buffer name,
allocate zero-filled outputs with the lowerer's shape (`:288-315`), compile
through the kernel cache (`:323-338`), execute (`:347`), publish outputs under
their names (`:357-372`); the root's buffer is found by name, else the
highest-numbered `bufN` is returned (`:389-447`).

Backends that offer `compile_program` get the whole Program at once (buffer
table attached) so they can fuse across kernels; results are identical.
"""

from __future__ import annotations

import os
from typing import Dict, List, Sequence

from .ast import AstNode
from .device import (DeviceError, compile_ast_with_cache, compile_program_with_cache,
                     get_default_device)
from .graph import GraphNode, collect_inputs
from .lowerer import lower_graph
from .optimize import optimize_program


class ExecutionError(Exception):
    pass


def _const_shape(shape) -> List[int]:
    return [int(e.evaluate()) for e in shape]


def buffer_table(program: AstNode, lowerer, input_names: Sequence[str],
                 output_names: Sequence[str], constants: Dict[str, str] = None) -> List[dict]:
    """Name, dtype, shape and role (input | output | temp | ones | zeros) of every
    buffer the program's kernels touch, in first-use order.  `constants` names the inputs
    the executor itself filled with 1.0 / 0.0."""
    constants = constants or {}
    seen, table = set(), []
    for kern in program.args:
        for p in kern.attrs["params"]:
            if not p.dtype.is_ptr() or p.name in seen:
                continue
            seen.add(p.name)
            info = lowerer.get_buffer_info_by_name(p.name)
            if info is None:
                raise ExecutionError(f"no shape known for buffer '{p.name}'")
            role = (constants[p.name] if p.name in constants
                    else "input" if p.name in input_names
                    else "output" if p.name in output_names else "temp")
            table.append({"name": p.name, "dtype": info[1],
                          "shape": _const_shape(info[0]), "role": role})
    return table


def _root_buffer_name(root: GraphNode, lowerer, available: Sequence[str], opt_root=None):
    name = lowerer.lookup_buffer_name(root)
    if name is not None and name in available:
        return name
    # the optimised graph's root (graph passes rebuild nodes), or -- when that root is a view
    # that was inlined -- the node whose buffer it views
    n = opt_root
    while n is not None and not n.is_external():
        name = lowerer.lookup_buffer_name(n)
        if name is not None and name in available:
            return name
        n = n.src[0] if (n.op.kind == "view" and n.src) else None
    best = None
    for k in available:
        if k.startswith("buf") and k[3:].isdigit():
            n = int(k[3:])
            if best is None or n > best[0]:
                best = (n, k)
    return best[1] if best else None


def execute_graph(roots: Sequence[GraphNode], input_buffers: Dict[int, object],
                  fuse_program: bool = None, constant_inputs: Dict[int, str] = None):
    """Returns one buffer per root (None where the reference finds none).
    `constant_inputs` maps id(input node) -> "ones" | "zeros" for inputs whose buffer
    the caller synthesised (realize.rs:391-421); a whole-program backend may fold them."""
    dev = get_default_device()
    if dev is None:
        raise ExecutionError("NoDevice")
    if not roots:
        return []
    program, lowerer, opt_roots = lower_graph(roots)
    # pipeline.optimize (executor.rs:169-176): ECLAT_OPT_LEVEL 0 leaves the program as lowered
    program = optimize_program(program)
    kernels = [k for k in program.args if k.op == "kernel"]

    input_nodes = collect_inputs(roots)
    buffer_map: Dict[str, object] = {}
    for n in input_nodes:
        if id(n) not in input_buffers:
            raise ExecutionError(f"MissingInput: {lowerer.lookup_buffer_name(n)}")
        buffer_map[lowerer.lookup_buffer_name(n) or ""] = input_buffers[id(n)].clone_buffer()

    if fuse_program is None:
        fuse_program = os.environ.get("ECLAT_HIP_FUSE", "1") != "0"
    if fuse_program and dev.supports_program() and kernels:
        produced = [p.name for k in kernels for p in k.attrs["params"]
                    if p.dtype.is_ptr() and p.mutable]
        all_names = list(buffer_map.keys()) + produced
        out_names = []
        for r, o in zip(roots, opt_roots):
            nm = _root_buffer_name(r, lowerer, all_names, o)
            if nm is not None and nm not in out_names:
                out_names.append(nm)
        consts = {}
        for n in input_nodes:
            kind = (constant_inputs or {}).get(id(n))
            if kind:
                consts[lowerer.lookup_buffer_name(n)] = kind
        table = buffer_table(program, lowerer, list(buffer_map.keys()), out_names, consts)
        prog_ast = AstNode.program(kernels, buffers=table)
        compiled = compile_program_with_cache(prog_ast)
        outs = compiled.execute({k: v for k, v in buffer_map.items()})
        buffer_map.update(outs)
    else:
        for kern in kernels:
            params = kern.attrs["params"]
            in_params = [p for p in params if p.dtype.is_ptr() and not p.mutable]
            out_params = [p for p in params if p.dtype.is_ptr() and p.mutable]
            k_inputs = []
            for p in in_params:
                if p.name not in buffer_map:
                    raise ExecutionError(f"MissingInput: Buffer '{p.name}' not found for "
                                         f"kernel '{kern.attrs['name']}'")
                k_inputs.append(buffer_map[p.name])
            k_outputs = []
            for p in out_params:
                info = lowerer.get_buffer_info_by_name(p.name)
                if info is None:
                    raise ExecutionError(f"no shape known for buffer '{p.name}'")
                k_outputs.append(dev.allocate_buffer(_const_shape(info[0]), info[1]))
            try:
                kernel = compile_ast_with_cache(AstNode.program([kern]))
            except Exception as e:
                raise ExecutionError(f"CompilationFailed: Failed to compile kernel "
                                     f"'{kern.attrs['name']}': {e}") from e
            kernel.execute(k_inputs, k_outputs)
            for p, b in zip(out_params, k_outputs):
                buffer_map[p.name] = b

    results = []
    for r, o in zip(roots, opt_roots):
        nm = _root_buffer_name(r, lowerer, list(buffer_map.keys()), o)
        results.append(buffer_map.get(nm) if nm is not None else None)
    return results
