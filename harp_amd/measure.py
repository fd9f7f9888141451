"""Timing of compiled programs on the device: buffer sets and event-bracketed launches.

Shared by the benchmark and the option search, so both measure the same way: inputs resident
in device memory, several independent bindings rotated between launches so that a launch does
not find its operands in the last-level cache, W untimed launches, then K launches between two
events on the launch stream with a device synchronisation on both sides.
"""

from __future__ import annotations

import time

import numpy as np

from . import backend as hb


def make_sets(dev, prog, arg_names, const_inputs, arrays, nsets):
    """`nsets` independent bindings of `prog`: inputs filled from `arrays` (in the order of
    `arg_names`), synthesised constants filled with their value, outputs allocated; temps are
    kept by the program itself.  Returns [(binding, {name: buffer})]."""
    sets = []
    for _ in range(nsets):
        named = {}
        for b in prog.buffers:
            if b["elided"] or b["role"] == "temp":
                continue
            buf = hb.HipBuffer(dev, [b["bytes"]], None, nbytes=b["bytes"])
            if b["name"] in arg_names:
                buf.write_array(np.ascontiguousarray(arrays[arg_names.index(b["name"])]))
            elif b["name"] in const_inputs:
                fill = {"ones": 1.0, "zeros": 0.0, "scalar": 1.0}[const_inputs[b["name"]]]
                buf.write_array(np.full(b["bytes"] // 4, fill, dtype=np.float32))
            named[b["name"]] = buf
        sets.append((prog.bind(named), named))
    return sets


def time_steps(dev, prog, sets, steps, warmup):
    """(event ms, wall ms) per step over exactly `steps` launches after `warmup` untimed ones."""
    for i in range(warmup):
        prog.run(sets[i % len(sets)][0], sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        prog.run(sets[i % len(sets)][0], sync=False)
    e1.record()
    e1.sync()
    dev.sync()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_ms(e1) / steps, wall / steps


def time_replays(dev, prog, sets, steps, warmup):
    """As `time_steps`, with each binding recorded once as a HIP graph and a step = one replay."""
    graphs = [prog.record(b) for b, _ in sets]
    for i in range(warmup):
        graphs[i % len(graphs)].replay(sync=False)
    dev.sync()
    e0, e1 = hb.Event(dev), hb.Event(dev)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        graphs[i % len(graphs)].replay(sync=False)
    e1.record()
    e1.sync()
    dev.sync()
    wall = (time.perf_counter() - t0) * 1e3
    return e0.elapsed_ms(e1) / steps, wall / steps
