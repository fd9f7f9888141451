"""Two entries of a program's buffer table bound to the same memory.

The planner orders, merges and overlaps launches by the dependences it reads off buffer names, so
an in-place update (one buffer as a parameter and as its new value) would race; the library
refuses it on the host, on every execute path, and leaves read-only sharing alone.
"""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _sgd_like(hip, dev):
    """w' = w - g as one Program: two inputs, one output."""
    from harp_amd import workloads as wl
    ast, names, out, _c, _ = wl.lower_with_table([(128, 64), (128, 64)], lambda w, g: w - g)
    return hip.HipProgram(dev, ast), names, out


def _table(prog, named):
    arr = (ctypes.c_void_p * len(prog.buffers))()
    for i, b in enumerate(prog.buffers):
        arr[i] = named[b["name"]]._h if b["name"] in named else None
    return arr


def test_in_place_update_is_refused_on_every_execute_path(frontend, hip):
    from harp_amd._lib import EhError, check, lib
    dev = hip.HipDevice(0)
    prog, names, out = _sgd_like(hip, dev)
    w = np.random.default_rng(0).normal(size=(128, 64)).astype(np.float32)
    g = np.random.default_rng(1).normal(size=(128, 64)).astype(np.float32)
    bw, bg, bo = dev.alloc(w.nbytes), dev.alloc(g.nbytes), dev.alloc(w.nbytes)
    bw.write_array(w)
    bg.write_array(g)
    assert [b["role"] for b in prog.buffers if not b["elided"]] == ["input", "input", "output"]
    extra = {}
    aliased = _table(prog, {**extra, names[0]: bw, names[1]: bg, out: bw})           # w' written over w
    for call in (lambda: lib.eh_program_execute(prog._h, aliased, len(prog.buffers), 1),
                 lambda: lib.eh_program_execute_static(prog._h, aliased, len(prog.buffers), 1),
                 lambda: lib.eh_program_record(prog._h, aliased, len(prog.buffers), ctypes.byref(ctypes.c_void_p()))):
        with pytest.raises(EhError, match="overlapping device memory") as e:
            check(call())
        assert e.value.code == 1                                                      # EH_ERR_INVALID
    assert np.array_equal(bw.read_array(np.float32).reshape(w.shape), w)             # nothing ran
    # distinct buffers: runs, and matches the statement
    ok = _table(prog, {**extra, names[0]: bw, names[1]: bg, out: bo})
    check(lib.eh_program_execute(prog._h, ok, len(prog.buffers), 1))
    got = bo.read_array(np.float32).reshape(w.shape)
    assert np.array_equal(got, w - g)
    # the same buffer bound to both inputs is only read: allowed (w - w)
    shared = _table(prog, {**extra, names[0]: bw, names[1]: bw, out: bo})
    check(lib.eh_program_execute(prog._h, shared, len(prog.buffers), 1))
    got = bo.read_array(np.float32).reshape(w.shape)
    assert np.all(got == 0)
