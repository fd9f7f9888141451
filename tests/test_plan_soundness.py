"""Invariants of a plan, checked on the host over many seeded random programs (no GPU): what a
launch reads exists when it runs.  The planner folds, inlines and elides kernels in a dozen
passes; each pass has its own tests, and this one holds their composition to the two facts the
executor relies on."""
import numpy as np
import pytest

import graph_fuzz


def _programs(frontend, seed, kind):
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    if kind == "cnn":
        shapes, fn, desc = graph_fuzz.build_cnn(seed, frontend)
    elif kind == "windows":
        shapes, fn, desc = graph_fuzz.build(seed, frontend, kinds=(8, 12))
    else:
        shapes, fn, desc = graph_fuzz.build(seed, frontend)
    ts = [Tensor.input(list(s)) for s in shapes]
    yield desc + " forward", wl.lower_multi(ts, [fn(*ts)])
    with frontend.exact_mode():
        ts = [Tensor.input(list(s)) for s in shapes]
        loss = fn(*ts)
        while loss.ndim() > 0:
            loss = loss.sum(loss.ndim() - 1)
        try:
            loss.backward_with_params(ts)
        except NotImplementedError:
            return
        roots = [t.grad().contiguous() for t in ts if t.grad() is not None] + [loss]
        yield desc + " gradients", wl.lower_multi(ts, roots)


def _check(plan, arg_names, outs, desc):
    buffers = {b["name"]: b for b in plan.buffers}
    written = set(arg_names) | {n for n, b in buffers.items() if b["role"] in ("input", "ones", "zeros")}
    for l in plan.launches:
        for a, w in zip(l["args"], l["written"]):
            b = buffers.get(a)
            assert b is not None, (desc, l["entry"], a)
            # (1) a buffer that never reaches memory is nobody's parameter
            assert not b["elided"], (desc, l["entry"], a, l["kernels"])
            # (2) what a launch only reads has been written by an earlier launch, or is an input
            if not w:
                assert a in written, (desc, l["entry"], a, l["kernels"])
        written |= {a for a, w in zip(l["args"], l["written"]) if w}
    for o in outs:
        assert o in written and not buffers[o]["elided"], (desc, o)


SEEDS = [("graph", s) for s in list(range(3000, 3300)) + [2438]] + [("windows", s) for s in range(3600, 3660)] + \
        [("cnn", s) for s in range(3750, 3790)]


@pytest.mark.parametrize("kind,seed", SEEDS)
def test_what_a_launch_reads_exists(frontend, kind, seed):
    """Seed 2438 (gradients of a permuted relu, axes 2 x 2 x 1): a short reduce whose gather had
    been folded into a window-reduce launch of its own was also taken as a stage by the row group
    in front of it, and read the gather's buffer, which no launch wrote any more."""
    from harp_amd import backend as hb
    for desc, (ast, arg_names, outs, _consts, _plain) in _programs(frontend, seed, kind):
        for options in (None, "merge_launches=0"):
            try:
                plan = hb.render_program(ast, options)
            except hb.EhError as e:
                assert "EH_ERR_UNSUPPORTED" in str(e) or "unsupported" in str(e).lower() or "refused" in str(e).lower(), (desc, str(e))
                continue
            _check(plan, arg_names, outs if isinstance(outs, list) else [outs], desc)
