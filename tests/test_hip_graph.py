"""eh_program_record / eh_graph_replay: a program's launches captured as a HIP graph give, on
every replay, exactly what eh_program_execute gives on the same buffers (bit for bit: the same
kernels run on the same data in the same order)."""

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _cnn_sets(hb, dev, batch, seed, options=None):
    from harp_amd import measure, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(batch, 28, 32, 64, 128, 10, seed=seed)
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    roots = wl.config5_graph(*ts, lr=0.05)
    prog_ast, arg_names, outs, consts, _ = wl.lower_multi(ts, roots)
    prog = hb.HipProgram(dev, prog_ast, options)
    sets = measure.make_sets(dev, prog, arg_names, consts, arrays, 2)
    return prog, sets, arg_names, outs, arrays


def _read_outputs(named, outs):
    return [named[o].read_array(np.float32, (named[o].byte_len() // 4,)).copy() for o in outs]


def test_graph_replays_match_eager_runs(hip):
    """The CNN training step (conv, pooling, K-split contractions with partial sums, 40+ launches
    over program-owned temps): eager on binding 0, recorded on binding 1, replayed four times with
    eager runs, host writes and synchronisations in between; every replay equals the eager result."""
    hb = hip
    dev = hb.HipDevice(0)
    prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 8, seed=91)
    prog.run(sets[0][0], sync=True)
    want = _read_outputs(sets[0][1], outs)
    graph = prog.record(sets[1][0])
    for replay in range(4):
        for o in outs:                       # stale results must not survive a replay
            n = sets[1][1][o].byte_len() // 4
            sets[1][1][o].write_array(np.full(n, np.nan, np.float32))
        graph.replay(sync=(replay % 2 == 0))
        got = _read_outputs(sets[1][1], outs)
        for g, w in zip(got, want):
            assert np.array_equal(g, w), f"replay {replay} differs from the eager run"
        prog.run(sets[0][0], sync=True)      # eager work between replays
        for g, w in zip(_read_outputs(sets[0][1], outs), want):
            assert np.array_equal(g, w)


def test_graph_reads_buffer_contents_at_replay_time_and_outlives_the_program(hip):
    """New inputs written into the recorded buffers are what the next replay computes on; the
    graph keeps the code objects and temps alive after the program handle is gone."""
    hb = hip
    dev = hb.HipDevice(0)
    prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 4, seed=92)
    graph = prog.record(sets[1][0])
    graph.replay()
    first = _read_outputs(sets[1][1], outs)
    x2 = np.ascontiguousarray(arrays[0][::-1])
    sets[0][1][arg_names[0]].write_array(x2)
    sets[1][1][arg_names[0]].write_array(x2)
    prog.run(sets[0][0], sync=True)
    want = _read_outputs(sets[0][1], outs)
    del prog
    graph.replay()
    got = _read_outputs(sets[1][1], outs)
    assert not np.array_equal(got[-1], first[-1])
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_record_rejects_a_missing_input(hip):
    hb = hip
    dev = hb.HipDevice(0)
    prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 4, seed=93)
    named = dict(sets[0][1])
    del named[arg_names[0]]
    with pytest.raises(Exception, match="MissingInput"):
        prog.record(prog.bind(named))
    prog.run(sets[0][0], sync=True)          # the stream is still usable (no capture left open)


def test_other_threads_may_use_the_device_while_a_graph_is_recorded(hip):
    """Recording captures the device's one stream.  A second thread that allocates (a fill),
    writes, reads back and runs another program on the same device meanwhile must neither fail
    nor end up inside the graph: its work waits for the capture to end.  Every recorded graph
    still replays to the eager result, and everything the other thread read back is right."""
    import threading
    hb = hip
    dev = hb.HipDevice(0)
    prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 4, seed=94)
    prog.run(sets[0][0], sync=True)
    want = _read_outputs(sets[0][1], outs)
    from harp_amd import workloads as wl
    ast, names, out, consts, _ = wl.lower_with_table([(64, 96)], lambda t: t * t + t)
    other = hb.HipProgram(dev, ast, None)
    stop, errors, rounds = threading.Event(), [], [0]

    def churn():
        rng = np.random.default_rng(5)
        try:
            while not stop.is_set():
                x = rng.normal(0, 1, (64, 96)).astype(np.float32)
                xin, res = dev.alloc(x.nbytes), dev.alloc(x.nbytes)        # alloc = a fill on the stream
                assert not res.read_array(np.float32).any()
                xin.write_array(x)
                other.run(other.bind({names[0]: xin, out: res}), sync=True)
                assert np.array_equal(res.read_array(np.float32, x.shape), x * x + x)
                rounds[0] += 1
        except Exception as e:                                             # noqa: BLE001
            errors.append(e)

    t = threading.Thread(target=churn)
    t.start()
    try:
        for _ in range(12):
            graph = prog.record(sets[1][0])
            graph.replay(sync=True)
            for g, w in zip(_read_outputs(sets[1][1], outs), want):
                assert np.array_equal(g, w)
            del graph
    finally:
        stop.set()
        t.join(60)
    assert not errors, errors
    assert rounds[0] > 0


def test_lanes_change_nothing_but_the_timing(hip):
    """The CNN training step with its launches on one stream (the default), on two and spread over
    four lanes with no size limit: the same kernels see the same inputs, so every output is equal
    bit for bit -- on back-to-back executes that reuse the program's temps (a launch of the next
    execute must not overtake a side-lane launch of the one before), and as a recorded graph."""
    hb = hip
    dev = hb.HipDevice(0)
    want = None
    for options in (None, "lanes=2,merge_launches=0", "lanes=4,lane_us=0,merge_launches=0", "lanes=4,lane_us=0"):
        prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 16, seed=94, options=options)
        lanes = {l["lane"] for l in prog.launches}
        assert (len(lanes) == 1) == (options is None) or "merge_launches" not in options, lanes
        for _ in range(3):
            prog.run(sets[0][0], sync=False)
        dev.sync()
        got = _read_outputs(sets[0][1], outs)
        if want is None:
            want = got
        for g, w in zip(got, want):
            assert np.array_equal(g, w), options
        graph = prog.record(sets[1][0])
        for _ in range(2):
            graph.replay()
        for g, w in zip(_read_outputs(sets[1][1], outs), want):
            assert np.array_equal(g, w), options
        del graph, prog, sets
        dev.trim()


def test_contractions_issued_together_change_nothing_but_the_timing(hip):
    """A layer's input gradient and weight gradient as one launch (the kernel templates compiled
    as parts that share the launch's block of LDS) and as launches of their own; the poolings as
    tails of their convolutions' launches and as launches of their own: the same arithmetic on
    the same inputs, so every output of the CNN training step is equal bit for bit -- also on
    back-to-back executes and as a recorded graph."""
    hb = hip
    dev = hb.HipDevice(0)
    want = None
    for options in ("merge_templates=0,gemm_tail=0", "gemm_tail=0", None):
        prog, sets, arg_names, outs, arrays = _cnn_sets(hb, dev, 32, seed=95, options=options)
        pairs = [l for l in prog.launches if l["schedule"].startswith("together(mfma")]
        assert len(pairs) == (0 if options and "merge_templates" in options else 3), [l["schedule"] for l in prog.launches]
        # (and the poolings in their convolutions' launches, reading the workgroup's results from LDS)
        assert sum(",tail=" in l["schedule"] for l in prog.launches) == (0 if options else 2)
        for _ in range(2):
            prog.run(sets[0][0], sync=False)
        dev.sync()
        got = _read_outputs(sets[0][1], outs)
        if want is None:
            want = got
        for g, w in zip(got, want):
            assert np.array_equal(g, w), options
        graph = prog.record(sets[1][0])
        graph.replay()
        for g, w in zip(_read_outputs(sets[1][1], outs), want):
            assert np.array_equal(g, w), options
        del graph, prog, sets
        dev.trim()
