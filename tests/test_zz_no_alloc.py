"""eh_program_execute_static: the execute entry point that allocates no device memory.

Its kernels are the ones eh_program_execute launches; only the scratch temps the plan appended
(pieces of cut reduce lines, chunk totals of scans, split-K partial tiles) sit in the device's
static block instead of buffers of their own.  Results must therefore equal eh_program_execute's
bit for bit, call after call, also when a later call uses less of the block than the one before
it and finds that call's leftovers there.
"""

import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RNG = lambda seed: np.random.default_rng(seed)  # noqa: E731


def _program(hip, dev, shapes, fn, options=None):
    from harp_amd import workloads as wl
    ast, names, out, _consts, _ = wl.lower_with_table(list(shapes), fn)
    return hip.HipProgram(dev, ast, options), names, out


def _run_both(hip, dev, prog, names, out, arrays):
    """Runs the program through eh_program_execute and through eh_program_execute_static on
    separate output buffers; returns both results and the scratch bytes the plan needs."""
    from harp_amd._lib import lib, check
    bufs = {}
    for n, a in zip(names, arrays):
        bufs[n] = dev.alloc(a.nbytes)
        bufs[n].write_array(a)
    own = [b for b in prog.buffers if not b["name"].startswith("eh_")]
    scratch = [b for b in prog.buffers if b["name"].startswith("eh_") and not b["elided"]]
    assert scratch, "the plan under test must use a scratch temp"
    out_bytes = next(b["bytes"] for b in prog.buffers if b["name"] == out)
    results = []
    for entry in (lib.eh_program_execute, lib.eh_program_execute_static):
        res = dev.alloc(out_bytes)
        res.write_array(np.full(out_bytes // 4, np.nan, np.float32))
        named = dict(bufs)
        named[out] = res
        # the caller's own temps must be given to the entry point that does not allocate
        temps = {b["name"]: dev.alloc(b["bytes"]) for b in own
                 if b["role"] == "temp" and not b["elided"]}
        named.update(temps)
        arr = (ctypes.c_void_p * len(own))()
        for i, b in enumerate(own):
            arr[i] = named[b["name"]]._h if b["name"] in named else None
        check(entry(prog._h, arr, len(own), 1))
        results.append(res.read_array(np.float32))
    return results[0], results[1], sum((b["bytes"] + 255) // 256 * 256 for b in scratch)


CASES = [
    # (name, input shapes, graph, float64 statement, options) -- each plan appends a scratch temp
    ("sum_4x1M", [(4, 1 << 20)], lambda t: t.sum(1), lambda x: x.sum(1), None),
    ("max_2x300k", [(2, 300_000)], lambda t: t.max(1), lambda x: x.max(1), None),
    ("cumsum_2x1M", [(2, 1 << 20)], lambda t: t.cumsum(1), lambda x: np.cumsum(x, 1), None),
    ("cumsum_3x40k", [(3, 40_000)], lambda t: t.cumsum(1), lambda x: np.cumsum(x, 1), None),
    ("matmul_96x8192x80_split", [(96, 8192), (8192, 80)], None, lambda a, b: a @ b, "gemm_split_k=8"),
    ("matmul_64x2048x48_split", [(64, 2048), (2048, 48)], None, lambda a, b: a @ b, "gemm_split_k=4"),
]


def _graph(case):
    from harp_amd.frontend import nn
    return case[2] if case[2] is not None else (lambda a, b: nn.matmul(a, b))


@pytest.mark.parametrize("pair", [(0, 1), (2, 3), (4, 5), (2, 1)], ids=lambda p: f"{CASES[p[0]][0]}-then-{CASES[p[1]][0]}")
def test_static_scratch_execute_equals_the_allocating_execute(frontend, hip, pair):
    """Two calls in a row on one device, the second with a smaller input (and a smaller share of
    the block): each equals eh_program_execute bit for bit and float64 within the reduction
    tolerance."""
    dev = hip.HipDevice(0)
    used = []
    for ci in pair:
        name, shapes, _fn, exact_fn, options = CASES[ci]
        arrays = [RNG(7 + ci + k).uniform(-1.0, 1.5, s).astype(np.float32) for k, s in enumerate(shapes)]
        prog, names, out = _program(hip, dev, shapes, _graph(CASES[ci]), options)
        ref, got, need = _run_both(hip, dev, prog, names, out, arrays)
        used.append(need)
        assert 0 < need <= (8 << 20), (name, need)
        assert not np.isnan(got).any(), name
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32)), name
        x64 = [a.astype(np.float64) for a in arrays]
        exact = exact_fn(*x64).ravel()
        scale = exact_fn(*[np.abs(a) for a in x64]).ravel()
        assert np.all(np.abs(got.ravel().astype(np.float64) - exact) <= 1e-5 * scale + 1e-30), name
    assert used[1] < used[0], used


def test_static_scratch_execute_refuses_what_does_not_fit(frontend, hip):
    """Split-K partial tiles of 1024 x 1024 x 8 floats are 32 MiB: more than the 8 MiB block.
    The call fails with a size error before anything is launched, and the allocating entry point
    still runs the same program."""
    from harp_amd._lib import lib, check, EhError
    from harp_amd.frontend import nn
    dev = hip.HipDevice(0)
    shapes = [(1024, 4096), (4096, 1024)]
    prog, names, out = _program(hip, dev, shapes, lambda a, b: nn.matmul(a, b), "gemm_split_k=8")
    scratch = [b for b in prog.buffers if b["name"].startswith("eh_part_")]
    assert scratch and scratch[0]["bytes"] == 8 * 1024 * 1024 * 4
    a = RNG(1).uniform(-1, 1, shapes[0]).astype(np.float32)
    b = RNG(2).uniform(-1, 1, shapes[1]).astype(np.float32)
    bufs = {names[0]: dev.alloc(a.nbytes), names[1]: dev.alloc(b.nbytes), out: dev.alloc(4 << 20)}
    bufs[names[0]].write_array(a)
    bufs[names[1]].write_array(b)
    own = [x for x in prog.buffers if not x["name"].startswith("eh_")]
    arr = (ctypes.c_void_p * len(own))()
    for i, x in enumerate(own):
        arr[i] = bufs[x["name"]]._h
    with pytest.raises(EhError, match="static scratch block holds 8388608") as e:
        check(lib.eh_program_execute_static(prog._h, arr, len(own), 1))
    assert e.value.code == 6            # EH_ERR_SIZE
    assert np.all(bufs[out].read_array(np.float32) == 0)      # nothing ran
    check(lib.eh_program_execute(prog._h, arr, len(own), 1))
    got = bufs[out].read_array(np.float32).reshape(1024, 1024)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    assert np.allclose(got, ref, rtol=0, atol=1e-3 * float(np.abs(a).astype(np.float64).sum(1).max()))


def test_static_scratch_execute_needs_every_buffer_of_the_caller(frontend, hip):
    """A missing output is an error, not an allocation."""
    from harp_amd._lib import lib, check, EhError
    dev = hip.HipDevice(0)
    prog, names, out = _program(hip, dev, [(2, 300_000)], lambda t: t.max(1))
    x = dev.alloc(2 * 300_000 * 4)
    arr = (ctypes.c_void_p * 2)()
    for i, b in enumerate(prog.buffers[:2]):
        arr[i] = x._h if b["name"] == names[0] else None
    with pytest.raises(EhError, match="allocates nothing"):
        check(lib.eh_program_execute_static(prog._h, arr, 2, 1))


def _hip_runtime():
    rt = ctypes.CDLL("libamdhip64.so")
    rt.hipMemGetInfo.argtypes = [ctypes.POINTER(ctypes.c_size_t), ctypes.POINTER(ctypes.c_size_t)]
    rt.hipStreamBeginCapture.argtypes = [ctypes.c_void_p, ctypes.c_int]
    rt.hipStreamEndCapture.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]
    rt.hipGraphInstantiate.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
    rt.hipGraphLaunch.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    rt.hipStreamSynchronize.argtypes = [ctypes.c_void_p]
    rt.hipGraphExecDestroy.argtypes = [ctypes.c_void_p]
    rt.hipGraphDestroy.argtypes = [ctypes.c_void_p]
    return rt


def _free_bytes(rt):
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert rt.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _bound(hip, dev, prog, names, out, arrays):
    """Every buffer of the caller's table allocated and filled; (pointer array, count, output buffer)."""
    bufs = {}
    for n, a in zip(names, arrays):
        bufs[n] = dev.alloc(a.nbytes)
        bufs[n].write_array(a)
    own = [b for b in prog.buffers if not b["name"].startswith("eh_")]
    for b in own:
        if b["name"] not in bufs and not b["elided"]:
            bufs[b["name"]] = dev.alloc(b["bytes"])
    arr = (ctypes.c_void_p * len(own))()
    for i, b in enumerate(own):
        arr[i] = bufs[b["name"]]._h if b["name"] in bufs else None
    return arr, len(own), bufs[out], bufs


def test_static_scratch_execute_allocates_no_device_memory(frontend, hip):
    """What the entry point is for: after a first call (which settles the output's deferred zero
    fill), further calls leave the driver's free memory and the device's pool of released blocks
    exactly as they were -- for a cut reduce line and for a split contraction."""
    from harp_amd._lib import lib, check
    rt = _hip_runtime()
    dev = hip.HipDevice(0)
    for ci in (0, 4):
        name, shapes, _fn, _exact, options = CASES[ci]
        arrays = [RNG(17 + k).uniform(-1.0, 1.5, s).astype(np.float32) for k, s in enumerate(shapes)]
        prog, names, out = _program(hip, dev, shapes, _graph(CASES[ci]), options)
        arr, n, res, _bufs = _bound(hip, dev, prog, names, out, arrays)
        check(lib.eh_program_execute_static(prog._h, arr, n, 1))
        want = res.read_array(np.float32).copy()
        kept = ctypes.c_size_t()
        free_before = _free_bytes(rt)
        for _ in range(3):
            check(lib.eh_program_execute_static(prog._h, arr, n, 1))
        assert _free_bytes(rt) == free_before, name
        assert np.array_equal(res.read_array(np.float32).view(np.uint32), want.view(np.uint32)), name


def test_static_scratch_execute_under_stream_capture(frontend, hip):
    """The advertised use: the launches of eh_program_execute_static(sync = 0) captured into a
    caller's graph on the device's stream (eh_device_stream), replayed twice with the output
    overwritten in between; every replay equals eh_program_execute bit for bit.  Also with the
    program's launches spread over two lanes (the fork and join of the side stream are recorded
    into the same graph).  Free device memory is not compared here: instantiating a graph takes
    a few MiB for the runtime's own argument pool; the test above measures the entry point."""
    from harp_amd._lib import lib, check
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    rt = _hip_runtime()
    dev = hip.HipDevice(0)
    stream = ctypes.c_void_p()
    check(lib.eh_device_stream(dev._h, ctypes.byref(stream)))
    assert stream.value

    def cnn_step(options):
        arrays = wl.config5_inputs(16, 28, 32, 64, 128, 10, seed=93)
        ts = [Tensor.input(list(a.shape)) for a in arrays]
        ast, names, outs, consts, _ = wl.lower_multi(ts, wl.config5_graph(*ts, lr=0.05))
        prog = hip.HipProgram(dev, ast, options)
        bufs = {}
        for nme, a in zip(names, arrays):
            bufs[nme] = dev.alloc(a.nbytes)
            bufs[nme].write_array(a)
        for nme, val in consts.items():
            b = next(x for x in prog.buffers if x["name"] == nme)
            if not b["elided"]:
                bufs[nme] = dev.alloc(b["bytes"])
                bufs[nme].write_array(np.full(b["bytes"] // 4, val, np.float32))
        own = [b for b in prog.buffers if not b["name"].startswith("eh_")]
        for b in own:
            if b["name"] not in bufs and not b["elided"]:
                bufs[b["name"]] = dev.alloc(b["bytes"])
        arr = (ctypes.c_void_p * len(own))()
        for i, b in enumerate(own):
            arr[i] = bufs[b["name"]]._h if b["name"] in bufs else None
        return prog, arr, len(own), [bufs[o] for o in outs], bufs      # (bufs: the handles in arr stay alive)

    name, shapes, _fn, _exact, options = CASES[4]
    arrays = [RNG(27 + k).uniform(-1.0, 1.5, s).astype(np.float32) for k, s in enumerate(shapes)]
    prog, names, out = _program(hip, dev, shapes, _graph(CASES[4]), options)
    arr, n, res, _bufs = _bound(hip, dev, prog, names, out, arrays)
    cases = [("split contraction", prog, arr, n, [res])]
    alive = [_bufs]
    for opts in ("lanes=1", "lanes=2,lane_us=0,merge_launches=0"):
        p2, a2, n2, outs2, keep = cnn_step(opts)
        alive.append(keep)
        assert any(b["name"].startswith("eh_") and not b["elided"] for b in p2.buffers)
        if "lanes=2" in opts:
            assert len({l["lane"] for l in p2.launches}) == 2
        cases.append(("cnn step " + opts, p2, a2, n2, outs2))
    for what, prg, ar, cnt, outs in cases:
        check(lib.eh_program_execute(prg._h, ar, cnt, 1))
        want = [o.read_array(np.float32).copy() for o in outs]
        check(lib.eh_program_execute_static(prg._h, ar, cnt, 1))           # settles fills, creates the lanes' streams and events
        check(lib.eh_device_sync(dev._h))
        graph, exe = ctypes.c_void_p(), ctypes.c_void_p()
        assert rt.hipStreamBeginCapture(stream, 2) == 0                     # hipStreamCaptureModeRelaxed
        rc = lib.eh_program_execute_static(prg._h, ar, cnt, 0)
        assert rt.hipStreamEndCapture(stream, ctypes.byref(graph)) == 0
        check(rc)
        assert rt.hipGraphInstantiate(ctypes.byref(exe), graph, None, None, 0) == 0
        for replay in range(2):
            for o in outs:
                o.write_array(np.full(o.byte_len() // 4, np.nan, np.float32))
            assert rt.hipGraphLaunch(exe, stream) == 0
            assert rt.hipStreamSynchronize(stream) == 0
            for o, w in zip(outs, want):
                assert np.array_equal(o.read_array(np.float32).view(np.uint32), w.view(np.uint32)), (what, replay)
        assert rt.hipGraphExecDestroy(exe) == 0 and rt.hipGraphDestroy(graph) == 0
