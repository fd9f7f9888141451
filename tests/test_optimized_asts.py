"""Kernels as the reference's AST optimiser may hand them over (ECLAT_OPT_LEVEL > 0,
`src/backend/executor.rs:169-176`): shifts for power-of-two strides, sums re-associated, loops
tiled with a remainder or a guard, tile and remainder loops unrolled, loops interchanged.

CPU part: the backend plans them exactly as it plans the lowered kernel; the normalised AST
computes, through the C oracle, bit for bit what the rewritten one computes (and the rewritten
one what the lowered one computes, which pins the test's own transforms); a kernel nothing
recognises is refused instead of run in one work-item.  GPU part: parity with the oracle on the
rewritten ASTs.
"""

import ctypes
import os

import numpy as np
import pytest

from conftest import bits_equal_mod_zero, realize_on

RNG = np.random.default_rng

TRANSFORMS = [
    [], ["tile=7"], ["tile=2"], ["guard=5"], ["tile=7", "unroll"], ["guard=3", "unroll"],
    ["tile_all=3"], ["tile_all=5", "unroll"], ["tile_outer=7"], ["interchange"],
    ["tile_outer=3", "unroll"], ["unroll"], ["tile_outer=5", "tile=3"], ["tile=5", "interchange", "unroll"],
    ["fma"], ["tile=7", "fma"],
]
IDS = ["+".join(t) or "rules" for t in TRANSFORMS]
# forms whose normalisation gives a sum back the order the lowerer wrote (an interchanged tile
# loop): the normalised kernel equals the rewritten one up to the order of the additions
REORDERING = {"tile=5+interchange+unroll"}


@pytest.fixture
def opt_env(monkeypatch):
    def set_(level, transforms=()):
        monkeypatch.setenv("ECLAT_OPT_LEVEL", str(level))
        monkeypatch.setenv("ECLAT_OPT_TRANSFORMS", ",".join(transforms))
    return set_


def _headline(name):
    from harp_amd import workloads as wl
    shapes = {"config1_relu_sum": [(1024, 1024)] * 3, "config2_softmax": [(4096, 4096)],
              "config3_matmul": [(4096, 4096)] * 2}[name]
    return shapes, wl.CONFIGS[name][1]


@pytest.mark.parametrize("transforms", TRANSFORMS, ids=IDS)
@pytest.mark.parametrize("config", ["config1_relu_sum", "config2_softmax", "config3_matmul"])
def test_rewritten_headline_kernels_are_planned_like_the_lowered_ones(frontend, opt_env, config, transforms):
    """Same schedule, grid and block as the as-lowered AST, on the whole-program path and kernel
    by kernel (what `compile_ast` receives)."""
    from harp_amd import backend as hb
    from harp_amd import workloads as wl
    from harp_amd.frontend import AstNode
    shapes, fn = _headline(config)
    opt_env(0)
    table0, _, _, _, plain0 = wl.lower_with_table(shapes, fn)
    opt_env(3, transforms)
    table1, _, _, _, plain1 = wl.lower_with_table(shapes, fn)
    if transforms or config != "config2_softmax":
        assert table1.to_sexpr() != table0.to_sexpr()          # the optimiser did rewrite something
    if config != "config2_softmax":
        assert "(shl " in table1.to_sexpr()                      # power-of-two strides became shifts

    def dispatch(ast):
        return [(l["schedule"], l["grid"], l["block"]) for l in hb.render_program(ast).launches]
    assert dispatch(table1) == dispatch(table0)
    for k0, k1 in zip(plain0.args, plain1.args):
        assert dispatch(AstNode.program([k1])) == dispatch(AstNode.program([k0])), k0.attrs["name"]


def _graphs(fe):
    nn = fe.nn
    return {
        "mul_add_bcast": ([(6, 23), (23,)], lambda a, b: a * b.unsqueeze(0).expand(0, 6) + a),
        "sum_last": ([(5, 37)], lambda a: (a * a).sum(1)),
        "max_first": ([(9, 16)], lambda a: a.max(0)),
        "softmax": ([(7, 19)], lambda a: nn.softmax(a, 1)),
        "matmul": ([(10, 21), (21, 8)], lambda a, b: nn.matmul(a, b)),
        "permute_copy": ([(4, 9, 8)], lambda a: a.permute([2, 0, 1]).contiguous() + a.permute([2, 0, 1])),
        "pad": ([(5, 11)], lambda a: a.pad([(1, 2), (3, 0)]) * a.pad([(1, 2), (3, 0)])),
        "cumsum": ([(4, 29)], lambda a: a.cumsum(1)),
    }


GRAPHS = ["mul_add_bcast", "sum_last", "max_first", "softmax", "matmul", "permute_copy", "pad", "cumsum"]


@pytest.mark.parametrize("name", GRAPHS)
def test_normalised_kernels_compute_what_the_rewritten_ones_compute(frontend, opt_env, name):
    """Every kernel of the graph, in every rewritten form, through the C oracle: the rewritten
    kernel against the lowered one (equal bits unless the rules re-associated a float sum), and
    the backend's normalised AST against the rewritten one (equal bits always)."""
    from harp_amd import backend as hb
    from harp_amd.frontend import AstNode, lower_graph, optimize
    from oracle.c_backend import CKernel
    from oracle.c_renderer import render_program
    shapes, fn = _graphs(frontend)[name]
    opt_env(0)
    ts = [frontend.Tensor.input(list(s)) for s in shapes]
    prog, lw, _ = lower_graph([fn(*ts).graph])
    rng = RNG(len(name))
    for kern in prog.args:
        params = [p for p in kern.attrs["params"] if p.dtype.is_ptr()]
        variants = {"lowered": kern}
        for t, tid in zip(TRANSFORMS, IDS):
            rewritten = optimize.optimize_kernel(kern, t)
            variants["rw_" + tid] = rewritten
            variants["nm_" + tid] = hb.normalize_ast(rewritten)
        # one translation unit: every variant under its own entry point
        funcs, entries = {}, {}
        for i, (vid, k) in enumerate(variants.items()):
            text = k if isinstance(k, str) else k.to_sexpr()
            entry = f"v{i}_{kern.attrs['name']}"
            assert text.startswith(f'(kernel "{kern.attrs["name"]}"')
            funcs[vid] = text.replace(f'(kernel "{kern.attrs["name"]}"', f'(kernel "{entry}"', 1)
            entries[vid] = entry

        def build(vids):
            # strict IEEE arithmetic: with -ffast-math gcc re-associates a reduction differently for
            # every loop structure, and equal evaluation order could not be seen in the bits
            return CKernel(render_program("(program " + " ".join(funcs[v] for v in vids) + ")"),
                           entries["lowered"], len(params), gcc_args=["-O1", "-shared", "-fPIC"])
        live = list(variants)
        try:
            lib = build(live)
        except RuntimeError:
            # The reference renders a nested block without braces (src/backend/renderer.rs:604-624),
            # so a rewritten form that repeats a block with a declaration (an unrolled loop around
            # an accumulator) is not valid C for its own C backend either: such forms are left out
            # here (the GPU test still runs them).
            live = ["lowered"]
            for tid in IDS:
                try:
                    build(["lowered", "rw_" + tid])
                    live += ["rw_" + tid, "nm_" + tid]
                except RuntimeError as e:
                    assert "redeclaration" in str(e), str(e)
            lib = build(live)
        assert len(live) >= 1 + 2 * 8, live
        sizes = {p.name: int(np.prod([int(e.evaluate()) for e in lw.get_buffer_info_by_name(p.name)[0]]))
                 for p in params}
        inputs = {p.name: rng.uniform(-2, 2, sizes[p.name]).astype(np.float32) for p in params if not p.mutable}

        def run(entry):
            outs = {p.name: np.zeros(sizes[p.name], np.float32) for p in params if p.mutable}
            args = [inputs[p.name] if not p.mutable else outs[p.name] for p in params]
            fn_ = getattr(lib._lib, entry)
            fn_.restype = None
            fn_(*[ctypes.c_void_p(a.ctypes.data) for a in args])
            return np.concatenate([outs[p.name] for p in params if p.mutable])
        base = run(entries["lowered"])
        for tid in IDS:
            if "rw_" + tid not in live:
                continue
            rw, nm = run(entries["rw_" + tid]), run(entries["nm_" + tid])
            # (interchanging the two loops of a tiled scan reorders a recurrence: the reference's
            # suggester does not check dependences, loop_transforms.rs:710-793, and the form no longer
            # computes the scan; the normalised kernel must still compute what that form computes)
            if not (tid in REORDERING and kern.attrs["name"].startswith("P_")):
                assert np.allclose(rw, base, rtol=1e-5, atol=1e-6), (kern.attrs["name"], tid)
            if tid in REORDERING and kern.attrs["name"].startswith("R_"):
                assert np.allclose(nm, rw, rtol=1e-5, atol=1e-6), (kern.attrs["name"], tid)
                assert bits_equal_mod_zero(nm, base) or name == "softmax", (kern.attrs["name"], tid)   # the lowered order is back
            else:
                assert bits_equal_mod_zero(nm, rw), (kern.attrs["name"], tid)


def test_normalisation_restores_the_lowered_loop_nest(frontend, opt_env):
    """For the plain forms the normalised text is the lowered text itself, shifts, tiles and
    unrolled remainders gone."""
    from harp_amd import backend as hb
    from harp_amd.frontend import lower_graph, optimize
    opt_env(0)
    a, b = frontend.Tensor.input([64, 100]), frontend.Tensor.input([64, 100])
    prog, _, _ = lower_graph([(a * b).graph])
    kern = prog.args[0]
    want = hb.normalize_ast(kern)
    assert "(shl" not in want and "ridx" in want
    for t in (["tile=7"], ["tile=7", "unroll"], ["guard=3"], ["tile_all=3"], ["tile_outer=5", "tile=3"]):
        rewritten = optimize.optimize_kernel(kern, t)
        assert rewritten.to_sexpr() != kern.to_sexpr()
        assert hb.normalize_ast(rewritten) == want, t


def _odd_kernel(n):
    """out[i] = t, t = t * 0.5 + x[i]: a recurrence no schedule recognises."""
    from harp_amd.frontend import AstNode as A
    from harp_amd.frontend.ast import DType, F32, VarDecl
    c = A.const_i64
    step = A.assign("t", A.add(A.mul(A.var("t"), A.const_f32(0.5)), A.load(A.var("x"), A.var("i"), F32)))
    body = A.block([A.assign("t", A.const_f32(0.0)),
                    A.range("i", c(0), c(1), c(n), A.block([step, A.store(A.var("y"), A.var("i"), A.var("t"))]))],
                   decls=[("t", F32)])
    params = [VarDecl("x", DType.ptr(F32)), VarDecl("y", DType.ptr(F32), mutable=True)]
    return A.program([A.kernel("odd_recurrence", params, body)])


def test_long_serial_kernels_are_refused_not_run_in_one_work_item():
    from harp_amd import backend as hb
    from harp_amd._lib import EhError
    small = hb.render_program(_odd_kernel(1000)).launches
    assert [l["schedule"] for l in small] == ["as-written"] and small[0]["grid"] == [1, 1, 1]
    with pytest.raises(EhError, match="would run its 300000 loop iterations in one work-item") as e:
        hb.render_program(_odd_kernel(300_000))
    assert e.value.code == 3                         # EH_ERR_UNSUPPORTED
    forced = hb.render_program(_odd_kernel(300_000), "allow_serial=1").launches
    assert [l["schedule"] for l in forced] == ["as-written"]


def _plain_kernels(config, transforms, opt_env):
    from harp_amd import workloads as wl
    from harp_amd.frontend import optimize
    shapes, fn = _headline(config)
    opt_env(0)
    plain = wl.lower_with_table(shapes, fn)[4]
    return [(k, optimize.optimize_kernel(k, transforms)) for k in plain.args]


@pytest.mark.parametrize("config", ["config1_relu_sum", "config2_softmax"])
def test_nested_tiling_with_moving_bounds_is_refused(frontend, opt_env, config):
    """The inner loops of a tiling tiled again (src/opt/ast/suggesters/loop_transforms.rs:86-110
    proposes tiling for every step-1 loop, nested ones included): re-tiling a remainder loop that
    does not start at 0 (`tile_loop`, src/opt/ast/transforms.rs:450-461) leaves a nest whose inner
    bound moves with an outer variable.  Counted over the outer loop's range it is millions of
    iterations for one work-item: refused, never launched at 1x1x1."""
    from harp_amd import backend as hb
    from harp_amd._lib import EhError
    from harp_amd.frontend import AstNode
    for k, rw in _plain_kernels(config, ["tile=2", "tile=3"], opt_env):
        nm = hb.normalize_ast(rw)
        assert "eh_u" in nm or "eh_c" in nm                       # a rolled loop with a moving bound survived normalisation
        with pytest.raises(EhError, match="loop iterations in one work-item") as e:
            hb.render_program(AstNode.program([rw]))
        assert e.value.code == 3, k.attrs["name"]                 # EH_ERR_UNSUPPORTED


def test_forms_no_schedule_recovers_are_marked_degraded(frontend, opt_env, capfd):
    """`tile_all=7` then `tile=2` re-tiles the remainder loop [4095, 4096) of a 4096-long axis with the
    reference's wrong main-loop bound: the rewritten kernel itself reads one element past the axis.
    Nothing is recovered from that; the plan says so (`degraded`) and the library logs it once, for
    the elementwise and row kernels as for the contraction that misses the matrix cores.  Where the
    same composition is clean (1024 = 7 * 146 + 2) the lowered schedules come back."""
    from harp_amd import backend as hb
    from harp_amd.frontend import AstNode
    for k, rw in _plain_kernels("config3_matmul", ["tile_all=7", "tile=2"], opt_env):
        sched = [l["schedule"] for l in hb.render_program(AstNode.program([rw])).launches]
        assert sched == ["outer-parallel(work-items=16777216,degraded)"]
        hb.render_program(AstNode.program([rw]))
    assert capfd.readouterr().err.count("plan marked 'degraded'") <= 1        # logged once per kernel
    for k, rw in _plain_kernels("config2_softmax", ["tile_all=7", "tile=2"], opt_env):
        sched = [l["schedule"] for l in hb.render_program(AstNode.program([rw])).launches]
        assert sched == ["outer-parallel(work-items=4096,degraded)"], k.attrs["name"]
    for k, rw in _plain_kernels("config1_relu_sum", ["tile_all=7", "tile=2"], opt_env):
        want = [l["schedule"] for l in hb.render_program(AstNode.program([k])).launches]
        assert [l["schedule"] for l in hb.render_program(AstNode.program([rw])).launches] == want


# ---------------------------------------------------------------------------------------------
# GPU
# ---------------------------------------------------------------------------------------------

GPU_TRANSFORMS = [[], ["tile=7"], ["guard=5"], ["tile=7", "unroll"], ["tile_all=3"], ["tile_outer=7"],
                  ["interchange"], ["tile=7", "interchange"], ["tile=5", "interchange", "unroll"], ["fma"]]


@pytest.mark.gpu
@pytest.mark.parametrize("transforms", GPU_TRANSFORMS, ids=["+".join(t) or "rules" for t in GPU_TRANSFORMS])
@pytest.mark.parametrize("fuse", [False, True])
def test_rewritten_kernels_match_the_oracle_on_the_gpu(frontend, hip, opt_env, transforms, fuse):
    """Configs 1 to 3 (reduced sizes), both paths, HIP and oracle on the same rewritten AST:
    elementwise outputs bit-exact, reductions within 1e-5, matmul within 1e-3 of the row scale."""
    from harp_amd import workloads as wl
    opt_env(3, transforms)
    a, b, c = [RNG(s).normal(0, 1, (300, 1000)).astype(np.float32) for s in (1, 2, 3)]
    ref = realize_on(frontend, "c", lambda x, y, z: x * y + z, [a, b, c])
    got = realize_on(frontend, "hip", lambda x, y, z: x * y + z, [a, b, c], fuse=fuse)
    assert bits_equal_mod_zero(ref, got)
    ref = realize_on(frontend, "c", wl.config1_graph, [a, b, c])
    got = realize_on(frontend, "hip", wl.config1_graph, [a, b, c], fuse=fuse)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-5)
    x = RNG(4).normal(0, 2, (257, 4096)).astype(np.float32)
    ref = realize_on(frontend, "c", wl.config2_graph, [x])
    got = realize_on(frontend, "hip", wl.config2_graph, [x], fuse=fuse)
    assert np.allclose(got, ref, rtol=1e-5, atol=1e-12)
    p, q = RNG(5).uniform(-1, 1, (192, 640)).astype(np.float32), RNG(6).uniform(-1, 1, (640, 160)).astype(np.float32)
    ref = realize_on(frontend, "c", wl.config3_graph, [p, q])
    got = realize_on(frontend, "hip", wl.config3_graph, [p, q], fuse=fuse)
    scale = np.abs(p).astype(np.float64) @ np.abs(q).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - ref.reshape(got.shape)) <= 1e-3 * scale.reshape(got.shape))
    assert np.allclose(got.reshape(192, 160), p.astype(np.float64) @ q.astype(np.float64), rtol=0, atol=1e-4 * scale.max())


@pytest.mark.gpu
def test_opt_levels_give_the_same_results_on_the_gpu(frontend, hip, opt_env):
    """Level 0 and level 3 (rule set) differ in the AST text only."""
    from harp_amd import workloads as wl
    x = RNG(9).normal(0, 2, (128, 2048)).astype(np.float32)
    outs = []
    for level in (0, 3):
        opt_env(level)
        outs.append(realize_on(frontend, "hip", wl.config2_graph, [x]))
    assert np.allclose(outs[0], outs[1], rtol=1e-6, atol=1e-12)


@pytest.mark.gpu
def test_fused_multiply_add_forms_match_the_oracle_on_the_gpu(frontend, hip, opt_env):
    """What the multiply-add rules produce for a device that reports `DeviceInstruction::Fma`
    (src/opt/ast/rules/mod.rs:117-143; algebraic.rs:218-282), as `Pipeline::optimize_ast` would
    hand it over.  Elementwise `fma(a, b, c)` is bit-identical to the C backend's `fma(a, b, c)`
    (double-precision fma on promoted floats, converted back), also where float arithmetic in
    two steps or a single-precision fused multiply-add would give another value; a reduce whose
    step is `acc = fma(a, b, acc)` is planned as the sum of products it is (row, column and MFMA
    schedules) and stays within the reduction tolerances."""
    from harp_amd.frontend import AstNode as A
    from harp_amd.frontend.ast import DType, F32, VarDecl
    from oracle.c_backend import CBuffer, compile_program_text
    dev = hip.HipDevice(0)
    n = 1 << 16
    idx = A.var("ridx0")
    body = A.range("ridx0", A.const_i64(0), A.const_i64(1), A.const_i64(n),
                   A.store(A.var("buf6"), idx, A("fma", [A.load(A.var("buf0"), idx, F32), A.load(A.var("buf2"), idx, F32),
                                                         A.load(A.var("buf4"), idx, F32)])))
    params = [VarDecl(v, DType.ptr(F32)) for v in ("buf0", "buf2", "buf4")] + [VarDecl("buf6", DType.ptr(F32), mutable=True)]
    prog = A.program([A.kernel("E_fma", params, body)])
    rng = RNG(11)
    x, y = (rng.uniform(1, 2, n).astype(np.float32) for _ in range(2))
    z = (-(x.astype(np.float64) * y.astype(np.float64))).astype(np.float32)        # cancels all but the product's low bits
    x[:4] = [1 + 2.0 ** -12, 1 + 2.0 ** -23, 3.0, 1.5]
    y[:4] = [1 + 2.0 ** -12, 1 - 2.0 ** -23, 7.0, -2.0]
    z[:4] = [-1.0, -1.0, 0.25, 3.0]
    k = hip.HipKernel(dev, prog)
    assert k.launches[0]["schedule"].startswith("flat(") and "fma((double)" in k.launches[0]["source"]
    bufs = [dev.alloc(4 * n) for _ in range(4)]
    for b, a in zip(bufs, (x, y, z)):
        b.write_array(a)
    k.execute(bufs[:3], bufs[3:])
    got = bufs[3].read_array(np.float32)
    ck = compile_program_text(prog.to_sexpr())
    cb = [CBuffer([n], "f32") for _ in range(4)]
    for b, a in zip(cb, (x, y, z)):
        b.write_from_host(a.tobytes())
    ck.execute(cb[:3], cb[3:])
    ref = np.frombuffer(cb[3].read_to_host(), np.float32)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    want = (x.astype(np.float64) * y.astype(np.float64) + z.astype(np.float64)).astype(np.float32)
    assert np.array_equal(got, want)
    assert np.count_nonzero(got != (x * y + z)) > n // 4            # two float roundings lose the residue

    # reductions in fma form: a row dot product, a column one, a contraction
    opt_env(3, ["fma"])
    a = RNG(12).normal(0, 1, (300, 1000)).astype(np.float32)
    b = RNG(13).normal(0, 1, (300, 1000)).astype(np.float32)
    for axis in (1, 0):
        fn = lambda p, q: (p * q).sum(axis)                                          # noqa: E731
        ref = realize_on(frontend, "c", fn, [a, b])
        for fuse in (False, True):
            got = realize_on(frontend, "hip", fn, [a, b], fuse=fuse)
            scale = (np.abs(a.astype(np.float64)) * np.abs(b)).sum(axis)
            assert np.all(np.abs(got.astype(np.float64).ravel() - ref.ravel()) <= 1e-5 * scale.ravel())
    from harp_amd import workloads as wl
    table = wl.lower_with_table([(192, 640), (640, 160)], wl.config3_graph)[0]
    assert "(fma " in table.to_sexpr()
    assert hip.render_program(table).launches[0]["schedule"].startswith("mfma32x32x2(")


def _fuzz_graph(frontend, seed):
    import graph_fuzz
    kinds = (0, 8) if seed % 3 else (8, 12)
    return graph_fuzz.build(seed, frontend, kinds=kinds)


@pytest.mark.parametrize("seed", [60022, 60028, 60112, 60130])
def test_unrolled_loop_around_a_reduction_compiles(frontend, opt_env, seed):
    """`tile_outer=3` + `unroll` repeats a reduction's block, accumulator declaration and all.  The
    reference prints a block inside a block without braces (src/backend/renderer.rs:604-624), which
    makes the second `float acc;` a redefinition -- for its own C backend too.  Rendered as written
    here, such a block gets its braces and compiles."""
    from harp_amd import backend as hb
    from harp_amd.frontend import AstNode, lower_graph, optimize
    opt_env(0)
    shapes, fn, desc = _fuzz_graph(frontend, seed)
    ts = [frontend.Tensor.input(list(s)) for s in shapes]
    prog, _, _ = lower_graph([fn(*ts).graph])
    repeated = 0
    for kern in prog.args:
        rw = optimize.optimize_kernel(kern, ["tile_outer=3", "unroll"])
        # (normalize=0: the form as it arrives; normalised, the loops come back and nothing repeats)
        for l in hb.render_program(AstNode.program([rw]), "normalize=0").launches:
            repeated += l["source"].count("float acc;") > 1
            assert len(hb.compile_source(l["source"])) > 500, (desc, kern.attrs["name"])
    assert repeated >= 1, desc


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [60022, 60040, 60085, 60130])
@pytest.mark.parametrize("transforms", [["tile_outer=3", "unroll"], ["guard=3", "unroll"]], ids=["tile_outer=3+unroll", "guard=3+unroll"])
def test_rewritten_random_graphs_match_the_oracle_on_the_gpu(frontend, hip, opt_env, seed, transforms):
    """Random graphs in forms that mostly fall back to the as-written and outer-parallel schedules
    (small axes, unrolled tile loops): HIP on the rewritten AST against the oracle on the lowered one."""
    import graph_fuzz
    large = seed % 5 == 0
    kinds = (0, 8) if seed % 3 else (8, 12)
    shapes, fn, desc = graph_fuzz.build(seed, frontend, kinds=kinds, dims=graph_fuzz.LARGE_DIMS if large else graph_fuzz.SMALL_DIMS,
                                        max_rank=2 if large else 3)
    arrays = [RNG(seed).uniform(-1.5, 1.5, s).astype(np.float32) for s in shapes]
    with frontend.exact_mode():
        opt_env(0)
        ref = np.asarray(realize_on(frontend, "c", fn, arrays))
        opt_env(3, transforms)
        for fuse in (True, False):
            got = np.asarray(realize_on(frontend, "hip", fn, arrays, fuse=fuse))
            scale = max(1.0, float(np.abs(ref).max()))
            assert got.shape == ref.shape and np.allclose(got, ref, rtol=5e-5, atol=5e-6 * scale), (desc, fuse)


@pytest.mark.parametrize("seed", [50002, 50005, 50007, 50062])
def test_unrolled_tilings_of_small_axes_are_planned_like_the_lowered_kernels(frontend, opt_env, seed):
    """Axes of a few elements are unrolled whole.  Two things the normaliser undoes there: a guarded
    tiling whose tile loops were both unrolled and rolled back leaves `for v < 6 { if (v < 5) S }`,
    which is `for v < 5 S`; and the repetitions of an unrolled outer loop each hold inner loops
    that an earlier roll made, under fresh names (`eh_u0`, `eh_u1`, ...), which are renamed by
    position before repetitions (and a loop and its remainder) are compared."""
    from harp_amd import backend as hb
    from harp_amd.frontend import AstNode, lower_graph, optimize
    opt_env(0)
    shapes, fn, desc = _fuzz_graph(frontend, seed)
    ts = [frontend.Tensor.input(list(s)) for s in shapes]
    prog, _, _ = lower_graph([fn(*ts).graph])

    def dispatch(k):
        return [(l["schedule"], l["grid"], l["block"]) for l in hb.render_program(AstNode.program([k])).launches]
    rewritten = 0
    for kern in prog.args:
        if any(int(e) == 1 for e in kern.attrs["name"].split("_")[1:-1]):
            continue                      # (a loop that runs once and was unrolled away leaves no loop to find)
        for t in (["guard=3", "unroll"], ["tile_outer=3", "unroll"]):
            rw = optimize.optimize_kernel(kern, t)
            rewritten += rw.to_sexpr() != kern.to_sexpr()
            assert dispatch(rw) == dispatch(kern), (desc, kern.attrs["name"], t)
    assert rewritten >= 2, desc
