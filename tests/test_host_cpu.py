"""Host-side checks that need no GPU: the C ABI exports what the header declares, the AST
reader, the renderer's schedules for the benchmark configurations, hiprtc compilation for gfx950,
and the front end's lowering structure."""

import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from harp_amd import _lib
    with open(os.path.join(ROOT, "include", "eclat_hip.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(eh_[a-z_0-9]+)\s*\(", header))
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(_lib.lib, name), f"{name} declared in eclat_hip.h but not exported"
    assert declared == set(_lib.EXPORTED)
    assert _lib.lib.eh_version() >= 100


def test_rust_binding_names_only_declared_symbols():
    """The Rust shim (never compiled here) may only bind what the header declares, with the
    same number of parameters."""
    with open(os.path.join(ROOT, "include", "eclat_hip.h")) as f:
        header = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    with open(os.path.join(ROOT, "crates", "backend-hip", "src", "ffi.rs")) as f:
        ffi = f.read()

    def arity(params):
        params = params.strip()
        return 0 if params in ("", "void") else params.count(",") + 1

    declared = {m.group(1): arity(m.group(2)) for m in re.finditer(r"\b(eh_[a-z_0-9]+)\s*\(([^)]*)\)", header)}
    bound = {m.group(1): arity(m.group(2)) for m in re.finditer(r"pub fn (eh_[a-z_0-9]+)\(([^)]*)\)", ffi)}
    assert len(bound) >= 15
    for name, n in bound.items():
        assert name in declared, f"{name} bound in ffi.rs but not declared in eclat_hip.h"
        assert declared[name] == n, f"{name}: {n} parameters in ffi.rs, {declared[name]} in the header"

    # parameter and return types, each side brought to one spelling: base type, then one
    # "*const" or "*mut" per level of indirection, outermost last
    def c_type(decl, is_param=True):
        decl = decl.strip()
        array = is_param and decl.endswith("]")
        decl = re.sub(r"\[[0-9]*\]$", "", decl).strip()
        if is_param:
            decl = re.sub(r"\b[A-Za-z_][A-Za-z_0-9]*$", "", decl).strip() if not decl.endswith("*") else decl
        toks = re.findall(r"\*|[A-Za-z_][A-Za-z_0-9]*", decl)
        # a `const` ahead of the first `*` qualifies the base type; one behind a `*` qualifies that pointer
        base, levels, base_const = [], [], False
        for t in toks:
            if t == "const":
                if levels:
                    levels[-1] = "ptrconst"
                else:
                    base_const = True
            elif t == "*":
                levels.append("*")
            else:
                base.append(t)
        base = " ".join(base)
        base = {"unsigned": "c_uint", "int": "c_int", "char": "c_char", "void": "c_void", "size_t": "usize",
                "unsigned long long": "u64", "float": "f32", "double": "f64"}.get(base, base)
        out, pointee_const = base, base_const
        for lv in levels:
            out += " *const" if pointee_const else " *mut"
            pointee_const = lv == "ptrconst"      # constness of this pointer matters for the next level out
        if array:
            out += " *const" if base_const else " *mut"
        return out

    def rust_type(t):
        t = t.strip()
        levels = []
        while t.startswith("*"):
            m = re.match(r"\*(const|mut)\s+", t)
            levels.append("*" + m.group(1))
            t = t[m.end():]
        t = {"c_ulonglong": "u64", "i32": "c_int", "u32": "c_uint"}.get(t, t)
        return " ".join([t] + list(reversed(levels)))

    def c_signature(name):
        m = re.search(r"([A-Za-z_][A-Za-z_0-9 ]*?[ \*]+)\b" + name + r"\s*\(([^)]*)\)", header)
        ret, params = m.group(1), m.group(2).strip()
        ps = [] if params in ("", "void") else [c_type(p) for p in params.split(",")]
        return c_type(ret.replace("extern", ""), is_param=False), ps

    def rust_signature(name):
        m = re.search(r"pub fn " + name + r"\(([^)]*)\)\s*(->\s*([^;]+))?;", ffi)
        params = m.group(1).strip()
        ps = [rust_type(p.split(":", 1)[1]) for p in params.split(",")] if params else []
        return rust_type(m.group(3)) if m.group(3) else "c_void", ps

    assert c_type("const char* ast_text") == "c_char *const" and c_type("eh_buffer* const* bufs") == "eh_buffer *mut *const"
    assert c_type("const unsigned grid[3]") == "c_uint *const" and c_type("const void** blob") == "c_void *const *mut"
    assert rust_type("*const *mut eh_buffer") == "eh_buffer *mut *const" and rust_type("*mut *const c_void") == "c_void *const *mut"
    for name in bound:
        assert rust_signature(name) == c_signature(name), (name, rust_signature(name), c_signature(name))
    # the whole-program path of the binding
    assert {"eh_program_num_buffers", "eh_program_buffer", "eh_program_execute"} <= set(bound)
    with open(os.path.join(ROOT, "crates", "backend-hip", "src", "lib.rs")) as f:
        lib_rs = f.read()
    for name in re.findall(r"ffi::(eh_[a-z_0-9]+)\(", lib_rs):
        assert name in bound, f"lib.rs calls ffi::{name}, which ffi.rs does not declare"
    assert "fn execute_program(" in lib_rs and "panic!" not in lib_rs
    with open(os.path.join(ROOT, "crates", "backend-hip", "src", "ser.rs")) as f:
        assert "panic!" not in f.read()


def test_core_edits_patch_is_well_formed():
    """Every hunk header of crates/backend-hip/core-edits.patch counts its own lines right, new
    line numbers follow from the old ones, and the executor hunks (skip of the optimisation
    stage for the HIP device, whole-program hook) are there."""
    with open(os.path.join(ROOT, "crates", "backend-hip", "core-edits.patch")) as f:
        lines = f.read().split("\n")
    delta, seen_files, i = 0, [], 0
    while i < len(lines):
        l = lines[i]
        if l.startswith("diff "):
            delta = 0
            seen_files.append(l.split(" b/")[1])
        m = re.match(r"@@ -(\d+)(?:,(\d+))? \+(\d+)(?:,(\d+))? @@", l)
        if m:
            old_start, old_n = int(m.group(1)), int(m.group(2) or 1)
            new_start, new_n = int(m.group(3)), int(m.group(4) or 1)
            body = []
            i += 1
            while i < len(lines) and lines[i][:1] in ("+", "-") and not lines[i].startswith(("+++", "---")):
                body.append(lines[i])
                i += 1
            assert sum(b[0] == "-" for b in body) == old_n, l
            assert sum(b[0] == "+" for b in body) == new_n, l
            if old_start or old_n:
                assert new_start == old_start + delta + (1 if old_n == 0 else 0), l
            delta += new_n - old_n
            continue
        i += 1
    assert {"src/backend/executor.rs", "src/backend/device.rs", "src/backend/program_exec.rs"} <= set(seen_files)
    text = "\n".join(lines)
    assert "if device_kind == DeviceKind::Hip" in text and "try_execute_program" in text


def test_c_client_renders_and_compiles_without_a_gpu():
    """tests/capi_client.c is strict C99 against include/eclat_hip.h: it builds with -Werror
    and renders + compiles a kernel for gfx950 with no Python and no device involved."""
    import subprocess
    from harp_amd import build as hb_build
    exe = hb_build.build_capi_client()
    r = subprocess.run([exe, "render"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    assert "render ok: ehk_E_4_0" in r.stdout and "gfx950" in r.stdout


def _program_with_table(fe, tensor):
    from harp_amd.frontend.executor import buffer_table
    from harp_amd.frontend.graph import collect_inputs
    prog, lw, _ = fe.lower_graph([tensor.graph])
    ins = [lw.lookup_buffer_name(n) for n in collect_inputs([tensor.graph])]
    outs = [p.name for k in prog.args for p in k.attrs["params"] if p.mutable]
    last = max(outs, key=lambda s: int(s[3:]))
    return fe.AstNode.program(prog.args, buffers=buffer_table(prog, lw, ins, [last]))


def test_config2_softmax_is_one_row_kernel(frontend):
    from harp_amd import backend as hb
    x = frontend.Tensor.input([4096, 4096])
    plan = hb.render_program(_program_with_table(frontend, frontend.nn.softmax(x, 1)))
    assert len(plan.launches) == 1
    l = plan.launches[0]
    assert l["schedule"].startswith("row(") and "V=4" in l["schedule"] and "reg" in l["schedule"]
    assert l["kernels"] == ["R_4096_1_0", "E_4096_4096_1", "E_4096_4096_2", "R_4096_1_3", "E_4096_4096_4"]
    assert l["algo_bytes"] == 2 * 4096 * 4096 * 4                 # one read + one write
    assert l["grid"][0] * (l["block"][0] // int(re.search(r"T=(\d+)", l["schedule"]).group(1))) >= 4096
    assert sum(b["elided"] for b in plan.buffers) == 4            # max, shifted, exp, sum never reach HBM
    assert "eh_row_reduce<EhMax" in l["source"] and "eh_row_reduce<EhSum" in l["source"]
    assert len(hb.compile_source(l["source"])) > 1000             # hiprtc -> gfx950 code object


def test_config1_fuses_into_one_launch(frontend):
    from harp_amd import backend as hb
    a, b, c = (frontend.Tensor.input([1024, 1024]) for _ in range(3))
    plan = hb.render_program(_program_with_table(frontend, frontend.nn.relu(a * b + c).sum(1)))
    assert len(plan.launches) == 1 and plan.launches[0]["kernels"][-1].startswith("R_1024_1")
    # separate graph nodes keep separate roundings: no fused multiply-add in the text
    assert "fmaf" not in plan.launches[0]["source"]
    assert len(hb.compile_source(plan.launches[0]["source"])) > 1000


def test_config3_matmul_takes_the_mfma_schedule(frontend):
    from harp_amd import backend as hb
    a, b = frontend.Tensor.input([4096, 4096]), frontend.Tensor.input([4096, 4096])
    plan = hb.render_program(_program_with_table(frontend, frontend.nn.matmul(a, b)))
    assert len(plan.launches) == 1
    l = plan.launches[0]
    assert l["schedule"].startswith("mfma32x32x2(") and l["flops"] == 2.0 * 4096 ** 3
    assert "__builtin_amdgcn_mfma_f32_32x32x2f32" in l["source"]
    assert len(hb.compile_source(l["source"])) > 1000
    # option fuse=0 / gemm=0 fall back to other schedules and still compile
    plan2 = hb.render_program(_program_with_table(frontend, frontend.nn.matmul(a, b)), {"gemm": 0})
    assert not plan2.launches[0]["schedule"].startswith("mfma")


def test_unfused_per_kernel_rendering(frontend):
    from harp_amd import backend as hb
    x = frontend.Tensor.input([64, 100])
    prog, _, _ = frontend.lower_graph([frontend.nn.softmax(x, 1).graph])
    assert [k.attrs["name"][0] for k in prog.args] == ["R", "E", "E", "R", "E"]
    for k in prog.args:                                          # what compile_ast receives
        plan = hb.render_program(frontend.AstNode.program([k]))
        assert len(plan.launches) == 1
        assert len(hb.compile_source(plan.launches[0]["source"])) > 500


def test_rendering_of_scatter_and_scan(frontend):
    from harp_amd import backend as hb
    x = frontend.Tensor.input([4, 4])
    y = x.unfold([0, 1], [2, 2], [2, 2], [1, 1]).fold([4, 4], [0, 1], [2, 2], [2, 2], [1, 1])
    prog, _, _ = frontend.lower_graph([y.graph])
    names = [k.attrs["name"] for k in prog.args]
    assert names[0].startswith("C_") and names[1].startswith("S_")
    plan = hb.render_program(prog)
    # zero-fill and scatter-add nests become two launches; tiling windows cannot collide, so
    # both are spread over work-items (16 outputs, 16 window slots)
    assert [l["schedule"] for l in plan.launches[1:]] == ["outer-parallel(work-items=16)"] * 2
    assert "atomicAdd" in plan.launches[2]["source"]
    for l in plan.launches:
        hb.compile_source(l["source"])
    # overlapping windows collide: the AST's atomic adds become device atomics
    z = x.unfold([0, 1], [2, 2], [1, 1], [1, 1]).fold([4, 4], [0, 1], [2, 2], [1, 1], [1, 1])
    plan_z = hb.render_program(frontend.lower_graph([z.graph])[0])
    assert [l["schedule"] for l in plan_z.launches[1:]] == ["outer-parallel(work-items=16)",
                                                           "outer-parallel(work-items=36,atomics)"]
    prog2, _, _ = frontend.lower_graph([x.cumsum(1).graph])
    plan2 = hb.render_program(prog2)
    assert plan2.launches[0]["schedule"] == "outer-parallel(work-items=4)"
    hb.compile_source(plan2.launches[0]["source"])
    # a scan over axis 0 is lowered with one accumulator for the whole tensor: nothing to spread
    plan3 = hb.render_program(frontend.lower_graph([x.cummax(0).graph])[0])
    assert plan3.launches[0]["schedule"] == "as-written"


@pytest.mark.parametrize("text,needle", [
    ("(program", "missing ')'"),
    ("(program (kernel \"k\" (params) (frobnicate)))", "frobnicate"),
    ("(bogus 1 2)", "unknown AST node"),
    ("(program)", "no kernel"),
    ("(add (const f32 1.0))", "takes 2 operands"),
])
def test_malformed_ast_is_reported(text, needle):
    from harp_amd import backend as hb
    with pytest.raises(hb.EhError) as e:
        hb.render_program(text)
    assert needle in str(e.value)


def test_bad_options_and_bad_source_are_reported(frontend):
    from harp_amd import backend as hb
    a = frontend.Tensor.input([8])
    prog, _, _ = frontend.lower_graph([(a + a).graph])
    with pytest.raises(hb.EhError) as e:
        hb.render_program(prog, "no_such_option=1")
    assert "unknown option" in str(e.value)
    with pytest.raises(hb.EhError) as e:
        hb.render_program(prog, "row_threads=100")
    assert "power of two" in str(e.value)
    with pytest.raises(hb.EhError) as e:
        hb.compile_source("this is not HIP")
    assert e.value.code == 4 and "hiprtc" in str(e.value)


@pytest.mark.parametrize("expr,value", [
    ("(const i64 42)", 42),                                             # pipeline.rs:719-723
    ("(mul (const i64 10) (const i64 20))", 200),                       # pipeline.rs:740-752
    ("(add (const i64 10) (const i64 20))", 30),
    ("(idiv (const i64 100) (const i64 10))", 10),
    ("(idiv (add (const i64 1000) (const i64 63)) (const i64 64))", 16),   # ceil_div, parallelization_common.rs:575
    ("(max (const i64 3) (rem (const i64 17) (const i64 5)))", 3),
])
def test_dispatch_size_expressions(expr, value):
    """Grid sizes of kernels the reference has parallelised are expressions; they evaluate as
    the reference's `evaluate_ast_expr` does (src/backend/pipeline.rs:505-553, cases of its
    tests :718-752).  A shape variable is an error here, not a silent 1."""
    from harp_amd import backend as hb
    text = ('(program (kernel "k" (params ("g" i64 imm (group_id 0)) ("o" (ptr f32 global) mut normal)) '
            f'(grid {expr} (const i64 1) (const i64 1)) (tg (const i64 1) (const i64 1) (const i64 1)) '
            '(block (decls) (store (var "o") (var "g") (const f32 1.0)))))')
    l, = hb.render_program(text).launches
    assert l["schedule"] == "as-written" and l["grid"] == [value, 1, 1]
    with pytest.raises(hb.EhError, match="cannot be evaluated"):
        hb.render_program(text.replace(expr, '(var "n")'))


def _fit(global_, preferred, max_wg=1024):
    import ctypes
    from harp_amd._lib import check, lib
    g = (ctypes.c_size_t * 3)(*global_)
    p = (ctypes.c_size_t * 3)(*preferred)
    out = (ctypes.c_size_t * 3)()
    check(lib.eh_fit_local_size(g, p, max_wg, out))
    return list(out)


def test_local_size_is_fitted_as_the_reference_pipeline_does():
    """`compute_compatible_local_size` (src/backend/pipeline.rs:475-489): the largest divisor of
    the global size not above the preferred size; then the workgroup is shrunk, largest
    dimension first, to the next smaller divisor until it fits the device (:176-192)."""
    assert _fit([1000, 1, 1], [48, 1, 1]) == [40, 1, 1]           # 48 does not divide 1000; 40 does
    assert _fit([1000, 1, 1], [1000, 1, 1]) == [1000, 1, 1]
    assert _fit([1000, 1, 1], [2000, 1, 1]) == [1000, 1, 1]       # never above the global size
    assert _fit([997, 1, 1], [256, 1, 1]) == [1, 1, 1]            # a prime has no other divisor
    assert _fit([0, 1, 1], [64, 1, 1]) == [1, 1, 1]               # global 0 -> 1 (:476-478)
    assert _fit([2048, 2048, 1], [64, 64, 1]) == [32, 32, 1]      # 64x64 > 1024: 32x64, then 32x32
    assert _fit([4096, 6, 1], [2048, 3, 1]) == [256, 3, 1]        # only the largest dimension steps down
    assert _fit([96, 96, 96], [16, 16, 16], 256) == [6, 6, 6]     # 16^3 -> 12,16,16 -> ... by turns
    from harp_amd._lib import EhError
    with pytest.raises(EhError):
        _fit([8, 8, 8], [0, 1, 1])


def test_kernels_with_their_own_dispatch_get_the_fitted_local_size():
    """global = grid x thread group; a thread group beyond the device's 1024 work-items is shrunk
    to a divisor of the global size and the workgroup count grows to match."""
    from harp_amd import backend as hb

    def text(grid, tg):
        c = lambda v: f"(const i64 {v})"
        return ('(program (kernel "k" (params ("g" i64 imm (group_id 0)) ("o" (ptr f32 global) mut normal)) '
                f'(grid {c(grid[0])} {c(grid[1])} {c(grid[2])}) (tg {c(tg[0])} {c(tg[1])} {c(tg[2])}) '
                '(block (decls) (store (var "o") (var "g") (const f32 1.0)))))')
    l, = hb.render_program(text([25, 1, 1], [40, 1, 1])).launches
    assert (l["grid"], l["block"]) == ([25, 1, 1], [40, 1, 1])             # fits: launched as given
    l, = hb.render_program(text([4, 4, 1], [64, 64, 1])).launches          # 4096 work-items a group
    assert (l["grid"], l["block"]) == ([8, 8, 1], [32, 32, 1])
    l, = hb.render_program(text([3, 1, 1], [2048, 1, 1])).launches         # global 6144
    assert (l["grid"], l["block"]) == ([6, 1, 1], [1024, 1, 1])


def test_no_device_is_an_error_not_a_fallback():
    from harp_amd import backend as hb
    if hb.device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(hb.EhError) as e:
        hb.HipDevice(0)
    assert "no HIP device" in str(e.value)
    assert not hb.HipBackendRegistry().is_available()


def test_lowering_structure(frontend):
    # src/lowerer/lower.rs:1335-1441: kernel name prefixes, parameter order
    a = frontend.Tensor.input([32, 64])
    b = frontend.Tensor.input([32, 64])
    prog, lw, _ = frontend.lower_graph([(a + b).graph])
    (k,) = prog.args
    assert k.attrs["name"] == "E_32_64_0"
    ps = k.attrs["params"]
    assert [p.mutable for p in ps] == [False, False, True]
    assert [p.name for p in ps] == ["buf0", "buf2", "buf4"]      # counter advances by two
    prog, _, _ = frontend.lower_graph([a.sum(1).graph])
    assert prog.args[0].attrs["name"].startswith("R_32_1_")
    # a view with two consumers is materialised by a copy kernel, a single-consumer view is inlined
    t = a.permute([1, 0])
    prog, _, _ = frontend.lower_graph([(t + t).graph])
    assert [k.attrs["name"][0] for k in prog.args] == ["C", "E"]
    prog, _, _ = frontend.lower_graph([(a.permute([1, 0]) + b.permute([1, 0])).graph])
    assert [k.attrs["name"][0] for k in prog.args] == ["E"]


def test_view_algebra(frontend):
    # spot checks mirroring src/graph/shape/view.rs tests
    V, E = frontend.View, frontend.Expr
    v = V.contiguous([3, 4])
    assert v.strides == [E.const(4), E.const(1)] and v.is_contiguous()
    p = v.permute([1, 0])
    assert p.shape() == [E.const(4), E.const(3)] and p.strides == [E.const(1), E.const(4)]
    assert not p.is_contiguous() and not p.is_innermost_contiguous()
    u = v.unsqueeze(0)
    assert u.shape()[0] == E.const(1) and u.strides[0] == E.const(0)
    assert u.squeeze(0) == v
    ex = u.expand(0, 5)
    assert ex.shape()[0] == E.const(5) and ex.strides[0] == E.const(0)
    pd = V.padded(v, [(1, 1), (1, 1)], "zero")
    assert pd.shape() == [E.const(5), E.const(6)] and pd.has_bounds()
    un = V.contiguous([2, 3, 8, 10]).unfold([2, 3], [3, 3], [1, 1], [1, 1])
    assert [d.evaluate() for d in un.shape()] == [2, 3, 6, 8, 3, 3]
    assert V.contiguous([6, 4]).reshape([2, 12]).is_contiguous()
    with pytest.raises(AssertionError):
        p.reshape([12])


def test_tensor_api_errors(frontend):
    frontend.clear_default_device()
    t = frontend.Tensor.input([4])
    with pytest.raises(frontend.ExecutionError) as e:
        t.set_data([1, 2, 3, 4])
    assert "NoDevice" in str(e.value)
    frontend.set_device_str("c")
    with pytest.raises(frontend.ExecutionError) as e:
        t.set_data([1, 2, 3])
    assert "ShapeMismatch" in str(e.value)
    u = frontend.Tensor.input([4])
    with pytest.raises(frontend.ExecutionError) as e:
        (t + u).realize()
    assert "MissingInput" in str(e.value)
    with pytest.raises(frontend.ExecutionError):
        u.to_vec()
    with pytest.raises(frontend.DeviceError):
        frontend.set_device_str("nosuchbackend")


def test_tensor_constructors_and_small_api(frontend):
    T = frontend.Tensor
    assert T.scalar(3.5).shape() == [] and T.scalar(3.5).graph.name == "scalar"     # value not recorded
    t = T.from_shape_data([2, 3], [0.0] * 6)
    assert t.shape() == [2, 3] and not t.is_realized() and t.try_buffer() is None     # data not attached
    with pytest.raises(ValueError):
        T.from_shape_data([2, 3], [0.0] * 5)
    x = T.input([2, 3, 10])
    assert x.unfold_1d(3, 1, 1).shape() == [2, 3, 8, 3]
    y = T.input([2, 3, 8, 9])
    assert y.unfold_2d((3, 2), (1, 1), (1, 1)).shape() == [2, 3, 6, 8, 3, 2]
    z = T.input([1, 2, 5, 6, 7])
    assert z.unfold_3d((2, 2, 2), (1, 2, 1), (1, 1, 1)).shape() == [1, 2, 4, 3, 6, 2, 2, 2]
    p = T.input([4])
    p.accumulate_grad(T.ones([4]))
    first = p.grad()
    p.accumulate_grad(T.ones([4]))
    assert p.grad() is not first and p.grad().graph.op.kind == "map_reduce" and p.grad().shape() == [4]


def test_kernel_cache_counts(frontend):
    # crates/backend-c/src/lib.rs:246-297: second realize of the same graph hits the cache
    frontend.set_device_str("c")
    frontend.clear_cache()
    import numpy as np
    from conftest import realize_on
    a = np.ones(16, dtype=np.float32)
    realize_on(frontend, "c", lambda x: x + x, [a])
    s1 = frontend.cache_stats()
    realize_on(frontend, "c", lambda x: x + x, [a])
    s2 = frontend.cache_stats()
    assert s1["misses"] == 1 and s1["hits"] == 0
    assert s2["misses"] == 1 and s2["hits"] == 1 and s2["entries"] == 1


def test_config4_training_step_plan(frontend):
    """The MLP step (forward, loss, exact backward, SGD) lowers to one multi-root Program whose
    matmuls all take the MFMA schedule, whose bias gradients take the two-launch column
    reduce, and whose synthesised ones/zeros inputs never become device buffers."""
    from harp_amd import backend as hb, workloads as wl
    batch, dims = 192, (128, 256, 128, 128)       # a batch no weight dimension equals
    shapes = [(batch, dims[0]), (batch, dims[-1])]
    for a, b in zip(dims[:-1], dims[1:]):
        shapes += [(b, a), (b,)]
    ts = [frontend.Tensor.input(list(s)) for s in shapes]
    roots = wl.config4_graph(*ts)
    prog_ast, arg_names, outs, consts, plain = wl.lower_multi(ts, roots)
    assert len(outs) == len(set(outs)) == 7 and len(arg_names) == 8
    plan = hb.render_program(prog_ast)
    assert len(plan.launches) < len(plain.args) // 2
    scheds = [l["schedule"] for l in plan.launches]
    assert sum(s.count("mfma32x32x2(") for s in scheds) == 8         # 3 forward, 3 dW, 2 dX (a layer's dW and dX as one launch)
    assert sum(s.count("-reduce(") for s in scheds) == 3               # bias gradients (column sums) ...
    together = [l for l in plan.launches if l["schedule"].startswith("together(") and "mfma" not in l["schedule"]]
    assert len(together) == 1 and len(together[0]["kernels"]) == 9      # ... and their updates, issued as one launch
    apart = hb.render_program(prog_ast, {"merge_launches": 0})
    assert len(apart.launches) == len(plan.launches) + 4 and not any("together(" in l["schedule"] for l in apart.launches)
    # bias add and activation chains ride on the forward contractions' accumulators
    epi = [l for l in plan.launches if "epilogue=" in l["schedule"]]
    assert len(epi) >= 3 and all("eh_epilogue(" in l["source"] for l in epi)
    assert any(len(l["kernels"]) >= 6 for l in epi)
    # every weight's SGD update (lr * dW, then W - that read through a transposing view) is
    # part of its gradient contraction: no elementwise launch over a weight matrix is left,
    # and the gradient itself never reaches memory
    weight_kernels = {f"E_{b}_{a}" for a, b in zip(dims[:-1], dims[1:])} | {f"E_{a}_{b}" for a, b in zip(dims[:-1], dims[1:])}
    for l in plan.launches:
        if l["schedule"].startswith("flat("):
            assert not any(k.rsplit("_", 1)[0] in weight_kernels for k in l["kernels"]), l["kernels"]
    # the tanh' products of the backward pass (one stage squares a saved activation and reads
    # nothing of the chain) ride on the dX contractions
    assert sum(len(l["kernels"]) >= 8 for l in epi) >= 2
    off = hb.render_program(prog_ast, {"gemm_epilogue": 0})
    assert not any("epilogue=" in l["schedule"] for l in off.launches) and len(off.launches) > len(plan.launches)
    by_name = {b["name"]: b for b in plan.buffers}
    assert by_name[outs[-1]]["bytes"] == 4 and by_name[outs[-1]]["role"] == "output"   # scalar loss
    for name in consts:
        assert by_name[name]["elided"], name
    for src in {l["source"] for l in plan.launches}:
        assert len(hb.compile_source(src)) > 1000


def test_few_very_long_reduce_lines_are_planned_as_two_reduces(frontend):
    """Four lines of ten million elements: the plan cuts every line into pieces that start on
    a 16-byte boundary (one workgroup each), adds the scratch buffer for the pieces and then
    reduces those; without the buffer table (nowhere to put the scratch) or with fusion off
    the kernel stays whole, and lines of ordinary length are never cut."""
    from harp_amd import backend as hb, workloads as wl
    ast = wl.lower_with_table([(4, 10_000_000)], lambda t: t.sum(1))[0]
    plan = hb.render_program(ast)
    assert [l["entry"][-5:] for l in plan.launches][0] == "_rows" and len(plan.launches) == 2
    part, final = plan.launches
    assert part["schedule"].startswith("row(") and part["grid"][0] == 4000 and ",V=4," in part["schedule"]
    scratch = [b for b in plan.buffers if b["name"].startswith("eh_rowpart_")]
    assert len(scratch) == 1 and scratch[0]["bytes"] == 4 * 4000 and scratch[0]["role"] == "temp"
    assert scratch[0]["name"] in part["args"] and scratch[0]["name"] in final["args"]
    for src in (part["source"], final["source"]):
        assert len(hb.compile_source(src)) > 1000
    assert len(hb.render_program(ast, {"fuse": False}).launches) == 1
    t = frontend.Tensor.input([4, 10_000_000])
    bare = frontend.lower_graph([t.sum(1).graph])[0]
    assert len(hb.render_program(bare).launches) == 1
    short = wl.lower_with_table([(4, 1 << 16)], lambda t: t.sum(1))[0]
    assert len(hb.render_program(short).launches) == 1


def test_few_very_long_scan_lines_are_planned_as_totals_then_scan(frontend):
    """A scan over axis 0 is lowered with one accumulator for the whole tensor: one line of a
    million elements.  With a buffer table the plan totals chunks of whole 1024-element tiles
    first and scans every chunk from the totals ahead of it; without one it stays a single
    workgroup per line."""
    from harp_amd import backend as hb, workloads as wl
    ast = wl.lower_with_table([(2048, 512)], lambda t: t.cumsum(0))[0]
    plan = hb.render_program(ast)
    assert [l["schedule"] for l in plan.launches] == ["scan-row-totals(lines=1,chunks=256)",
                                                       "scan-row(lines=1,length=1048576,chunks=256)"]
    tot, scan = plan.launches
    scratch = [b for b in plan.buffers if b["name"].startswith("eh_scanpart_")]
    assert len(scratch) == 1 and scratch[0]["bytes"] == 4 * 256 and scratch[0]["role"] == "temp"
    assert tot["args"][-1] == scan["args"][-1] == scratch[0]["name"] and tot["grid"] == scan["grid"] == [256, 1, 1]
    for l in plan.launches:
        assert len(hb.compile_source(l["source"])) > 1000
    assert [l["schedule"] for l in hb.render_program(ast, {"fuse": False}).launches] == ["scan-row(lines=1,length=1048576)"]
    ragged = hb.render_program(wl.lower_with_table([(3, 700001)], lambda t: t.cummax(1))[0])
    assert [l["schedule"] for l in ragged.launches][-1] == "scan-row(lines=3,length=700001,chunks=171)"
    many = hb.render_program(wl.lower_with_table([(512, 1 << 14)], lambda t: t.cumsum(1))[0])
    assert [l["schedule"] for l in many.launches] == ["scan-row(lines=512,length=16384)"]


def test_pooling_plan_reads_the_source_through_the_gathers(frontend):
    """max-pool as lowered (unfold gather, a second gather through the same view, reduce over the
    window): one launch, both window buffers elided, the gathers as device functions whose
    loop variables the caller passes without divisions where the indices line up.  Switched
    off, or when something else reads the windows too, the gathers stay launches."""
    from harp_amd import backend as hb, workloads as wl
    fn = lambda t: frontend.nn.max_pool2d(t, (2, 2))
    ast = wl.lower_with_table([(2, 3, 8, 8)], fn)[0]
    plan = hb.render_program(ast)
    assert [l["schedule"] for l in plan.launches] == ["window-reduce(window=4,gathers=2)"]
    (l,) = plan.launches
    assert len(l["kernels"]) == 3 and l["args"] == ["buf0", "buf6"]
    assert sorted(b["name"] for b in plan.buffers if b["elided"]) == ["buf2", "buf4"]
    assert "eh_win_buf4(buf0, (ridx0), (ridx1), (ridx2), (ridx3), ((ridx4 / 2)), ((ridx4) % 2))" in l["source"]
    assert "eh_win_buf2(buf0, (ridx0), (ridx1), (ridx2), ((ridx3 / 2) + ridx4 * 2), ((ridx3) % 2), (ridx5))" in l["source"]
    assert len(hb.compile_source(l["source"])) > 1000
    off = hb.render_program(ast, {"window": 0})
    assert len(off.launches) == 3 and not any(b["elided"] for b in off.buffers)
    with frontend.exact_mode():
        shared = wl.lower_with_table([(2, 3, 8, 8)], lambda t: (lambda w: w.max(4).sum(3) + w.sum(4).sum(3))(
            t.unfold([2, 3], [2, 2], [2, 2], [1, 1]).contiguous().reshape([2, 3, 4, 4, 4])))[0]
    assert not any(s["schedule"].startswith("window") for s in hb.render_program(shared).launches)


def test_convolution_plan_folds_both_gathers(frontend):
    """A 3x3 convolution as the reference lowers it (gather, gather through the same view,
    contraction): one MFMA launch whose A loader calls the first gather as a device function;
    both window buffers are elided.  In exact mode (one gather) and for a pointwise
    convolution (window loops that run once) the single gather is folded."""
    from harp_amd import backend as hb, workloads as wl
    conv = lambda x, w: frontend.nn.conv2d(x, w, None, (1, 1), (1, 1))
    shapes = [(2, 4, 10, 10), (8, 4, 3, 3)]
    plan = hb.render_program(wl.lower_with_table(shapes, conv)[0])
    (l,) = plan.launches
    assert l["schedule"].startswith("mfma32x32x2(") and "A:m/folded" in l["schedule"] and len(l["args"]) == 3
    assert sum(b["elided"] for b in plan.buffers) == 2
    assert "__device__ __forceinline__ float eh_win_" in l["source"] and "? eh_win_" in l["source"]
    assert len(hb.compile_source(l["source"])) > 1000
    assert len(hb.render_program(wl.lower_with_table(shapes, conv)[0], {"gemm_fold": 0}).launches) == 3
    with frontend.exact_mode():
        exact = hb.render_program(wl.lower_with_table(shapes, conv)[0])
        point = hb.render_program(wl.lower_with_table([(2, 16, 9, 9), (8, 16, 1, 1)], lambda x, w: frontend.nn.conv2d(x, w))[0])
    for p in (exact, point):
        assert len(p.launches) == 1 and sum(b["elided"] for b in p.buffers) == 1
    # the single padded 3x3 gather is taken apart and staged in LDS (one image's channels with their
    # zero border per workgroup); a 1x1 window has nothing to stage and stays in the tile loader
    assert exact.launches[0]["schedule"].startswith("mfma16x16x4(window,group=100,M=8,K=36,") and exact.launches[0]["grid"] == [2, 1, 1]
    assert "/folded" in point.launches[0]["schedule"]
    with frontend.exact_mode():
        loader = hb.render_program(wl.lower_with_table(shapes, conv)[0], {"gemm_window": 0})
    assert len(loader.launches) == 1 and "/folded" in loader.launches[0]["schedule"]


def test_option_beam_search_on_a_synthetic_cost():
    """The schedule search without a device: suggesters propose neighbours by the schedules in
    the plan, the beam keeps the cheapest states, the search stops when nothing improves."""
    from harp_amd import tune

    class Fake:
        def __init__(self):
            self.calls = 0

        def schedules(self, opts):
            return ["mfma32x32x2(tile=...)", "row(T=64)"]

        def cost(self, opts):
            self.calls += 1
            d = dict(opts)
            c = 10.0
            c -= 3.0 if (d.get("gemm_bm"), d.get("gemm_bn")) == (256, 256) else 0.0
            c -= 1.0 if d.get("gemm_waves") == 4 else 0.0
            c -= 0.5 if d.get("row_threads") == 512 else 0.0
            return c

    est = Fake()
    best, cost, history = tune.beam_search(est, beam_width=2, max_steps=6)
    d = dict(best)
    assert (d["gemm_bm"], d["gemm_bn"]) == (256, 256) and d["gemm_waves"] == 4 and d["row_threads"] == 512
    assert cost == 5.5 and history[0] == (0, "", 10.0)
    assert len({h[1] for h in history}) == len(history)              # no state measured twice
    # flat-only plans get no contraction or row proposals
    assert list(tune.suggest_gemm({}, ["flat(V=4,block=256)"])) == []
    assert all("flat_" in k or k == "nontemporal" for sg in (tune.suggest_flat, tune.suggest_streaming)
               for st in sg({}, ["flat(V=4,block=256)"]) for k in st)
    assert tune.options_string(tune._freeze({"b": 2, "a": 1})) == "a=1,b=2"


def test_dump_directory_receives_every_launch(frontend, tmp_path, monkeypatch):
    """ECLAT_HIP_DUMP=<dir>: the generated HIP source and the dispatch of every launch."""
    from harp_amd import backend as hb
    from harp_amd import workloads as wl
    monkeypatch.setenv("ECLAT_HIP_DUMP", str(tmp_path / "dump"))
    plan = hb.render_program(wl.lower_with_table([(64, 256)], wl.config2_graph)[0])
    for l in plan.launches:
        src = (tmp_path / "dump" / (l["entry"] + ".hip")).read_text()
        assert src == l["source"] and "__global__" in src
        info = (tmp_path / "dump" / (l["entry"] + ".txt")).read_text()
        assert "schedule: " + l["schedule"] in info and "grid: %d %d %d" % tuple(l["grid"]) in info


def test_contraction_with_more_batches_than_grid_z_allows_is_not_put_on_mfma(frontend):
    """The batch axis of a contraction rides on blockIdx.z, which holds at most 65535 workgroups: a
    per-group contraction over 70000 groups is planned with another reduce schedule instead of a
    launch the runtime would refuse."""
    from harp_amd import backend as hb
    from harp_amd import workloads as wl
    fn = lambda g, c: (g.unsqueeze(3) * c.unsqueeze(2)).sum(1)          # [G,R,O],[G,R,K] -> [G,O,K]
    small = hb.render_program(wl.lower_with_table([(6, 16, 8), (6, 16, 8)], fn)[0]).launches
    assert any(l["schedule"].startswith("mfma32x32x2(") for l in small)
    big = hb.render_program(wl.lower_with_table([(70000, 16, 8), (70000, 16, 8)], fn)[0]).launches
    assert not any(l["schedule"].startswith("mfma") for l in big), [l["schedule"] for l in big]
    for l in big:
        assert l["grid"][2] <= 65535 and l["grid"][1] <= 65535 and l["grid"][0] < 2 ** 31, l["grid"]


def _lane_plan_is_sound(launches):
    """Issue order is a valid sequential order, and every dependence between launches on different
    lanes is covered by a wait (directly, or by a later launch of the producer's lane that the
    consumer's lane has waited for: lanes run in order)."""
    lanes = max(l["lane"] for l in launches) + 1
    waited = [[-1] * lanes for _ in range(lanes)]          # [consumer lane][producer lane] -> launch
    for j, lj in enumerate(launches):
        for w in lj["waits"]:
            assert w < j and launches[w]["lane"] != lj["lane"]
            waited[lj["lane"]][launches[w]["lane"]] = max(waited[lj["lane"]][launches[w]["lane"]], w)
        for i in range(j):
            li = launches[i]
            hazard = any(a == b and (wa or wb) for a, wa in zip(li["args"], li["written"])
                         for b, wb in zip(lj["args"], lj["written"]))
            if hazard and li["lane"] != lj["lane"]:
                assert waited[lj["lane"]][li["lane"]] >= i, (i, li["entry"], j, lj["entry"])
    return lanes


def test_training_step_launches_are_spread_over_lanes_soundly(frontend):
    """The CNN training step: independent launches (the gradients of the parameters beside the
    chain that carries the gradient back) go to a side lane.  Producers come before consumers in
    the issue order, every buffer has its writer marked, and every cross-lane dependence is
    covered by a wait; with lanes=1 (the default) the plan is the same set of launches on lane 0."""
    from harp_amd import backend as hb
    from harp_amd import workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(8, *wl.cnn_sizes(False)[1:])
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    prog_ast, arg_names, outs, consts, _ = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))
    plan = hb.render_program(prog_ast, "lanes=3,lane_us=0,merge_launches=0")
    assert _lane_plan_is_sound(plan.launches) == 3
    assert sum(l["lane"] > 0 for l in plan.launches) >= 8
    roles = {b["name"]: b["role"] for b in plan.buffers}
    written = {a for l in plan.launches for a, w in zip(l["args"], l["written"]) if w}
    read_first = set()
    seen = set()
    for l in plan.launches:
        for a, w in zip(l["args"], l["written"]):
            if not w and a not in seen and roles.get(a) != "input" and roles.get(a) not in ("ones", "zeros"):
                read_first.add(a)
        seen.update(a for a, w in zip(l["args"], l["written"]) if w)
    assert not read_first, read_first                      # nothing but inputs is read before it is written
    assert {n for n, r in roles.items() if r == "output"} <= written
    one = hb.render_program(prog_ast, "lanes=1,merge_launches=0")
    assert all(l["lane"] == 0 and not l["waits"] for l in one.launches)
    assert sorted(l["entry"] for l in one.launches) == sorted(l["entry"] for l in plan.launches)
    two = hb.render_program(prog_ast, "lanes=2,merge_launches=0")
    assert _lane_plan_is_sound(two.launches) == 2
    default = hb.render_program(prog_ast, "merge_launches=0")   # one lane unless asked (or tuned) otherwise
    assert [l["entry"] for l in default.launches] == [l["entry"] for l in one.launches]
    merged = hb.render_program(prog_ast, "lanes=2")        # with the updates issued together: still sound
    assert _lane_plan_is_sound(merged.launches) in (1, 2) and len(merged.launches) < len(two.launches)
    # a single softmax has nothing to spread
    from harp_amd import workloads
    sm = hb.render_program(workloads.lower_with_table([(64, 256)], workloads.config2_graph)[0])
    assert all(l["lane"] == 0 for l in sm.launches)


def _regrouped_chain(x, y):
    """[8,6,4] squared, permuted and made contiguous, its axes regrouped to [4,4,12], then used twice."""
    a = (x * x).permute([2, 0, 1]).contiguous().reshape([4, 4, 12])
    return a * y.unsqueeze(0) + a


def test_elementwise_producers_are_evaluated_where_another_index_space_reads_them(frontend):
    """A square, a permuting copy and a regrouping copy in front of the kernel that uses them: as
    lowered that is three launches through three temps; planned, the consumer's loops are split at
    the producers' loop boundaries, the producers' expressions take the place of the loads, and one
    launch reads x directly.  reindex=0 keeps the kernels apart."""
    from harp_amd import backend as hb, workloads as wl
    ast = wl.lower_with_table([(8, 6, 4), (4, 12)], _regrouped_chain)[0]
    plan = hb.render_program(ast)
    (l,) = plan.launches
    roles = {b["name"]: b["role"] for b in plan.buffers}
    assert l["schedule"].startswith("flat(")
    assert sorted(roles[a] for a in l["args"]) == ["input", "input", "output"], l["args"]
    assert sum(b["elided"] for b in plan.buffers) == 4
    src = l["source"]
    apart = hb.render_program(ast, "reindex=0")
    assert len(apart.launches) == 3 and sum(b["elided"] for b in apart.buffers) == 2
    assert len(hb.compile_source(src)) > 1000


def test_convolution_input_gradient_temp_is_stored_for_its_reader(frontend):
    """The input gradient of a 3x3 convolution: `dY x W` writes columns [pixels, channels*9] that
    nine shifted, guarded reads sum up along the image's rows.  Stored as written, neighbouring
    lanes of that sum read 288 floats apart; the plan stores the temp transposed (the contraction
    computes the transposed product), and the guarded reads carry no branch."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(64, *wl.cnn_sizes(True)[1:])
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]
    plan = hb.render_program(ast, "lanes=1,gemm_window=0,merge_templates=0")
    # (transposed product: W as rows; dY, a copy through a view, read from its source with strides)
    cols = [l for l in plan.launches if l["schedule"].startswith("mfma") and "A:m,B:n,B:source" in l["schedule"]]
    assert len(cols) == 1, [l["schedule"] for l in plan.launches]
    temp = cols[0]["args"][-1]
    (reader,) = [l for l in plan.launches if temp in l["args"] and l is not cols[0]]
    # (the reader may have gone out together with an independent launch: its part of the source then)
    src = reader["source"]
    body = src[src.rindex("\n", 0, src.index("eh_rs_" + temp)):]
    body = body[:body.index("}  // namespace")] if "}  // namespace" in body else body
    assert body.count("eh_ranged_load(eh_rs_" + temp + ",") == 9   # guarded loads: out of range where the guard fails
    assert "if (" not in body.replace("if (eh_", "") and temp + "[" not in body
    clamped = hb.render_program(ast, "lanes=1,ranged_loads=0,gemm_window=0,merge_templates=0")
    (reader0,) = [l for l in clamped.launches if temp in l["args"] and not l["schedule"].startswith("mfma")]
    assert reader0["source"].count(temp + "[") == 9             # ... or a clamped index and a select
    plain = hb.render_program(ast, "lanes=1,reindex=0")
    assert not any("A:m,B:n,B:source" in l["schedule"] for l in plain.launches)
    # the weight gradients' dY operand is a copy through a view (NCHW read as [image, pixel, channel]):
    # read from its source with strides, not through an element function
    direct = [l for l in plan.launches if "A:source" in l["schedule"]]
    assert len(direct) == 2 and all("A:k,B:n/folded" in l["schedule"] for l in direct), [l["schedule"] for l in plan.launches]


def test_only_guarded_reads_go_through_a_buffer_resource(frontend):
    """A padded operand (guarded reads) beside an operand read as it is: the guarded reads are
    buffer-resource loads that come back zero beyond the buffer, the unguarded ones keep their
    pointer -- also reads of the padded buffer itself that sit under no guard -- so an index that
    runs out of its buffer is not turned into a quiet zero."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor

    def graph(x, w):
        return [(x.pad([(1, 1), (2, 2)]).contiguous() * w).contiguous(), (x * x).contiguous()]

    ts = [Tensor.input([30, 60]), Tensor.input([32, 64])]
    ast = wl.lower_multi(ts, graph(*ts))[0]
    plan = hb.render_program(ast, "merge_launches=0")
    names = wl.lower_multi(ts, graph(*ts))[1]
    x_buf, w_buf = names[0], names[1]
    padded = [l for l in plan.launches if "eh_ranged_load(" in l["source"]]
    assert len(padded) == 1
    src = padded[0]["source"]
    body = src[src.index("__global__"):]
    assert body.count("eh_ranged_load(eh_rs_" + x_buf + ",") >= 1 and "eh_rs_" + w_buf not in src
    assert w_buf + " + " in body or w_buf + "[" in body                     # w through its pointer
    squares = [l for l in plan.launches if l is not padded[0]]
    assert squares and all("eh_ranged_load" not in l["source"] for l in squares)
    assert all(len(hb.compile_source(l["source"])) > 1000 for l in plan.launches)


def test_convolution_windows_are_staged_in_lds(frontend):
    """The padded 3x3 gathers of the CNN step's convolutions are taken apart (row digit + window
    digit = source coordinate, guards = where that coordinate leaves the image) and what one
    image's rows read is staged in LDS once per workgroup: the forward contractions of both
    convolutions (rows = the image's pixels, the four k of a step along the channels, or along
    the taps where there is one channel) and the second convolution's weight gradient (rows =
    channel x tap, k = the image's pixels, two offset patterns where a step of four pixels runs
    over the end of a row of fourteen).  The multiply loop holds no vector instruction but the
    MFMAs.  A's rows are staged too, so the first convolution's weight gradient (K = 784 pixels, 196 steps)
    fits as well."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(*wl.cnn_sizes(True))
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]
    plan = hb.render_program(ast, "merge_templates=0,gemm_tail=0")   # (every contraction a launch of its own, and every pooling)
    win = {l["entry"]: l for l in plan.launches if l["schedule"].startswith("mfma16x16x4(window,")}
    assert sorted(win) == ["ehk_R_256_196_1_288_59", "ehk_R_256_196_64_1_9", "ehk_R_256_1_32_9_79", "ehk_R_256_1_64_288_88",
                           "ehk_R_256_784_32_1_1"]
    fwd2, wg2, fwd1 = win["ehk_R_256_196_64_1_9"], win["ehk_R_256_1_64_288_88"], win["ehk_R_256_784_32_1_1"]
    assert fwd2["schedule"].startswith("mfma16x16x4(window,group=196,M=64,K=288,waves=4x1,blocks=1x13,steps=72,patterns=1,")
    assert fwd2["grid"] == [256, 1, 1] and fwd2["block"] == [256, 1, 1] and "epilogue=1" in fwd2["schedule"]   # (bias; the relu is the pooling's to apply)
    assert wg2["schedule"].startswith("mfma16x16x4(window,group=288,M=64,K=196,waves=4x1,blocks=1x18,steps=49,patterns=2,")
    assert wg2["grid"] == [1, 1, 256]
    assert fwd1["schedule"].startswith("mfma16x16x4(window,group=784,M=32,K=9,waves=2x2,blocks=1x25,steps=3,patterns=3,")
    for l in win.values():
        assert len(hb.compile_source(l["source"])) > 1000
    # one image: 32 channels of 16 x 16 (14 x 14 and its border), the channel stride padded off the banks
    import re
    m = re.search(r"axes \[32 x stride 196, valid 0\.\.32, lds (\d+)\] \[16 x stride 14, valid 1\.\.15, lds 16\] "
                  r"\[16 x stride 1, valid 1\.\.15, lds 1\]", fwd2["source"])
    assert m and 256 < int(m.group(1)) < 320
    # (the four pixels of a step: consecutive, or two at the end of a row and two at the start of the next, a padded row stride apart)
    assert "if (p == 0) return 0 + b0 * 1 + b1 * 2 + (b0 & b1) * 0;" in wg2["source"]
    assert re.search(r"if \(p == 1\) return 0 \+ b0 \* 1 \+ b1 \* (\d+) \+ \(b0 & b1\) \* 0;", wg2["source"])
    wg1 = win["ehk_R_256_1_32_9_79"]
    assert wg1["schedule"].startswith("mfma16x16x4(window,group=9,M=32,K=784,waves=2x1,blocks=1x1,steps=196,patterns=1,")
    assert wg1["grid"] == [1, 1, 256] and wg1["block"] == [256, 1, 1]      # two waves multiply, all four fetch
    assert not any("/folded" in l["schedule"] for l in plan.launches)
    # the same buffers elided either way (the tile loader splits K for the first convolution's weight
    # gradient and needs a scratch buffer and a summing launch for it; the staged form does not)
    loader = hb.render_program(ast, "gemm_window=0,merge_templates=0")
    assert not any("(window," in l["schedule"] for l in loader.launches) and len(loader.launches) >= len(plan.launches)
    gone = lambda p: {b["name"] for b in p.buffers if b["elided"]}          # noqa: E731
    # (with K split, the per-image results of that weight gradient are summed from the partial tiles and never exist)
    # (and the columns of the second convolution's input gradient exist only in the tile-loader plan)
    assert len(gone(loader) - gone(plan)) <= 1 and len(gone(plan) - gone(loader)) == 1


def test_convolution_input_gradient_is_one_window_contraction(frontend):
    """The input gradient of the second convolution as the reference lowers it: dY x W into
    columns [pixel, channel x tap], then eight kernels that add up nine shifted, guarded reads of
    the columns into the padded image.  The nine reads join the contraction's sum (K = 64
    channels x 3 x 3 shifts, the shifts walking dY against the pixel), dY is read at its NCHW
    source rather than through the permuting copy folded into the product, and the one-pixel
    border that the next kernel slices away is not computed: one launch for nine kernels, and
    neither the columns (58 MB) nor the partial sums reach memory."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    import re
    arrays = wl.config5_inputs(*wl.cnn_sizes(True))
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]
    plan = hb.render_program(ast, "merge_templates=0,gemm_tail=0")   # (every contraction a launch of its own, and every pooling)
    (dx,) = [l for l in plan.launches if "shifts=" in l["schedule"]]
    assert dx["schedule"].startswith("mfma16x16x4(window,group=196,M=32,K=576,waves=2x2,blocks=1x7,steps=144,patterns=1,")
    assert dx["schedule"].endswith(",shifts=9)") and dx["grid"] == [256, 1, 1]
    assert dx["kernels"] == ["R_256_196_1_288_59"] + ["E_256_32_16_16_%d" % q for q in range(60, 68)]
    assert len(dx["args"]) == 3 and dx["written"] == [False, False, True]
    # dY's channels, and its 14 x 14 pixels inside a border of one: source coordinate = pixel - shift
    assert re.search(r"axes \[64 x stride 196, valid 0\.\.64, lds \d+\] \[16 x stride 14, valid 1\.\.15, lds 16\] "
                     r"\[16 x stride 1, valid 1\.\.15, lds 1\]", dx["source"])
    # the result's interior only (offset 17 = one row and one column into the 16 x 16 image)
    assert "return 17LL + 0LL;" in dx["source"] and "(u / 14u) % 14u) * 16LL" in dx["source"]
    out = dx["args"][2]
    assert dx["overwrites"] == [False, False, False]           # ... so the output is not overwritten as a whole
    gone = {b["name"] for b in plan.buffers if b["elided"]}
    assert len(gone & {"buf%d" % q for q in range(145, 161, 2)}) == 8 and out not in gone
    assert len(hb.compile_source(dx["source"])) > 1000
    # without the LDS-staged schedules the product and the shifted sums are two launches
    off = hb.render_program(ast, "gemm_window=0,merge_templates=0")
    assert not any("shifts=" in l["schedule"] for l in off.launches) and len(off.launches) == len(plan.launches) + 1


def test_loss_bookkeeping_joins_the_launch_it_continues(frontend):
    """The roots of a training step are lowered one after another, so what is left of the loss's
    value (a few kernels on [batch] and [batch, classes]) comes behind a hundred kernels of the
    gradients.  Those kernels carry on with the rows of the log-softmax launch and nothing in
    between touches their buffers: they join that launch (their own launch goes), and the last
    of them, the sum over the batch, depends on nothing later and is issued with the other final
    launches."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(*wl.cnn_sizes(True))
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]
    plan = hb.render_program(ast)
    (rows,) = [l for l in plan.launches if l["entry"] == "ehk_R_256_1_28"]
    assert {"E_256_109", "E_256_10_110", "R_256_1_111"} <= set(rows["kernels"]), rows["kernels"]
    assert rows["kernels"].index("E_256_109") > rows["kernels"].index("E_256_10_43")
    assert sum("R_256_1_111" in l["kernels"] for l in plan.launches) == 1
    (total,) = [l for l in plan.launches if "R_1_112" in l["kernels"]]
    assert total["schedule"].startswith("together(") and plan.launches.index(total) > plan.launches.index(rows)
    assert len(plan.launches) == 14
    apart = hb.render_program(ast, "merge_launches=0")
    assert not any("E_256_109" in l["kernels"] and "R_256_1_28" in l["kernels"] for l in apart.launches)


def test_convolution_rows_run_across_images(frontend):
    """196 pixels an image are no multiple of a 64-wide tile: the second convolution's forward
    contraction takes (image, pixel) as one axis (784 tiles for 256 images, none padded per
    image, where one image at a time would need 1024) and only the result's NCHW address keeps
    the two extents.  The first convolution's weight gradient, 32 channels by 9 taps per image,
    takes the one-wave tile."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config5_inputs(*wl.cnn_sizes(True))
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config5_graph(*ts, lr=1e-2))[0]
    plan = hb.render_program(ast, "lanes=1,gemm_window=0")           # the tile-loader schedule
    (fwd,) = [l for l in plan.launches if l["entry"] == "ehk_R_256_196_64_1_9"]
    assert "C:split" in fwd["schedule"] and "edges" not in fwd["schedule"], fwd["schedule"]
    assert fwd["grid"] == [256 * 196 // 64, 1, 1]
    assert "#define EH_C_NSPLIT 196LL" in fwd["source"] and "#define EH_C_SN2 12544LL" in fwd["source"]
    small = [l for l in plan.launches if "tile=32x32x16" in l["schedule"]]
    assert [l["entry"] for l in small] == ["ehk_R_256_1_32_9_79_part"], [l["schedule"] for l in plan.launches]
    # the kernel that prepares the second fully connected layer's operand is lowered behind two
    # small kernels of the loss (another root); it moves up behind its producer and rides on the
    # first layer's contraction like the rest of that chain
    fc1 = [l for l in plan.launches if "R_256_1_128_16" in l["kernels"] and "E_256_128_23" in l["kernels"]]
    assert len(fc1) == 1 and "epilogue=4" in fc1[0]["schedule"], [l["kernels"] for l in plan.launches]


def _bias_gradient_step(x, b, lr):
    """A bias's gradient as the reference lowers it (sums over columns, rows, then the batch) and its update."""
    return b - x.sum(3).sum(2).sum(0) * lr


def test_bias_gradient_chain_is_two_launches(frontend):
    """Sums over an image's columns and then its rows are one sum along memory (the second
    kernel is taken into the first), and the update rides in the launch that finishes the sum
    over the batch: four launches become two.  A total over everything is not merged into one
    long line, and reindex=0 / gemm_epilogue=0 plan the kernels as lowered."""
    from harp_amd import backend as hb, workloads as wl
    shapes = [(64, 32, 14, 14), (32,), (32,)]
    ast = wl.lower_with_table(shapes, _bias_gradient_step)[0]
    plan = hb.render_program(ast)
    assert [l["kernels"] for l in plan.launches] == [["R_64_32_14_1_0", "R_64_32_1_1"], ["R_1_32_2", "E_32_3", "E_32_4"]]
    assert plan.launches[0]["schedule"].startswith("row(T=32,V=4") and "epilogue=2" in plan.launches[1]["schedule"]
    assert "eh_epilogue(" in plan.launches[1]["source"]
    elided = {b["name"] for b in plan.buffers if b["elided"]}
    assert len(elided) == 3                                # the two partial sums' buffers and the gradient itself
    plain = hb.render_program(ast, "reindex=0,gemm_epilogue=0")
    assert len(plain.launches) == 4
    total = hb.render_program(wl.lower_with_table([(8192, 1024)], lambda t: t.sum(1).sum(0))[0])
    assert [l["kernels"] for l in total.launches] == [["R_8192_1_0"], ["R_1_1"]]


def test_backward_pass_recomputes_cheap_saved_values(frontend):
    """The MLP training step: the exact tanh saves exp(-2x), 1 + exp(-2x) and the activation for the
    backward pass.  The second is one addition away from the first, which stays in memory
    anyway: its backward reader evaluates it again instead of loading it, and the forward
    contraction's epilogue no longer stores it (one tensor less per tanh layer);
    rematerialize=0 keeps every saved value."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    arrays = wl.config4_inputs(512, [64, 256, 256, 64])       # (activations beyond what counts as a small kernel)
    ts = [Tensor.input(list(a.shape)) for a in arrays]
    ast = wl.lower_multi(ts, wl.config4_graph(*ts, lr=1e-3))[0]
    stored = lambda plan: sorted(b["name"] for b in plan.buffers if b["role"] == "temp" and not b["elided"])
    with_remat, without = hb.render_program(ast), hb.render_program(ast, "rematerialize=0")
    assert len(with_remat.launches) == len(without.launches)
    gone = set(stored(without)) - set(stored(with_remat))
    assert len(gone) == 2 and set(stored(with_remat)) <= set(stored(without)), gone
    fwd = [l for l in with_remat.launches if "epilogue=8" in l["schedule"]]
    fwd0 = [l for l in without.launches if "epilogue=8" in l["schedule"]]
    assert len(fwd) == len(fwd0) == 2 and all(len(a["args"]) + 1 == len(b["args"]) for a, b in zip(fwd, fwd0))


def _value_and_its_row_sums(x, m):
    """x*m + x as one root and the row sums of the same expression, written out again, as another."""
    return [x * m + x, (x * m + x).sum(1)]


def test_a_stored_value_is_read_back_instead_of_computed_again(frontend):
    """Two roots: an elementwise result and a reduction over the same expression built a second
    time (as a training step's bias gradient repeats the masked gradient its weight gradient
    reads).  The second product is not lowered into a kernel of its own: the reduction takes what
    the first root's kernels hold.  reindex=0 plans all four lowered kernels."""
    from harp_amd import backend as hb, workloads as wl
    from harp_amd.frontend import Tensor
    ts = [Tensor.input([64, 256]), Tensor.input([64, 256])]
    ast = wl.lower_multi(ts, _value_and_its_row_sums(*ts))[0]
    kernels = lambda plan: [k for l in plan.launches for k in l["kernels"]]
    assert len(kernels(hb.render_program(ast, "reindex=0"))) == 4
    plan = hb.render_program(ast)
    assert len(kernels(plan)) == 3 and len(plan.launches) == 1
    assert len(hb.compile_source(plan.launches[0]["source"])) > 1000


def test_tuned_options_are_filed_and_applied(frontend, tmp_path, monkeypatch):
    """What the measured search found is kept: a line "<key> <options>" in the file that
    ECLAT_HIP_TUNE names makes every later compile of that program take those options; explicit
    options still win, other programs and a missing file change nothing."""
    from harp_amd import backend as hb, tune, workloads as wl
    softmax = wl.lower_with_table([(64, 2048)], wl.config2_graph)[0]
    other = wl.lower_with_table([(32, 2048)], wl.config2_graph)[0]
    key = hb.tune_key(softmax)
    assert len(key) == 16 and key != hb.tune_key(other) and key == hb.tune_key(softmax)
    sched = lambda ast, o=None: hb.render_program(ast, o).launches[0]["schedule"]
    default = sched(softmax)
    assert "row(T=256," in default
    path = tmp_path / "tuned.txt"
    monkeypatch.setenv("ECLAT_HIP_TUNE", str(path))
    assert sched(softmax) == default                                   # no file yet
    tune.save_tuned(str(path), key, "row_threads=64", "an older result")
    tune.save_tuned(str(path), key, "row_threads=512,nontemporal=1", "softmax 64x2048")
    path.write_text("# tuned on MI355X\n" + path.read_text())
    assert "row(T=512," in sched(softmax) and "nt-store" in sched(softmax)
    assert "row(T=128," in sched(softmax, "row_threads=128") and "nt-store" in sched(softmax, "row_threads=128")
    assert "row(T=256," in sched(other)
    monkeypatch.delenv("ECLAT_HIP_TUNE")
    assert sched(softmax) == default
    assert {"gemm_prefetch", "gemm_dma", "lanes"} <= {k for st in tune.suggest_pipeline({}, ["mfma32x32x2(...)"] * 8) for k in st}
    # the key is of the canonical text: spacing does not matter
    assert hb.tune_key(softmax.to_sexpr().replace(" (", "  (")) == key


def test_options_filed_for_one_launch(frontend, tmp_path, monkeypatch):
    """Options can be filed for a single launch: under the key the plan reports for it (the hash
    of the canonical text of the first lowered kernel the launch covers), in the tuned-options
    file beside program keys or as "@<key>:name=value" in an options string.  They apply to that
    launch alone, in whatever program the kernel turns up, on top of the program's options."""
    import subprocess, sys, os
    from harp_amd import backend as hb, tune, workloads as wl

    def two(x, w):
        return [x.softmax(1) if hasattr(x, "softmax") else frontend.nn.softmax(x, 1), frontend.nn.softmax(w, 1)]

    from harp_amd.frontend import Tensor
    ts = [Tensor.input([64, 2048]), Tensor.input([32, 1024])]
    ast = wl.lower_multi(ts, two(*ts))[0]
    plan = hb.render_program(ast, "merge_launches=0")
    rows = [l for l in plan.launches if l["schedule"].startswith("row(")]
    assert len(rows) == 2 and rows[0]["tune_key"] != rows[1]["tune_key"] and all(len(l["tune_key"]) == 16 for l in rows)
    k0 = rows[0]["tune_key"]
    tuned = hb.render_program(ast, f"merge_launches=0,@{k0}:row_threads=64")
    by_key = {l["tune_key"]: l["schedule"] for l in tuned.launches if l["schedule"].startswith("row(")}
    assert "row(T=64," in by_key[k0] and by_key[rows[1]["tune_key"]] == rows[1]["schedule"]
    # the same kernel in another program has the same key
    alone = wl.lower_multi(ts[:1], [frontend.nn.softmax(ts[0], 1)])[0]
    assert k0 in [l["tune_key"] for l in hb.render_program(alone).launches]
    with pytest.raises(hb.EhError):
        hb.render_program(ast, f"@{k0}:no_such_option=1")
    with pytest.raises(hb.EhError):
        hb.render_program(ast, "@123:row_threads=64")
    # in the file: a program's line and a launch's line side by side
    path = tmp_path / "tuned.txt"
    tune.save_tuned(str(path), hb.tune_key(ast), "merge_launches=0", "the program")
    tune.save_tuned(str(path), k0, "row_threads=128", "one launch")
    monkeypatch.setenv("ECLAT_HIP_TUNE", str(path))
    filed = hb.render_program(ast)
    assert len(filed.launches) == len(plan.launches)
    assert ["row(T=128," in l["schedule"] for l in filed.launches if l["tune_key"] == k0] == [True]
    assert "row(T=128," in [l for l in hb.render_program(alone).launches if l["tune_key"] == k0][0]["schedule"]
    # a file that cannot be read is reported once and ignored
    env = dict(os.environ, ECLAT_HIP_TUNE=str(tmp_path / "missing" / "tuned.txt"), PYTHONPATH=os.path.dirname(os.path.dirname(__file__)))
    code = ("from harp_amd import backend as hb, workloads as wl\n"
            "ast = wl.lower_with_table([(64, 2048)], wl.config2_graph)[0]\n"
            "print(hb.render_program(ast).launches[0]['schedule']); print(hb.render_program(ast).launches[0]['schedule'])\n")
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.count("row(T=256,") == 2
    assert out.stderr.count("cannot read the tuned-options file") == 1
