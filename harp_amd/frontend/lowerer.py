"""Graph -> kernel AST lowering: one GraphNode becomes one Kernel.

Host-side mirror of the reference's `src/lowerer/`:
`lower.rs` (`Lowerer::lower` `:303-330`, `lower_node` `:335-388`, view
inlining `:150-224`, buffer/kernel naming `:227-279`, `lower_view` `:448`,
`lower_elementwise` `:504`, `lower_reduce` `:525`, `lower_scatter` `:580`,
`lower_scan` `:691`, `lower_matmul` `:745`, `make_kernel` `:1047-1105`,
`substitute_wildcards` `:1127-1163`), `loop_gen.rs` (`generate_loops` `:51`,
`generate_loops_with_reduce` `:87`, `generate_scan` `:237`), `index_gen.rs`
(`view_to_expr` `:45`, `view_to_reduce_output_index` `:107`) and `fusion.rs`
(`ViewFusion` `:28-56`, `ElementwiseReduceFusion` `:83-128`, `AllFusions`
`:147-155`).
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

from .ast import AstNode, DType, F32, I64, VarDecl, expr_to_ast
from .expr import Expr
from .graph import (GraphNode, GraphOp, apply_transform, collect_inputs,
                    reduce_combine, reduce_identity, topological_sort)
from .view import PAD_VALUES, View


# --------------------------------------------------------------------------
# fusion passes
# --------------------------------------------------------------------------

def _view_fusion(node: GraphNode) -> Optional[GraphNode]:
    if node.op.kind != "view" or len(node.src) != 1:
        return None
    inner = node.src[0]
    if inner.op.kind != "view" or len(inner.src) != 1:
        return None
    composed = View.compose(node.op.view, inner.op.view)
    return GraphNode(inner.src, node.view, GraphOp("view", view=composed), node.dtype)


def _elementwise_reduce_fusion(node: GraphNode) -> Optional[GraphNode]:
    op = node.op
    if op.kind != "map_reduce" or op.reduce is None:
        return None
    m = op.map
    if not (m.op == "wildcard" and m.attrs["name"] == "0"):
        return None
    if len(node.src) != 1:
        return None
    s = node.src[0]
    if s.op.kind == "map_reduce" and s.op.reduce is None:
        # the producer's consumer count is not checked (fusion.rs:83-128)
        return GraphNode(s.src, node.view,
                         GraphOp("map_reduce", map=s.op.map, reduce=op.reduce), node.dtype)
    return None


def fuse_views(roots, share=False): return apply_transform(_view_fusion, roots, share)


def fuse_elementwise_reduce(roots, share=False):
    return apply_transform(_elementwise_reduce_fusion, roots, share)


def all_fusions(roots: Sequence[GraphNode], share: bool = False) -> List[GraphNode]:
    return fuse_elementwise_reduce(fuse_views(roots, share), share)


# --------------------------------------------------------------------------
# index / loop generation
# --------------------------------------------------------------------------

def view_to_expr(view: View) -> Expr:
    if view.kind == "linear":
        e = view.offset
        for i, s in enumerate(view.strides):
            e = e + Expr.idx(i) * s
        return e
    return view.index_expr


def view_to_index(view: View) -> AstNode:
    return expr_to_ast(view_to_expr(view))


def view_to_reduce_output_index(view: View, axis: int) -> AstNode:
    return expr_to_ast(view_to_expr(view).substitute_idx(axis, Expr.const(0)).simplify())


def _range(var: str, stop: Expr, body: AstNode) -> AstNode:
    return AstNode.range(var, AstNode.const_i64(0), AstNode.const_i64(1),
                         expr_to_ast(stop), body)


def generate_loops(shape: Sequence[Expr], inner: AstNode) -> AstNode:
    res = inner
    for i in range(len(shape) - 1, -1, -1):
        res = _range(f"ridx{i}", shape[i], res)
    return res


def generate_reduce(shape, axis, out_ptr, out_idx, acc, acc_dtype, identity, combine):
    pre = AstNode.assign(acc, identity)
    body = AstNode.assign(acc, combine)
    post = AstNode.store(out_ptr, out_idx, AstNode.var(acc))
    red = _range(f"ridx{axis}", shape[axis], body)
    res = AstNode.block([pre, red, post], decls=[(acc, acc_dtype)])
    # loops after the reduce axis wrap the block first, then the ones before it
    for i in range(len(shape) - 1, axis, -1):
        res = _range(f"ridx{i}", shape[i], res)
    for i in range(axis - 1, -1, -1):
        res = _range(f"ridx{i}", shape[i], res)
    return res


def generate_scan(shape, axis, out_ptr, out_idx, acc, acc_dtype, identity, combine):
    body = AstNode.block([AstNode.assign(acc, combine),
                          AstNode.store(out_ptr, out_idx, AstNode.var(acc))])
    inner = body
    for i in range(len(shape) - 1, axis, -1):
        inner = _range(f"ridx{i}", shape[i], inner)
    scan_loop = _range(f"ridx{axis}", shape[axis], inner)
    res = AstNode.block([AstNode.assign(acc, identity), scan_loop], decls=[(acc, acc_dtype)])
    for i in range(axis - 1, -1, -1):
        res = _range(f"ridx{i}", shape[i], res)
    return res


# --------------------------------------------------------------------------
# Lowerer
# --------------------------------------------------------------------------

class LoweringError(Exception):
    pass


class Lowerer:
    def __init__(self):
        self.buffer_counter = 0
        self.kernel_counter = 0
        self.buffer_map: Dict[int, str] = {}
        self.dtype_map: Dict[int, DType] = {}
        self.shape_map: Dict[int, List[Expr]] = {}
        self._nodes: Dict[int, GraphNode] = {}     # keeps ids alive
        self.kernels: List[AstNode] = []
        self.consumer_counts: Dict[int, int] = {}

    # -- view inlining -------------------------------------------------------
    @staticmethod
    def count_consumers(nodes: Sequence[GraphNode]) -> Dict[int, int]:
        counts: Dict[int, int] = {}
        visited = set()
        for root in nodes:
            stack = [root]
            while stack:
                n = stack.pop()
                if id(n) in visited:
                    continue
                visited.add(id(n))
                for s in n.src:
                    counts[id(s)] = counts.get(id(s), 0) + 1
                    stack.append(s)
        return counts

    def can_inline_view(self, node: GraphNode) -> bool:
        if node.is_external() or not node.src:
            return False
        return self.consumer_counts.get(id(node), 0) <= 1

    def resolve_view_chain(self, node: GraphNode) -> Tuple[GraphNode, View]:
        if node.op.kind == "view" and self.can_inline_view(node):
            inner_src, inner_view = self.resolve_view_chain(node.src[0])
            return inner_src, View.compose(node.view, inner_view)
        return node, node.view

    # -- naming ------------------------------------------------------------------
    def get_buffer_name(self, node: GraphNode) -> str:
        k = id(node)
        if k in self.buffer_map:
            return self.buffer_map[k]
        if node.name is not None:
            name = f"{node.name}_{self.buffer_counter}"
        else:
            name = f"buf{self.buffer_counter}"
            self.buffer_counter += 1
        self.buffer_counter += 1        # incremented a second time (lower.rs:273)
        self.buffer_map[k] = name
        self.dtype_map[k] = node.dtype
        self.shape_map[k] = node.shape()
        self._nodes[k] = node
        return name

    def generate_kernel_name(self, prefix: str, node: GraphNode) -> str:
        dims = []
        for d in node.shape():
            c = d.as_const()
            dims.append("N" if c is None else str(c))
        name = f"{prefix}_{'_'.join(dims)}_{self.kernel_counter}"
        self.kernel_counter += 1
        return name

    def lookup_buffer_name(self, node: GraphNode) -> Optional[str]:
        return self.buffer_map.get(id(node))

    def get_buffer_info_by_name(self, name: str):
        for k, n in self.buffer_map.items():
            if n == name:
                return self.shape_map[k], self.dtype_map[k]
        return None

    # -- entry point ---------------------------------------------------------------
    def lower(self, roots: Sequence[GraphNode]) -> AstNode:
        order = topological_sort(roots)
        self.consumer_counts = self.count_consumers(order)
        for inp in collect_inputs(roots):
            self.get_buffer_name(inp)
        for node in order:
            if not node.is_external():
                k = self.lower_node(node)
                if k is not None:
                    self.kernels.append(k)
        return AstNode.program(list(self.kernels))

    def lower_node(self, node: GraphNode) -> Optional[AstNode]:
        kind = node.op.kind
        if kind == "view" and self.can_inline_view(node):
            return None
        out = self.get_buffer_name(node)
        if kind == "view" or kind == "unfold":
            return self.lower_view(node, out)
        if kind == "map_reduce":
            if node.op.reduce is not None:
                rop, axis = node.op.reduce
                return self.lower_reduce(node, out, node.op.map, rop, axis)
            return self.lower_elementwise(node, out, node.op.map)
        if kind == "scatter":
            return self.lower_scatter(node, out)
        if kind == "scan":
            return self.lower_scan(node, out)
        if kind == "matmul":
            return self.lower_matmul(node, out)
        raise LoweringError(f"Unsupported operation: {kind}")

    # -- helpers -----------------------------------------------------------------------
    def collect_input_buffers(self, node: GraphNode):
        seen, res = set(), []
        for s in node.src:
            actual, _ = self.resolve_view_chain(s)
            name = self.get_buffer_name(actual)
            if name not in seen:
                seen.add(name)
                res.append((name, self.dtype_map.get(id(actual), F32), actual.shape()))
        return res

    def _context(self, node, out, prefix, output_shape=None):
        inputs = self.collect_input_buffers(node)
        output = (out, node.dtype, output_shape if output_shape is not None else node.shape())
        return self.generate_kernel_name(prefix, node), inputs, output

    def make_kernel(self, name, body, inputs, output) -> AstNode:
        syms = set()

        def collect(e: Expr):
            if e.kind == "sym":
                syms.add(e.a)
            for c in (e.a, e.b):
                if isinstance(c, Expr):
                    collect(c)
        for _, _, shp in list(inputs) + [output]:
            for d in shp:
                collect(d)
        params = [VarDecl(n, DType.ptr(dt), mutable=False) for n, dt, _ in inputs]
        params.append(VarDecl(output[0], DType.ptr(output[1]), mutable=True))
        params += [VarDecl(s, I64, mutable=False) for s in sorted(syms)]
        return AstNode.kernel(name, params, body)

    def _load_with_bounds(self, buf: str, view: View, dtype: DType) -> AstNode:
        load = AstNode.load(AstNode.var(buf), view_to_index(view), dtype)
        dv = view.default_value()
        if dv is None:
            return load
        # pad literal is always F32 (lower.rs:1149)
        return AstNode.select(expr_to_ast(view.condition()), load,
                              AstNode.const_f32(PAD_VALUES[dv]))

    def substitute_wildcards(self, node: GraphNode, expr: AstNode) -> AstNode:
        mapping = {}
        for i, s in enumerate(node.src):
            actual, view = self.resolve_view_chain(s)
            mapping[str(i)] = self._load_with_bounds(self.get_buffer_name(actual), view, s.dtype)
        return expr.substitute(mapping)

    # -- per-op lowering -------------------------------------------------------------------
    def lower_view(self, node, out) -> AstNode:
        name, inputs, output = self._context(node, out, "C")
        shape = node.shape()
        out_idx = view_to_index(View.contiguous(shape))
        actual, inner_view = self.resolve_view_chain(node.src[0])
        composed = View.compose(node.view, inner_view)
        value = self._load_with_bounds(self.get_buffer_name(actual), composed, node.dtype)
        body = generate_loops(shape, AstNode.store(AstNode.var(out), out_idx, value))
        return self.make_kernel(name, body, inputs, output)

    def lower_elementwise(self, node, out, map_) -> AstNode:
        name, inputs, output = self._context(node, out, "E")
        out_idx = view_to_index(node.view)
        value = self.substitute_wildcards(node, map_)
        body = generate_loops(node.shape(), AstNode.store(AstNode.var(out), out_idx, value))
        return self.make_kernel(name, body, inputs, output)

    def lower_reduce(self, node, out, map_, rop, axis) -> AstNode:
        name, inputs, output = self._context(node, out, "R")
        src_shape = node.src[0].shape()
        out_idx = view_to_reduce_output_index(node.view, axis)
        lit_dt, lit_v = reduce_identity(rop, node.dtype)
        value = self.substitute_wildcards(node, map_)
        combine = reduce_combine(rop, AstNode.var("acc"), value)
        body = generate_reduce(src_shape, axis, AstNode.var(out), out_idx, "acc",
                               node.dtype, AstNode.const(lit_dt, lit_v), combine)
        return self.make_kernel(name, body, inputs, output)

    def lower_scan(self, node, out) -> AstNode:
        name, inputs, output = self._context(node, out, "P")
        op = node.op
        src_shape = node.src[0].shape()
        out_idx = view_to_index(node.view)
        lit_dt, lit_v = reduce_identity(op.scan_op, node.dtype)
        value = self.substitute_wildcards(node, op.map)
        combine = reduce_combine(op.scan_op, AstNode.var("acc"), value)
        body = generate_scan(src_shape, op.axis, AstNode.var(out), out_idx, "acc",
                             node.dtype, AstNode.const(lit_dt, lit_v), combine)
        return self.make_kernel(name, body, inputs, output)

    def lower_scatter(self, node, out) -> AstNode:
        op = node.op
        output_shape, axes = op.output_shape, op.axes
        name, inputs, output = self._context(node, out, "S", output_shape)
        src = node.src[0]
        src_shape = src.shape()
        zero_store = AstNode.store(AstNode.var(out),
                                   view_to_index(View.contiguous(output_shape)),
                                   AstNode.const_f32(0.0))
        init_loop = generate_loops(output_shape, zero_store)
        nd, nu = len(output_shape), len(axes)
        npres = nd - nu
        # the source is addressed through its own view, not a resolved chain (lower.rs:623-630)
        load = AstNode.load(AstNode.var(self.get_buffer_name(src)),
                            view_to_index(src.view), node.dtype)
        dst, dst_stride = Expr.const(0), Expr.const(1)
        for axis in range(nd - 1, -1, -1):
            if axis in axes:
                ui = axes.index(axis)
                coord = (Expr.idx(npres + ui) * op.strides[ui]
                         + Expr.idx(npres + nu + ui) * op.dilations[ui]).simplify()
            else:
                coord = Expr.idx(sum(1 for a in range(axis) if a not in axes))
            dst = (dst + coord * dst_stride).simplify()
            dst_stride = (dst_stride * output_shape[axis]).simplify()
        atomic = AstNode.atomic_add(AstNode.var(out), expr_to_ast(dst), load, node.dtype)
        scatter_loop = generate_loops(src_shape, atomic)
        return self.make_kernel(name, AstNode.block([init_loop, scatter_loop]), inputs, output)

    def lower_matmul(self, node, out) -> AstNode:
        name, inputs, output = self._context(node, out, "R")
        op = node.op
        if len(node.src) < 2:
            return self.make_kernel(name, AstNode.block([]), inputs, output)
        a, b = node.src[0], node.src[1]
        ta, tb = op.transpose
        a_buf, b_buf = self.get_buffer_name(a), self.get_buffer_name(b)
        ash, bsh = a.shape(), b.shape()
        one = Expr.const(1)
        m = (ash[1] if ta else ash[0]) if len(ash) > (1 if ta else 0) else one
        k = (ash[0] if ta else ash[1]) if len(ash) > (0 if ta else 1) else one
        n = (bsh[0] if tb else bsh[1]) if len(bsh) > (0 if tb else 1) else one
        acc_dt = op.accumulator_dtype or F32
        dims_ok = all((d.as_const() or 0) > 0 and d.as_const() % 16 == 0 for d in (m, k, n))
        if node.dtype.name == "f16" and dims_ok:
            zero = AstNode.const_i64(0)
            args = [AstNode.var(a_buf), zero, expr_to_ast(m if ta else k),
                    AstNode.var(b_buf), zero, expr_to_ast(k if tb else n),
                    AstNode.var(out), zero, expr_to_ast(n),
                    expr_to_ast(m), expr_to_ast(k), expr_to_ast(n)]
            body = AstNode("wmma_matmul", args, dtype_ab=node.dtype, dtype_c=acc_dt)
            return self.make_kernel(name, body, inputs, output)
        i, j, kk = AstNode.var("ridx_m"), AstNode.var("ridx_n"), AstNode.var("ridx_k")
        a_idx = (AstNode.add(AstNode.mul(kk, expr_to_ast(m)), i) if ta
                 else AstNode.add(AstNode.mul(i, expr_to_ast(k)), kk))
        b_idx = (AstNode.add(AstNode.mul(j, expr_to_ast(k)), kk) if tb
                 else AstNode.add(AstNode.mul(kk, expr_to_ast(n)), j))
        c_idx = AstNode.add(AstNode.mul(i, expr_to_ast(n)), j)
        prod = AstNode.mul(AstNode.load(AstNode.var(a_buf), a_idx, a.dtype),
                           AstNode.load(AstNode.var(b_buf), b_idx, b.dtype))
        k_loop = AstNode.range("ridx_k", AstNode.const_i64(0), AstNode.const_i64(1),
                               expr_to_ast(k),
                               AstNode.assign("acc", AstNode.add(AstNode.var("acc"), prod)))
        init_dt = acc_dt if acc_dt.name in ("f16", "f32", "f64") else F32
        inner = AstNode.block([AstNode.assign("acc", AstNode.const(init_dt, 0.0)), k_loop,
                               AstNode.store(AstNode.var(out), c_idx, AstNode.var("acc"))],
                              decls=[("acc", acc_dt)])
        n_loop = AstNode.range("ridx_n", AstNode.const_i64(0), AstNode.const_i64(1),
                               expr_to_ast(n), inner)
        m_loop = AstNode.range("ridx_m", AstNode.const_i64(0), AstNode.const_i64(1),
                               expr_to_ast(m), n_loop)
        return self.make_kernel(name, m_loop, inputs, output)


def unshare_views(roots: Sequence[GraphNode]) -> List[GraphNode]:
    """Gives every consumer its own copy of each View node it reads, so that all views have
    one consumer and are inlined.  Not in the reference: there a view with several consumers
    is materialised contiguously by a copy kernel but still indexed through its own
    (possibly strided) view by the readers (`lower.rs:209-224` vs `:452-455`), which is only
    right for contiguous views.  Used by the exact mode.

    Unfold nodes become plain views here as well: the reference materialises an unfold into
    a contiguous window buffer and then lets its readers index that buffer through the
    unfold's own (input-space) view (`lower.rs:344-348` vs `:221-224`), which reads the
    wrong elements; as an inlined view the windows are read straight from the input."""
    memo: Dict[int, GraphNode] = {}
    order = topological_sort(roots)

    def is_view(n: GraphNode) -> bool:
        return n.op.kind in ("view", "unfold") and not n.is_external() and bool(n.src)

    def fresh(n: GraphNode) -> GraphNode:
        # a private copy of a view chain, down to the first node that computes something
        if is_view(n):
            op = n.op if n.op.kind == "view" else GraphOp("view", view=n.src[0].view)
            return GraphNode([fresh(n.src[0])], n.view, op, n.dtype, None, n.name, n.hint)
        return memo[id(n)]

    for n in order:
        if is_view(n):
            continue                      # rebuilt on demand by fresh()
        new_src = [fresh(s) for s in n.src]
        changed = any(a is not b for a, b in zip(new_src, n.src))
        memo[id(n)] = n.with_new_sources(new_src) if changed else n
    return [fresh(r) for r in roots]


def lower_graph(roots: Sequence[GraphNode], optimize: bool = True, exact_views: bool = None):
    """`CompilationPipeline::lower_with_lowerer` (compile.rs:227-244) with the
    level-0 graph optimisation (`AllFusions`, compile.rs:366-371).  Returns
    (program AST, lowerer, optimised roots)."""
    from . import config
    if exact_views is None:
        exact_views = config.EXACT
    if exact_views:
        roots = unshare_views(roots)
    opt_roots = all_fusions(roots, share=exact_views) if optimize else list(roots)
    lw = Lowerer()
    program = lw.lower(opt_roots)
    return program, lw, opt_roots
