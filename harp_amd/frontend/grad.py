"""Reverse-mode differentiation by graph construction.

Host-side mirror of the reference's `src/grad/`: `backward` (`backward.rs:41-108`),
`GradContext` (`context.rs`), and the per-op VJP rules of `rules.rs`
(`compute_vjp` `:28-84`, matmul `:95-190`, elementwise `:196-345`, reduce
`:348-445`, scan `:448-530`, view `:534-712`, `categorize_map` `:736-778`).

The rules are restated as written, not as calculus would have them.  In
particular: a map is classified by its top AST node, so `a - b`
(= `Add(a, Mul(b, -1))`) is an Add and passes `+g` to `b`, `a / b`
(= `Mul(a, Recip(b))`) is a Mul, and `exp(x)` (= `Exp2(Mul(x, c))`) takes the
Exp2 rule; `create_scalar_like` ignores its value and returns ones
(`rules.rs:854-860`), so the `ln 2` factors of exp2/log2 are dropped; the VJP
of a same-rank view that is not an expand is `contiguous().reshape()`, which
for a permute is a reshape, not the inverse permutation.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence

from .ast import AstNode
from .expr import Expr
from .graph import GraphNode, GraphOp, ones, topological_sort, zeros
from .view import View


class GradContext:
    def __init__(self):
        self.grad_map: Dict[int, GraphNode] = {}
        self.requires: set = set()
        self._keep: List[GraphNode] = []

    def mark_requires_grad(self, n: GraphNode) -> None:
        self.requires.add(id(n))
        self._keep.append(n)

    def requires_grad(self, n: GraphNode) -> bool:
        return id(n) in self.requires

    def get_grad(self, n: GraphNode) -> Optional[GraphNode]:
        return self.grad_map.get(id(n))

    def set_grad(self, n: GraphNode, g: GraphNode) -> None:
        self.grad_map[id(n)] = g
        self._keep.append(n)

    def accumulate_grad(self, n: GraphNode, g: GraphNode) -> None:
        cur = self.grad_map.get(id(n))
        self.grad_map[id(n)] = (cur + g) if cur is not None else g
        self._keep.append(n)


class GradResult:
    def __init__(self, ctx: GradContext, params: Sequence[GraphNode]):
        self.context = ctx
        self.params = list(params)

    def get(self, param: GraphNode) -> Optional[GraphNode]:
        return self.context.get_grad(param)

    def grads(self) -> List[Optional[GraphNode]]:
        return [self.context.get_grad(p) for p in self.params]


def backward(output: GraphNode, params: Sequence[GraphNode], exact: bool = False) -> GradResult:
    """`exact=False` restates the reference's rules as written; `exact=True` applies the
    mathematically correct VJPs (see `compute_vjp_exact`), which the reference does not have."""
    ctx = GradContext()
    for p in params:
        ctx.mark_requires_grad(p)
    ctx.set_grad(output, ones(output.shape(), output.dtype))
    memo: Dict[int, bool] = {}

    def needs_grad(n: GraphNode) -> bool:
        k = id(n)
        if k in memo:
            return memo[k]
        r = ctx.requires_grad(n) or any(needs_grad(s) for s in n.src)
        memo[k] = r
        return r

    for node in reversed(topological_sort([output])):
        g = ctx.get_grad(node)
        if g is None or not node.src:
            continue
        for src, gi in zip(node.src, compute_vjp_exact(node, g) if exact else compute_vjp(node, g)):
            if gi is not None and needs_grad(src):
                ctx.accumulate_grad(src, gi)
    return GradResult(ctx, params)


# ---------------------------------------------------------------------------
# VJP rules
# ---------------------------------------------------------------------------

def _zeros_like(n: GraphNode) -> GraphNode:
    return zeros(n.shape(), n.dtype)


def _ones_like(n: GraphNode) -> GraphNode:
    return ones(n.shape(), n.dtype)


def _scalar_like(n: GraphNode, _value: float) -> GraphNode:
    return _ones_like(n)


def compute_vjp(node: GraphNode, g: GraphNode) -> List[Optional[GraphNode]]:
    op = node.op
    k = op.kind
    if k == "view":
        return _view_vjp(node, g)
    if k == "map_reduce":
        if op.reduce is not None:
            return _reduce_vjp(node, g, op.reduce[0], op.reduce[1])
        return _elementwise_vjp(node, g, op.map)
    if k == "unfold":
        return [g.fold(op.input_shape, op.axes, op.sizes, op.strides, op.dilations)]
    if k == "scatter":
        return [g.unfold(op.axes, op.sizes, op.strides, op.dilations)]
    if k == "scan":
        return _scan_vjp(node, g, op.scan_op, op.axis)
    if k == "matmul":
        return _matmul_vjp(node, g, op.transpose)
    raise ValueError(k)


def _is_const_neg_one(n: AstNode) -> bool:
    return (n.op == "const" and n.attrs["dtype"].name in ("f32", "i32")
            and n.attrs["value"] == -1)


def _is_constant_expr(n: AstNode) -> bool:
    if n.op == "const":
        return True
    if n.op == "recip":
        return _is_constant_expr(n.args[0])
    if n.op in ("mul", "add"):
        return _is_constant_expr(n.args[0]) and _is_constant_expr(n.args[1])
    return False


def categorize_map(m: AstNode) -> str:
    if m.op == "mul" and (_is_const_neg_one(m.args[0]) or _is_const_neg_one(m.args[1])):
        return "neg"
    if m.op == "mul" and m.args[0].op == "log2" and _is_constant_expr(m.args[1]):
        return "log"
    table = {"add": "add", "mul": "mul", "recip": "recip", "sqrt": "sqrt", "exp2": "exp2",
             "log2": "log2", "sin": "sin", "floor": "floor", "max": "max", "lt": "comparison",
             "and": "comparison", "not": "comparison", "select": "select", "cast": "cast"}
    return table.get(m.op, "unknown")


def _elementwise_vjp(node, g, m) -> List[Optional[GraphNode]]:
    ins = node.src
    cat = categorize_map(m)
    if cat == "add":
        return [g, g]
    if cat == "mul":
        if len(ins) < 2:
            return [g]
        return [g * ins[1], g * ins[0]]
    if cat == "neg":
        return [-g]
    if cat == "recip":
        return [(-g) / (ins[0] * ins[0])]
    if cat == "sqrt":
        s = ins[0].sqrt()
        return [g / (s + s)]
    if cat == "log":
        return [g / ins[0]]
    if cat == "exp2":
        return [(g * ins[0].exp2()) * _scalar_like(g, 0.6931472)]
    if cat == "log2":
        return [(g / ins[0]) * _scalar_like(g, 1.442695)]
    if cat == "sin":
        return [g * ins[0].cos()]
    if cat == "floor":
        return [_zeros_like(g)]
    if cat == "max":
        mask_a = ins[0].ge(ins[1])
        mask_b = ins[1].gt(ins[0])
        z = _zeros_like(g)
        return [g.where_cond(mask_a, z), g.where_cond(mask_b, z)]
    if cat == "comparison":
        return [None] * len(ins)
    if cat == "select":
        z = _zeros_like(g)
        cond = ins[0]
        return [None, g.where_cond(cond, z), z.where_cond(cond, g)]
    if cat == "cast":
        return [g.cast(ins[0].dtype)]
    return [_zeros_like(g) for _ in ins]


def _reduce_vjp(node, g, rop, axis) -> List[Optional[GraphNode]]:
    x = node.src[0]
    axis_size = x.shape()[axis]
    gw = g.unsqueeze(axis) if g.ndim() < x.ndim() else g
    if rop == "sum":
        return [gw.expand(axis, axis_size)]
    nw = node.unsqueeze(axis) if node.ndim() < x.ndim() else node
    full = nw.expand(axis, axis_size)
    ge = gw.expand(axis, axis_size)
    if rop in ("max", "min"):
        mask = x.eq_node(full).cast(x.dtype)
        return [ge * mask]
    return [(ge * full) / x]                       # prod


def _scan_vjp(node, g, sop, axis) -> List[Optional[GraphNode]]:
    x = node.src[0]
    if sop == "sum":
        return [g.flip(axis).cumsum(axis).flip(axis)]
    if sop == "prod":
        return [(g * node).flip(axis).cumsum(axis).flip(axis) / x]
    mask = x.eq_node(node).cast(x.dtype)           # max / min
    return [g * mask]


def _numel(shape) -> Optional[int]:
    n = 1
    for d in shape:
        if d.kind != "const":
            return None
        n *= d.a
    return n


def _is_squeeze_or_unsqueeze(a, b) -> bool:
    longer, shorter = (a, b) if len(a) > len(b) else (b, a)
    si = 0
    one = Expr.const(1)
    for d in longer:
        if si < len(shorter) and d == shorter[si]:
            si += 1
        elif d != one:
            return False
    return si == len(shorter)


def _view_vjp(node, g) -> List[Optional[GraphNode]]:
    orig, cur = node.src[0].shape(), node.shape()
    on, cn = _numel(orig), _numel(cur)
    one = Expr.const(1)
    if orig == cur:
        return [g]
    if on is not None and cn is not None and on != cn:
        if cn > on and len(orig) == len(cur):      # padding: slice the centre back out
            r = g
            for axis, (o, n) in enumerate(zip(orig, cur)):
                if o.kind == "const" and n.kind == "const" and n.a > o.a:
                    r = r.slice_axis(axis, Expr.const((n.a - o.a) // 2), o)
            return [r]
        if cn < on and len(orig) == len(cur):      # slicing: pad back
            padding = []
            for o, n in zip(orig, cur):
                if o.kind == "const" and n.kind == "const":
                    diff = o.a - n.a
                    padding.append((diff // 2, diff - diff // 2))
                else:
                    padding.append((0, 0))
            return [g.pad(padding, "zero")]
        return [g.contiguous().reshape(orig)]
    if len(orig) != len(cur) and not _is_squeeze_or_unsqueeze(orig, cur):
        return [g.contiguous().reshape(orig)]
    if len(orig) > len(cur):                       # squeeze -> unsqueeze the gradient
        r, oi = g, 0
        for ii, d in enumerate(orig):
            if oi >= len(cur) or d != cur[oi]:
                r = r.unsqueeze(ii)
            else:
                oi += 1
        return [r]
    if len(orig) < len(cur):                       # unsqueeze -> squeeze the gradient
        axes, ii = [], 0
        for oi, d in enumerate(cur):
            if ii >= len(orig) or d != orig[ii]:
                axes.append(oi)
            else:
                ii += 1
        r = g
        for a in reversed(axes):
            r = r.squeeze(a)
        return [r]
    r, is_expand = g, False
    for i, (o, n) in enumerate(zip(orig, cur)):
        if o == one and n != one:
            is_expand = True
            r = r.sum(i)
    if is_expand:
        return [r]
    return [g.contiguous().reshape(orig)]


def _matmul_vjp(node, g, transpose) -> List[Optional[GraphNode]]:
    ins = node.src
    if len(ins) < 2:
        return [None] * len(ins)
    a, b = ins[0], ins[1]
    ta, tb = transpose
    ash, bsh, csh = a.shape(), b.shape(), g.shape()
    if len(ash) < 2 or len(bsh) < 2:
        return [None] * len(ins)
    k = ash[0] if ta else ash[1]
    n = bsh[0] if tb else bsh[1]
    gc = g.unsqueeze(1).expand(1, k)
    bt = b if tb else b.permute([1, 0])
    ga = (gc * bt.unsqueeze(0).expand(0, csh[0])).sum(2).squeeze(2)
    if ta:
        ga = ga.permute([1, 0])
    at = a if ta else a.permute([1, 0])
    gb = (at.unsqueeze(2).expand(2, n) * g.unsqueeze(0).expand(0, k)).sum(0).squeeze(0)
    if tb:
        gb = gb.permute([1, 0])
    return [ga, gb]


# ---------------------------------------------------------------------------
# exact VJPs (not in the reference)
# ---------------------------------------------------------------------------

def _dense_unary(g: GraphNode, f) -> GraphNode:
    """f(g) stored contiguously.  `unary_op` hands its operand's view to the result, and
    the lowerer stores through the result's view: over a slice that writes past a buffer
    sized by the shape, over a broadcast it writes one element many times."""
    if g.view.is_contiguous():
        return g.unary_op(f)
    return GraphNode([g], View.contiguous(g.shape()),
                     GraphOp("map_reduce", map=f(AstNode.wildcard("0")), reduce=None), g.dtype)


def _scaled(g: GraphNode, c: float) -> GraphNode:
    return _dense_unary(g, lambda x: AstNode.mul(x, AstNode.const_f32(c)))


def _dense(n: GraphNode) -> GraphNode:
    """A node whose own view is contiguous (elementwise results inherit the view of
    their first operand, which may be a broadcast)."""
    return n if n.view.is_contiguous() else n.contiguous()


def _is_w(n: AstNode, i: int) -> bool:
    return n.op == "wildcard" and n.attrs["name"] == str(i)


def _is_f32(n: AstNode, v: float) -> bool:
    return n.op == "const" and n.attrs["dtype"].name == "f32" and abs(n.attrs["value"] - v) < 1e-6


def compute_vjp_exact(node: GraphNode, g: GraphNode) -> List[Optional[GraphNode]]:
    op = node.op
    if op.kind == "view":
        return _view_vjp_exact(node, g)
    if op.kind == "map_reduce" and op.reduce is not None:
        rop, axis = op.reduce
        x = node.src[0]
        size = x.shape()[axis]
        gw = g.unsqueeze(axis) if g.ndim() < x.ndim() else g
        ge = gw.repeat(axis, size)                      # stride 0 along the reduced axis
        if _is_w(op.map, 0):
            if rop == "sum":
                return [ge]
            nw = node.unsqueeze(axis) if node.ndim() < x.ndim() else node
            full = nw.repeat(axis, size)
            if rop in ("max", "min"):
                return [ge * x.eq_node(full).cast(x.dtype)]
            return [(ge * full) / x]
        raise NotImplementedError("exact VJP of a reduce with a fused map: differentiate before fusion")
    if op.kind == "map_reduce":
        return _elementwise_vjp_exact(node, g, op.map)
    if op.kind == "unfold":
        return [_unfold_adjoint(g, op)]
    return compute_vjp(node, g)                          # scatter / scan / matmul


def _elementwise_vjp_exact(node, g, m) -> List[Optional[GraphNode]]:
    ins = node.src
    # g may be a broadcast view; unary results inherit that view (stored compactly), which
    # every reader then indexes consistently, so only selects need a dense operand
    if m.op == "add" and _is_w(m.args[0], 0) and m.args[1].op == "mul" and \
            _is_w(m.args[1].args[0], 1) and _is_f32(m.args[1].args[1], -1.0):
        return [g, -g]                                   # a - b
    if m.op == "mul" and _is_w(m.args[0], 0) and m.args[1].op == "recip" and _is_w(m.args[1].args[0], 1):
        a, b = ins
        return [g / b, (-(g * a)) / (b * b)]             # a / b
    if m.op == "exp2" and m.args[0].op == "mul" and _is_w(m.args[0].args[0], 0) and \
            m.args[0].args[1].op == "const":
        return [g * node]                                # exp(x): d/dx = exp(x) itself
    if m.op == "exp2" and _is_w(m.args[0], 0):
        return [_scaled(g * node, 0.6931471805599453)]
    if m.op == "log2" and _is_w(m.args[0], 0):
        return [_scaled(g / ins[0], 1.4426950408889634)]
    if m.op == "sin" and m.args[0].op == "add" and _is_w(m.args[0].args[0], 0):
        return [-(g * ins[0].sin())]                     # cos(x)
    if m.op == "mul" and len(ins) == 1 and _is_w(m.args[0], 0) and m.args[1].op == "const":
        return [_scaled(g, m.args[1].attrs["value"])]    # x * c
    if m.op == "wildcard":
        return [g]                                       # contiguous(): identity map
    if m.op == "max" and len(ins) == 2:
        z = _zeros_like(g)
        return [_select_dense(ins[0].ge(ins[1]), g, z), _select_dense(ins[1].gt(ins[0]), g, z)]
    if m.op == "select" and len(ins) == 3:
        z = _zeros_like(g)
        return [None, _select_dense(ins[0], g, z), _select_dense(ins[0], z, g)]
    if m.op == "select" and len(ins) == 2 and m.args[0].op == "lt" and _is_w(m.args[0].args[0], 0) and \
            _is_w(m.args[0].args[1], 1) and _is_w(m.args[1], 0) and _is_w(m.args[2], 1):
        z = _zeros_like(g)                               # minimum(a, b) = a < b ? a : b
        cond = ins[0].lt(ins[1])
        return [_select_dense(cond, g, z), _select_dense(cond, z, g)]
    if categorize_map(m) not in ("add", "mul", "neg", "recip", "sqrt", "log", "sin", "floor", "cast", "comparison"):
        raise NotImplementedError(f"no exact VJP for the elementwise map {m.to_sexpr()}")
    return _elementwise_vjp(node, g, m)                  # rules that are right as written


def _unfold_adjoint(g: GraphNode, op) -> GraphNode:
    """Adjoint of a sliding-window unfold as a gather (no scatter, no atomics): every input
    position sums the window slots that read it.  g: [preserved..., out_0.., k_0..].

    Windows that tile the axis (stride == size, dilation 1) are a pure re-indexing:
    interleave (out_i, k_i) and merge.  Unit-stride windows are a sum over the window
    offsets of g's slice at that offset, zero-padded back to the input extent."""
    in_shape = [int(e.evaluate()) for e in op.input_shape]
    sizes = [int(e.evaluate()) for e in op.sizes]
    strides = [int(e.evaluate()) for e in op.strides]
    dils = [int(e.evaluate()) for e in op.dilations]
    axes, nu = list(op.axes), len(op.axes)
    npres = len(in_shape) - nu
    if axes != list(range(npres, npres + nu)):
        raise NotImplementedError("exact unfold adjoint: windowed axes must be the trailing ones")
    outs = [int(e.evaluate()) for e in g.shape()[npres:npres + nu]]
    if all(s == k and d == 1 for s, k, d in zip(strides, sizes, dils)):
        perm = list(range(npres))
        for i in range(nu):
            perm += [npres + i, npres + nu + i]
        merged = g.permute(perm).contiguous().reshape(
            in_shape[:npres] + [o * k for o, k in zip(outs, sizes)])
        padding = [(0, 0)] * npres + [(0, n - o * k) for n, o, k in zip(in_shape[npres:], outs, sizes)]
        return merged.pad(padding, "zero") if any(a for _, a in padding) else merged
    if all(s == 1 for s in strides):
        import itertools
        total = None
        for ks in itertools.product(*[range(k) for k in sizes]):
            term = g
            for i in range(nu - 1, -1, -1):                      # drop the window axes, last first
                term = term.slice_axis(npres + nu + i, ks[i], 1).squeeze(npres + nu + i)
            padding = [(0, 0)] * npres
            for i in range(nu):
                before = ks[i] * dils[i]
                padding.append((before, in_shape[npres + i] - outs[i] - before))
            term = term.pad(padding, "zero")
            total = term if total is None else total + term
        return total
    raise NotImplementedError("exact unfold adjoint: strided overlapping windows")


def _select_dense(cond: GraphNode, a: GraphNode, b: GraphNode) -> GraphNode:
    from .graph import GraphOp, _w
    from .view import View
    return GraphNode([cond, a, b], View.contiguous(a.shape()),
                     GraphOp("map_reduce", map=AstNode.select(_w(0), _w(1), _w(2)), reduce=None),
                     a.dtype)


def _view_vjp_exact(node, g) -> List[Optional[GraphNode]]:
    src = node.src[0]
    h = node.hint
    if h is None:
        if src.shape() == node.shape():
            return [g]
        raise NotImplementedError("exact VJP needs to know which view transformation was applied")
    kind = h[0]
    if kind == "permute":
        inv = [0] * len(h[1])
        for new_axis, old_axis in enumerate(h[1]):
            inv[old_axis] = new_axis
        return [g.permute(inv)]
    if kind == "unsqueeze":
        return [g.squeeze(h[1])]
    if kind == "squeeze":
        return [g.unsqueeze(h[1])]
    if kind == "expand":
        return [g.sum(h[1])]
    if kind == "reshape":
        return [_dense(g).reshape(src.shape())]
    if kind == "flip":
        return [g.flip(h[1])]
    if kind == "pad":
        r = g
        for axis, ((before, _after), size) in enumerate(zip(h[1], src.shape())):
            r = r.slice_axis(axis, before, size)
        return [r]
    if kind == "slice":
        axis, start = h[1], h[2]
        full = src.shape()[axis]
        after = (full - start - node.shape()[axis]).simplify()
        padding = [(0, 0)] * src.ndim()
        padding[axis] = (start, after)
        return [g.pad(padding, "zero")]
    raise NotImplementedError(kind)
