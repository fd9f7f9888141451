"""Computation-graph nodes and the operations that build them.

Host-side mirror of the reference's `src/graph/node.rs` (ReduceOp `:16-77`,
GraphOp `:86-182`, GraphNode view transforms `:325-560`, reductions
`:592-628`, scans `:635-676`, cast `:685`), `src/graph/ops.rs` (broadcast
`:17-67`, binary ops `:70-97`, Sub/Div/Neg sugar `:151-236`, math `:262-367`,
comparisons `:373-441`, where/maximum/minimum/clamp `:443-485`),
`src/graph/builder.rs:40-100` (input/constant/zeros/ones/scalar) and
`src/graph/traversal.rs` (DFS post-order, `GraphTransform`).
Node identity is object identity, as the reference compares `Rc` pointers.
"""

from __future__ import annotations

import itertools
from typing import Callable, Dict, List, Optional, Sequence, Tuple

from .ast import AstNode, DType, F32, BOOL
from .expr import Expr, ExprLike, shape_of
from .view import View

LOG2_E = 1.4426950408889634   # std::f32::consts::LOG2_E, rounded to f32 on use
FRAC_PI_2 = 1.5707963267948966

_buffer_ids = itertools.count()


def _w(i: int) -> AstNode:
    return AstNode.wildcard(str(i))


def reduce_identity(op: str, dtype: DType):
    """ReduceOp::identity (node.rs:29-60). Returns (literal dtype, value)."""
    fam = dtype.name if dtype.name in ("f32", "f64", "i32", "i64") else "f32"
    lit = DType(fam)
    if op == "sum":
        return lit, (0.0 if fam[0] == "f" else 0)
    if op == "prod":
        return lit, (1.0 if fam[0] == "f" else 1)
    if op == "max":
        if fam[0] == "f":
            return lit, float("-inf")
        return lit, (-(2 ** 31) if fam == "i32" else -(2 ** 63))
    if op == "min":
        if fam[0] == "f":
            return lit, float("inf")
        return lit, ((2 ** 31) - 1 if fam == "i32" else (2 ** 63) - 1)
    raise ValueError(op)


def reduce_combine(op: str, acc: AstNode, val: AstNode) -> AstNode:
    """ReduceOp::combine (node.rs:63-77)."""
    if op == "sum":
        return AstNode.add(acc, val)
    if op == "max":
        return AstNode.max(acc, val)
    if op == "prod":
        return AstNode.mul(acc, val)
    if op == "min":
        return AstNode.select(AstNode.lt(acc, val), acc, val)
    raise ValueError(op)


class GraphOp:
    """kind: view | map_reduce | unfold | scatter | scan | matmul."""

    __slots__ = ("kind", "f")

    def __init__(self, kind: str, **fields):
        self.kind = kind
        self.f = fields

    def __getattr__(self, name):
        try:
            return self.f[name]
        except KeyError:
            raise AttributeError(name)


class GraphNode:
    __slots__ = ("src", "view", "op", "dtype", "name", "buffer_id", "hint", "__weakref__")

    def __init__(self, src: Sequence["GraphNode"], view: View, op: GraphOp, dtype: DType,
                 buffer_id: Optional[int] = None, name: Optional[str] = None, hint=None):
        self.src = list(src)
        self.view = view
        self.op = op
        self.dtype = dtype
        self.name = name
        self.buffer_id = buffer_id
        # which view transformation built this node, e.g. ("permute", [1, 0]); the reference
        # keeps no such record -- only the exact-gradient mode reads it
        self.hint = hint

    # -- accessors ---------------------------------------------------------
    def shape(self) -> List[Expr]:
        return self.view.shape()

    def ndim(self) -> int:
        return self.view.ndim()

    def sources(self) -> List["GraphNode"]:
        return self.src

    def is_external(self) -> bool:
        return self.buffer_id is not None

    def with_name(self, name: str) -> "GraphNode":
        return GraphNode(self.src, self.view, self.op, self.dtype, self.buffer_id, name, self.hint)

    def with_new_sources(self, src) -> "GraphNode":
        return GraphNode(src, self.view, self.op, self.dtype, self.buffer_id, self.name, self.hint)

    def __repr__(self):
        return f"GraphNode(name={self.name}, dtype={self.dtype}, shape={self.shape()}, op={self.op.kind})"

    # -- view transformations (node.rs:325-480): op holds the SOURCE view ----
    def _view_node(self, new_view: View, hint=None) -> "GraphNode":
        return GraphNode([self], new_view, GraphOp("view", view=self.view), self.dtype, hint=hint)

    def permute(self, axes):
        return self._view_node(self.view.permute(list(axes)), ("permute", list(axes)))

    def unsqueeze(self, axis): return self._view_node(self.view.unsqueeze(axis), ("unsqueeze", axis))
    def squeeze(self, axis): return self._view_node(self.view.squeeze(axis), ("squeeze", axis))
    def expand(self, axis, size): return self._view_node(self.view.expand(axis, size), ("expand", axis))
    def reshape(self, shape): return self._view_node(self.view.reshape(shape), ("reshape",))
    def flip(self, axis): return self._view_node(self.view.flip(axis), ("flip", axis))
    def repeat(self, axis, times): return self._view_node(self.view.repeat(axis, times), ("expand", axis))

    def slice_axis(self, axis, start, length):
        return self._view_node(self.view.slice_axis(axis, start, length),
                               ("slice", axis, Expr.of(start)))

    def pad(self, padding, value: str = "zero"):
        padding = [(Expr.of(b), Expr.of(a)) for b, a in padding]
        return self._view_node(View.padded(self.view, padding, value), ("pad", padding))

    def contiguous(self) -> "GraphNode":
        return GraphNode([self], View.contiguous(self.shape()),
                         GraphOp("map_reduce", map=_w(0), reduce=None), self.dtype)

    def unfold(self, axes, sizes, strides, dilations) -> "GraphNode":
        nv = self.view.unfold(axes, sizes, strides, dilations)
        op = GraphOp("unfold", input_shape=self.shape(), axes=list(axes),
                     sizes=shape_of(sizes), strides=shape_of(strides),
                     dilations=shape_of(dilations))
        return GraphNode([self], nv, op, self.dtype)

    def fold(self, output_shape, axes, sizes, strides, dilations) -> "GraphNode":
        output_shape = shape_of(output_shape)
        op = GraphOp("scatter", output_shape=output_shape, axes=list(axes),
                     sizes=shape_of(sizes), strides=shape_of(strides),
                     dilations=shape_of(dilations))
        return GraphNode([self], View.contiguous(output_shape), op, self.dtype)

    # -- reductions / scans ----------------------------------------------------
    def _reduce(self, op: str, axis: int) -> "GraphNode":
        shape = self.shape()
        shape[axis] = Expr.const(1)
        return GraphNode([self], View.contiguous(shape),
                         GraphOp("map_reduce", map=_w(0), reduce=(op, axis)), self.dtype)

    def sum(self, axis): return self._reduce("sum", axis)
    def max(self, axis): return self._reduce("max", axis)
    def min(self, axis): return self._reduce("min", axis)
    def prod(self, axis): return self._reduce("prod", axis)

    def _scan(self, op: str, axis: int, exclusive: bool = False) -> "GraphNode":
        return GraphNode([self], View.contiguous(self.shape()),
                         GraphOp("scan", map=_w(0), scan_op=op, axis=axis,
                                 exclusive=exclusive), self.dtype)

    def cumsum(self, axis): return self._scan("sum", axis)
    def cumprod(self, axis): return self._scan("prod", axis)
    def cummax(self, axis): return self._scan("max", axis)

    def cast(self, dtype: DType) -> "GraphNode":
        return GraphNode([self], self.view,
                         GraphOp("map_reduce", map=AstNode.cast(_w(0), dtype), reduce=None),
                         dtype)

    # -- elementwise -------------------------------------------------------------
    def unary_op(self, f: Callable[[AstNode], AstNode]) -> "GraphNode":
        # the result keeps this node's view, not a contiguous one (ops.rs:255-274)
        return GraphNode([self], self.view,
                         GraphOp("map_reduce", map=f(_w(0)), reduce=None), self.dtype)

    def __add__(self, o): return binary_op(self, o, AstNode.add)
    def __mul__(self, o): return binary_op(self, o, AstNode.mul)

    def __sub__(self, o):
        return binary_op(self, o, lambda a, b: AstNode.add(
            a, AstNode.mul(b, AstNode.const_f32(-1.0))))

    def __truediv__(self, o):
        return binary_op(self, o, lambda a, b: AstNode.mul(a, AstNode.recip(b)))

    def __neg__(self):
        return self.unary_op(lambda x: AstNode.mul(x, AstNode.const_f32(-1.0)))

    def sqrt(self): return self.unary_op(lambda x: AstNode.unary("sqrt", x))
    def recip(self): return self.unary_op(lambda x: AstNode.unary("recip", x))
    def log2(self): return self.unary_op(lambda x: AstNode.unary("log2", x))
    def exp2(self): return self.unary_op(lambda x: AstNode.unary("exp2", x))
    def sin(self): return self.unary_op(lambda x: AstNode.unary("sin", x))
    def floor(self): return self.unary_op(lambda x: AstNode.unary("floor", x))

    def ln(self):
        return self.unary_op(lambda x: AstNode.mul(
            AstNode.unary("log2", x), AstNode.recip(AstNode.const_f32(LOG2_E))))

    def exp(self):
        return self.unary_op(lambda x: AstNode.unary(
            "exp2", AstNode.mul(x, AstNode.const_f32(LOG2_E))))

    def cos(self):
        return self.unary_op(lambda x: AstNode.unary(
            "sin", AstNode.add(x, AstNode.const_f32(FRAC_PI_2))))

    def abs(self):
        def f(x):
            sign = AstNode.select(AstNode.lt(x, AstNode.const_f32(0.0)),
                                  AstNode.const_f32(-1.0), AstNode.const_f32(1.0))
            return AstNode.mul(x, sign)
        return self.unary_op(f)

    def lt(self, other: "GraphNode") -> "GraphNode":
        r = binary_op(self, other, AstNode.lt)
        return GraphNode(r.src, r.view, r.op, BOOL)

    def gt(self, other): return other.lt(self)
    def le(self, other): return other.lt(self).logical_not()
    def ge(self, other): return self.lt(other).logical_not()
    def eq_node(self, other): return self.le(other).logical_and(other.le(self))
    def ne_node(self, other): return self.eq_node(other).logical_not()

    def logical_and(self, other):
        return binary_op(self, other, lambda a, b: AstNode("and", [a, b]))

    def logical_not(self):
        return self.unary_op(lambda x: AstNode("not", [x]))

    def logical_or(self, other):
        return self.logical_not().logical_and(other.logical_not()).logical_not()

    def where_cond(self, cond: "GraphNode", other: "GraphNode") -> "GraphNode":
        sel = AstNode.select(_w(0), _w(1), _w(2))
        return GraphNode([cond, self, other], self.view,
                         GraphOp("map_reduce", map=sel, reduce=None), self.dtype)

    def maximum(self, other): return binary_op(self, other, AstNode.max)

    def minimum(self, other):
        return binary_op(self, other,
                         lambda a, b: AstNode.select(AstNode.lt(a, b), a, b))

    def clamp(self, lo, hi): return self.maximum(lo).minimum(hi)


def broadcast(lhs: GraphNode, rhs: GraphNode) -> Tuple[GraphNode, GraphNode]:
    """ops.rs:17-67."""
    ls, rs = lhs.shape(), rhs.shape()
    if ls == rs:
        return lhs, rhs
    nd = max(len(ls), len(rs))
    for _ in range(nd - len(ls)):
        lhs = lhs.unsqueeze(0)
    for _ in range(nd - len(rs)):
        rhs = rhs.unsqueeze(0)
    ls, rs = lhs.shape(), rhs.shape()
    for i in range(nd):
        if ls[i] != rs[i]:
            if ls[i] == Expr.const(1):
                lhs = lhs.expand(i, rs[i])
            elif rs[i] == Expr.const(1):
                rhs = rhs.expand(i, ls[i])
            else:
                raise ValueError(f"Cannot broadcast shapes: {ls} and {rs} at dimension {i}")
    return lhs, rhs


def binary_op(lhs: GraphNode, rhs: GraphNode, combine) -> GraphNode:
    """ops.rs:70-97: result is contiguous with the broadcast shape, lhs dtype."""
    l, r = broadcast(lhs, rhs)
    return GraphNode([l, r], View.contiguous(l.shape()),
                     GraphOp("map_reduce", map=combine(_w(0), _w(1)), reduce=None), l.dtype)


# -- builder (builder.rs:40-100) ----------------------------------------------

def input(shape: Sequence[ExprLike], dtype: DType = F32) -> GraphNode:
    v = View.contiguous(shape)
    return GraphNode([], v, GraphOp("view", view=v), dtype, buffer_id=next(_buffer_ids))


def named_input(name: str, shape, dtype: DType = F32) -> GraphNode:
    return input(shape, dtype).with_name(name)


def constant(shape, dtype: DType = F32) -> GraphNode:
    return input(shape, dtype).with_name("const")


def zeros(shape, dtype: DType = F32) -> GraphNode:
    return constant(shape, dtype).with_name("zeros")


def ones(shape, dtype: DType = F32) -> GraphNode:
    return constant(shape, dtype).with_name("ones")


def scalar(dtype: DType = F32) -> GraphNode:
    return input([], dtype).with_name("scalar")


# -- traversal (traversal.rs) ---------------------------------------------------

def topological_sort(roots: Sequence[GraphNode]) -> List[GraphNode]:
    """DFS post-order, sources first, each node once."""
    seen = set()
    out: List[GraphNode] = []
    for root in roots:
        stack = [(root, 0)]
        while stack:
            node, i = stack.pop()
            if i == 0:
                if id(node) in seen:
                    continue
                seen.add(id(node))
            if i < len(node.src):
                stack.append((node, i + 1))
                child = node.src[i]
                if id(child) not in seen:
                    stack.append((child, 0))
            else:
                out.append(node)
    return out


def collect_inputs(roots: Sequence[GraphNode]) -> List[GraphNode]:
    return [n for n in topological_sort(roots) if n.is_external()]


def apply_transform(transform: Callable[[GraphNode], Optional[GraphNode]],
                    roots: Sequence[GraphNode], share_cache: bool = False) -> List[GraphNode]:
    """GraphTransform::apply (traversal.rs:197-245): bottom-up, a fresh cache
    per root, nodes rebuilt only when a source changed.  `share_cache` keeps one cache
    for all roots, so nodes common to several roots stay common (the reference rebuilds
    them once per root)."""
    out = []
    shared: Dict[int, GraphNode] = {}
    keep = []
    for root in roots:
        cache: Dict[int, GraphNode] = shared if share_cache else {}
        order = topological_sort([root])
        keep.append(order)
        for node in order:
            if id(node) in cache:
                continue
            new_src = [cache[id(s)] for s in node.src]
            changed = any(a is not b for a, b in zip(new_src, node.src))
            cur = node.with_new_sources(new_src) if changed else node
            res = transform(cur)
            cache[id(node)] = res if res is not None else cur
        out.append(cache[id(root)])
    return out
