"""Views: the logical shape of a tensor plus how a logical index maps to a
buffer offset, and an optional bounds condition with a pad value.

Host-side mirror of the reference's `src/graph/shape/view.rs`:
`View::{Linear, IndexExpr}` `:116-133`, `contiguous` `:136`, `to_index_expr`
`:198`, `compose` `:240-323`, `permute` `:350`, `unsqueeze` `:392`, `squeeze`
`:430`, `expand` `:487`, `flip` `:531`, `slice_axis` `:588`, `repeat` `:642`,
`tile` `:711`, `reshape` `:786`, `is_contiguous` `:841`, `padded` `:980`,
`masked` `:1076`, `unfold` `:1162-1384`.  Behaviour is restated as written,
including `compose` keeping only the outer index expression.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

from .expr import Expr, ExprLike, shape_of

PAD_VALUES = {"zero": 0.0, "one": 1.0, "neg_inf": float("-inf")}


class ViewBounds:
    """Condition under which an access is valid, and the value used otherwise."""

    __slots__ = ("condition", "default_value")

    def __init__(self, condition: Expr, default_value: str = "zero"):
        self.condition = condition
        self.default_value = default_value

    @staticmethod
    def none() -> "ViewBounds":
        return ViewBounds(Expr.boolean(True), "zero")

    def has_condition(self) -> bool:
        return not self.condition.is_always_true()

    def substitute_idx(self, idx: int, e: Expr) -> "ViewBounds":
        return ViewBounds(self.condition.substitute_idx(idx, e), self.default_value)

    def shift_indices(self, threshold: int, delta: int) -> "ViewBounds":
        return ViewBounds(self.condition.shift_idx(threshold, delta), self.default_value)

    def permute_idx(self, axes: Sequence[int]) -> "ViewBounds":
        return ViewBounds(self.condition.permute_idx(axes), self.default_value)

    def and_(self, other: "ViewBounds") -> "ViewBounds":
        # the left operand's pad value wins (view.rs:75-84)
        return ViewBounds(self.condition.and_(other.condition).simplify(), self.default_value)

    def __eq__(self, o):
        return (isinstance(o, ViewBounds) and self.condition == o.condition
                and self.default_value == o.default_value)


class View:
    """kind == 'linear': offset + sum(idx[i] * strides[i]);
    kind == 'index_expr': an arbitrary Expr over Idx(0..ndim)."""

    __slots__ = ("kind", "_shape", "strides", "offset", "index_expr", "bounds")

    def __init__(self, kind: str, shape: List[Expr], strides=None, offset=None,
                 index_expr=None, bounds: Optional[ViewBounds] = None):
        self.kind = kind
        self._shape = list(shape)
        self.strides = list(strides) if strides is not None else None
        self.offset = offset
        self.index_expr = index_expr
        self.bounds = bounds if bounds is not None else ViewBounds.none()

    # -- constructors ---------------------------------------------------
    @staticmethod
    def linear(shape, strides, offset, bounds=None) -> "View":
        return View("linear", shape, strides=strides, offset=offset, bounds=bounds)

    @staticmethod
    def from_index_expr(shape, index_expr: Expr, bounds=None) -> "View":
        return View("index_expr", shape_of(shape), index_expr=index_expr, bounds=bounds)

    @staticmethod
    def contiguous(shape: Sequence[ExprLike]) -> "View":
        shape = shape_of(shape)
        if not shape:
            return View.linear([], [], Expr.const(0))
        strides = [Expr.const(1)] * len(shape)
        for i in range(len(shape) - 2, -1, -1):
            strides[i] = (strides[i + 1] * shape[i + 1]).simplify()
        return View.linear(shape, strides, Expr.const(0))

    # -- accessors --------------------------------------------------------
    def shape(self) -> List[Expr]:
        return list(self._shape)

    def ndim(self) -> int:
        return len(self._shape)

    def is_linear(self) -> bool:
        return self.kind == "linear"

    def has_bounds(self) -> bool:
        return self.bounds.has_condition()

    def default_value(self) -> Optional[str]:
        return self.bounds.default_value if self.bounds.has_condition() else None

    def condition(self) -> Optional[Expr]:
        return self.bounds.condition if self.bounds.has_condition() else None

    def __eq__(self, o):
        if not isinstance(o, View) or self.kind != o.kind or self._shape != o._shape:
            return False
        if self.bounds != o.bounds:
            return False
        if self.kind == "linear":
            return self.strides == o.strides and self.offset == o.offset
        return self.index_expr == o.index_expr

    def __repr__(self):
        if self.kind == "linear":
            return f"Linear(shape={self._shape}, strides={self.strides}, offset={self.offset})"
        return f"IndexExpr(shape={self._shape}, expr={self.index_expr})"

    def is_contiguous(self) -> bool:
        if self.kind != "linear" or self.bounds.has_condition():
            return False
        return self == View.contiguous(self._shape)

    def is_innermost_contiguous(self) -> bool:
        if self.kind != "linear" or self.bounds.has_condition():
            return False
        return (not self.strides) or self.strides[-1] == Expr.const(1)

    # -- conversions --------------------------------------------------------
    def to_index_expr(self) -> "View":
        if self.kind == "index_expr":
            return self
        e = self.offset
        for i, s in enumerate(self.strides):
            e = (e + Expr.idx(i) * s).simplify()
        return View("index_expr", self._shape, index_expr=e, bounds=self.bounds)

    @staticmethod
    def compose(outer: "View", inner: "View") -> "View":
        """Result has outer's shape and outer's index expression; the two bounds
        are and-ed without re-indexing (view.rs:240-323)."""
        o = outer.to_index_expr()
        return View("index_expr", o._shape, index_expr=o.index_expr,
                    bounds=o.bounds.and_(inner.bounds))

    # -- transformations ------------------------------------------------------
    def permute(self, axes: Sequence[int]) -> "View":
        axes = list(axes)
        assert len(axes) == self.ndim() and len(set(axes)) == len(axes), "bad permutation"
        if self.kind == "linear":
            return View.linear([self._shape[a].simplify() for a in axes],
                               [self.strides[a].simplify() for a in axes],
                               self.offset, self.bounds.permute_idx(axes))
        return View("index_expr", [self._shape[a] for a in axes],
                    index_expr=self.index_expr.permute_idx(axes),
                    bounds=self.bounds.permute_idx(axes))

    def unsqueeze(self, axis: int) -> "View":
        assert axis <= self.ndim()
        shape = self.shape()
        shape.insert(axis, Expr.const(1))
        if self.kind == "linear":
            strides = list(self.strides)
            strides.insert(axis, Expr.const(0))
            return View.linear(shape, strides, self.offset, self.bounds.shift_indices(axis, 1))
        return View("index_expr", shape, index_expr=self.index_expr.shift_idx(axis, 1),
                    bounds=self.bounds.shift_indices(axis, 1))

    def squeeze(self, axis: int) -> "View":
        assert axis < self.ndim()
        assert self._shape[axis] == Expr.const(1), "can only squeeze an axis of size 1"
        shape = self.shape()
        del shape[axis]
        b = self.bounds.substitute_idx(axis, Expr.const(0)).shift_indices(axis + 1, -1)
        if self.kind == "linear":
            strides = list(self.strides)
            del strides[axis]
            return View.linear(shape, strides, self.offset, b)
        e = self.index_expr.substitute_idx(axis, Expr.const(0)).shift_idx(axis + 1, -1)
        return View("index_expr", shape, index_expr=e, bounds=b)

    def expand(self, axis: int, size: ExprLike) -> "View":
        assert axis < self.ndim(), "axis out of bounds"
        assert self._shape[axis] == Expr.const(1), "can only expand an axis of size 1"
        shape = self.shape()
        shape[axis] = Expr.of(size)
        if self.kind == "linear":
            # the stride of the expanded axis is left as it was (view.rs:505-516)
            return View.linear(shape, self.strides, self.offset, self.bounds)
        return View("index_expr", shape, index_expr=self.index_expr, bounds=self.bounds)

    def flip(self, axis: int) -> "View":
        assert axis < self.ndim()
        flipped = (self._shape[axis] - Expr.const(1) - Expr.idx(axis)).simplify()
        if self.kind == "linear":
            strides = list(self.strides)
            off = (self.offset + (self._shape[axis] - Expr.const(1)) * strides[axis]).simplify()
            strides[axis] = (-strides[axis]).simplify()
            return View.linear(self._shape, strides, off,
                               self.bounds.substitute_idx(axis, flipped))
        return View("index_expr", self._shape,
                    index_expr=self.index_expr.substitute_idx(axis, flipped),
                    bounds=self.bounds.substitute_idx(axis, flipped))

    def slice_axis(self, axis: int, start: ExprLike, length: ExprLike) -> "View":
        start, length = Expr.of(start), Expr.of(length)
        assert axis < self.ndim()
        shape = self.shape()
        shape[axis] = length
        shifted = (Expr.idx(axis) + start).simplify()
        if self.kind == "linear":
            off = (self.offset + start * self.strides[axis]).simplify()
            return View.linear(shape, self.strides, off,
                               self.bounds.substitute_idx(axis, shifted))
        return View("index_expr", shape,
                    index_expr=self.index_expr.substitute_idx(axis, shifted),
                    bounds=self.bounds.substitute_idx(axis, shifted))

    def repeat(self, axis: int, times: ExprLike) -> "View":
        assert axis < self.ndim()
        assert self._shape[axis] == Expr.const(1), "can only repeat an axis of size 1"
        shape = self.shape()
        shape[axis] = Expr.of(times)
        if self.kind == "linear":
            strides = list(self.strides)
            strides[axis] = Expr.const(0)
            return View.linear(shape, strides, self.offset, self.bounds)
        return View("index_expr", shape,
                    index_expr=self.index_expr.substitute_idx(axis, Expr.const(0)),
                    bounds=self.bounds)

    def tile(self, axis: int, times: ExprLike) -> "View":
        assert axis < self.ndim()
        original = self._shape[axis]
        shape = self.shape()
        shape[axis] = (original * Expr.of(times)).simplify()
        cyclic = (Expr.idx(axis) % original).simplify()
        if self.kind == "linear":
            e = self.offset
            for i, s in enumerate(self.strides):
                idx = cyclic if i == axis else Expr.idx(i)
                e = (e + idx * s).simplify()
            return View("index_expr", shape, index_expr=e,
                        bounds=self.bounds.substitute_idx(axis, cyclic))
        return View("index_expr", shape,
                    index_expr=self.index_expr.substitute_idx(axis, cyclic),
                    bounds=self.bounds.substitute_idx(axis, cyclic))

    def reshape(self, new_shape: Sequence[ExprLike]) -> "View":
        assert self.is_contiguous(), "reshape can only be applied to contiguous views"
        new_shape = shape_of(new_shape)
        old_n = Expr.const(1)
        for s in self._shape:
            old_n = old_n * s
        new_n = Expr.const(1)
        for s in new_shape:
            new_n = new_n * s
        o, n = old_n.simplify(), new_n.simplify()
        if o.kind == "const" and n.kind == "const":
            assert o.a == n.a, "reshape requires the number of elements to match"
        r = View.contiguous(new_shape)
        r.offset = self.offset
        r.bounds = self.bounds
        return r

    @staticmethod
    def padded(inner: "View", padding: Sequence[Tuple[ExprLike, ExprLike]],
               default_value: str = "zero") -> "View":
        assert inner.ndim() == len(padding), "padding dimensions must match"
        padding = [(Expr.of(b), Expr.of(a)) for b, a in padding]
        inner_shape = inner.shape()
        padded_shape = [(s + b + a).simplify() for s, (b, a) in zip(inner_shape, padding)]
        cond = Expr.boolean(True)
        for i, ((before, _), size) in enumerate(zip(padding, inner_shape)):
            idx = Expr.idx(i)
            cond = cond.and_(idx.lt(before).not_()).and_(idx.lt(before + size))
        cond = cond.simplify()
        icond = inner.bounds.condition
        for i, (before, _) in enumerate(padding):
            icond = icond.substitute_idx(i, Expr.idx(i) - before)
        adjusted = ViewBounds(icond.simplify(), inner.bounds.default_value)
        bounds = ViewBounds(cond, default_value).and_(adjusted)
        if inner.kind == "linear":
            e = inner.offset
            for i, (stride, (before, _)) in enumerate(zip(inner.strides, padding)):
                e = (e + (Expr.idx(i) - before) * stride).simplify()
        else:
            e = inner.index_expr
            for i, (before, _) in enumerate(padding):
                e = e.substitute_idx(i, Expr.idx(i) - before)
            e = e.simplify()
        return View("index_expr", padded_shape, index_expr=e, bounds=bounds)

    @staticmethod
    def masked(inner: "View", condition: Expr, default_value: str) -> "View":
        nb = ViewBounds(condition, default_value).and_(inner.bounds)
        if inner.kind == "linear":
            return View.linear(inner._shape, inner.strides, inner.offset, nb)
        return View("index_expr", inner._shape, index_expr=inner.index_expr, bounds=nb)

    def unfold(self, axes: Sequence[int], sizes, strides, dilations) -> "View":
        axes = list(axes)
        sizes, strides, dilations = shape_of(sizes), shape_of(strides), shape_of(dilations)
        assert len(axes) == len(sizes) == len(strides) == len(dilations)
        ndim = self.ndim()
        for i, a in enumerate(axes):
            assert a < ndim, "axis out of bounds"
            assert i == 0 or axes[i] > axes[i - 1], "axes must be sorted and unique"
        nu = len(axes)
        npres = ndim - nu
        shape = self._shape
        new_shape = [d for i, d in enumerate(shape) if i not in axes]
        for i, axis in enumerate(axes):
            eff = ((sizes[i] - Expr.const(1)) * dilations[i] + Expr.const(1)).simplify()
            new_shape.append(((shape[axis] - eff) // strides[i] + Expr.const(1)).simplify())
        new_shape += list(sizes)

        def window_index(ui: int) -> Expr:
            return (Expr.idx(npres + ui) * strides[ui]
                    + Expr.idx(npres + nu + ui) * dilations[ui]).simplify()

        if self.kind == "linear":
            e = self.offset
            preserved = 0
            for axis, stride in enumerate(self.strides):
                if axis in axes:
                    e = (e + window_index(axes.index(axis)) * stride).simplify()
                else:
                    e = (e + Expr.idx(preserved) * stride).simplify()
                    preserved += 1
        else:
            e = self.index_expr
            for ui in range(nu - 1, -1, -1):
                e = e.substitute_idx(axes[ui], window_index(ui))
            mapping = []
            new_i = 0
            for i in range(ndim):
                if i not in axes:
                    mapping.append((i, new_i))
                    new_i += 1
            for old, new in reversed(mapping):
                if old != new:
                    e = e.substitute_idx(old, Expr.idx(ndim + nu + old))
            for old, new in mapping:
                if old != new:
                    e = e.substitute_idx(ndim + nu + old, Expr.idx(new))
            e = e.simplify()
        nb = self._unfold_bounds(ndim, axes, window_index)
        return View("index_expr", new_shape, index_expr=e, bounds=nb)

    def _unfold_bounds(self, ndim, axes, window_index) -> ViewBounds:
        if not self.bounds.has_condition():
            return ViewBounds.none()
        temp = 1000
        cond = self.bounds.condition
        preserved = 0
        for orig in range(ndim):
            cond = cond.substitute_idx(orig, Expr.idx(temp + orig))
            if orig in axes:
                cond = cond.substitute_idx(temp + orig, window_index(axes.index(orig)))
            else:
                cond = cond.substitute_idx(temp + orig, Expr.idx(preserved))
                preserved += 1
        return ViewBounds(cond.simplify(), self.bounds.default_value)
