"""Symbolic index expressions (`Expr`) used by views and the lowerer.

Host-side mirror of the reference's `src/graph/shape/expr.rs`:
variants `:7-59`, `simplify` `:545-663`, `substitute_idx` `:378`,
`permute_idx` `:439`, `shift_idx` `:499`, conversion to the kernel AST
`:62-105`.  Expressions are immutable tuples-with-a-tag so they can be
compared and hashed structurally, as the reference's derive(PartialEq, Hash).
"""

from __future__ import annotations

from typing import Sequence, Union

ExprLike = Union["Expr", int, bool]


class Expr:
    """One node of an index expression.  `kind` is one of
    const, bool, idx, add, sub, mul, div, rem, lt, and, not, sym."""

    __slots__ = ("kind", "a", "b")

    def __init__(self, kind: str, a=None, b=None):
        self.kind = kind
        self.a = a
        self.b = b

    # -- constructors -------------------------------------------------
    @staticmethod
    def const(v: int) -> "Expr":
        return Expr("const", int(v))

    @staticmethod
    def boolean(v: bool) -> "Expr":
        return Expr("bool", bool(v))

    @staticmethod
    def idx(i: int) -> "Expr":
        return Expr("idx", int(i))

    @staticmethod
    def sym(name: str) -> "Expr":
        return Expr("sym", name)

    @staticmethod
    def of(v: ExprLike) -> "Expr":
        if isinstance(v, Expr):
            return v
        if isinstance(v, bool):
            return Expr.boolean(v)
        return Expr.const(int(v))

    # -- structural equality -------------------------------------------
    def _key(self):
        return (self.kind, self.a._key() if isinstance(self.a, Expr) else self.a,
                self.b._key() if isinstance(self.b, Expr) else self.b)

    def __eq__(self, other):
        return isinstance(other, Expr) and self._key() == other._key()

    def __ne__(self, other):
        return not self.__eq__(other)

    def __hash__(self):
        return hash(self._key())

    # -- operators (no simplification, as expr.rs:790-803) --------------
    def __add__(self, o): return Expr("add", self, Expr.of(o))
    def __radd__(self, o): return Expr("add", Expr.of(o), self)
    def __sub__(self, o): return Expr("sub", self, Expr.of(o))
    def __rsub__(self, o): return Expr("sub", Expr.of(o), self)
    def __mul__(self, o): return Expr("mul", self, Expr.of(o))
    def __rmul__(self, o): return Expr("mul", Expr.of(o), self)
    def __floordiv__(self, o): return Expr("div", self, Expr.of(o))
    def __mod__(self, o): return Expr("rem", self, Expr.of(o))
    def __neg__(self): return Expr("sub", Expr.const(0), self)

    def lt(self, o): return Expr("lt", self, Expr.of(o))
    def ge(self, o): return Expr("not", Expr("lt", self, Expr.of(o)))
    def le(self, o): return Expr("not", Expr("lt", Expr.of(o), self))
    def gt(self, o): return Expr("lt", Expr.of(o), self)
    def and_(self, o): return Expr("and", self, Expr.of(o))
    def not_(self): return Expr("not", self)

    # -- predicates ---------------------------------------------------
    def is_always_true(self) -> bool:
        return self.kind == "bool" and self.a is True

    def as_const(self):
        if self.kind == "const":
            return self.a
        s = self.simplify()
        return s.a if s.kind == "const" else None

    def evaluate(self) -> int:
        v = self.as_const()
        if v is None:
            raise ValueError(f"expression is not a constant: {self}")
        return v

    # -- rewriting ----------------------------------------------------
    def _map(self, f) -> "Expr":
        k = self.kind
        if k in ("add", "sub", "mul", "div", "rem", "lt", "and"):
            return Expr(k, f(self.a), f(self.b))
        if k == "not":
            return Expr(k, f(self.a))
        return self

    def substitute_idx(self, idx: int, repl: "Expr") -> "Expr":
        if self.kind == "idx":
            return repl if self.a == idx else self
        return self._map(lambda e: e.substitute_idx(idx, repl))

    def permute_idx(self, axes: Sequence[int]) -> "Expr":
        """axes[new] = old, so Idx(old) becomes Idx(new) (expr.rs:439-447)."""
        inverse = [0] * len(axes)
        for new_axis, old_axis in enumerate(axes):
            inverse[old_axis] = new_axis
        return self._permute_inv(inverse)

    def _permute_inv(self, inverse) -> "Expr":
        if self.kind == "idx":
            return Expr.idx(inverse[self.a]) if self.a < len(inverse) else self
        return self._map(lambda e: e._permute_inv(inverse))

    def shift_idx(self, threshold: int, delta: int) -> "Expr":
        if self.kind == "idx":
            return Expr.idx(self.a + delta) if self.a >= threshold else self
        return self._map(lambda e: e.shift_idx(threshold, delta))

    def simplify(self) -> "Expr":
        k = self.kind
        if k == "add":
            l, r = self.a.simplify(), self.b.simplify()
            if l.kind == "const" and l.a == 0:
                return r
            if r.kind == "const" and r.a == 0:
                return l
            if l.kind == "const" and r.kind == "const":
                return Expr.const(l.a + r.a)
            return l + r
        if k == "sub":
            l, r = self.a.simplify(), self.b.simplify()
            if r.kind == "const" and r.a == 0:
                return l
            if l == r:
                return Expr.const(0)
            if l.kind == "const" and r.kind == "const":
                return Expr.const(l.a - r.a)
            if l.kind == "add" and l.b == r:
                return l.a
            if l.kind == "add" and l.a == r:
                return l.b
            if l.kind == "const" and l.a == 0 and r.kind == "sub":
                return (r.b - r.a).simplify()
            return l - r
        if k == "mul":
            l, r = self.a.simplify(), self.b.simplify()
            if (l.kind == "const" and l.a == 0) or (r.kind == "const" and r.a == 0):
                return Expr.const(0)
            if l.kind == "const" and l.a == 1:
                return r
            if r.kind == "const" and r.a == 1:
                return l
            if l.kind == "const" and l.a == -1:
                return (-r).simplify()
            if r.kind == "const" and r.a == -1:
                return (-l).simplify()
            if l.kind == "const" and r.kind == "const":
                return Expr.const(l.a * r.a)
            return l * r
        if k == "div":
            l, r = self.a.simplify(), self.b.simplify()
            if r.kind == "const" and r.a == 0:
                raise ZeroDivisionError("division by zero")
            if r.kind == "const" and r.a == 1:
                return l
            if l == r:
                return Expr.const(1)
            if l.kind == "const" and l.a == 0:
                return Expr.const(0)
            if l.kind == "const" and r.kind == "const":
                # Rust i64 division truncates toward zero
                q = abs(l.a) // abs(r.a)
                return Expr.const(q if (l.a >= 0) == (r.a >= 0) else -q)
            return l // r
        if k == "rem":
            l, r = self.a.simplify(), self.b.simplify()
            if r.kind == "const" and r.a == 0:
                raise ZeroDivisionError("division by zero")
            if r.kind == "const" and r.a == 1:
                return Expr.const(0)
            if l == r:
                return Expr.const(0)
            if l.kind == "const" and l.a == 0:
                return Expr.const(0)
            if l.kind == "const" and r.kind == "const":
                m = abs(l.a) % abs(r.a)
                return Expr.const(m if l.a >= 0 else -m)
            return l % r
        if k == "lt":
            l, r = self.a.simplify(), self.b.simplify()
            if l.kind == "const" and r.kind == "const":
                return Expr.const(1 if l.a < r.a else 0)
            if l == r:
                return Expr.const(0)
            return Expr("lt", l, r)
        if k == "and":
            l, r = self.a.simplify(), self.b.simplify()
            if l.kind == "bool" and l.a is True:
                return r
            if r.kind == "bool" and r.a is True:
                return l
            if (l.kind == "bool" and l.a is False) or (r.kind == "bool" and r.a is False):
                return Expr.boolean(False)
            if (l.kind == "const" and l.a == 0) or (r.kind == "const" and r.a == 0):
                return Expr.const(0)
            if l.kind == "const" and r.kind == "const":
                return Expr.const(1 if (l.a != 0 and r.a != 0) else 0)
            if l.kind == "const":
                return r
            if r.kind == "const":
                return l
            if l == r:
                return l
            if r.kind == "not" and r.a == l:
                return Expr.const(0)
            if l.kind == "not" and l.a == r:
                return Expr.const(0)
            return Expr("and", l, r)
        if k == "not":
            a = self.a.simplify()
            if a.kind == "bool":
                return Expr.boolean(not a.a)
            if a.kind == "const":
                return Expr.const(1 if a.a == 0 else 0)
            if a.kind == "not":
                return a.a
            return Expr("not", a)
        return self

    def __repr__(self):
        k = self.kind
        if k == "const":
            return str(self.a)
        if k == "bool":
            return "true" if self.a else "false"
        if k == "idx":
            return f"idx{self.a}"
        if k == "sym":
            return self.a
        if k == "not":
            return f"!({self.a})"
        sym = {"add": "+", "sub": "-", "mul": "*", "div": "/", "rem": "%",
               "lt": "<", "and": "&&"}[k]
        return f"({self.a} {sym} {self.b})"


def shape_of(dims: Sequence[ExprLike]) -> list:
    return [Expr.of(d) for d in dims]
