"""Kernel-level AST: the data model handed to a backend's `compile_ast`.

Host-side mirror of the reference's `src/ast/mod.rs:107-385` (node variants),
`src/ast/types.rs:100-160` (DType, Literal) and `src/ast/scope.rs:8-41`
(VarDecl, Mutability, VarKind).  `to_sexpr` is the text form the C-ABI
library parses; it carries every field a renderer needs.
"""

from __future__ import annotations

import math
import struct
from typing import Dict, List, Optional, Sequence, Tuple

from .expr import Expr

# --------------------------------------------------------------------------
# DType
# --------------------------------------------------------------------------

SCALAR_DTYPES = ("void", "bool", "i8", "i16", "i32", "i64", "u8", "u16", "u32",
                 "u64", "f16", "bf16", "f32", "f64", "int", "unknown")


class DType:
    """Scalar dtype name, or a composite ('ptr', inner, space) / ('vec', inner, n)."""

    __slots__ = ("name", "inner", "extra")

    def __init__(self, name: str, inner: Optional["DType"] = None, extra=None):
        self.name = name
        self.inner = inner
        self.extra = extra

    @staticmethod
    def ptr(inner: "DType", space: str = "global") -> "DType":
        return DType("ptr", inner, space)

    @staticmethod
    def vec(inner: "DType", n: int) -> "DType":
        return DType("vec", inner, n)

    def is_ptr(self) -> bool:
        return self.name == "ptr"

    def is_float(self) -> bool:
        return self.name in ("f16", "bf16", "f32", "f64")

    def itemsize(self) -> int:
        return {"bool": 1, "i8": 1, "u8": 1, "i16": 2, "u16": 2, "f16": 2, "bf16": 2,
                "i32": 4, "u32": 4, "f32": 4, "i64": 8, "u64": 8, "f64": 8,
                "int": 8}[self.name]

    def __eq__(self, o):
        return (isinstance(o, DType) and self.name == o.name and self.inner == o.inner
                and self.extra == o.extra)

    def __hash__(self):
        return hash((self.name, self.inner, self.extra))

    def to_sexpr(self) -> str:
        if self.name == "ptr":
            return f"(ptr {self.inner.to_sexpr()} {self.extra})"
        if self.name == "vec":
            return f"(vec {self.inner.to_sexpr()} {self.extra})"
        return self.name

    def __repr__(self):
        return self.to_sexpr()


F32 = DType("f32")
F64 = DType("f64")
I32 = DType("i32")
I64 = DType("i64")
BOOL = DType("bool")
VOID = DType("void")
INT = DType("int")


def _fmt_float(v: float, bits32: bool) -> str:
    if math.isnan(v):
        return "nan"
    if math.isinf(v):
        return "inf" if v > 0 else "-inf"
    if bits32:
        # exact: the IEEE-754 bit pattern, so no decimal round trip is involved
        return "#%08x" % struct.unpack("<I", struct.pack("<f", v))[0]
    return "#%016x" % struct.unpack("<Q", struct.pack("<d", v))[0]


# --------------------------------------------------------------------------
# AstNode
# --------------------------------------------------------------------------

BINARY = ("add", "mul", "max", "rem", "idiv", "lt", "and", "bitand", "bitor",
          "bitxor", "shl", "shr")
UNARY = ("recip", "sqrt", "log2", "exp2", "sin", "floor", "not", "bitnot")


class VarDecl:
    """Function/kernel parameter or block-scope variable (scope.rs:8-13)."""

    __slots__ = ("name", "dtype", "mutable", "kind", "axis")

    def __init__(self, name: str, dtype: DType, mutable: bool = False,
                 kind: str = "normal", axis: int = 0):
        self.name = name
        self.dtype = dtype
        self.mutable = mutable
        self.kind = kind          # normal | group_id | local_id | group_size | grid_size
        self.axis = axis

    def to_sexpr(self) -> str:
        k = self.kind if self.kind == "normal" else f"({self.kind} {self.axis})"
        return f'("{self.name}" {self.dtype.to_sexpr()} {"mut" if self.mutable else "imm"} {k})'


class AstNode:
    """Tagged tree node.  `op` names follow the reference's variant names in
    snake_case; `args` are child nodes; `attrs` holds the non-node fields."""

    __slots__ = ("op", "args", "attrs")

    def __init__(self, op: str, args: Sequence["AstNode"] = (), **attrs):
        self.op = op
        self.args = list(args)
        self.attrs = attrs

    # -- constructors mirroring the reference's helper functions --------
    @staticmethod
    def const_f32(v: float) -> "AstNode":
        v32 = struct.unpack("<f", struct.pack("<f", v))[0]
        return AstNode("const", dtype=F32, value=v32)

    @staticmethod
    def const_i64(v: int) -> "AstNode":
        return AstNode("const", dtype=I64, value=int(v))

    @staticmethod
    def const(dtype: DType, v) -> "AstNode":
        return AstNode("const", dtype=dtype, value=v)

    @staticmethod
    def var(name: str) -> "AstNode":
        return AstNode("var", name=name)

    @staticmethod
    def wildcard(name: str) -> "AstNode":
        return AstNode("wildcard", name=name)

    @staticmethod
    def binary(op: str, a: "AstNode", b: "AstNode") -> "AstNode":
        assert op in BINARY, op
        return AstNode(op, [a, b])

    @staticmethod
    def unary(op: str, a: "AstNode") -> "AstNode":
        assert op in UNARY, op
        return AstNode(op, [a])

    @staticmethod
    def add(a, b): return AstNode("add", [a, b])
    @staticmethod
    def mul(a, b): return AstNode("mul", [a, b])
    @staticmethod
    def max(a, b): return AstNode("max", [a, b])
    @staticmethod
    def lt(a, b): return AstNode("lt", [a, b])
    @staticmethod
    def recip(a): return AstNode("recip", [a])

    @staticmethod
    def select(c, t, e): return AstNode("select", [c, t, e])

    @staticmethod
    def cast(a, dtype: DType): return AstNode("cast", [a], dtype=dtype)

    @staticmethod
    def load(ptr, offset, dtype: DType, count: int = 1):
        return AstNode("load", [ptr, offset], dtype=dtype, count=count)

    @staticmethod
    def store(ptr, offset, value): return AstNode("store", [ptr, offset, value])

    @staticmethod
    def assign(name: str, value): return AstNode("assign", [value], name=name)

    @staticmethod
    def atomic_add(ptr, offset, value, dtype: DType):
        return AstNode("atomic_add", [ptr, offset, value], dtype=dtype)

    @staticmethod
    def block(stmts: Sequence["AstNode"], decls: Sequence[Tuple[str, DType]] = ()):
        return AstNode("block", stmts, decls=list(decls))

    @staticmethod
    def range(var: str, start, step, stop, body, parallel: str = "sequential"):
        return AstNode("range", [start, step, stop, body], name=var, parallel=parallel)

    @staticmethod
    def kernel(name: str, params: Sequence[VarDecl], body, grid=None, tg=None):
        one = AstNode.const_i64(1)
        return AstNode("kernel", [body], name=name, params=list(params),
                       return_type=VOID, grid=list(grid or [one, one, one]),
                       tg=list(tg or [one, one, one]))

    @staticmethod
    def program(functions: Sequence["AstNode"], buffers=None):
        return AstNode("program", functions, buffers=buffers)

    # -- traversal -------------------------------------------------------
    def substitute(self, mapping: Dict[str, "AstNode"]) -> "AstNode":
        """Replace Wildcard(name) by mapping[name] (AstNode::substitute)."""
        if self.op == "wildcard":
            return mapping.get(self.attrs["name"], self)
        return AstNode(self.op, [a.substitute(mapping) for a in self.args], **self.attrs)

    def walk(self):
        yield self
        for a in self.args:
            yield from a.walk()

    def __eq__(self, o):
        return isinstance(o, AstNode) and self.to_sexpr() == o.to_sexpr()

    def __hash__(self):
        return hash(self.to_sexpr())

    # -- text form ---------------------------------------------------------
    def to_sexpr(self) -> str:
        op, a, at = self.op, self.args, self.attrs
        if op == "const":
            dt: DType = at["dtype"]
            v = at["value"]
            if dt.name in ("f32", "f16", "bf16"):
                return f"(const {dt.name} {_fmt_float(v, True)})"
            if dt.name == "f64":
                return f"(const f64 {_fmt_float(v, False)})"
            if dt.name == "bool":
                return f"(const bool {1 if v else 0})"
            return f"(const {dt.name} {int(v)})"
        if op in ("var", "wildcard"):
            return f'({op} "{at["name"]}")'
        if op in BINARY or op in UNARY or op in ("select", "fma", "store", "if",
                                                 "return", "shared_store", "deallocate"):
            return "(" + " ".join([op] + [x.to_sexpr() for x in a]) + ")"
        if op == "cast":
            return f"(cast {at['dtype'].to_sexpr()} {a[0].to_sexpr()})"
        if op == "load":
            return (f"(load {a[0].to_sexpr()} {a[1].to_sexpr()} {at['count']} "
                    f"{at['dtype'].to_sexpr()})")
        if op == "shared_load":
            return f"(shared_load {a[0].to_sexpr()} {a[1].to_sexpr()} {at['dtype'].to_sexpr()})"
        if op == "shared_alloc":
            return f'(shared_alloc "{at["name"]}" {at["dtype"].to_sexpr()} {a[0].to_sexpr()})'
        if op == "allocate":
            return f"(allocate {at['dtype'].to_sexpr()} {a[0].to_sexpr()})"
        if op in ("atomic_add", "atomic_max"):
            return ("(" + " ".join([op] + [x.to_sexpr() for x in a]) +
                    f" {at['dtype'].to_sexpr()})")
        if op == "assign":
            return f'(assign "{at["name"]}" {a[0].to_sexpr()})'
        if op == "block":
            decls = " ".join(f'("{n}" {d.to_sexpr()})' for n, d in at.get("decls", []))
            body = " ".join(x.to_sexpr() for x in a)
            return f"(block (decls {decls}) {body})".replace("  ", " ")
        if op == "range":
            return (f'(range "{at["name"]}" {a[0].to_sexpr()} {a[1].to_sexpr()} '
                    f'{a[2].to_sexpr()} {a[3].to_sexpr()} {at.get("parallel", "sequential")})')
        if op in ("barrier", "rand"):
            return f"({op})"
        if op == "call":
            return '(call "%s" %s)' % (at["name"], " ".join(x.to_sexpr() for x in a))
        if op in ("kernel", "function"):
            params = " ".join(p.to_sexpr() for p in at["params"])
            head = f'({op} "{at["name"]}" (params {params})'
            if op == "kernel":
                g = " ".join(x.to_sexpr() for x in at["grid"])
                t = " ".join(x.to_sexpr() for x in at["tg"])
                head += f" (grid {g}) (tg {t})"
            else:
                head += f" (ret {at['return_type'].to_sexpr()})"
            return head + " " + a[0].to_sexpr() + ")"
        if op == "program":
            parts = ["(program"]
            bufs = at.get("buffers")
            if bufs:
                items = " ".join(
                    f'("{b["name"]}" {b["dtype"].to_sexpr()} (shape {" ".join(str(d) for d in b["shape"])}) {b["role"]})'
                    for b in bufs)
                parts.append(f"(buffers {items})")
            parts += [f.to_sexpr() for f in a]
            return " ".join(parts) + ")"
        if op == "wmma_matmul":
            return ("(wmma_matmul " + " ".join(x.to_sexpr() for x in a) +
                    f" {at['dtype_ab'].to_sexpr()} {at['dtype_c'].to_sexpr()})")
        raise ValueError(f"cannot serialise AST node '{op}'")

    def __repr__(self):
        return self.to_sexpr()


def expr_to_ast(expr: Expr) -> AstNode:
    """`impl From<Expr> for AstNode` (expr.rs:62-105): simplify, then map
    Idx(i) -> Var("ridx{i}"), a-b -> a + (-1 * b), a/b -> a * recip(b)."""
    return _expr_to_ast(expr.simplify())


def _expr_to_ast(e: Expr) -> AstNode:
    # every sub-conversion re-simplifies, as the recursive `.into()` does
    e = e.simplify()
    k = e.kind
    if k == "const":
        return AstNode.const_i64(e.a)
    if k == "bool":
        return AstNode.const_i64(1 if e.a else 0)
    if k == "idx":
        return AstNode.var(f"ridx{e.a}")
    if k == "sym":
        return AstNode.var(e.a)
    if k == "add":
        return AstNode.add(_expr_to_ast(e.a), _expr_to_ast(e.b))
    if k == "sub":
        return AstNode.add(_expr_to_ast(e.a),
                           AstNode.mul(AstNode.const_i64(-1), _expr_to_ast(e.b)))
    if k == "mul":
        return AstNode.mul(_expr_to_ast(e.a), _expr_to_ast(e.b))
    if k == "div":
        return AstNode.mul(_expr_to_ast(e.a), AstNode.recip(_expr_to_ast(e.b)))
    if k == "rem":
        return AstNode("rem", [_expr_to_ast(e.a), _expr_to_ast(e.b)])
    if k == "lt":
        return AstNode.lt(_expr_to_ast(e.a), _expr_to_ast(e.b))
    if k == "and":
        return AstNode("and", [_expr_to_ast(e.a), _expr_to_ast(e.b)])
    if k == "not":
        return AstNode("not", [_expr_to_ast(e.a)])
    raise ValueError(f"cannot convert {e} to AstNode")
