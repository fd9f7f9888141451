"""AST text -> C99 source, as the reference's C backend renders it
(test infrastructure; see package docstring).

Follows `CLikeRenderer` in `src/backend/renderer.rs` -- `render_literal`
`:182-265`, `render_expr` `:268-441`, `render_statement` `:444-573`,
`render_block` `:604-624`, `render_range` `:627-660`,
`render_program_clike` `:715-771`, `render_function_node` `:774-847` -- with
the `CRenderer` overrides of `crates/backend-c/src/renderer.rs:117-224`
(type names, header, `fmaxf/sqrtf/log2f/exp2f/sinf/floorf`, sequential
atomics) and the default `fma(a, b, c)` of `src/backend/renderer.rs:107-109`.
"""

from __future__ import annotations

import math
import struct

import numpy as np

from .sexpr import Str, parse

HEADER = ("/* Generated C code by Harp */\n"
          "/* This code is pure C99 without parallelization */\n\n"
          "#include <math.h>\n#include <stdlib.h>\n#include <stdint.h>\n\n")

_CTYPE = {"void": "void", "bool": "unsigned char", "i8": "signed char", "i16": "short",
          "i32": "int", "i64": "long long", "u8": "unsigned char", "u16": "unsigned short",
          "u32": "unsigned int", "u64": "unsigned long long", "f16": "_Float16",
          "bf16": "__bf16", "f32": "float", "f64": "double", "int": "long long",
          "unknown": "/* unknown */"}

_MATH = {"max": "fmaxf", "min": "fminf", "sqrt": "sqrtf", "log2": "log2f",
         "exp2": "exp2f", "sin": "sinf", "floor": "floorf"}

_INFIX = {"add": "+", "mul": "*", "rem": "%", "idiv": "/", "lt": "<", "and": "&&",
          "bitand": "&", "bitor": "|", "bitxor": "^", "shl": "<<", "shr": ">>"}


def render_dtype(dt) -> str:
    if isinstance(dt, list):
        if dt[0] == "ptr":
            return render_dtype(dt[1]) + "*"
        if dt[0] == "vec":
            return f"{render_dtype(dt[1])}[{dt[2]}]"
        raise ValueError(dt)
    return _CTYPE[dt]


def _decode_float(tok: str, bits32: bool) -> float:
    if tok.startswith("#"):
        if bits32:
            return struct.unpack("<f", struct.pack("<I", int(tok[1:], 16)))[0]
        return struct.unpack("<d", struct.pack("<Q", int(tok[1:], 16)))[0]
    return float(tok)


def _rust_display_f32(v: float) -> str:
    """Rust's `{}` for f32: shortest digits that round-trip, never scientific."""
    s = np.format_float_positional(np.float32(v), unique=True, trim="-")
    return s


def render_literal(dt: str, tok: str) -> str:
    if dt in ("f32", "f16", "bf16"):
        v = _decode_float(tok, True)
        cast = {"f32": "", "f16": "(half)", "bf16": "(bfloat)"}[dt]
        if math.isnan(v):
            return cast + "NAN"
        if math.isinf(v):
            return cast + ("INFINITY" if v > 0 else "(-INFINITY)")
        s = _rust_display_f32(v)
        if dt != "f32":
            return f"{cast}{s}f"
        if "." not in s and "e" not in s and "E" not in s:
            return s + ".0f"
        return s + "f"
    if dt == "f64":
        v = _decode_float(tok, False)
        if math.isnan(v):
            return "NAN"
        if math.isinf(v):
            return "INFINITY" if v > 0 else "(-INFINITY)"
        s = np.format_float_positional(np.float64(v), unique=True, trim="-")
        return s if "." in s else s + ".0"
    if dt == "bool":
        return "1" if int(tok) else "0"
    if dt in ("u8", "u16", "u32"):
        return f"{int(tok)}u"
    if dt == "u64":
        return f"{int(tok)}ull"
    return str(int(tok))


class CRenderer:
    def __init__(self):
        self.level = 0

    def indent(self) -> str:
        return " " * (4 * self.level)

    # -- expressions -------------------------------------------------------
    def expr(self, n) -> str:
        op = n[0]
        if op == "const":
            return render_literal(n[1], n[2])
        if op in ("var", "wildcard"):
            return str(n[1])
        if op in _INFIX:
            return f"({self.expr(n[1])} {_INFIX[op]} {self.expr(n[2])})"
        if op == "max":
            return f"fmaxf({self.expr(n[1])}, {self.expr(n[2])})"
        if op == "recip":
            return f"(1.0f / {self.expr(n[1])})"
        if op in ("sqrt", "log2", "exp2", "sin", "floor"):
            return f"{_MATH[op]}({self.expr(n[1])})"
        if op == "rand":
            return "((float)rand() / (float)RAND_MAX)"
        if op == "bitnot":
            return f"(~{self.expr(n[1])})"
        if op == "not":
            return f"(!{self.expr(n[1])})"
        if op == "select":
            return f"({self.expr(n[1])} ? {self.expr(n[2])} : {self.expr(n[3])})"
        if op == "cast":
            return f"({render_dtype(n[1])})({self.expr(n[2])})"
        if op == "load":
            if int(n[3]) == 1:
                return f"{self.expr(n[1])}[{self.expr(n[2])}]"
            return f"*reinterpret_cast<{render_dtype(n[4])} *>(&{self.expr(n[1])}[{self.expr(n[2])}])"
        if op == "call":
            return f"{n[1]}({', '.join(self.expr(a) for a in n[2:])})"
        if op == "return":
            return f"return {self.expr(n[1])}"
        if op == "fma":
            return f"fma({self.expr(n[1])}, {self.expr(n[2])}, {self.expr(n[3])})"
        if op == "atomic_add":
            return (f"/* atomic_add (sequential) */ ({self.expr(n[1])}[{self.expr(n[2])}] "
                    f"+= {self.expr(n[3])})")
        if op == "atomic_max":
            p, o, v = self.expr(n[1]), self.expr(n[2]), self.expr(n[3])
            return (f"/* atomic_max (sequential) */ ({{float __tmp = {p}[{o}]; "
                    f"{p}[{o}] = __tmp > {v} ? __tmp : {v}; __tmp;}})")
        if op == "shared_load":
            return f"{self.expr(n[1])}[{self.expr(n[2])}]"
        return f"/* unsupported expression: {op} */"

    # -- statements -----------------------------------------------------------
    def stmt(self, n) -> str:
        op = n[0]
        ind = self.indent()
        if op == "store":
            return f"{ind}{self.expr(n[1])}[{self.expr(n[2])}] = {self.expr(n[3])};"
        if op == "assign":
            return f"{ind}{n[1]} = {self.expr(n[2])};"
        if op == "block":
            out = ""
            for name, dt in n[1][1:]:
                out += f"{ind}{render_dtype(dt)} {name};\n"
            for s in n[2:]:
                out += self.stmt(s) + "\n"
            return out
        if op == "range":
            var, start, step, stop, body = n[1], n[2], n[3], n[4], n[5]
            out = (f"{ind}for (long long {var} = {self.expr(start)}; {var} < "
                   f"{self.expr(stop)}; {var} += {self.expr(step)}) {{\n")
            self.level += 1
            b = self.stmt(body)
            out += b
            if not b.endswith("\n"):
                out += "\n"
            self.level -= 1
            return out + f"{self.indent()}}}"
        if op == "if":
            out = f"{ind}if ({self.expr(n[1])}) {{\n"
            self.level += 1
            t = self.stmt(n[2])
            out += t + ("" if t.endswith("\n") else "\n")
            self.level -= 1
            out += f"{self.indent()}}}"
            if len(n) > 3:
                out += " else {\n"
                self.level += 1
                e = self.stmt(n[3])
                out += e + ("" if e.endswith("\n") else "\n")
                self.level -= 1
                out += f"{self.indent()}}}"
            return out
        if op == "return":
            return f"{ind}return {self.expr(n[1])};"
        if op == "barrier":
            return f"{ind}/* barrier (no-op in sequential C) */"
        if op == "shared_alloc":
            return f"{ind}{render_dtype(n[2])}* {n[1]} = 0; // shared alloc size={self.expr(n[3])}"
        if op == "shared_store":
            return f"{ind}{self.expr(n[1])}[{self.expr(n[2])}] = {self.expr(n[3])};"
        if op == "wmma_matmul":
            return f"{ind}/* WMMA matmul not supported on this backend */"
        return f"{ind}{self.expr(n)};"

    # -- functions / program --------------------------------------------------------
    def function(self, f) -> str:
        name = f[1]
        params = f[2][1:]
        body = f[-1]
        ret = "void"
        for item in f[3:-1]:
            if isinstance(item, list) and item and item[0] == "ret":
                ret = render_dtype(item[1])
        ps = ", ".join(f"{render_dtype(p[1])} {p[0]}" for p in params)
        out = f"{ret} {name}({ps}) {{\n"
        self.level += 1
        b = self.stmt(body)
        out += b + ("" if b.endswith("\n") else "\n")
        self.level -= 1
        return out + f"{self.indent()}}}\n"

    def program(self, tree) -> str:
        assert tree[0] == "program"
        funcs = [x for x in tree[1:] if isinstance(x, list) and x[0] in ("kernel", "function")]
        kernels = sorted((f for f in funcs if f[0] == "kernel"), key=lambda f: f[1])
        helpers = sorted((f for f in funcs if f[0] == "function"), key=lambda f: f[1])
        out = HEADER
        if kernels:
            out += "// === Kernel Functions ===\n"
            for f in kernels:
                out += self.function(f) + "\n"
        if helpers:
            out += "// === Helper Functions ===\n"
            for f in helpers:
                out += self.function(f) + "\n"
        return out


def render_program(ast_text: str) -> str:
    return CRenderer().program(parse(ast_text))


def render_expr(ast_text: str) -> str:
    return CRenderer().expr(parse(ast_text))
