"""The AST optimisation stage of `execute_graph` (`pipeline.optimize`).

Host-side mirror of what the reference runs over the lowered Program before any
backend sees a kernel (`src/backend/executor.rs:169-176`,
`src/backend/compile.rs:246-265`; suggesters `compile.rs:326-337`):

* the algebraic rule set `all_algebraic_rules` (`src/opt/ast/rules/mod.rs:67-108`):
  constant folding (`rules/const_folding.rs`), identities and zero elements on
  integer literals (`rules/algebraic.rs:17-46`, `rules/macros.rs`), idempotent and
  inverse pairs (`algebraic.rs:52-100`), single-statement block unwrapping
  (`algebraic.rs:150-174`), multiplication by a power of two as a left shift
  (`rules/bit_ops.rs:19-83`), re-association of sums and products to the right
  (`algebraic.rs:113-127`);
* the loop transforms its suggesters draw from (`src/opt/ast/transforms.rs`):
  `tile_loop` (`:393-500`), `tile_loop_with_guard` (`:520-630`),
  `inline_small_loop` (`:238-361`), and loop interchange
  (`src/opt/ast/suggesters/loop_transforms.rs:710-793`).

The reference picks among these with a beam search over a static cost model
(`src/opt/ast/optimizer/beam_search.rs`); which candidates win can only be
learnt from a live run of the reference, so `optimize_program` applies the rule
set to a fixed point (every rule shrinks or normalises the tree) and applies
loop transforms only when asked to by name.  The transforms are here so that
tests can hand a backend every form the reference may send.
"""

from __future__ import annotations

import math
import os
from typing import Callable, List, Optional, Sequence

import numpy as np

from .ast import AstNode, I64, F32

_F32 = np.float32


# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------

def _is_const(n: AstNode, dtype_name: str = None) -> bool:
    return n.op == "const" and (dtype_name is None or n.attrs["dtype"].name == dtype_name)


def _is_i64(n: AstNode, value: int = None) -> bool:
    return _is_const(n, "i64") and (value is None or n.attrs["value"] == value)


def _rebuild(n: AstNode, args: Sequence[AstNode]) -> AstNode:
    return AstNode(n.op, args, **n.attrs)


def collect_var_names(n: AstNode) -> set:
    """transforms.rs:13-201: names of variables, loop variables, assignment targets, parameters."""
    names = set()
    for x in n.walk():
        if x.op in ("var", "range", "assign"):
            names.add(x.attrs["name"])
        if x.op in ("kernel", "function"):
            names.update(p.name for p in x.attrs["params"])
    return names


def find_next_ridx_names(used: set):
    """transforms.rs:206-219: the first three `ridxN` names not in `used`."""
    out, i = [], 0
    while len(out) < 3:
        name = f"ridx{i}"
        if name not in used:
            out.append(name)
        i += 1
    return tuple(out)


def replace_var(n: AstNode, name: str, by: AstNode) -> AstNode:
    """transforms.rs:645-: every Var(name) replaced."""
    if n.op == "var" and n.attrs["name"] == name:
        return by
    return _rebuild(n, [replace_var(a, name, by) for a in n.args])


# --------------------------------------------------------------------------
# loop transforms
# --------------------------------------------------------------------------

def tile_loop(loop: AstNode, tile: int) -> Optional[AstNode]:
    """transforms.rs:393-500.  `for v in s..e` becomes a block of
    `for o in s..(e/T)*T step T { for i in 0..T { v = o + i; body } }` and the remainder
    `for r in (e/T)*T..e { v = r; body }`; `v` is declared in both inner blocks."""
    if tile <= 1 or loop.op != "range":
        return None
    start, step, stop, body = loop.args
    if not _is_i64(step, 1):
        return None
    var = loop.attrs["name"]
    outer, inner, rem = find_next_ridx_names(collect_var_names(loop))
    c = AstNode.const_i64
    inner_body = AstNode.block([AstNode.assign(var, AstNode.add(AstNode.var(outer), AstNode.var(inner))), body],
                               decls=[(var, I64)])
    inner_loop = AstNode.range(inner, c(0), c(1), c(tile), inner_body)
    aligned = AstNode.mul(AstNode("idiv", [stop, c(tile)]), c(tile))
    outer_loop = AstNode.range(outer, start, c(tile), aligned, inner_loop)
    rem_body = AstNode.block([AstNode.assign(var, AstNode.var(rem)), body], decls=[(var, I64)])
    rem_loop = AstNode.range(rem, aligned, step, stop, rem_body)
    return AstNode.block([outer_loop, rem_loop])


def tile_loop_with_guard(loop: AstNode, tile: int) -> Optional[AstNode]:
    """transforms.rs:520-630.  `for o in 0..ceil(e/T) { for i in 0..T { v = o*T + i;
    if (v < e) { body } } }`; needs start 0 and step 1."""
    if tile <= 1 or loop.op != "range":
        return None
    start, step, stop, body = loop.args
    if not _is_i64(step, 1) or not _is_i64(start, 0):
        return None
    var = loop.attrs["name"]
    outer, inner, _ = find_next_ridx_names(collect_var_names(loop))
    c = AstNode.const_i64
    index = AstNode.add(AstNode.mul(AstNode.var(outer), c(tile)), AstNode.var(inner))
    guarded = AstNode("if", [AstNode.lt(AstNode.var(var), stop), body])
    inner_body = AstNode.block([AstNode.assign(var, index), guarded], decls=[(var, I64)])
    inner_loop = AstNode.range(inner, c(0), c(1), c(tile), inner_body)
    if _is_i64(stop):
        outer_stop = c(-(-stop.attrs["value"] // tile))
    else:
        outer_stop = AstNode("idiv", [AstNode.add(stop, c(tile - 1)), c(tile)])
    return AstNode.range(outer, c(0), c(1), outer_stop, inner_loop)


def inline_small_loop(loop: AstNode, max_iterations: int = 8) -> Optional[AstNode]:
    """transforms.rs:238-361.  A loop with constant bounds and at most `max_iterations`
    iterations becomes a block of its bodies with the variable replaced by each value; bodies
    that are blocks are flattened into it, and the block keeps the body's declarations."""
    if loop.op != "range":
        return None
    start, step, stop, body = loop.args
    if not (_is_i64(start) and _is_i64(step) and _is_i64(stop)) or step.attrs["value"] <= 0:
        return None
    s, st, e = start.attrs["value"], step.attrs["value"], stop.attrs["value"]
    if s >= e:
        return AstNode.block([])
    if -(-(e - s) // st) > max_iterations:
        return None
    stmts: List[AstNode] = []
    cur = s
    while cur < e:
        replaced = replace_var(body, loop.attrs["name"], AstNode.const_i64(cur))
        if replaced.op == "block":
            stmts.extend(replaced.args)
        else:
            stmts.append(replaced)
        cur += st
    decls = body.attrs.get("decls", []) if body.op == "block" else []
    return AstNode.block(stmts, decls=decls)


def interchange(loop: AstNode) -> Optional[AstNode]:
    """loop_transforms.rs:710-793: swaps a loop with the loop directly inside it (or inside its
    single-statement block)."""
    if loop.op != "range":
        return None
    body = loop.args[3]
    through_block = body.op == "block" and len(body.args) == 1 and body.args[0].op == "range"
    inner = body if body.op == "range" else body.args[0] if through_block else None
    if inner is None:
        return None
    new_inner = AstNode("range", list(loop.args[:3]) + [inner.args[3]], **loop.attrs)
    if through_block:
        new_inner = AstNode("block", [new_inner], **body.attrs)
    return AstNode("range", list(inner.args[:3]) + [new_inner], **inner.attrs)


def rewrite_loops(n: AstNode, pick: Callable[[AstNode], bool], f: Callable[[AstNode], Optional[AstNode]]) -> AstNode:
    """`n` with every loop `pick` accepts replaced by `f(loop)` (innermost first; loops `f`
    declines stay)."""
    args = [rewrite_loops(a, pick, f) for a in n.args]
    out = _rebuild(n, args)
    if out.op == "range" and pick(out):
        r = f(out)
        if r is not None:
            return r
    return out


def is_innermost(loop: AstNode) -> bool:
    return not any(x.op == "range" for x in loop.args[3].walk())


# --------------------------------------------------------------------------
# rewrite rules
# --------------------------------------------------------------------------

def _f32_const(v) -> AstNode:
    return AstNode("const", dtype=F32, value=float(_F32(v)))


def _fold(n: AstNode) -> Optional[AstNode]:
    """One application of a rule of `all_algebraic_rules` at the root of `n`, or None."""
    op, a = n.op, n.args
    # constant folding (rules/const_folding.rs:188-260)
    if op in ("add", "mul", "max") and _is_const(a[0]) and _is_const(a[1]):
        if _is_i64(a[0]) and _is_i64(a[1]):
            x, y = a[0].attrs["value"], a[1].attrs["value"]
            return AstNode.const_i64(x + y if op == "add" else x * y if op == "mul" else max(x, y))
        if _is_const(a[0], "f32") and _is_const(a[1], "f32"):
            x, y = _F32(a[0].attrs["value"]), _F32(a[1].attrs["value"])
            with np.errstate(all="ignore"):
                if op == "max":        # f32::max: a NaN operand yields the other one
                    r = y if np.isnan(x) else x if np.isnan(y) else max(x, y)
                else:
                    r = x + y if op == "add" else x * y
            return _f32_const(r)
    if op in ("rem", "idiv") and _is_i64(a[0]) and _is_i64(a[1]) and a[1].attrs["value"] != 0:
        x, y = a[0].attrs["value"], a[1].attrs["value"]
        q = abs(x) // abs(y) * (1 if (x >= 0) == (y >= 0) else -1)      # truncating, as Rust's / and %
        return AstNode.const_i64(q if op == "idiv" else x - q * y)
    if op in ("recip", "sqrt", "log2", "exp2", "sin") and _is_const(a[0], "f32"):
        v = _F32(a[0].attrs["value"])
        with np.errstate(all="ignore"):
            if op == "recip" and v != 0:
                return _f32_const(_F32(1.0) / v)
            if op == "sqrt" and v >= 0:
                return _f32_const(np.sqrt(v))
            if op == "log2" and v > 0:
                return _f32_const(np.log2(v))
            if op == "exp2":
                return _f32_const(np.exp2(v))
            if op == "sin":
                return _f32_const(np.sin(v))
    # identities and zero elements, integer literals only (rules/algebraic.rs:17-46)
    if op == "add":
        if _is_i64(a[1], 0):
            return a[0]
        if _is_i64(a[0], 0):
            return a[1]
    if op == "mul":
        if _is_i64(a[1], 1):
            return a[0]
        if _is_i64(a[0], 1):
            return a[1]
        if _is_i64(a[1], 0) or _is_i64(a[0], 0):
            return AstNode.const_i64(0)
    # idempotent and inverse pairs (algebraic.rs:52-100)
    if op == "max" and a[0] == a[1]:
        return a[0]
    if op == "recip" and a[0].op == "recip":
        return a[0].args[0]
    if op == "mul" and a[0].op == "sqrt" and a[1].op == "sqrt" and a[0].args[0] == a[1].args[0]:
        return a[0].args[0]
    if op == "log2" and a[0].op == "exp2":
        return a[0].args[0]
    if op == "exp2" and a[0].op == "log2":
        return a[0].args[0]
    # a block of one statement is that statement; its scope goes (algebraic.rs:150-174)
    if op == "block" and len(a) == 1:
        return a[0]
    # x * 2^n -> x << n, either side (rules/bit_ops.rs:19-83)
    if op == "mul":
        for x, k in ((a[0], a[1]), (a[1], a[0])):
            if _is_i64(k) and k.attrs["value"] > 0 and k.attrs["value"] & (k.attrs["value"] - 1) == 0:
                return AstNode("shl", [x, AstNode.const_i64(k.attrs["value"].bit_length() - 1)])
    # (a op b) op c -> a op (b op c) (algebraic.rs:113-127)
    if op in ("add", "mul") and a[0].op == op:
        return AstNode(op, [a[0].args[0], AstNode(op, [a[0].args[1], a[1]])])
    return None


def apply_rules(n: AstNode, max_passes: int = 64) -> AstNode:
    """The rule set applied bottom-up until nothing changes."""
    def once(x: AstNode) -> AstNode:
        x = _rebuild(x, [once(c) for c in x.args])
        for _ in range(max_passes):
            r = _fold(x)
            if r is None:
                return x
            x = _rebuild(r, [once(c) for c in r.args]) if r.args else r
        return x
    return once(n)


# --------------------------------------------------------------------------
# fused multiply-add rules (devices that report DeviceInstruction::Fma)
# --------------------------------------------------------------------------

def infer_type(n: AstNode) -> Optional[str]:
    """`AstNode::infer_type` (src/ast/mod.rs:781-860) as far as expressions go: a dtype name,
    or None for Unknown.  A variable's type is unknown (it depends on the context); a binary
    operation has its operands' type when they agree; a math function keeps its operand's type
    and is f32 when that is unknown."""
    op = n.op
    if op == "const":
        return n.attrs["dtype"].name
    if op == "cast":
        return n.attrs["dtype"].name
    if op == "load":
        return n.attrs["dtype"].name
    if op in ("var", "wildcard"):
        return None
    if op in ("add", "mul", "max", "rem", "idiv", "and", "or", "xor", "shl", "shr", "bitand", "bitor", "bitxor"):
        l, r = infer_type(n.args[0]), infer_type(n.args[1])
        return l if l == r else None
    if op in ("lt", "not", "logical_and"):
        return "bool"
    if op == "select":
        return infer_type(n.args[1])
    if op in ("recip", "sqrt", "log2", "exp2", "sin", "floor", "bitnot"):
        return infer_type(n.args[0]) or "f32"
    if op == "fma":
        return infer_type(n.args[0])
    return None


def _to_fma(n: AstNode) -> Optional[AstNode]:
    """`mul_add_to_fma` and `add_mul_to_fma` (src/opt/ast/rules/algebraic.rs:218-282):
    a * b + c and c + a * b become fma(a, b, c) when `a` infers to f32."""
    if n.op != "add":
        return None
    l, r = n.args
    if l.op == "mul" and infer_type(l.args[0]) == "f32":
        return AstNode("fma", [l.args[0], l.args[1], r])
    if r.op == "mul" and infer_type(r.args[0]) == "f32":
        return AstNode("fma", [r.args[0], r.args[1], l])
    return None


def apply_fma_rules(n: AstNode) -> AstNode:
    """`fma_rules` (src/opt/ast/rules/mod.rs:117-123) applied bottom-up, once per node: what
    `rules_for_capabilities` (:136-143) adds to the rule set for a device whose
    `supports_instruction(Fma)` is true, as `Pipeline::optimize_ast` uses it
    (src/backend/pipeline.rs:219-224)."""
    x = _rebuild(n, [apply_fma_rules(c) for c in n.args])
    r = _to_fma(x)
    return r if r is not None else x


# --------------------------------------------------------------------------
# the stage itself
# --------------------------------------------------------------------------

def optimize_kernel(kernel: AstNode, transforms: Sequence[str] = (), rules: bool = True) -> AstNode:
    """`kernel` after the named loop transforms and then the rule set.  Transform names:
    `tile=T` / `guard=T` (innermost loops), `tile_all=T` (every loop, innermost first),
    `tile_outer=T` (outermost loop only), `unroll` (loops of at most eight iterations, which
    after a tiling are the tile loops and the remainders), `interchange` (the outermost pair),
    `fma` (the multiply-add rules, applied after the rule set as the last step)."""
    body = kernel.args[0]
    for t in transforms:
        name, _, arg = t.partition("=")
        if name == "tile":
            body = rewrite_loops(body, is_innermost, lambda l: tile_loop(l, int(arg)))
        elif name == "guard":
            body = rewrite_loops(body, is_innermost, lambda l: tile_loop_with_guard(l, int(arg)))
        elif name == "tile_all":
            body = rewrite_loops(body, lambda l: True, lambda l: tile_loop(l, int(arg)))
        elif name == "tile_outer":
            outer = body
            while outer.op == "block" and len(outer.args) == 1:
                outer = outer.args[0]
            first = [outer]
            body = rewrite_loops(body, lambda l: l.to_sexpr() == first[0].to_sexpr(), lambda l: tile_loop(l, int(arg)))
        elif name == "unroll":
            body = rewrite_loops(body, lambda l: True, lambda l: inline_small_loop(l, 8))
        elif name == "interchange":
            done = [False]

            def swap(l):
                if done[0]:
                    return None
                r = interchange(l)
                done[0] = r is not None
                return r
            # outermost first: try the top loop, then go down
            def top_down(x: AstNode) -> AstNode:
                if x.op == "range":
                    r = swap(x)
                    if r is not None:
                        return r
                return _rebuild(x, [top_down(c) for c in x.args])
            body = top_down(body)
        elif name == "fma":
            pass
        elif name:
            raise ValueError(f"unknown loop transform '{t}'")
    if rules:
        body = apply_rules(body)
    if "fma" in transforms:
        body = apply_fma_rules(body)
    return AstNode("kernel", [body], **kernel.attrs)


def optimize_program(program: AstNode, level: Optional[int] = None, transforms: Sequence[str] = None) -> AstNode:
    """`pipeline.optimize(ast)` (compile.rs:246-265): level 0 returns the program as lowered;
    any other level applies the rule set, after the loop transforms named in `transforms` or in
    ECLAT_OPT_TRANSFORMS (comma-separated; none by default)."""
    if level is None:
        level = opt_level()
    if level == 0:
        return program
    if transforms is None:
        transforms = [t for t in os.environ.get("ECLAT_OPT_TRANSFORMS", "").split(",") if t]
    funcs = [optimize_kernel(f, transforms) if f.op == "kernel" else f for f in program.args]
    return AstNode("program", funcs, **program.attrs)


def opt_level() -> int:
    """ECLAT_OPT_LEVEL, 0-3, default 3 (executor.rs:169-173)."""
    try:
        v = int(os.environ.get("ECLAT_OPT_LEVEL", "3"))
    except ValueError:
        return 3
    return v if 0 <= v <= 255 else 3
