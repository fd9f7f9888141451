//! `AstNode` -> the s-expression text `libeclat_hip` reads.  Source only: never compiled.
//! One form per variant of `eclat::ast::AstNode`; float literals travel as IEEE bit patterns.

use eclat::ast::{AddressSpace, AstNode, DType, Literal, Mutability, VarDecl, VarKind};
use eclat::backend::device::ProgramBuffer;

/// A node the text form has no spelling for (`Allocate`, `Deallocate`, `CallKernel`,
/// `WmmaMatmul`, `src/ast/mod.rs:246-290`): compiling such a program is an error, not a panic.
pub type SerResult = Result<String, String>;

pub fn first_kernel_name(program: &AstNode) -> Option<String> {
    if let AstNode::Program { functions, .. } = program {
        for f in functions {
            if let AstNode::Kernel { name, .. } = f { return name.clone(); }
        }
    }
    None
}

pub fn dtype_text(d: &DType) -> String { dtype(d) }

fn dtype(d: &DType) -> String {
    match d {
        DType::Void => "void".into(), DType::Bool => "bool".into(),
        DType::I8 => "i8".into(), DType::I16 => "i16".into(), DType::I32 => "i32".into(), DType::I64 => "i64".into(),
        DType::U8 => "u8".into(), DType::U16 => "u16".into(), DType::U32 => "u32".into(), DType::U64 => "u64".into(),
        DType::F16 => "f16".into(), DType::BF16 => "bf16".into(), DType::F32 => "f32".into(), DType::F64 => "f64".into(),
        DType::Int => "int".into(), DType::Unknown => "unknown".into(),
        DType::Ptr(inner, space) => format!("(ptr {} {})", dtype(inner), match space {
            AddressSpace::Global => "global", AddressSpace::Shared => "shared",
            AddressSpace::Local => "local", AddressSpace::Constant => "constant" }),
        DType::Vec(inner, n) => format!("(vec {} {})", dtype(inner), n),
        DType::Tuple(_) => "unknown".into(),
    }
}

fn literal(l: &Literal) -> String {
    match l {
        Literal::Bool(v) => format!("(const bool {})", *v as u8),
        Literal::I8(v) => format!("(const i8 {v})"), Literal::I16(v) => format!("(const i16 {v})"),
        Literal::I32(v) => format!("(const i32 {v})"), Literal::I64(v) => format!("(const i64 {v})"),
        Literal::U8(v) => format!("(const u8 {v})"), Literal::U16(v) => format!("(const u16 {v})"),
        Literal::U32(v) => format!("(const u32 {v})"), Literal::U64(v) => format!("(const u64 {v})"),
        Literal::F32(v) => format!("(const f32 #{:08x})", v.to_bits()),
        Literal::F64(v) => format!("(const f64 #{:016x})", v.to_bits()),
        Literal::F16(v) => format!("(const f16 #{:08x})", v.to_f32().to_bits()),
        Literal::BF16(v) => format!("(const bf16 #{:08x})", v.to_f32().to_bits()),
    }
}

fn param(p: &VarDecl) -> String {
    let m = if matches!(p.mutability, Mutability::Mutable) { "mut" } else { "imm" };
    let k = match p.kind {
        VarKind::Normal => "normal".to_string(),
        VarKind::GroupId(a) => format!("(group_id {a})"), VarKind::LocalId(a) => format!("(local_id {a})"),
        VarKind::GroupSize(a) => format!("(group_size {a})"), VarKind::GridSize(a) => format!("(grid_size {a})"),
    };
    format!("(\"{}\" {} {} {})", p.name, dtype(&p.dtype), m, k)
}

fn list(op: &str, items: &[&AstNode]) -> SerResult {
    let mut s = format!("({op}");
    for i in items { s.push(' '); s.push_str(&to_text(i)?); }
    s.push(')');
    Ok(s)
}

/// `(buffers ("name" dtype (shape ...) role) ...)`: the table that lets the library compile the
/// program as a whole (fuse kernels, keep temporaries out of memory).
pub fn buffer_table(table: &[ProgramBuffer]) -> String {
    let mut s = String::from("(buffers");
    for b in table {
        let dims: Vec<String> = b.shape.iter().map(|d| d.to_string()).collect();
        s.push_str(&format!(" (\"{}\" {} (shape {}) {})", b.name, dtype(&b.dtype), dims.join(" "), b.role.as_str()));
    }
    s.push(')');
    s
}

/// A Program with its buffer table in front of the kernels.
pub fn program_text(kernels: &[AstNode], table: &[ProgramBuffer]) -> SerResult {
    let mut s = String::from("(program ");
    s.push_str(&buffer_table(table));
    for k in kernels { s.push(' '); s.push_str(&to_text(k)?); }
    s.push(')');
    Ok(s)
}

pub fn to_text(n: &AstNode) -> SerResult {
    use AstNode::*;
    Ok(match n {
        Wildcard(s) => format!("(wildcard \"{s}\")"),
        Const(l) => literal(l),
        Var(s) => format!("(var \"{s}\")"),
        Add(a, b) => list("add", &[a, b])?, Mul(a, b) => list("mul", &[a, b])?, Max(a, b) => list("max", &[a, b])?,
        Rem(a, b) => list("rem", &[a, b])?, Idiv(a, b) => list("idiv", &[a, b])?, Lt(a, b) => list("lt", &[a, b])?,
        And(a, b) => list("and", &[a, b])?, BitwiseAnd(a, b) => list("bitand", &[a, b])?,
        BitwiseOr(a, b) => list("bitor", &[a, b])?, BitwiseXor(a, b) => list("bitxor", &[a, b])?,
        LeftShift(a, b) => list("shl", &[a, b])?, RightShift(a, b) => list("shr", &[a, b])?,
        Recip(a) => list("recip", &[a])?, Sqrt(a) => list("sqrt", &[a])?, Log2(a) => list("log2", &[a])?,
        Exp2(a) => list("exp2", &[a])?, Sin(a) => list("sin", &[a])?, Floor(a) => list("floor", &[a])?,
        Not(a) => list("not", &[a])?, BitwiseNot(a) => list("bitnot", &[a])?,
        Cast(a, d) => format!("(cast {} {})", dtype(d), to_text(a)?),
        Fma { a, b, c } => list("fma", &[a, b, c])?,
        Select { cond, then_val, else_val } => list("select", &[cond, then_val, else_val])?,
        Load { ptr, offset, count, dtype: d } => format!("(load {} {} {} {})", to_text(ptr)?, to_text(offset)?, count, dtype(d)),
        Store { ptr, offset, value } => list("store", &[ptr, offset, value])?,
        Assign { var, value } => format!("(assign \"{var}\" {})", to_text(value)?),
        AtomicAdd { ptr, offset, value, dtype: d } =>
            format!("(atomic_add {} {} {} {})", to_text(ptr)?, to_text(offset)?, to_text(value)?, dtype(d)),
        AtomicMax { ptr, offset, value, dtype: d } =>
            format!("(atomic_max {} {} {} {})", to_text(ptr)?, to_text(offset)?, to_text(value)?, dtype(d)),
        Rand => "(rand)".into(),
        Barrier => "(barrier)".into(),
        Block { statements, scope } => {
            let mut s = String::from("(block (decls");
            for v in scope.local_variables() { s.push_str(&format!(" (\"{}\" {})", v.name, dtype(&v.dtype))); }
            s.push(')');
            for st in statements { s.push(' '); s.push_str(&to_text(st)?); }
            s.push(')');
            s
        }
        Range { var, start, step, stop, body, parallel } => {
            let kind = if parallel.is_parallel { format!("{:?}", parallel.kind).to_lowercase() } else { "sequential".into() };
            format!("(range \"{var}\" {} {} {} {} {kind})", to_text(start)?, to_text(step)?, to_text(stop)?, to_text(body)?)
        }
        If { condition, then_body, else_body } => match else_body {
            Some(e) => list("if", &[condition, then_body, e])?,
            None => list("if", &[condition, then_body])?,
        },
        Call { name, args } => {
            let mut s = format!("(call \"{name}\"");
            for a in args { s.push(' '); s.push_str(&to_text(a)?); }
            s.push(')');
            s
        }
        Return { value } => list("return", &[value])?,
        SharedAlloc { name, dtype: d, size } => format!("(shared_alloc \"{name}\" {} {})", dtype(d), to_text(size)?),
        SharedLoad { ptr, offset, dtype: d } => format!("(shared_load {} {} {})", to_text(ptr)?, to_text(offset)?, dtype(d)),
        SharedStore { ptr, offset, value } => list("shared_store", &[ptr, offset, value])?,
        Kernel { name, params, body, default_grid_size: g, default_thread_group_size: t, .. } => {
            let ps: Vec<String> = params.iter().map(param).collect();
            format!("(kernel \"{}\" (params {}) (grid {} {} {}) (tg {} {} {}) {})",
                    name.clone().unwrap_or_else(|| "kernel".into()), ps.join(" "),
                    to_text(&g[0])?, to_text(&g[1])?, to_text(&g[2])?,
                    to_text(&t[0])?, to_text(&t[1])?, to_text(&t[2])?, to_text(body)?)
        }
        Function { name, params, return_type, body } => {
            let ps: Vec<String> = params.iter().map(param).collect();
            format!("(function \"{}\" (params {}) (ret {}) {})", name.clone().unwrap_or_else(|| "anonymous".into()),
                    ps.join(" "), dtype(return_type), to_text(body)?)
        }
        Program { functions, .. } => {
            let mut s = String::from("(program");
            for f in functions { s.push(' '); s.push_str(&to_text(f)?); }
            s.push(')');
            s
        }
        other => return Err(format!("backend-hip: AST node has no text form: {other:?}")),
    })
}
