// Kernel-level AST as received from the host: the C++ image of the reference's
// AstNode / DType / Literal / VarDecl (src/ast/mod.rs:107-385, src/ast/types.rs:100-160,
// src/ast/scope.rs:8-41), plus the reader for its text form.
#pragma once

#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace eh {

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

enum class Ty : uint8_t {
  Void, Bool, I8, I16, I32, I64, U8, U16, U32, U64, F16, BF16, F32, F64, Int, Unknown, Ptr, Vec
};

struct DType {
  Ty ty = Ty::Unknown;
  std::shared_ptr<DType> inner;  // Ptr / Vec
  int extra = 0;                 // Ptr: address space (0 global,1 shared,2 local,3 constant); Vec: lanes

  bool is_ptr() const { return ty == Ty::Ptr; }
  bool is_float() const { return ty == Ty::F16 || ty == Ty::BF16 || ty == Ty::F32 || ty == Ty::F64; }
  const DType& elem() const { return inner ? *inner : *this; }
  size_t itemsize() const;
  std::string name() const;  // text form, e.g. "f32" or "(ptr f32 global)"
  bool operator==(const DType& o) const;
};

enum class Op : uint8_t {
  Const, Var, Wildcard,
  Add, Mul, Max, Rem, Idiv, Lt, And, BitAnd, BitOr, BitXor, Shl, Shr,
  Recip, Sqrt, Log2, Exp2, Sin, Floor, Not, BitNot,
  Cast, Fma, Select, Load, Store, Assign, AtomicAdd, AtomicMax,
  Block, Range, If, Barrier, Rand, Call, Return,
  SharedAlloc, SharedLoad, SharedStore, Allocate, Deallocate, WmmaMatmul,
  Kernel, Function, Program
};

const char* op_name(Op op);
bool is_binary(Op op);
bool is_unary(Op op);

enum class VarKind : uint8_t { Normal, GroupId, LocalId, GroupSize, GridSize };

struct Param {
  std::string name;
  DType dtype;
  bool mut_ = false;
  VarKind kind = VarKind::Normal;
  int axis = 0;
};

struct BufferInfo {
  std::string name;
  DType dtype;
  std::vector<int64_t> shape;
  std::string role;  // input | output | temp | ones | zeros
  bool shape_known = true;  // false when the program came without a buffer table
  size_t numel() const {
    size_t n = 1;
    for (auto d : shape) n *= static_cast<size_t>(d);
    return n;
  }
  size_t bytes() const { return numel() * dtype.itemsize(); }
};

struct Node;
using NodePtr = std::shared_ptr<Node>;

struct Node {
  Op op;
  std::vector<NodePtr> args;
  std::string name;          // Var/Wildcard/Assign/Range var/Call/Kernel/SharedAlloc
  DType dtype;               // Const/Cast/Load/Atomic*/SharedAlloc/...; Function: return type
  DType dtype2;              // WmmaMatmul: accumulator type
  // literal payload (Const)
  int64_t ival = 0;
  double fval = 0.0;         // value of float literals (f32 literals hold the exact f32 value)
  int count = 1;             // Load lanes
  std::string parallel;      // Range: sequential | openmp | gpu_thread | rayon
  std::vector<std::pair<std::string, DType>> decls;  // Block scope variables
  std::vector<Param> params;                         // Kernel / Function
  std::vector<NodePtr> grid, tg;                     // Kernel dispatch hints
  std::vector<BufferInfo> buffers;                   // Program buffer table (optional)

  explicit Node(Op o) : op(o) {}
};

NodePtr make(Op op, std::vector<NodePtr> args = {});
NodePtr make_var(const std::string& name);
NodePtr make_i64(int64_t v);

// Parses the text form; throws eh::Error with position info on malformed input.
NodePtr parse_ast(const std::string& text);
// Writes the text form back (round-trips parse_ast output).
std::string to_text(const Node& n);
DType parse_dtype_text(const std::string& text);

}  // namespace eh
