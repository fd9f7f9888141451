// Text reader/writer for the kernel AST.
#include "ast.hpp"

#include <cmath>
#include <cstring>
#include <map>
#include <sstream>

namespace eh {

namespace {

struct OpInfo {
  Op op;
  const char* name;
  int arity;  // -1: variadic / special
};

const OpInfo kOps[] = {
    {Op::Const, "const", -1},       {Op::Var, "var", -1},           {Op::Wildcard, "wildcard", -1},
    {Op::Add, "add", 2},            {Op::Mul, "mul", 2},            {Op::Max, "max", 2},
    {Op::Rem, "rem", 2},            {Op::Idiv, "idiv", 2},          {Op::Lt, "lt", 2},
    {Op::And, "and", 2},            {Op::BitAnd, "bitand", 2},      {Op::BitOr, "bitor", 2},
    {Op::BitXor, "bitxor", 2},      {Op::Shl, "shl", 2},            {Op::Shr, "shr", 2},
    {Op::Recip, "recip", 1},        {Op::Sqrt, "sqrt", 1},          {Op::Log2, "log2", 1},
    {Op::Exp2, "exp2", 1},          {Op::Sin, "sin", 1},            {Op::Floor, "floor", 1},
    {Op::Not, "not", 1},            {Op::BitNot, "bitnot", 1},      {Op::Cast, "cast", -1},
    {Op::Fma, "fma", 3},            {Op::Select, "select", 3},      {Op::Load, "load", -1},
    {Op::Store, "store", 3},        {Op::Assign, "assign", -1},     {Op::AtomicAdd, "atomic_add", -1},
    {Op::AtomicMax, "atomic_max", -1}, {Op::Block, "block", -1},    {Op::Range, "range", -1},
    {Op::If, "if", -1},             {Op::Barrier, "barrier", 0},    {Op::Rand, "rand", 0},
    {Op::Call, "call", -1},         {Op::Return, "return", 1},      {Op::SharedAlloc, "shared_alloc", -1},
    {Op::SharedLoad, "shared_load", -1}, {Op::SharedStore, "shared_store", 3},
    {Op::Allocate, "allocate", -1}, {Op::Deallocate, "deallocate", 1},
    {Op::WmmaMatmul, "wmma_matmul", -1}, {Op::Kernel, "kernel", -1}, {Op::Function, "function", -1},
    {Op::Program, "program", -1},
};

const std::map<std::string, Ty>& ty_names() {
  static const std::map<std::string, Ty> m = {
      {"void", Ty::Void}, {"bool", Ty::Bool}, {"i8", Ty::I8},   {"i16", Ty::I16}, {"i32", Ty::I32},
      {"i64", Ty::I64},   {"u8", Ty::U8},     {"u16", Ty::U16}, {"u32", Ty::U32}, {"u64", Ty::U64},
      {"f16", Ty::F16},   {"bf16", Ty::BF16}, {"f32", Ty::F32}, {"f64", Ty::F64}, {"int", Ty::Int},
      {"unknown", Ty::Unknown}};
  return m;
}

const char* kSpaces[] = {"global", "shared", "local", "constant"};

// ---- tokenizer -------------------------------------------------------------
struct Tok {
  enum Kind { LP, RP, Atom, Str, End } kind;
  std::string text;
  size_t pos;
};

struct Lexer {
  const std::string& s;
  size_t i = 0;
  explicit Lexer(const std::string& src) : s(src) {}
  Tok next() {
    while (i < s.size() && isspace(static_cast<unsigned char>(s[i]))) ++i;
    if (i >= s.size()) return {Tok::End, "", i};
    size_t p = i;
    char c = s[i];
    if (c == '(') { ++i; return {Tok::LP, "(", p}; }
    if (c == ')') { ++i; return {Tok::RP, ")", p}; }
    if (c == '"') {
      size_t j = s.find('"', i + 1);
      if (j == std::string::npos) throw Error("AST text: unterminated string at " + std::to_string(p));
      std::string t = s.substr(i + 1, j - i - 1);
      i = j + 1;
      return {Tok::Str, t, p};
    }
    size_t j = i;
    while (j < s.size() && !isspace(static_cast<unsigned char>(s[j])) && s[j] != '(' && s[j] != ')' &&
           s[j] != '"')
      ++j;
    std::string t = s.substr(i, j - i);
    i = j;
    return {Tok::Atom, t, p};
  }
};

// generic s-expression tree
struct SX {
  bool is_list = false;
  bool is_str = false;
  std::string atom;
  std::vector<SX> items;
  size_t pos = 0;
};

SX read_sx(Lexer& lx, Tok t) {
  SX r;
  r.pos = t.pos;
  if (t.kind == Tok::LP) {
    r.is_list = true;
    for (;;) {
      Tok n = lx.next();
      if (n.kind == Tok::RP) break;
      if (n.kind == Tok::End) throw Error("AST text: missing ')' for list opened at " + std::to_string(t.pos));
      r.items.push_back(read_sx(lx, n));
    }
    return r;
  }
  if (t.kind == Tok::RP) throw Error("AST text: unexpected ')' at " + std::to_string(t.pos));
  if (t.kind == Tok::End) throw Error("AST text: unexpected end of input");
  r.atom = t.text;
  r.is_str = (t.kind == Tok::Str);
  return r;
}

[[noreturn]] void fail(const SX& s, const std::string& msg) {
  throw Error("AST text: " + msg + " (at offset " + std::to_string(s.pos) + ")");
}

const std::string& head(const SX& s) {
  if (!s.is_list || s.items.empty() || s.items[0].is_list) fail(s, "expected (op ...)");
  return s.items[0].atom;
}

DType to_dtype(const SX& s) {
  DType d;
  if (!s.is_list) {
    auto it = ty_names().find(s.atom);
    if (it == ty_names().end()) fail(s, "unknown dtype '" + s.atom + "'");
    d.ty = it->second;
    return d;
  }
  const std::string& h = head(s);
  if (h == "ptr") {
    if (s.items.size() != 3) fail(s, "ptr needs (ptr <dtype> <space>)");
    d.ty = Ty::Ptr;
    d.inner = std::make_shared<DType>(to_dtype(s.items[1]));
    d.extra = -1;
    for (int i = 0; i < 4; ++i)
      if (s.items[2].atom == kSpaces[i]) d.extra = i;
    if (d.extra < 0) fail(s, "unknown address space '" + s.items[2].atom + "'");
    return d;
  }
  if (h == "vec") {
    if (s.items.size() != 3) fail(s, "vec needs (vec <dtype> <n>)");
    d.ty = Ty::Vec;
    d.inner = std::make_shared<DType>(to_dtype(s.items[1]));
    d.extra = std::stoi(s.items[2].atom);
    return d;
  }
  fail(s, "unknown composite dtype '" + h + "'");
}

int64_t to_int(const SX& s) {
  if (s.is_list) fail(s, "expected integer");
  try {
    size_t used = 0;
    long long v = std::stoll(s.atom, &used, 10);
    if (used != s.atom.size()) fail(s, "bad integer '" + s.atom + "'");
    return v;
  } catch (const std::logic_error&) {
    // u64 literals above i64::MAX
    try {
      return static_cast<int64_t>(std::stoull(s.atom));
    } catch (const std::logic_error&) {
      fail(s, "bad integer '" + s.atom + "'");
    }
  }
}

double to_float(const SX& s, bool bits32) {
  const std::string& a = s.atom;
  if (a == "nan") return std::nan("");
  if (a == "inf") return INFINITY;
  if (a == "-inf") return -INFINITY;
  if (!a.empty() && a[0] == '#') {
    uint64_t bits = 0;
    try {
      size_t used = 0;
      bits = std::stoull(a.substr(1), &used, 16);
      if (used + 1 != a.size()) fail(s, "bad float bit pattern '" + a + "'");
    } catch (const std::logic_error&) {
      fail(s, "bad float bit pattern '" + a + "'");
    }
    if (bits32) {
      uint32_t b = static_cast<uint32_t>(bits);
      float f;
      std::memcpy(&f, &b, 4);
      return f;
    }
    double d;
    std::memcpy(&d, &bits, 8);
    return d;
  }
  try {
    return std::stod(a);
  } catch (const std::logic_error&) {
    fail(s, "bad float literal '" + a + "'");
  }
}

NodePtr to_node(const SX& s);

std::vector<Param> to_params(const SX& s) {
  if (!s.is_list || head(s) != "params") fail(s, "expected (params ...)");
  std::vector<Param> out;
  for (size_t i = 1; i < s.items.size(); ++i) {
    const SX& p = s.items[i];
    if (!p.is_list || p.items.size() != 4) fail(p, "param needs (\"name\" dtype imm|mut kind)");
    Param q;
    q.name = p.items[0].atom;
    q.dtype = to_dtype(p.items[1]);
    if (p.items[2].atom == "mut") q.mut_ = true;
    else if (p.items[2].atom != "imm") fail(p, "mutability must be imm or mut");
    const SX& k = p.items[3];
    if (!k.is_list) {
      if (k.atom != "normal") fail(k, "unknown param kind '" + k.atom + "'");
    } else {
      const std::string& kh = head(k);
      if (kh == "group_id") q.kind = VarKind::GroupId;
      else if (kh == "local_id") q.kind = VarKind::LocalId;
      else if (kh == "group_size") q.kind = VarKind::GroupSize;
      else if (kh == "grid_size") q.kind = VarKind::GridSize;
      else fail(k, "unknown param kind '" + kh + "'");
      q.axis = static_cast<int>(to_int(k.items.at(1)));
    }
    out.push_back(std::move(q));
  }
  return out;
}

NodePtr to_node(const SX& s) {
  const std::string& h = head(s);
  const OpInfo* info = nullptr;
  for (const auto& o : kOps)
    if (h == o.name) info = &o;
  if (!info) fail(s, "unknown AST node '" + h + "'");
  auto n = std::make_shared<Node>(info->op);
  const auto& it = s.items;
  auto need = [&](size_t k) {
    if (it.size() != k + 1) fail(s, "'" + h + "' takes " + std::to_string(k) + " operands");
  };
  if (info->arity >= 0) {
    need(static_cast<size_t>(info->arity));
    for (size_t i = 1; i < it.size(); ++i) n->args.push_back(to_node(it[i]));
    return n;
  }
  switch (info->op) {
    case Op::Const: {
      need(2);
      n->dtype = to_dtype(it[1]);
      if (n->dtype.is_float()) {
        n->fval = to_float(it[2], n->dtype.ty != Ty::F64);
      } else {
        n->ival = to_int(it[2]);
        n->fval = static_cast<double>(n->ival);
      }
      break;
    }
    case Op::Var:
    case Op::Wildcard:
      need(1);
      n->name = it[1].atom;
      break;
    case Op::Cast:
      need(2);
      n->dtype = to_dtype(it[1]);
      n->args.push_back(to_node(it[2]));
      break;
    case Op::Load:
      need(4);
      n->args.push_back(to_node(it[1]));
      n->args.push_back(to_node(it[2]));
      n->count = static_cast<int>(to_int(it[3]));
      n->dtype = to_dtype(it[4]);
      break;
    case Op::SharedLoad:
      need(3);
      n->args.push_back(to_node(it[1]));
      n->args.push_back(to_node(it[2]));
      n->dtype = to_dtype(it[3]);
      break;
    case Op::SharedAlloc:
      need(3);
      n->name = it[1].atom;
      n->dtype = to_dtype(it[2]);
      n->args.push_back(to_node(it[3]));
      break;
    case Op::Allocate:
      need(2);
      n->dtype = to_dtype(it[1]);
      n->args.push_back(to_node(it[2]));
      break;
    case Op::Assign:
      need(2);
      n->name = it[1].atom;
      n->args.push_back(to_node(it[2]));
      break;
    case Op::AtomicAdd:
    case Op::AtomicMax:
      need(4);
      for (int i = 1; i <= 3; ++i) n->args.push_back(to_node(it[i]));
      n->dtype = to_dtype(it[4]);
      break;
    case Op::Block: {
      if (it.size() < 2 || !it[1].is_list || head(it[1]) != "decls") fail(s, "block needs (decls ...) first");
      for (size_t i = 1; i < it[1].items.size(); ++i) {
        const SX& d = it[1].items[i];
        if (!d.is_list || d.items.size() != 2) fail(d, "decl needs (\"name\" dtype)");
        n->decls.emplace_back(d.items[0].atom, to_dtype(d.items[1]));
      }
      for (size_t i = 2; i < it.size(); ++i) n->args.push_back(to_node(it[i]));
      break;
    }
    case Op::Range: {
      if (it.size() != 6 && it.size() != 7) fail(s, "range needs (range \"v\" start step stop body [kind])");
      n->name = it[1].atom;
      for (int i = 2; i <= 5; ++i) n->args.push_back(to_node(it[i]));
      n->parallel = it.size() == 7 ? it[6].atom : "sequential";
      break;
    }
    case Op::If:
      if (it.size() != 3 && it.size() != 4) fail(s, "if needs (if cond then [else])");
      for (size_t i = 1; i < it.size(); ++i) n->args.push_back(to_node(it[i]));
      break;
    case Op::Call:
      if (it.size() < 2) fail(s, "call needs a name");
      n->name = it[1].atom;
      for (size_t i = 2; i < it.size(); ++i) n->args.push_back(to_node(it[i]));
      break;
    case Op::WmmaMatmul:
      need(14);
      for (int i = 1; i <= 12; ++i) n->args.push_back(to_node(it[i]));
      n->dtype = to_dtype(it[13]);
      n->dtype2 = to_dtype(it[14]);
      break;
    case Op::Kernel:
    case Op::Function: {
      if (it.size() < 4) fail(s, "kernel/function needs a name, params and a body");
      n->name = it[1].atom;
      n->params = to_params(it[2]);
      n->dtype.ty = Ty::Void;
      for (size_t i = 3; i + 1 < it.size(); ++i) {
        const std::string& sh = head(it[i]);
        if (sh == "grid" || sh == "tg") {
          if (it[i].items.size() != 4) fail(it[i], sh + " needs three sizes");
          auto& dst = sh == "grid" ? n->grid : n->tg;
          for (int k = 1; k <= 3; ++k) dst.push_back(to_node(it[i].items[k]));
        } else if (sh == "ret") {
          n->dtype = to_dtype(it[i].items.at(1));
        } else {
          fail(it[i], "unexpected section '" + sh + "'");
        }
      }
      n->args.push_back(to_node(it.back()));
      break;
    }
    case Op::Program: {
      for (size_t i = 1; i < it.size(); ++i) {
        const std::string& sh = head(it[i]);
        if (sh == "buffers") {
          for (size_t k = 1; k < it[i].items.size(); ++k) {
            const SX& b = it[i].items[k];
            if (!b.is_list || b.items.size() != 4) fail(b, "buffer needs (\"name\" dtype (shape ...) role)");
            BufferInfo bi;
            bi.name = b.items[0].atom;
            bi.dtype = to_dtype(b.items[1]);
            if (!b.items[2].is_list || head(b.items[2]) != "shape") fail(b, "expected (shape ...)");
            for (size_t d = 1; d < b.items[2].items.size(); ++d) {
              int64_t v = to_int(b.items[2].items[d]);
              if (v < 0) fail(b, "negative dimension");
              bi.shape.push_back(v);
            }
            bi.role = b.items[3].atom;
            if (bi.role != "input" && bi.role != "output" && bi.role != "temp" && bi.role != "ones" &&
                bi.role != "zeros")
              fail(b, "role must be input, output, temp, ones or zeros");
            n->buffers.push_back(std::move(bi));
          }
        } else {
          n->args.push_back(to_node(it[i]));
        }
      }
      break;
    }
    default:
      fail(s, "unhandled node '" + h + "'");
  }
  return n;
}

}  // namespace

size_t DType::itemsize() const {
  switch (ty) {
    case Ty::Bool: case Ty::I8: case Ty::U8: return 1;
    case Ty::I16: case Ty::U16: case Ty::F16: case Ty::BF16: return 2;
    case Ty::I32: case Ty::U32: case Ty::F32: return 4;
    case Ty::I64: case Ty::U64: case Ty::F64: case Ty::Int: case Ty::Ptr: return 8;
    case Ty::Vec: return inner->itemsize() * static_cast<size_t>(extra);
    default: throw Error("dtype '" + name() + "' has no size");
  }
}

std::string DType::name() const {
  if (ty == Ty::Ptr) return "(ptr " + inner->name() + " " + kSpaces[extra] + ")";
  if (ty == Ty::Vec) return "(vec " + inner->name() + " " + std::to_string(extra) + ")";
  for (const auto& kv : ty_names())
    if (kv.second == ty) return kv.first;
  return "unknown";
}

bool DType::operator==(const DType& o) const {
  if (ty != o.ty || extra != o.extra) return false;
  if (static_cast<bool>(inner) != static_cast<bool>(o.inner)) return false;
  return !inner || *inner == *o.inner;
}

const char* op_name(Op op) {
  for (const auto& o : kOps)
    if (o.op == op) return o.name;
  return "?";
}

bool is_binary(Op op) {
  for (const auto& o : kOps)
    if (o.op == op) return o.arity == 2;
  return false;
}

bool is_unary(Op op) {
  for (const auto& o : kOps)
    if (o.op == op) return o.arity == 1 && op != Op::Return && op != Op::Deallocate;
  return false;
}

NodePtr make(Op op, std::vector<NodePtr> args) {
  auto n = std::make_shared<Node>(op);
  n->args = std::move(args);
  return n;
}

NodePtr make_var(const std::string& name) {
  auto n = std::make_shared<Node>(Op::Var);
  n->name = name;
  return n;
}

NodePtr make_i64(int64_t v) {
  auto n = std::make_shared<Node>(Op::Const);
  n->dtype.ty = Ty::I64;
  n->ival = v;
  n->fval = static_cast<double>(v);
  return n;
}

NodePtr parse_ast(const std::string& text) {
  Lexer lx(text);
  SX root = read_sx(lx, lx.next());
  if (lx.next().kind != Tok::End) throw Error("AST text: trailing input after the top-level form");
  return to_node(root);
}

DType parse_dtype_text(const std::string& text) {
  Lexer lx(text);
  return to_dtype(read_sx(lx, lx.next()));
}

static void write_float(std::ostringstream& os, const Node& n) {
  if (std::isnan(n.fval)) { os << "nan"; return; }
  if (std::isinf(n.fval)) { os << (n.fval > 0 ? "inf" : "-inf"); return; }
  char buf[32];
  if (n.dtype.ty == Ty::F64) {
    uint64_t b;
    std::memcpy(&b, &n.fval, 8);
    snprintf(buf, sizeof buf, "#%016llx", static_cast<unsigned long long>(b));
  } else {
    float f = static_cast<float>(n.fval);
    uint32_t b;
    std::memcpy(&b, &f, 4);
    snprintf(buf, sizeof buf, "#%08x", b);
  }
  os << buf;
}

static void write(std::ostringstream& os, const Node& n) {
  os << "(" << op_name(n.op);
  auto kids = [&]() {
    for (const auto& a : n.args) { os << " "; write(os, *a); }
  };
  switch (n.op) {
    case Op::Const:
      os << " " << n.dtype.name() << " ";
      if (n.dtype.is_float()) write_float(os, n);
      else os << n.ival;
      break;
    case Op::Var: case Op::Wildcard:
      os << " \"" << n.name << "\"";
      break;
    case Op::Cast: case Op::Allocate:
      os << " " << n.dtype.name();
      kids();
      break;
    case Op::Load:
      kids();
      os << " " << n.count << " " << n.dtype.name();
      break;
    case Op::SharedLoad: case Op::AtomicAdd: case Op::AtomicMax:
      kids();
      os << " " << n.dtype.name();
      break;
    case Op::SharedAlloc:
      os << " \"" << n.name << "\" " << n.dtype.name();
      kids();
      break;
    case Op::Assign: case Op::Call:
      os << " \"" << n.name << "\"";
      kids();
      break;
    case Op::Block:
      os << " (decls";
      for (const auto& d : n.decls) os << " (\"" << d.first << "\" " << d.second.name() << ")";
      os << ")";
      kids();
      break;
    case Op::Range:
      os << " \"" << n.name << "\"";
      kids();
      os << " " << (n.parallel.empty() ? "sequential" : n.parallel);
      break;
    case Op::WmmaMatmul:
      kids();
      os << " " << n.dtype.name() << " " << n.dtype2.name();
      break;
    case Op::Kernel: case Op::Function: {
      os << " \"" << n.name << "\" (params";
      for (const auto& p : n.params) {
        os << " (\"" << p.name << "\" " << p.dtype.name() << " " << (p.mut_ ? "mut" : "imm") << " ";
        static const char* kn[] = {"normal", "group_id", "local_id", "group_size", "grid_size"};
        if (p.kind == VarKind::Normal) os << "normal";
        else os << "(" << kn[static_cast<int>(p.kind)] << " " << p.axis << ")";
        os << ")";
      }
      os << ")";
      if (n.op == Op::Kernel) {
        if (n.grid.size() == 3) { os << " (grid"; for (auto& g : n.grid) { os << " "; write(os, *g); } os << ")"; }
        if (n.tg.size() == 3) { os << " (tg"; for (auto& g : n.tg) { os << " "; write(os, *g); } os << ")"; }
      } else {
        os << " (ret " << n.dtype.name() << ")";
      }
      kids();
      break;
    }
    case Op::Program:
      if (!n.buffers.empty()) {
        os << " (buffers";
        for (const auto& b : n.buffers) {
          os << " (\"" << b.name << "\" " << b.dtype.name() << " (shape";
          for (auto d : b.shape) os << " " << d;
          os << ") " << b.role << ")";
        }
        os << ")";
      }
      kids();
      break;
    default:
      kids();
  }
  os << ")";
}

std::string to_text(const Node& n) {
  std::ostringstream os;
  write(os, n);
  return os.str();
}

}  // namespace eh
