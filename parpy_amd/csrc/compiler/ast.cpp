// Constructors, structural equality and debug printers for the compiler AST.
#include "ast.hpp"

#include <sstream>

namespace parpy {

const char* elem_tag(ElemSize s) {
  switch (s) {
    case ElemSize::Bool: return "bool";
    case ElemSize::I8: return "i8";
    case ElemSize::I16: return "i16";
    case ElemSize::I32: return "i32";
    case ElemSize::I64: return "i64";
    case ElemSize::U8: return "u8";
    case ElemSize::U16: return "u16";
    case ElemSize::U32: return "u32";
    case ElemSize::U64: return "u64";
    case ElemSize::F16: return "f16";
    case ElemSize::F32: return "f32";
    case ElemSize::F64: return "f64";
  }
  return "?";
}

const char* elem_pyname(ElemSize s) {
  switch (s) {
    case ElemSize::Bool: return "bool";
    case ElemSize::I8: return "int8";
    case ElemSize::I16: return "int16";
    case ElemSize::I32: return "int32";
    case ElemSize::I64: return "int64";
    case ElemSize::U8: return "uint8";
    case ElemSize::U16: return "uint16";
    case ElemSize::U32: return "uint32";
    case ElemSize::U64: return "uint64";
    case ElemSize::F16: return "float16";
    case ElemSize::F32: return "float32";
    case ElemSize::F64: return "float64";
  }
  return "?";
}

// C type names of the emitted device code (reference: src/gpu/pprint.rs:9-27)
const char* elem_ctype(ElemSize s) {
  switch (s) {
    case ElemSize::Bool: return "bool";
    case ElemSize::I8: return "int8_t";
    case ElemSize::I16: return "int16_t";
    case ElemSize::I32: return "int32_t";
    case ElemSize::I64: return "int64_t";
    case ElemSize::U8: return "uint8_t";
    case ElemSize::U16: return "uint16_t";
    case ElemSize::U32: return "uint32_t";
    case ElemSize::U64: return "uint64_t";
    case ElemSize::F16: return "_Float16";
    case ElemSize::F32: return "float";
    case ElemSize::F64: return "double";
  }
  return "?";
}

bool parse_elem_tag(const std::string& t, ElemSize* out) {
  static const ElemSize all[] = {ElemSize::Bool, ElemSize::I8, ElemSize::I16, ElemSize::I32,
                                 ElemSize::I64, ElemSize::U8, ElemSize::U16, ElemSize::U32,
                                 ElemSize::U64, ElemSize::F16, ElemSize::F32, ElemSize::F64};
  for (auto s : all)
    if (t == elem_tag(s)) { *out = s; return true; }
  return false;
}

bool Type::operator==(const Type& o) const {
  if (k != o.k) return false;
  switch (k) {
    case Unknown: case Void: case Str: return true;
    case Tensor: return sz == o.sz && shape == o.shape;
    case Pointer: return sz == o.sz && mem == o.mem;
    case Dict:
      if (fields.size() != o.fields.size()) return false;
      for (size_t i = 0; i < fields.size(); ++i)
        if (fields[i].first != o.fields[i].first || fields[i].second != o.fields[i].second) return false;
      return true;
    case Tuple: return elems == o.elems;
  }
  return false;
}

std::string Type::str() const {
  std::ostringstream os;
  switch (k) {
    case Unknown: return "?";
    case Void: return "void";
    case Str: return "str";
    case Tensor:
      os << elem_pyname(sz);
      if (!shape.empty()) {
        os << "[";
        for (size_t i = 0; i < shape.size(); ++i) os << (i ? "," : "") << shape[i];
        os << "]";
      }
      return os.str();
    case Pointer: return std::string(elem_pyname(sz)) + (mem == Mem::LDS ? "*lds" : "*");
    case Dict:
      os << "{";
      for (size_t i = 0; i < fields.size(); ++i) os << (i ? ", " : "") << fields[i].first << ": " << fields[i].second.str();
      os << "}";
      return os.str();
    case Tuple:
      os << "(";
      for (size_t i = 0; i < elems.size(); ++i) os << (i ? ", " : "") << elems[i].str();
      os << ")";
      return os.str();
  }
  return "?";
}

const char* unop_name(UnOp op) {
  switch (op) {
    case UnOp::Sub: return "-";
    case UnOp::Not: return "!";
    case UnOp::BitNeg: return "~";
    case UnOp::Exp: return "exp";
    case UnOp::Log: return "log";
    case UnOp::Cos: return "cos";
    case UnOp::Sin: return "sin";
    case UnOp::Sqrt: return "sqrt";
    case UnOp::Tanh: return "tanh";
    case UnOp::Abs: return "abs";
  }
  return "?";
}

const char* binop_name(BinOp op) {
  switch (op) {
    case BinOp::Add: return "+";
    case BinOp::Sub: return "-";
    case BinOp::Mul: return "*";
    case BinOp::Div: return "/";
    case BinOp::FloorDiv: return "//";
    case BinOp::Rem: return "%";
    case BinOp::Pow: return "**";
    case BinOp::And: return "&&";
    case BinOp::Or: return "||";
    case BinOp::BitAnd: return "&";
    case BinOp::BitOr: return "|";
    case BinOp::BitXor: return "^";
    case BinOp::BitShl: return "<<";
    case BinOp::BitShr: return ">>";
    case BinOp::Eq: return "==";
    case BinOp::Neq: return "!=";
    case BinOp::Leq: return "<=";
    case BinOp::Geq: return ">=";
    case BinOp::Lt: return "<";
    case BinOp::Gt: return ">";
    case BinOp::Max: return "max";
    case BinOp::Min: return "min";
    case BinOp::Atan2: return "atan2";
  }
  return "?";
}

bool is_compare(BinOp op) { return op >= BinOp::Eq && op <= BinOp::Gt; }

bool LoopPar::try_merge(const LoopPar& o) {
  auto merge = [](int64_t l, int64_t r, int64_t dflt, int64_t* out) {
    if (l == dflt || l == r) { *out = r; return true; }
    if (r == dflt) { *out = l; return true; }
    return false;
  };
  int64_t n, t;
  if (!merge(nthreads, o.nthreads, 0, &n)) return false;
  if (!merge(tpb, o.tpb, DEFAULT_TPB, &t)) return false;
  nthreads = n;
  tpb = t;
  reduction = reduction || o.reduction;
  return true;
}

std::string LoopPar::str() const {
  std::ostringstream os;
  os << "{nthreads = " << nthreads << ", reduction = " << (reduction ? "true" : "false") << ", tpb = " << tpb << "}";
  return os.str();
}

// ---------------------------------------------------------------- constructors
static std::shared_ptr<Expr> new_expr(Expr::Kind k, const Type& ty, const Info& i) {
  auto e = std::make_shared<Expr>();
  e->k = k;
  e->ty = ty;
  e->i = i;
  return e;
}

E mk_var(const Name& n, const Type& ty, const Info& i) {
  auto e = new_expr(Expr::Var, ty, i);
  e->name = n;
  return e;
}
E mk_int(int64_t v, ElemSize sz, const Info& i) {
  auto e = new_expr(Expr::Int, Type::scalar(sz), i);
  e->iv = v;
  return e;
}
E mk_float(double v, ElemSize sz, const Info& i) {
  auto e = new_expr(Expr::Float, Type::scalar(sz), i);
  e->fv = v;
  return e;
}
E mk_bool(bool v, const Info& i) {
  auto e = new_expr(Expr::Bool, Type::scalar(ElemSize::Bool), i);
  e->bv = v;
  return e;
}
E mk_unop(UnOp op, E a, const Type& ty, const Info& i) {
  auto e = new_expr(Expr::UnOpE, ty, i);
  e->uop = op;
  e->args = {std::move(a)};
  return e;
}
E mk_binop(BinOp op, E a, E b, const Type& ty, const Info& i) {
  auto e = new_expr(Expr::BinOpE, ty, i);
  e->bop = op;
  e->args = {std::move(a), std::move(b)};
  return e;
}
E mk_convert(E a, ElemSize sz) {
  if (a->ty.is_scalar() && a->ty.sz == sz) return a;
  auto e = new_expr(Expr::Convert, Type::scalar(sz), a->i);
  e->args = {std::move(a)};
  return e;
}
E mk_index(E base, E idx, const Type& elem_ty, const Info& i) {
  auto e = new_expr(Expr::Index, elem_ty, i);
  e->args = {std::move(base), std::move(idx)};
  return e;
}
E mk_raw(const std::string& text, const Type& ty) {
  auto e = new_expr(Expr::Raw, ty, Info());
  e->sval = text;
  return e;
}
E mk_ifexpr(E c, E a, E b, const Type& ty, const Info& i) {
  auto e = new_expr(Expr::IfExpr, ty, i);
  e->args = {std::move(c), std::move(a), std::move(b)};
  return e;
}
E with_type(const E& e, const Type& ty) {
  if (e->ty == ty) return e;
  auto r = std::make_shared<Expr>(*e);
  r->ty = ty;
  return r;
}

bool expr_eq(const E& a, const E& b) {
  if (a == b) return true;
  if (!a || !b) return false;
  if (a->k != b->k || a->args.size() != b->args.size()) return false;
  switch (a->k) {
    case Expr::Var: case Expr::RegElem: if (a->name != b->name) return false; break;
    case Expr::Int: case Expr::ThreadIdx: case Expr::BlockIdx: if (a->iv != b->iv) return false; break;
    case Expr::Float:
      if (!(a->fv == b->fv || (std::isnan(a->fv) && std::isnan(b->fv)))) return false;
      break;
    case Expr::Bool: if (a->bv != b->bv) return false; break;
    case Expr::Str: case Expr::Call: case Expr::Raw: if (a->sval != b->sval) return false; break;
    case Expr::UnOpE: if (a->uop != b->uop) return false; break;
    case Expr::BinOpE: case Expr::NeutralElement: if (a->bop != b->bop) return false; break;
    case Expr::BuiltinE: if (a->fn != b->fn || a->has_axis != b->has_axis || a->iv != b->iv) return false; break;
    case Expr::Convert: if (a->ty != b->ty) return false; break;
    default: break;
  }
  if ((a->k == Expr::Int || a->k == Expr::Float) && a->ty != b->ty) return false;
  for (size_t i = 0; i < a->args.size(); ++i)
    if (!expr_eq(a->args[i], b->args[i])) return false;
  return true;
}

static std::shared_ptr<Stmt> new_stmt(Stmt::Kind k, const Info& i) {
  auto s = std::make_shared<Stmt>();
  s->k = k;
  s->i = i;
  return s;
}

S mk_def(const Name& id, const Type& ty, E expr, const Info& i) {
  auto s = new_stmt(Stmt::Def, i);
  s->id = id;
  s->ty = ty;
  s->expr = std::move(expr);
  return s;
}
S mk_assign(E dst, E expr, const Info& i) {
  auto s = new_stmt(Stmt::Assign, i);
  s->dst = std::move(dst);
  s->expr = std::move(expr);
  return s;
}
S mk_for(const Name& id, E lo, E hi, int64_t step, Stmts body, const LoopPar& par, const Info& i) {
  auto s = new_stmt(Stmt::For, i);
  s->id = id;
  s->lo = std::move(lo);
  s->hi = std::move(hi);
  s->step = step;
  s->body = std::move(body);
  s->par = par;
  return s;
}
S mk_if(E cond, Stmts thn, Stmts els, const Info& i) {
  auto s = new_stmt(Stmt::If, i);
  s->expr = std::move(cond);
  s->body = std::move(thn);
  s->els = std::move(els);
  return s;
}
S mk_sync() { return new_stmt(Stmt::Sync, Info()); }
S mk_scope(Stmts body) {
  auto s = new_stmt(Stmt::Scope, Info());
  s->body = std::move(body);
  return s;
}
S mk_rawstmt(const std::string& text) {
  auto s = new_stmt(Stmt::RawStmt, Info());
  s->fname = text;
  return s;
}

// ---------------------------------------------------------------- printers
static std::string fmt_double(double v) {
  if (std::isinf(v)) return v > 0 ? "inf" : "-inf";
  if (std::isnan(v)) return "nan";
  char buf[64];
  snprintf(buf, sizeof buf, "%.17g", v);
  return buf;
}

std::string print_expr(const E& e) {
  if (!e) return "<null>";
  std::ostringstream os;
  switch (e->k) {
    case Expr::Var: return e->name.str();
    case Expr::Int: return std::to_string(e->iv);
    case Expr::Float: return fmt_double(e->fv);
    case Expr::Bool: return e->bv ? "true" : "false";
    case Expr::Str: return "\"" + e->sval + "\"";
    case Expr::UnOpE: {
      std::string n = unop_name(e->uop);
      if (n.size() == 1) return "(" + n + print_expr(e->args[0]) + ")";
      return n + "(" + print_expr(e->args[0]) + ")";
    }
    case Expr::BinOpE: {
      std::string n = binop_name(e->bop);
      if (e->bop == BinOp::Max || e->bop == BinOp::Min || e->bop == BinOp::Atan2)
        return n + "(" + print_expr(e->args[0]) + ", " + print_expr(e->args[1]) + ")";
      return "(" + print_expr(e->args[0]) + " " + n + " " + print_expr(e->args[1]) + ")";
    }
    case Expr::IfExpr:
      return "(" + print_expr(e->args[1]) + " if " + print_expr(e->args[0]) + " else " + print_expr(e->args[2]) + ")";
    case Expr::Subscript: return print_expr(e->args[0]) + "[" + print_expr(e->args[1]) + "]";
    case Expr::Slice:
      return (e->args[0] ? print_expr(e->args[0]) : "") + ":" + (e->args[1] ? print_expr(e->args[1]) : "");
    case Expr::Tuple: {
      for (size_t i = 0; i < e->args.size(); ++i) os << (i ? ", " : "") << print_expr(e->args[i]);
      return os.str();
    }
    case Expr::BuiltinE: {
      static const char* names[] = {"exp", "inf", "log", "min", "max", "abs", "cos", "sin", "sqrt",
                                    "tanh", "atan2", "sum", "prod", "convert", "label", "gpu"};
      os << names[(int)e->fn];
      if (e->fn == Builtin::Convert) os << "<" << elem_pyname(e->ty.sz) << ">";
      if (e->fn == Builtin::Inf && e->args.empty()) return os.str();
      os << "(";
      for (size_t i = 0; i < e->args.size(); ++i) os << (i ? ", " : "") << print_expr(e->args[i]);
      if (e->has_axis) os << ", axis=" << e->iv;
      os << ")";
      return os.str();
    }
    case Expr::Call: {
      os << e->sval << "(";
      for (size_t i = 0; i < e->args.size(); ++i) os << (i ? ", " : "") << print_expr(e->args[i]);
      os << ")";
      return os.str();
    }
    case Expr::Convert: return std::string(elem_pyname(e->ty.sz)) + "(" + print_expr(e->args[0]) + ")";
    case Expr::NeutralElement: return std::string("neutral<") + binop_name(e->bop) + ">";
    case Expr::Index: return print_expr(e->args[0]) + "[" + print_expr(e->args[1]) + "]";
    case Expr::AddrOf: return "&" + print_expr(e->args[0]) + "[" + print_expr(e->args[1]) + "]";
    case Expr::ThreadIdx: return std::string("threadIdx.") + "xyz"[e->iv];
    case Expr::BlockIdx: return std::string("blockIdx.") + "xyz"[e->iv];
    case Expr::RegElem: return e->name.str() + "<" + print_expr(e->args[0]) + ">";
    case Expr::Raw: return e->sval;
  }
  return "?";
}

static void print_stmt(std::ostringstream& os, const S& s, int ind) {
  std::string pad(ind, ' ');
  auto labels = [&]() {
    if (s->labels.empty()) return std::string();
    std::string r = " [";
    for (size_t i = 0; i < s->labels.size(); ++i) r += (i ? ", " : "") + s->labels[i];
    return r + "]";
  };
  switch (s->k) {
    case Stmt::Def:
      os << pad << s->id.str() << " : " << s->ty.str() << " = " << print_expr(s->expr) << labels() << "\n";
      break;
    case Stmt::Assign:
      os << pad << print_expr(s->dst) << " = " << print_expr(s->expr) << labels() << "\n";
      break;
    case Stmt::For:
      os << pad << "for " << s->id.str() << " in range(" << print_expr(s->lo) << ", " << print_expr(s->hi) << ", "
         << s->step << ")" << labels();
      if (s->par.is_parallel() || s->par.reduction) os << " " << s->par.str();
      os << ":\n" << print_stmts(s->body, ind + 2);
      break;
    case Stmt::While:
      os << pad << "while " << print_expr(s->expr) << ":\n" << print_stmts(s->body, ind + 2);
      break;
    case Stmt::If:
      os << pad << "if " << print_expr(s->expr) << ":\n" << print_stmts(s->body, ind + 2);
      if (!s->els.empty()) os << pad << "else:\n" << print_stmts(s->els, ind + 2);
      break;
    case Stmt::WithGpu:
      os << pad << "with gpu:\n" << print_stmts(s->body, ind + 2);
      break;
    case Stmt::CallStmt: {
      os << pad << s->fname << "(";
      for (size_t i = 0; i < s->args.size(); ++i) os << (i ? ", " : "") << print_expr(s->args[i]);
      os << ")\n";
      break;
    }
    case Stmt::Label: os << pad << "label(" << s->fname << ")\n"; break;
    case Stmt::Return: os << pad << "return " << print_expr(s->expr) << "\n"; break;
    case Stmt::SyncPoint:
      os << pad << "<sync point: " << (s->sync == SyncKind::BlockLocal ? "block" : "inter-block") << ">\n";
      break;
    case Stmt::Sync: os << pad << "sync()\n"; break;
    case Stmt::Alloc: os << pad << s->id.str() << " = alloc<" << elem_pyname(s->ty.sz) << ">(" << s->iv << ")\n"; break;
    case Stmt::Free: os << pad << "free(" << s->id.str() << ")\n"; break;
    case Stmt::Launch: {
      os << pad << "launch " << s->fname << "<<<(" << s->grid.x << ", " << s->grid.y << ", " << s->grid.z << "), ("
         << s->block.x << ", " << s->block.y << ", " << s->block.z << ")>>>(";
      for (size_t i = 0; i < s->args.size(); ++i) os << (i ? ", " : "") << print_expr(s->args[i]);
      os << ")\n";
      break;
    }
    case Stmt::Scope: os << pad << "{\n" << print_stmts(s->body, ind + 2) << pad << "}\n"; break;
    case Stmt::WaveReduce: os << pad << s->id.str() << " = wave_reduce<" << binop_name(s->bop) << ">(" << s->id.str() << ")\n"; break;
    case Stmt::LdsDecl: os << pad << "lds " << elem_pyname(s->ty.sz) << " " << s->id.str() << "[" << s->iv << "]\n"; break;
    case Stmt::RegDecl: os << pad << "reg " << elem_pyname(s->ty.sz) << " " << s->id.str() << "[" << s->iv << "]\n"; break;
    case Stmt::RawStmt: os << pad << s->fname << "\n"; break;
  }
}

std::string print_stmts(const Stmts& ss, int indent) {
  std::ostringstream os;
  for (auto& s : ss) print_stmt(os, s, indent);
  return os.str();
}

std::string print_fun(const FunDef& f) {
  std::ostringstream os;
  os << "def " << f.id.s << "(";
  for (size_t i = 0; i < f.params.size(); ++i) {
    os << (i ? ", " : "") << f.params[i].id.str();
    if (f.params[i].ty.k != Type::Unknown) os << ": " << f.params[i].ty.str();
  }
  os << "):\n" << print_stmts(f.body, 2);
  return os.str();
}

}  // namespace parpy
