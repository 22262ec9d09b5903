// Constant folding, reduction neutral elements and integer interval analysis.
//
// Folding follows src/utils/constant_fold.rs:139-292 of the reference: integer
// `//` and `%` fold with truncating division (equal to Python's for the
// non-negative operands index arithmetic produces); transcendental calls are
// never folded so that host-side folding cannot differ from the device
// intrinsics.
#include <cmath>
#include <limits>

#include "passes.hpp"

namespace parpy {

namespace {

int64_t wrap_int(int64_t v, const Type& ty) {
  if (ty.k != Type::Tensor) return v;
  switch (ty.sz) {
    case ElemSize::I8: return (int8_t)v;
    case ElemSize::I16: return (int16_t)v;
    case ElemSize::I32: return (int32_t)v;
    case ElemSize::U8: return (uint8_t)v;
    case ElemSize::U16: return (uint16_t)v;
    case ElemSize::U32: return (uint32_t)v;
    default: return v;
  }
}

double round_float(double v, const Type& ty) {
  if (ty.k == Type::Tensor && ty.sz == ElemSize::F32) return (double)(float)v;
  if (ty.k == Type::Tensor && ty.sz == ElemSize::F16) return (double)(float)v;  // half literals are rounded when emitted
  return v;
}

E lit_int(int64_t v, const Type& ty, const Info& i) {
  auto e = std::make_shared<Expr>();
  e->k = Expr::Int;
  e->ty = ty;
  e->i = i;
  e->iv = wrap_int(v, ty);
  return e;
}
E lit_float(double v, const Type& ty, const Info& i) {
  auto e = std::make_shared<Expr>();
  e->k = Expr::Float;
  e->ty = ty;
  e->i = i;
  e->fv = round_float(v, ty);
  return e;
}
E lit_bool(bool v, const Info& i) { return mk_bool(v, i); }

bool is_int_lit(const E& e, int64_t v) { return e->k == Expr::Int && e->iv == v; }

E fold_binop(const E& e, const E& a, const E& b) {
  const Type& ty = e->ty;
  BinOp op = e->bop;
  if (a->k == Expr::Int && b->k == Expr::Int) {
    int64_t x = a->iv, y = b->iv;
    Type rty = ty.k == Type::Unknown ? a->ty : ty;
    switch (op) {
      case BinOp::Add: return lit_int(x + y, rty, e->i);
      case BinOp::Sub: return lit_int(x - y, rty, e->i);
      case BinOp::Mul: return lit_int(x * y, rty, e->i);
      case BinOp::FloorDiv: if (y != 0) return lit_int(x / y, rty, e->i); break;
      case BinOp::Div: if (y != 0 && ty.k == Type::Tensor && is_int(ty.sz)) return lit_int(x / y, rty, e->i); break;
      case BinOp::Rem: if (y != 0) return lit_int(x % y, rty, e->i); break;
      case BinOp::BitAnd: return lit_int(x & y, rty, e->i);
      case BinOp::BitOr: return lit_int(x | y, rty, e->i);
      case BinOp::BitXor: return lit_int(x ^ y, rty, e->i);
      case BinOp::BitShl: if (y >= 0 && y < 63) return lit_int(x << y, rty, e->i); break;
      case BinOp::BitShr: if (y >= 0 && y < 63) return lit_int(x >> y, rty, e->i); break;
      case BinOp::Max: return lit_int(x > y ? x : y, rty, e->i);
      case BinOp::Min: return lit_int(x < y ? x : y, rty, e->i);
      case BinOp::Eq: return lit_bool(x == y, e->i);
      case BinOp::Neq: return lit_bool(x != y, e->i);
      case BinOp::Leq: return lit_bool(x <= y, e->i);
      case BinOp::Geq: return lit_bool(x >= y, e->i);
      case BinOp::Lt: return lit_bool(x < y, e->i);
      case BinOp::Gt: return lit_bool(x > y, e->i);
      default: break;
    }
  }
  if (a->k == Expr::Float && b->k == Expr::Float) {
    double x = a->fv, y = b->fv;
    Type rty = ty.k == Type::Unknown ? a->ty : ty;
    switch (op) {
      case BinOp::Add: return lit_float(x + y, rty, e->i);
      case BinOp::Sub: return lit_float(x - y, rty, e->i);
      case BinOp::Mul: return lit_float(x * y, rty, e->i);
      case BinOp::Div: return lit_float(x / y, rty, e->i);
      case BinOp::Max: return lit_float(std::fmax(x, y), rty, e->i);
      case BinOp::Min: return lit_float(std::fmin(x, y), rty, e->i);
      case BinOp::Eq: return lit_bool(x == y, e->i);
      case BinOp::Neq: return lit_bool(x != y, e->i);
      case BinOp::Leq: return lit_bool(x <= y, e->i);
      case BinOp::Geq: return lit_bool(x >= y, e->i);
      case BinOp::Lt: return lit_bool(x < y, e->i);
      case BinOp::Gt: return lit_bool(x > y, e->i);
      default: break;
    }
  }
  if (a->k == Expr::Bool && b->k == Expr::Bool) {
    switch (op) {
      case BinOp::And: return lit_bool(a->bv && b->bv, e->i);
      case BinOp::Or: return lit_bool(a->bv || b->bv, e->i);
      case BinOp::Eq: return lit_bool(a->bv == b->bv, e->i);
      case BinOp::Neq: return lit_bool(a->bv != b->bv, e->i);
      default: break;
    }
  }
  // integer identities (index arithmetic); floats are left alone to keep NaN/-0 semantics
  bool int_ty = (ty.k == Type::Tensor && is_int(ty.sz)) ||
                (ty.k == Type::Unknown && (a->k == Expr::Int || b->k == Expr::Int));
  if (int_ty) {
    bool same = ty.k == Type::Unknown || (a->ty == ty && b->ty == ty);
    if (same) {
      if (op == BinOp::Add && is_int_lit(a, 0)) return b;
      if ((op == BinOp::Add || op == BinOp::Sub) && is_int_lit(b, 0)) return a;
      if (op == BinOp::Mul && is_int_lit(a, 1)) return b;
      if ((op == BinOp::Mul || op == BinOp::FloorDiv) && is_int_lit(b, 1)) return a;
      if (op == BinOp::Mul && (is_int_lit(a, 0) || is_int_lit(b, 0)) && ty.k == Type::Tensor) return lit_int(0, ty, e->i);
      if (op == BinOp::Rem && is_int_lit(b, 1) && ty.k == Type::Tensor) return lit_int(0, ty, e->i);
    }
  }
  if (a == e->args[0] && b == e->args[1]) return e;
  auto r = std::make_shared<Expr>(*e);
  r->args = {a, b};
  return r;
}

}  // namespace

E fold_expr(const E& e) {
  if (!e) return e;
  switch (e->k) {
    case Expr::UnOpE: {
      E a = fold_expr(e->args[0]);
      if (e->uop == UnOp::Sub && a->k == Expr::Int) return lit_int(-a->iv, e->ty.k == Type::Unknown ? a->ty : e->ty, e->i);
      if (e->uop == UnOp::Sub && a->k == Expr::Float) return lit_float(-a->fv, e->ty.k == Type::Unknown ? a->ty : e->ty, e->i);
      if (e->uop == UnOp::Not && a->k == Expr::Bool) return lit_bool(!a->bv, e->i);
      if (e->uop == UnOp::BitNeg && a->k == Expr::Int) return lit_int(~a->iv, e->ty.k == Type::Unknown ? a->ty : e->ty, e->i);
      if (a == e->args[0]) return e;
      auto r = std::make_shared<Expr>(*e);
      r->args = {a};
      return r;
    }
    case Expr::BinOpE: return fold_binop(e, fold_expr(e->args[0]), fold_expr(e->args[1]));
    case Expr::Convert: {
      E a = fold_expr(e->args[0]);
      ElemSize sz = e->ty.sz;
      if (a->k == Expr::Int) {
        if (is_int(sz)) return lit_int(a->iv, e->ty, e->i);
        if (is_float(sz)) return lit_float((double)a->iv, e->ty, e->i);
        if (sz == ElemSize::Bool) return lit_bool(a->iv != 0, e->i);
      }
      if (a->k == Expr::Float) {
        if (is_float(sz)) return lit_float(a->fv, e->ty, e->i);
        if (is_int(sz) && std::isfinite(a->fv)) return lit_int((int64_t)a->fv, e->ty, e->i);
      }
      if (a->k == Expr::Bool) {
        if (is_int(sz)) return lit_int(a->bv ? 1 : 0, e->ty, e->i);
        if (sz == ElemSize::Bool) return a;
      }
      if (a->ty == e->ty) return a;
      if (a == e->args[0]) return e;
      auto r = std::make_shared<Expr>(*e);
      r->args = {a};
      return r;
    }
    case Expr::IfExpr: {
      E c = fold_expr(e->args[0]), a = fold_expr(e->args[1]), b = fold_expr(e->args[2]);
      if (c->k == Expr::Bool) return c->bv ? a : b;
      if (c->k == Expr::Int) return c->iv != 0 ? a : b;
      auto r = std::make_shared<Expr>(*e);
      r->args = {c, a, b};
      return r;
    }
    default:
      return map_children(e, [](const E& c) { return fold_expr(c); });
  }
}

Stmts fold_stmts(const Stmts& ss) {
  Stmts out;
  for (auto& s0 : ss) {
    S s = map_exprs(s0, [](const E& e) { return fold_expr(e); });
    if (s->k == Stmt::If) {
      E c = s->expr;
      if (c->k == Expr::Bool || c->k == Expr::Int) {
        bool t = c->k == Expr::Bool ? c->bv : c->iv != 0;
        for (auto& b : fold_stmts(t ? s->body : s->els)) out.push_back(b);
        continue;
      }
    }
    if (s->k == Stmt::For && s->lo->k == Expr::Int && s->hi->k == Expr::Int) {
      bool empty = s->step > 0 ? s->lo->iv >= s->hi->iv : s->lo->iv <= s->hi->iv;
      if (empty) continue;
    }
    if (!s->body.empty() || !s->els.empty()) {
      auto r = std::make_shared<Stmt>(*s);
      r->body = fold_stmts(s->body);
      r->els = fold_stmts(s->els);
      s = r;
    }
    out.push_back(s);
  }
  return out;
}

E neutral_element(BinOp op, ElemSize sz, const Info& i) {
  Type ty = Type::scalar(sz);
  auto f = [&](double v) { return lit_float(v, ty, i); };
  auto n = [&](int64_t v) { return lit_int(v, ty, i); };
  auto int_min = [&]() -> int64_t {
    switch (sz) {
      case ElemSize::I8: return INT8_MIN;
      case ElemSize::I16: return INT16_MIN;
      case ElemSize::I32: return INT32_MIN;
      case ElemSize::I64: return INT64_MIN;
      default: return 0;
    }
  };
  auto int_max = [&]() -> int64_t {
    switch (sz) {
      case ElemSize::I8: return INT8_MAX;
      case ElemSize::I16: return INT16_MAX;
      case ElemSize::I32: return INT32_MAX;
      case ElemSize::I64: return INT64_MAX;
      case ElemSize::U8: return UINT8_MAX;
      case ElemSize::U16: return UINT16_MAX;
      case ElemSize::U32: return UINT32_MAX;
      case ElemSize::U64: return -1;  // all ones
      default: return 0;
    }
  };
  switch (op) {
    case BinOp::Add: return is_float(sz) ? f(0.0) : n(0);
    case BinOp::Mul: return is_float(sz) ? f(1.0) : n(1);
    case BinOp::Max: return is_float(sz) ? f(-HUGE_VAL) : n(int_min());
    case BinOp::Min: return is_float(sz) ? f(HUGE_VAL) : n(int_max());
    case BinOp::And: case BinOp::BitAnd:
      if (sz == ElemSize::Bool) return lit_bool(true, i);
      return n(-1);
    case BinOp::Or: case BinOp::BitOr: case BinOp::BitXor:
      if (sz == ElemSize::Bool) return lit_bool(false, i);
      return n(0);
    default:
      fail_rt(i, std::string("Reduction operation ") + binop_name(op) + " has unknown neutral element.");
  }
}

// ---------------------------------------------------------------- intervals
namespace {
Interval iv(int64_t lo, int64_t hi) { Interval r; r.known = true; r.lo = lo; r.hi = hi; return r; }
bool mul_ok(int64_t a, int64_t b, int64_t* out) { return !__builtin_mul_overflow(a, b, out); }
}  // namespace

namespace {
// what the value's own type guarantees: small integer types bound their values
Interval type_range(const Type& ty) {
  Interval none;
  if (!(ty.k == Type::Tensor && ty.shape.empty())) return none;
  switch (ty.sz) {
    case ElemSize::Bool: return iv(0, 1);
    case ElemSize::I8: return iv(INT8_MIN, INT8_MAX);
    case ElemSize::I16: return iv(INT16_MIN, INT16_MAX);
    case ElemSize::U8: return iv(0, UINT8_MAX);
    case ElemSize::U16: return iv(0, UINT16_MAX);
    default: return none;
  }
}
Interval range_impl(const E& e, const RangeEnv& env);
}  // namespace

Interval expr_range(const E& e, const RangeEnv& env) {
  if (!e) return Interval();
  Interval r = range_impl(e, env);
  Interval t = type_range(e->ty);
  if (!r.known) return t;
  if (t.known) { r.lo = std::max(r.lo, t.lo); r.hi = std::min(r.hi, t.hi); if (r.lo > r.hi) return t; }
  return r;
}

namespace {
Interval range_impl(const E& e, const RangeEnv& env) {
  Interval none;
  if (!e) return none;
  switch (e->k) {
    case Expr::Int: return iv(e->iv, e->iv);
    case Expr::Bool: return iv(0, 1);
    case Expr::Var: {
      auto it = env.find(e->name);
      return it == env.end() ? none : it->second;
    }
    case Expr::ThreadIdx: {
      auto it = env.find(Name{std::string("threadIdx.") + "xyz"[e->iv], -1});
      return it == env.end() ? none : it->second;
    }
    case Expr::BlockIdx: {
      auto it = env.find(Name{std::string("blockIdx.") + "xyz"[e->iv], -1});
      return it == env.end() ? none : it->second;
    }
    case Expr::Convert: {
      if (!(e->ty.k == Type::Tensor && is_int(e->ty.sz))) return none;
      Interval a = expr_range(e->args[0], env);
      if (!a.known) return none;
      int bits = elem_bytes(e->ty.sz) * 8;
      if (bits < 64) {
        int64_t lo = is_signed(e->ty.sz) ? -(int64_t(1) << (bits - 1)) : 0;
        int64_t hi = is_signed(e->ty.sz) ? (int64_t(1) << (bits - 1)) - 1 : (int64_t(1) << bits) - 1;
        if (a.lo < lo || a.hi > hi) return none;
      }
      return a;
    }
    case Expr::IfExpr: {
      Interval a = expr_range(e->args[1], env), b = expr_range(e->args[2], env);
      if (!a.known || !b.known) return none;
      return iv(std::min(a.lo, b.lo), std::max(a.hi, b.hi));
    }
    case Expr::UnOpE: {
      if (e->uop != UnOp::Sub) return none;
      Interval a = expr_range(e->args[0], env);
      if (!a.known || a.lo == INT64_MIN) return none;
      return iv(-a.hi, -a.lo);
    }
    case Expr::BinOpE: {
      Interval a = expr_range(e->args[0], env), b = expr_range(e->args[1], env);
      // the smaller of two values is bounded above by either one alone (a loop that runs to min(n, len[i]))
      if (e->bop == BinOp::Min && a.known != b.known) return iv(INT64_MIN, a.known ? a.hi : b.hi);
      if (e->bop == BinOp::Max && a.known != b.known) return iv(a.known ? a.lo : b.lo, INT64_MAX);
      if (!a.known || !b.known) return none;
      int64_t r0, r1, r2, r3;
      switch (e->bop) {
        case BinOp::Add:
          if (__builtin_add_overflow(a.lo, b.lo, &r0) || __builtin_add_overflow(a.hi, b.hi, &r1)) return none;
          return iv(r0, r1);
        case BinOp::Sub:
          if (__builtin_sub_overflow(a.lo, b.hi, &r0) || __builtin_sub_overflow(a.hi, b.lo, &r1)) return none;
          return iv(r0, r1);
        case BinOp::Mul:
          if (!mul_ok(a.lo, b.lo, &r0) || !mul_ok(a.lo, b.hi, &r1) || !mul_ok(a.hi, b.lo, &r2) || !mul_ok(a.hi, b.hi, &r3)) return none;
          return iv(std::min(std::min(r0, r1), std::min(r2, r3)), std::max(std::max(r0, r1), std::max(r2, r3)));
        case BinOp::FloorDiv: case BinOp::Div:
          if (e->bop == BinOp::Div && !(e->ty.k == Type::Tensor && is_int(e->ty.sz))) return none;
          if (b.lo <= 0 || a.lo < 0) return none;
          return iv(a.lo / b.hi, a.hi / b.lo);
        case BinOp::Rem:
          if (b.lo <= 0 || a.lo < 0) return none;
          if (a.hi < b.lo) return a;
          return iv(0, b.hi - 1);
        case BinOp::BitAnd:
          if (a.lo < 0 || b.lo < 0) return none;
          return iv(0, std::min(a.hi, b.hi));
        case BinOp::BitShl:
          if (b.lo != b.hi || b.lo < 0 || b.lo > 40 || a.lo < 0) return none;
          if (!mul_ok(a.hi, int64_t(1) << b.lo, &r0)) return none;
          return iv(a.lo << b.lo, r0);
        case BinOp::BitShr:
          if (b.lo != b.hi || b.lo < 0 || b.lo > 62 || a.lo < 0) return none;
          return iv(a.lo >> b.lo, a.hi >> b.lo);
        case BinOp::Max: return iv(std::max(a.lo, b.lo), std::max(a.hi, b.hi));
        case BinOp::Min: return iv(std::min(a.lo, b.lo), std::min(a.hi, b.hi));
        case BinOp::Eq: case BinOp::Neq: case BinOp::Leq: case BinOp::Geq: case BinOp::Lt: case BinOp::Gt:
          return iv(0, 1);
        default: return none;
      }
    }
    default: return none;
  }
}

}  // namespace

}  // namespace parpy
