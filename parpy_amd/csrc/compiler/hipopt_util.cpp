// gfx950 memory passes, helpers over the kernel IR.
#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

bool mentions(const E& e, const Name& v) {
  bool m = false;
  visit_exprs(e, [&](const E& x) { if (x->k == Expr::Var && x->name == v) m = true; });
  return m;
}

bool has_load(const E& e) {
  bool m = false;
  visit_exprs(e, [&](const E& x) { if (x->k == Expr::Index || x->k == Expr::AddrOf || x->k == Expr::RegElem) m = true; });
  return m;
}

// idx == rest + d with rest free of d
bool affine_unit(const E& idx, const Name& d, E* rest) {
  if (idx->k == Expr::Var && idx->name == d) { *rest = mk_int(0, idx->ty.sz); return true; }
  if (idx->k == Expr::BinOpE && (idx->bop == BinOp::Add || idx->bop == BinOp::Sub)) {
    E r;
    if (affine_unit(idx->args[0], d, &r) && !mentions(idx->args[1], d)) {
      *rest = fold_expr(mk_binop(idx->bop, r, idx->args[1], idx->ty));
      return true;
    }
    if (idx->bop == BinOp::Add && affine_unit(idx->args[1], d, &r) && !mentions(idx->args[0], d)) {
      *rest = fold_expr(mk_binop(BinOp::Add, idx->args[0], r, idx->ty));
      return true;
    }
  }
  return false;
}

int64_t const_extent(const S& loop) {
  if (loop->lo->k != Expr::Int || loop->hi->k != Expr::Int || loop->step <= 0) return -1;
  return (loop->hi->iv - loop->lo->iv + loop->step - 1) / loop->step;
}

// iterations every thread runs in a thread-mapped loop, when that is a compile-time constant
int64_t per_thread_trips(const S& loop) {
  return counted_trips(const_extent(loop), loop->map.n);
}

// the per-thread iteration counter of a mapped loop as the printer names it
E counter_var(const S& loop, ElemSize isz) {
  if (per_thread_trips(loop) == 1) return mk_int(0, isz);
  return mk_var(Name{loop->id.str() + "_k", 0}, Type::scalar(isz));
}

E subst_vars(const E& e, const std::map<Name, E>& m) {
  if (!e) return e;
  if (e->k == Expr::Var) {
    auto it = m.find(e->name);
    return it == m.end() ? e : it->second;
  }
  return map_children(e, [&](const E& c) { return subst_vars(c, m); });
}

}  // namespace hipopt
}  // namespace parpy
