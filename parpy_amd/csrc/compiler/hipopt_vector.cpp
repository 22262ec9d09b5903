// gfx950 memory passes, several consecutive elements per thread; MFMA dot products.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ vectorised iteration remap
// Elements per thread that turn the unit-stride accesses of `loop` into 16-byte accesses, 0 when the
// rewrite does not pay.  It does not pay when such an access goes through a local pointer into global
// memory (`src = a if t & 1 else b`): loads and stores through pointers that may coincide cannot be
// merged, so every lane would issue four 4-byte accesses 16 bytes apart from its neighbour's -- a
// quarter of each cache line per request -- where the plain loop has neighbouring lanes on
// neighbouring words.  (Measured on a 262144-state HMM step kept in global memory: 158 us per step
// with the rewrite, 60 us without.)  Pointers into LDS have no such cost.
int Pass::vector_width(const S& loop) {
  int v = 0;
  bool through_global_alias = false, owns_runs = false;
  std::set<Name> params = param_names();
  std::function<void(const E&)> scan = [&](const E& e) {
    visit_exprs(e, [&](const E& x) {
      if (x->k != Expr::Index) return;
      E rest;
      if (!affine_unit(x->args[1], loop->id, &rest)) {
        // an iteration that already owns a run of 16 bytes or more (`a[4*d + c]`): neighbouring lanes sit on
        // neighbouring runs, and giving a thread V consecutive iterations would put them V runs apart
        if (strided_run(x->args[1], loop->id) * elem_bytes(x->ty.sz) >= 16) owns_runs = true;
        return;
      }
      const E& base = x->args[0];
      if (base->k == Expr::Var && !params.count(base->name) && base->ty.mem != Mem::LDS) through_global_alias = true;
      // (the same holds for every global array when the call passed one that is not 16-byte aligned)
      if (base->k == Expr::Var && base->ty.mem != Mem::LDS && !opts.assume_aligned) through_global_alias = true;
      int w = elem_bytes(x->ty.sz) == 8 ? 2 : elem_bytes(x->ty.sz) == 4 ? 4 : 0;
      if (w == 0) return;
      v = v == 0 ? w : std::min(v, w);
    });
  };
  visit_stmts(loop->body, [&](const S& s) { scan(s->dst); scan(s->expr); scan(s->lo); scan(s->hi); });
  return through_global_alias || owns_runs ? 0 : v;
}

// c when idx == c * d + rest with rest free of d and c a constant > 1, else 0
int64_t Pass::strided_run(const E& idx, const Name& d) {
  if (idx->k != Expr::BinOpE) return 0;
  const E &a = idx->args[0], &b = idx->args[1];
  if (idx->bop == BinOp::Mul) {
    if (a->k == Expr::Int && b->k == Expr::Var && b->name == d) return a->iv > 1 ? a->iv : 0;
    if (b->k == Expr::Int && a->k == Expr::Var && a->name == d) return b->iv > 1 ? b->iv : 0;
    return 0;
  }
  if (idx->bop == BinOp::Add || idx->bop == BinOp::Sub) {
    if (!mentions(b, d)) return strided_run(a, d);
    if (idx->bop == BinOp::Add && !mentions(a, d)) return strided_run(b, d);
  }
  return 0;
}

Stmts Pass::vectorize(const Stmts& ss) {
  Stmts out;
  for (auto& s : ss) {
    bool done = false;
    // grid-wide loops qualify too when the launch has no partial block (no bounds guard)
    bool grid_wide = s->k == Stmt::For && s->map.k == GpuMap::ThreadBlock && s->map.tpb > 0 && s->map.n % s->map.tpb == 0;
    if ((thread_mapped(s) || grid_wide) && s->step == 1 && s->lo->k == Expr::Int && s->hi->k == Expr::Int) {
      int64_t extent = const_extent(s);
      int V = vector_width(s);
      bool nested = false;
      visit_stmts(s->body, [&](const S& c) { if (c->k == Stmt::For && c->map.k != GpuMap::None) nested = true; });
      // a block-level loop only needs whole vectors (threads may run different trip counts); a grid-wide
      // one must also fill its launch exactly, since it has no bounds guard
      // (fewer vectors than threads would leave threads idle that the scalar loop keeps busy)
      if (V > 0 && !nested && extent >= s->map.n * V && extent % V == 0 && (!grid_wide || extent % (s->map.n * V) == 0)) {
        Type ity = Type::scalar(isz);
        Name q = gen.fresh(s->id.s + "_q"), u = gen.fresh(s->id.s + "_u");
        E d = fold_expr(mk_binop(BinOp::Add, s->lo,
                                 mk_binop(BinOp::Add, mk_binop(BinOp::Mul, mk_var(q, ity), mk_int(V, isz), ity), mk_var(u, ity), ity), ity));
        Stmts ib;
        ib.push_back(mk_def(s->id, ity, d, s->i));
        for (auto& b : s->body) ib.push_back(b);
        auto inner = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(
            mk_for(u, mk_int(0, isz), mk_int(V, isz), 1, ib, LoopPar(), s->i)));
        inner->unroll = true;
        auto outer = clone(s);
        outer->id = q;
        outer->lo = mk_int(0, isz);
        outer->hi = mk_int(extent / V, isz);
        outer->body = {S(inner)};
        out.push_back(outer);
        done = true;
      }
    }
    if (done) continue;
    auto r = clone(s);
    r->body = vectorize(s->body);
    r->els = vectorize(s->els);
    out.push_back(r);
  }
  return out;
}

// ================================================================ dot products on the matrix cores
// `t = t + X[..] * Y[..]` in an innermost sequential f32 loop of constant length is a dot
// product that every thread computes for itself.  v_mfma_f32_4x4x1 multiplies, for each group
// of four lanes, the four X values by the four Y values of the group (a 4 x 4 outer product
// accumulated over the loop); the product a thread wants is element [lane % 4] of its own
// column.  Three quarters of the multiplications are thrown away and the instruction takes two
// passes, so this is no faster than v_fmac on the vector ALU: there is no operand reuse between
// the dot products of different threads for a matrix unit to exploit.  Kept as an option so
// that the comparison can be measured.
Stmts Pass::mfma_dot(const Stmts& ss) {
  Stmts out;
  for (auto& s : ss) {
    bool inner = s->k == Stmt::For && s->map.k == GpuMap::None && s->step == 1 && s->hi->k == Expr::Int && s->lo->k == Expr::Int &&
                 s->body.size() == 1 && s->body[0]->k == Stmt::Assign && s->body[0]->dst->k == Expr::Var;
    if (inner) {
      const S& a = s->body[0];
      const E& t = a->dst;
      E mul;
      if (a->expr->k == Expr::BinOpE && a->expr->bop == BinOp::Add) {
        const E &l = a->expr->args[0], &r = a->expr->args[1];
        if (l->k == Expr::Var && l->name == t->name) mul = r;
        else if (r->k == Expr::Var && r->name == t->name) mul = l;
      }
      bool ok = mul && mul->k == Expr::BinOpE && mul->bop == BinOp::Mul && t->ty.is_scalar() && t->ty.sz == ElemSize::F32 &&
                mul->args[0]->k == Expr::Index && mul->args[1]->k == Expr::Index && mul->args[0]->ty.sz == ElemSize::F32 &&
                mul->args[1]->ty.sz == ElemSize::F32 && !mentions(mul, t->name);
      if (ok) {
        Name acc = gen.fresh(t->name.s + "_acc");
        Type f32 = Type::scalar(ElemSize::F32);
        out.push_back(mk_rawstmt("parpy_f32x4 " + acc.str() + " = {0.0f, 0.0f, 0.0f, 0.0f};"));
        auto call = std::make_shared<Expr>();
        call->k = Expr::Call;
        call->ty = f32;
        call->sval = "__builtin_amdgcn_mfma_f32_4x4x1f32";
        call->args = {mul->args[0], mul->args[1], mk_var(acc, f32), mk_raw("0", f32), mk_raw("0", f32), mk_raw("0", f32)};
        auto loop = clone(s);
        loop->body = {mk_assign(mk_var(acc, f32), call)};
        out.push_back(loop);
        out.push_back(mk_assign(t, mk_binop(BinOp::Add, t, mk_raw(acc.str() + "[parpy_lane_id() & 3]", f32), f32)));
        continue;
      }
    }
    auto r = clone(s);
    r->body = mfma_dot(s->body);
    r->els = mfma_dot(s->els);
    out.push_back(r);
  }
  return out;
}

}  // namespace hipopt
}  // namespace parpy
