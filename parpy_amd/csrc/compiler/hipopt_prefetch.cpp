// gfx950 memory passes, loads issued a step ahead of their use.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ loads that depend on the step counter alone
// Inside a sequential loop that a workgroup walks step by step (a barrier per step), `o = data[i, t]`
// is needed at the very start of step t and everything else of the step hangs on it (it selects the
// emission row).  The array is never written and the address is a function of t and of values that
// do not change in the loop, so the load for step t + 1 is issued at the start of step t into a second
// variable: its latency passes behind a whole step of work.  The index must be provably in bounds
// over the static range of the loop (the last iteration re-reads its own element instead of t + 1).
Stmts Pass::prefetch_counter_loads(const Stmts& ss, RangeEnv env) {
  std::set<Name> params = param_names();
  std::set<Name> written = written_arrays();
  Stmts out;
  for (size_t pos = 0; pos < ss.size(); ++pos) {
    const S& s = ss[pos];
    bool seq = s->k == Stmt::For && s->map.k == GpuMap::None && !s->unroll && s->step == 1 && s->lo->k == Expr::Int;
    // static upper bound of the loop: a literal, or a variable defined just before as min(literal, ...)
    int64_t HI = -1;
    if (seq) {
      if (s->hi->k == Expr::Int) HI = s->hi->iv;
      else if (s->hi->k == Expr::Var)
        for (size_t b = 0; b < out.size(); ++b)
          if (out[b]->k == Stmt::Def && out[b]->id == s->hi->name && out[b]->expr->k == Expr::BinOpE && out[b]->expr->bop == BinOp::Min) {
            for (auto& a : out[b]->expr->args) if (a->k == Expr::Int) HI = a->iv;
          }
    }
    bool barrier_inside = false;
    if (seq) visit_stmts(s->body, [&](const S& c) { if (c->k == Stmt::Sync || c->k == Stmt::SyncPoint) barrier_inside = true; });
    if (seq && HI > s->lo->iv && barrier_inside) {
      std::set<Name> varying{s->id}, reassigned;
      visit_stmts(s->body, [&](const S& c) {
        if (c->k == Stmt::Def || c->k == Stmt::For) varying.insert(c->id);
        if (c->k == Stmt::Assign && c->dst->k == Expr::Var) { varying.insert(c->dst->name); reassigned.insert(c->dst->name); }
      });
      varying.erase(s->id);
      RangeEnv le = env;
      Interval tr;
      tr.known = true;
      tr.lo = s->lo->iv;
      tr.hi = HI - 1;
      le[s->id] = tr;
      Stmts pre, body;
      for (auto& c : s->body) {
        E ld = c->k == Stmt::Def && c->expr ? strip_converts(c->expr) : E();
        bool ok = ld && ld->k == Expr::Index && c->ty.is_scalar() && !reassigned.count(c->id) && ld->args[0]->k == Expr::Var &&
                  params.count(ld->args[0]->name) && !written.count(ld->args[0]->name) && !ld->dim_shape.empty() && mentions(ld->args[1], s->id);
        if (ok) {
          visit_exprs(ld->args[1], [&](const E& x) {
            if (x->k == Expr::Var && varying.count(x->name)) ok = false;
            if (x->k == Expr::Index || x->k == Expr::RegElem || x->k == Expr::ThreadIdx || x->k == Expr::Call || x->k == Expr::Raw) ok = false;
          });
        }
        if (ok) {
          int64_t numel = 1;
          for (auto d : ld->dim_shape) numel *= d;
          Interval r = expr_range(ld->args[1], le);
          ok = r.known && r.lo >= 0 && r.hi < numel;
        }
        if (!ok) { body.push_back(c); continue; }
        Type ity = s->lo->ty;
        auto at = [&](const E& t) {
          std::map<Name, E> m{{s->id, t}};
          return subst_vars(c->expr, m);
        };
        Name nxt = gen.fresh(c->id.s + "_next");
        pre.push_back(mk_def(nxt, c->ty, at(s->lo), c->i));
        body.push_back(mk_def(c->id, c->ty, mk_var(nxt, c->ty), c->i));
        E t1 = mk_binop(BinOp::Min, mk_binop(BinOp::Add, mk_var(s->id, ity), mk_int(1, ity.sz), ity), mk_int(HI - 1, ity.sz), ity);
        body.push_back(mk_assign(mk_var(nxt, c->ty), at(t1), c->i));
      }
      if (!pre.empty()) {
        for (auto& d : pre) out.push_back(d);
        auto r = clone(s);
        r->body = body;
        out.push_back(r);
        continue;
      }
    }
    auto r = clone(s);
    RangeEnv ne = env;
    if (s->k == Stmt::For && s->lo && s->hi && s->lo->k == Expr::Int && s->hi->k == Expr::Int && s->hi->iv > s->lo->iv) {
      Interval v;
      v.known = true;
      v.lo = s->lo->iv;
      v.hi = s->hi->iv - 1;
      ne[s->id] = v;
    }
    r->body = prefetch_counter_loads(s->body, ne);
    r->els = prefetch_counter_loads(s->els, ne);
    out.push_back(r);
  }
  return out;
}

// ================================================================ rows selected by a value loaded one step ahead
// Second level of the step-ahead loads above: `o = o_next; o_next = data[i, t + 1]` makes the observation of
// the next step known while the current one runs, so the elements of a never-written table that a thread
// reads at `tab[o, f(iteration)]` can be fetched for step t + 1 as soon as the thread has consumed those of
// step t.  They travel in a per-thread register array (one slot per iteration the thread runs): filled
// before the loop for the first step, refilled right after the thread's loop over its iterations, so the
// latency of the table passes behind the barrier and the shared-memory phase of the next step.  Costs one
// register per element and is only done while the register budget lasts.
Stmts Pass::prefetch_selected_rows(const Stmts& ss, int64_t* budget) {
  std::set<Name> params = param_names();
  std::set<Name> written = written_arrays();
  Stmts out;
  for (auto& s : ss) {
    bool seq = s->k == Stmt::For && s->map.k == GpuMap::None && !s->unroll;
    // the pairs `o = o_next; o_next = ...` at the top level of the loop body
    std::map<Name, Name> ahead;   // o -> o_next
    if (seq)
      for (size_t i = 0; i + 1 < s->body.size(); ++i) {
        const S &d = s->body[i], &a = s->body[i + 1];
        if (d->k == Stmt::Def && d->expr && d->expr->k == Expr::Var && a->k == Stmt::Assign && a->dst->k == Expr::Var &&
            a->dst->name == d->expr->name && has_load(a->expr))
          ahead[d->id] = d->expr->name;
      }
    if (!seq || ahead.empty()) {
      auto r = clone(s);
      r->body = prefetch_selected_rows(s->body, budget);
      r->els = prefetch_selected_rows(s->els, budget);
      out.push_back(r);
      continue;
    }
    std::set<Name> varying, reassigned;
    visit_stmts(s->body, [&](const S& c) {
      if (c->k == Stmt::Def || c->k == Stmt::For) varying.insert(c->id);
      if (c->k == Stmt::Assign && c->dst->k == Expr::Var) { varying.insert(c->dst->name); reassigned.insert(c->dst->name); }
    });
    Stmts pre, body;
    for (auto& c : s->body) {
      IterSpace is;
      if (!(thread_mapped(c) && iter_space(c, &is))) { body.push_back(c); continue; }
      std::set<Name> iter_vars{c->id};
      if (is.inner) iter_vars.insert(is.inner->id);
      std::map<Name, E> defs;   // definitions in the body that are pure functions of the iteration
      std::function<void(const Stmts&)> collect_defs = [&](const Stmts& b) {
        for (auto& d : b) {
          if (d->k == Stmt::Def && d->ty.is_scalar() && !has_load(d->expr) && !reassigned.count(d->id)) {   // a name assigned again stands for several values
            E e = subst_vars(d->expr, defs);
            bool pure = true;
            visit_exprs(e, [&](const E& x) { if (x->k == Expr::Var && !iter_vars.count(x->name)) pure = false; });
            if (pure) defs[d->id] = e;
          }
          collect_defs(d->body);
          collect_defs(d->els);
        }
      };
      collect_defs(*is.body);
      struct Row { E load; Name reg; ElemSize sz; };
      std::vector<Row> rows;
      auto take = [&](const E& e) -> E {
        if (e->k != Expr::Index || e->args[0]->k != Expr::Var) return e;
        const Name& base = e->args[0]->name;
        if (!params.count(base) || written.count(base) || e->dim_shape.empty() || elem_bytes(e->ty.sz) > 4) return e;
        E idx = fold_expr(subst_vars(e->args[1], defs));
        bool selected = false, ok = true;
        visit_exprs(idx, [&](const E& x) {
          if (x->k == Expr::Var && ahead.count(x->name)) selected = true;
          else if (x->k == Expr::Var && !iter_vars.count(x->name) && varying.count(x->name)) ok = false;
          if (x->k == Expr::Index || x->k == Expr::RegElem || x->k == Expr::ThreadIdx || x->k == Expr::Call || x->k == Expr::Raw) ok = false;
        });
        if (!selected || !ok) return e;
        auto elem = [&](const Name& reg) {
          auto re = std::make_shared<Expr>();
          re->k = Expr::RegElem;
          re->ty = e->ty;
          re->name = reg;
          re->args = {is.slot};
          return E(re);
        };
        for (auto& r : rows)
          if (r.load->args[0]->name == base && expr_eq(r.load->args[1], idx)) return elem(r.reg);
        auto ld = std::make_shared<Expr>(*e);
        ld->args = {e->args[0], idx};
        ld->dim_idx.clear();
        rows.push_back({E(ld), gen.fresh("row_" + base.s), e->ty.sz});
        return elem(rows.back().reg);
      };
      Stmts nbody = rewrite_stmts(*is.body, take);
      // all elements of the row that the thread reads, or none (a part of them would split the 16-byte loads)
      int64_t cost = (int64_t)rows.size() * is.slots;
      if (rows.empty() || *budget < cost) { body.push_back(c); continue; }
      *budget -= cost;
      // the loop nest that fills the registers from the row of the step to come
      auto fill_nest = [&]() {
        std::map<Name, E> rv;
        Type ity = Type::scalar(isz);
        Name nq = gen.fresh(c->id.s), nu;
        rv[c->id] = mk_var(nq, ity);
        if (is.inner) { nu = gen.fresh(is.inner->id.s); rv[is.inner->id] = mk_var(nu, ity); }
        for (auto& kv : ahead) rv[kv.first] = mk_var(kv.second, Type::scalar(ElemSize::I8));
        auto outer = clone(c);
        outer->id = nq;
        outer->unroll = true;
        E kq = counter_var(outer, isz), slot = kq;
        if (is.inner) {
          int64_t V = const_extent(is.inner);
          slot = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, kq, mk_int(V, isz), ity), mk_var(nu, ity), ity));
        }
        Stmts fills;
        for (auto& r : rows) {
          auto re = std::make_shared<Expr>();
          re->k = Expr::RegElem;
          re->ty = Type::scalar(r.sz);
          re->name = r.reg;
          re->args = {slot};
          fills.push_back(mk_assign(E(re), subst_vars(r.load, rv)));
        }
        if (is.inner) {
          auto fi = clone(is.inner);
          fi->id = nu;
          fi->body = fills;
          outer->body = {S(fi)};
        } else {
          outer->body = fills;
        }
        return S(outer);
      };
      for (auto& r : rows) {
        auto d = std::make_shared<Stmt>();
        d->k = Stmt::RegDecl;
        d->id = r.reg;
        d->ty = Type::scalar(r.sz);
        d->iv = is.slots;
        pre.push_back(d);
      }
      pre.push_back(fill_nest());
      auto nc = clone(c);
      nc->unroll = true;
      if (is.inner) {
        auto ni = clone(is.inner);
        ni->body = nbody;
        nc->body = {S(ni)};
      } else {
        nc->body = nbody;
      }
      body.push_back(nc);
      body.push_back(fill_nest());
    }
    for (auto& d : pre) out.push_back(d);
    auto r = clone(s);
    r->body = body;
    out.push_back(r);
  }
  return out;
}

}  // namespace hipopt
}  // namespace parpy
