// gfx950 memory passes, values a thread stored in a step and reads back itself.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ values a thread has just stored, read again by itself
// Inside one iteration of a sequential loop a thread-mapped loop stores a row through a pointer (`dst[V q + c] = e`
// for c = 0 .. V-1, a thread owning the same q in every such loop), and later in the same iteration -- possibly
// under a test of the step counter -- a thread-mapped loop of the same shape reads exactly those elements back
// through a pointer that selects the same array under the same condition (`x = a; if (t & 1) x = b` written twice:
// the row maximum every eighth step of the rescaled HMM forward pass).  The values travel in a register array
// from the storing loop to the reading one; the stores stay (other threads read the row in the next iteration),
// the loads from LDS and their wait go.  7-mer batch 16.9 -> 15.5 ms.

// `name = a; if (cond) { ...; name = b; ... }` among the statements of `ss` before position `upto`, no other assignment
Pass::AliasDef Pass::alias_definition(const Stmts& ss, size_t upto, const Name& name) {
  AliasDef d;
  int assigns = 0;
  for (size_t i = 0; i < upto && i < ss.size(); ++i) {
    const S& st = ss[i];
    if (st->k == Stmt::Def && st->id == name && st->expr && st->expr->k == Expr::Var) { d.a = st->expr->name; ++assigns; continue; }
    if (st->k == Stmt::If && st->els.empty()) {
      for (auto& c : st->body)
        if (c->k == Stmt::Assign && c->dst->k == Expr::Var && c->dst->name == name) {
          if (c->expr->k != Expr::Var) return d;
          d.b = c->expr->name;
          d.cond = st->expr;
          ++assigns;
        }
      continue;
    }
    bool touches = false;
    visit_stmts({st}, [&](const S& c) { if ((c->k == Stmt::Assign && c->dst->k == Expr::Var && c->dst->name == name) || (c->k == Stmt::Def && c->id == name)) touches = true; });
    if (touches) return d;
  }
  d.ok = assigns == 2 && d.cond != nullptr;
  return d;
}

// idx == V * var + c with 0 <= c < V
bool Pass::scaled_index(const E& idx, const Name& var, int64_t* V, int64_t* c) {
  std::vector<E> terms;
  std::function<void(const E&)> flat = [&](const E& e) {
    if (e->k == Expr::BinOpE && e->bop == BinOp::Add) { flat(e->args[0]); flat(e->args[1]); }
    else if (e->k == Expr::Convert) flat(e->args[0]);
    else terms.push_back(e);
  };
  flat(idx);
  int64_t v = 0, k0 = 0;
  for (auto& t : terms) {
    if (t->k == Expr::Int) { k0 += t->iv; continue; }
    if (t->k == Expr::BinOpE && t->bop == BinOp::Mul && v == 0) {
      const E &x = t->args[0], &y = t->args[1];
      if (x->k == Expr::Int && y->k == Expr::Var && y->name == var) { v = x->iv; continue; }
      if (y->k == Expr::Int && x->k == Expr::Var && x->name == var) { v = y->iv; continue; }
    }
    return false;
  }
  if (v <= 1 || k0 < 0 || k0 >= v) return false;
  *V = v;
  *c = k0;
  return true;
}

Stmts Pass::keep_stored_rows(const Stmts& ss, int64_t* budget) {
  Stmts out;
  for (auto& st : ss) {
    auto r = clone(st);
    r->body = keep_stored_rows(st->body, budget);
    r->els = keep_stored_rows(st->els, budget);
    bool seq = st->k == Stmt::For && st->map.k == GpuMap::None && !st->unroll;
    if (seq) {
      Stmts pre;
      r->body = keep_in_iteration(r->body, budget, st, &pre);
      for (auto& p : pre) out.push_back(p);
    }
    out.push_back(r);
  }
  return out;
}

// `t & 1` on the variable of a loop with step one (possibly compared with zero): true in every other iteration
bool Pass::alternates(const E& cond, const S& loop) {
  E c = cond;
  while (c->k == Expr::Convert) c = c->args[0];
  if (c->k == Expr::BinOpE && c->bop == BinOp::Neq && c->args[1]->k == Expr::Int && c->args[1]->iv == 0) c = c->args[0];
  while (c->k == Expr::Convert) c = c->args[0];
  if (!(c->k == Expr::BinOpE && c->bop == BinOp::BitAnd && loop->step == 1)) return false;
  E v = c->args[0], one = c->args[1];
  while (v->k == Expr::Convert) v = v->args[0];
  return v->k == Expr::Var && v->name == loop->id && one->k == Expr::Int && one->iv == 1;
}

// The second half: when the pointer pair of the step swaps its arrays every iteration (`src = a, dst = b`, the
// other way round when `t & 1`), what a thread reads of its own elements through `src` in one iteration is what
// it stored through `dst` in the iteration before.  The register array then lives across the iterations: filled
// from the start row in front of the loop, read where the loop read its own elements from LDS, overwritten by the
// stores.  A third of the LDS bytes of the rescaled HMM step (the 16-byte loads of the own states) go.
// Returns the rewritten body of the storing loop, or an empty list when the conditions do not hold.
Stmts Pass::carry_across_iterations(const Stmts& B, size_t p1, const S& L1, const IterSpace& is1, const S& seq_loop, const AliasDef& dx,
                              int64_t V, const std::map<int64_t, size_t>& store_at, const Name& reg, ElemSize sz, Stmts* pre) {
  Type ity = Type::scalar(isz);
  if (!alternates(dx.cond, seq_loop) || seq_loop->lo->k != Expr::Int) return {};
  // the pointer the own elements are read through: the swapped pair, same test
  Name Xs;
  bool ok = true;
  std::map<int64_t, size_t> last_read;     // c -> last statement of the body that reads element c through Xs
  for (size_t i = 0; i < L1->body.size() && ok; ++i)
    visit_stmts({L1->body[i]}, [&](const S& c) {
      visit_stmt_exprs(c, [&](const E& x) {
        if (x->k != Expr::Index || x->args[0]->k != Expr::Var) return;
        int64_t v = 0, k0 = 0;
        if (!scaled_index(x->args[1], L1->id, &v, &k0) || v != V || x->ty.sz != sz) return;
        if (c->k == Stmt::Assign && c->dst.get() == x.get()) return;      // the store itself
        AliasDef d = alias_definition(B, p1, x->args[0]->name);
        if (!(d.ok && d.a == dx.b && d.b == dx.a && expr_eq(d.cond, dx.cond))) return;
        if (Xs.s.empty()) Xs = x->args[0]->name;
        else if (!(Xs == x->args[0]->name)) ok = false;
        last_read[k0] = i;
      });
    });
  if (!ok || Xs.s.empty()) return {};
  // an element is read before the thread overwrites it (the register slot holds the old value until then)
  for (auto& kv : last_read)
    if (kv.second > store_at.at(kv.first)) return {};
  // nothing else in the iteration stores to memory through a pointer (the emission refill writes registers, the
  // look-up only reads), so the rows change through this loop alone
  bool clean = true;
  for (size_t i = 0; i < B.size(); ++i) {
    if (i == p1) continue;
    visit_stmts({B[i]}, [&](const S& c) {
      if (c->k == Stmt::Assign && c->dst->k == Expr::Index) clean = false;
      if (c->k == Stmt::CallStmt || c->k == Stmt::While) clean = false;
    });
  }
  if (!clean) return {};
  auto reg_elem = [&](const E& slot) {
    auto re = std::make_shared<Expr>();
    re->k = Expr::RegElem;
    re->ty = Type::scalar(sz);
    re->name = reg;
    re->args = {slot};
    return E(re);
  };
  auto slot_of = [&](int64_t c) { return fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, is1.slot, mk_int(V, isz), ity), mk_int(c, isz), ity)); };
  // in front of the loop: the thread's elements of the row that the first iteration reads
  Name first = (seq_loop->lo->iv & 1) ? dx.a : dx.b;      // src is the pair swapped: b in even iterations, a in odd ones
  Type pty = Type::pointer(sz);
  pty.mem = Mem::LDS;
  if (!lds_array_names().count(first)) return {};
  Stmts fill;
  for (int64_t c = 0; c < V; ++c) {
    E idx = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, mk_int(V, isz), mk_var(L1->id, ity), ity), mk_int(c, isz), ity));
    fill.push_back(mk_assign(reg_elem(slot_of(c)), mk_index(mk_var(first, pty), idx, Type::scalar(sz))));
  }
  auto init = clone(L1);
  init->body = fill;
  init->unroll = true;
  pre->push_back(mk_sync());       // what other threads stored into the start row is in place
  pre->push_back(init);
  return rewrite_stmts(L1->body, [&](const E& e) -> E {
    if (e->k != Expr::Index || e->args[0]->k != Expr::Var || !(e->args[0]->name == Xs)) return e;
    int64_t v = 0, k0 = 0;
    if (!scaled_index(e->args[1], L1->id, &v, &k0) || v != V) return e;
    return reg_elem(slot_of(k0));
  });
}

std::set<Name> Pass::lds_array_names() const {
  std::set<Name> r;
  visit_stmts(k.body, [&](const S& c) { if (c->k == Stmt::LdsDecl) r.insert(c->id); });
  return r;
}

Stmts Pass::keep_in_iteration(const Stmts& B, int64_t* budget, const S& seq_loop, Stmts* pre) {
  Type ity = Type::scalar(isz);
  for (size_t p1 = 0; p1 < B.size(); ++p1) {
    const S& L1 = B[p1];
    IterSpace is1;
    if (!thread_mapped(L1) || L1->par.reduction || !iter_space(L1, &is1) || is1.inner || L1->lo->k != Expr::Int || L1->lo->iv != 0) continue;
    // the stores of the loop: top-level statements of its body, all through one pointer variable, one per c
    Name X;
    int64_t V = 0;
    std::map<int64_t, size_t> store_at;
    bool ok = true;
    ElemSize sz = ElemSize::F32;
    for (size_t i = 0; i < L1->body.size() && ok; ++i) {
      const S& c = L1->body[i];
      if (c->k != Stmt::Assign || c->dst->k != Expr::Index) continue;
      int64_t v = 0, k0 = 0;
      if (c->dst->args[0]->k != Expr::Var || !scaled_index(c->dst->args[1], L1->id, &v, &k0)) { ok = false; break; }
      if (V == 0) { V = v; X = c->dst->args[0]->name; sz = c->dst->ty.sz; }
      if (v != V || !(c->dst->args[0]->name == X) || store_at.count(k0) || c->dst->ty.sz != sz) { ok = false; break; }
      store_at[k0] = i;
    }
    // (stores under a condition or in a nested loop would leave register slots unset)
    visit_stmts(L1->body, [&](const S& c) { if (c->k == Stmt::Assign && c->dst->k == Expr::Index) { bool top = false; for (auto& t : L1->body) top = top || t == c; if (!top) ok = false; } });
    if (!ok || V == 0 || (int64_t)store_at.size() != V || elem_bytes(sz) != 4) continue;
    AliasDef dx = alias_definition(B, p1, X);
    if (!dx.ok) continue;
    int64_t slots = is1.slots * V;
    // (a thread with a single vector reloads it with one LDS instruction: measured 3 % slower kept than reloaded
    // on the 1024-state model with 256 threads, so only rows of at least two vectors per thread are kept)
    if (slots < 2 * V || slots > 32 || slots > *budget) continue;
    // the reader: later in the iteration, directly or as a statement of an `if` on scalars only
    for (size_t p2 = p1 + 1; p2 < B.size(); ++p2) {
      const S& outer = B[p2];
      const Stmts* list = &B;
      size_t pos = p2;
      if (outer->k == Stmt::If && outer->els.empty() && !has_load(outer->expr)) {
        list = &outer->body;
        pos = 0;
      }
      bool found = false;
      for (; pos < list->size() && !found; ++pos) {
        const S& L2 = (*list)[pos];
        IterSpace is2;
        if (!thread_mapped(L2) || !iter_space(L2, &is2) || !is2.inner || is2.slots != slots || const_extent(is2.inner) != V ||
            L2->map.n != L1->map.n || const_extent(L2) != const_extent(L1) || L2->lo->k != Expr::Int || L2->lo->iv != 0)
          { if (list == &B) break; else continue; }
        if (is2.body->empty() || (*is2.body)[0]->k != Stmt::Def) break;
        const S& edef = (*is2.body)[0];
        // element = V * q2 + u, exactly the element (q, c) of the storing loop
        E want = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, mk_var(L2->id, ity), mk_int(V, isz), ity), mk_var(is2.inner->id, ity), ity));
        if (!expr_eq(fold_expr(edef->expr), want)) break;
        // every access to an array in the loop is a read of Y[element]
        Name Y;
        bool good = true;
        visit_stmts(*is2.body, [&](const S& c) {
          if (c->k == Stmt::Assign && c->dst->k == Expr::Index) good = false;
          visit_stmt_exprs(c, [&](const E& x) {
            if (x->k != Expr::Index) return;
            if (x->args[0]->k != Expr::Var || !(x->args[1]->k == Expr::Var && x->args[1]->name == edef->id) || x->ty.sz != sz) { good = false; return; }
            if (Y.s.empty()) Y = x->args[0]->name;
            else if (!(Y == x->args[0]->name)) good = false;
          });
        });
        if (!good || Y.s.empty()) break;
        AliasDef dy = alias_definition(*list, pos, Y);
        if (!dy.ok || !(dy.a == dx.a) || !(dy.b == dx.b) || !expr_eq(dy.cond, dx.cond)) break;
        // nothing between the two loops stores to memory through a pointer or to the two arrays, and the
        // condition of the selection still means the same (its variables are not assigned)
        std::set<Name> cond_vars;
        visit_exprs(dx.cond, [&](const E& x) { if (x->k == Expr::Var) cond_vars.insert(x->name); });
        bool clean = true;
        auto check = [&](const Stmts& span, size_t lo, size_t hi) {
          for (size_t i = lo; i < hi && i < span.size(); ++i)
            visit_stmts({span[i]}, [&](const S& c) {
              if (c->k == Stmt::Assign && c->dst->k == Expr::Index) clean = false;
              if (c->k == Stmt::Assign && c->dst->k == Expr::Var && cond_vars.count(c->dst->name)) clean = false;
              if (c->k == Stmt::CallStmt || c->k == Stmt::While) clean = false;
            });
        };
        check(B, p1 + 1, p2);
        if (list != &B) check(*list, 0, pos);
        if (!clean) break;
        // ---- rewrite
        Name reg = gen.fresh("kept_" + X.s);
        auto reg_elem = [&](const E& slot) {
          auto re = std::make_shared<Expr>();
          re->k = Expr::RegElem;
          re->ty = Type::scalar(sz);
          re->name = reg;
          re->args = {slot};
          return E(re);
        };
        Stmts carried = opts.opt_keep_own ? carry_across_iterations(B, p1, L1, is1, seq_loop, dx, V, store_at, reg, sz, pre) : Stmts();
        const Stmts& body1 = carried.empty() ? L1->body : carried;
        Stmts nb1;
        for (size_t i = 0; i < body1.size(); ++i) {
          const S& c = body1[i];
          int64_t cc = -1;
          for (auto& kv : store_at) if (kv.second == i) cc = kv.first;
          if (cc < 0) { nb1.push_back(c); continue; }
          E slot = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, is1.slot, mk_int(V, isz), ity), mk_int(cc, isz), ity));
          nb1.push_back(mk_assign(reg_elem(slot), c->expr, c->i));
          nb1.push_back(mk_assign(c->dst, reg_elem(slot), c->i));
        }
        auto n1 = clone(L1);
        n1->body = nb1;
        n1->unroll = true;
        Stmts inner2 = rewrite_stmts(*is2.body, [&](const E& e) -> E {
          if (e->k == Expr::Index && e->args[0]->k == Expr::Var && e->args[0]->name == Y) return reg_elem(is2.slot);
          return e;
        });
        auto ni = clone(is2.inner);
        ni->body = inner2;
        auto n2 = clone(L2);
        n2->body = {S(ni)};
        n2->unroll = true;
        auto decl = std::make_shared<Stmt>();
        decl->k = Stmt::RegDecl;
        decl->id = reg;
        decl->ty = Type::scalar(sz);
        decl->iv = slots;
        Stmts nb;
        if (!carried.empty()) pre->insert(pre->begin(), S(decl));      // the array lives across the iterations
        for (size_t i = 0; i < B.size(); ++i) {
          if (i == p1) { if (carried.empty()) nb.push_back(decl); nb.push_back(n1); continue; }
          if (i == p2) {
            if (list == &B) nb.push_back(n2);
            else {
              auto no = clone(outer);
              Stmts lb = *list;
              lb[pos] = n2;
              no->body = lb;
              nb.push_back(no);
            }
            continue;
          }
          nb.push_back(B[i]);
        }
        *budget -= slots;
        return nb;
      }
      // a statement between that may change the arrays ends the search
      bool barrier_like = true;
      visit_stmts({outer}, [&](const S& c) { if (c->k == Stmt::Assign && c->dst->k == Expr::Index) barrier_like = false; });
      if (!barrier_like) break;
    }
  }
  return B;
}

}  // namespace hipopt
}  // namespace parpy
