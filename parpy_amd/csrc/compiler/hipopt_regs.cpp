// gfx950 memory passes, values kept in registers: the register budget, loads hoisted out of sequential loops, sections cached between loops.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ hoisting of thread-private invariant loads
// The iteration structure of a thread-mapped loop: the mapped loop itself and,
// after vectorisation, the unrolled inner loop over the V consecutive elements.
bool Pass::iter_space(const S& loop, IterSpace* is) {
  int64_t per = per_thread_trips(loop);
  if (per <= 0) return false;
  is->outer = loop;
  Type ity = Type::scalar(isz);
  E kq = counter_var(loop, isz);
  if (loop->body.size() == 1 && loop->body[0]->k == Stmt::For && loop->body[0]->unroll &&
      loop->body[0]->map.k == GpuMap::None && const_extent(loop->body[0]) > 0 && loop->body[0]->lo->k == Expr::Int &&
      loop->body[0]->lo->iv == 0) {
    is->inner = loop->body[0];
    int64_t V = const_extent(is->inner);
    is->slots = per * V;
    is->slot = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, kq, mk_int(V, isz), ity), mk_var(is->inner->id, ity), ity));
    is->body = &is->inner->body;
  } else {
    is->slots = per;
    is->slot = kq;
    is->body = &loop->body;
  }
  return true;
}

std::set<Name> Pass::written_arrays() {
  std::set<Name> w;
  visit_stmts(k.body, [&](const S& s) {
    if (s->k == Stmt::Assign && s->dst->k == Expr::Index) {
      visit_exprs(s->dst->args[0], [&](const E& x) { if (x->k == Expr::Var) w.insert(x->name); });
    }
  });
  return w;
}

int64_t Pass::reg_budget() const {
  if (opts.reg_budget > 0) return opts.reg_budget;
  int64_t threads = k.block.x * k.block.y * k.block.z;
  // a 1024-thread block leaves 128 VGPRs per lane; 88 cached values plus the
  // working set fit without spilling (measured on the HMM kernels; 96 spills a few)
  // (workgroups of up to 512 threads leave a wave 256 registers or more: 192 cached values and the working set fit;
  // with 128 the 7-mer HMM forms on 512 threads cache a part of their tables and run up to 2.6 times slower)
  int64_t base = threads <= 512 ? 192 : step_has_transcendentals() ? 88 : 112;
  // (a per-element step body without exponentials or logarithms keeps few values alive besides the cached ones)
  // The driver reads the spill count of the compiled code object and asks again with a smaller share when the
  // register allocator did not get by.
  return std::max<int64_t>(base * opts.reg_budget_scale / 100, 8);
}

// whether the per-element body of a step loop (a thread-mapped loop inside a sequential loop) takes exponentials
// or logarithms: such a step is bound by the vector ALU, one without them by what it moves
bool Pass::step_has_transcendentals() const {
  bool transcendental = false;
  std::function<void(const Stmts&, bool, bool)> walk = [&](const Stmts& ss, bool in_seq, bool in_threads) {
    for (auto& st : ss) {
      if (in_seq && in_threads) {
        auto scan = [&](const E& e) {
          visit_exprs(e, [&](const E& x) { if (x->k == Expr::UnOpE && (x->uop == UnOp::Exp || x->uop == UnOp::Log)) transcendental = true; });
        };
        scan(st->expr);
        scan(st->dst);
      }
      bool seq = st->k == Stmt::For && st->map.k == GpuMap::None && !st->unroll;
      bool thr = st->k == Stmt::For && st->map.k == GpuMap::Thread;
      // (reductions of a whole row every few steps are not the step body: only straight element loops count)
      bool reduction_like = thr && st->par.reduction;
      walk(st->body, in_seq || seq, in_threads || (thr && !reduction_like));
      walk(st->els, in_seq, in_threads);
    }
  };
  walk(k.body, false, false);
  return transcendental;
}

// hoist out of the sequential loop `seq` (a statement of `parent`)
Stmts Pass::hoist_from_seq_loop(const S& seq, int64_t* budget) {
  std::set<Name> params = param_names();
  std::set<Name> written = written_arrays();
  std::set<Name> reassigned;
  visit_stmts(k.body, [&](const S& s) { if (s->k == Stmt::Assign && s->dst->k == Expr::Var) reassigned.insert(s->dst->name); });

  Stmts pre;  // statements to run before the sequential loop
  std::function<Stmts(const Stmts&)> walk = [&](const Stmts& ss) -> Stmts {
    Stmts out;
    for (auto& s : ss) {
      IterSpace is;
      if (thread_mapped(s) && iter_space(s, &is)) {
        // definitions inside the body that are pure functions of the iteration
        std::map<Name, E> defs;
        std::set<Name> iter_vars{s->id};
        if (is.inner) iter_vars.insert(is.inner->id);
        std::function<void(const Stmts&)> collect_defs = [&](const Stmts& b) {
          for (auto& c : b) {
            if (c->k == Stmt::Def && c->ty.is_scalar() && !reassigned.count(c->id) && !has_load(c->expr)) {
              E e = subst_vars(c->expr, defs);
              bool pure = true;
              visit_exprs(e, [&](const E& x) { if (x->k == Expr::Var && !iter_vars.count(x->name)) pure = false; });
              if (pure) defs[c->id] = e;
            }
            collect_defs(c->body);
            collect_defs(c->els);
          }
        };
        collect_defs(*is.body);
        RangeEnv env;
        {
          Interval r;
          r.known = true;
          r.lo = s->lo->iv;
          r.hi = s->hi->iv - 1;
          env[s->id] = r;
          if (is.inner) { Interval u; u.known = true; u.lo = 0; u.hi = const_extent(is.inner) - 1; env[is.inner->id] = u; }
        }
        std::vector<Hoisted> hoisted;
        auto try_hoist = [&](const E& e) -> E {
          if (e->k != Expr::Index || e->args[0]->k != Expr::Var) return e;
          const Name& base = e->args[0]->name;
          if (!params.count(base) || written.count(base) || e->dim_shape.empty()) return e;
          E idx = fold_expr(subst_vars(e->args[1], defs));
          bool pure = true;
          visit_exprs(idx, [&](const E& x) {
            if (x->k == Expr::Var && !iter_vars.count(x->name)) pure = false;
            if (x->k == Expr::Index || x->k == Expr::RegElem || x->k == Expr::ThreadIdx || x->k == Expr::BlockIdx) pure = false;
          });
          if (!pure) return e;
          int64_t numel = 1;
          for (auto d : e->dim_shape) numel *= d;
          Interval r = expr_range(idx, env);
          if (!r.known || r.lo < 0 || r.hi >= numel) return e;  // the load is executed unconditionally once hoisted
          for (auto& h : hoisted)
            if (h.load->k == Expr::Index && h.load->args[0]->name == base && expr_eq(h.load->args[1], idx)) {
              auto re = std::make_shared<Expr>();
              re->k = Expr::RegElem;
              re->ty = e->ty;
              re->name = h.reg;
              re->args = {is.slot};
              return re;
            }
          int64_t cost = is.slots * std::max(1, elem_bytes(e->ty.sz) / 4);
          if (*budget < cost) return e;
          *budget -= cost;
          Hoisted h;
          auto ld = std::make_shared<Expr>(*e);
          ld->args = {e->args[0], idx};
          h.load = ld;
          h.reg = gen.fresh("inv_" + base.s);
          h.sz = e->ty.sz;
          hoisted.push_back(h);
          auto re = std::make_shared<Expr>();
          re->k = Expr::RegElem;
          re->ty = e->ty;
          re->name = h.reg;
          re->args = {is.slot};
          return re;
        };
        Stmts nbody = rewrite_stmts(*is.body, try_hoist);
        // Arithmetic whose operands are all hoisted values (or literals) is invariant too: `trans1[..] +
        // trans2[..]` is computed once and takes one register per element instead of two.  Only values
        // with a single use are combined, so the register count never grows; same operations in the
        // same order, hence the same bits.
        {
          // `t = hoisted[slot]` is only a name for the value: uses of t become the register element
          std::map<Name, E> alias;
          visit_stmts(nbody, [&](const S& st) {
            if (st->k == Stmt::Def && st->expr && st->expr->k == Expr::RegElem && !reassigned.count(st->id)) alias[st->id] = st->expr;
          });
          if (!alias.empty()) {
            std::function<Stmts(const Stmts&)> drop = [&](const Stmts& b) {
              Stmts o;
              for (auto& c : b) {
                if (c->k == Stmt::Def && alias.count(c->id)) continue;
                auto n = clone(c);
                n->body = drop(c->body);
                n->els = drop(c->els);
                o.push_back(n);
              }
              return o;
            };
            nbody = rewrite_stmts(drop(nbody), [&](const E& x) -> E {
              if (x->k != Expr::Var) return x;
              auto it = alias.find(x->name);
              return it == alias.end() ? x : it->second;
            });
          }
        }
        for (bool changed = true; changed;) {
          changed = false;
          std::map<Name, int> uses;
          visit_stmts(nbody, [&](const S& st) {
            auto scan = [&](const E& root) { visit_exprs(root, [&](const E& x) { if (x->k == Expr::RegElem) uses[x->name]++; }); };
            scan(st->dst); scan(st->expr); scan(st->lo); scan(st->hi);
          });
          auto index_of = [&](const Name& r) { for (size_t q = 0; q < hoisted.size(); ++q) if (hoisted[q].reg == r) return (int)q; return -1; };
          auto merge = [&](const E& e) -> E {
            if (e->k != Expr::BinOpE || !e->ty.is_scalar() || elem_bytes(e->ty.sz) > 4) return e;
            if (!(e->bop == BinOp::Add || e->bop == BinOp::Sub || e->bop == BinOp::Mul || e->bop == BinOp::Max || e->bop == BinOp::Min)) return e;
            auto reg = [&](const E& x) { return x->k == Expr::RegElem && index_of(x->name) >= 0 && expr_eq(x->args[0], is.slot); };
            auto lit = [](const E& x) { return x->k == Expr::Float || x->k == Expr::Int; };
            const E &a = e->args[0], &b = e->args[1];
            if (!((reg(a) && (reg(b) || lit(b))) || (lit(a) && reg(b)))) return e;
            if (reg(a) && reg(b) && a->name == b->name) return e;
            // the combined value takes the place of an operand that has no other use, so registers never grow
            if (!((reg(a) && uses[a->name] == 1) || (reg(b) && uses[b->name] == 1))) return e;
            Hoisted h;
            E la = reg(a) ? hoisted[index_of(a->name)].load : a, lb = reg(b) ? hoisted[index_of(b->name)].load : b;
            h.load = mk_binop(e->bop, la, lb, e->ty, e->i);
            h.reg = gen.fresh("inv_expr");
            h.sz = e->ty.sz;
            if (reg(a)) uses[a->name]--;
            if (reg(b)) uses[b->name]--;
            hoisted.push_back(h);
            uses[h.reg] = 1;
            changed = true;
            auto re = std::make_shared<Expr>();
            re->k = Expr::RegElem;
            re->ty = e->ty;
            re->name = h.reg;
            re->args = {is.slot};
            return re;
          };
          nbody = rewrite_stmts(nbody, merge);
        }
        {
          std::map<Name, int> uses;
          visit_stmts(nbody, [&](const S& st) {
            auto scan = [&](const E& root) { visit_exprs(root, [&](const E& x) { if (x->k == Expr::RegElem) uses[x->name]++; }); };
            scan(st->dst); scan(st->expr); scan(st->lo); scan(st->hi);
          });
          std::vector<Hoisted> live;
          for (auto& h : hoisted) {
            int64_t cost = is.slots * std::max(1, elem_bytes(h.sz) / 4);
            if (uses[h.reg] > 0) live.push_back(h);
            else if (h.load->k == Expr::Index) *budget += cost;   // a load that only feeds a combined value
          }
          for (auto& h : live)
            if (h.load->k != Expr::Index) *budget -= is.slots * std::max(1, elem_bytes(h.sz) / 4);
          hoisted = live;
        }
        // Values picked by tests on the iteration alone (`layer == 15 ? gamma : layer == 14 ? tail : 0`, and the
        // predecessor index chosen the same way) are invariant as well: a compare and a select per test and
        // step otherwise.  The largest such expressions move into a register per iteration.
        {
                      std::function<bool(const E&)> has_select = [&](const E& e) {
            bool f = false;
            visit_exprs(e, [&](const E& x) { if (x->k == Expr::IfExpr) f = true; });
            return f;
          };
          std::function<E(const E&)> pick = [&](const E& e) -> E {
            if (!e) return e;
            if (e->k == Expr::IfExpr && e->ty.is_scalar() && has_select(e)) {
              E v = fold_expr(subst_vars(e, defs));
              bool pure = true;
              visit_exprs(v, [&](const E& x) {
                if (x->k == Expr::Var && !iter_vars.count(x->name)) pure = false;
                if (x->k == Expr::Index || x->k == Expr::RegElem || x->k == Expr::ThreadIdx || x->k == Expr::BlockIdx || x->k == Expr::Call ||
                    x->k == Expr::Raw || x->k == Expr::AddrOf)
                  pure = false;
              });
              int64_t cost = is.slots * std::max(1, elem_bytes(e->ty.sz) / 4);
              if (pure && *budget >= cost) {
                for (auto& h : hoisted)
                  if (h.load->k != Expr::Index && expr_eq(h.load, v)) {
                    auto re = std::make_shared<Expr>();
                    re->k = Expr::RegElem; re->ty = e->ty; re->name = h.reg; re->args = {is.slot};
                    return re;
                  }
                *budget -= cost;
                Hoisted h;
                h.load = v;
                h.reg = gen.fresh("inv_pick");
                h.sz = e->ty.sz;
                hoisted.push_back(h);
                auto re = std::make_shared<Expr>();
                re->k = Expr::RegElem; re->ty = e->ty; re->name = h.reg; re->args = {is.slot};
                return re;
              }
            }
            return map_children(e, pick);
          };
          std::function<Stmts(const Stmts&)> walk_picks = [&](const Stmts& b) {
            Stmts o;
            for (auto& c : b) {
              auto nn = clone(c);
              if (c->k == Stmt::Assign || c->k == Stmt::Def) nn->expr = pick(c->expr);
              nn->body = walk_picks(c->body);
              nn->els = walk_picks(c->els);
              o.push_back(nn);
            }
            return o;
          };
          nbody = walk_picks(nbody);
        }
        if (hoisted.empty()) { out.push_back(s); continue; }
        // loop nest that fills the registers, with the same thread mapping
        std::map<Name, Name> ren;
        Name nq = gen.fresh(s->id.s);
        ren[s->id] = nq;
        Name nu;
        if (is.inner) { nu = gen.fresh(is.inner->id.s); ren[is.inner->id] = nu; }
        std::map<Name, E> rv;
        Type ity = Type::scalar(isz);
        for (auto& kv : ren) rv[kv.first] = mk_var(kv.second, ity);
        auto fill_outer = clone(s);
        fill_outer->id = nq;
        fill_outer->unroll = true;
        // the counter of the fill loop has its own name: rebuild the slot expression for it
        E fill_slot;
        {
          E kq = counter_var(fill_outer, isz);
          if (is.inner) {
            int64_t V = const_extent(is.inner);
            fill_slot = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, kq, mk_int(V, isz), ity), mk_var(nu, ity), ity));
          } else {
            fill_slot = kq;
          }
        }
        Stmts fills;
        for (auto& h : hoisted) {
          auto d = std::make_shared<Stmt>();
          d->k = Stmt::RegDecl;
          d->id = h.reg;
          d->ty = Type::scalar(h.sz);
          d->iv = is.slots;
          pre.push_back(d);
          auto re = std::make_shared<Expr>();
          re->k = Expr::RegElem;
          re->ty = Type::scalar(h.sz);
          re->name = h.reg;
          re->args = {fill_slot};
          E ld = rewrite_expr(subst_vars(h.load, rv), [](const E& x) -> E {
            if (x->k != Expr::Index || x->dim_idx.empty()) return x;
            auto c = std::make_shared<Expr>(*x);
            c->dim_idx.clear();
            return c;
          });
          fills.push_back(mk_assign(re, ld));
        }
        if (is.inner) {
          auto fi = clone(is.inner);
          fi->id = nu;
          fi->body = fills;
          fill_outer->body = {S(fi)};
        } else {
          fill_outer->body = fills;
        }
        pre.push_back(fill_outer);
        // the loop itself must be fully unrolled so that the arrays stay in registers
        auto ns = clone(s);
        ns->unroll = true;
        if (is.inner) {
          auto ni = clone(is.inner);
          ni->body = nbody;
          ns->body = {S(ni)};
        } else {
          ns->body = nbody;
        }
        out.push_back(ns);
        continue;
      }
      auto r = clone(s);
      r->body = walk(s->body);
      r->els = walk(s->els);
      out.push_back(r);
    }
    return out;
  };
  auto nseq = clone(seq);
  nseq->body = walk(seq->body);
  pre.push_back(nseq);
  return pre;
}

Stmts Pass::hoist_invariant(const Stmts& ss, int64_t* budget, bool in_seq) {
  Stmts out;
  for (auto& s : ss) {
    bool seq = (s->k == Stmt::For && s->map.k == GpuMap::None && !s->unroll) || s->k == Stmt::While;
    if (seq && !in_seq) {
      for (auto& r : hoist_from_seq_loop(s, budget)) out.push_back(r);
      continue;
    }
    auto r = clone(s);
    r->body = hoist_invariant(s->body, budget, in_seq);
    r->els = hoist_invariant(s->els, budget, in_seq);
    out.push_back(r);
  }
  return out;
}

// ================================================================ what the iterations of one thread share
// A parallel loop of `per * N` iterations on N threads gives thread g the iterations g, g + N, ..., g + (per-1) N.
// When N is a multiple of what the body divides by, much of the body is the same in all of them: with one thread
// per k-mer of a 16-layer model (`state = g + layer * N`) the four predecessors `(state // 4) % (N // 4)`, their
// table rows, their scores and the emission `output_prob[o, state % N]` depend on g alone.  The loop variable is
// replaced by `g + k * N`, quotients and remainders of such sums are taken apart where the constants divide
// ((a + k * N) // c = a // c + k * (N // c), (a + k * N) % c = a % c for c | N and a, k >= 0; a // c = 0 and
// a % c = a where the range of a says so), and the largest subexpressions that are free of k -- loads
// included -- are evaluated once per thread in front of the counted loop (the statements kept in `els` of the
// loop, printed before it).  A load may move there because the iterations of a parallel loop do not depend on
// each other: what one reads no other writes.  On top of that the array must not be stored to by name in the
// body, and must be either never written by the kernel or known to differ from every array the body stores to
// (pointer parameters carry the no-alias promise; local pointers that never coincide).
struct Pass::OwnIterations {
  Pass& p;
  Name gname, kname;
  int64_t N = 0, per = 0;
  RangeEnv env;
  std::set<Name> variant;            // names whose value changes with k
  std::set<Name> stored;             // arrays the body stores to
  std::set<Name> never_written;      // parameters the kernel only reads
  Stmts pre;
  ElemSize isz;

  bool divides_all(const E& e, int64_t c) const {   // e is a multiple of c for every value of its variables
    if (e->k == Expr::Int) return e->iv % c == 0;
    if (e->k == Expr::Convert) return divides_all(e->args[0], c);
    if (e->k != Expr::BinOpE) return false;
    if (e->bop == BinOp::Mul)
      return (e->args[0]->k == Expr::Int && e->args[0]->iv % c == 0) || (e->args[1]->k == Expr::Int && e->args[1]->iv % c == 0);
    if (e->bop == BinOp::Add) return divides_all(e->args[0], c) && divides_all(e->args[1], c);
    return false;
  }
  bool non_negative(const E& e) const {
    Interval r = expr_range(e, env);
    return r.known && r.lo >= 0;
  }
  E divide(const E& e, int64_t c) const {            // e / c for e with divides_all(e, c)
    if (e->k == Expr::Int) return mk_int(e->iv / c, e->ty.sz, e->i);
    if (e->k == Expr::Convert) return mk_convert(divide(e->args[0], c), e->ty.sz);
    if (e->bop == BinOp::Mul) {
      if (e->args[0]->k == Expr::Int && e->args[0]->iv % c == 0)
        return fold_expr(mk_binop(BinOp::Mul, mk_int(e->args[0]->iv / c, e->args[0]->ty.sz), e->args[1], e->ty, e->i));
      return fold_expr(mk_binop(BinOp::Mul, e->args[0], mk_int(e->args[1]->iv / c, e->args[1]->ty.sz), e->ty, e->i));
    }
    return fold_expr(mk_binop(BinOp::Add, divide(e->args[0], c), divide(e->args[1], c), e->ty, e->i));
  }
  E simplify(const E& e0) const {
    return rewrite_expr(e0, [&](const E& e) -> E {
      if (e->k != Expr::BinOpE || !e->ty.is_scalar() || !is_int(e->ty.sz)) return e;
      bool div = e->bop == BinOp::FloorDiv || e->bop == BinOp::Div, rem = e->bop == BinOp::Rem;
      if (!(div || rem) || e->args[1]->k != Expr::Int || e->args[1]->iv <= 0) return e;
      int64_t c = e->args[1]->iv;
      const E& a = e->args[0];
      Interval r = expr_range(a, env);
      if (r.known && r.lo >= 0 && r.hi < c) return div ? mk_int(0, e->ty.sz, e->i) : a;
      if (a->k == Expr::BinOpE && a->bop == BinOp::Add && a->ty == e->ty) {
        for (int side = 0; side < 2; ++side) {
          const E &m = a->args[side], &rest = a->args[1 - side];
          if (!divides_all(m, c) || !non_negative(m) || !non_negative(rest)) continue;
          if (rem) return simplify(mk_binop(BinOp::Rem, rest, e->args[1], e->ty, e->i));
          return fold_expr(mk_binop(BinOp::Add, simplify(mk_binop(e->bop, rest, e->args[1], e->ty, e->i)), divide(m, c), e->ty, e->i));
        }
      }
      return e;
    });
  }
  bool load_may_move(const E& x) const {
    if (x->args[0]->k != Expr::Var) return false;
    const Name& b = x->args[0]->name;
    if (stored.count(b)) return false;
    if (never_written.count(b)) return true;
    for (auto& sb : stored)
      if (!p.distinct_names(b, sb)) return false;
    return true;
  }
  bool shared(const E& e) const {                    // the same in every iteration of the thread
    bool ok = true;
    visit_exprs(e, [&](const E& x) {
      if (x->k == Expr::Var && (x->name == kname || variant.count(x->name))) ok = false;
      if (x->k == Expr::Index && !load_may_move(x)) ok = false;
      if (x->k == Expr::Call || x->k == Expr::Raw || x->k == Expr::RegElem || x->k == Expr::AddrOf) ok = false;
    });
    return ok;
  }
  static bool worth(const E& e) {
    bool w = false;
    visit_exprs(e, [&](const E& x) {
      if (x->k == Expr::Index) w = true;
      if (x->k == Expr::BinOpE && (x->bop == BinOp::FloorDiv || x->bop == BinOp::Div || x->bop == BinOp::Rem)) w = true;
    });
    return w;
  }
  E lift(const E& e) {
    if (!e) return e;
    if (e->ty.is_scalar() && shared(e) && worth(e)) {
      for (auto& d : pre)
        if (d->k == Stmt::Def && d->ty == e->ty && expr_eq(d->expr, e)) return mk_var(d->id, d->ty, e->i);
      Name n = p.gen.fresh("own");
      pre.push_back(mk_def(n, e->ty, e, e->i));
      Interval r = expr_range(e, env);
      if (r.known) env[n] = r;
      return mk_var(n, e->ty, e->i);
    }
    // what a selection or a short-circuit operator may skip stays where it is (a test can guard an index)
    if (e->k == Expr::IfExpr || (e->k == Expr::BinOpE && (e->bop == BinOp::And || e->bop == BinOp::Or))) {
      auto n = std::make_shared<Expr>(*e);
      n->args[0] = lift(e->args[0]);
      return n;
    }
    return map_children(e, [&](const E& c) { return lift(c); });
  }
};

bool Pass::distinct_names(const Name& a, const Name& b) const {
  if (a == b) return false;
  bool pa = false, pb = false;
  for (auto& q : k.params) {
    if (!q.ty.is_pointer()) continue;
    pa = pa || q.id == a;
    pb = pb || q.id == b;
  }
  if (pa && pb && !k.no_restrict) return true;
  for (auto& g : k.distinct_pointers)
    if (std::find(g.begin(), g.end(), a) != g.end() && std::find(g.begin(), g.end(), b) != g.end()) return true;
  return false;
}

Stmts Pass::share_own_iterations(const Stmts& ss) {
  Stmts out;
  for (auto& s : ss) {
    bool mapped = s->k == Stmt::For && (s->map.k == GpuMap::Thread || s->map.k == GpuMap::ThreadBlock);
    int64_t extent = mapped ? const_extent(s) : -1;
    bool fits = mapped && s->els.empty() && s->step == 1 && extent > 0 && s->lo->iv == 0 && extent % s->map.n == 0 &&
                extent / s->map.n > 1 && (s->map.k == GpuMap::Thread || s->map.n % s->map.tpb == 0) && !s->unroll;
    if (fits) {
      for (auto& c : s->body)
        if (c->k != Stmt::Def && c->k != Stmt::Assign) fits = false;
      visit_stmts(s->body, [&](const S& c) {
        visit_stmt_exprs(c, [&](const E& x) { if (x->k == Expr::RegElem || x->k == Expr::AddrOf) fits = false; });
      });
    }
    if (!fits) {
      auto r = clone(s);
      r->body = share_own_iterations(s->body);
      if (s->k != Stmt::For) r->els = share_own_iterations(s->els);
      out.push_back(r);
      continue;
    }
    OwnIterations oi{*this};
    oi.isz = isz;
    oi.N = s->map.n;
    oi.per = extent / s->map.n;
    oi.gname = Name{s->id.str() + "_g", 0};
    oi.kname = Name{s->id.str() + "_k", 0};
    Type ity = s->lo->ty;
    Interval gr, kr;
    gr.known = kr.known = true;
    gr.lo = kr.lo = 0;
    gr.hi = oi.N - 1;
    kr.hi = oi.per - 1;
    oi.env[oi.gname] = gr;
    oi.env[oi.kname] = kr;
    std::set<Name> written = written_arrays();
    for (auto& q : k.params)
      if (q.ty.is_pointer() && !written.count(q.id)) oi.never_written.insert(q.id);
    std::set<Name> defined, reassigned;
    bool ok = true;
    for (auto& c : s->body) {
      if (c->k == Stmt::Def) defined.insert(c->id);
      if (c->k == Stmt::Assign && c->dst->k == Expr::Var) {
        if (!defined.count(c->dst->name)) ok = false;   // a value that lives across iterations: not ours to move
        reassigned.insert(c->dst->name);
      }
      if (c->k == Stmt::Assign && c->dst->k == Expr::Index) {
        if (c->dst->args[0]->k == Expr::Var) oi.stored.insert(c->dst->args[0]->name); else ok = false;
      }
    }
    if (!ok) { out.push_back(s); continue; }
    oi.variant = reassigned;
    E sum = mk_binop(BinOp::Add, mk_var(oi.gname, ity), mk_binop(BinOp::Mul, mk_var(oi.kname, ity), mk_int(oi.N, ity.sz), ity), ity);
    std::map<Name, E> sub;
    sub[s->id] = sum;
    Stmts body;
    for (auto& c : s->body) {
      auto r = clone(c);
      E e = oi.simplify(fold_expr(subst_vars(c->expr, sub)));
      if (c->k == Stmt::Def && c->ty.is_scalar() && !reassigned.count(c->id) && oi.shared(e)) {
        // the whole definition is the same for all iterations of the thread
        r->expr = e;
        oi.pre.push_back(r);
        Interval rg = expr_range(e, oi.env);
        if (rg.known) oi.env[c->id] = rg;
        continue;
      }
      r->expr = oi.lift(e);
      if (c->k == Stmt::Def) {
        oi.variant.insert(c->id);
        Interval rg = expr_range(r->expr, oi.env);
        if (rg.known && !reassigned.count(c->id)) oi.env[c->id] = rg;
      } else if (c->dst->k == Expr::Index) {
        r->dst = map_children(c->dst, [&](const E& x) { return oi.lift(oi.simplify(fold_expr(subst_vars(x, sub)))); });
      }
      body.push_back(r);
    }
    if (oi.pre.empty()) { out.push_back(s); continue; }
    auto ns = clone(s);
    ns->body = body;
    ns->els = oi.pre;
    out.push_back(ns);
  }
  return out;
}

// ================================================================ register caching across parallel loops
// Consecutive thread-mapped loops with the same iteration structure give each
// thread the same elements every time.  An array that is only ever accessed
// as a[inv + d] inside those loops (d the loop's element) is therefore private
// to the thread between them: it is read from memory once, kept in registers
// across the loops (and the block synchronisations between them), and written
// back by the last loop that stores to it.
void Pass::reg_cache(int64_t* budget) {
  if (k.body.size() != 1 || k.body[0]->k != Stmt::For || k.body[0]->map.k != GpuMap::Block) return;
  const S root = k.body[0];
  struct Cand { size_t pos; S loop; IterSpace is; Name elem; };
  std::vector<Cand> cands;
  for (size_t pos = 0; pos < root->body.size(); ++pos) {
    const S& s = root->body[pos];
    Cand c;
    if (!thread_mapped(s) || !iter_space(s, &c.is)) continue;
    c.pos = pos;
    c.loop = s;
    // element variable: the loop variable, or the definition at the head of the unrolled element loop
    if (c.is.inner) {
      if (c.is.body->empty() || (*c.is.body)[0]->k != Stmt::Def) continue;
      c.elem = (*c.is.body)[0]->id;
    } else {
      c.elem = s->id;
    }
    cands.push_back(c);
  }
  if (cands.size() < 2) return;
  // loops must agree on extent, mapping and element width
  auto same = [&](const Cand& a, const Cand& b) {
    return const_extent(a.loop) == const_extent(b.loop) && a.loop->map.n == b.loop->map.n && a.is.slots == b.is.slots &&
           a.loop->lo->iv == b.loop->lo->iv && (a.is.inner != nullptr) == (b.is.inner != nullptr);
  };
  std::vector<Cand> group;
  for (auto& c : cands)
    if (same(cands[0], c)) group.push_back(c);
  if (group.size() < 2) return;
  std::map<Name, size_t> elem_loop;  // element variable -> index in group
  for (size_t g = 0; g < group.size(); ++g) elem_loop[group[g].elem] = g;

  // arrays: every access in the kernel is a[inv + elem] inside a group loop, with one common inv
  struct Arr { bool ok = true; E inv; ElemSize sz = ElemSize::F32; std::vector<bool> reads, writes; bool seen = false; };
  std::map<Name, Arr> arrs;
  for (auto& p : k.params)
    if (p.ty.is_pointer()) { Arr a; a.reads.assign(group.size(), false); a.writes.assign(group.size(), false); arrs[p.id] = a; }
  std::set<Name> locals;  // pointer aliases defeat the analysis: any array reachable through one is left alone
  visit_stmts(k.body, [&](const S& s) {
    if ((s->k == Stmt::Def && !s->ty.is_scalar()) || (s->k == Stmt::Assign && s->dst->k == Expr::Var && !s->dst->ty.is_scalar()))
      visit_exprs(s->expr, [&](const E& x) { if (x->k == Expr::Var && arrs.count(x->name)) arrs[x->name].ok = false; });
  });
  std::function<void(const E&, int, bool)> scan = [&](const E& e, int g, bool store) {
    if (!e) return;
    if ((e->k == Expr::Index || e->k == Expr::AddrOf) && e->args[0]->k == Expr::Var && arrs.count(e->args[0]->name)) {
      Arr& a = arrs[e->args[0]->name];
      E inv;
      bool good = e->k == Expr::Index && g >= 0 && affine_unit(e->args[1], group[g].elem, &inv);
      if (good) {
        // inv must be uniform over the block: only the root variable and constants
        visit_exprs(inv, [&](const E& x) {
          if (x->k == Expr::Var && x->name != root->id) good = false;
          if (x->k == Expr::Index || x->k == Expr::ThreadIdx || x->k == Expr::RegElem) good = false;
        });
      }
      if (good && a.seen && (!expr_eq(a.inv, inv) || a.sz != e->ty.sz)) good = false;
      if (!good) a.ok = false;
      else {
        a.seen = true;
        a.inv = inv;
        a.sz = e->ty.sz;
        (store ? a.writes : a.reads)[g] = true;
      }
      scan(e->args[1], g, false);
      return;
    }
    if (e->k == Expr::Var && arrs.count(e->name)) { arrs[e->name].ok = false; return; }
    for (auto& c : e->args) scan(c, g, false);
  };
  // accesses under a condition inside a loop body are not cached: a register
  // slot that was neither loaded nor written must never be stored back
  std::function<void(const Stmts&, int, bool)> scan_stmts = [&](const Stmts& ss, int g, bool cond) {
    for (auto& s : ss) {
      int gg = g;
      if (g < 0)
        for (size_t i = 0; i < group.size(); ++i)
          if (group[i].loop == s) gg = (int)i;
      int ag = cond ? -1 : gg;  // a conditional access is treated like one outside the loops
      if (s->dst) scan(s->dst, ag, s->k == Stmt::Assign);
      if (s->expr) scan(s->expr, ag, false);
      if (s->lo) scan(s->lo, ag, false);
      if (s->hi) scan(s->hi, ag, false);
      for (auto& a : s->args) scan(a, ag, false);
      bool c = cond || (gg >= 0 && (s->k == Stmt::If || s->k == Stmt::While));
      scan_stmts(s->body, gg, c);
      scan_stmts(s->els, gg, c);
    }
  };
  scan_stmts(k.body, -1, false);

  struct Chosen { Name arr, reg; ElemSize sz; E inv; int first, last, last_write; bool load_first; int64_t cost; };
  std::vector<Chosen> chosen;
  int64_t slots = group[0].is.slots;
  // Registers are budgeted by what is live at once, loop by loop: an array occupies its slots from the first
  // loop that touches it to the last.  Where one array is read for the last time in the very loop that first
  // writes another (out[e] = f(x[e]) with x dead afterwards), each iteration frees a slot as it fills one,
  // so the pair needs the larger of the two, not the sum.
  const int G = (int)group.size();
  auto peak_with = [&](const std::vector<Chosen>& cs) {
    int64_t peak = 0;
    for (int g = 0; g < G; ++g) {
      int64_t live = 0, dying = 0, born = 0;
      for (auto& c : cs) {
        if (c.first > g || c.last < g) continue;
        live += c.cost;
        if (c.last == g && c.first < g) dying += c.cost;
        if (c.first == g && !c.load_first && c.last > g) born += c.cost;
      }
      peak = std::max(peak, live - std::min(dying, born));
    }
    return peak;
  };
  for (auto& p : k.params) {
    auto it = arrs.find(p.id);
    if (it == arrs.end() || !it->second.ok || !it->second.seen) continue;
    const Arr& a = it->second;
    int touched = 0, first = -1, last = -1, last_write = -1;
    for (size_t g = 0; g < group.size(); ++g) {
      if (a.reads[g] || a.writes[g]) { ++touched; if (first < 0) first = (int)g; last = (int)g; }
      if (a.writes[g]) last_write = (int)g;
    }
    if (touched < 2) continue;
    // registers that would be held through a whole sequential loop between two of the array's loops (the copy
    // into LDS in front of a time loop and the copy back behind it) cost every step of that loop a register
    // per slot and save one load: not cached
    bool spans_loop = false;
    for (size_t pos = group[first].pos + 1; pos < group[last].pos; ++pos) {
      const S& between = root->body[pos];
      if (between->k == Stmt::For && between->map.k == GpuMap::None && !between->unroll) spans_loop = true;
      if (between->k == Stmt::While) spans_loop = true;
    }
    if (spans_loop) continue;
    Chosen c;
    c.arr = p.id;
    c.sz = a.sz;
    c.inv = a.inv;
    c.first = first;
    c.last = last;
    c.last_write = last_write;
    c.load_first = a.reads[first];
    c.cost = slots * std::max(1, elem_bytes(a.sz) / 4);
    chosen.push_back(c);
    if (peak_with(chosen) > *budget) { chosen.pop_back(); continue; }
    chosen.back().reg = gen.fresh("row_" + p.id.s);
  }
  if (!chosen.empty()) *budget -= peak_with(chosen);
  if (chosen.empty()) return;

  Type ity = Type::scalar(isz);
  Stmts nb;
  for (auto& c : chosen) {
    auto d = std::make_shared<Stmt>();
    d->k = Stmt::RegDecl;
    d->id = c.reg;
    d->ty = Type::scalar(c.sz);
    d->iv = slots;
    nb.push_back(d);
  }
  for (size_t pos = 0; pos < root->body.size(); ++pos) {
    const S& s = root->body[pos];
    int g = -1;
    for (size_t i = 0; i < group.size(); ++i)
      if (group[i].loop == s) g = (int)i;
    if (g < 0) { nb.push_back(s); continue; }
    const Cand& c = group[g];
    auto reg_elem = [&](const Chosen& ch) {
      auto re = std::make_shared<Expr>();
      re->k = Expr::RegElem;
      re->ty = Type::scalar(ch.sz);
      re->name = ch.reg;
      re->args = {c.is.slot};
      return E(re);
    };
    auto global_elem = [&](const Chosen& ch) {
      E idx = fold_expr(mk_binop(BinOp::Add, ch.inv, mk_var(c.elem, ity), ity));
      return mk_index(mk_var(ch.arr, Type::pointer(ch.sz)), idx, Type::scalar(ch.sz));
    };
    auto rw = [&](const E& e) -> E {
      if (e->k == Expr::Index && e->args[0]->k == Expr::Var)
        for (auto& ch : chosen)
          if (ch.arr == e->args[0]->name) return reg_elem(ch);
      return e;
    };
    Stmts body = rewrite_stmts(*c.is.body, rw);
    Stmts head, tail;
    for (auto& ch : chosen) {
      if (g == ch.first && ch.load_first) head.push_back(mk_assign(reg_elem(ch), global_elem(ch)));
      if (g == ch.last_write) tail.push_back(mk_assign(global_elem(ch), reg_elem(ch)));
    }
    Stmts full;
    size_t start = 0;
    if (c.is.inner) { full.push_back(body[0]); start = 1; }  // the element definition stays first
    for (auto& h : head) full.push_back(h);
    for (size_t i = start; i < body.size(); ++i) full.push_back(body[i]);
    for (auto& t : tail) full.push_back(t);
    auto ns = clone(s);
    ns->unroll = true;
    if (c.is.inner) {
      auto ni = clone(c.is.inner);
      ni->body = full;
      ns->body = {S(ni)};
    } else {
      ns->body = full;
    }
    nb.push_back(ns);
  }
  auto nr = clone(root);
  nr->body = nb;
  k.body = {nr};
}

}  // namespace hipopt
}  // namespace parpy
