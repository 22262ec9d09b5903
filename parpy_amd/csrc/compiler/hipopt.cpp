// gfx950 memory code generation passes over the extracted kernels.
//
// The reference's backends print the loop nest as it stands
// (src/cuda/codegen.rs:120-358): every access goes to global memory with one
// element per thread and per iteration.  These passes restructure the kernels
// for CDNA4's memory system instead:
//
//   lds_rows        rows of arrays that only one workgroup touches (a[blk, *])
//                   and that are revisited inside an in-kernel sequential loop
//                   live in LDS for the whole kernel (160 KB per workgroup);
//   vectorize       thread-mapped loops with unit-stride accesses give every
//                   thread V consecutive elements so that loads and stores
//                   become dwordx4 / ds_*_b128;
//   hoist_invariant loads from read-only arrays whose address depends only on
//                   the thread's own iteration, inside a sequential loop, are
//                   done once before the loop into per-thread registers;
//   reg_cache       array sections that a thread alone reads and writes across
//                   consecutive parallel loops stay in registers in between;
//   hoist_uniform_conditions
//                   `for x: if (c) A else B` with c the same for every x becomes
//                   `if (c) for x: A else for x: B`;
//   drop_barriers   barriers between regions that share no written array go.
//
// Three rewrites work on the whole program because they change a launch:
//   GatherTranspose column gathers X[d, c] over an innermost sequential d read a
//                   transposed copy made by a tiled kernel in front of the launch;
//   LaneSplit       eight adjacent lanes share one iteration's sequential sum
//                   (constant bounds: 16-byte pieces of each line; bounds that
//                   are data, as in a CSR row: one element each, stride 8);
//   Coarsen         a large element-wise launch with one element per thread is
//                   cut to a quarter so that vectorize gives each thread four.
//
// Each pass can be switched off through the options (tests compare the
// results with and without them).
#include <algorithm>
#include <functional>

#include "passes.hpp"

namespace parpy {

namespace {

using StmtP = std::shared_ptr<Stmt>;
StmtP clone(const S& s) { return std::make_shared<Stmt>(*s); }

constexpr int64_t LDS_BUDGET_BYTES = 160 * 1024 - 4096;  // leave room for reduction slots

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

bool thread_mapped(const S& s) { return s->k == Stmt::For && s->map.k == GpuMap::Thread; }

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

template <class F> E rewrite_expr(const E& e, F f) {  // bottom-up rewrite
  if (!e) return e;
  E r = map_children(e, [&](const E& c) { return rewrite_expr(c, f); });
  return f(r);
}

template <class F> Stmts rewrite_stmts(const Stmts& ss, F f) {  // f : E -> E applied to every expression, deep
  Stmts out;
  for (auto& s : ss) {
    auto r = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(s, [&](const E& e) { return rewrite_expr(e, f); })));
    r->body = rewrite_stmts(s->body, f);
    r->els = rewrite_stmts(s->els, f);
    out.push_back(r);
  }
  return out;
}

struct Pass {
  Kernel& k;
  const Options& opts;
  NameGen& gen;
  ElemSize isz;

  Pass(Kernel& kernel, const Options& o, NameGen& g) : k(kernel), opts(o), gen(g), isz(o.int_size()) {}

  std::set<Name> param_names() const {
    std::set<Name> r;
    for (auto& p : k.params) r.insert(p.id);
    return r;
  }

  // ================================================================ unswitching of array aliases
  // `src = a; dst = b; if (c) { src = b; dst = a; } <rest>` becomes
  // `if (c) { <rest with src=b, dst=a> } else { <rest with src=a, dst=b> }`.
  // Every access then names its array directly, which is what lets the target
  // compiler prove that loads from one buffer do not alias stores to the other
  // (it merges and reorders LDS accesses accordingly) and what the LDS and
  // register passes below analyse.  The condition is evaluated where it was.
  struct Unswitch {
    bool failed = false;
    int clones = 0;

    static bool is_alias_type(const Type& t) { return t.k == Type::Tensor ? !t.shape.empty() : t.k == Type::Pointer; }

    E resolve(const E& e, const std::map<Name, E>& env) {
      if (e->k == Expr::Var) {
        auto it = env.find(e->name);
        return it == env.end() ? e : it->second;
      }
      return e;
    }

    // a statement that does nothing but (conditionally) repoint aliases
    bool pure_select(const S& s, const std::map<Name, E>& env) {
      if (s->k == Stmt::Assign) return s->dst->k == Expr::Var && env.count(s->dst->name) && s->expr->k == Expr::Var;
      if (s->k == Stmt::If) {
        if (s->body.empty() && s->els.empty()) return false;
        for (auto& c : s->body) if (!pure_select(c, env)) return false;
        for (auto& c : s->els) if (!pure_select(c, env)) return false;
        return true;
      }
      return false;
    }

    void apply_selects(const Stmts& ss, std::map<Name, E>& env) {
      for (auto& s : ss)
        if (s->k == Stmt::Assign) env[s->dst->name] = resolve(s->expr, env);
    }

    bool has_nested_if(const Stmts& ss) {
      for (auto& s : ss)
        if (s->k == Stmt::If) return true;
      return false;
    }

    E subst(const E& e, const std::map<Name, E>& env) {
      if (!e) return e;
      if (e->k == Expr::Var) {
        auto it = env.find(e->name);
        return it == env.end() ? e : it->second;
      }
      return map_children(e, [&](const E& c) { return subst(c, env); });
    }

    Stmts run(const Stmts& ss, size_t from, std::map<Name, E> env) {
      Stmts out;
      for (size_t i = from; i < ss.size(); ++i) {
        const S& s = ss[i];
        if (s->k == Stmt::Def && is_alias_type(s->ty) && s->expr->k == Expr::Var) {
          env[s->id] = resolve(s->expr, env);
          continue;
        }
        if (s->k == Stmt::Assign && s->dst->k == Expr::Var && env.count(s->dst->name)) {
          if (s->expr->k != Expr::Var) { failed = true; return out; }
          env[s->dst->name] = resolve(s->expr, env);
          continue;
        }
        if (s->k == Stmt::If && !env.empty() && pure_select(s, env)) {
          if (has_nested_if(s->body) || has_nested_if(s->els) || ++clones > 4) { failed = true; return out; }
          std::map<Name, E> et = env, ee = env;
          apply_selects(s->body, et);
          apply_selects(s->els, ee);
          auto n = clone(s);
          n->expr = subst(s->expr, env);
          n->body = run(ss, i + 1, et);
          n->els = run(ss, i + 1, ee);
          out.push_back(n);
          return out;
        }
        // an alias assigned anywhere else (inside a loop body, say) cannot be tracked
        bool bad = false;
        std::function<void(const Stmts&)> check = [&](const Stmts& b) {
          for (auto& c : b) {
            if (c->k == Stmt::Assign && c->dst->k == Expr::Var && env.count(c->dst->name)) bad = true;
            check(c->body);
            check(c->els);
          }
        };
        check(s->body);
        check(s->els);
        if (bad) { failed = true; return out; }
        auto n = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(s, [&](const E& e) { return subst(e, env); })));
        n->body = run(s->body, 0, env);
        n->els = run(s->els, 0, env);
        out.push_back(n);
      }
      return out;
    }
  };

  // ================================================================ short counted loops inside one iteration
  // `for u in range(4): ...` written inside the body of a parallel loop (the four states of a group, the
  // taps of a small stencil) is expanded in place: one copy of the body per value of u, with the copy's
  // local variables renamed and u replaced by its value.  Every index then depends on the thread's own
  // iteration alone, which is the form the invariant-load and register passes below work on, and the tests
  // on u fold away.  Only loops of at most 8 iterations whose body is straight-line code and value-picking
  // branches are expanded.
  static bool straight_line(const Stmts& ss) {
    for (auto& s : ss) {
      if (s->k == Stmt::If) { if (!straight_line(s->body) || !straight_line(s->els)) return false; continue; }
      if (s->k != Stmt::Def && s->k != Stmt::Assign) return false;
    }
    return true;
  }

  // Local names that are defined once with a literal value (`nq = hmm["num_states"] // 4` after the shapes
  // are known) stand for that value wherever they are read: index arithmetic written with them folds like
  // arithmetic written with the numbers, which the passes that compare offsets rely on.
  Stmts propagate_constants(const Stmts& ss) {
    std::set<Name> reassigned;
    visit_stmts(ss, [&](const S& c) {
      if (c->k == Stmt::Assign && c->dst->k == Expr::Var) reassigned.insert(c->dst->name);
    });
    std::map<Name, E> env;
    std::function<Stmts(const Stmts&)> run = [&](const Stmts& b) {
      Stmts out;
      for (auto& c : b) {
        auto fix = [&](const E& e) {
          if (env.empty()) return e;
          return fold_expr(rewrite_expr(e, [&](const E& x) -> E {
            if (x->k != Expr::Var) return x;
            auto it = env.find(x->name);
            return it == env.end() ? x : it->second;
          }));
        };
        auto r = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(c, fix)));
        if (r->k == Stmt::Def && r->expr && r->ty.is_scalar() && !reassigned.count(r->id) &&
            (r->expr->k == Expr::Int || r->expr->k == Expr::Float || r->expr->k == Expr::Bool) && r->expr->ty == r->ty) {
          env[r->id] = r->expr;   // (the definition itself stays: it is what the listing shows for the name)
        }
        r->body = run(c->body);
        r->els = run(c->els);
        out.push_back(r);
      }
      return out;
    };
    return run(ss);
  }

  static size_t count_stmts(const Stmts& ss) {
    size_t n = 0;
    visit_stmts(ss, [&](const S&) { ++n; });
    return n;
  }

  Stmts expand_short_loops(const Stmts& ss0, bool in_par) {
    // inner loops first: a short loop around a short loop is straight-line code once the inner one is expanded
    Stmts ss;
    for (auto& s : ss0) {
      if (s->body.empty() && s->els.empty()) { ss.push_back(s); continue; }
      auto r = clone(s);
      bool par = in_par || (s->k == Stmt::For && s->map.k != GpuMap::None);
      r->body = expand_short_loops(s->body, par);
      r->els = expand_short_loops(s->els, par);
      ss.push_back(r);
    }
    Stmts out;
    for (auto& s : ss) {
      int64_t n = s->k == Stmt::For && s->map.k == GpuMap::None ? const_extent(s) : -1;
      if (in_par && n >= 1 && n <= 8 && straight_line(s->body) && count_stmts(s->body) * (size_t)n <= 256) {
        std::vector<Name> locals;
        visit_stmts(s->body, [&](const S& c) { if (c->k == Stmt::Def) locals.push_back(c->id); });
        for (int64_t it = 0; it < n; ++it) {
          std::map<Name, E> sub;
          std::map<Name, Name> ren;
          sub[s->id] = mk_int(s->lo->iv + it * s->step, isz);
          for (auto& l : locals) ren[l] = gen.fresh(l.s);
          std::function<Stmts(const Stmts&)> copy = [&](const Stmts& b) {
            Stmts o;
            for (auto& c : b) {
              auto r = clone(c);
              auto fix = [&](const E& e) {
                return rewrite_expr(e, [&](const E& x) -> E {
                  if (x->k != Expr::Var) return x;
                  auto si = sub.find(x->name);
                  if (si != sub.end()) return si->second;
                  auto ri = ren.find(x->name);
                  if (ri == ren.end()) return x;
                  auto v = std::make_shared<Expr>(*x);
                  v->name = ri->second;
                  return E(v);
                });
              };
              if (r->dst) r->dst = fix(r->dst);
              if (r->expr) r->expr = fix(r->expr);
              if (r->k == Stmt::Def) r->id = ren[c->id];
              r->body = copy(c->body);
              r->els = copy(c->els);
              o.push_back(r);
            }
            return o;
          };
          for (auto& c : fold_stmts(copy(s->body))) out.push_back(c);
        }
        continue;
      }
      out.push_back(s);
    }
    return out;
  }

  // ================================================================ guards that only ever switch off
  // `for t in range(lo, hi): ... if t < X: <work>` where X does not change while the loop runs, every
  // effect of the body sits under that test and X is the same for all threads of the workgroup: once
  // t reaches X no later iteration does anything, so the loop runs to min(hi, X) and the test goes.
  // The HMM kernels walk every read to the length of the longest one this way; with the bound in the
  // loop a workgroup ends with its read (its compute unit is free for the next one) and the step no
  // longer carries the test through every state.
  static E strip_converts(const E& e) { return e->k == Expr::Convert ? strip_converts(e->args[0]) : e; }

  Stmts guards_to_bounds(const Stmts& ss) {
    std::set<Name> params = param_names();
    std::set<Name> written = written_arrays();
    Stmts out;
    for (auto& s : ss) {
      bool seq = s->k == Stmt::For && s->map.k == GpuMap::None && !s->unroll && s->step == 1;
      E bound;
      bool ok = seq;
      std::set<Name> local;
      if (seq) {
        local.insert(s->id);
        visit_stmts(s->body, [&](const S& c) {
          if (c->k == Stmt::Def || c->k == Stmt::For) local.insert(c->id);
          if (c->k == Stmt::Assign && c->dst->k == Expr::Var) local.insert(c->dst->name);
        });
      }
      auto guard_of = [&](const S& c, E* x) {
        if (c->k != Stmt::If || !c->els.empty() || c->expr->k != Expr::BinOpE) return false;
        const E &a = c->expr->args[0], &b = c->expr->args[1];
        E t, other;
        if (c->expr->bop == BinOp::Lt) { t = a; other = b; }
        else if (c->expr->bop == BinOp::Gt) { t = b; other = a; }
        else return false;
        E tv = strip_converts(t);
        if (tv->k != Expr::Var || tv->name != s->id) return false;
        bool uniform = true;
        visit_exprs(other, [&](const E& y) {
          if (y->k == Expr::Var && local.count(y->name)) uniform = false;
          if (y->k == Expr::Index && !(y->args[0]->k == Expr::Var && params.count(y->args[0]->name) && !written.count(y->args[0]->name)))
            uniform = false;
          if (y->k == Expr::Call || y->k == Expr::Raw || y->k == Expr::RegElem || y->k == Expr::ThreadIdx || y->k == Expr::AddrOf) uniform = false;
        });
        if (!uniform || !other->ty.is_scalar() || !is_int(other->ty.sz)) return false;
        *x = other;
        return true;
      };
      // statements without effects outside the iteration: definitions and assignments of the iteration's own scalars
      std::function<bool(const Stmts&)> effect_free = [&](const Stmts& b) {
        for (auto& c : b) {
          if (c->k == Stmt::Def) continue;
          if (c->k == Stmt::Assign && c->dst->k == Expr::Var) continue;
          if (c->k == Stmt::If && effect_free(c->body) && effect_free(c->els)) continue;
          return false;
        }
        return true;
      };
      int guards = 0;
      std::function<Stmts(const Stmts&)> strip = [&](const Stmts& b) -> Stmts {
        Stmts o;
        for (auto& c : b) {
          E x;
          if (guard_of(c, &x)) {
            if (bound && !expr_eq(bound, x)) { ok = false; return o; }
            bound = x;
            ++guards;
            for (auto& g : c->body) o.push_back(g);
            continue;
          }
          if (c->k == Stmt::Sync || c->k == Stmt::SyncPoint) { o.push_back(c); continue; }
          if (c->k == Stmt::For && c->map.k != GpuMap::None) {
            auto r = clone(c);
            r->body = strip(c->body);
            o.push_back(r);
            continue;
          }
          if (effect_free({c})) { o.push_back(c); continue; }
          ok = false;
          return o;
        }
        return o;
      };
      if (seq) {
        // an assignment outside the tests to a variable that lives beyond the loop would see fewer iterations
        std::set<Name> defined_inside;
        visit_stmts(s->body, [&](const S& c) { if (c->k == Stmt::Def || c->k == Stmt::For) defined_inside.insert(c->id); });
        Stmts body = strip(s->body);
        std::function<void(const Stmts&, bool)> check = [&](const Stmts& b, bool) {};
        if (ok && guards > 0) {
          bool escapes = false;
          std::function<void(const Stmts&)> scan = [&](const Stmts& b) {
            for (auto& c : b) {
              E x;
              if (guard_of(c, &x)) continue;   // what a test covers ran in the same iterations before
              if (c->k == Stmt::Assign && c->dst->k == Expr::Var && !defined_inside.count(c->dst->name)) escapes = true;
              scan(c->body);
              scan(c->els);
            }
          };
          scan(s->body);
          if (!escapes) {
            auto r = clone(s);
            E x = bound->ty.sz == s->hi->ty.sz ? bound : mk_convert(bound, s->hi->ty.sz);
            // evaluated once, in front of the loop: a load in the loop test would be repeated behind every barrier
            Name end = gen.fresh(s->id.s + "_end");
            out.push_back(mk_def(end, s->hi->ty, mk_binop(BinOp::Min, s->hi, x, s->hi->ty, s->i), s->i));
            r->hi = mk_var(end, s->hi->ty);
            r->body = guards_to_bounds(body);
            out.push_back(r);
            continue;
          }
        }
      }
      auto r = clone(s);
      r->body = guards_to_bounds(s->body);
      r->els = guards_to_bounds(s->els);
      out.push_back(r);
    }
    return out;
  }

  // ================================================================ loads that depend on the step counter alone
  // Inside a sequential loop that a workgroup walks step by step (a barrier per step), `o = data[i, t]`
  // is needed at the very start of step t and everything else of the step hangs on it (it selects the
  // emission row).  The array is never written and the address is a function of t and of values that
  // do not change in the loop, so the load for step t + 1 is issued at the start of step t into a second
  // variable: its latency passes behind a whole step of work.  The index must be provably in bounds
  // over the static range of the loop (the last iteration re-reads its own element instead of t + 1).
  Stmts prefetch_counter_loads(const Stmts& ss, RangeEnv env) {
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
  Stmts prefetch_selected_rows(const Stmts& ss, int64_t* budget) {
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

  // ================================================================ conditions no iteration changes
  // A parallel loop whose whole body is `if (c) A else B`, with c the same for every iteration (it
  // mentions neither the loop variable nor anything the body defines or assigns, and loads only from
  // arrays the kernel never writes), becomes `if (c) { loop A } else { loop B }`.  The HMM step tests
  // `t < lens[inst]` (and `t == lens[inst]` in the else branch) once per state; inside the unrolled
  // loop that is a branch between any two states, which keeps the instructions of neighbouring
  // states from being scheduled together.  Only tests with an else branch are rewritten: a plain
  // `if (c) A` the device compiler unswitches by itself, and doing it here first was measured to
  // cost 5 % on the single-layer HMM step (60.4 -> 63.4 ms; the 16-layer model gains 6 %).
  Stmts hoist_uniform_conditions(const Stmts& ss) {
    std::set<Name> params = param_names();
    std::set<Name> written = written_arrays();
    std::function<Stmts(const Stmts&)> walk = [&](const Stmts& in) -> Stmts {
      Stmts out;
      for (auto& s : in) {
        bool done = false;
        if (s->k == Stmt::For && s->map.k != GpuMap::None && s->body.size() == 1 && s->body[0]->k == Stmt::If && !s->body[0]->els.empty()) {
          const S& test = s->body[0];
          std::set<Name> local{s->id};
          visit_stmts(s->body, [&](const S& c) {
            if (c->k == Stmt::Def || c->k == Stmt::For) local.insert(c->id);
            if (c->k == Stmt::Assign && c->dst->k == Expr::Var) local.insert(c->dst->name);
          });
          bool uniform = true;
          visit_exprs(test->expr, [&](const E& x) {
            if (x->k == Expr::Var && local.count(x->name)) uniform = false;
            if (x->k == Expr::Index && !(x->args[0]->k == Expr::Var && params.count(x->args[0]->name) && !written.count(x->args[0]->name)))
              uniform = false;
            if (x->k == Expr::Call || x->k == Expr::Raw || x->k == Expr::RegElem || x->k == Expr::ThreadIdx) uniform = false;
          });
          if (uniform) {
            auto loop_over = [&](const Stmts& body) {
              auto n = clone(s);
              n->body = body;
              return walk({S(n)});
            };
            Stmts els;
            if (!test->els.empty()) els = loop_over(test->els);
            out.push_back(mk_if(test->expr, loop_over(test->body), els, test->i));
            done = true;
          }
        }
        if (done) continue;
        auto r = clone(s);
        r->body = walk(s->body);
        r->els = walk(s->els);
        out.push_back(r);
      }
      return out;
    };
    return walk(ss);
  }

  // ================================================================ branches that only pick values
  // `if (c) { x = a; y = b } else { x = d }` where every statement assigns a scalar variable a value that
  // is free to compute either way (no memory access, no call, no division) becomes
  // `x = c ? a : d; y = c ? b : y`.  The HMM step picks the predecessor and the score of the stay
  // transition with an if / elif / else over the duration layer of the state; as branches these were
  // eight execution-mask regions per sixteen states in the unrolled loop.
  Stmts if_convert(const Stmts& ss) {
    // variables that stand for a non-zero integer constant (`num_kmers = 1024`): dividing by them is safe to do early
    std::set<Name> reassigned, nonzero_const;
    visit_stmts(k.body, [&](const S& st) { if (st->k == Stmt::Assign && st->dst->k == Expr::Var) reassigned.insert(st->dst->name); });
    visit_stmts(k.body, [&](const S& st) {
      if (st->k == Stmt::Def && st->expr && st->expr->k == Expr::Int && st->expr->iv != 0 && !reassigned.count(st->id)) nonzero_const.insert(st->id);
    });
    return if_convert(ss, nonzero_const);
  }

  Stmts if_convert(const Stmts& ss, const std::set<Name>& nonzero_const) {
    auto cheap = [&](const E& e) {
      bool ok = true;
      visit_exprs(e, [&](const E& x) {
        if (x->k == Expr::Index || x->k == Expr::AddrOf || x->k == Expr::Call || x->k == Expr::Raw || x->k == Expr::RegElem) ok = false;
        if (x->k == Expr::BinOpE && (x->bop == BinOp::Div || x->bop == BinOp::FloorDiv || x->bop == BinOp::Rem) &&
            !((x->args[1]->k == Expr::Int && x->args[1]->iv != 0) || (x->args[1]->k == Expr::Var && nonzero_const.count(x->args[1]->name))))
          ok = false;
        if (x->k == Expr::BinOpE && x->bop == BinOp::Pow) ok = false;
      });
      return ok;
    };
    // a branch qualifies if it is a list of assignments to distinct scalar variables, none of which reads a
    // variable assigned in the same `if` (either branch): then the order of the selects does not matter
    auto values = [&](const Stmts& branch, std::vector<std::pair<E, E>>* out) {
      for (auto& st : branch) {
        if (st->k != Stmt::Assign || st->dst->k != Expr::Var || !st->dst->ty.is_scalar() || !cheap(st->expr)) return false;
        for (auto& kv : *out)
          if (kv.first->name == st->dst->name) return false;
        out->push_back({st->dst, st->expr});
      }
      return true;
    };
    Stmts out;
    for (auto& s : ss) {
      auto r = clone(s);
      r->body = if_convert(s->body, nonzero_const);
      r->els = if_convert(s->els, nonzero_const);
      bool done = false;
      // (the test itself is evaluated once, as before, so it may read memory)
      bool plain_test = true;
      if (r->k == Stmt::If)
        visit_exprs(r->expr, [&](const E& x) { if (x->k == Expr::Call || x->k == Expr::Raw || x->k == Expr::AddrOf) plain_test = false; });
      if (r->k == Stmt::If && plain_test && !(r->body.empty() && r->els.empty())) {
        std::vector<std::pair<E, E>> thn, els;
        if (values(r->body, &thn) && values(r->els, &els)) {
          std::set<Name> assigned;
          for (auto& kv : thn) assigned.insert(kv.first->name);
          for (auto& kv : els) assigned.insert(kv.first->name);
          bool independent = true;
          // (a value may read the variable it is assigned to -- its previous value, as in `w = c ? a : w` -- but no other)
          auto reads_assigned = [&](const E& e, const Name* self) {
            visit_exprs(e, [&](const E& x) { if (x->k == Expr::Var && assigned.count(x->name) && !(self && x->name == *self)) independent = false; });
          };
          for (auto& kv : thn) reads_assigned(kv.second, &kv.first->name);
          for (auto& kv : els) reads_assigned(kv.second, &kv.first->name);
          reads_assigned(r->expr, nullptr);
          if (independent && assigned.size() <= 4) {
            E test = r->expr;
            if (!cheap(test)) {   // reads memory: evaluated once, under a name (a cheap test is repeated, which lets a chain of elifs collapse)
              Name c = gen.fresh("pick");
              out.push_back(mk_def(c, Type::scalar(ElemSize::Bool), test, r->i));
              test = mk_var(c, Type::scalar(ElemSize::Bool), r->i);
            }
            for (auto& name : assigned) {
              E var, a, b;
              for (auto& kv : thn) if (kv.first->name == name) { var = kv.first; a = kv.second; }
              for (auto& kv : els) if (kv.first->name == name) { var = kv.first; b = kv.second; }
              if (!a) a = var;
              if (!b) b = var;
              if (a->ty.sz != var->ty.sz) a = fold_expr(mk_convert(a, var->ty.sz));
              if (b->ty.sz != var->ty.sz) b = fold_expr(mk_convert(b, var->ty.sz));
              E picked = mk_ifexpr(test, a, b, var->ty, r->i);
              // `x = init` a few statements up, nothing in between reading x or defining what the select reads:
              // the select takes init's place there (`w = 0.5; if c: w = 2` -> `w = c ? 2 : 0.5`), which leaves a
              // value that no longer depends on the variable's history
              bool merged = false;
              if (mentions(picked, name)) {
                std::set<Name> between;
                for (size_t back = out.size(); back-- > 0;) {
                  const S& prev = out[back];
                  bool def_like = (prev->k == Stmt::Def && prev->ty.is_scalar()) ||
                                  (prev->k == Stmt::Assign && prev->dst->k == Expr::Var && prev->dst->ty.is_scalar());
                  if (!def_like || !prev->expr || !cheap(prev->expr)) break;
                  const Name& pn = prev->k == Stmt::Def ? prev->id : prev->dst->name;
                  if (pn == name) {
                    bool clash = false;
                    visit_exprs(picked, [&](const E& x) { if (x->k == Expr::Var && between.count(x->name)) clash = true; });
                    if (!clash && !mentions(prev->expr, name)) {
                      std::map<Name, E> sub{{name, prev->expr}};
                      auto np = clone(prev);
                      np->expr = fold_expr(subst_vars(picked, sub));
                      out[back] = np;
                      merged = true;
                    }
                    break;
                  }
                  if (mentions(prev->expr, name)) break;
                  between.insert(pn);
                }
              }
              if (!merged) out.push_back(mk_assign(var, picked, r->i));
            }
            done = true;
          }
        }
      }
      if (!done) out.push_back(r);
    }
    return out;
  }

  void unswitch_aliases() {
    bool any = false;
    visit_stmts(k.body, [&](const S& s) { if (s->k == Stmt::Def && Unswitch::is_alias_type(s->ty)) any = true; });
    if (!any) return;
    Unswitch u;
    Stmts nb = u.run(k.body, 0, {});
    if (!u.failed) k.body = nb;
  }

  // ================================================================ LDS rows
  struct ArrayInfo {
    bool ok = true;
    int64_t rowlen = 0;
    ElemSize sz = ElemSize::F32;
    bool in_seq_loop = false;
    bool written = false;
    bool accessed = false;
  };

  void lds_rows() {
    if (k.body.size() != 1 || k.body[0]->k != Stmt::For || k.body[0]->map.k != GpuMap::Block) return;
    const S root = k.body[0];
    int64_t ext = const_extent(root);
    if (ext <= 0 || ext > root->map.n) return;  // a block must own exactly one value of the root variable
    if (k.block.y != 1 || k.block.z != 1) return;
    const Name r = root->id;

    std::map<Name, ArrayInfo> info;
    for (auto& p : k.params)
      if (p.ty.is_pointer()) info[p.id] = ArrayInfo();
    std::map<Name, std::set<Name>> alias;  // local -> parameters it may point to

    std::function<bool(const E&, std::set<Name>&)> sources = [&](const E& e, std::set<Name>& out) -> bool {
      if (e->k == Expr::Var) {
        if (info.count(e->name)) { out.insert(e->name); return true; }
        auto it = alias.find(e->name);
        if (it != alias.end()) { out.insert(it->second.begin(), it->second.end()); return true; }
        return false;
      }
      if (e->k == Expr::IfExpr) return sources(e->args[1], out) && sources(e->args[2], out);
      return false;
    };
    // aliases first (two sweeps reach a fixed point for loop-carried selects)
    for (int sweep = 0; sweep < 2; ++sweep)
      visit_stmts(k.body, [&](const S& s) {
        if (s->k == Stmt::Def && !s->ty.is_scalar()) { std::set<Name> src; if (sources(s->expr, src)) alias[s->id].insert(src.begin(), src.end()); }
        if (s->k == Stmt::Assign && s->dst->k == Expr::Var && !s->dst->ty.is_scalar()) {
          std::set<Name> src;
          if (sources(s->expr, src)) alias[s->dst->name].insert(src.begin(), src.end());
        }
      });

    // every use of an array (or alias) must be a two-dimensional access a[r, e]
    std::function<void(const E&, bool, bool)> scan = [&](const E& e, bool in_seq, bool is_store_dst) {
      if (!e) return;
      if (e->k == Expr::Index || e->k == Expr::AddrOf) {
        std::set<Name> src;
        if (sources(e->args[0], src)) {
          bool row = e->k == Expr::Index && e->dim_idx.size() == 2 && e->dim_idx[0]->k == Expr::Var && e->dim_idx[0]->name == r;
          for (auto& a : src) {
            ArrayInfo& ai = info[a];
            if (!row) { ai.ok = false; continue; }
            int64_t len = e->dim_shape[1];
            if (ai.accessed && (ai.rowlen != len || ai.sz != e->ty.sz)) ai.ok = false;
            ai.accessed = true;
            ai.rowlen = len;
            ai.sz = e->ty.sz;
            ai.in_seq_loop = ai.in_seq_loop || in_seq;
            ai.written = ai.written || is_store_dst;
          }
          scan(e->args[1], in_seq, false);
          for (auto& d : e->dim_idx) scan(d, in_seq, false);
          return;
        }
      }
      if (e->k == Expr::Var) {
        // a bare use of an array value that is not an alias definition (handled by the caller)
        std::set<Name> src;
        if (!e->ty.is_scalar() && sources(e, src))
          for (auto& a : src) info[a].ok = false;
        return;
      }
      for (auto& a : e->args) scan(a, in_seq, false);
    };
    std::function<void(const Stmts&, bool)> scan_stmts = [&](const Stmts& ss, bool in_seq) {
      for (auto& s : ss) {
        bool alias_def = (s->k == Stmt::Def && !s->ty.is_scalar()) ||
                         (s->k == Stmt::Assign && s->dst->k == Expr::Var && !s->dst->ty.is_scalar());
        if (alias_def) {
          std::set<Name> src;
          if (!sources(s->expr, src)) scan(s->expr, in_seq, false);
        } else {
          if (s->dst) scan(s->dst, in_seq, s->k == Stmt::Assign);
          if (s->expr) scan(s->expr, in_seq, false);
        }
        if (s->lo) scan(s->lo, in_seq, false);
        if (s->hi) scan(s->hi, in_seq, false);
        for (auto& a : s->args) scan(a, in_seq, false);
        bool seq = in_seq || (s->k == Stmt::For && s->map.k == GpuMap::None) || s->k == Stmt::While;
        scan_stmts(s->body, seq);
        scan_stmts(s->els, seq);
      }
    };
    scan_stmts(root->body, false);

    // arrays reachable through a common alias are promoted together or not at all
    bool changed = true;
    while (changed) {
      changed = false;
      for (auto& kv : alias) {
        bool all_ok = true, any_seq = false, any_written = false;
        int64_t len = -1;
        ElemSize sz = ElemSize::F32;
        for (auto& a : kv.second) {
          const ArrayInfo& ai = info[a];
          if (!ai.ok || !ai.accessed) { if (!ai.ok) all_ok = false; continue; }
          if (len >= 0 && (len != ai.rowlen || sz != ai.sz)) all_ok = false;
          len = ai.rowlen;
          sz = ai.sz;
          any_seq = any_seq || ai.in_seq_loop;
          any_written = any_written || ai.written;
        }
        for (auto& a : kv.second) {
          ArrayInfo& ai = info[a];
          if (!all_ok && ai.ok) { ai.ok = false; changed = true; }
          if (all_ok && len >= 0) {
            if (!ai.accessed) { ai.accessed = true; ai.rowlen = len; ai.sz = sz; changed = true; }
            if (any_seq && !ai.in_seq_loop) { ai.in_seq_loop = true; changed = true; }
            if (any_written && !ai.written) { ai.written = true; changed = true; }
          }
        }
      }
    }

    // choose what fits
    std::map<Name, Name> lds_name;
    int64_t used = 0;
    for (auto& p : k.params) {
      auto it = info.find(p.id);
      if (it == info.end()) continue;
      const ArrayInfo& ai = it->second;
      if (!ai.ok || !ai.accessed || !ai.in_seq_loop || !ai.written) continue;  // read-only tables stream better from L2
      int64_t bytes = ai.rowlen * elem_bytes(ai.sz);
      if (used + bytes > LDS_BUDGET_BYTES) { used = LDS_BUDGET_BYTES + 1; break; }
      used += bytes;
      lds_name[p.id] = gen.fresh("lds_" + p.id.s);
    }
    if (used > LDS_BUDGET_BYTES || lds_name.empty()) return;
    // an alias must not mix promoted and non-promoted arrays
    for (auto& kv : alias) {
      size_t n = 0;
      for (auto& a : kv.second) n += lds_name.count(a);
      if (n != 0 && n != kv.second.size()) return;
    }
    std::set<Name> lds_alias;
    for (auto& kv : alias)
      if (!kv.second.empty() && lds_name.count(*kv.second.begin())) lds_alias.insert(kv.first);

    auto lds_var = [&](const Name& a, const Info& i) { return mk_var(lds_name.at(a), Type::pointer(info[a].sz, Mem::LDS), i); };
    auto rw = [&](const E& e) -> E {
      if (e->k == Expr::Index && e->args[0]->k == Expr::Var) {
        const Name& b = e->args[0]->name;
        if (lds_name.count(b)) {
          auto n = std::make_shared<Expr>(*e);
          n->args = {lds_var(b, e->i), e->dim_idx[1]};
          n->dim_idx.clear();
          n->dim_shape.clear();
          return n;
        }
        if (lds_alias.count(b)) {
          auto n = std::make_shared<Expr>(*e);
          n->args = {mk_var(b, Type::pointer(e->ty.sz, Mem::LDS), e->i), e->dim_idx[1]};
          n->dim_idx.clear();
          n->dim_shape.clear();
          return n;
        }
      }
      return e;
    };
    Stmts body = rewrite_stmts(root->body, rw);
    // alias definitions now select between LDS arrays
    std::function<E(const E&)> to_lds = [&](const E& e) -> E {
      if (e->k == Expr::Var && lds_name.count(e->name)) return lds_var(e->name, e->i);
      if (e->k == Expr::Var && lds_alias.count(e->name)) return mk_var(e->name, Type::pointer(e->ty.sz, Mem::LDS), e->i);
      if (e->k == Expr::IfExpr) {
        E a = to_lds(e->args[1]), b = to_lds(e->args[2]);
        return mk_ifexpr(e->args[0], a, b, a->ty, e->i);
      }
      return e;
    };
    std::function<Stmts(const Stmts&)> fix_alias = [&](const Stmts& ss) {
      Stmts out;
      for (auto& s : ss) {
        auto n = clone(s);
        if (s->k == Stmt::Def && lds_alias.count(s->id)) {
          n->expr = to_lds(s->expr);
          n->ty = n->expr->ty;
        } else if (s->k == Stmt::Assign && s->dst->k == Expr::Var && lds_alias.count(s->dst->name)) {
          n->expr = to_lds(s->expr);
          n->dst = mk_var(s->dst->name, n->expr->ty, s->dst->i);
        }
        n->body = fix_alias(s->body);
        n->els = fix_alias(s->els);
        out.push_back(n);
      }
      return out;
    };
    body = fix_alias(body);

    // prologue: bring the rows in; epilogue: write them back
    Type ity = Type::scalar(isz);
    auto copy_loop = [&](const Name& a, bool to_lds_dir) {
      const ArrayInfo& ai = info[a];
      Name e = gen.fresh("e");
      E ev = mk_var(e, ity);
      E rv = mk_var(r, ity);
      E flat = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, rv, mk_int(ai.rowlen, isz), ity), ev, ity));
      Type elem = Type::scalar(ai.sz);
      E g = mk_index(mk_var(a, Type::pointer(ai.sz)), flat, elem);
      E l = mk_index(lds_var(a, Info()), ev, elem);
      LoopPar par;
      par.nthreads = k.block.x;
      auto loop = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(
          mk_for(e, mk_int(0, isz), mk_int(ai.rowlen, isz), 1, {to_lds_dir ? mk_assign(l, g) : mk_assign(g, l)}, par)));
      loop->map.k = GpuMap::Thread;
      loop->map.dim = 0;
      loop->map.n = k.block.x;
      return S(loop);
    };
    Stmts nb;
    for (auto& kv : lds_name) {
      auto d = std::make_shared<Stmt>();
      d->k = Stmt::LdsDecl;
      d->id = kv.second;
      d->ty = Type::scalar(info[kv.first].sz);
      d->iv = info[kv.first].rowlen;
      nb.push_back(d);
    }
    for (auto& kv : lds_name) nb.push_back(copy_loop(kv.first, true));
    nb.push_back(mk_sync());
    for (auto& s : body) nb.push_back(s);
    nb.push_back(mk_sync());
    for (auto& kv : lds_name)
      if (info[kv.first].written) nb.push_back(copy_loop(kv.first, false));
    auto nr = clone(root);
    nr->body = nb;
    k.body = {nr};
    int64_t total = 0;
    for (auto& kv : lds_name) total += info[kv.first].rowlen * elem_bytes(info[kv.first].sz);
    k.lds_bytes += total;
  }

  // ================================================================ vectorised iteration remap
  // Elements per thread that turn the unit-stride accesses of `loop` into 16-byte accesses, 0 when the
  // rewrite does not pay.  It does not pay when such an access goes through a local pointer into global
  // memory (`src = a if t & 1 else b`): loads and stores through pointers that may coincide cannot be
  // merged, so every lane would issue four 4-byte accesses 16 bytes apart from its neighbour's -- a
  // quarter of each cache line per request -- where the plain loop has neighbouring lanes on
  // neighbouring words.  (Measured on a 262144-state HMM step kept in global memory: 158 us per step
  // with the rewrite, 60 us without.)  Pointers into LDS have no such cost.
  int vector_width(const S& loop) {
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
  static int64_t strided_run(const E& idx, const Name& d) {
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

  Stmts vectorize(const Stmts& ss) {
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

  // ================================================================ hoisting of thread-private invariant loads
  // The iteration structure of a thread-mapped loop: the mapped loop itself and,
  // after vectorisation, the unrolled inner loop over the V consecutive elements.
  struct IterSpace {
    S outer;                 // thread-mapped loop
    S inner;                 // unrolled element loop, or null
    E slot;                  // per-thread iteration number (register array index)
    int64_t slots = 0;
    const Stmts* body = nullptr;  // innermost body
  };

  bool iter_space(const S& loop, IterSpace* is) {
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

  std::set<Name> written_arrays() {
    std::set<Name> w;
    visit_stmts(k.body, [&](const S& s) {
      if (s->k == Stmt::Assign && s->dst->k == Expr::Index) {
        visit_exprs(s->dst->args[0], [&](const E& x) { if (x->k == Expr::Var) w.insert(x->name); });
      }
    });
    return w;
  }

  struct Hoisted { E load; Name reg; ElemSize sz; };

  int64_t reg_budget() const {
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
  bool step_has_transcendentals() const {
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
  Stmts hoist_from_seq_loop(const S& seq, int64_t* budget) {
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

  Stmts hoist_invariant(const Stmts& ss, int64_t* budget, bool in_seq) {
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
  struct OwnIterations {
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

  bool distinct_names(const Name& a, const Name& b) const {
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

  Stmts share_own_iterations(const Stmts& ss) {
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
  void reg_cache(int64_t* budget) {
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

  // ================================================================ values a thread has just stored, read again by itself
  // Inside one iteration of a sequential loop a thread-mapped loop stores a row through a pointer (`dst[V q + c] = e`
  // for c = 0 .. V-1, a thread owning the same q in every such loop), and later in the same iteration -- possibly
  // under a test of the step counter -- a thread-mapped loop of the same shape reads exactly those elements back
  // through a pointer that selects the same array under the same condition (`x = a; if (t & 1) x = b` written twice:
  // the row maximum every eighth step of the rescaled HMM forward pass).  The values travel in a register array
  // from the storing loop to the reading one; the stores stay (other threads read the row in the next iteration),
  // the loads from LDS and their wait go.  7-mer batch 16.9 -> 15.5 ms.
  struct AliasDef { Name a, b; E cond; bool ok = false; };

  // `name = a; if (cond) { ...; name = b; ... }` among the statements of `ss` before position `upto`, no other assignment
  static AliasDef alias_definition(const Stmts& ss, size_t upto, const Name& name) {
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
  static bool scaled_index(const E& idx, const Name& var, int64_t* V, int64_t* c) {
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

  Stmts keep_stored_rows(const Stmts& ss, int64_t* budget) {
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
  static bool alternates(const E& cond, const S& loop) {
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
  Stmts carry_across_iterations(const Stmts& B, size_t p1, const S& L1, const IterSpace& is1, const S& seq_loop, const AliasDef& dx,
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

  std::set<Name> lds_array_names() const {
    std::set<Name> r;
    visit_stmts(k.body, [&](const S& c) { if (c->k == Stmt::LdsDecl) r.insert(c->id); });
    return r;
  }

  Stmts keep_in_iteration(const Stmts& B, int64_t* budget, const S& seq_loop, Stmts* pre) {
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

  // ================================================================ barriers that order nothing
  // The generic pipeline puts a barrier after every parallel loop.  Once rows live in registers, a
  // loop may touch no memory at all (softmax's `exp` and scaling steps), and the barrier after it --
  // or the one before the next memory access -- orders nothing.  A barrier between two straight-line
  // regions of the workgroup's top-level statement list is kept only if an array written on one
  // side is accessed on the other; accesses through pointer variables, helper calls and raw
  // statements count as touching everything.  Barriers inside sequential loops are left alone (the
  // region after them wraps round to the loop head).  Reduction sites own their LDS slots and
  // synchronise internally.
  struct Touched {
    std::set<Name> r, w;
    bool any = false;
  };

  void touched(const Stmts& ss, const std::set<Name>& arrays, Touched& t) {
    std::function<void(const E&, bool)> scan = [&](const E& e, bool store) {
      if (!e) return;
      if (e->k == Expr::Index || e->k == Expr::AddrOf) {
        const E& b = e->args[0];
        if (b->k == Expr::Var && arrays.count(b->name)) (store && e->k == Expr::Index ? t.w : t.r).insert(b->name);
        else t.any = true;
        if (e->k == Expr::AddrOf) t.any = true;   // the address escapes (an external may write through it)
        scan(e->args[1], false);
        return;
      }
      if (e->k == Expr::Call) t.any = true;
      for (auto& a : e->args) scan(a, false);
    };
    for (auto& st : ss) {
      if (st->k == Stmt::RawStmt || st->k == Stmt::CallStmt) t.any = true;
      scan(st->dst, st->k == Stmt::Assign);
      scan(st->expr, false);
      scan(st->lo, false);
      scan(st->hi, false);
      for (auto& a : st->args) scan(a, false);
      touched(st->body, arrays, t);
      touched(st->els, arrays, t);
    }
  }

  Stmts drop_barriers_in(const Stmts& ss, const std::set<Name>& arrays) {
    // split into regions at the barriers of this level
    std::vector<Stmts> regions(1);
    for (auto& st : ss) {
      if (st->k == Stmt::Sync) regions.emplace_back();
      else regions.back().push_back(st);
    }
    if (regions.size() == 1) {
      Stmts out;
      for (auto& st : ss) {
        if (st->k == Stmt::For && st->map.k == GpuMap::Block) {  // the workgroup's statement list is further in
          auto r = clone(st);
          r->body = drop_barriers_in(st->body, arrays);
          out.push_back(r);
        } else out.push_back(st);
      }
      return out;
    }
    Stmts out = regions[0];
    Touched before;
    touched(regions[0], arrays, before);
    for (size_t q = 1; q < regions.size(); ++q) {
      Touched after;
      touched(regions[q], arrays, after);
      bool conflict = before.any || after.any;
      for (auto& n : before.w) if (after.r.count(n) || after.w.count(n)) conflict = true;
      for (auto& n : before.r) if (after.w.count(n)) conflict = true;
      if (conflict) {
        out.push_back(mk_sync());
        before = after;
      } else {   // merged into one region
        before.r.insert(after.r.begin(), after.r.end());
        before.w.insert(after.w.begin(), after.w.end());
      }
      for (auto& st : regions[q]) out.push_back(st);
    }
    return out;
  }

  void drop_barriers() {
    std::set<Name> arrays;
    for (auto& p : k.params) if (p.ty.is_pointer()) arrays.insert(p.id);
    visit_stmts(k.body, [&](const S& st) { if (st->k == Stmt::LdsDecl) arrays.insert(st->id); });
    k.body = drop_barriers_in(k.body, arrays);
  }

  // ================================================================ no-alias scopes for array aliases
  // `src = a; dst = b; if (c) { src = b; dst = a; } <rest>`: in <rest> the two aliases always name
  // different arrays, but the target compiler only sees two selected pointers that may be equal, so
  // it keeps every load from `src` behind the preceding store to `dst`.  When every combination of
  // the selections gives pairwise different arrays, and <rest> reaches those arrays through the
  // aliases only, <rest> is put into a scope whose parameters are the aliases, declared not to
  // alias each other.  Loads of the (independent) iterations that a thread runs of a parallel loop
  // can then be shared and merged: the four states of a thread that have the same predecessors load
  // them once, and own-state loads and stores become 128-bit LDS accesses.
  static bool is_alias_type(const Type& t) { return t.k == Type::Pointer || (t.k == Type::Tensor && !t.shape.empty()); }

  using AliasCfg = std::map<Name, Name>;

  static bool alias_target(const E& e, const AliasCfg& cfg, Name* out) {
    if (!e || e->k != Expr::Var) return false;
    auto it = cfg.find(e->name);
    *out = it == cfg.end() ? e->name : it->second;
    return true;
  }

  // statements that only (re)point aliases: applies them to every configuration, false if anything else is found
  static bool apply_alias_stmt(const S& st, std::vector<AliasCfg>& cfgs, std::vector<Name>& order) {
    if ((st->k == Stmt::Def && is_alias_type(st->ty)) ||
        (st->k == Stmt::Assign && st->dst->k == Expr::Var && is_alias_type(st->dst->ty))) {
      Name a = st->k == Stmt::Def ? st->id : st->dst->name;
      for (auto& c : cfgs) {
        Name t;
        if (!alias_target(st->expr, c, &t)) return false;
        c[a] = t;
      }
      if (std::find(order.begin(), order.end(), a) == order.end()) order.push_back(a);
      return true;
    }
    if (st->k == Stmt::If && !(st->body.empty() && st->els.empty())) {
      std::vector<AliasCfg> then_c = cfgs, else_c = cfgs;
      for (auto& c : st->body) if (!apply_alias_stmt(c, then_c, order)) return false;
      for (auto& c : st->els) if (!apply_alias_stmt(c, else_c, order)) return false;
      cfgs = then_c;
      cfgs.insert(cfgs.end(), else_c.begin(), else_c.end());
      return cfgs.size() <= 16;
    }
    return false;
  }

  // With `wrap` the rest of the block goes into a scope whose pointer parameters carry the promise; without it the
  // kernel only records which local pointers never coincide (the printer's access packing asks).
  Stmts noalias_scopes(const Stmts& ss, bool wrap) {
    Stmts cur;
    for (auto& s : ss) {
      auto r = clone(s);
      r->body = noalias_scopes(s->body, wrap);
      r->els = noalias_scopes(s->els, wrap);
      cur.push_back(r);
    }
    // the first run of alias-only statements of this block
    size_t a = 0;
    while (a < cur.size() && !(cur[a]->k == Stmt::Def && is_alias_type(cur[a]->ty))) ++a;
    if (a == cur.size()) return cur;
    std::vector<AliasCfg> cfgs(1);
    std::vector<Name> order;
    size_t b = a;
    while (b < cur.size()) {
      std::vector<AliasCfg> trial = cfgs;
      std::vector<Name> otrial = order;
      if (!apply_alias_stmt(cur[b], trial, otrial)) break;
      cfgs = trial;
      order = otrial;
      ++b;
    }
    if (order.size() < 2 || b == cur.size()) return cur;
    std::set<Name> targets;
    for (auto& c : cfgs) {
      std::set<Name> seen;
      for (auto& n : order) {
        auto it = c.find(n);
        if (it == c.end() || !seen.insert(it->second).second) return cur;  // two aliases may name one array
        targets.insert(it->second);
      }
    }
    // the rest of the block must reach the arrays through the aliases only and leave the aliases alone
    bool clean = true;
    std::map<Name, Type> types;
    Stmts rest(cur.begin() + b, cur.end());
    visit_stmts(rest, [&](const S& st) {
      if (st->k == Stmt::Def && (targets.count(st->id) || std::count(order.begin(), order.end(), st->id))) clean = false;
      if (st->k == Stmt::Assign && st->dst->k == Expr::Var && std::count(order.begin(), order.end(), st->dst->name)) clean = false;
      if (wrap && (st->k == Stmt::Def || (st->k == Stmt::Assign && st->dst->k == Expr::Var)) && is_alias_type(st->k == Stmt::Def ? st->ty : st->dst->ty))
        clean = false;  // a further alias inside the scope could name the same arrays
      auto scan = [&](const E& e) {
        visit_exprs(e, [&](const E& x) {
          if (x->k != Expr::Var) return;
          if (wrap && targets.count(x->name)) clean = false;
          if (std::count(order.begin(), order.end(), x->name)) types[x->name] = x->ty;
        });
      };
      scan(st->dst); scan(st->expr); scan(st->lo); scan(st->hi);
      for (auto& e : st->args) scan(e);
    });
    if (!clean) return cur;
    std::vector<E> params;
    for (auto& n : order)
      if (types.count(n) && types[n].k == Type::Pointer) params.push_back(mk_var(n, types[n]));
    if (!wrap) {
      std::vector<Name> group;
      for (auto& n : order)
        if (types.count(n)) group.push_back(n);
      if (group.size() >= 2) k.distinct_pointers.push_back(group);
      return cur;
    }
    if (params.size() < 2) return cur;
    auto scope = std::make_shared<Stmt>();
    scope->k = Stmt::Scope;
    scope->args = params;
    scope->body = rest;
    Stmts out(cur.begin(), cur.begin() + b);
    out.push_back(scope);
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
  Stmts mfma_dot(const Stmts& ss) {
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

  // ================================================================ read-only parameters
  // A pointer parameter is read-only when nothing in the kernel stores through
  // it, directly or through a local alias initialised from it.
  void mark_read_only() {
    std::set<Name> written;
    std::map<Name, std::set<Name>> alias_of;
    std::function<void(const E&, std::set<Name>&)> bases = [&](const E& e, std::set<Name>& out) {
      if (!e) return;
      if (e->k == Expr::Var) {
        auto it = alias_of.find(e->name);
        if (it != alias_of.end()) out.insert(it->second.begin(), it->second.end());
        else out.insert(e->name);
        return;
      }
      if (e->k == Expr::AddrOf || e->k == Expr::Index) { bases(e->args[0], out); return; }
      if (e->k == Expr::IfExpr) { bases(e->args[1], out); bases(e->args[2], out); }
    };
    for (int sweep = 0; sweep < 2; ++sweep) {
      visit_stmts(k.body, [&](const S& s) {
        if (s->k == Stmt::Def && (s->ty.is_array() || s->ty.is_pointer())) bases(s->expr, alias_of[s->id]);
        if (s->k == Stmt::Assign && s->dst->k == Expr::Var && (s->dst->ty.is_array() || s->dst->ty.is_pointer()))
          bases(s->expr, alias_of[s->dst->name]);
        if (s->k == Stmt::Assign && s->dst->k == Expr::Index) bases(s->dst->args[0], written);
        // an array handed to an external device function may be written by it
        auto calls = [&](const E& root) {
          visit_exprs(root, [&](const E& x) {
            if (x->k != Expr::Call || !x->ext) return;
            for (auto& a : x->args)
              if (a->k == Expr::AddrOf || (a->k == Expr::Var && !a->ty.is_scalar())) bases(a, written);
          });
        };
        calls(s->expr); calls(s->dst); calls(s->lo); calls(s->hi);
      });
    }
    for (auto& p : k.params) p.read_only = p.ty.is_pointer() && !written.count(p.id);
  }
};

// ================================================================ transposed staging of column gathers
// A read-only matrix X[K, N] that a kernel only reads as X[d, c] with d the
// variable of an innermost sequential loop over all K rows and c fixed per
// thread is a column gather: every step of the loop touches one 4-byte word
// in each of up to 64 different cache lines per wavefront.  Staging X^T once
// in a device temporary turns each thread's column into K contiguous words
// (dwordx4 loads, whole cache lines used).  The transposition costs two
// passes over X; it is applied to kernels launched once per call.
struct GatherTranspose {
  Program& p;
  const Options& opts;
  NameGen& gen;
  ElemSize isz;

  GatherTranspose(Program& prog, const Options& o, NameGen& g) : p(prog), opts(o), gen(g), isz(o.int_size()) {}

  struct Cand { Name arr; int64_t K = 0, N = 0; ElemSize sz = ElemSize::F32; bool ok = true; bool seen = false; };

  void scan_expr(const E& e, const std::vector<std::pair<Name, int64_t>>& seq_loops, std::map<Name, Cand>& cands) {
    if (!e) return;
    if ((e->k == Expr::Index || e->k == Expr::AddrOf) && e->args[0]->k == Expr::Var && cands.count(e->args[0]->name)) {
      Cand& c = cands[e->args[0]->name];
      bool good = e->k == Expr::Index && e->dim_idx.size() == 2 && e->dim_idx[0]->k == Expr::Var && !seq_loops.empty() &&
                  e->dim_idx[0]->name == seq_loops.back().first && e->dim_shape[0] == seq_loops.back().second &&
                  !mentions(e->dim_idx[1], seq_loops.back().first) && !has_load(e->dim_idx[1]);
      if (good && c.seen && (c.K != e->dim_shape[0] || c.N != e->dim_shape[1])) good = false;
      if (!good) c.ok = false;
      else { c.seen = true; c.K = e->dim_shape[0]; c.N = e->dim_shape[1]; c.sz = e->ty.sz; }
      scan_expr(e->args[1], seq_loops, cands);
      return;
    }
    if (e->k == Expr::Var && cands.count(e->name)) { cands[e->name].ok = false; return; }
    for (auto& a : e->args) scan_expr(a, seq_loops, cands);
  }

  void scan(const Stmts& ss, std::vector<std::pair<Name, int64_t>>& seq_loops, std::map<Name, Cand>& cands) {
    for (auto& s : ss) {
      scan_expr(s->dst, seq_loops, cands);
      scan_expr(s->expr, seq_loops, cands);
      scan_expr(s->lo, seq_loops, cands);
      scan_expr(s->hi, seq_loops, cands);
      for (auto& a : s->args) scan_expr(a, seq_loops, cands);
      bool seq = s->k == Stmt::For && s->map.k == GpuMap::None && s->step == 1 && s->lo->k == Expr::Int && s->lo->iv == 0 &&
                 s->hi->k == Expr::Int;
      // only innermost loops qualify: a nested loop hides the enclosing one
      if (seq) seq_loops.emplace_back(s->id, s->hi->iv);
      else if (s->k == Stmt::For || s->k == Stmt::While) seq_loops.emplace_back(Name{"", -1}, -1);
      scan(s->body, seq_loops, cands);
      if (s->k == Stmt::For || s->k == Stmt::While) seq_loops.pop_back();
      scan(s->els, seq_loops, cands);
    }
  }

  Kernel make_transpose(const Name& x, const Name& xt, const Cand& c) {
    KernelParam px, pxt;
    px.id = x;
    px.ty = Type::pointer(c.sz);
    px.read_only = true;
    pxt.id = xt;
    pxt.ty = Type::pointer(c.sz);
    if (c.K >= 16 && c.N >= 64 && elem_bytes(c.sz) >= 4) {
      // 64 x 64 tiles turned round in LDS by a device helper, whole lines on both sides (edge tiles are guarded)
      Kernel k;
      k.name = p.name + "_transpose_" + x.s + "_" + std::to_string(gen.next++);
      k.grid.x = (c.N + 63) / 64;
      k.grid.y = (c.K + 63) / 64;
      k.block.x = 256;
      k.lds_bytes = 64 * 65 * elem_bytes(c.sz);
      k.cached_stores = true;
      k.opaque_body = true;
      k.body = {mk_rawstmt("parpy_transpose_tile<" + std::string(elem_ctype(c.sz)) + ", " + std::to_string(c.K) + ", " +
                           std::to_string(c.N) + ">(" + x.str() + ", " + xt.str() + ");")};
      k.params = {px, pxt};
      return k;
    }
    // one thread per column c; reads are coalesced across the wavefront, each thread writes its own row of X^T
    Type ity = Type::scalar(isz);
    Type elem = Type::scalar(c.sz);
    Name cv = gen.fresh("c"), dv = gen.fresh("d");
    E ce = mk_var(cv, ity), de = mk_var(dv, ity);
    E src = mk_index(mk_var(x, Type::pointer(c.sz)), fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, de, mk_int(c.N, isz), ity), ce, ity)), elem);
    E dst = mk_index(mk_var(xt, Type::pointer(c.sz)), fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, ce, mk_int(c.K, isz), ity), de, ity)), elem);
    S inner = mk_for(dv, mk_int(0, isz), mk_int(c.K, isz), 1, {mk_assign(dst, src)}, LoopPar());
    LoopPar par;
    par.nthreads = c.N;
    par.tpb = 256;
    auto outer = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(mk_for(cv, mk_int(0, isz), mk_int(c.N, isz), 1, {inner}, par)));
    int64_t n = (c.N + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
    Kernel k;
    k.name = p.name + "_transpose_" + x.s + "_" + std::to_string(gen.next++);
    if (n > 256) {
      outer->map.k = GpuMap::ThreadBlock;
      outer->map.n = n;
      outer->map.tpb = 256;
      k.grid.x = (n + 255) / 256;
      k.block.x = 256;
    } else {
      outer->map.k = GpuMap::Thread;
      outer->map.n = n;
      k.block.x = n;
    }
    outer->map.dim = 0;
    k.body = {S(outer)};
    k.cached_stores = true;
    k.params = {px, pxt};
    return k;
  }

  void run() {
    Stmts host;
    std::vector<Kernel> extra;
    for (auto& s : p.host) {
      if (s->k != Stmt::Launch) { host.push_back(s); continue; }
      Kernel* k = nullptr;
      for (auto& kk : p.kernels)
        if (kk.name == s->fname) k = &kk;
      if (!k) { host.push_back(s); continue; }
      std::map<Name, Cand> cands;
      std::set<Name> written;
      visit_stmts(k->body, [&](const S& st) {
        if (st->k == Stmt::Assign && st->dst->k == Expr::Index)
          visit_exprs(st->dst->args[0], [&](const E& x) { if (x->k == Expr::Var) written.insert(x->name); });
        if ((st->k == Stmt::Def && !st->ty.is_scalar()) || (st->k == Stmt::Assign && st->dst->k == Expr::Var && !st->dst->ty.is_scalar()))
          visit_exprs(st->expr, [&](const E& x) { if (x->k == Expr::Var) written.insert(x->name); });  // aliased: leave alone
      });
      for (auto& q : k->params)
        if (q.ty.is_pointer() && !written.count(q.id)) { Cand c; c.arr = q.id; cands[q.id] = c; }
      std::vector<std::pair<Name, int64_t>> seq_loops;
      scan(k->body, seq_loops, cands);
      std::map<Name, Name> staged;
      Stmts pre, post;
      for (auto& kv : cands) {
        const Cand& c = kv.second;
        // worth it when the stride is at least a cache line and the matrix is re-read many times
        if (!c.ok || !c.seen || c.N < 32 || c.K < 8 || c.K * c.N * elem_bytes(c.sz) > (int64_t(1) << 30)) continue;
        Name xt = gen.fresh(c.arr.s + "_T");
        staged[c.arr] = xt;
        auto a = std::make_shared<Stmt>();
        a->k = Stmt::Alloc;
        a->id = xt;
        a->ty = Type::scalar(c.sz);
        a->iv = c.K * c.N;
        pre.push_back(a);
        Kernel tk = make_transpose(c.arr, xt, c);
        auto l = std::make_shared<Stmt>();
        l->k = Stmt::Launch;
        l->fname = tk.name;
        l->grid = tk.grid;
        l->block = tk.block;
        // the launch argument is whatever the consumer was given for this parameter
        E src_arg;
        for (size_t i = 0; i < k->params.size(); ++i)
          if (k->params[i].id == c.arr) src_arg = s->args[i];
        l->args = {src_arg, mk_var(xt, Type::pointer(c.sz))};
        pre.push_back(l);
        extra.push_back(tk);
        auto f = std::make_shared<Stmt>();
        f->k = Stmt::Free;
        f->id = xt;
        post.push_back(f);
      }
      if (staged.empty()) { host.push_back(s); continue; }
      Type ity = Type::scalar(isz);
      k->body = rewrite_stmts(k->body, [&](const E& e) -> E {
        if (e->k == Expr::Index && e->args[0]->k == Expr::Var && staged.count(e->args[0]->name)) {
          const Cand& c = cands[e->args[0]->name];
          auto n = std::make_shared<Expr>(*e);
          E idx = fold_expr(mk_binop(BinOp::Add, mk_binop(BinOp::Mul, e->dim_idx[1], mk_int(c.K, isz), ity), e->dim_idx[0], ity));
          n->args = {mk_var(staged.at(e->args[0]->name), Type::tensor(c.sz, {c.N, c.K}), e->i), idx};
          n->dim_idx = {e->dim_idx[1], e->dim_idx[0]};
          n->dim_shape = {c.N, c.K};
          return n;
        }
        return e;
      });
      auto ns = std::make_shared<Stmt>(*s);
      for (size_t i = 0; i < k->params.size(); ++i)
        if (staged.count(k->params[i].id)) {
          Name xt = staged.at(k->params[i].id);
          ns->args[i] = mk_var(xt, Type::pointer(k->params[i].ty.sz));
          k->params[i].id = xt;
        }
      for (auto& q : pre) host.push_back(q);
      host.push_back(ns);
      for (auto& q : post) host.push_back(q);
    }
    for (auto& e : extra) p.kernels.push_back(e);
    p.host = host;
  }
};

// ================================================================ lane groups for per-thread dot products
// A grid-wide loop whose every iteration runs a long sequential sum over unit-stride rows
// (`t += X[a*K + d] * Y[b*K + d]`, d = 0..K) makes each lane walk its own rows: one wavefront load
// touches 64 different cache lines and uses 16 bytes of each, and the line is fetched again for
// each of the following iterations unless it survives in L1.  Here G = 8 adjacent lanes share one
// iteration instead: lane g takes the g-th 16-byte piece of every 128-byte line, so each line is
// requested once, and the eight partial sums are added with three DPP steps.  The launch grows by
// G; statements after the sum that store to memory are executed by lane 0 of each group.
struct LaneSplit {
  Program& p;
  const Options& opts;
  NameGen& gen;
  ElemSize isz;
  static constexpr int64_t G = 8;

  LaneSplit(Program& prog, const Options& o, NameGen& g) : p(prog), opts(o), gen(g), isz(o.int_size()) {}

  // the sum loop: a sequential loop over [0, K) whose body is `acc = acc + e`, where acc is a scalar
  // variable or an array element that does not depend on d, and all d-dependent accesses are unit-stride
  // (*vec = 0 stands for the second form: bounds that are data, as in a CSR row -- then lane g of a group takes
  // the elements lo+g, lo+g+8, ... one at a time, since nothing is known about where the row starts.)
  bool sum_loop(const S& s, int* vec, E* term_out) {
    if (!(s->k == Stmt::For && s->map.k == GpuMap::None && !s->unroll && s->step == 1 && s->body.size() == 1)) return false;
    const bool fixed = s->lo->k == Expr::Int && s->lo->iv == 0 && s->hi->k == Expr::Int;
    if (!fixed && s->lo->k == Expr::Int && s->hi->k == Expr::Int) return false;  // constant bounds that do not start at 0: not handled
    const S& a = s->body[0];
    if (a->k != Stmt::Assign) return false;
    const E& acc = a->dst;
    bool scalar_acc = acc->k == Expr::Var && acc->ty.is_scalar();
    bool elem_acc = acc->k == Expr::Index && acc->args[0]->k == Expr::Var && !mentions(acc->args[1], s->id) && !has_load(acc->args[1]);
    if (!(scalar_acc || elem_acc) || !is_float(acc->ty.sz)) return false;
    if (!(a->expr->k == Expr::BinOpE && a->expr->bop == BinOp::Add)) return false;
    const E &l = a->expr->args[0], &r = a->expr->args[1];
    E term;
    if (expr_eq(l, acc)) term = r;
    else if (expr_eq(r, acc)) term = l;
    if (!term) return false;
    const Name& acc_name = scalar_acc ? acc->name : acc->args[0]->name;
    if (mentions(term, acc_name) || mentions(s->lo, acc_name) || mentions(s->hi, acc_name)) return false;
    int v = 0, loads = 0;
    bool ok = true;
    visit_exprs(term, [&](const E& x) {
      if (x->k == Expr::Call || x->k == Expr::AddrOf) ok = false;
      if (x->k != Expr::Index) return;
      if (!mentions(x->args[1], s->id)) return;
      E rest;
      if (!affine_unit(x->args[1], s->id, &rest)) { if (fixed) ok = false; return; }  // (a gather `x[cols[d]]` is fine lane by lane)
      int w = elem_bytes(x->ty.sz) == 4 ? 4 : elem_bytes(x->ty.sz) == 8 ? 2 : 0;
      if (w == 0) { ok = false; return; }
      v = v == 0 ? w : std::min(v, w);
      ++loads;
    });
    if (!ok || loads < 1) return false;
    if (fixed && (s->hi->iv % v != 0 || s->hi->iv < 2 * v * G)) return false;  // whole vectors, and enough of them
    *vec = fixed ? v : 0;
    *term_out = term;
    return true;
  }

  bool apply(Kernel& k, const StmtP& launch) {
    if (k.body.size() != 1) return false;
    const S& root = k.body[0];
    // the iterations of the whole launch: spread over the grid, or over the threads of a single workgroup
    // (which then becomes a grid, since eight times as many threads may not fit one workgroup)
    bool one_group = root->k == Stmt::For && root->map.k == GpuMap::Thread && k.grid.x == 1;
    if (!(root->k == Stmt::For && (root->map.k == GpuMap::ThreadBlock || one_group) && root->map.dim == 0 && root->step == 1 &&
          root->lo->k == Expr::Int && root->lo->iv == 0 && root->hi->k == Expr::Int))
      return false;
    int64_t N = root->hi->iv;
    if (one_group && N > root->map.n) return false;  // a strided loop inside the workgroup: iterations are not one per thread
    if (N < 64 || k.grid.y != 1 || k.grid.z != 1 || k.block.y != 1 || k.block.z != 1) return false;  // (less than a wavefront of iterations: nothing to share)
    int pos = -1, vec = 0;
    E term;
    for (size_t q = 0; q < root->body.size(); ++q) {
      const S& st = root->body[q];
      int v = 0;
      E t;
      if (sum_loop(st, &v, &t)) {
        if (pos >= 0) return false;
        pos = (int)q;
        vec = v;
        term = t;
        continue;
      }
      bool simple = st->k == Stmt::Def || (st->k == Stmt::Assign && (st->dst->k == Expr::Index || st->dst->k == Expr::Var));
      if (!simple) return false;
    }
    if (pos < 0) return false;
    const S& loop = root->body[pos];
    const E& acc = loop->body[0]->dst;
    bool elem_acc = acc->k == Expr::Index;
    // an array element as accumulator: nothing else in the iteration may touch that array but plain
    // stores to the very element in front of the loop (its initialisation)
    if (elem_acc)
      for (size_t q = 0; q < root->body.size(); ++q) {
        if ((int)q == pos) continue;
        const S& st = root->body[q];
        bool init = (int)q < pos && st->k == Stmt::Assign && expr_eq(st->dst, acc) && !mentions(st->expr, acc->args[0]->name);
        if (init) continue;
        bool touches = false;
        auto scan = [&](const E& e) { if (e && mentions(e, acc->args[0]->name)) touches = true; };
        scan(st->dst); scan(st->expr);
        if (touches) return false;
      }
    for (int q = 0; q < pos; ++q)   // other stores in front of the sum would be repeated by every lane of a group: harmless, same value
      if (root->body[q]->k == Stmt::Assign && root->body[q]->dst->k == Expr::Index && !expr_eq(root->body[q]->dst, acc)) return false;
    Type ity = Type::scalar(isz);
    Name gi = gen.fresh(root->id.s + "_lane"), g = gen.fresh("g"), d0 = gen.fresh(loop->id.s + "_c"), u = gen.fresh(loop->id.s + "_u");
    E giv = mk_var(gi, ity), gv = mk_var(g, ity);
    E lane0 = mk_binop(BinOp::Eq, gv, mk_int(0, isz), Type::scalar(ElemSize::Bool));
    Stmts body;
    body.push_back(mk_def(root->id, ity, mk_binop(BinOp::FloorDiv, giv, mk_int(G, isz), ity), root->i));
    body.push_back(mk_def(g, ity, mk_binop(BinOp::Rem, giv, mk_int(G, isz), ity), root->i));
    for (int q = 0; q < pos; ++q) {
      const S& st = root->body[q];
      if (st->k == Stmt::Assign && st->dst->k == Expr::Index) body.push_back(mk_if(lane0, {st}, {}));
      else body.push_back(st);
    }
    E t = acc;
    if (elem_acc) {
      Name tn = gen.fresh("part");
      body.push_back(mk_def(tn, acc->ty, mk_float(0.0, acc->ty.sz), loop->i));
      t = mk_var(tn, acc->ty);
    }
    if (vec == 0) {
      // bounds that are data: for (d = lo + g; d < hi; d += G) t += term
      auto strided = clone(loop);
      strided->lo = mk_binop(BinOp::Add, loop->lo, gv, ity);
      strided->step = G;
      strided->body = {mk_assign(t, mk_binop(BinOp::Add, t, term, t->ty), loop->i)};
      body.push_back(strided);
    } else {
    // d = (d0 * G + g) * V + u
    E d = mk_binop(BinOp::Add,
                   mk_binop(BinOp::Mul, mk_binop(BinOp::Add, mk_binop(BinOp::Mul, mk_var(d0, ity), mk_int(G, isz), ity), gv, ity),
                            mk_int(vec, isz), ity),
                   mk_var(u, ity), ity);
    Stmts ib;
    ib.push_back(mk_def(loop->id, ity, d, loop->i));
    ib.push_back(mk_assign(t, mk_binop(BinOp::Add, t, term, t->ty), loop->i));
    auto inner = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(
        mk_for(u, mk_int(0, isz), mk_int(vec, isz), 1, ib, LoopPar(), loop->i)));
    inner->unroll = true;
    auto outer = clone(loop);
    outer->id = d0;
    const int64_t K = loop->hi->iv, chunk = vec * G;
    outer->hi = mk_int((K + chunk - 1) / chunk, isz);
    if (K % chunk == 0) {
      outer->body = {S(inner)};
    } else {
      // the last round covers only part of the group: lanes whose vector starts past the end sit it out
      E base = mk_binop(BinOp::Mul, mk_binop(BinOp::Add, mk_binop(BinOp::Mul, mk_var(d0, ity), mk_int(G, isz), ity), gv, ity),
                        mk_int(vec, isz), ity);
      outer->body = {mk_if(mk_binop(BinOp::Lt, base, mk_int(K, isz), Type::scalar(ElemSize::Bool)), {S(inner)}, {})};
    }
    body.push_back(outer);
    }
    body.push_back(mk_assign(t, mk_raw("parpy_sum8(" + t->name.str() + ")", t->ty)));
    Stmts stores;
    if (elem_acc) {
      // a group that lies wholly in one lane-0 store: the synchronisation between the initialising store
      // and this read-modify-write is program order of lane 0
      stores.push_back(mk_assign(acc, mk_binop(BinOp::Add, acc, t, acc->ty), loop->i));
    }
    for (size_t q = pos + 1; q < root->body.size(); ++q) {
      const S& st = root->body[q];
      if (st->k == Stmt::Assign && st->dst->k == Expr::Index) stores.push_back(st);
      else {
        if (!stores.empty()) return false;  // a definition after a store: not the shape this pass handles
        body.push_back(st);
      }
    }
    if (!stores.empty()) body.push_back(mk_if(lane0, stores, {}));
    auto nr = clone(root);
    nr->id = gi;
    nr->hi = mk_int(N * G, isz);
    nr->body = body;
    int64_t tpb = one_group ? 256 : root->map.tpb;
    nr->map.k = GpuMap::ThreadBlock;
    nr->map.tpb = tpb;
    nr->map.n = (N * G + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
    k.body = {S(nr)};
    k.block.x = tpb;
    k.grid.x = (nr->map.n + tpb - 1) / tpb;
    launch->grid = k.grid;
    launch->block = k.block;
    return true;
  }

  void run() {
    Stmts host;
    for (auto& s : p.host) {
      if (s->k != Stmt::Launch) { host.push_back(s); continue; }
      Kernel* k = nullptr;
      for (auto& kk : p.kernels)
        if (kk.name == s->fname) k = &kk;
      auto ns = std::make_shared<Stmt>(*s);
      if (k && !k->opaque_body) apply(*k, ns);
      host.push_back(ns);
    }
    p.host = host;
  }
};

// ================================================================ four elements per thread for element-wise launches
// `parpy.threads(n)` on a loop of n iterations gives every thread one element, and a thread cannot
// turn one 4-byte access into a 16-byte one.  When the iteration is nothing but straight-line
// element-wise work on unit-stride data, the launch is cut to n/4 threads; the vectorised remap then
// gives each of them four consecutive elements (y = a*x + y on 2^28 floats: 5.5 -> 5.9 TB/s).  Launches
// that would drop below 64 threads per CU keep their shape, as do iterations that contain loops (those
// want more threads, not fewer: see the lane groups below).
struct Coarsen {
  Program& p;
  const Options& opts;
  NameGen& gen;
  Coarsen(Program& prog, const Options& o, NameGen& g) : p(prog), opts(o), gen(g) {}

  bool apply(Kernel& k, const StmtP& launch) {
    if (k.body.size() != 1) return false;
    const S& root = k.body[0];
    if (!(root->k == Stmt::For && root->map.k == GpuMap::ThreadBlock && root->map.dim == 0 && root->step == 1 &&
          root->lo->k == Expr::Int && root->lo->iv == 0 && root->hi->k == Expr::Int))
      return false;
    const int64_t n = root->hi->iv, tpb = root->map.tpb;
    const int64_t launched = (n + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
    if (launched != root->map.n || tpb <= 0 || n / 4 < 256 * 64) return false;   // exactly one iteration per thread, and plenty
    if (k.grid.y != 1 || k.grid.z != 1 || k.block.y != 1 || k.block.z != 1) return false;
    bool straight = true;
    visit_stmts(root->body, [&](const S& c) {
      if (c->k == Stmt::For || c->k == Stmt::While || c->k == Stmt::Sync || c->k == Stmt::RawStmt) straight = false;
    });
    if (!straight) return false;
    Pass probe(k, opts, gen);
    if (probe.vector_width(root) != 4) return false;   // 4-byte elements through parameters only
    if (n % (4 * tpb) == 0) {
      // whole workgroups of whole vectors: shrink the launch and let the vectorised remap do the rest
      auto nr = clone(root);
      nr->map.n = n / 4;
      k.body = {S(nr)};
      k.grid.x = n / 4 / tpb;
      launch->grid = k.grid;
      return true;
    }
    // any other n: thread q takes elements 4q .. 4q+3; the last thread may hold fewer and tests each of its own
    ElemSize isz = opts.int_size();
    Type ity = Type::scalar(isz);
    const int64_t quads = (n + 3) / 4;
    Name q = gen.fresh(root->id.s + "_q");
    E qv = mk_var(q, ity);
    auto elements = [&](bool guarded) {
      Name u = gen.fresh(root->id.s + "_u");
      E d = mk_binop(BinOp::Add, mk_binop(BinOp::Mul, qv, mk_int(4, isz), ity), mk_var(u, ity), ity);
      Stmts ib;
      ib.push_back(mk_def(root->id, ity, d, root->i));
      for (auto& b : root->body) ib.push_back(b);
      if (guarded) {
        Stmts inner = {ib.begin() + 1, ib.end()};
        ib = {ib[0], mk_if(mk_binop(BinOp::Lt, mk_var(root->id, ity), mk_int(n, isz), Type::scalar(ElemSize::Bool)), inner, {})};
      }
      auto loop = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(
          mk_for(u, mk_int(0, isz), mk_int(4, isz), 1, ib, LoopPar(), root->i)));
      loop->unroll = true;
      return S(loop);
    };
    Stmts body;
    if (n % 4 == 0) {
      body = {elements(false)};
    } else {
      E whole = mk_binop(BinOp::Leq, mk_binop(BinOp::Add, mk_binop(BinOp::Mul, qv, mk_int(4, isz), ity), mk_int(4, isz), ity), mk_int(n, isz),
                         Type::scalar(ElemSize::Bool));
      body = {mk_if(whole, {elements(false)}, {elements(true)})};
    }
    auto nr = clone(root);
    nr->id = q;
    nr->hi = mk_int(quads, isz);
    nr->body = body;
    nr->map.n = (quads + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
    k.body = {S(nr)};
    k.grid.x = (nr->map.n + tpb - 1) / tpb;
    launch->grid = k.grid;
    return true;
  }

  void run() {
    Stmts host;
    for (auto& s : p.host) {
      if (s->k != Stmt::Launch) { host.push_back(s); continue; }
      Kernel* k = nullptr;
      for (auto& kk : p.kernels)
        if (kk.name == s->fname) k = &kk;
      auto ns = std::make_shared<Stmt>(*s);
      if (k && !k->opaque_body) apply(*k, ns);
      host.push_back(ns);
    }
    p.host = host;
  }
};

// ================================================================ host loops of launches inside one kernel
// A sequential loop that had to move to the host because its steps need all workgroups to meet
// (`for t: launch step(t)`) pays the fixed cost of a dependent launch per step -- several microseconds
// on the device, more than the step itself when the launch is small.  With `persistent_loops` the loop
// also exists as one kernel: the bodies of the step kernels in a `for t` loop, each followed by a barrier
// over all workgroups of the launch (a counter in device memory, what the workgroups exchange loaded and
// stored at device scope, a bounded wait).  The runtime uses that kernel only when the whole grid fits on
// the device at once -- otherwise workgroups would wait for others that cannot start -- and runs the loop
// of launches as before when it does not.  When the steps keep the values of one grid dimension apart
// (the reads of a batch), the barrier is one per value of that dimension instead of one over the grid.
struct PersistentLoops {
  Program& p;
  const Options& opts;
  NameGen& gen;
  ElemSize isz;

  PersistentLoops(Program& prog, const Options& o, NameGen& g) : p(prog), opts(o), gen(g), isz(o.int_size()) {}

  Kernel* find(const std::string& name) {
    for (auto& k : p.kernels)
      if (k.name == name) return &k;
    return nullptr;
  }

  // The outermost loop of a step kernel when it runs over one whole grid dimension and every access to memory that the
  // steps write names its variable as the first index: workgroups with different values of it never touch the same
  // element, so after a step only the workgroups of one value have to meet.  Null when that cannot be shown.
  const Stmt* group_loop(const Kernel& k, const std::set<Name>& written) {
    if (k.body.size() != 1) return nullptr;
    const Stmt* root = k.body[0].get();
    while (root->k == Stmt::Scope && root->body.size() == 1) root = root->body[0].get();
    if (!(root->k == Stmt::For && root->map.k == GpuMap::Block && root->map.mult == 1 && root->step == 1 && root->lo &&
          root->lo->k == Expr::Int && root->lo->iv == 0))
      return nullptr;
    int64_t extent = root->map.dim == 0 ? k.grid.x : root->map.dim == 1 ? k.grid.y : k.grid.z;
    if (extent != root->map.n || root->map.n < 2) return nullptr;
    std::set<Name> exchanged = written;   // and the local variables that take one of them as value
    bool ok = true;
    auto names_exchanged = [&](E rhs) {
      while (rhs && rhs->k == Expr::Convert) rhs = rhs->args[0];
      return rhs && rhs->k == Expr::Var && exchanged.count(rhs->name) > 0;
    };
    visit_stmts(root->body, [&](const S& s) {
      // one variable taking another's value is how the source and the destination of a step are chosen
      if (s->k == Stmt::Def && names_exchanged(s->expr)) exchanged.insert(s->id);
      if (s->k == Stmt::RawStmt || s->k == Stmt::CallStmt) ok = false;
      if ((s->k == Stmt::Def || s->k == Stmt::For) && s->id == root->id) ok = false;
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var && s->dst->name == root->id) ok = false;
    });
    std::function<void(const E&)> look = [&](const E& e) {
      if (!e || !ok) return;
      if (e->k == Expr::Raw) { ok = false; return; }
      if (e->k == Expr::Var && exchanged.count(e->name)) { ok = false; return; }   // a pointer that goes somewhere unseen
      if ((e->k == Expr::Index || e->k == Expr::AddrOf) && e->args[0]->k == Expr::Var) {
        if (exchanged.count(e->args[0]->name) &&
            !(e->dim_idx.size() >= 2 && e->dim_idx[0]->k == Expr::Var && e->dim_idx[0]->name == root->id && !e->dim_shape.empty() &&
              e->dim_shape[0] == root->map.n))
          ok = false;
        for (size_t a = 1; a < e->args.size(); ++a) look(e->args[a]);
        return;
      }
      for (auto& a : e->args) look(a);
    };
    visit_stmts(root->body, [&](const S& s) {
      bool alias = (s->k == Stmt::Def && exchanged.count(s->id)) || (s->k == Stmt::Assign && s->dst->k == Expr::Var && exchanged.count(s->dst->name));
      if (!(alias && names_exchanged(s->expr))) look(s->expr);
      if (!(s->dst && s->dst->k == Expr::Var)) look(s->dst);
      look(s->lo);
      look(s->hi);
      for (auto& a : s->args) look(a);
    });
    return ok ? root : nullptr;
  }

  S fuse(const S& loop) {
    if (!(loop->k == Stmt::For && loop->map.k == GpuMap::None && loop->step == 1 && !loop->body.empty())) return S();
    std::vector<Kernel*> ks;
    for (auto& l : loop->body) {
      if (l->k != Stmt::Launch) return S();
      Kernel* k = find(l->fname);
      if (!k || k->opaque_body) return S();
      // the argument of every parameter must be the host variable of the same name (how launches are generated)
      for (size_t i = 0; i < k->params.size(); ++i)
        if (!(l->args[i]->k == Expr::Var && l->args[i]->name == k->params[i].id)) return S();
      ks.push_back(k);
    }
    const Kernel& k0 = *ks[0];
    for (auto* k : ks)
      if (k->grid.x != k0.grid.x || k->grid.y != k0.grid.y || k->grid.z != k0.grid.z || k->block.x != k0.block.x ||
          k->block.y != k0.block.y || k->block.z != k0.block.z)
        return S();
    int64_t nblocks = k0.grid.x * k0.grid.y * k0.grid.z;
    // the barrier counter runs up to (number of barriers) x (number of workgroups) in 32 bits
    if (loop->lo->k != Expr::Int || loop->hi->k != Expr::Int) return S();
    int64_t trips = loop->hi->iv - loop->lo->iv;
    if (trips < 2 || trips * (int64_t)ks.size() * nblocks >= (int64_t(1) << 32)) return S();
    Kernel f;
    f.name = p.name + "_steps_" + std::to_string(gen.next++);
    f.grid = k0.grid;
    f.block = k0.block;
    f.cached_stores = true;
    f.no_restrict = true;
    f.aligned_params = k0.aligned_params;
    std::map<Name, size_t> seen;
    for (auto* k : ks)
      for (auto& q : k->params) {
        if (q.id == loop->id) continue;
        auto it = seen.find(q.id);
        if (it == seen.end()) { seen[q.id] = f.params.size(); f.params.push_back(q); }
        else if (!q.read_only) f.params[it->second].read_only = false;
      }
    // What the workgroups exchange is loaded and stored at device scope, which the printer does for elements of
    // four bytes and more; narrower elements would keep plain cached accesses and a compute unit could serve a line
    // that another workgroup rewrote a step ago.  Such loops stay a loop of launches.
    for (auto& q : f.params)
      if (q.ty.k == Type::Pointer && !q.read_only && elem_bytes(q.ty.sz) < 4) return S();
    // Workgroups that never touch each other's elements (those of different reads of a batch) need not wait for each
    // other: each value of the grid dimension that keeps them apart gets a counter of its own, 128 bytes apart.
    std::set<Name> written;
    for (auto& q : f.params)
      if (q.ty.k == Type::Pointer && !q.read_only) written.insert(q.id);
    int group_dim = -1;
    int64_t groups = 1;
    for (auto* k : ks) {
      const Stmt* g = group_loop(*k, written);
      if (!g || (group_dim >= 0 && g->map.dim != group_dim)) { group_dim = -1; groups = 1; break; }
      group_dim = g->map.dim;
      groups = g->map.n;
    }
    Type u32 = Type::scalar(ElemSize::U32);
    KernelParam counter, status, limit;
    counter.id = gen.fresh("parpy_bar_counter"); counter.ty = Type::pointer(ElemSize::U32);
    status.id = gen.fresh("parpy_bar_status"); status.ty = Type::pointer(ElemSize::U32);
    limit.id = gen.fresh("parpy_bar_limit"); limit.ty = u32;
    std::string which = groups > 1 ? counter.id.str() + " + 32u * blockIdx." + std::string(1, "xyz"[group_dim]) : counter.id.str();
    std::string bar = "if (!parpy_grid_barrier(" + which + ", " + status.id.str() + ", " + std::to_string(nblocks / groups) +
                      "u, parpy_bar_epoch, " + limit.id.str() + ")) return;";
    Stmts step;
    for (auto* k : ks) {
      step.push_back(mk_scope(k->body));
      step.push_back(mk_rawstmt(bar));
    }
    auto t = clone(loop);
    t->body = step;
    f.body = {mk_rawstmt("unsigned parpy_bar_epoch = 0;"), S(t)};
    auto l = std::make_shared<Stmt>();
    l->k = Stmt::PersistentLaunch;
    l->fname = f.name;
    l->grid = f.grid;
    l->block = f.block;
    l->i = loop->i;
    l->iv = groups;   // counters the barrier needs
    for (auto& q : f.params) l->args.push_back(mk_var(q.id, q.ty));
    l->body = {loop};
    f.params.push_back(counter);
    f.params.push_back(status);
    f.params.push_back(limit);
    p.kernels.push_back(f);
    return l;
  }

  Stmts walk(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (S f = fuse(s)) { out.push_back(f); continue; }
      auto r = clone(s);
      if (s->k == Stmt::For || s->k == Stmt::While || s->k == Stmt::If) {
        r->body = walk(s->body);
        r->els = walk(s->els);
      }
      out.push_back(r);
    }
    return out;
  }

  void run() { p.host = walk(p.host); }
};

}  // namespace

void hip_optimize(Program& p, const Options& opts, NameGen& gen) {
  if (opts.opt_gather_transpose) GatherTranspose(p, opts, gen).run();
  if (opts.opt_lane_split && !opts.opt_mfma_sddmm) LaneSplit(p, opts, gen).run();
  if (opts.opt_vectorize) Coarsen(p, opts, gen).run();
  for (auto& k : p.kernels) {
    if (k.opaque_body) { k.aligned_params = opts.assume_aligned; continue; }
    Pass pass(k, opts, gen);
    if (opts.opt_unswitch) pass.unswitch_aliases();
    if (opts.opt_mfma_sddmm) k.body = pass.mfma_dot(k.body);
    k.body = pass.propagate_constants(k.body);
    if (opts.opt_expand_short_loops) k.body = pass.expand_short_loops(k.body, false);
    if (opts.opt_guard_bounds) k.body = pass.guards_to_bounds(k.body);
    if (opts.opt_prefetch_steps) k.body = pass.prefetch_counter_loads(k.body, RangeEnv());
    if (opts.opt_unswitch_uniform) k.body = pass.hoist_uniform_conditions(k.body);
    if (opts.opt_if_convert) k.body = pass.if_convert(k.body);
    if (opts.opt_lds_rows) pass.lds_rows();
    if (opts.opt_vectorize) k.body = pass.vectorize(k.body);
    int64_t budget = pass.reg_budget();
    if (opts.opt_hoist_invariant) k.body = pass.hoist_invariant(k.body, &budget, false);
    if (opts.opt_prefetch_steps) k.body = pass.prefetch_selected_rows(k.body, &budget);
    if (opts.opt_keep_stored) k.body = pass.keep_stored_rows(k.body, &budget);
    if (opts.opt_reg_cache) pass.reg_cache(&budget);
    if (opts.opt_share_iterations) {
      k.distinct_pointers.clear();
      pass.noalias_scopes(k.body, false);
      k.body = pass.share_own_iterations(k.body);
    }
    if (opts.opt_drop_barriers) pass.drop_barriers();
    k.distinct_pointers.clear();
    k.body = pass.noalias_scopes(k.body, opts.opt_noalias_scopes);
    k.fence_lds_iterations = opts.opt_fence_iterations && !pass.step_has_transcendentals();
    pass.mark_read_only();
    k.aligned_params = opts.assume_aligned;
  }
  if (opts.persistent_loops) PersistentLoops(p, opts, gen).run();
}

}  // namespace parpy
