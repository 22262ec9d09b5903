// gfx950 memory passes, control flow inside a kernel: constants, short loops, guards, uniform and value-picking branches, array aliases.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

std::set<Name> Pass::param_names() const {
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
struct Pass::Unswitch {
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
bool Pass::straight_line(const Stmts& ss) {
  for (auto& s : ss) {
    if (s->k == Stmt::If) { if (!straight_line(s->body) || !straight_line(s->els)) return false; continue; }
    if (s->k != Stmt::Def && s->k != Stmt::Assign) return false;
  }
  return true;
}

// Local names that are defined once with a literal value (`nq = hmm["num_states"] // 4` after the shapes
// are known) stand for that value wherever they are read: index arithmetic written with them folds like
// arithmetic written with the numbers, which the passes that compare offsets rely on.
Stmts Pass::propagate_constants(const Stmts& ss) {
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

size_t Pass::count_stmts(const Stmts& ss) {
  size_t n = 0;
  visit_stmts(ss, [&](const S&) { ++n; });
  return n;
}

Stmts Pass::expand_short_loops(const Stmts& ss0, bool in_par) {
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
E Pass::strip_converts(const E& e) { return e->k == Expr::Convert ? strip_converts(e->args[0]) : e; }

Stmts Pass::guards_to_bounds(const Stmts& ss) {
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

// ================================================================ conditions no iteration changes
// A parallel loop whose whole body is `if (c) A else B`, with c the same for every iteration (it
// mentions neither the loop variable nor anything the body defines or assigns, and loads only from
// arrays the kernel never writes), becomes `if (c) { loop A } else { loop B }`.  The HMM step tests
// `t < lens[inst]` (and `t == lens[inst]` in the else branch) once per state; inside the unrolled
// loop that is a branch between any two states, which keeps the instructions of neighbouring
// states from being scheduled together.  Only tests with an else branch are rewritten: a plain
// `if (c) A` the device compiler unswitches by itself, and doing it here first was measured to
// cost 5 % on the single-layer HMM step (60.4 -> 63.4 ms; the 16-layer model gains 6 %).
Stmts Pass::hoist_uniform_conditions(const Stmts& ss) {
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
Stmts Pass::if_convert(const Stmts& ss) {
  // variables that stand for a non-zero integer constant (`num_kmers = 1024`): dividing by them is safe to do early
  std::set<Name> reassigned, nonzero_const;
  visit_stmts(k.body, [&](const S& st) { if (st->k == Stmt::Assign && st->dst->k == Expr::Var) reassigned.insert(st->dst->name); });
  visit_stmts(k.body, [&](const S& st) {
    if (st->k == Stmt::Def && st->expr && st->expr->k == Expr::Int && st->expr->iv != 0 && !reassigned.count(st->id)) nonzero_const.insert(st->id);
  });
  return if_convert(ss, nonzero_const);
}

Stmts Pass::if_convert(const Stmts& ss, const std::set<Name>& nonzero_const) {
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

void Pass::unswitch_aliases() {
  bool any = false;
  visit_stmts(k.body, [&](const S& s) { if (s->k == Stmt::Def && Unswitch::is_alias_type(s->ty)) any = true; });
  if (!any) return;
  Unswitch u;
  Stmts nb = u.run(k.body, 0, {});
  if (!u.failed) k.body = nb;
}

}  // namespace hipopt
}  // namespace parpy
