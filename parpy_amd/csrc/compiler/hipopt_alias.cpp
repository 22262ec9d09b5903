// gfx950 memory passes, what the target compiler may assume about pointers: distinct arrays, read-only parameters.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ no-alias scopes for array aliases
// `src = a; dst = b; if (c) { src = b; dst = a; } <rest>`: in <rest> the two aliases always name
// different arrays, but the target compiler only sees two selected pointers that may be equal, so
// it keeps every load from `src` behind the preceding store to `dst`.  When every combination of
// the selections gives pairwise different arrays, and <rest> reaches those arrays through the
// aliases only, <rest> is put into a scope whose parameters are the aliases, declared not to
// alias each other.  Loads of the (independent) iterations that a thread runs of a parallel loop
// can then be shared and merged: the four states of a thread that have the same predecessors load
// them once, and own-state loads and stores become 128-bit LDS accesses.
bool Pass::is_alias_type(const Type& t) { return t.k == Type::Pointer || (t.k == Type::Tensor && !t.shape.empty()); }

bool Pass::alias_target(const E& e, const AliasCfg& cfg, Name* out) {
  if (!e || e->k != Expr::Var) return false;
  auto it = cfg.find(e->name);
  *out = it == cfg.end() ? e->name : it->second;
  return true;
}

// statements that only (re)point aliases: applies them to every configuration, false if anything else is found
bool Pass::apply_alias_stmt(const S& st, std::vector<AliasCfg>& cfgs, std::vector<Name>& order) {
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
Stmts Pass::noalias_scopes(const Stmts& ss, bool wrap) {
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

// ================================================================ read-only parameters
// A pointer parameter is read-only when nothing in the kernel stores through
// it, directly or through a local alias initialised from it.
void Pass::mark_read_only() {
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

}  // namespace hipopt
}  // namespace parpy
