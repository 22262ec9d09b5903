// gfx950 memory passes, rows that live in LDS for a whole kernel, and the barriers between regions that share nothing.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

// ================================================================ LDS rows
void Pass::lds_rows() {
  if (k.body.size() != 1 || k.body[0]->k != Stmt::For || k.body[0]->map.k != GpuMap::Block) return;
  const S root = k.body[0];
  int64_t ext = const_extent(root);
  if (ext <= 0 || ext > root->map.n) return;  // a block must own exactly one value of the root variable
  if (k.block.y != 1 || k.block.z != 1) return;
  // one workgroup per value of the root variable: when the loops below spread over several workgroups, each of them
  // would copy the whole row in and out and overwrite what the others computed
  if (k.grid.x * k.grid.y * k.grid.z != root->map.n) return;
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

// ================================================================ barriers that order nothing
// The generic pipeline puts a barrier after every parallel loop.  Once rows live in registers, a
// loop may touch no memory at all (softmax's `exp` and scaling steps), and the barrier after it --
// or the one before the next memory access -- orders nothing.  A barrier between two straight-line
// regions of the workgroup's top-level statement list is kept only if an array written on one
// side is accessed on the other; accesses through pointer variables, helper calls and raw
// statements count as touching everything.  Barriers inside sequential loops are left alone (the
// region after them wraps round to the loop head).  Reduction sites own their LDS slots and
// synchronise internally.
void Pass::touched(const Stmts& ss, const std::set<Name>& arrays, Touched& t) {
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

Stmts Pass::drop_barriers_in(const Stmts& ss, const std::set<Name>& arrays) {
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

void Pass::drop_barriers() {
  std::set<Name> arrays;
  for (auto& p : k.params) if (p.ty.is_pointer()) arrays.insert(p.id);
  visit_stmts(k.body, [&](const S& st) { if (st->k == Stmt::LdsDecl) arrays.insert(st->id); });
  k.body = drop_barriers_in(k.body, arrays);
}

}  // namespace hipopt
}  // namespace parpy
