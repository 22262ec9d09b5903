// GPU structuring: synchronisation points, multi-block reduction split,
// hoisting of sequential loops that need grid-wide synchronisation, kernel
// splitting, device temporaries, the wave64 grid mapper, kernel extraction,
// reduction lowering and the block-wide store hazard pass.
//
// Behavioural counterparts in the reference: src/gpu/inter_block.rs:17-1116,
// src/gpu/par.rs:105-335 (grid mapper; WARP_SIZE 32 there, 64 here),
// src/gpu/codegen.rs:106-604, src/gpu/reduce.rs:17-480,
// src/gpu/global_mem.rs:102-205, src/gpu/sync_elim.rs:4-39,
// src/gpu/free_vars.rs:64-67.
#include <algorithm>
#include <functional>
#include <optional>

#include "passes.hpp"

namespace parpy {

namespace {

using StmtP = std::shared_ptr<Stmt>;
StmtP clone(const S& s) { return std::make_shared<Stmt>(*s); }

S mk_syncpoint(SyncKind k, const Info& i) {
  auto s = std::make_shared<Stmt>();
  s->k = Stmt::SyncPoint;
  s->sync = k;
  s->i = i;
  return s;
}

bool is_par_for(const S& s) { return s->k == Stmt::For && s->par.is_parallel(); }
bool is_ib_sync(const S& s) { return s->k == Stmt::SyncPoint && s->sync == SyncKind::InterBlock; }

SyncKind classify_parallelism(const LoopPar& p) {  // src/gpu/inter_block.rs:46-58 without clusters
  int64_t n = (p.nthreads + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
  if (p.nthreads > 0 && (p.nthreads <= p.tpb || n <= p.tpb)) return SyncKind::BlockLocal;
  return SyncKind::InterBlock;
}

int par_height(const Stmts& ss) {
  int h = 0;
  for (auto& s : ss) {
    int inner = std::max(par_height(s->body), par_height(s->els));
    if (is_par_for(s)) inner += 1;
    h = std::max(h, inner);
  }
  return h;
}

bool contains_ib_sync(const Stmts& ss) {
  for (auto& s : ss)
    if (is_ib_sync(s) || contains_ib_sync(s->body) || contains_ib_sync(s->els)) return true;
  return false;
}

bool contains_par(const Stmts& ss) {
  for (auto& s : ss)
    if (is_par_for(s) || contains_par(s->body) || contains_par(s->els)) return true;
  return false;
}

E rename_expr(const E& e, const std::map<Name, Name>& m) {
  if (!e) return e;
  if (e->k == Expr::Var) {
    auto it = m.find(e->name);
    if (it == m.end()) return e;
    auto r = std::make_shared<Expr>(*e);
    r->name = it->second;
    return r;
  }
  return map_children(e, [&](const E& c) { return rename_expr(c, m); });
}

E subst_expr(const E& e, const std::map<Name, E>& m) {
  if (!e) return e;
  if (e->k == Expr::Var) {
    auto it = m.find(e->name);
    return it == m.end() ? e : it->second;
  }
  return map_children(e, [&](const E& c) { return subst_expr(c, m); });
}

// ================================================================ restructuring
struct Restructure {
  const Options& opts;
  NameGen& gen;
  ElemSize isz;

  Restructure(const Options& o, NameGen& g) : opts(o), gen(g), isz(o.int_size()) {}

  // ---- 1. a synchronisation point after every parallel loop (inter_block.rs:17-36)
  Stmts insert_sync(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      auto r = clone(s);
      r->body = insert_sync(s->body);
      r->els = insert_sync(s->els);
      out.push_back(r);
      if (is_par_for(s)) out.push_back(mk_syncpoint(SyncKind::InterBlock, s->i));
    }
    return out;
  }

  // ---- 2. classification (inter_block.rs:60-148)
  Stmts classify_par(const Stmts& ss, int inner_height) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::SyncPoint) {
        SyncKind prev = SyncKind::InterBlock;
        if (!out.empty() && out.back()->k == Stmt::For) prev = classify_parallelism(out.back()->par);
        out.push_back(mk_syncpoint(inner_height == 1 ? prev : SyncKind::InterBlock, s->i));
        continue;
      }
      auto r = clone(s);
      if (s->k == Stmt::For) {
        r->body = classify_par(s->body, par_height(s->body));
      } else {
        r->body = classify_par(s->body, inner_height);
        r->els = classify_par(s->els, inner_height);
      }
      out.push_back(r);
    }
    return out;
  }

  Stmts classify(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      auto r = clone(s);
      if (is_par_for(s)) {
        r->body = classify_par(s->body, par_height(s->body));
      } else {
        r->body = classify(s->body);
        r->els = classify(s->els);
      }
      out.push_back(r);
    }
    return out;
  }

  // ---- 3. multi-block reductions (inter_block.rs:150-433)
  static BinOp non_short_circuit(BinOp op) { return op == BinOp::And ? BinOp::BitAnd : op == BinOp::Or ? BinOp::BitOr : op; }

  Stmts split_reductions(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::For && s->par.is_parallel() && s->par.reduction &&
          classify_parallelism(s->par) == SyncKind::InterBlock) {
        const LoopPar& par = s->par;
        if (par.nthreads % par.tpb != 0)
          fail_rt(s->i, "Multi-block reductions must use a multiple of " + std::to_string(par.tpb) + " threads.");
        int64_t nblocks = par.nthreads / par.tpb;
        E lhs, rhs;
        BinOp op;
        ElemSize sz;
        extract_reduction(s, &lhs, &op, &rhs, &sz);
        Type ty = Type::scalar(sz);
        Type ity = Type::scalar(isz);
        Name bid = gen.fresh("block_idx");
        Name tmp = gen.fresh("tmp");
        E tmpv = mk_var(tmp, ty, s->i);
        E block = mk_var(bid, ity, s->i);
        // contiguous chunk of the iteration space for each block
        E ofs = mk_binop(BinOp::FloorDiv,
                         mk_binop(BinOp::Add, mk_binop(BinOp::Sub, s->hi, s->lo, ity), mk_int(nblocks - 1, isz), ity),
                         mk_int(nblocks, isz), ity);
        E lo = mk_binop(BinOp::Add, s->lo, mk_binop(BinOp::Mul, ofs, block, ity), ity);
        E hi = mk_binop(BinOp::Min, mk_binop(BinOp::Add, lo, ofs, ity), s->hi, ity);
        LoopPar ipar;
        ipar.nthreads = par.tpb;
        ipar.reduction = true;
        ipar.tpb = par.tpb;
        S inner = mk_for(s->id, fold_expr(lo), fold_expr(hi), s->step,
                         {mk_assign(tmpv, mk_binop(op, tmpv, rhs, ty, s->i), s->i)}, ipar, s->i);
        LoopPar opar;
        opar.nthreads = nblocks;
        opar.tpb = par.tpb;
        S outer = mk_for(bid, mk_int(0, isz), mk_int(nblocks, isz), 1,
                         {mk_def(tmp, ty, neutral_element(op, sz, s->i), s->i), inner}, opar, s->i);
        out.push_back(outer);
        out.push_back(mk_syncpoint(SyncKind::InterBlock, s->i));
        LoopPar spar;
        spar.nthreads = std::min<int64_t>(nblocks, DEFAULT_TPB);
        spar.reduction = true;
        // the partial results are reduced by one workgroup, also when there are more of them than the first stage's
        // workgroups have threads (8192 threads in workgroups of 64: 128 partial results)
        spar.tpb = std::max(par.tpb, spar.nthreads);
        out.push_back(mk_for(bid, mk_int(0, isz), mk_int(nblocks, isz), 1,
                             {mk_assign(lhs, mk_binop(op, lhs, tmpv, ty, s->i), s->i)}, spar, s->i));
        continue;
      }
      auto r = clone(s);
      r->body = split_reductions(s->body);
      r->els = split_reductions(s->els);
      out.push_back(r);
    }
    return out;
  }

 public:
  // The body of a reduction loop must be `x = x op e` (src/gpu/reduce.rs:97-137).
  static void extract_reduction(const S& loop, E* lhs, BinOp* op, E* rhs, ElemSize* sz) {
    if (loop->body.size() != 1) fail_rt(loop->i, "Reduction for-loop must contain a single statement.");
    const S& a = loop->body[0];
    if (a->k != Stmt::Assign) fail_rt(loop->i, "Reduction for-loop statement must be an assignment.");
    E e = a->expr;
    while (e->k == Expr::Convert) e = e->args[0];
    if (e->k != Expr::BinOpE) fail_rt(a->i, "RHS of reduction statement should be a binary operation.");
    if (!e->ty.is_scalar()) fail_rt(a->i, "Expected the result of reduction to be a scalar value, found " + e->ty.str());
    E l = e->args[0];
    while (l->k == Expr::Convert) l = l->args[0];
    if (a->dst->k != Expr::Var && a->dst->k != Expr::Index)
      fail_rt(a->i, "Left-hand side of reduction must be a variable or tensor access.");
    if (!expr_eq(a->dst, l))
      fail_rt(a->i, "Invalid reduction. Left-hand side of binary operation " + print_expr(e->args[0]) +
                        " is not equal to the assignment target " + print_expr(a->dst) + ".");
    *lhs = a->dst;
    *op = non_short_circuit(e->bop);
    *rhs = e->args[1];
    *sz = e->ty.sz;
  }

 private:
  // ---- 4. hoisting (inter_block.rs:448-633)
  static bool is_seq_loop_with_ib(const S& s) { return s->k == Stmt::For && !s->par.is_parallel() && contains_ib_sync(s->body); }

  template <class P> static std::vector<Stmts> split_inclusive(const Stmts& ss, P pred) {
    std::vector<Stmts> chunks;
    Stmts cur;
    for (auto& s : ss) {
      cur.push_back(s);
      if (pred(s)) { chunks.push_back(cur); cur.clear(); }
    }
    if (!cur.empty()) chunks.push_back(cur);
    return chunks;
  }

  S with_body(const S& loop, Stmts body) {
    auto r = clone(loop);
    r->body = std::move(body);
    return r;
  }

  Stmts hoist_chunk(const S& root, const Stmts& chunk) {
    const S& last = chunk.back();
    Stmts out;
    if (is_seq_loop_with_ib(last)) {
      Stmts pre = hoist_inner(Stmts(chunk.begin(), chunk.end() - 1));
      if (!pre.empty()) out.push_back(with_body(root, pre));
      Stmts inner;
      for (auto& sub : split_inclusive(last->body, is_ib_sync)) {
        Stmts piece{with_body(root, sub)};
        if (sub.back()->k == Stmt::SyncPoint) piece.push_back(sub.back());
        for (auto& s : hoist_inner(piece)) inner.push_back(s);
      }
      out.push_back(with_body(last, inner));
      return out;
    }
    Stmts body = hoist_inner(chunk);
    if (std::any_of(body.begin(), body.end(), is_seq_loop_with_ib)) return hoist_seq_loops(with_body(root, body));
    out.push_back(with_body(root, body));
    return out;
  }

  Stmts hoist_seq_loops(const S& root) {
    Stmts out;
    for (auto& chunk : split_inclusive(root->body, is_seq_loop_with_ib))
      for (auto& s : hoist_chunk(root, chunk)) out.push_back(s);
    return out;
  }

  Stmts hoist_inner(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        for (auto& r : hoist_seq_loops(s)) out.push_back(r);
      } else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = hoist_inner(s->body);
        r->els = hoist_inner(s->els);
        out.push_back(r);
      } else {
        out.push_back(s);
      }
    }
    return out;
  }

  Stmts hoist(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        for (auto& r : hoist_inner({s})) out.push_back(r);
      } else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = hoist(s->body);
        r->els = hoist(s->els);
        out.push_back(r);
      } else {
        out.push_back(s);
      }
    }
    return out;
  }

  // ---- 5. split kernels at the remaining grid-wide synchronisation points (inter_block.rs:639-678)
  // A nested parallel loop that is cut into several pieces takes its enclosing loops with it: the grid-wide
  // synchronisation between two pieces (a multi-block reduction under two parallel levels: partial results per
  // block, then their reduction) is repeated one level up, where it cuts the enclosing loop in the same place, so
  // that the first kernel maps (outer loops, blocks, threads) and the second (outer loops, threads).
  void push_pieces(Stmts& body, const S& child, const Stmts& pieces) {
    for (size_t k = 0; k < pieces.size(); ++k) {
      body.push_back(pieces[k]);
      if (k + 1 < pieces.size() && child->par.is_parallel()) body.push_back(mk_syncpoint(SyncKind::InterBlock, child->i));
    }
  }

  // Only sequential for-loops are moved out of a parallel loop to make room for a synchronisation of all workgroups
  // (src/gpu/inter_block.rs:448-633 does the same); a conditional or a while loop cannot be.
  void refuse_grid_sync_under(const S& s) {
    if ((s->k == Stmt::If || s->k == Stmt::While) && (contains_ib_sync(s->body) || contains_ib_sync(s->els)))
      fail_rt(s->i, std::string("A parallel statement that spans several workgroups (more threads than fit one workgroup, or a "
                                "reduction over them) sits under ") + (s->k == Stmt::If ? "a conditional" : "a while loop") +
                        " inside a parallel loop, where all workgroups cannot meet; give it at most one workgroup's threads or "
                        "move the condition into it");
  }

  Stmts split_kernel(const S& loop) {
    Stmts body;
    for (auto& s : loop->body) {
      refuse_grid_sync_under(s);
      if (s->k == Stmt::For) push_pieces(body, s, split_kernel(s));
      else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = split_in_kernel(s->body);
        r->els = split_in_kernel(s->els);
        body.push_back(r);
      } else body.push_back(s);
    }
    Stmts out;
    for (auto& chunk : split_inclusive(body, is_ib_sync)) out.push_back(with_body(loop, chunk));
    return out;
  }

  Stmts split_in_kernel(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::For) push_pieces(out, s, split_kernel(s));
      else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = split_in_kernel(s->body);
        r->els = split_in_kernel(s->els);
        out.push_back(r);
      } else out.push_back(s);
    }
    return out;
  }

  Stmts split_sync(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        for (auto& r : split_kernel(s)) out.push_back(r);
      } else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = split_sync(s->body);
        r->els = split_sync(s->els);
        out.push_back(r);
      } else out.push_back(s);
    }
    return out;
  }

  // ---- 6. drop synchronisation points that do nothing (inter_block.rs:680-748)
  Stmts drop_syncs(const Stmts& ss0, bool in_par, bool par_body) {
    Stmts ss = ss0;
    if (par_body && !ss.empty() && ss.back()->k == Stmt::SyncPoint) ss.pop_back();
    Stmts out;
    for (auto& s : ss) {
      if (is_ib_sync(s) && !in_par) continue;
      if (s->k == Stmt::For) {
        auto r = clone(s);
        bool p = s->par.is_parallel();
        r->body = drop_syncs(s->body, in_par || p, p);
        if (p && r->body.empty()) continue;  // a kernel that does nothing
        out.push_back(r);
      } else if (s->k == Stmt::While) {
        auto r = clone(s);
        r->body = drop_syncs(s->body, in_par, false);
        out.push_back(r);
      } else if (s->k == Stmt::If) {
        auto r = clone(s);
        r->body = drop_syncs(s->body, in_par, par_body && false);
        r->els = drop_syncs(s->els, in_par, false);
        out.push_back(r);
      } else {
        out.push_back(s);
      }
    }
    return out;
  }

  // ---- 7. locals that now cross kernels live in device temporaries (inter_block.rs:795-1053)
  struct DefUse { std::set<Name> defs, uses; };

  static void collect_kernel(const Stmts& ss, DefUse& du) {
    for (auto& s : ss) {
      if (s->k == Stmt::Def || s->k == Stmt::For) du.defs.insert(s->id);
      auto use = [&](const E& e) { visit_exprs(e, [&](const E& x) { if (x->k == Expr::Var) du.uses.insert(x->name); }); };
      use(s->dst); use(s->expr); use(s->lo); use(s->hi);
      for (auto& a : s->args) use(a);
      collect_kernel(s->body, du);
      collect_kernel(s->els, du);
    }
  }

  static void collect_host(const Stmts& ss, std::vector<DefUse>& kernels, std::set<Name>& bound) {
    for (auto& s : ss) {
      if (s->k == Stmt::Def) bound.insert(s->id);
      if (s->k == Stmt::For) {
        if (s->par.is_parallel()) {
          DefUse du;
          du.defs.insert(s->id);
          collect_kernel(s->body, du);
          kernels.push_back(du);
          continue;
        }
        bound.insert(s->id);
      }
      collect_host(s->body, kernels, bound);
      collect_host(s->els, kernels, bound);
    }
  }

  struct TempData { Name id; Type elem; E access; int64_t size; };

  void collect_temp_data(const Stmts& ss, const std::set<Name>& temp_vars, std::map<Name, TempData>& data,
                         std::vector<std::pair<S, int64_t>>& par_structure) {
    for (auto& s : ss) {
      if (s->k == Stmt::Def && temp_vars.count(s->id) && !data.count(s->id)) {
        if (!s->ty.is_scalar())
          fail_rt(s->i, "Cannot allocate temporary data for non-scalar variable " + s->id.s + ".");
        Type ity = Type::scalar(isz);
        E idx = mk_int(0, isz);
        int64_t size = 1;
        for (size_t k = par_structure.size(); k-- > 0;) {
          const S& loop = par_structure[k].first;
          E lo = fold_expr(loop->lo), hi = fold_expr(loop->hi);
          if (lo->k != Expr::Int || hi->k != Expr::Int)
            fail_rt(loop->i, "A parallel loop around a variable that crosses kernels must have constant bounds.");
          int64_t extent = loop->step > 0 ? (hi->iv - lo->iv + loop->step - 1) / loop->step
                                          : (lo->iv - hi->iv - loop->step - 1) / (-loop->step);
          E rel = mk_binop(BinOp::FloorDiv, mk_binop(BinOp::Sub, mk_var(loop->id, ity), loop->lo, ity),
                           mk_int(loop->step, isz), ity);
          idx = mk_binop(BinOp::Add, idx, mk_binop(BinOp::Mul, rel, mk_int(size, isz), ity), ity);
          size *= std::max<int64_t>(extent, 1);
        }
        Name nid = gen.fresh(s->id.s + "_tmp");
        TempData td;
        td.id = nid;
        td.elem = s->ty;
        td.size = size;
        td.access = mk_index(mk_var(nid, Type::pointer(s->ty.sz)), fold_expr(idx), s->ty, s->i);
        data[s->id] = td;
      }
      if (is_par_for(s)) {
        par_structure.emplace_back(s, 0);
        collect_temp_data(s->body, temp_vars, data, par_structure);
        par_structure.pop_back();
      } else {
        collect_temp_data(s->body, temp_vars, data, par_structure);
        collect_temp_data(s->els, temp_vars, data, par_structure);
      }
    }
  }

  Stmts replace_temps(const Stmts& ss, const std::map<Name, TempData>& data) {
    std::map<Name, E> m;
    for (auto& kv : data) m[kv.first] = kv.second.access;
    Stmts out;
    for (auto& s : ss) {
      S t = map_exprs(s, [&](const E& e) { return subst_expr(e, m); });
      auto r = clone(t);
      if (s->k == Stmt::Def && data.count(s->id)) {
        r->k = Stmt::Assign;
        r->dst = data.at(s->id).access;
      }
      r->body = replace_temps(s->body, data);
      r->els = replace_temps(s->els, data);
      out.push_back(r);
    }
    return out;
  }

  // Array aliases (`alpha = alpha2; if c: alpha = alpha1`) that end up defined
  // in one kernel and used in a later one are recomputed where they are used:
  // the statements that select the pointer are copied to the start of every
  // kernel that needs them, which costs nothing compared with a device array
  // of pointers.
  static bool only_assigns_to(const Stmts& ss, const Name& v) {
    for (auto& s : ss) {
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var && s->dst->name == v) continue;
      if (s->k == Stmt::If && only_assigns_to(s->body, v) && only_assigns_to(s->els, v)) continue;
      return false;
    }
    return true;
  }

  Stmts rematerialize_aliases(const Stmts& ss, std::map<Name, Stmts>& slices) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        DefUse du;
        du.defs.insert(s->id);
        collect_kernel(s->body, du);
        Stmts body;
        for (auto& kv : slices)
          if (du.uses.count(kv.first) && !du.defs.count(kv.first))
            for (auto& d : kv.second) body.push_back(d);
        for (auto& c : s->body) {
          body.push_back(c);
          if (c->k == Stmt::Def && !c->ty.is_scalar()) slices[c->id] = {c};
          else if (c->k == Stmt::Assign && c->dst->k == Expr::Var && slices.count(c->dst->name)) slices[c->dst->name].push_back(c);
          else if (c->k == Stmt::If)
            for (auto& kv : slices)
              if (only_assigns_to({c}, kv.first)) kv.second.push_back(c);
        }
        out.push_back(with_body(s, body));
      } else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = rematerialize_aliases(s->body, slices);
        r->els = rematerialize_aliases(s->els, slices);
        out.push_back(r);
      } else {
        out.push_back(s);
      }
    }
    return out;
  }

  // An assignment at the top level of a kernel to a variable that the kernel
  // neither defined nor read before is a definition there: the value does not
  // come from another kernel (src/gpu/inter_block.rs:1095-1099).
  Stmts promote_assignments(const Stmts& ss, const std::set<Name>& host_bound) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        std::set<Name> defs{s->id}, used;
        Stmts body;
        for (auto& c : s->body) {
          bool promote = c->k == Stmt::Assign && c->dst->k == Expr::Var && c->dst->ty.is_scalar() &&
                         !defs.count(c->dst->name) && !used.count(c->dst->name) && !host_bound.count(c->dst->name);
          if (promote) {
            bool self = false;
            visit_exprs(c->expr, [&](const E& x) { if (x->k == Expr::Var && x->name == c->dst->name) self = true; });
            promote = !self;
          }
          DefUse du;
          collect_kernel({c}, du);
          if (promote) {
            body.push_back(mk_def(c->dst->name, c->dst->ty, c->expr, c->i));
            defs.insert(c->dst->name);
          } else {
            body.push_back(c);
          }
          defs.insert(du.defs.begin(), du.defs.end());
          used.insert(du.uses.begin(), du.uses.end());
        }
        out.push_back(with_body(s, body));
      } else if (!s->body.empty() || !s->els.empty()) {
        auto r = clone(s);
        r->body = promote_assignments(s->body, host_bound);
        r->els = promote_assignments(s->els, host_bound);
        out.push_back(r);
      } else {
        out.push_back(s);
      }
    }
    return out;
  }

  Stmts allocate_temporaries(const Stmts& body0, const std::vector<Param>& params) {
    std::map<Name, Stmts> slices;
    Stmts body = rematerialize_aliases(body0, slices);
    {
      std::vector<DefUse> ks;
      std::set<Name> host_bound;
      for (auto& p : params) host_bound.insert(p.id);
      collect_host(body, ks, host_bound);
      body = promote_assignments(body, host_bound);
    }
    std::vector<DefUse> kernels;
    std::set<Name> bound;
    for (auto& p : params) bound.insert(p.id);
    collect_host(body, kernels, bound);
    std::set<Name> temp_vars;
    for (auto& du : kernels)
      for (auto& u : du.uses)
        if (!du.defs.count(u) && !bound.count(u)) temp_vars.insert(u);
    if (temp_vars.empty()) return body;
    std::map<Name, TempData> data;
    std::vector<std::pair<S, int64_t>> ps;
    collect_temp_data(body, temp_vars, data, ps);
    for (auto& v : temp_vars)
      if (!data.count(v)) fail_name(Info(), "Variable " + v.s + " is used in a kernel in which it is not defined");
    Stmts out;
    for (auto& kv : data) {
      auto a = std::make_shared<Stmt>();
      a->k = Stmt::Alloc;
      a->id = kv.second.id;
      a->ty = kv.second.elem;
      a->iv = kv.second.size;
      out.push_back(a);
    }
    for (auto& s : replace_temps(body, data)) out.push_back(s);
    for (auto& kv : data) {
      auto f = std::make_shared<Stmt>();
      f->k = Stmt::Free;
      f->id = kv.second.id;
      out.push_back(f);
    }
    return out;
  }

  // ---- 8. every kernel gets its own loop variables and locals (inter_block.rs:763-793)
  Stmts rename_defs(const Stmts& ss, std::map<Name, Name>& m, std::set<Name>& seen) {
    Stmts out;
    for (auto& s : ss) {
      auto r = clone(s);
      if (s->k == Stmt::For || s->k == Stmt::Def) {
        if (seen.count(s->id)) {
          Name n = gen.fresh(s->id.s);
          m[s->id] = n;
        } else {
          seen.insert(s->id);
          m.erase(s->id);
        }
      }
      auto ren = [&](const E& e) { return rename_expr(e, m); };
      if (s->k == Stmt::For) {
        // bounds are evaluated outside the scope of the new loop variable
        auto saved = m.find(s->id) != m.end() ? std::optional<Name>(m[s->id]) : std::nullopt;
        m.erase(s->id);
        r->lo = ren(s->lo);
        r->hi = ren(s->hi);
        if (saved) m[s->id] = *saved;
      }
      if (r->dst) r->dst = ren(r->dst);
      if (r->expr) r->expr = ren(r->expr);
      for (auto& a : r->args) a = ren(a);
      if ((s->k == Stmt::For || s->k == Stmt::Def) && m.count(s->id)) r->id = m[s->id];
      r->body = rename_defs(s->body, m, seen);
      r->els = rename_defs(s->els, m, seen);
      out.push_back(r);
    }
    return out;
  }

 public:
  Stmts run(const Stmts& body0, const std::vector<Param>& params) {
    Stmts body = insert_sync(body0);
    body = classify(body);
    body = split_reductions(body);
    body = hoist(body);
    body = split_sync(body);
    body = drop_syncs(body, false, false);
    body = allocate_temporaries(body, params);
    std::map<Name, Name> m;
    std::set<Name> seen;
    body = rename_defs(body, m, seen);
    return body;
  }
};

// ================================================================ grid mapping
struct ParLayer { int64_t threads = 0, tpb = DEFAULT_TPB; };

struct GridMapper {
  // src/gpu/par.rs:105-154: the parallel loops at each depth below a kernel
  // root must agree on their thread counts
  static std::vector<ParLayer> unify(const std::vector<ParLayer>& a, const std::vector<ParLayer>& b, const Info& i) {
    if (a.empty()) return b;
    if (b.empty()) return a;
    if (a.size() != b.size()) fail_rt(i, "Found statements with inconsistent parallel structure (different nesting depth)");
    for (size_t k = 0; k < a.size(); ++k)
      if (a[k].threads != b[k].threads)
        fail_rt(i, "Found statements with inconsistent parallel structure: " + std::to_string(a[k].threads) + " != " +
                       std::to_string(b[k].threads) + " threads");
    std::vector<ParLayer> r = a;
    for (size_t k = 0; k < r.size(); ++k)
      if (r[k].tpb == DEFAULT_TPB) r[k].tpb = b[k].tpb;
    return r;
  }

  static std::vector<ParLayer> structure(const Stmts& ss) {
    std::vector<ParLayer> acc;
    for (auto& s : ss) {
      std::vector<ParLayer> p;
      if (s->k == Stmt::If) {
        auto t = structure(s->body), e = structure(s->els);
        if (!t.empty() && !e.empty()) p = unify(t, e, s->i);
        else p = t.empty() ? e : t;
      } else {
        p = structure(s->body);
        if (is_par_for(s)) {
          ParLayer l;
          l.threads = s->par.nthreads;
          l.tpb = s->par.tpb;
          p.insert(p.begin(), l);
        }
      }
      acc = unify(acc, p, s->i);
    }
    return acc;
  }

  struct Mapping { Dim3 blocks, threads; std::vector<GpuMap> maps; int64_t tpb; };

  static Mapping map_root(const S& root) {
    std::vector<ParLayer> layers = structure(root->body);
    ParLayer l0;
    l0.threads = root->par.nthreads;
    l0.tpb = root->par.tpb;
    layers.insert(layers.begin(), l0);
    int64_t tpb = DEFAULT_TPB;
    for (auto& l : layers) {
      if (tpb == DEFAULT_TPB || tpb == l.tpb) tpb = l.tpb;
      else if (l.tpb != DEFAULT_TPB)
        fail_rt(root->i, "Found inconsistent number of threads per block: " + std::to_string(tpb) + " != " + std::to_string(l.tpb));
    }
    // whole wavefronts on the innermost level, or cross-lane reductions misbehave
    layers.back().threads = (layers.back().threads + WAVE_SIZE - 1) / WAVE_SIZE * WAVE_SIZE;
    Mapping m;
    m.tpb = tpb;
    m.maps.resize(layers.size());
    auto block_dim = [&](int d) -> int64_t& { return d == 0 ? m.blocks.x : d == 1 ? m.blocks.y : m.blocks.z; };
    for (size_t k = layers.size(); k-- > 0;) {
      int64_t n = layers[k].threads;
      GpuMap g;
      if (k + 1 == layers.size()) {
        if (n > tpb) {
          g.k = GpuMap::ThreadBlock;
          g.dim = 0;
          g.n = n;
          g.tpb = tpb;
          m.blocks.x = (n + tpb - 1) / tpb;
          m.threads.x = tpb;
        } else {
          g.k = GpuMap::Thread;
          g.dim = 0;
          g.n = n;
          m.threads.x = n;
        }
      } else {
        int d = n > MAX_GRID_YZ ? 0 : m.blocks.y == 1 ? 1 : m.blocks.z == 1 ? 2 : 0;
        g.k = GpuMap::Block;
        g.dim = d;
        g.n = n;
        g.mult = block_dim(d);
        block_dim(d) *= n;
      }
      m.maps[k] = g;
    }
    return m;
  }
};

// ================================================================ kernel generation
struct KernelGen {
  const Options& opts;
  NameGen& gen;
  ElemSize isz;
  GridMapper::Mapping map;
  int seq_loop_depth = 0;

  KernelGen(const Options& o, NameGen& g) : opts(o), gen(g), isz(o.int_size()) {}

  // ---- reduction lowering (wave64): strided partials, cross-lane reduce,
  // one LDS slot per wavefront, second cross-lane pass over the partials
  Stmts expand_reduction(const S& loop, const GpuMap& gm, const S* prev) {
    if (gm.k != GpuMap::Thread)
      fail_rt(loop->i, "Parallel reductions must be performed within one thread block (internal error)");
    E lhs, rhs;
    BinOp op;
    ElemSize sz;
    Restructure::extract_reduction(loop, &lhs, &op, &rhs, &sz);
    Type ty = Type::scalar(sz);
    Name t = gen.fresh("t");
    E tv = mk_var(t, ty);
    Stmts out;
    out.push_back(mk_def(t, ty, neutral_element(op, sz, loop->i), loop->i));
    auto l = clone(loop);
    l->map = gm;
    l->par.reduction = false;
    l->body = {mk_assign(tv, mk_binop(op, tv, rhs, ty, loop->i), loop->i)};
    out.push_back(l);
    auto wr = std::make_shared<Stmt>();
    wr->k = Stmt::WaveReduce;
    wr->id = t;
    wr->ty = ty;
    wr->bop = op;
    wr->iv = gm.n;  // threads taking part (a multiple of the wavefront size)
    wr->i = loop->i;
    wr->unroll = seq_loop_depth > 0;  // the LDS slots are reused when the site sits in a sequential loop
    out.push_back(wr);
    // `x = neutral` directly before the loop followed by `x = x op t` is `x = t`
    bool init_before = prev && (*prev)->k == Stmt::Assign && expr_eq((*prev)->dst, lhs) &&
                       expr_eq(fold_expr((*prev)->expr), neutral_element(op, sz, loop->i));
    if (init_before) out.push_back(mk_assign(lhs, tv, loop->i));
    else out.push_back(mk_assign(lhs, mk_binop(op, lhs, tv, ty, loop->i), loop->i));
    return out;
  }

  Stmts gen_stmts(const Stmts& ss, size_t depth) {
    Stmts out;
    for (size_t k = 0; k < ss.size(); ++k) {
      const S& s = ss[k];
      switch (s->k) {
        case Stmt::SyncPoint:
          if (s->sync != SyncKind::BlockLocal)
            fail_rt(s->i, "Found an inter-block synchronization point remaining in parallel code after the inter-block "
                          "transformation. This is likely caused by a bug in the compiler.");
          out.push_back(mk_sync());
          break;
        case Stmt::For: {
          if (s->par.is_parallel()) {
            if (depth >= map.maps.size()) fail_rt(s->i, "Parallel nesting deeper than the mapped grid (internal error)");
            const GpuMap& gm = map.maps[depth];
            if (s->par.reduction) {
              bool fused = false;
              const S* prev = nullptr;
              if (!out.empty() && out.back()->k == Stmt::Assign) prev = &out.back();
              Stmts red = expand_reduction(s, gm, prev);
              // the initialisation is subsumed when the update was rewritten to a plain store
              if (prev && red.back()->expr->k == Expr::Var) { out.pop_back(); fused = true; }
              (void)fused;
              for (auto& r : red) out.push_back(r);
            } else {
              auto r = clone(s);
              r->map = gm;
              r->body = gen_stmts(s->body, depth + 1);
              out.push_back(r);
            }
          } else {
            auto r = clone(s);
            ++seq_loop_depth;
            r->body = gen_stmts(s->body, depth);
            --seq_loop_depth;
            out.push_back(r);
          }
          break;
        }
        case Stmt::While: {
          auto r = clone(s);
          ++seq_loop_depth;
          r->body = gen_stmts(s->body, depth);
          --seq_loop_depth;
          out.push_back(r);
          break;
        }
        case Stmt::If: {
          auto r = clone(s);
          r->body = gen_stmts(s->body, depth);
          r->els = gen_stmts(s->els, depth);
          out.push_back(r);
          break;
        }
        case Stmt::Alloc: fail_rt(s->i, "Memory allocation is not supported in parallel code.");
        case Stmt::Free: fail_rt(s->i, "Memory deallocation is not supported in parallel code.");
        default:
          out.push_back(s);
      }
    }
    return out;
  }

  // ---- block-wide store hazard (src/gpu/global_mem.rs:102-205)
  static bool thread_mapped(const S& s) {
    return s->k == Stmt::For && (s->map.k == GpuMap::Thread || s->map.k == GpuMap::ThreadBlock);
  }

  static bool depends(const E& e, const std::set<Name>& vars) {
    bool d = false;
    visit_exprs(e, [&](const E& x) {
      if (x->k == Expr::ThreadIdx) d = true;
      if (x->k == Expr::Var && vars.count(x->name)) d = true;
    });
    return d;
  }

  static void thread_dependent_vars(const Stmts& ss, std::set<Name>& vars, bool& changed) {
    for (auto& s : ss) {
      if (thread_mapped(s) && !vars.count(s->id)) { vars.insert(s->id); changed = true; }
      if (s->k == Stmt::For && !thread_mapped(s) && (depends(s->lo, vars) || depends(s->hi, vars)) && !vars.count(s->id)) {
        vars.insert(s->id);
        changed = true;
      }
      if (s->k == Stmt::Def && depends(s->expr, vars) && !vars.count(s->id)) { vars.insert(s->id); changed = true; }
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var && depends(s->expr, vars) && !vars.count(s->dst->name)) {
        vars.insert(s->dst->name);
        changed = true;
      }
      if (s->k == Stmt::WaveReduce) { /* result is uniform across the block */ }
      thread_dependent_vars(s->body, vars, changed);
      thread_dependent_vars(s->els, vars, changed);
    }
  }

  Stmts first_thread_stores(const Stmts& ss, const std::set<Name>& vars) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::Assign && s->dst->k == Expr::Index && !depends(s->dst->args[1], vars) &&
          !depends(s->dst->args[0], vars)) {
        Name t = gen.fresh("t");
        out.push_back(mk_def(t, s->dst->ty, s->expr, s->i));
        E cond = mk_binop(BinOp::Eq, thread_idx(0), mk_int(0, isz), Type::scalar(ElemSize::Bool));
        out.push_back(mk_if(cond, {mk_assign(s->dst, mk_var(t, s->dst->ty), s->i)}, {}, s->i));
        out.push_back(mk_sync());
        continue;
      }
      auto r = clone(s);
      r->body = first_thread_stores(s->body, vars);
      r->els = first_thread_stores(s->els, vars);
      out.push_back(r);
    }
    return out;
  }

  E thread_idx(int dim) {
    auto e = std::make_shared<Expr>();
    e->k = Expr::ThreadIdx;
    e->iv = dim;
    e->ty = Type::scalar(isz);
    return e;
  }

  // ---- src/gpu/sync_elim.rs:4-39: repeated synchronisations and a trailing one
  static Stmts sync_elim(const Stmts& ss, bool top) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::Sync && !out.empty() && out.back()->k == Stmt::Sync) continue;
      auto r = clone(s);
      r->body = sync_elim(s->body, false);
      r->els = sync_elim(s->els, false);
      out.push_back(r);
    }
    if (top)
      while (!out.empty() && out.back()->k == Stmt::Sync) out.pop_back();
    return out;
  }

  Kernel generate(const S& root, const std::string& fun_name) {
    map = GridMapper::map_root(root);
    Kernel k;
    k.name = fun_name + "_" + root->id.s + "_" + std::to_string(gen.next++);
    k.grid = map.blocks;
    k.block = map.threads;
    Stmts body = gen_stmts({root}, 0);
    std::set<Name> tvars;
    bool changed = true;
    while (changed) { changed = false; thread_dependent_vars(body, tvars, changed); }
    body = first_thread_stores(body, tvars);
    body = sync_elim(fold_stmts(body), true);
    // the root loop runs once per block when the grid covers its extent: a
    // synchronisation at the end of its body is then the end of the kernel
    if (body.size() == 1 && body[0]->k == Stmt::For && body[0]->lo->k == Expr::Int && body[0]->hi->k == Expr::Int) {
      const S& r = body[0];
      int64_t extent = r->step > 0 ? (r->hi->iv - r->lo->iv + r->step - 1) / r->step : (r->lo->iv - r->hi->iv - r->step - 1) / (-r->step);
      if (extent <= r->map.n && r->map.k == GpuMap::Block) {
        auto rr = clone(r);
        rr->body = sync_elim(r->body, true);
        body = {rr};
      }
    }
    k.body = body;
    return k;
  }
};

// ================================================================ host side
struct HostGen {
  const Options& opts;
  NameGen& gen;
  Program& prog;
  std::set<Name> host_scalars;   // names bound on the host (loop variables, scalar locals)
  std::map<Name, Type> host_vars;

  static void free_vars(const Stmts& ss, std::set<Name>& defined, std::vector<std::pair<Name, Type>>& fv, std::set<Name>& seen) {
    for (auto& s : ss) {
      auto use = [&](const E& e) {
        visit_exprs(e, [&](const E& x) {
          if (x->k == Expr::Var && !defined.count(x->name) && !seen.count(x->name)) {
            seen.insert(x->name);
            fv.emplace_back(x->name, x->ty);
          }
        });
      };
      use(s->lo); use(s->hi);
      if (s->k == Stmt::Def || s->k == Stmt::For) defined.insert(s->id);
      use(s->dst); use(s->expr);
      for (auto& a : s->args) use(a);
      free_vars(s->body, defined, fv, seen);
      free_vars(s->els, defined, fv, seen);
    }
  }

  static bool touches_memory(const E& e) {
    bool m = false;
    visit_exprs(e, [&](const E& x) { if (x->k == Expr::Index) m = true; });
    return m;
  }

  Stmts run(const Stmts& ss) {
    Stmts out;
    for (auto& s : ss) {
      if (is_par_for(s)) {
        KernelGen kg(opts, gen);
        Kernel k = kg.generate(s, prog.name);
        std::set<Name> defined, seen;
        std::vector<std::pair<Name, Type>> fv;
        free_vars(k.body, defined, fv, seen);
        auto l = std::make_shared<Stmt>();
        l->k = Stmt::Launch;
        l->fname = k.name;
        l->grid = k.grid;
        l->block = k.block;
        l->i = s->i;
        for (auto& v : fv) {
          KernelParam p;
          p.id = v.first;
          p.ty = v.second.is_array() ? Type::pointer(v.second.sz) : v.second;
          k.params.push_back(p);
          l->args.push_back(mk_var(v.first, v.second));
        }
        prog.kernels.push_back(k);
        out.push_back(l);
        continue;
      }
      switch (s->k) {
        case Stmt::For: case Stmt::While: case Stmt::If: {
          if (s->k != Stmt::If && !contains_par(s->body))
            fail_rt(s->i, "Loops outside parallel code must contain parallel code");
          if (s->expr && touches_memory(s->expr)) fail_rt(s->i, "Array accesses are not allowed outside parallel code");
          if (s->lo && (touches_memory(s->lo) || touches_memory(s->hi)))
            fail_rt(s->i, "Array accesses are not allowed outside parallel code");
          auto r = clone(s);
          r->body = run(s->body);
          r->els = run(s->els);
          out.push_back(r);
          break;
        }
        case Stmt::Def:
          if (touches_memory(s->expr)) fail_rt(s->i, "Assignments are not allowed outside parallel code");
          out.push_back(s);
          break;
        case Stmt::Assign:
          if (s->dst->k != Expr::Var || touches_memory(s->expr))
            fail_rt(s->i, "Assignments are not allowed outside parallel code");
          out.push_back(s);
          break;
        case Stmt::SyncPoint: break;
        default: out.push_back(s);
      }
    }
    return out;
  }
};

}  // namespace

Program gpu_codegen(const FunDef& f, const Options& opts, NameGen& gen) {
  Program prog;
  prog.name = f.id.s;
  prog.entry_params = f.params;
  prog.includes = opts.includes;
  for (auto& d : f.device_funs) prog.device_funs.push_back(*d);
  Restructure rs(opts, gen);
  Stmts body = rs.run(f.body, f.params);
  HostGen hg{opts, gen, prog, {}, {}};
  prog.host = hg.run(body);
  return prog;
}

}  // namespace parpy
