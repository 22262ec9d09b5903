// Lowering of the typed tree to the loop-level IR the GPU passes consume:
// N-d subscripts become row-major flat indices in the default integer type,
// labels become a LoopPar on each loop, `with gpu` becomes a one-iteration
// loop on one thread unless it is already inside parallel code.
//
// Counterpart of the reference's src/ir/from_py_ast.rs:176-214,283-297
// (indexing), :342-386 (labels -> LoopPar), :402-413 (GPU context) and
// src/ir/eliminate_gpu_context.rs:5-30.
#include <functional>

#include "passes.hpp"

namespace parpy {

namespace {

struct Lowerer {
  const Options& opts;
  NameGen& gen;

  E lower_expr(const E& e) {
    if (!e) return e;
    if (e->k == Expr::Subscript) {
      E target = lower_expr(e->args[0]);
      const auto& idxs = e->args[1]->args;
      const auto& shape = e->args[0]->ty.shape;
      ElemSize isz = opts.int_size();
      Type ity = Type::scalar(isz);
      E flat;
      std::vector<E> dims;
      for (size_t d = 0; d < idxs.size(); ++d) {
        E x = lower_expr(idxs[d]);
        dims.push_back(x);
        if (!flat) flat = x;
        else flat = mk_binop(BinOp::Add, mk_binop(BinOp::Mul, flat, mk_int(shape[d], isz), ity), x, ity);
      }
      int64_t rest = 1;
      for (size_t d = idxs.size(); d < shape.size(); ++d) rest *= shape[d];
      bool partial = idxs.size() < shape.size();
      if (partial) flat = mk_binop(BinOp::Mul, flat, mk_int(rest, isz), ity);
      flat = fold_expr(flat);
      // (&b[o])[j] == b[o + j]
      E base = target;
      if (base->k == Expr::AddrOf) {
        flat = fold_expr(mk_binop(BinOp::Add, base->args[1], flat, ity));
        base = base->args[0];
        dims.clear();
      }
      auto r = std::make_shared<Expr>();
      r->k = partial ? Expr::AddrOf : Expr::Index;
      r->ty = e->ty;
      r->i = e->i;
      r->args = {base, flat};
      if (!partial && !dims.empty() && base->k == Expr::Var) {
        r->dim_idx = dims;
        r->dim_shape = shape;
      }
      return r;
    }
    return map_children(e, [&](const E& c) { return lower_expr(c); });
  }

  // An external declared with `parallelize=threads(n)` is executed by n threads of a workgroup
  // together (it indexes its data with threadIdx.x itself).  The statement that calls it becomes
  // a parallel layer of n threads, every one of which makes the call (src/gpu/par.rs:88-103);
  // the value is then stored by the statement proper, which the store-hazard pass limits to one thread.
  int64_t parallel_external_threads(const S& s) {
    if (s->k != Stmt::Assign && s->k != Stmt::Def) return 0;
    int64_t n = 0;
    visit_exprs(s->expr, [&](const E& x) {
      if (x->k != Expr::Call || !x->ext || x->ext->par_threads <= 0) return;
      if (n != 0 && n != x->ext->par_threads) fail_rt(s->i, "Found calls of externals with different numbers of threads in one statement");
      n = x->ext->par_threads;
    });
    return n;
  }

  S cooperative_call(const S& s, int64_t n) {
    if (s->k == Stmt::Def) fail_rt(s->i, "The result of an external that runs on several threads must be assigned to an array element");
    Stmts body;
    std::function<E(const E&)> pull = [&](const E& e) -> E {
      if (!e) return e;
      if (e->k == Expr::Call && e->ext && e->ext->par_threads > 0) {
        Name t = gen.fresh("ext_res");
        body.push_back(mk_def(t, e->ty, lower_expr(e), e->i));
        return mk_var(t, e->ty, e->i);
      }
      return map_children(e, pull);
    };
    E rhs = pull(s->expr);
    body.push_back(mk_assign(lower_expr(s->dst), lower_expr(rhs), s->i));
    LoopPar p;
    p.nthreads = n;
    return mk_for(gen.fresh("ext_lane"), mk_int(0, opts.int_size()), mk_int(n, opts.int_size()), 1, body, p, s->i);
  }

  LoopPar loop_par(const S& s) {
    LoopPar p;
    for (auto& l : s->labels) {
      LoopPar o;
      if (l == REDUCE_PAR_LABEL) o.reduction = true;
      else {
        auto it = opts.parallelize.find(l);
        if (it == opts.parallelize.end()) continue;
        o = it->second;
      }
      if (!p.try_merge(o))
        fail_rt(s->i, "The labels associated with this statement specify conflicting parallelism");
    }
    return p;
  }

  Stmts lower_stmts(const Stmts& ss, bool in_par) {
    Stmts out;
    for (auto& s : ss) {
      if (s->k == Stmt::WithGpu) {
        Stmts body = lower_stmts(s->body, true);
        if (in_par) {
          for (auto& b : body) out.push_back(b);
        } else {
          LoopPar p;
          p.nthreads = 1;
          Name v = gen.fresh("_gpu_context");
          out.push_back(mk_for(v, mk_int(0, opts.int_size()), mk_int(1, opts.int_size()), 1, body, p, s->i));
        }
        continue;
      }
      if (int64_t n = parallel_external_threads(s)) {
        out.push_back(cooperative_call(s, n));
        continue;
      }
      auto r = std::const_pointer_cast<Stmt>(std::static_pointer_cast<const Stmt>(map_exprs(s, [&](const E& e) { return lower_expr(e); })));
      bool par_here = in_par;
      if (s->k == Stmt::For) {
        r->par = loop_par(s);
        par_here = in_par || r->par.is_parallel();
      }
      r->body = lower_stmts(s->body, par_here);
      r->els = lower_stmts(s->els, par_here);
      out.push_back(r);
    }
    return out;
  }
};

}  // namespace

FunDef lower(const FunDef& f, const Options& opts, NameGen& gen) {
  Lowerer lw{opts, gen};
  FunDef out = f;
  out.body = fold_stmts(lw.lower_stmts(f.body, false));
  out.device_funs.clear();
  for (auto& d : f.device_funs) {
    auto c = std::make_shared<FunDef>(*d);
    c->body = fold_stmts(lw.lower_stmts(d->body, false));
    out.device_funs.push_back(c);
  }
  return out;
}

}  // namespace parpy
