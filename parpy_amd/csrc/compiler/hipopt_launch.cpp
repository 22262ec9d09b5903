// gfx950 memory passes, rewrites that change a launch: transposed staging of column gathers, lane groups, coarsened element-wise launches.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

namespace {

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

}  // namespace

void gather_transpose(Program& p, const Options& opts, NameGen& gen) { GatherTranspose(p, opts, gen).run(); }
void lane_split(Program& p, const Options& opts, NameGen& gen) { LaneSplit(p, opts, gen).run(); }
void coarsen(Program& p, const Options& opts, NameGen& gen) { Coarsen(p, opts, gen).run(); }

}  // namespace hipopt
}  // namespace parpy
