// gfx950 memory passes, host loops of launches that also exist as one kernel.
#include <algorithm>
#include <functional>

#include "hipopt_pass.hpp"

namespace parpy {
namespace hipopt {

namespace {

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

void persistent_loops(Program& p, const Options& opts, NameGen& gen) { PersistentLoops(p, opts, gen).run(); }

}  // namespace hipopt
}  // namespace parpy
