// gfx950 memory code generation passes over the extracted kernels.
#include "passes.hpp"

namespace parpy {

namespace {

// A pointer parameter is read-only when nothing in the kernel stores through
// it, directly or through a local alias initialised from it.
void mark_read_only(Kernel& k) {
  std::set<Name> written;
  std::map<Name, std::set<Name>> alias_of;  // local pointer -> parameters it may point into
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
  // two sweeps so that aliases assigned after their first use inside loops are seen
  for (int sweep = 0; sweep < 2; ++sweep) {
    visit_stmts(k.body, [&](const S& s) {
      if (s->k == Stmt::Def && (s->ty.is_array() || s->ty.is_pointer())) bases(s->expr, alias_of[s->id]);
      if (s->k == Stmt::Assign && s->dst->k == Expr::Var && (s->dst->ty.is_array() || s->dst->ty.is_pointer()))
        bases(s->expr, alias_of[s->dst->name]);
      if (s->k == Stmt::Assign && s->dst->k == Expr::Index) bases(s->dst->args[0], written);
    });
  }
  for (auto& p : k.params) p.read_only = p.ty.is_pointer() && !written.count(p.id);
}

}  // namespace

void hip_optimize(Program& p, const Options& opts, NameGen& gen) {
  (void)opts;
  (void)gen;
  for (auto& k : p.kernels) mark_read_only(k);
}

}  // namespace parpy
