// What the gfx950 memory passes share: helpers over the kernel IR and the per-kernel pass object.  The methods of
// `Pass` are defined by concern in hipopt_control.cpp, hipopt_prefetch.cpp, hipopt_lds.cpp, hipopt_vector.cpp,
// hipopt_regs.cpp, hipopt_keep.cpp and hipopt_alias.cpp; the rewrites that change a launch are in hipopt_launch.cpp
// and hipopt_persist.cpp; hipopt.cpp holds the order in which they run.
#pragma once
#include <algorithm>
#include <functional>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "passes.hpp"

namespace parpy {
namespace hipopt {

using StmtP = std::shared_ptr<Stmt>;
inline StmtP clone(const S& s) { return std::make_shared<Stmt>(*s); }

constexpr int64_t LDS_BUDGET_BYTES = 160 * 1024 - 4096;  // leave room for reduction slots

bool mentions(const E& e, const Name& v);                 // e reads variable v
bool has_load(const E& e);                                // e reads memory or a register array
bool affine_unit(const E& idx, const Name& d, E* rest);   // idx == rest + d with rest free of d
int64_t const_extent(const S& loop);                      // iterations of a loop with literal bounds, else -1
inline bool thread_mapped(const S& s) { return s->k == Stmt::For && s->map.k == GpuMap::Thread; }
int64_t per_thread_trips(const S& loop);                  // iterations every thread runs in a thread-mapped loop, when that is a compile-time constant
E counter_var(const S& loop, ElemSize isz);               // the per-thread iteration counter of a mapped loop as the printer names it
E subst_vars(const E& e, const std::map<Name, E>& m);

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

  struct ArrayInfo {
    bool ok = true;
    int64_t rowlen = 0;
    ElemSize sz = ElemSize::F32;
    bool in_seq_loop = false;
    bool written = false;
    bool accessed = false;
  };
  struct IterSpace {
    S outer;                 // thread-mapped loop
    S inner;                 // unrolled element loop, or null
    E slot;                  // per-thread iteration number (register array index)
    int64_t slots = 0;
    const Stmts* body = nullptr;  // innermost body
  };
  struct Hoisted { E load; Name reg; ElemSize sz; };
  struct AliasDef { Name a, b; E cond; bool ok = false; };
  struct Touched {
    std::set<Name> r, w;
    bool any = false;
  };
  using AliasCfg = std::map<Name, Name>;

  // hipopt_control.cpp: control flow inside a kernel: constants, short loops, guards, uniform and value-picking branches, array aliases
  std::set<Name> param_names() const;
  struct Unswitch;
  static bool straight_line(const Stmts& ss);
  Stmts propagate_constants(const Stmts& ss);
  static size_t count_stmts(const Stmts& ss);
  Stmts expand_short_loops(const Stmts& ss0, bool in_par);
  static E strip_converts(const E& e);
  Stmts guards_to_bounds(const Stmts& ss);
  Stmts hoist_uniform_conditions(const Stmts& ss);
  Stmts if_convert(const Stmts& ss);
  Stmts if_convert(const Stmts& ss, const std::set<Name>& nonzero_const);
  void unswitch_aliases();

  // hipopt_prefetch.cpp: loads issued a step ahead of their use
  Stmts prefetch_counter_loads(const Stmts& ss, RangeEnv env);
  Stmts prefetch_selected_rows(const Stmts& ss, int64_t* budget);

  // hipopt_lds.cpp: rows that live in LDS for a whole kernel, and the barriers between regions that share nothing
  void lds_rows();
  void touched(const Stmts& ss, const std::set<Name>& arrays, Touched& t);
  Stmts drop_barriers_in(const Stmts& ss, const std::set<Name>& arrays);
  void drop_barriers();

  // hipopt_vector.cpp: several consecutive elements per thread; MFMA dot products
  int vector_width(const S& loop);
  static int64_t strided_run(const E& idx, const Name& d);
  Stmts vectorize(const Stmts& ss);
  Stmts mfma_dot(const Stmts& ss);

  // hipopt_regs.cpp: values kept in registers: the register budget, loads hoisted out of sequential loops, sections cached between loops
  bool iter_space(const S& loop, IterSpace* is);
  std::set<Name> written_arrays();
  int64_t reg_budget() const;
  bool step_has_transcendentals() const;
  Stmts hoist_from_seq_loop(const S& seq, int64_t* budget);
  Stmts hoist_invariant(const Stmts& ss, int64_t* budget, bool in_seq);
  struct OwnIterations;
  bool distinct_names(const Name& a, const Name& b) const;
  Stmts share_own_iterations(const Stmts& ss);
  void reg_cache(int64_t* budget);

  // hipopt_keep.cpp: values a thread stored in a step and reads back itself
  static AliasDef alias_definition(const Stmts& ss, size_t upto, const Name& name);
  static bool scaled_index(const E& idx, const Name& var, int64_t* V, int64_t* c);
  Stmts keep_stored_rows(const Stmts& ss, int64_t* budget);
  static bool alternates(const E& cond, const S& loop);
  Stmts carry_across_iterations(const Stmts& B, size_t p1, const S& L1, const IterSpace& is1, const S& seq_loop, const AliasDef& dx,
                                int64_t V, const std::map<int64_t, size_t>& store_at, const Name& reg, ElemSize sz, Stmts* pre);
  std::set<Name> lds_array_names() const;
  Stmts keep_in_iteration(const Stmts& B, int64_t* budget, const S& seq_loop, Stmts* pre);

  // hipopt_alias.cpp: what the target compiler may assume about pointers: distinct arrays, read-only parameters
  static bool is_alias_type(const Type& t);
  static bool alias_target(const E& e, const AliasCfg& cfg, Name* out);
  static bool apply_alias_stmt(const S& st, std::vector<AliasCfg>& cfgs, std::vector<Name>& order);
  Stmts noalias_scopes(const Stmts& ss, bool wrap);
  void mark_read_only();
};

// ---- rewrites of the whole program (they change a launch)
void gather_transpose(Program& p, const Options& opts, NameGen& gen);   // hipopt_launch.cpp
void lane_split(Program& p, const Options& opts, NameGen& gen);         // hipopt_launch.cpp
void coarsen(Program& p, const Options& opts, NameGen& gen);            // hipopt_launch.cpp
void persistent_loops(Program& p, const Options& opts, NameGen& gen);   // hipopt_persist.cpp

}  // namespace hipopt
}  // namespace parpy
