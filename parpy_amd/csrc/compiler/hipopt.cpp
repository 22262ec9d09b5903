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
// results with and without them).  This file holds the order in which they
// run; the passes themselves are methods of `hipopt::Pass` (hipopt_pass.hpp),
// defined by concern in hipopt_control.cpp (constants, short loops, guards,
// branches, aliases), hipopt_prefetch.cpp, hipopt_lds.cpp, hipopt_vector.cpp,
// hipopt_regs.cpp (budget, hoisting, register caching), hipopt_keep.cpp and
// hipopt_alias.cpp; the whole-program rewrites are in hipopt_launch.cpp and
// hipopt_persist.cpp.
#include "hipopt_pass.hpp"

namespace parpy {

void hip_optimize(Program& p, const Options& opts, NameGen& gen) {
  if (opts.opt_gather_transpose) hipopt::gather_transpose(p, opts, gen);
  if (opts.opt_lane_split && !opts.opt_mfma_sddmm) hipopt::lane_split(p, opts, gen);
  if (opts.opt_vectorize) hipopt::coarsen(p, opts, gen);
  for (auto& k : p.kernels) {
    if (k.opaque_body) { k.aligned_params = opts.assume_aligned; continue; }
    hipopt::Pass pass(k, opts, gen);
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
  if (opts.persistent_loops) hipopt::persistent_loops(p, opts, gen);
}

}  // namespace parpy
