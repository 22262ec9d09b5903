/*
 * C ABI of the ParPy HIP runtime library (libparpy_hip.so) for MI355X (gfx950).
 *
 * First group: the seven runtime entry points of the reference's native
 * runtime, python/parpy/native/parpy_cuda.h:15-25 (bound from ctypes in
 * python/parpy/runtime.py:11-26), with identical names, argument meaning and
 * return conventions so that the reference's Python driver binds them
 * unchanged.
 *
 * Second group: what replaces the reference's "generate a host translation
 * unit, run nvcc, dlopen the result" step (python/parpy/compile.py:29-54,
 * 123-184): runtime compilation of the generated device source with hiprtc,
 * code-object loading, and execution of the generated launch plan with
 * hipModuleLaunchKernel.  parpy_hip_plan_run plays the role of the generated
 * `extern "C" int32_t <fun>(...)` entry point (src/gpu/codegen.rs:540-547):
 * same flattened pointer arguments, same 0 / non-zero status, message through
 * parpy_get_error_message.
 *
 * All work is enqueued on the null stream and is not synchronised before
 * returning (like the reference).  No torch or Python types appear here.
 * Threads: the error message is a per-thread buffer owned by the library;
 * runs of one launch plan from several host threads take turns, different
 * plans run side by side; nothing else is promised beyond what HIP gives.
 * Host-side integer expressions of a plan are evaluated in signed 64-bit
 * arithmetic (unsigned 64-bit values above 2^63 are not represented); a
 * division by zero there fails the run with a message.
 */
#ifndef PARPY_HIP_H
#define PARPY_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- reference runtime surface (python/parpy/native/parpy_cuda.h:15-25) ---- */
void parpy_init(int64_t unused);                                   /* parpy_cuda.cpp:3-5   */
int32_t parpy_sync(void);                                          /* parpy_cuda.cpp:7-9   */
void* parpy_alloc_buffer(int64_t nbytes);                          /* parpy_cuda.cpp:11-17; NULL on failure */
int32_t parpy_memcpy(void* dst, void* src, int64_t nbytes, int64_t kind); /* :19-31; kind 0 H2H, 1 H2D, 2 D2H, 3 D2D */
int32_t parpy_memset(void* ptr, int64_t nbytes, int8_t value);     /* parpy_cuda.cpp:33-35 */
int32_t parpy_free_buffer(void* ptr);                              /* parpy_cuda.cpp:37-39 */
const char* parpy_get_error_message(void);                         /* parpy_cuda.h:22-25   */

/* ---- runtime compilation and loading (replaces python/parpy/compile.py:29-54) ---- */

/* Compile HIP C++ `source` with hiprtc.  `options` are compiler flags; the
 * target architecture defaults to gfx950 when no --offload-arch is given.
 * On success *code / *size receive the code object (free it with
 * parpy_hip_free_code).  On failure the hiprtc log is the error message.
 * Does not need a GPU. */
int32_t parpy_hip_compile(const char* source, const char* const* options,
                          int32_t noptions, void** code, size_t* size);
void parpy_hip_free_code(void* code);

/* Load / unload a code object on the current device (hipModuleLoadData). */
int32_t parpy_hip_module_load(const void* code, size_t size, void** module);
int32_t parpy_hip_module_unload(void* module);

/* Launch one kernel of a loaded module on the null stream
 * (hipModuleLaunchKernel); `args` are pointers to the argument values. */
int32_t parpy_hip_launch(void* module, const char* kernel,
                         const int64_t grid[3], const int64_t block[3],
                         int64_t lds_bytes, void** args);

/* ---- launch plans (replaces the generated host entry point) ---- */

/* Build an executable plan from the text emitted by parpy_hipc_compile.
 * Kernel functions are resolved once, here. */
int32_t parpy_hip_plan_create(void* module, const char* plan_text, void** plan);

/* Run the plan: `args` are the flattened pointer arguments in call order
 * (dict fields sorted by key, python/parpy/compile.py:142-146); scalars were
 * folded into the code at compile time.  Returns 0 or non-zero.  A plan holds
 * the state of its host loops and its device temporaries: runs of one plan
 * from several host threads take turns (different plans run concurrently);
 * the error message is per thread.  Temporaries stay allocated between runs up
 * to 1 GiB per plan and 8 GiB over all plans of the process (beyond that they
 * are allocated and freed per run); a run that fails half way frees what it
 * had allocated for itself. */
int32_t parpy_hip_plan_run(void* plan, void* const* args, int32_t nargs);

/* Same as parpy_hip_plan_run, bracketed by HIP events recorded on the null
 * stream right before the first and after the last launch; waits for the
 * work to finish and returns the device time in milliseconds.  This is what
 * the reference's benchmarks do with CUDA events around a call
 * (benchmarks/common.py:76-89), without the Python overhead in between. */
int32_t parpy_hip_plan_run_timed(void* plan, void* const* args, int32_t nargs,
                                 float* elapsed_ms);

/* Graph replay for plans whose host side is a long loop of launches: the
 * analogue of the reference's use_cuda_graphs option (src/option.rs:60-63,
 * src/cuda/graphs.rs).  With it enabled the first run is eager (it allocates
 * the device temporaries), the second is captured into a HIP graph, and later
 * runs with the same pointer arguments are one hipGraphLaunch on the null
 * stream; other pointers trigger a new capture.  A plan that would have to
 * allocate during capture falls back to eager launches. */
int32_t parpy_hip_plan_set_graph(void* plan, int32_t enable);

/* Number of runs of this plan that were served by a graph replay so far
 * (0 for a plan that runs eagerly or that fell back). */
int64_t parpy_hip_plan_graph_replays(void* plan);

/* Loops of launches inside one kernel (the plan's `persist` statements, emitted with the
 * persistent_loops option): the counterpart of the reference's answer to launch-bound host loops
 * (src/option.rs:60-63, src/gpu/inter_block.rs:466-563 hoists such loops to the host).  The
 * kernel separates the steps by a barrier over all workgroups (or over those of one value of a grid
 * dimension each, when the steps keep those values apart: the statement names the number of such
 * groups, one counter each), so the runtime uses it only when the whole grid is resident at once (occupancy query when the plan is created) and runs the loop of
 * launches otherwise.  The barrier's wait is bounded (PARPY_HIP_BARRIER_POLLS polls, about two
 * seconds by default): a barrier that times out makes every workgroup leave the kernel, and the next
 * parpy_sync or parpy_hip_plan_run_timed returns non-zero with a message.  This returns the number
 * of runs of the plan that used such a kernel. */
int64_t parpy_hip_plan_persistent_launches(void* plan);

/* Number of kernel launches the last run of this plan enqueued. */
int64_t parpy_hip_plan_launch_count(void* plan);

int32_t parpy_hip_plan_destroy(void* plan);

/* ---- a run that allocates nothing ---- */

/* No counterpart in the reference (its generated entry points call
 * cudaMallocAsync for every temporary, src/cuda/codegen.rs:179-202).  For
 * callers that cannot allocate device memory: tight serving loops, code under
 * a HIP graph capture elsewhere in the process, harnesses that forbid
 * hipMalloc.  Same arguments, result and status as parpy_hip_plan_run, but the
 * plan's device temporaries (partial results of multi-block reductions, locals
 * that cross kernels, transposed operands) are carved out of one array of
 * PARPY_HIP_SCRATCH_BYTES that is part of the library's code object, and no
 * hipMalloc / hipFree or other allocating call is made.  A plan whose
 * temporaries need more fails with a message and runs nothing.  Launches are
 * eager on the null stream (graph replay and kept temporaries do not apply).
 * Every call on a GPU uses that GPU's one array and temporaries start with
 * whatever the previous call left there (the kernels write a temporary before
 * they read it, as with a fresh allocation); two calls that overlap on one
 * GPU -- from two host threads, or on work still in flight on another stream
 * -- race on it. */
#define PARPY_HIP_SCRATCH_BYTES (16u << 20)
int32_t parpy_hip_plan_run_noalloc(void* plan, void* const* args, int32_t nargs);

#ifdef __cplusplus
}
#endif
#endif
