/*
 * C ABI of the ParPy compiler core for the HIP (gfx950) backend.
 *
 * This is the boundary the reference crosses through pyo3 (src/lib.rs:120-137):
 * the Python package hands over a serialised function at decoration time and
 * argument / option descriptors at call time and gets text back.  Everything
 * is passed as NUL-terminated S-expression strings; no Python or torch types
 * appear in the signatures.  The library does not touch the GPU.
 *
 * Threading: calls may come from any thread; error state is thread-local.
 * Ownership: strings returned through `char**` belong to the caller and are
 * released with parpy_hipc_free_string; handles with parpy_hipc_fun_free.
 */
#ifndef PARPY_HIPC_H
#define PARPY_HIPC_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct parpy_hipc_fun parpy_hipc_fun;

/* Replaces parpy.python_to_ir (src/lib.rs:18-36): parse one serialised
 * function, bind names, attach labels and inline statement calls to the
 * previously parsed functions given in (top_names, tops).  0 on success. */
int32_t parpy_hipc_parse(const char* sexpr, const char* const* top_names,
                         const parpy_hipc_fun* const* tops, int32_t ntops,
                         parpy_hipc_fun** out);

void parpy_hipc_fun_free(parpy_hipc_fun* f);

/* Replaces parpy.get_function_name (src/lib.rs:62-70). */
const char* parpy_hipc_fun_name(const parpy_hipc_fun* f);

/* Replaces parpy.print_ast (src/lib.rs:53-60); the text feeds the in-memory
 * cache key (python/parpy/key.py:32-37). */
const char* parpy_hipc_fun_print(const parpy_hipc_fun* f);

/* Replaces parpy.compile_ir (src/lib.rs:72-118) for the HIP backend:
 * specialise on `args`, lower, map to the wave64 grid and emit
 *   device_src : HIP C++ for hiprtc (--offload-arch=gfx950),
 *   plan       : host launch plan for parpy_hip_plan_create (parpy_hip.h),
 *   listing    : both in human-readable form (what print_compiled returns),
 *   debug_log  : per-pass dumps when the options enable debug_print (may be NULL).
 * Returns 0 on success; on failure see parpy_hipc_last_error*. */
int32_t parpy_hipc_compile(const parpy_hipc_fun* f, const char* args,
                           const char* opts, char** device_src, char** plan,
                           char** listing, char** debug_log);

void parpy_hipc_free_string(char* s);

/* Error of the last failed call on this thread: message, kind (0 runtime,
 * 1 type, 2 name; src/utils/err.rs:79-87) and source span
 * {first line, first column, last line, last column} (src/utils/info.rs). */
const char* parpy_hipc_last_error(void);
int32_t parpy_hipc_last_error_kind(void);
void parpy_hipc_last_error_span(int32_t* span4);

#ifdef __cplusplus
}
#endif
#endif
