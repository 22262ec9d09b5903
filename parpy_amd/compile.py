"""Build, cache, load and wrap compiled functions.

Counterpart of python/parpy/compile.py of the reference.  What changes: the
generated code is device-only HIP C++ compiled in-process by hiprtc (through
the runtime library) instead of a host+device translation unit compiled by an
nvcc subprocess, and the object that is loaded is a code object plus a launch
plan instead of a shared library.  What stays: the on-disk cache keyed by the
sha256 of the generated code and flags (python/parpy/compile.py:4-12,108-115),
the error text of a failed build (:17-27), dict arguments expanded sorted by
key (:142-146) and a non-zero status turned into RuntimeError with the runtime's
message (:172-182).
"""
import ctypes
import os
from pathlib import Path

cache_path = Path(os.environ.get("PARPY_CACHE_DIR", f"{os.path.expanduser('~')}/.cache/parpy_amd"))
cache_path.mkdir(parents=True, exist_ok=True)

# code generation flags for every generated kernel: no packed fp32 instructions
HIPRTC_FLAGS = ["-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

_modules = {}   # key -> (module handle, code bytes) kept alive for the process lifetime


def _get_code_path(key):
    return cache_path / f"{key}.hsaco"


def _is_cached(key):
    return os.path.isfile(_get_code_path(key))


_pinned = set()  # keys of modules behind callables handed to the user (compile_string): never unloaded
_plans = []     # (runtime library, plan handle) of every launch plan created, released by clear_cache


def clear_cache():
    """Remove every cached code object; release the launch plans (with the device temporaries they
    keep) and the loaded modules once the device has finished what was enqueued."""
    import shutil
    shutil.rmtree(f"{cache_path}", ignore_errors=True)
    cache_path.mkdir(parents=True, exist_ok=True)
    if _plans or _modules:
        lib = _plans[0][0] if _plans else None
        if lib is None:
            from .runtime import load_hip_runtime_lib
            lib = load_hip_runtime_lib()
        if _plans:
            lib.parpy_sync()
        for l, plan in _plans:
            l.parpy_hip_plan_destroy(plan)
        for key, (module, _) in _modules.items():
            if key not in _pinned:
                lib.parpy_hip_module_unload(module)
    _plans.clear()
    for key in [k for k in _modules if k not in _pinned]:
        del _modules[key]


def hiprtc_compile(source, opts, lib=None):
    """Compile device source to a gfx950 code object (bytes).  Needs no GPU."""
    from .runtime import load_hip_runtime_lib
    lib = lib or load_hip_runtime_lib()
    flags = list(HIPRTC_FLAGS) + [f"-I{inc}" for inc in opts.includes] + list(opts.extra_flags)
    cflags = (ctypes.c_char_p * len(flags))(*[f.encode() for f in flags])
    code = ctypes.c_void_p()
    size = ctypes.c_size_t()
    rc = lib.parpy_hip_compile(source.encode("utf-8"), cflags, len(flags), ctypes.byref(code), ctypes.byref(size))
    if rc != 0:
        msg = lib.parpy_get_error_message().decode("utf-8", "replace")
        msg = f"Compilation of generated HIP code failed with exit code {rc}:\n{msg}"
        if opts.write_output:
            import uuid
            temp_file = f"{uuid.uuid4().hex}.hip"
            with open(temp_file, "w+") as f:
                f.write(source)
            msg += f"\nWrote generated code to file {temp_file}."
        raise RuntimeError(msg)
    data = ctypes.string_at(code.value, size.value)
    lib.parpy_hip_free_code(code)
    return data


def build_code_object(key, source, opts):
    """Compile `source` unless a code object for `key` is already cached on disk."""
    from .options import CompileBackend
    if opts.backend != CompileBackend.Hip:
        raise RuntimeError(f"Cannot build for unsupported backend {opts.backend}")
    path = _get_code_path(key)
    if not _is_cached(key):
        data = hiprtc_compile(source, opts)
        tmp = path.with_suffix(f".tmp{os.getpid()}")
        with open(tmp, "wb") as f:
            f.write(data)
        os.replace(tmp, path)
    if opts.write_output:
        with open(cache_path / f"{key}.hip", "w") as f:
            f.write(source)
    return path


def _load_module(key, lib):
    if key not in _modules:
        with open(_get_code_path(key), "rb") as f:
            data = f.read()
        buf = ctypes.create_string_buffer(data, len(data))
        module = ctypes.c_void_p()
        rc = lib.parpy_hip_module_load(buf, len(data), ctypes.byref(module))
        if rc != 0:
            raise RuntimeError(lib.parpy_get_error_message().decode("ascii", "replace"))
        _modules[key] = (module, buf)
    return _modules[key][0]


def _expand_arg(arg):
    if isinstance(arg, dict):
        return [v for (_, v) in sorted(arg.items())]
    return [arg]


def get_wrapper(name, key, plan_text, opts):
    """Callable that runs the launch plan of a compiled function on its (validated) arguments."""
    from .buffer import Buffer
    from .runtime import _compile_runtime_lib
    lib = _compile_runtime_lib(opts.backend)
    module = _load_module(key, lib)
    plan = ctypes.c_void_p()
    rc = lib.parpy_hip_plan_create(module, plan_text.encode("utf-8"), ctypes.byref(plan))
    if rc != 0:
        raise RuntimeError(lib.parpy_get_error_message().decode("ascii", "replace"))

    _plans.append((lib, plan))
    if opts.use_cuda_graphs:
        lib.parpy_hip_plan_set_graph(plan, 1)

    def wrapper(*args):
        flat = [x for a in args for x in _expand_arg(a)]
        # scalars and 0-d buffers were folded into the code; what is passed are array pointers
        ptrs = [a._get_ptr() for a in flat if isinstance(a, Buffer) and len(a.shape) > 0]
        arr = (ctypes.c_void_p * max(1, len(ptrs)))(*ptrs)
        status = lib.parpy_hip_plan_run(plan, arr, len(ptrs))
        if status != 0:
            msg = lib.parpy_get_error_message()
            raise RuntimeError(f"{msg.decode('ascii', 'replace')}")
    def timed(*args):
        """Run once and return the device time in ms between the first and the last launch."""
        flat = [x for a in args for x in _expand_arg(a)]
        ptrs = [a._get_ptr() for a in flat if isinstance(a, Buffer) and len(a.shape) > 0]
        arr = (ctypes.c_void_p * max(1, len(ptrs)))(*ptrs)
        ms = ctypes.c_float()
        status = lib.parpy_hip_plan_run_timed(plan, arr, len(ptrs), ctypes.byref(ms))
        if status != 0:
            raise RuntimeError(f"{lib.parpy_get_error_message().decode('ascii', 'replace')}")
        return ms.value

    def run_pointers(ptrs):
        """Run on device pointers that were validated before (same order as `wrapper` derives them)."""
        arr = (ctypes.c_void_p * max(1, len(ptrs)))(*ptrs)
        if lib.parpy_hip_plan_run(plan, arr, len(ptrs)) != 0:
            raise RuntimeError(f"{lib.parpy_get_error_message().decode('ascii', 'replace')}")

    def run_noalloc(ptrs):
        """As `run_pointers`, through the entry point that allocates nothing: the plan's temporaries
        come out of the runtime library's fixed scratch array (parpy_hip_plan_run_noalloc)."""
        arr = (ctypes.c_void_p * max(1, len(ptrs)))(*ptrs)
        if lib.parpy_hip_plan_run_noalloc(plan, arr, len(ptrs)) != 0:
            raise RuntimeError(f"{lib.parpy_get_error_message().decode('ascii', 'replace')}")

    wrapper.__name__ = name
    wrapper.run_pointers = run_pointers
    wrapper.run_noalloc = run_noalloc
    wrapper.timed = timed
    wrapper.plan = plan
    wrapper.launch_count = lambda: lib.parpy_hip_plan_launch_count(plan)
    wrapper.graph_replays = lambda: lib.parpy_hip_plan_graph_replays(plan)
    wrapper.persistent_launches = lambda: lib.parpy_hip_plan_persistent_launches(plan)
    return wrapper


def get_string_wrapper(kernel_name, key, grid, block, opts):
    """Wrapper for parpy.compile_string: one hand-written kernel launched with a fixed grid."""
    from .buffer import Buffer
    from .options import ScalarSizes
    from .runtime import _compile_runtime_lib
    lib = _compile_runtime_lib(opts.backend)
    module = _load_module(key, lib)
    _pinned.add(key)
    sizes = ScalarSizes(opts)
    g = (ctypes.c_int64 * 3)(*grid)
    b = (ctypes.c_int64 * 3)(*block)

    def wrapper(*args):
        flat = [x for a in args for x in _expand_arg(a)]
        storage = []
        for a in flat:
            if isinstance(a, bool):
                storage.append(ctypes.c_bool(a))
            elif isinstance(a, int):
                storage.append(sizes.int.to_ctype()(a))
            elif isinstance(a, float):
                storage.append(sizes.float.to_ctype()(a))
            elif isinstance(a, Buffer):
                if len(a.shape) == 0:
                    storage.append(a.dtype.to_ctype()(a.numpy().item()))
                else:
                    storage.append(ctypes.c_void_p(a._get_ptr()))
            else:
                raise RuntimeError(f"Argument {a} has unsupported type {type(a)}")
        ptrs = (ctypes.c_void_p * max(1, len(storage)))(*[ctypes.cast(ctypes.pointer(s), ctypes.c_void_p) for s in storage])
        status = lib.parpy_hip_launch(module, kernel_name.encode(), ctypes.byref(g), ctypes.byref(b), 0, ptrs)
        if status != 0:
            raise RuntimeError(lib.parpy_get_error_message().decode("ascii", "replace"))
    wrapper.__name__ = kernel_name
    return wrapper
