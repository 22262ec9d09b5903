"""ctypes binding of the C++ compiler core (libparpy_hipc.so, include/parpy_hipc.h).

Offers the four entry points the reference's pyo3 module exposes to its
Python driver (src/lib.rs:120-127): python_to_ir, compile_ir, print_ast and
get_function_name.  Arguments and options cross the boundary as S-expression
text; errors come back as (kind, message, source span) and are re-raised as
RuntimeError / TypeError / NameError with the offending source lines attached,
like the reference does (src/utils/err.rs:79-87, src/utils/info.rs:90-121).
"""
import concurrent.futures
import ctypes
import linecache
import os
import pathlib
import subprocess
import tempfile

from . import _buildstamp, frontend
from .options import CompileBackend, LoopPar, ElemSize

CSRC = pathlib.Path(__file__).parent / "csrc" / "compiler"
LIB_PATH = pathlib.Path(__file__).parent / "libparpy_hipc.so"
SOURCES = ["ast.cpp", "front.cpp", "constfold.cpp", "specialize.cpp", "lower.cpp",
           "gpu.cpp", "hipopt.cpp", "hipopt_util.cpp", "hipopt_control.cpp", "hipopt_prefetch.cpp", "hipopt_lds.cpp",
           "hipopt_vector.cpp", "hipopt_regs.cpp", "hipopt_keep.cpp", "hipopt_alias.cpp", "hipopt_launch.cpp",
           "hipopt_persist.cpp", "hipprint.cpp", "capi.cpp"]

_lib = None


def _deps():
    return [CSRC / s for s in SOURCES] + sorted(CSRC.glob("*.hpp")) + [pathlib.Path(__file__).parent.parent / "include" / "parpy_hipc.h"]


def _command():
    return ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-sign-compare"]


def build_library(force=False):
    """Compile the compiler core with g++ (no GPU toolchain needed)."""
    srcs = [CSRC / s for s in SOURCES]
    if not force and LIB_PATH.exists() and _buildstamp.is_current(LIB_PATH, _deps(), _command()):
        return LIB_PATH
    # one object per source file, compiled side by side, then one link
    with tempfile.TemporaryDirectory(prefix="parpy_hipc_") as tmp:
        def compile_one(src):
            obj = os.path.join(tmp, src.stem + ".o")
            cmd = [c for c in _command() if c != "-shared"] + ["-c", "-o", obj, str(src)]
            return obj, subprocess.run(cmd, capture_output=True, text=True)
        with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
            done = list(pool.map(compile_one, srcs))
        failed = [r for _, r in done if r.returncode != 0]
        if failed:
            raise RuntimeError("Compilation of the ParPy compiler core failed:\n" + "\n".join(r.stdout + r.stderr for r in failed))
        r = subprocess.run(_command() + ["-o", str(LIB_PATH)] + [o for o, _ in done], capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"Linking the ParPy compiler core failed:\n{r.stdout}\n{r.stderr}")
    _buildstamp.write_stamp(LIB_PATH, _deps(), _command())
    return LIB_PATH


def _load():
    global _lib
    if _lib is not None:
        return _lib
    # what is built is loaded; a library that does not match its sources (by content) is rebuilt first
    _buildstamp.ensure_current(LIB_PATH, _deps(), _command(), lambda: build_library(force=True))
    lib = ctypes.CDLL(str(LIB_PATH))
    vp, cp, i32 = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int32
    lib.parpy_hipc_parse.argtypes = [cp, ctypes.POINTER(cp), ctypes.POINTER(vp), i32, ctypes.POINTER(vp)]
    lib.parpy_hipc_parse.restype = i32
    lib.parpy_hipc_fun_free.argtypes = [vp]
    lib.parpy_hipc_fun_free.restype = None
    lib.parpy_hipc_fun_name.argtypes = [vp]
    lib.parpy_hipc_fun_name.restype = cp
    lib.parpy_hipc_fun_print.argtypes = [vp]
    lib.parpy_hipc_fun_print.restype = cp
    lib.parpy_hipc_compile.argtypes = [vp, cp, cp] + [ctypes.POINTER(vp)] * 4
    lib.parpy_hipc_compile.restype = i32
    lib.parpy_hipc_free_string.argtypes = [vp]
    lib.parpy_hipc_free_string.restype = None
    lib.parpy_hipc_last_error.argtypes = []
    lib.parpy_hipc_last_error.restype = cp
    lib.parpy_hipc_last_error_kind.argtypes = []
    lib.parpy_hipc_last_error_kind.restype = i32
    lib.parpy_hipc_last_error_span.argtypes = [ctypes.POINTER(i32 * 4)]
    lib.parpy_hipc_last_error_span.restype = None
    _lib = lib
    return lib


class IrAst:
    """Owner of a parsed function held by the compiler core (the reference's PyCapsule)."""

    def __init__(self, handle, filepath):
        self.handle = handle
        self.filepath = filepath

    def __del__(self):
        if self.handle and _lib is not None:
            _lib.parpy_hipc_fun_free(self.handle)
            self.handle = None


def _raise_last_error(lib, filepath):
    msg = lib.parpy_hipc_last_error().decode("utf-8", "replace")
    kind = lib.parpy_hipc_last_error_kind()
    span = (ctypes.c_int32 * 4)()
    lib.parpy_hipc_last_error_span(ctypes.byref(span))
    l0, c0, l1, c1 = list(span)
    if l0 > 0 and filepath:
        lines = [linecache.getline(filepath, n).rstrip("\n") for n in range(l0, max(l0, l1) + 1)]
        excerpt = "\n".join(f"{n:4d} | {t}" for n, t in zip(range(l0, l1 + 1), lines) if t)
        where = f"line {l0}" if l0 == l1 else f"lines {l0}-{l1}"
        msg = f"{msg}\n\nOn {where} of file {filepath}:\n{excerpt}"
    exc = {0: RuntimeError, 1: TypeError, 2: NameError}.get(kind, RuntimeError)
    raise exc(msg)


def python_to_ir(tree, info, tops, vars):
    """Parse a Python function (ast.Module) into the compiler's untyped IR."""
    lib = _load()
    try:
        text = frontend.to_sexpr(tree, info, tops, vars)
    except frontend.FrontendError as e:
        raise RuntimeError(str(e)) from None
    names = [n for n, t in tops.items() if isinstance(t, IrAst)]
    cnames = (ctypes.c_char_p * max(1, len(names)))(*[n.encode() for n in names])
    chandles = (ctypes.c_void_p * max(1, len(names)))(*[tops[n].handle for n in names])
    out = ctypes.c_void_p()
    rc = lib.parpy_hipc_parse(text.encode("utf-8"), cnames, chandles, len(names), ctypes.byref(out))
    if rc != 0:
        _raise_last_error(lib, info[0])
    return IrAst(out.value, info[0])


def declare_external(fn, ext_name, backend, header, parallelize, vars):
    """Parsed declaration of an external device function (the reference's parpy.declare_external)."""
    import ast as pyast
    import inspect
    import textwrap
    lib = _load()
    src, first = inspect.getsourcelines(fn)
    tree = pyast.parse(textwrap.dedent("".join(src)))
    filepath = inspect.getfile(fn)
    try:
        text = frontend.external_to_sexpr(tree, (filepath, first - 1, 0), vars, ext_name, header,
                                          {CompileBackend.Auto: 0, CompileBackend.Cuda: 1, CompileBackend.Metal: 2,
                                           CompileBackend.Hip: 3}[backend], parallelize.nthreads)
    except frontend.FrontendError as e:
        raise RuntimeError(str(e)) from None
    out = ctypes.c_void_p()
    cnames = (ctypes.c_char_p * 1)()
    chandles = (ctypes.c_void_p * 1)()
    rc = lib.parpy_hipc_parse(text.encode("utf-8"), cnames, chandles, 0, ctypes.byref(out))
    if rc != 0:
        _raise_last_error(lib, filepath)
    return IrAst(out.value, filepath)


def get_function_name(ir_ast):
    return _load().parpy_hipc_fun_name(ir_ast.handle).decode()


def print_ast(ir_ast):
    return _load().parpy_hipc_fun_print(ir_ast.handle).decode()


# ---------------------------------------------------------------- descriptors
def _quote(s):
    return '"' + s.replace("\\", "\\\\").replace('"', '\\"') + '"'


def _fmt_float(v):
    import math
    if math.isinf(v):
        return "inf" if v > 0 else "-inf"
    if math.isnan(v):
        return "nan"
    return repr(float(v))


def describe_arg(arg):
    """S-expression descriptor of one (validated) argument: kind, dtype, shape or value."""
    from .buffer import Buffer
    if isinstance(arg, bool):
        return f"(scalar bool {'true' if arg else 'false'})"
    if isinstance(arg, int):
        return f"(int {arg})"
    if isinstance(arg, float):
        return f"(float {_fmt_float(arg)})"
    if isinstance(arg, dict):
        fields = " ".join(f"({_quote(k)} {describe_arg(v)})" for k, v in sorted(arg.items()))
        return f"(dict {fields})"
    if isinstance(arg, Buffer):
        tag = arg.dtype.sz.value
        if len(arg.shape) == 0:
            v = arg.numpy().item()
            if arg.dtype.sz == ElemSize.Bool:
                return f"(scalar bool {'true' if v else 'false'})"
            if arg.dtype.is_floating_point():
                return f"(scalar {tag} {_fmt_float(float(v))})"
            return f"(scalar {tag} {int(v)})"
        return f"(tensor {tag} ({' '.join(str(int(d)) for d in arg.shape)}))"
    raise RuntimeError(f"Argument {arg} has unsupported type {type(arg)}")


def describe_opts(opts):
    par = []
    for label, p in sorted(opts.parallelize.items()):
        if not isinstance(p, LoopPar):
            raise TypeError(f"Parallelization of label {label} must be a LoopPar")
        par.append(f"({_quote(label)} {p.nthreads} {1 if p.reduction else 0} {p._tpb})")
    backend = {CompileBackend.Hip: "hip", CompileBackend.Cuda: "cuda", CompileBackend.Metal: "metal"}.get(opts.backend, "auto")
    parts = [f"(par {' '.join(par)})", f"(backend {backend})",
             f"(debug_print {1 if opts.debug_print else 0})",
             f"(use_graphs {1 if opts.use_cuda_graphs else 0})",
             f"(persistent_loops {1 if getattr(opts, 'persistent_loops', False) else 0})",
             f"(device_functions {1 if getattr(opts, 'device_functions', False) else 0})"]
    if opts.force_int_size is not None:
        parts.append(f"(force_int_size {opts.force_int_size.value})")
    if opts.force_float_size is not None:
        parts.append(f"(force_float_size {opts.force_float_size.value})")
    for name in ("opt_vectorize", "opt_lds_rows", "opt_reg_cache", "opt_hoist_invariant",
                 "opt_narrow_index", "opt_mfma_sddmm", "opt_unswitch", "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_unswitch_uniform", "opt_offset32", "opt_if_convert", "opt_noalias_scopes", "opt_expand_short_loops", "opt_guard_bounds", "opt_prefetch_steps", "opt_pack_accesses", "opt_share_iterations", "opt_fence_iterations", "opt_keep_stored", "opt_keep_own", "assume_aligned"):
        v = getattr(opts, name, None)
        if v is not None:
            parts.append(f"({name} {1 if v else 0})")
    if getattr(opts, "reg_budget", None):
        parts.append(f"(reg_budget {int(opts.reg_budget)})")
    if getattr(opts, "reg_budget_scale", None):
        parts.append(f"(reg_budget_scale {int(opts.reg_budget_scale)})")
    return f"(opts {' '.join(parts)})"


class Compiled:
    """Result of compile_ir: device source, launch plan and the readable listing."""

    def __init__(self, device_src, plan, listing, debug_log):
        self.device_src = device_src
        self.plan = plan
        self.listing = listing
        self.debug_log = debug_log


def compile_ir(ir_ast, args, opts, tops=None):
    """Specialise `ir_ast` on `args` and generate HIP code (src/lib.rs:72-118)."""
    if opts.backend not in (CompileBackend.Hip, CompileBackend.Auto):
        raise RuntimeError(f"Cannot generate code for unsupported backend {opts.backend}; "
                           "this build of the compiler targets CompileBackend.Hip only")
    if opts.use_cuda_thread_block_clusters:
        raise RuntimeError("Thread block clusters are a CUDA (sm_90) feature and are not available in the HIP backend")
    lib = _load()
    args_text = "(args " + " ".join(describe_arg(a) for a in args) + ")"
    outs = [ctypes.c_void_p() for _ in range(4)]
    rc = lib.parpy_hipc_compile(ir_ast.handle, args_text.encode(), describe_opts(opts).encode(),
                                *[ctypes.byref(o) for o in outs])
    if rc != 0:
        _raise_last_error(lib, ir_ast.filepath)
    texts = []
    for o in outs:
        texts.append(ctypes.string_at(o.value).decode() if o.value else "")
        if o.value:
            lib.parpy_hipc_free_string(o)
    res = Compiled(*texts)
    if opts.debug_print and res.debug_log:
        print(res.debug_log)
    return res
