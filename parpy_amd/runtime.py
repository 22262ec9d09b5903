"""Loader of the native HIP runtime library (libparpy_hip.so, include/parpy_hip.h).

Counterpart of python/parpy/runtime.py:11-98 of the reference: declares the
ctypes signatures of the seven runtime exports plus the hiprtc / module /
launch-plan entry points.  The library is built ahead of time by
`__graft_entry__.build()`; loading it compiles nothing when the built file
matches its sources.
"""
import ctypes
import os
import pathlib
import subprocess

from . import _buildstamp
from .options import CompileBackend

PARPY_NATIVE_PATH = pathlib.Path(__file__).parent / "csrc" / "runtime"
PARPY_HIP_BASE_LIB_PATH = pathlib.Path(__file__).parent / "libparpy_hip.so"
HIPCC_FLAGS = ["-O2", "-fPIC", "-shared", "-std=c++17", "--offload-arch=gfx950",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

libs = {}


def _runtime_deps():
    return [PARPY_NATIVE_PATH / "parpy_hip.cpp", pathlib.Path(__file__).parent / "csrc" / "compiler" / "sexpr.hpp",
            pathlib.Path(__file__).parent.parent / "include" / "parpy_hip.h"]


def build_library(force=False):
    """Compile csrc/runtime/parpy_hip.cpp with hipcc for gfx950 (host code plus the device scratch array;
    cross-compiles without a GPU)."""
    src = PARPY_NATIVE_PATH / "parpy_hip.cpp"
    deps = _runtime_deps()
    lib = PARPY_HIP_BASE_LIB_PATH
    if not force and lib.exists() and _buildstamp.is_current(lib, deps, HIPCC_FLAGS):
        return lib
    cmd = ["hipcc"] + HIPCC_FLAGS + ["-o", str(lib), str(src), "-lhiprtc"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"Compilation of the HIP runtime library failed.\nstdout:\n{r.stdout}\nstderr:\n{r.stderr}")
    _buildstamp.write_stamp(lib, deps, HIPCC_FLAGS)
    return lib


def init_library(libpath):
    lib = ctypes.cdll.LoadLibrary(str(libpath))
    vp, cp, i32, i64 = ctypes.c_void_p, ctypes.c_char_p, ctypes.c_int32, ctypes.c_int64
    lib.parpy_init.argtypes = [i64]
    lib.parpy_init.restype = None
    lib.parpy_sync.argtypes = []
    lib.parpy_sync.restype = i32
    lib.parpy_alloc_buffer.argtypes = [i64]
    lib.parpy_alloc_buffer.restype = vp
    lib.parpy_memcpy.argtypes = [vp, vp, i64, i64]
    lib.parpy_memcpy.restype = i32
    lib.parpy_memset.argtypes = [vp, i64, ctypes.c_int8]
    lib.parpy_memset.restype = i32
    lib.parpy_free_buffer.argtypes = [vp]
    lib.parpy_free_buffer.restype = i32
    lib.parpy_get_error_message.argtypes = []
    lib.parpy_get_error_message.restype = cp
    lib.parpy_hip_compile.argtypes = [cp, ctypes.POINTER(cp), i32, ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_size_t)]
    lib.parpy_hip_compile.restype = i32
    lib.parpy_hip_free_code.argtypes = [vp]
    lib.parpy_hip_free_code.restype = None
    lib.parpy_hip_module_load.argtypes = [vp, ctypes.c_size_t, ctypes.POINTER(vp)]
    lib.parpy_hip_module_load.restype = i32
    lib.parpy_hip_module_unload.argtypes = [vp]
    lib.parpy_hip_module_unload.restype = i32
    lib.parpy_hip_launch.argtypes = [vp, cp, ctypes.POINTER(i64 * 3), ctypes.POINTER(i64 * 3), i64, ctypes.POINTER(vp)]
    lib.parpy_hip_launch.restype = i32
    lib.parpy_hip_plan_create.argtypes = [vp, cp, ctypes.POINTER(vp)]
    lib.parpy_hip_plan_create.restype = i32
    lib.parpy_hip_plan_run.argtypes = [vp, ctypes.POINTER(vp), i32]
    lib.parpy_hip_plan_run.restype = i32
    lib.parpy_hip_plan_run_timed.argtypes = [vp, ctypes.POINTER(vp), i32, ctypes.POINTER(ctypes.c_float)]
    lib.parpy_hip_plan_run_timed.restype = i32
    lib.parpy_hip_plan_run_noalloc.argtypes = [vp, ctypes.POINTER(vp), i32]
    lib.parpy_hip_plan_run_noalloc.restype = i32
    lib.parpy_hip_plan_set_graph.argtypes = [vp, i32]
    lib.parpy_hip_plan_set_graph.restype = i32
    lib.parpy_hip_plan_graph_replays.argtypes = [vp]
    lib.parpy_hip_plan_graph_replays.restype = i64
    lib.parpy_hip_plan_persistent_launches.argtypes = [vp]
    lib.parpy_hip_plan_persistent_launches.restype = i64
    lib.parpy_hip_plan_launch_count.argtypes = [vp]
    lib.parpy_hip_plan_launch_count.restype = i64
    lib.parpy_hip_plan_destroy.argtypes = [vp]
    lib.parpy_hip_plan_destroy.restype = i32
    return lib


def load_hip_runtime_lib():
    """Load the runtime library without requiring a GPU (hiprtc compilation works on any host)."""
    if "hip-nogpu" not in libs:
        # what is built is loaded; a library that does not match its sources (by content, not by file time) is
        # rebuilt first, so that a forgotten build step cannot put old code under test
        _buildstamp.ensure_current(PARPY_HIP_BASE_LIB_PATH, _runtime_deps(), HIPCC_FLAGS, lambda: build_library(force=True))
        libs["hip-nogpu"] = init_library(PARPY_HIP_BASE_LIB_PATH)
    return libs["hip-nogpu"]


def _compile_runtime_lib(backend):
    """Return the runtime library of `backend`; fails loudly when the backend is not usable."""
    if backend not in libs:
        from .backend import is_enabled
        if backend != CompileBackend.Hip:
            raise RuntimeError(f"Failed to load runtime library for backend {backend}: only CompileBackend.Hip is built")
        if not is_enabled(backend):
            raise RuntimeError(f"Cannot use the runtime library for {backend} as it is disabled")
        lib = load_hip_runtime_lib()
        lib.parpy_init(0)
        libs[backend] = lib
    return libs[backend]
