"""The two C-ABI libraries load and export every symbol their headers declare (no GPU calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(parpy_[a-z0-9_]+)\s*\(", text)))


def test_runtime_library_exports():
    from parpy_amd import runtime
    lib = ctypes.CDLL(str(runtime.PARPY_HIP_BASE_LIB_PATH))
    names = _declared("parpy_hip.h")
    assert {"parpy_init", "parpy_sync", "parpy_alloc_buffer", "parpy_memcpy", "parpy_memset", "parpy_free_buffer",
            "parpy_get_error_message", "parpy_hip_compile", "parpy_hip_plan_run"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n


def test_compiler_library_exports():
    from parpy_amd import compiler
    lib = ctypes.CDLL(str(compiler.LIB_PATH))
    names = _declared("parpy_hipc.h")
    assert {"parpy_hipc_parse", "parpy_hipc_compile", "parpy_hipc_fun_print", "parpy_hipc_fun_name"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n


def test_hiprtc_compile_error_path():
    """A broken source fails through the C ABI with the compiler log as message (test/test_cuda.py:143-153)."""
    import parpy_amd as parpy
    from parpy_amd.compile import hiprtc_compile
    with pytest.raises(RuntimeError, match="Compilation of generated HIP code failed"):
        hiprtc_compile("extern \"C\" __global__ void k(float* a) { a[0] = undeclared_name; }", parpy.CompileOptions())


def test_plan_rejects_malformed_text_and_wrong_arity():
    from parpy_amd import runtime
    lib = runtime.load_hip_runtime_lib()
    plan = ctypes.c_void_p()
    assert lib.parpy_hip_plan_create(None, b"(not-a-plan)", ctypes.byref(plan)) != 0
    assert b"invalid launch plan" in lib.parpy_get_error_message()
    text = b'(plan "f" (params ("x" ptr)) (kernels) (body ))'
    assert lib.parpy_hip_plan_create(None, text, ctypes.byref(plan)) == 0
    args = (ctypes.c_void_p * 2)(None, None)
    assert lib.parpy_hip_plan_run(plan, args, 2) != 0
    assert b"expects 1 pointer arguments" in lib.parpy_get_error_message()
    assert lib.parpy_hip_plan_run(plan, args, 1) != 0   # no module loaded: refuses to run
    assert lib.parpy_hip_plan_destroy(plan) == 0


def test_a_library_that_does_not_match_its_sources_is_rebuilt_on_load(monkeypatch, tmp_path):
    """Staleness goes by content (a stamp with the hash of the sources written at build time), not by file
    times, which do not survive copying the tree: a library whose stamp differs is rebuilt with a warning,
    PARPY_AMD_REBUILD=0 loads it as it is, and a matching one is loaded silently."""
    import warnings
    from parpy_amd import runtime, _buildstamp
    built = []
    monkeypatch.setattr(runtime, "build_library", lambda force=False: built.append(force))
    monkeypatch.delenv("PARPY_AMD_REBUILD", raising=False)
    monkeypatch.delitem(runtime.libs, "hip-nogpu", raising=False)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        assert runtime.load_hip_runtime_lib() is not None      # as built: no warning, no compilation
    assert built == []
    monkeypatch.setattr(_buildstamp, "source_hash", lambda paths, command: "another hash")
    monkeypatch.delitem(runtime.libs, "hip-nogpu", raising=False)
    with pytest.warns(RuntimeWarning, match="does not match its sources: rebuilding"):
        runtime.load_hip_runtime_lib()
    assert built == [True]
    monkeypatch.delitem(runtime.libs, "hip-nogpu", raising=False)
    monkeypatch.setenv("PARPY_AMD_REBUILD", "0")
    with pytest.warns(RuntimeWarning, match="PARPY_AMD_REBUILD=0 keeps it"):
        runtime.load_hip_runtime_lib()
    assert built == [True]
    # the hash covers contents and the command line
    a = tmp_path / "a.cpp"
    a.write_text("int x;")
    monkeypatch.undo()
    h1 = _buildstamp.source_hash([a], ["cc"])
    assert h1 == _buildstamp.source_hash([a], ["cc"]) and h1 != _buildstamp.source_hash([a], ["cc", "-O2"])
    a.write_text("int y;")
    assert h1 != _buildstamp.source_hash([a], ["cc"])


def test_running_without_a_device_fails_loudly():
    """No CPU path stands in for the HIP backend: with no ROCm device a call raises (the reference's messages,
    python/parpy/backend.py), it does not fall back to anything."""
    import numpy as np
    import parpy_amd as parpy
    if parpy.backend.is_enabled(parpy.CompileBackend.Hip):
        pytest.skip("a ROCm device is visible")

    @parpy.jit
    def set_first(x):
        with parpy.gpu:
            x[0] = 1.0
    o = parpy.par({})
    o.backend = parpy.CompileBackend.Hip
    with pytest.raises(RuntimeError, match="Specified backend CompileBackend.Hip is not available"):
        set_first(np.zeros(4, dtype=np.float32), opts=o)
    with pytest.raises(RuntimeError, match="Found no enabled GPU backends"):
        set_first(np.zeros(4, dtype=np.float32), opts=parpy.par({}))
