"""Backend resolution (python/parpy/backend.py:6-77 of the reference, with the Hip member)."""
import shutil

from .options import CompileBackend

backends = [
    CompileBackend.Hip,
]


def _assert_hip_is_enabled():
    import torch
    if getattr(torch.version, "hip", None) is None:
        raise RuntimeError("Torch was not built with ROCm support")
    if not torch.cuda.is_available():
        raise RuntimeError("No ROCm device is visible to Torch")
    from .runtime import PARPY_HIP_BASE_LIB_PATH
    if not PARPY_HIP_BASE_LIB_PATH.exists() and not shutil.which("hipcc"):
        raise RuntimeError("The HIP runtime library is not built and 'hipcc' is not in the path to build it")


def is_enabled(backend, verbose=False):
    """Whether `backend` can execute code on this machine."""
    try:
        if backend == CompileBackend.Hip:
            _assert_hip_is_enabled()
        elif backend in (CompileBackend.Cuda, CompileBackend.Metal):
            raise RuntimeError(f"Backend {backend} is not part of this build (HIP only)")
        else:
            raise RuntimeError(f"Unsupported backend {backend}")
        return True
    except RuntimeError as e:
        if verbose:
            print(f"Backend {backend} is not enabled: {e}")
        return False


available = [b for b in backends if is_enabled(b, False)]


def _resolve_backend(opts, strict):
    """Resolve CompileBackend.Auto to the single enabled backend (python/parpy/backend.py:49-77).

    When code is only generated (strict=False) and nothing is enabled, Auto
    resolves to Hip: this build has exactly one code generator.
    """
    if opts.verbose_backend_resolution:
        [b for b in backends if is_enabled(b, True)]
    if opts.backend == CompileBackend.Auto:
        if len(available) == 1:
            opts.backend = available[0]
            return opts
        if len(available) == 0:
            if not strict:
                opts.backend = CompileBackend.Hip
                return opts
            raise RuntimeError("Found no enabled GPU backends. For detailed information on why this is, "
                               "enable the 'verbose_backend_resolution' flag in the compiler options.")
        raise RuntimeError(f"Found multiple supported GPU backends: {available}. Please explicitly specify which "
                           "backend to use by setting the 'backend' field of the 'opts' argument to the desired backend.")
    if strict and opts.backend not in available:
        raise RuntimeError(f"Specified backend {opts.backend} is not available. For more information, enable the "
                           "'verbose_backend_resolution' flag in the compiler options.")
    return opts
