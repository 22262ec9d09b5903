"""Which backends can run here, and what `CompileBackend.Auto` stands for
(python/parpy/backend.py:6-77 of the reference, with Hip as the only member)."""
import shutil

from .options import CompileBackend

backends = [CompileBackend.Hip]


def _why_not(backend):
    """Reason why `backend` cannot execute code on this machine, or None when it can."""
    if backend in (CompileBackend.Cuda, CompileBackend.Metal):
        return f"Backend {backend} is not part of this build (HIP only)"
    if backend != CompileBackend.Hip:
        return f"Unsupported backend {backend}"
    import torch
    if getattr(torch.version, "hip", None) is None:
        return "Torch was not built with ROCm support"
    if not torch.cuda.is_available():
        return "No ROCm device is visible to Torch"
    from .runtime import PARPY_HIP_BASE_LIB_PATH
    if not PARPY_HIP_BASE_LIB_PATH.exists() and not shutil.which("hipcc"):
        return "The HIP runtime library is not built and 'hipcc' is not in the path to build it"
    return None


def is_enabled(backend, verbose=False):
    """Whether `backend` can execute code on this machine."""
    reason = _why_not(backend)
    if reason is not None and verbose:
        print(f"Backend {backend} is not enabled: {reason}")
    return reason is None


available = [b for b in backends if is_enabled(b)]


def _resolve_backend(opts, strict):
    """Replace CompileBackend.Auto in `opts` by the one enabled backend and check a named backend.

    `strict` is set when the code is going to run.  When it is only generated and no backend is enabled, Auto
    stands for Hip: this build has exactly one code generator.
    """
    if opts.verbose_backend_resolution:
        for b in backends:
            is_enabled(b, verbose=True)
    if opts.backend != CompileBackend.Auto:
        if strict and opts.backend not in available:
            raise RuntimeError(f"Specified backend {opts.backend} is not available. For more information, enable the "
                               "'verbose_backend_resolution' flag in the compiler options.")
        return opts
    if len(available) > 1:
        raise RuntimeError(f"Found multiple supported GPU backends: {available}. Please explicitly specify which "
                           "backend to use by setting the 'backend' field of the 'opts' argument to the desired backend.")
    if not available and strict:
        raise RuntimeError("Found no enabled GPU backends. For detailed information on why this is, "
                           "enable the 'verbose_backend_resolution' flag in the compiler options.")
    opts.backend = available[0] if available else CompileBackend.Hip
    return opts
