"""Normalisation of call arguments (python/parpy/validate.py:6-43 of the reference).

Every argument of a jitted function ends up as one of: a Python number (folded into the code), a Buffer,
or a flat dictionary of those.  What each kind of foreign object becomes:

  torch tensor on the device, other device array   HipBuffer over the same memory
  host array with dimensions                       device copy that is written back after the call
                                                   (a shape carrier when code is only generated)
  0-d host array                                   shape carrier: its value is folded into the code
"""
from .options import CompileBackend
from .buffer import Buffer, HipBuffer, _torch_tensor_info, from_array


class _Checker:
    def __init__(self, opts, execute):
        self.hip = opts.backend == CompileBackend.Hip
        self.backend = opts.backend
        self.execute = execute

    def value(self, arg, where, nested=False):
        if isinstance(arg, (int, float, Buffer)):
            return arg
        if isinstance(arg, dict):
            return self.fields(arg, where, nested)
        if self.hip:
            d = _torch_tensor_info(arg)
            if d is not None:
                return HipBuffer(arg, d.shape, d.dtype, ptr=d.ptr)
        if hasattr(arg, "__cuda_array_interface__"):
            if not self.hip:
                raise RuntimeError(f"Argument {where} is a GPU array, which is not supported in {self.backend}.")
            return from_array(arg, CompileBackend.Hip)
        if hasattr(arg, "__array_interface__") or hasattr(arg, "__array__"):
            on_device = self.execute and getattr(arg, "ndim", None) != 0
            return from_array(arg, self.backend if on_device else None)
        raise RuntimeError(f"Argument {where} has unsupported type {type(arg)}")

    def fields(self, arg, where, nested):
        if nested:
            raise RuntimeError(f"Dictionary argument {where} contains nested dictionary")
        out = {}
        for key, v in arg.items():
            if not isinstance(key, str):
                raise RuntimeError(f"Dictionary argument {where} contains non-string key {key}")
            out[key] = self.value(v, f"{where}[\"{key}\"]", nested=True)
        return out


def check_arguments(args, opts, execute):
    c = _Checker(opts, execute)
    return [c.value(arg, f"#{pos}") for pos, arg in enumerate(args, 1)]
