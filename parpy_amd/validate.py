"""Argument validation (python/parpy/validate.py:6-43 of the reference)."""
from .options import CompileBackend
from .buffer import Buffer, HipBuffer, _torch_tensor_info, from_array


def check_dict(arg, i, in_dict, opts, execute):
    if in_dict:
        raise RuntimeError(f"Dictionary argument {i} contains nested dictionary")
    arg_res = {}
    for k, v in arg.items():
        if not isinstance(k, str):
            raise RuntimeError(f"Dictionary argument {i} contains non-string key {k}")
        arg_res[k] = check_arg(v, f"{i}[\"{k}\"]", True, opts, execute)
    return arg_res


def check_arg(arg, i, in_dict, opts, execute):
    if isinstance(arg, (int, float)):
        return arg
    if isinstance(arg, dict):
        return check_dict(arg, i, in_dict, opts, execute)
    if isinstance(arg, Buffer):
        return arg
    if opts.backend == CompileBackend.Hip:
        info = _torch_tensor_info(arg)
        if info is not None:
            return HipBuffer(arg, info[0], info[1], ptr=info[2])
    if hasattr(arg, "__cuda_array_interface__"):
        # torch on ROCm publishes device tensors through this protocol: wrap zero-copy
        if opts.backend == CompileBackend.Hip:
            return from_array(arg, CompileBackend.Hip)
        raise RuntimeError(f"Argument {i} is a GPU array, which is not supported in {opts.backend}.")
    if hasattr(arg, "__array_interface__") or hasattr(arg, "__array__"):
        # Host data is copied to the device for the call and copied back when the
        # temporary buffer dies; when only generating code nothing is copied.  A 0-d
        # host array is a scalar that gets folded into the code: it needs no device copy.
        if getattr(arg, "ndim", None) == 0:
            return from_array(arg, None)
        return from_array(arg, opts.backend if execute else None)
    raise RuntimeError(f"Argument {i} has unsupported type {type(arg)}")


def check_arguments(args, opts, execute):
    return [check_arg(arg, f"#{i+1}", False, opts, execute) for i, arg in enumerate(args)]
