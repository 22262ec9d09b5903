"""Device buffers (python/parpy/buffer.py of the reference; HipBuffer takes the place of CudaBuffer).

A HipBuffer wraps a torch tensor that lives on the ROCm device.  Device arrays
(anything exposing __cuda_array_interface__, which is what torch-ROCm
publishes) are wrapped zero-copy; host arrays are copied in through the
runtime library and copied back when the last view of the temporary dies.
"""
from .options import CompileBackend, DataType, ElemSize
from .runtime import _compile_runtime_lib


def _check_errors(lib, rescode):
    if rescode != 0:
        msg = lib.parpy_get_error_message().decode("ascii", "replace")
        raise RuntimeError(f"Runtime library error: {msg} (code={rescode})")


def _check_not_nullptr(lib, resptr):
    if not resptr:
        raise RuntimeError(f"Runtime library error: {lib.parpy_get_error_message()}")
    return resptr


def _check_array_interface(intf):
    shape = intf["shape"]
    dtype = DataType(intf["typestr"])
    if "data" in intf:
        data, ro = intf["data"]
        if ro is True:
            raise ValueError("Cannot construct buffer from read-only memory")
    else:
        raise ValueError("Buffer protocol not supported")
    if "strides" in intf and intf["strides"] is not None:
        raise ValueError("Buffers must only operate on contiguous memory")
    return shape, dtype, data


_TORCH_DTYPES = {}


def _torch_tensor_info(t):
    """(shape, dtype, device pointer) of a plain torch tensor on the device without going through
    its array-interface property (which builds a dict on every access), or None."""
    import sys
    torch = sys.modules.get("torch")
    if torch is None or type(t) is not torch.Tensor or not t.is_cuda or t.requires_grad:
        return None
    if not t.is_contiguous():
        raise ValueError("Buffers must only operate on contiguous memory")
    if not _TORCH_DTYPES:
        for sz in ElemSize:
            dt = DataType.from_elem_size(sz)
            _TORCH_DTYPES.setdefault(dt.to_torch(), dt)
    dtype = _TORCH_DTYPES.get(t.dtype)
    if dtype is None:
        return None
    return tuple(t.shape), dtype, t.data_ptr()


def _to_array_interface(ptr, dtype, shape):
    return {"data": (ptr, False), "strides": None, "typestr": str(dtype), "shape": shape, "version": 3}


def _extract_array_interface(a, allow_cuda=False):
    if allow_cuda and hasattr(a, "__cuda_array_interface__"):
        return _check_array_interface(a.__cuda_array_interface__)
    if hasattr(a, "__array_interface__"):
        return _check_array_interface(a.__array_interface__)
    if hasattr(a, "__array__"):
        return _check_array_interface(a.__array__().__array_interface__)
    raise ValueError("Failed to extract array interface")


def _resolve_dtype(dtype):
    if isinstance(dtype, ElemSize):
        return DataType.from_elem_size(dtype)
    return dtype


def _size(shape, dtype):
    sz = dtype.size()
    for dim in shape:
        sz *= dim
    return sz


def sync(backend):
    """Wait until all work enqueued on the device has completed."""
    lib = _compile_runtime_lib(backend)
    _check_errors(lib, lib.parpy_sync())


def empty(shape, dtype, backend):
    dtype = _resolve_dtype(dtype)
    if backend == CompileBackend.Hip:
        import torch
        t = torch.empty(*shape, dtype=dtype.to_torch(), device="cuda")
        return HipBuffer(t, tuple(shape), dtype)
    raise ValueError(f"Cannot allocate a buffer for unsupported backend {backend}")


def empty_like(b):
    return empty(b.shape, b.dtype, b.backend)


def zeros(shape, dtype, backend):
    dtype = _resolve_dtype(dtype)
    if backend == CompileBackend.Hip:
        import torch
        t = torch.zeros(*shape, dtype=dtype.to_torch(), device="cuda")
        return HipBuffer(t, tuple(shape), dtype)
    raise ValueError(f"Cannot allocate a buffer for unsupported backend {backend}")


def zeros_like(b):
    return zeros(b.shape, b.dtype, b.backend)


def from_array(t, backend):
    if backend is None:
        return DummyBuffer._from_array(t)
    if backend == CompileBackend.Hip:
        return HipBuffer._from_array(t)
    raise ValueError(f"Cannot convert to buffer of unknown backend {backend}")


class Buffer:
    def __init__(self, buf, shape, dtype, src=None, refcount=None):
        if type(self) is Buffer:
            raise RuntimeError("Cannot construct instance of base Buffer class")
        self.buf = buf
        self.shape = tuple(shape)
        self.dtype = _resolve_dtype(dtype)
        self.src = src
        if refcount is None:
            self.refcount = [1]
        else:
            self.refcount = refcount
            self.refcount[0] += 1

    def __del__(self):
        self.refcount[0] -= 1
        if self.refcount[0] == 0:
            if self.src is not None:
                _, _, src_ptr = _extract_array_interface(self.src)
            else:
                src_ptr = None
            self._deconstruct(src_ptr)

    def __float__(self):
        if len(self.shape) == 0:
            return float(self.numpy().item())
        raise ValueError(f"Cannot convert buffer of shape {self.shape} to float")

    def __int__(self):
        if len(self.shape) == 0:
            return int(self.numpy().item())
        raise ValueError(f"Cannot convert buffer of shape {self.shape} to int")

    def __bool__(self):
        if len(self.shape) == 0:
            return bool(self.numpy().item())
        raise ValueError(f"Cannot convert buffer of shape {self.shape} to bool")

    def __index__(self):
        if len(self.shape) == 0 and self.dtype.is_integer():
            return self.__int__()
        raise ValueError(f"Cannot use buffer of shape {self.shape} and type {self.dtype} as index")

    def _deconstruct(self, src_ptr):
        pass

    def _get_ptr(self):
        return self.buf

    def sync(self):
        sync(self.backend)

    def size(self):
        return _size(self.shape, self.dtype)

    def numpy(self):
        import numpy as np
        return np.asarray(self)

    def torch(self):
        import torch
        return torch.as_tensor(self.numpy())

    def copy(self):
        raise RuntimeError("Cannot instantiate base Buffer class")

    def reshape(self, *dims):
        import math
        new_shape = tuple(dims)
        if math.prod(self.shape) == math.prod(new_shape):
            return type(self)(self.buf, new_shape, self.dtype, self.src, self.refcount)
        raise ValueError(f"Cannot reshape buffer of shape {self.shape} to {new_shape}")

    def with_type(self, new_dtype):
        raise RuntimeError("Cannot instantiate base Buffer class")


class DummyBuffer(Buffer):
    """Shape/dtype carrier used when code is generated but not run (no device needed)."""

    def __init__(self, buf, shape, dtype, src=None, refcount=None):
        super().__init__(buf, shape, dtype, src, refcount)
        self.__array_interface__ = _to_array_interface(self.buf, self.dtype, self.shape)
        self.backend = None

    @staticmethod
    def _from_array(t):
        try:
            shape, dtype, data_ptr = _extract_array_interface(t, allow_cuda=True)
        except ValueError:
            raise RuntimeError(f"Cannot convert argument {t} to CPU buffer")
        b = DummyBuffer(data_ptr, shape, dtype)
        b._keepalive = t
        return b

    def numpy(self):
        import numpy as np
        k = getattr(self, "_keepalive", None)
        if k is not None and hasattr(k, "cpu"):
            return np.asarray(k.cpu())
        return np.asarray(k if k is not None else self)

    def with_type(self, new_dtype):
        new_dtype = _resolve_dtype(new_dtype)
        if isinstance(new_dtype, DataType):
            return DummyBuffer(self.buf, self.shape, new_dtype, self.src, self.refcount)
        raise ValueError(f"Found unsupported data type: {type(new_dtype)}")


class HipBuffer(Buffer):
    """A torch tensor on the ROCm device, shared zero-copy with generated kernels."""

    def __init__(self, buf, shape, dtype, src=None, refcount=None, ptr=None):
        super().__init__(buf, shape, dtype, src, refcount)
        self._ptr = ptr
        self.backend = CompileBackend.Hip
        self.lib = _compile_runtime_lib(self.backend)

    @property
    def __cuda_array_interface__(self):
        return self.buf.__cuda_array_interface__

    def _deconstruct(self, src_ptr):
        if src_ptr is not None:
            _check_errors(self.lib, self.lib.parpy_memcpy(src_ptr, self._get_ptr(), self.size(), 2))
            self.sync()

    @staticmethod
    def _from_array(t):
        info = _torch_tensor_info(t)
        if info is not None:
            return HipBuffer(t, info[0], info[1], ptr=info[2])
        try:
            shape, dtype, data_ptr = _extract_array_interface(t, allow_cuda=True)
            if hasattr(t, "__cuda_array_interface__"):
                return HipBuffer(t, shape, dtype, ptr=data_ptr)
        except ValueError:
            raise ValueError(f"Cannot convert argument {t} to a HIP buffer")
        import torch
        if len(shape) == 0:
            data = torch.empty((), dtype=dtype.to_torch(), device="cuda")
        else:
            data = torch.empty(*shape, dtype=dtype.to_torch(), device="cuda")
        _, _, ptr = _extract_array_interface(data, allow_cuda=True)
        lib = _compile_runtime_lib(CompileBackend.Hip)
        _check_errors(lib, lib.parpy_memcpy(ptr, data_ptr, _size(shape, dtype), 1))
        # the host-to-device copy is asynchronous: the source must outlive it
        _check_errors(lib, lib.parpy_sync())
        return HipBuffer(data, shape, dtype, src=t, ptr=ptr)

    def _get_ptr(self):
        if self._ptr is None:
            _, _, self._ptr = _extract_array_interface(self.buf, allow_cuda=True)
        return self._ptr

    def numpy(self):
        import numpy as np
        return np.asarray(self.buf.cpu())

    def torch(self):
        return self.buf

    def copy(self):
        return HipBuffer(self.buf.detach().clone(), self.shape, self.dtype)

    def reshape(self, *dims):
        import math
        new_shape = tuple(dims)
        if math.prod(self.shape) != math.prod(new_shape):
            raise ValueError(f"Cannot reshape buffer of shape {self.shape} to {new_shape}")
        return HipBuffer(self.buf.reshape(new_shape), new_shape, self.dtype, self.src, self.refcount, self._ptr)

    def with_type(self, new_dtype):
        new_dtype = _resolve_dtype(new_dtype)
        if isinstance(new_dtype, DataType):
            if self.dtype.size() == new_dtype.size():
                return HipBuffer(self.buf, self.shape, new_dtype, self.src, self.refcount, self._ptr)
            t = self.buf.detach().clone().to(new_dtype.to_torch())
            return HipBuffer(t, self.shape, new_dtype)
        raise ValueError(f"Found unsupported data type: {type(new_dtype)}")
