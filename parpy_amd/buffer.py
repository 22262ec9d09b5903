"""Device buffers: the `parpy.buffer` interface of the reference (python/parpy/buffer.py) on ROCm.

Design.  A buffer is a typed, shaped *view*; what views share is a `_Storage`:
the torch tensor that owns the device memory and, when the data came from a
host array, that array.  Views made by `reshape` and same-width `with_type`
point at the same storage.  Python's own reference counting decides when a
storage dies, and a storage that mirrors a host array copies the device
contents back at that moment -- this is how a NumPy argument of a jitted
function receives its results.  The number of live views is observable as
`refcount` (a one-element list, as the reference's tests read it).

Device arrays (torch tensors on the ROCm device, or anything else publishing
`__cuda_array_interface__`) are wrapped without a copy.
"""
import math
import weakref
from collections import namedtuple

from .options import CompileBackend, DataType, ElemSize
from .runtime import _compile_runtime_lib

ArrayDesc = namedtuple("ArrayDesc", ["shape", "dtype", "ptr"])

H2D, D2H = 1, 2   # copy directions of parpy_memcpy


def _call(lib, status):
    """Turn a non-zero status of the runtime library into an exception carrying its message."""
    if status:
        text = lib.parpy_get_error_message().decode("ascii", "replace")
        raise RuntimeError(f"Runtime library error: {text} (code={status})")


# ---------------------------------------------------------------- describing foreign arrays
def _from_interface(intf):
    """ArrayDesc of an array-interface dictionary (version 3): writable, contiguous, little-endian."""
    if "data" not in intf:
        raise ValueError("Buffer protocol not supported")
    ptr, read_only = intf["data"]
    if read_only is True:
        raise ValueError("Cannot construct buffer from read-only memory")
    if intf.get("strides") is not None:
        raise ValueError("Buffers must only operate on contiguous memory")
    return ArrayDesc(intf["shape"], DataType(intf["typestr"]), ptr)


_torch_dtypes = {}


def _torch_tensor_info(t):
    """ArrayDesc of a plain torch tensor on the device, read from the tensor itself (its
    array-interface property builds a dictionary on every access); None for anything else."""
    import sys
    torch = sys.modules.get("torch")
    if torch is None or type(t) is not torch.Tensor or not t.is_cuda or t.requires_grad:
        return None
    if not t.is_contiguous():
        raise ValueError("Buffers must only operate on contiguous memory")
    if not _torch_dtypes:
        for sz in ElemSize:
            dt = DataType.from_elem_size(sz)
            _torch_dtypes.setdefault(dt.to_torch(), dt)   # unsigned 16/32/64 share the signed torch type
    dtype = _torch_dtypes.get(t.dtype)
    return None if dtype is None else ArrayDesc(tuple(t.shape), dtype, t.data_ptr())


def _describe(a, device_ok=False):
    """ArrayDesc of any object that publishes the (CUDA) array interface or converts to an array."""
    if device_ok:
        intf = getattr(a, "__cuda_array_interface__", None)
        if intf is not None:
            return _from_interface(intf)
    intf = getattr(a, "__array_interface__", None)
    if intf is None and hasattr(a, "__array__"):
        intf = a.__array__().__array_interface__
    if intf is None:
        raise ValueError("Failed to extract array interface")
    return _from_interface(intf)


def _as_dtype(dtype):
    return DataType.from_elem_size(dtype) if isinstance(dtype, ElemSize) else dtype


def _nbytes(shape, dtype):
    return math.prod(shape) * dtype.size()


# ---------------------------------------------------------------- shared storage
class _Storage:
    """What the views of one allocation share."""
    __slots__ = ("owner", "host", "views", "__weakref__")

    def __init__(self, owner, host=None):
        self.owner = owner            # torch tensor on the device, or the foreign object a carrier describes
        self.host = host              # host array that receives the contents when the storage dies
        self.views = weakref.WeakSet()

    def __del__(self):
        if self.host is None:
            return
        lib = _compile_runtime_lib(CompileBackend.Hip)
        dst = _describe(self.host)
        _call(lib, lib.parpy_memcpy(dst.ptr, self.owner.data_ptr(), _nbytes(dst.shape, dst.dtype), D2H))
        _call(lib, lib.parpy_sync())


# ---------------------------------------------------------------- module-level constructors
def sync(backend):
    """Wait until all work enqueued on the device has completed."""
    lib = _compile_runtime_lib(backend)
    _call(lib, lib.parpy_sync())


def _new_tensor(shape, dtype, zero):
    import torch
    make = torch.zeros if zero else torch.empty
    return make(tuple(shape), dtype=dtype.to_torch(), device="cuda")


def _allocate(shape, dtype, backend, zero):
    dtype = _as_dtype(dtype)
    if backend != CompileBackend.Hip:
        raise ValueError(f"Cannot allocate a buffer for unsupported backend {backend}")
    return HipBuffer(_new_tensor(shape, dtype, zero), tuple(shape), dtype)


def empty(shape, dtype, backend):
    return _allocate(shape, dtype, backend, zero=False)


def zeros(shape, dtype, backend):
    return _allocate(shape, dtype, backend, zero=True)


def empty_like(b):
    return empty(b.shape, b.dtype, b.backend)


def zeros_like(b):
    return zeros(b.shape, b.dtype, b.backend)


def from_array(t, backend):
    """Buffer over `t`: a shape/type carrier for backend None, a device buffer for Hip."""
    cls = {None: DummyBuffer, CompileBackend.Hip: HipBuffer}.get(backend)
    if cls is None:
        raise ValueError(f"Cannot convert to buffer of unknown backend {backend}")
    return cls._from_array(t)


# ---------------------------------------------------------------- views
class Buffer:
    backend = None

    def __init__(self, buf, shape, dtype, storage=None):
        if type(self) is Buffer:
            raise RuntimeError("Cannot construct instance of base Buffer class")
        self.buf = buf
        self.shape = tuple(shape)
        self.dtype = _as_dtype(dtype)
        self._storage = storage if storage is not None else _Storage(buf)
        self._storage.views.add(self)

    # the reference's tests read these two
    @property
    def src(self):
        return self._storage.host

    @property
    def refcount(self):
        return [len(self._storage.views)]

    def _scalar(self, kind, convert):
        if self.shape != ():
            raise ValueError(f"Cannot convert buffer of shape {self.shape} to {kind}")
        return convert(self.numpy().item())

    def __float__(self):
        return self._scalar("float", float)

    def __int__(self):
        return self._scalar("int", int)

    def __bool__(self):
        return self._scalar("bool", bool)

    def __index__(self):
        if self.shape == () and self.dtype.is_integer():
            return int(self)
        raise ValueError(f"Cannot use buffer of shape {self.shape} and type {self.dtype} as index")

    def _get_ptr(self):
        return self.buf

    def sync(self):
        sync(self.backend)

    def size(self):
        return _nbytes(self.shape, self.dtype)

    def numpy(self):
        import numpy as np
        return np.asarray(self)

    def torch(self):
        import torch
        return torch.as_tensor(self.numpy())

    def _checked_shape(self, dims):
        new_shape = tuple(dims)
        if math.prod(self.shape) != math.prod(new_shape):
            raise ValueError(f"Cannot reshape buffer of shape {self.shape} to {new_shape}")
        return new_shape

    def _checked_dtype(self, new_dtype):
        new_dtype = _as_dtype(new_dtype)
        if not isinstance(new_dtype, DataType):
            raise ValueError(f"Found unsupported data type: {type(new_dtype)}")
        return new_dtype

    def copy(self):
        raise RuntimeError("Cannot instantiate base Buffer class")

    reshape = with_type = copy


class DummyBuffer(Buffer):
    """Shape/type carrier for code generation without a device: it describes an array and never touches it."""

    def __init__(self, buf, shape, dtype, storage=None):
        super().__init__(buf, shape, dtype, storage)
        self.__array_interface__ = {"data": (self.buf, False), "strides": None, "typestr": str(self.dtype),
                                    "shape": self.shape, "version": 3}

    @staticmethod
    def _from_array(t):
        try:
            d = _describe(t, device_ok=True)
        except ValueError:
            raise RuntimeError(f"Cannot convert argument {t} to CPU buffer")
        return DummyBuffer(d.ptr, d.shape, d.dtype, _Storage(t))

    def numpy(self):
        import numpy as np
        described = self._storage.owner
        if hasattr(described, "cpu"):
            described = described.cpu()
        return np.asarray(self if isinstance(described, int) else described)

    def reshape(self, *dims):
        return DummyBuffer(self.buf, self._checked_shape(dims), self.dtype, self._storage)

    def with_type(self, new_dtype):
        return DummyBuffer(self.buf, self.shape, self._checked_dtype(new_dtype), self._storage)


class HipBuffer(Buffer):
    """View of a torch tensor on the ROCm device, shared zero-copy with generated kernels."""
    backend = CompileBackend.Hip

    def __init__(self, buf, shape, dtype, storage=None, ptr=None):
        super().__init__(buf, shape, dtype, storage)
        self._ptr = ptr

    @property
    def __cuda_array_interface__(self):
        return self.buf.__cuda_array_interface__

    @staticmethod
    def _from_array(t):
        d = _torch_tensor_info(t)
        if d is None and hasattr(t, "__cuda_array_interface__"):
            try:
                d = _describe(t, device_ok=True)
            except ValueError:
                raise ValueError(f"Cannot convert argument {t} to a HIP buffer")
        if d is not None:                    # already on the device: no copy
            return HipBuffer(t, d.shape, d.dtype, ptr=d.ptr)
        try:
            d = _describe(t)
        except ValueError:
            raise ValueError(f"Cannot convert argument {t} to a HIP buffer")
        tensor = _new_tensor(d.shape, d.dtype, zero=False)
        lib = _compile_runtime_lib(CompileBackend.Hip)
        _call(lib, lib.parpy_memcpy(tensor.data_ptr(), d.ptr, _nbytes(d.shape, d.dtype), H2D))
        _call(lib, lib.parpy_sync())         # the copy is asynchronous and the source must outlive it
        return HipBuffer(tensor, d.shape, d.dtype, _Storage(tensor, host=t), tensor.data_ptr())

    def _get_ptr(self):
        if self._ptr is None:
            self._ptr = _describe(self.buf, device_ok=True).ptr
        return self._ptr

    def numpy(self):
        import numpy as np
        return np.asarray(self.buf.cpu())

    def torch(self):
        return self.buf

    def copy(self):
        return HipBuffer(self.buf.detach().clone(), self.shape, self.dtype)

    def reshape(self, *dims):
        new_shape = self._checked_shape(dims)
        return HipBuffer(self.buf.reshape(new_shape), new_shape, self.dtype, self._storage, self._ptr)

    def with_type(self, new_dtype):
        new_dtype = self._checked_dtype(new_dtype)
        if new_dtype.size() == self.dtype.size():     # same width: the same bytes read differently
            return HipBuffer(self.buf, self.shape, new_dtype, self._storage, self._ptr)
        return HipBuffer(self.buf.detach().clone().to(new_dtype.to_torch()), self.shape, new_dtype)
