"""Value classes of the ParPy surface: element sizes, data types, loop
parallelisation specs and compile options.

Mirrors the reference's pyo3 classes (src/option.rs:8-162, src/par.rs:6-91,
src/buffer.rs:15-243, src/utils/ast.rs:9-110).  They are plain Python here
and are serialised as S-expressions for the C++ compiler core, which holds
its own copies of LoopPar / options (csrc/compiler/ast.hpp).
"""
import ctypes
import enum

WAVE_SIZE = 64          # CDNA wavefront width; the reference hard-codes 32-lane warps
DEFAULT_TPB = 1024      # src/par.rs:7
REDUCE_PAR_LABEL = "_reduce"   # src/par.rs:6


class CompileBackend(enum.Enum):
    """src/option.rs:8-12 plus the new Hip member."""
    Auto = 0
    Cuda = 1
    Metal = 2
    Hip = 3

    def __repr__(self):
        return f"CompileBackend.{self.name}"

    __str__ = __repr__


class Target(enum.Enum):
    Host = 0
    Device = 1


class ElemSize(enum.Enum):
    Bool = "bool"
    I8 = "i8"
    I16 = "i16"
    I32 = "i32"
    I64 = "i64"
    U8 = "u8"
    U16 = "u16"
    U32 = "u32"
    U64 = "u64"
    F16 = "f16"
    F32 = "f32"
    F64 = "f64"

    def is_signed_integer(self):
        return self in (ElemSize.I8, ElemSize.I16, ElemSize.I32, ElemSize.I64)

    def is_unsigned_integer(self):
        return self in (ElemSize.U8, ElemSize.U16, ElemSize.U32, ElemSize.U64)

    def is_integer(self):
        return self.is_signed_integer() or self.is_unsigned_integer()

    def is_floating_point(self):
        return self in (ElemSize.F16, ElemSize.F32, ElemSize.F64)

    def size(self):
        """Width of one element in bytes."""
        return _NBYTES[self]

    def __repr__(self):
        return f"ElemSize.{self.name}"

    __str__ = __repr__


class ExtType:
    """Type annotation of an external's pointer parameter (python/parpy/types.py:16-20)."""

    def __init__(self, sz):
        self.sz = sz

    @staticmethod
    def Pointer(sz):
        return ExtType(sz)

    def __eq__(self, other):
        return isinstance(other, ExtType) and self.sz == other.sz

    def __hash__(self):
        return hash(("ptr", self.sz))


# array-interface typestr <-> ElemSize (src/buffer.rs:15-30)
_TYPESTR = {
    "b1": ElemSize.Bool, "i1": ElemSize.I8, "i2": ElemSize.I16, "i4": ElemSize.I32,
    "i8": ElemSize.I64, "u1": ElemSize.U8, "u2": ElemSize.U16, "u4": ElemSize.U32,
    "u8": ElemSize.U64, "f2": ElemSize.F16, "f4": ElemSize.F32, "f8": ElemSize.F64,
}
_TYPESTR_INV = {v: k for k, v in _TYPESTR.items()}
_NBYTES = {ElemSize.Bool: 1, ElemSize.I8: 1, ElemSize.I16: 2, ElemSize.I32: 4,
           ElemSize.I64: 8, ElemSize.U8: 1, ElemSize.U16: 2, ElemSize.U32: 4,
           ElemSize.U64: 8, ElemSize.F16: 2, ElemSize.F32: 4, ElemSize.F64: 8}


class DataType:
    """Byte order + element size parsed from an array-interface typestr (src/buffer.rs:160-243)."""

    def __init__(self, typestr):
        if isinstance(typestr, DataType):
            self.byteorder, self.sz = typestr.byteorder, typestr.sz
            return
        typestr = str(typestr)
        if len(typestr) < 3 or typestr[0] not in "<>|=" or typestr[1:] not in _TYPESTR:
            raise ValueError(f"Unsupported array interface type string: {typestr}")
        if typestr[0] == ">":
            raise ValueError("Big-endian data is not supported")
        self.byteorder = typestr[0]
        self.sz = _TYPESTR[typestr[1:]]

    @staticmethod
    def from_elem_size(sz):
        bo = "|" if _NBYTES[sz] == 1 else "<"
        return DataType(bo + _TYPESTR_INV[sz])

    def size(self):
        return _NBYTES[self.sz]

    def is_integer(self):
        return self.sz.is_integer()

    def is_floating_point(self):
        return self.sz.is_floating_point()

    def __str__(self):
        return self.byteorder + _TYPESTR_INV[self.sz]

    __repr__ = __str__

    def __eq__(self, other):
        return isinstance(other, DataType) and self.sz == other.sz

    def __hash__(self):
        return hash(self.sz)

    def to_numpy(self):
        import numpy as np
        return np.dtype(str(self))

    def to_torch(self):
        # torch has no unsigned 16/32/64 arithmetic types worth using: the
        # reference maps them to the signed type of equal width (src/buffer.rs:93-109).
        import torch
        return {
            ElemSize.Bool: torch.bool, ElemSize.I8: torch.int8, ElemSize.I16: torch.int16,
            ElemSize.I32: torch.int32, ElemSize.I64: torch.int64, ElemSize.U8: torch.uint8,
            ElemSize.U16: torch.int16, ElemSize.U32: torch.int32, ElemSize.U64: torch.int64,
            ElemSize.F16: torch.float16, ElemSize.F32: torch.float32, ElemSize.F64: torch.float64,
        }[self.sz]

    def to_ctype(self):
        return {
            ElemSize.Bool: ctypes.c_bool, ElemSize.I8: ctypes.c_int8, ElemSize.I16: ctypes.c_int16,
            ElemSize.I32: ctypes.c_int32, ElemSize.I64: ctypes.c_int64, ElemSize.U8: ctypes.c_uint8,
            ElemSize.U16: ctypes.c_uint16, ElemSize.U32: ctypes.c_uint32, ElemSize.U64: ctypes.c_uint64,
            ElemSize.F16: ctypes.c_uint16, ElemSize.F32: ctypes.c_float, ElemSize.F64: ctypes.c_double,
        }[self.sz]


class LoopPar:
    """Per-label parallelisation: number of threads, reduction flag, threads per block.

    src/par.rs:11-91.  The only rule that changes for CDNA is tpb's granule:
    a multiple of the 64-lane wavefront instead of the 32-lane warp.
    """

    def __init__(self, nthreads=0, reduction=False, tpb=DEFAULT_TPB):
        self.nthreads = nthreads
        self.reduction = reduction
        self._tpb = tpb

    def is_parallel(self):
        return self.nthreads > 0

    def threads(self, nthreads):
        if self.nthreads == 0:
            return LoopPar(int(nthreads), self.reduction, self._tpb)
        raise RuntimeError("The number of threads can only be set once")

    def reduce(self):
        return LoopPar(self.nthreads, True, self._tpb)

    def tpb(self, tpb):
        if tpb > 0 and tpb % WAVE_SIZE == 0:
            return LoopPar(self.nthreads, self.reduction, int(tpb))
        raise RuntimeError("The number of threads per block must be a positive "
                           f"integer divisible by {WAVE_SIZE}.")

    def __eq__(self, other):
        return isinstance(other, LoopPar) and (self.nthreads, self.reduction, self._tpb) == \
            (other.nthreads, other.reduction, other._tpb)

    def __repr__(self):
        return f"LoopPar {{ nthreads: {self.nthreads}, reduction: {str(self.reduction).lower()}, tpb: {self._tpb} }}"

    __str__ = __repr__


_options_clock = [0]


class CompileOptions:
    """src/option.rs:14-108; __str__ feeds the in-memory cache key (python/parpy/key.py:29-30)."""

    def __setattr__(self, name, value):
        # every assignment to any options object gets a stamp that no other assignment has;
        # the stamp tells when the cached part of the fast key is stale
        _options_clock[0] += 1
        object.__setattr__(self, "_stamp", _options_clock[0])
        object.__setattr__(self, name, value)

    def _fast_key(self):
        """Hashable value of the whole options state: equal for two objects that hold equal settings,
        so that a call with a freshly built options object finds the code compiled for an earlier one.
        The fields assigned through attributes are cached per stamp; the containers, which can be
        changed in place, are read every time."""
        d = self.__dict__
        if d.get("_key_stamp") != d["_stamp"]:
            d["_key_fields"] = tuple(v for k, v in d.items()
                                     if (k[0] != "_" or k in CompileOptions._DEFAULTS) and not isinstance(v, (dict, list)))
            d["_key_stamp"] = d["_stamp"]
        return (d["_key_fields"], tuple(d["includes"]), tuple(d["libs"]), tuple(d["extra_flags"]),
                tuple((k, p.nthreads, p.reduction, p._tpb) for k, p in d["parallelize"].items()))

    # opt_*: HIP memory-codegen switches; None keeps the compiler's default.  They exist so that
    # tests and benchmarks can measure what each buys.
    # defaults of the fields that hold plain values, in the order the fast key reads them
    _DEFAULTS = {
        'verbose_backend_resolution': False,
        'debug_print': False,
        'write_output': False,
        'backend': CompileBackend.Auto,
        'use_cuda_thread_block_clusters': False,
        '_max_thread_blocks_per_cluster': 8,
        'use_cuda_graphs': False,
        'persistent_loops': False,   # host loops of launches run inside one kernel with device-wide barriers when the grid fits
        'device_functions': False,   # jitted functions called inside expressions stay functions on the device instead of being inlined
        '_force_int_size': None,
        '_force_float_size': None,
        'opt_vectorize': None,
        'opt_lds_rows': None,
        'opt_reg_cache': None,
        'opt_hoist_invariant': None,
        'opt_narrow_index': None,
        'opt_mfma_sddmm': None,
        'opt_unswitch': None,
        'opt_gather_transpose': None,
        'opt_nontemporal': None,
        'opt_lane_split': None,
        'opt_drop_barriers': None,
        'opt_unswitch_uniform': None,
        'opt_offset32': None,
        'opt_if_convert': None,
        'opt_noalias_scopes': None,
        'opt_expand_short_loops': None,
        'opt_guard_bounds': None,
        'opt_pack_accesses': None,
        'opt_share_iterations': None,
        'opt_fence_iterations': None,
        'opt_keep_stored': None,
        'opt_keep_own': None,
        'opt_prefetch_steps': None,
        'reg_budget': None,   # registers per thread the caching passes may claim (None: by block size)
        'reg_budget_scale': None,   # percent of the default budget (set by the register feedback of the driver)
        'reg_feedback': True,   # recompile with a smaller budget when the code object reports spilled vector registers
        'reg_feedback_timed': False,   # ... and pick between the two by timing them on the first call (runs the function several times)
        'assume_aligned': None,   # set by the driver: False when an array argument is not 16-byte aligned
    }

    def __init__(self):
        # written into the instance dictionary directly: building an options object is part of
        # many calls (`opts=parpy.par(...)`) and thirty stamped assignments would dominate them
        d = self.__dict__
        d.update(CompileOptions._DEFAULTS)
        d["parallelize"] = {}
        d["includes"] = []
        d["libs"] = []
        d["extra_flags"] = []
        _options_clock[0] += 1
        d["_stamp"] = d["_key_stamp"] = _options_clock[0]
        d["_key_fields"] = CompileOptions._DEFAULT_KEY

    @property
    def max_thread_blocks_per_cluster(self):
        return self._max_thread_blocks_per_cluster

    @max_thread_blocks_per_cluster.setter
    def max_thread_blocks_per_cluster(self, n):
        if n > 0 and (n & (n - 1)) == 0:
            self._max_thread_blocks_per_cluster = n
        else:
            raise RuntimeError("The number of thread blocks per cluster must be a power of two.")

    @property
    def force_int_size(self):
        return self._force_int_size

    @force_int_size.setter
    def force_int_size(self, sz):
        if not sz.is_integer():
            raise RuntimeError("Cannot use a non integer type for integer scalars.")
        self._force_int_size = sz

    @property
    def force_float_size(self):
        return self._force_float_size

    @force_float_size.setter
    def force_float_size(self, sz):
        if not sz.is_floating_point():
            raise RuntimeError("Cannot use a non floating-point type for floating-point scalars.")
        self._force_float_size = sz

    def __str__(self):
        par = ", ".join(f"{k!r}: {v}" for k, v in sorted(self.parallelize.items()))
        return (f"CompileOptions {{ parallelize: {{{par}}}, "
                f"verbose_backend_resolution: {self.verbose_backend_resolution}, "
                f"debug_print: {self.debug_print}, write_output: {self.write_output}, "
                f"backend: {self.backend}, "
                f"use_cuda_thread_block_clusters: {self.use_cuda_thread_block_clusters}, "
                f"max_thread_blocks_per_cluster: {self._max_thread_blocks_per_cluster}, "
                f"use_cuda_graphs: {self.use_cuda_graphs}, "
                f"force_int_size: {self._force_int_size}, force_float_size: {self._force_float_size}, "
                f"includes: {self.includes}, libs: {self.libs}, extra_flags: {self.extra_flags} }}")


CompileOptions._DEFAULT_KEY = tuple(CompileOptions._DEFAULTS.values())


class ScalarSizes:
    """Default scalar widths: int64 / float64 unless forced (src/utils/ast.rs:78-110)."""

    def __init__(self, opts):
        self.int = DataType.from_elem_size(opts.force_int_size or ElemSize.I64)
        self.float = DataType.from_elem_size(opts.force_float_size or ElemSize.F64)


def par(p):
    """Default options carrying the parallelisation mapping `p` (src/option.rs:157-162)."""
    opts = CompileOptions()
    for k, v in p.items():
        if not isinstance(k, str) or not isinstance(v, LoopPar):
            raise TypeError("parallelization specification must map label strings to LoopPar values")
    opts.__dict__["parallelize"] = dict(p)   # (no stamp needed: the fast key reads the mapping itself)
    return opts
