"""Element types, operators, comparisons, ranges, scalars and slice statements: what the language
accepts and rejects (test/test_arith.py, test_compare.py, test_bool.py, test_range.py,
test_scalar.py, test_slicing.py of the reference), compiled for gfx950 on the CPU and run against
the Python interpreter's result of the same function on the GPU."""
import linecache
import re

import numpy as np
import pytest

import parpy_amd as parpy
import parpy_amd.operators as ops
from parpy_amd.compile import hiprtc_compile
from parpy_amd.operators import min, sum

HIP = parpy.CompileBackend.Hip
INT_TYS = [np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64]
FLOAT_TYS = [np.float16, np.float32, np.float64]


def opts_for(p, **kw):
    o = parpy.par(p)
    o.backend = HIP
    for k, v in kw.items():
        setattr(o, k, v)
    return o


def compiles(s):
    hiprtc_compile(s[:s.index("// host side")], opts_for({}))
    return s


def make_fun(name, statement, params="dst, a, b"):
    """A one-statement GPU function; built from text so that one table covers all operators."""
    src = f"def {name}({params}):\n    with parpy.gpu:\n        {statement}\n"
    fname = f"<{name}>"
    linecache.cache[fname] = (len(src), None, src.splitlines(True), fname)
    ns = {"parpy": parpy, "ops": ops}
    exec(compile(src, fname, "exec"), ns)
    return ns[name]


BINOPS = {
    "add": "dst[0] = a[0] + b[0]", "sub": "dst[0] = a[0] - b[0]", "mul": "dst[0] = a[0] * b[0]",
    "floordiv": "dst[0] = a[0] // b[0]", "div": "dst[0] = a[0] / b[0]", "rem": "dst[0] = a[0] % b[0]",
    "pow": "dst[0] = a[0] ** b[0]", "abs": "dst[0] = abs(a[0]) + abs(b[0])", "bit_and": "dst[0] = a[0] & b[0]",
    "bit_or": "dst[0] = a[0] | b[0]", "bit_xor": "dst[0] = a[0] ^ b[0]", "shl": "dst[0] = a[0] << b[0]",
    "shr": "dst[0] = a[0] >> b[0]", "max": "dst[0] = ops.max(a[0], b[0])", "min": "dst[0] = ops.min(a[0], b[0])",
    "aug": "dst[0] += a[0]",
}
UNOPS = {"cos": "dst[0] = ops.cos(a[0])", "sin": "dst[0] = ops.sin(a[0])", "tanh": "dst[0] = ops.tanh(a[0])",
         "sqrt": "dst[0] = ops.sqrt(a[0])", "exp": "dst[0] = ops.exp(a[0])", "log": "dst[0] = ops.log(a[0])",
         "atan2": "dst[0] = ops.atan2(a[0], b[0])"}
BIN_FUNS = {k: make_fun("op_" + k, v) for k, v in BINOPS.items()}
UN_FUNS = {k: make_fun("op_" + k, v) for k, v in UNOPS.items()}
BITWISE = {"bit_and", "bit_or", "bit_xor", "shl", "shr"}


def expected_failure(op, ty):
    """The type errors of test/test_arith.py:129-141."""
    flt = ty in FLOAT_TYS
    if op in ("floordiv", "rem") and flt:
        return r"Invalid type .* of integer arithmetic operation"
    if op == "pow" and (not flt or ty == np.float16):
        return r"Invalid type .* of floating-point arithmetic operation"
    if op in BITWISE and flt:
        return r"Invalid type .* of bitwise operation"
    return None


def binop_args(ty):
    return [np.zeros(1, dtype=ty), np.array([7], dtype=ty), np.array([3], dtype=ty)]


# ---------------------------------------------------------------- operators x element types (no GPU)
@pytest.mark.parametrize("op", sorted(BINOPS))
def test_binary_operators_type_check(op):
    for ty in INT_TYS + FLOAT_TYS:
        msg = expected_failure(op, ty)
        if msg:
            with pytest.raises(TypeError, match=msg):
                parpy.print_compiled(BIN_FUNS[op], binop_args(ty), opts_for({}))
        else:
            s = parpy.print_compiled(BIN_FUNS[op], binop_args(ty), opts_for({}))
            if ty in (np.int8, np.uint16, np.int64, np.float16, np.float32, np.float64):
                compiles(s)


def test_mixed_width_operands_are_widened():
    for lt, rt in [(np.int8, np.int32), (np.int16, np.int64), (np.uint8, np.uint32), (np.float16, np.float32), (np.float32, np.float64)]:
        compiles(parpy.print_compiled(BIN_FUNS["add"], [np.zeros(1, dtype=rt), np.ones(1, dtype=lt), np.ones(1, dtype=rt)], opts_for({})))
    with pytest.raises(TypeError):   # no implicit conversion between families (src/py/type_check.rs:162-187)
        parpy.print_compiled(BIN_FUNS["add"], [np.zeros(1, dtype=np.float32), np.ones(1, dtype=np.int32), np.ones(1, dtype=np.float32)], opts_for({}))


@pytest.mark.parametrize("op", sorted(UNOPS))
def test_float_functions_type_check(op):
    for ty in FLOAT_TYS:
        compiles(parpy.print_compiled(UN_FUNS[op], binop_args(ty), opts_for({})))
    with pytest.raises(TypeError):
        parpy.print_compiled(UN_FUNS[op], binop_args(np.int32), opts_for({}))


CMP_FUNS = {k: make_fun("cmp_" + k, f"dst[0] = 1 if a[0] {v} b[0] else 0") for k, v in
            {"eq": "==", "neq": "!=", "leq": "<=", "geq": ">=", "lt": "<", "gt": ">"}.items()}


@pytest.mark.parametrize("op", sorted(CMP_FUNS))
def test_comparisons_compile(op):
    for ty in [np.int8, np.int16, np.int32, np.int64, np.float16, np.float32, np.float64]:
        s = parpy.print_compiled(CMP_FUNS[op], [np.zeros(1, dtype=np.int32), np.ones(1, dtype=ty), np.ones(1, dtype=ty)], opts_for({}))
        if ty in (np.int8, np.float16, np.float64):
            compiles(s)


# ---------------------------------------------------------------- booleans, ranges, scalars
def store_lt(x, y, out, N):
    parpy.label('i')
    out[:] = x[:] < y[:]


def reduce_and(x, out):
    with parpy.gpu:
        out[0] = out[0] and x[0]


def range_upper(x, N):
    parpy.label('i')
    for i in range(N):
        x[i] = i


def range_start(x, N):
    parpy.label('i')
    for i in range(1, N):
        x[i] = i


def range_step(x, N):
    parpy.label('i')
    for i in range(1, N, 2):
        x[i] = i


def range_down(x, N):
    parpy.label('i')
    for i in range(N - 1, -1, -1):
        x[i] = i


RANGE_FUNS = [range_upper, range_start, range_step, range_down]


@parpy.jit
def scalar_def(x):
    with parpy.gpu:
        y = x


def test_booleans_and_ranges_compile():
    x = np.zeros(100, dtype=np.float32)
    compiles(parpy.print_compiled(store_lt, [x, x, np.zeros(100, dtype=bool), 100], opts_for({'i': parpy.threads(64)})))
    compiles(parpy.print_compiled(reduce_and, [np.zeros(100, dtype=bool), np.zeros(1, dtype=bool)], opts_for({})))
    for f in RANGE_FUNS:
        compiles(parpy.print_compiled(f, [np.zeros(100, dtype=np.int64), 100], opts_for({'i': parpy.threads(64)})))
    with pytest.raises(RuntimeError, match=r"Range step size must be non-zero"):
        @parpy.jit
        def zero_step(x, N):
            for i in range(0, N, 0):
                x[i] = i


CTYPES = {parpy.ElemSize.I8: "int8_t", parpy.ElemSize.I16: "int16_t", parpy.ElemSize.I32: "int32_t", parpy.ElemSize.I64: "int64_t",
          parpy.ElemSize.U8: "uint8_t", parpy.ElemSize.U16: "uint16_t", parpy.ElemSize.U32: "uint32_t", parpy.ElemSize.U64: "uint64_t",
          parpy.ElemSize.F16: "_Float16", parpy.ElemSize.F32: "float", parpy.ElemSize.F64: "double"}


def test_python_scalars_take_the_default_or_the_forced_size():
    body = lambda s: s.split("extern \"C\" __global__")[1]
    # (a 64-bit integer whose value range is known to fit is otherwise computed in 32 bits)
    assert "int64_t y" in body(parpy.print_compiled(scalar_def, [1], opts_for({}, opt_narrow_index=False)))
    assert "double y" in body(parpy.print_compiled(scalar_def, [1.0], opts_for({})))
    for sz, c in CTYPES.items():
        if sz.is_integer():
            assert f"{c} y" in body(compiles(parpy.print_compiled(scalar_def, [1], opts_for({}, force_int_size=sz, opt_narrow_index=False))))
        else:
            assert f"{c} y" in body(compiles(parpy.print_compiled(scalar_def, [1.0], opts_for({}, force_float_size=sz))))


# ---------------------------------------------------------------- slice statements
def vec_add(x, y, out):
    parpy.label('N')
    out[:] = x[:] + y[:]


def mat_add(x, y, out):
    parpy.label('N')
    parpy.label('M')
    out[:, :] = x[:, :] + y[:, :]


def fill_zero(x):
    parpy.label('N')
    parpy.label('M')
    x[:, :] = 0.0


def sum_all(x, out):
    parpy.label('N')
    out[0] = sum(x[:, :])


def sum_interspersed(x, out):
    parpy.label('N')
    out[0] = sum(x[:, 0, :, 2])


def reduce_in_loop(x, y, N, out):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        out[i] = sum(x[i, :] * y[:, i])


def new_var_slice(x):
    with parpy.gpu:
        y = x[:]


def bad_axis_dims(x, y):
    with parpy.gpu:
        y[:] = sum(x[:, :, :], axis=0)


def bad_shapes(x, y, out):
    with parpy.gpu:
        out[0] = sum(x[:, :] * y[:], axis=0)


def bad_reduce_assign(x, y, z, N):
    parpy.label('N')
    for i in range(N):
        x[i, :] = min(y[i, :] + z[:, i])


def bad_dims(x, y, N):
    parpy.label('N')
    for i in range(N):
        x[i, :] = y[i, :, :]


def slice_in_range(x, y):
    parpy.label('N')
    for i in range(sum(y[:])):
        x[i] = i


def temp_slices(x, y, z):
    parpy.label('N')
    x[:] = (y[1:] + z[:-1])[1:-1]


def T(*shape):
    return np.random.default_rng(sum(shape)).standard_normal(shape).astype(np.float32)


SLICE_OK = [
    (vec_add, lambda: [T(10), T(10), T(10)]), (mat_add, lambda: [T(10, 15), T(10, 15), T(10, 15)]), (fill_zero, lambda: [T(10, 10)]),
    (sum_all, lambda: [T(12, 14), T(1)]), (sum_interspersed, lambda: [T(8, 10, 12, 14), T(1)]),
    (reduce_in_loop, lambda: [T(10, 10), T(10, 10), 10, T(10)]),
]
SLICE_BAD = [
    (new_var_slice, lambda: [T(10)], RuntimeError, r".*Slice statements cannot have more slice dim.*"),
    (bad_axis_dims, lambda: [T(10, 12, 14), T(12)], TypeError, r".*incompatible shapes.*"),
    (bad_shapes, lambda: [T(10, 12), T(10), T(1)], TypeError, r".*incompatible shapes.*"),
    (bad_reduce_assign, lambda: [T(10, 10), T(10, 10), T(10, 10), 10], RuntimeError, r"When reducing along all dimensions,.*"),
    (bad_dims, lambda: [T(10, 10), T(10, 10), 10], TypeError, r"Indexing with 3 dimensions on tensor of shape .*"),
    (slice_in_range, lambda: [T(10), T(10)], RuntimeError, r"Slice expressions are only allowed in assignment.*"),
    (temp_slices, lambda: [T(7), T(10), T(10)], RuntimeError, r"Target of slice must be a variable."),
]
SLICE_PAR = {'N': parpy.threads(64), 'M': parpy.threads(64), 'K': parpy.threads(64)}


@pytest.mark.parametrize("spec", SLICE_OK, ids=lambda s: s[0].__name__)
def test_slice_statements_compile(spec):
    compiles(parpy.print_compiled(spec[0], spec[1](), opts_for(SLICE_PAR)))


@pytest.mark.parametrize("spec", SLICE_BAD, ids=lambda s: s[0].__name__)
def test_invalid_slice_statements_are_rejected(spec):
    with pytest.raises(spec[2], match=spec[3]):
        parpy.print_compiled(spec[0], spec[1](), opts_for(SLICE_PAR))


# ---------------------------------------------------------------- results (GPU): device against the interpreter
@pytest.mark.gpu
@pytest.mark.parametrize("op", sorted(BINOPS))
def test_binary_operators_on_device(op):
    for ty in INT_TYS + FLOAT_TYS:
        if expected_failure(op, ty):
            continue
        want, got = binop_args(ty), binop_args(ty)
        with np.errstate(all="ignore"):
            BIN_FUNS[op](*want)
        parpy.jit(BIN_FUNS[op])(*got, opts=opts_for({}))
        assert np.allclose(got[0].astype(np.float64), want[0].astype(np.float64), atol=1e-5, rtol=1e-3 if ty == np.float16 else 1e-6), (op, ty)


@pytest.mark.gpu
@pytest.mark.parametrize("op", sorted(UNOPS))
def test_float_functions_on_device(op):
    for ty in FLOAT_TYS:
        want = [np.zeros(1, dtype=ty), np.array([0.5], dtype=ty), np.array([0.25], dtype=ty)]
        got = [w.copy() for w in want]
        UN_FUNS[op](*want)
        parpy.jit(UN_FUNS[op])(*got, opts=opts_for({}))
        assert np.allclose(got[0], want[0], atol=2e-3 if ty == np.float16 else 1e-6), (op, ty)


@pytest.mark.gpu
def test_comparisons_booleans_and_ranges_on_device():
    for op, f in CMP_FUNS.items():
        for ty in [np.int8, np.int64, np.float16, np.float32, np.float64]:
            for av, bv in [(3, 3), (2, 5), (5, 2)]:
                want = [np.zeros(1, dtype=np.int32), np.array([av], dtype=ty), np.array([bv], dtype=ty)]
                got = [w.copy() for w in want]
                f(*want)
                parpy.jit(f)(*got, opts=opts_for({}))
                assert got[0][0] == want[0][0], (op, ty, av, bv)
    rng = np.random.default_rng(4)
    x, y = rng.standard_normal(100).astype(np.float32), rng.standard_normal(100).astype(np.float32)
    flags = np.zeros(100, dtype=bool)
    parpy.jit(store_lt)(x, y, flags, 100, opts=opts_for({'i': parpy.threads(100)}))
    assert np.array_equal(flags, x < y)
    out = np.ones(1, dtype=bool)
    parpy.jit(reduce_and)(flags, out, opts=opts_for({}))
    assert out[0] == (True and flags[0])
    for f in RANGE_FUNS:
        want, got = np.zeros(100, dtype=np.int64), np.zeros(100, dtype=np.int64)
        f(want, 100)
        parpy.jit(f)(got, 100, opts=opts_for({'i': parpy.threads(64)}))
        assert np.array_equal(got, want), f.__name__


@pytest.mark.gpu
@pytest.mark.parametrize("spec", SLICE_OK, ids=lambda s: s[0].__name__)
def test_slice_statements_on_device(spec):
    want, got = spec[1](), spec[1]()
    spec[0](*want)
    parpy.jit(spec[0])(*got, opts=opts_for(SLICE_PAR))
    assert np.allclose(got[-1], want[-1], atol=1e-4)


# ---------------------------------------------------------------- constructs rejected when the function is parsed
def test_unsupported_statements_report_their_lines():
    """test/test_unsupported.py of the reference: the message names the lines of the offending statement."""
    import inspect
    here = inspect.currentframe().f_lineno
    with pytest.raises(RuntimeError, match=rf"lines {here + 5}-{here + 9}"):
        @parpy.jit
        def while_else(x, y, N):
            i = 0
            while i < N:
                y[i] = x[i]
                i += 1
            else:
                y[i] = 0.0
    here = inspect.currentframe().f_lineno
    with pytest.raises(RuntimeError, match=rf"lines {here + 4}-{here + 7}"):
        @parpy.jit
        def for_else(x, y, N):
            for i in range(N):
                y[i] = x[i]
            else:
                y[0] += 1
    here = inspect.currentframe().f_lineno
    with pytest.raises(RuntimeError, match=rf"lines {here + 4}-{here + 5}"):
        @parpy.jit
        def with_context():
            with 5:
                pass
    here = inspect.currentframe().f_lineno
    with pytest.raises(RuntimeError, match=rf"lines {here + 4}-{here + 5}"):
        @parpy.jit
        def with_as():
            with parpy.gpu as x:
                a = x + 1
    with pytest.raises(RuntimeError, match=r"Empty return statements are not supported"):
        @parpy.jit
        def empty_return():
            return


def test_entry_function_rules():
    @parpy.jit
    def dict_arg(a):
        with parpy.gpu:
            a["x"] = a["y"]
    # (without a GPU the call stops at backend resolution, as in the reference's own test)
    with pytest.raises(RuntimeError, match=r"(.*non-string key.*)|(.*backend.*not available.*)"):
        dict_arg({'x': 2, 'y': 4, 3: 5}, opts=opts_for({}))
    o = parpy.CompileOptions()
    with pytest.raises(RuntimeError, match=r".*number of thread blocks per cluster must be a power of two.*"):
        o.max_thread_blocks_per_cluster = 3

    @parpy.jit
    def f_return(x):
        with parpy.gpu:
            y = sum(x[:])
            return y
    with pytest.raises(RuntimeError, match=r"The called function f_return cannot return a value"):
        parpy.print_compiled(f_return, [np.ndarray(10)], opts_for({}))

    @parpy.jit
    def fun_with_args(x, y):
        with parpy.gpu:
            x[:] += y[:]
    with pytest.raises(RuntimeError, match="Missing required keyword argument opts in call to fun_with_args"):
        fun_with_args(np.ndarray((10,), dtype=np.float32), np.ndarray((10,), dtype=np.float32))


# ---------------------------------------------------------------- random expression trees: device against the interpreter
def _random_expr(rng, depth, kind):
    # `//` and `%` get non-negative operands: they compile to C's truncating operators, which agree
    # with Python's flooring ones only there (src/cuda/pprint.rs:146-147 of the reference does the same)
    leaves = ["a[i]", "b[i]", "c[i]"] + (["0.5", "2.0", "1.25"] if kind == "f" else ["3", "7", "2"])
    if depth == 0 or rng.random() < 0.2:
        return str(rng.choice(leaves))
    x, y = _random_expr(rng, depth - 1, kind), _random_expr(rng, depth - 1, kind)
    if kind == "f":
        forms = ["({x} + {y})", "({x} - {y})", "({x} * {y})", "({x} / (abs({y}) + 1.0))", "ops.max({x}, {y})", "ops.min({x}, {y})",
                 "abs({x})", "(-{x})", "ops.exp(ops.min({x}, 2.0))", "ops.sqrt(abs({x}))", "({x} if {x} < {y} else {y})",
                 "ops.tanh({x})", "ops.log(abs({x}) + 1.0)"]
    else:
        forms = ["({x} + {y})", "({x} - {y})", "({x} * {y})", "(abs({x}) // (abs({y}) + 1))", "(abs({x}) % (abs({y}) + 1))", "({x} & {y})",
                 "({x} | {y})", "({x} ^ {y})", "ops.max({x}, {y})", "ops.min({x}, {y})", "abs({x})", "(-{x})",
                 "({x} if {x} <= {y} else {y})", "(({x} & 7) << 2)", "(abs({x}) >> 1)"]
    return str(rng.choice(forms)).format(x=x, y=y)


def _loop_fun(name, expr):
    src = f"def {name}(out, a, b, c, N):\n    parpy.label('N')\n    for i in range(N):\n        out[i] = {expr}\n"
    fname = f"<{name}>"
    linecache.cache[fname] = (len(src), None, src.splitlines(True), fname)
    ns = {"parpy": parpy, "ops": ops}
    exec(compile(src, fname, "exec"), ns)
    return ns[name]


@pytest.mark.gpu
@pytest.mark.parametrize("kind,dtype", [("f", np.float32), ("f", np.float64), ("i", np.int32), ("i", np.int64)], ids=["f32", "f64", "i32", "i64"])
def test_random_expressions_on_device(kind, dtype):
    rng = np.random.default_rng(31)
    N = 96
    for case in range(25):
        expr = _random_expr(rng, 4, kind)
        f = _loop_fun(f"expr_{kind}_{case}", expr)
        if kind == "f":
            args = [rng.uniform(-2, 2, N).astype(dtype) for _ in range(3)]
        else:
            args = [rng.integers(-20, 20, N).astype(dtype) for _ in range(3)]
        want, got = np.zeros(N, dtype=dtype), np.zeros(N, dtype=dtype)
        with np.errstate(all="ignore"):
            f(want, *args, N)
        parpy.jit(f)(got, *args, N, opts=opts_for({'N': parpy.threads(N)}))
        if kind == "f":
            ok = np.allclose(got, want, rtol=2e-5 if dtype == np.float32 else 1e-12, atol=1e-6 if dtype == np.float32 else 1e-13, equal_nan=True)
        else:
            ok = np.array_equal(got, want)
        assert ok, (expr, got[:4], want[:4])


# ---------------------------------------------------------------- branches that only pick values
def pick_values(x, y, out, N):
    parpy.label('N')
    for i in range(N):
        a = ops.float32(0.0)
        k = 0
        if x[i] > 0.5:
            a = x[i] * 2.0
            k = i % 7
        elif y[i] < 0.0:
            a = ops.float32(-1.0)
        else:
            k = i // 3
        b = ops.float32(1.0)
        if y[i] > 0.25:            # one-sided: b keeps its value otherwise
            b = ops.float32(3.0)
        out[i] = a + b + ops.float32(k)


def test_branches_that_only_assign_scalars_become_selects():
    N = 256
    x, y, out = np.zeros(N, dtype=np.float32), np.zeros(N, dtype=np.int32), np.zeros(N, dtype=np.float32)
    on = compiles(parpy.print_compiled(pick_values, [x, y.astype(np.float32), out, N], opts_for({'N': parpy.threads(N)})))
    off = compiles(parpy.print_compiled(pick_values, [x, y.astype(np.float32), out, N], opts_for({'N': parpy.threads(N)}, opt_if_convert=False)))
    body = lambda s: s.split('extern "C" __global__')[1]
    # the branch that loads x[i] in its value stays a branch (a load is not free to do either way); the others go
    assert body(off).count("if (") - body(on).count("if (") >= 2 and " ? " in body(on)


@pytest.mark.gpu
def test_branches_that_only_assign_scalars_keep_their_meaning_as_selects():
    rng = np.random.default_rng(12)
    N = 1000
    x, y = rng.uniform(0, 1, N).astype(np.float32), rng.uniform(-1, 1, N).astype(np.float32)
    want = np.zeros(N, dtype=np.float32)
    pick_values(x, y, want, N)
    for flag in (True, False):
        got = np.zeros(N, dtype=np.float32)
        parpy.jit(pick_values)(x, y, got, N, opts=opts_for({'N': parpy.threads(N)}, opt_if_convert=flag))
        assert np.allclose(got, want, rtol=1e-6), flag


def relax(x, y, N, M, T):
    parpy.label('N')
    for i in range(N):
        for t in range(T):
            parpy.label('M')
            for j in range(M):
                w = ops.float32(0.5)
                k = j
                if j % 3 == 0:
                    w = ops.float32(2.0)
                    k = (j + 5) % M
                elif j % 3 == 1:
                    w = ops.float32(-1.0)
                y[i, j] = w * x[i, k] + ops.float32(t)
            parpy.label('M')
            for j in range(M):
                x[i, j] = y[i, j] * ops.float32(0.5)


def test_selects_on_the_iteration_alone_leave_the_time_loop():
    N, M, T = 4, 256, 3
    x = np.zeros((N, M), dtype=np.float32)
    s = compiles(parpy.print_compiled(relax, [x, x.copy(), N, M, T], opts_for({'N': parpy.threads(N), 'M': parpy.threads(64)})))
    body = s.split('extern "C" __global__')[1]
    loop = body[body.index("for (int t_"):]
    assert "inv_pick_" in body and " ? " not in loop[:loop.index("__syncthreads")]


@pytest.mark.gpu
@pytest.mark.parametrize("threads", [64, 100, 256])
def test_selects_on_the_iteration_alone_keep_their_values(threads):
    rng = np.random.default_rng(3)
    N, M, T = 5, 300, 4
    x0 = rng.uniform(-1, 1, (N, M)).astype(np.float32)
    want_x, want_y = x0.copy(), np.zeros_like(x0)
    relax(want_x, want_y, N, M, T)
    for flags in ({}, {"opt_if_convert": False}, {"opt_hoist_invariant": False}):
        got_x, got_y = x0.copy(), np.zeros_like(x0)
        parpy.jit(relax)(got_x, got_y, N, M, T, opts=opts_for({'N': parpy.threads(N), 'M': parpy.threads(threads)}, **flags))
        assert np.allclose(got_x, want_x, rtol=1e-5, atol=1e-6) and np.allclose(got_y, want_y, rtol=1e-5, atol=1e-6), flags


def test_rejections_the_reference_tests_for_contexts_dictionaries_returns_and_calls():
    """test/test_unsupported.py:33-67,82-95 and test/test_call.py:97-137,207-223 of the reference: same exception
    type and the same words in the message."""
    import parpy_amd.types as types

    with pytest.raises(RuntimeError, match=r"lines \d+-\d+"):
        @parpy.jit
        def with_context():
            with 5:
                pass

    @parpy.jit
    def dict_arg(a):
        with parpy.gpu:
            a["x"] = a["y"]
    with pytest.raises(RuntimeError, match="non-string key"):
        parpy.print_compiled(dict_arg, [{'x': 2, 'y': 4, 3: 5}], opts_for({}))

    @parpy.jit
    def f_return(x):
        with parpy.gpu:
            y = parpy.operators.sum(x[:])
            return y
    with pytest.raises(RuntimeError, match="The called function f_return cannot return a value"):
        parpy.print_compiled(f_return, [np.zeros(10)], opts_for({}))

    def non_decorated_add(x, y, M):
        for i in range(M):
            y[i] += x[i]
    with pytest.raises(RuntimeError, match="unknown function non_decorated_add"):
        @parpy.jit
        def add_2d(x, y, N, M):
            parpy.label('N')
            for i in range(N):
                non_decorated_add(x[i], y[i], M)

    @parpy.external("_zero", parpy.CompileBackend.Cuda, parpy.Target.Device)
    def zero() -> types.I32:
        return 0

    @parpy.jit
    def uses_zero(x):
        with parpy.gpu:
            x[:] = zero()
    with pytest.raises(RuntimeError, match="Call to unknown function zero"):
        parpy.print_compiled(uses_zero, [np.zeros(10, dtype=np.int32)], opts_for({}))

    @parpy.jit
    def needs_opts(x):
        with parpy.gpu:
            x[0] = 1.0
    with pytest.raises(RuntimeError, match="opts"):
        needs_opts(np.zeros(4, dtype=np.float32))
