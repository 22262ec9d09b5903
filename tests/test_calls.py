"""Calls between jitted functions and calls of external device functions
(test/test_call.py, test/test_cuda.py:113-225 of the reference, re-targeted to HIP;
the external targets live in tests/code/hip_utils.h)."""
import os

import re

import numpy as np
import pytest

import parpy_amd as parpy
import parpy_amd.types as types
from parpy_amd.compile import hiprtc_compile

HIP = parpy.CompileBackend.Hip
CODE_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "code")


def opts_for(p, **kw):
    o = parpy.par(p)
    o.backend = HIP
    o.includes += [CODE_DIR]
    for k, v in kw.items():
        setattr(o, k, v)
    return o


def compiles(s, o=None):
    hiprtc_compile(s[:s.index("// host side")], o or opts_for({}))
    return s


# ---------------------------------------------------------------- jitted callees
@parpy.jit
def add_call(x: types.F32, y: types.F32):
    return x + y


@parpy.jit
def mul_call(x: types.F32, y: types.F32):
    return x * y


@parpy.jit
def add_then_mul(x: types.F32, y: types.F32, z: types.F32):
    return mul_call(add_call(x, y), z)


@parpy.jit
def scaled_square(x: types.F32, s: types.F32):
    t = x * x
    u = t * s
    return u + t


@parpy.jit
def add_direct(x, y, N):
    parpy.label('N')
    y[:] = add_call(x[:], y[:])


@parpy.jit
def add_mul_nested(x, y, N):
    parpy.label('N')
    y[:] = add_then_mul(x[:], y[:], x[:])


@parpy.jit
def with_locals(x, y, N):
    parpy.label('N')
    for i in range(N):
        y[i] = scaled_square(x[i], 0.5)


@parpy.jit
def add_inplace(x, y, M):
    parpy.label("1d")
    y[:] += x[:]


@parpy.jit
def add_2d_inplace(x, y, N, M):
    parpy.label("2d")
    for i in range(N):
        add_inplace(x[i], y[i], M)


@parpy.jit
def add_2d_inplace_x2(x, y, z, w, N, M):
    parpy.label("2d")
    for i in range(N):
        add_inplace(x[i], y[i], M)
        add_inplace(z[i], w[i], M)


@parpy.jit
def add_3d_inplace(x, y, N, M, K):
    parpy.label('3d')
    for i in range(N):
        add_2d_inplace(x[i], y[i], M, K)


# ---------------------------------------------------------------- externals
@parpy.external("sqrtf", HIP, parpy.Target.Device)
def sqrt_ext(x: types.F32) -> types.F32:
    return np.sqrt(x)


@parpy.external("clamp", HIP, parpy.Target.Device, header="<hip_utils.h>")
def clamp(x: types.F32, lo: types.F32, hi: types.F32) -> types.F32:
    return min(max(x, lo), hi)


@parpy.external("sum_row_ext", HIP, parpy.Target.Device, header="<hip_utils.h>")
def sum_row(x: types.pointer(types.F64), n: types.I64) -> types.F64:
    return np.sum(x[:n])


@parpy.external("wave_sum", HIP, parpy.Target.Device, header="<hip_utils.h>", parallelize=parpy.threads(64))
def wave_sum_custom(x: types.pointer(types.F32)) -> types.F32:
    return np.sum(x)


@parpy.external("_zero", parpy.CompileBackend.Cuda, parpy.Target.Device)
def zero_for_cuda() -> types.I32:
    return 0


@parpy.jit
def ext_sqrt(x, y):
    with parpy.gpu:
        y[0] = sqrt_ext(x)


@parpy.jit
def clamp_many(out, x):
    parpy.label('N')
    out[:] = clamp(x[:], 0.0, 10.0)


@parpy.jit
def sum_ext_seq(x, y, N, M):
    parpy.label('N')
    for i in range(N):
        y[i] = sum_row(x[i], M)


@parpy.jit
def sum_rows_using_ext(out, x, N):
    parpy.label('N')
    for i in range(N):
        out[i] = wave_sum_custom(x[i])


# callees with more than one return statement (the reference keeps them as device functions,
# src/py/insert_called_functions.rs:12-88; here they are inlined with the returned value in a variable unless the
# device_functions option asks for functions)
@parpy.jit
def clamp_between(x, lo, hi):
    if x < lo:
        return lo
    if x > hi:
        return hi
    return x


@parpy.jit
def piecewise(x, y):
    t = x * y
    if t > 1.0:
        u = t - 1.0
        return u * u
    elif t < -1.0:
        return -t
    v = t + 2.0
    return v


@parpy.jit
def sign_of(x):
    if x > 0.0:
        return 1
    else:
        if x < 0.0:
            return -1
        else:
            return 0


@parpy.jit
def early_returns(x, y, sgn, N):
    parpy.label('N')
    for i in range(N):
        y[i] = clamp_between(x[i], parpy.operators.float32(-1.0), parpy.operators.float32(2.0)) + piecewise(x[i], y[i])
        sgn[i] = sign_of(x[i])


# callees that only work as functions of their own: a return inside a loop, a loop of data-dependent length
@parpy.jit
def first_at_least(x: types.F32):
    for k in range(4):
        if x <= parpy.operators.float32(k):
            return k
    return 4


@parpy.jit
def halvings(n):
    c = 0
    while n > 1:
        n2 = n // 2
        c = c + 1
        if n2 * 2 != n:
            return -c
        n = n2
    return c


@parpy.jit
def add_any(a, b):
    return a + b


@parpy.jit
def second_of(x, i):
    return x[i + 1]


@parpy.jit
def function_calls(x, y, steps, idx, N):
    parpy.label('N')
    for i in range(N):
        y[i] = parpy.operators.float32(first_at_least(x[i])) + add_any(x[i], y[i])
        steps[i] = add_any(halvings(idx[i]), 1)


@parpy.jit
def mixed_callees(x, y, N):
    parpy.label('N')
    for i in range(N - 1):
        y[i] = second_of(x, i) + add_call(x[i], 1.0)


F = np.float32


# ---------------------------------------------------------------- code generation (no GPU)
def test_expression_calls_are_inlined():
    x = np.zeros(10, dtype=F)
    s = compiles(parpy.print_compiled(add_direct, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)})))
    assert "add_call" not in s.split("extern \"C\" __global__")[1]
    compiles(parpy.print_compiled(add_mul_nested, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)})))
    compiles(parpy.print_compiled(with_locals, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)})))


def test_callees_with_several_returns_are_inlined_through_a_result_variable():
    x = np.zeros(10, dtype=F)
    s = compiles(parpy.print_compiled(early_returns, [x, x.copy(), np.zeros(10, dtype=np.int64), 10], opts_for({'N': parpy.threads(10)})))
    assert re.search(r"float clamp_between_result_\d+ = 0.0f;", s) and re.search(r"int64_t sign_of_result_\d+ = 0;", s)
    # a callee that returns from inside a loop cannot be inlined this way: accepted when it is declared (it compiles as
    # a device function), reported when the caller is compiled with inlined calls
    @parpy.jit
    def first_positive(x: types.F32):
        for k in range(3):
            if x > parpy.operators.float32(k):
                return k
        return 3

    @parpy.jit
    def use(x, y, N):
        parpy.label('N')
        for i in range(N):
            y[i] = parpy.operators.float32(first_positive(x[i]))
    with pytest.raises(RuntimeError, match="return statement inside a loop"):
        parpy.print_compiled(use, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)}))
    compiles(parpy.print_compiled(use, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)}, device_functions=True)))
    with pytest.raises(TypeError, match="Unknown return type"):
        @parpy.jit
        def maybe(x: types.F32):
            if x > 0.0:
                return x

        @parpy.jit
        def use2(x, y, N):
            parpy.label('N')
            for i in range(N):
                y[i] = maybe(x[i])


def test_expression_calls_as_device_functions():
    """`device_functions`: what the reference does with functions called inside expressions
    (src/py/insert_called_functions.rs:12-88, src/gpu/codegen.rs:573-585).  A callee becomes a `__device__` function
    once per combination of argument types, callees in front of their callers; a callee that indexes a parameter is
    inlined as before; statement calls are inlined in both modes."""
    x = np.zeros(10, dtype=F)
    dev = lambda p: opts_for(p, device_functions=True)
    s = compiles(parpy.print_compiled(add_mul_nested, [x, x.copy(), 10], dev({'N': parpy.threads(10)})))
    heads = re.findall(r"__device__ __forceinline__ float (\w+)_fn\d+\(float \w+, float \w+(?:, float \w+)?\)", s)
    assert heads[-1] == "add_then_mul" and sorted(heads[:-1]) == ["add_call", "mul_call"], heads
    assert re.search(r"= add_then_mul_fn\d+\(", s.split('extern "C" __global__')[1])
    s = compiles(parpy.print_compiled(early_returns, [x, x.copy(), np.zeros(10, dtype=np.int64), 10], dev({'N': parpy.threads(10)})))
    assert "clamp_between_result" not in s and re.search(r"__device__ __forceinline__ int64_t sign_of_fn\d+\(float", s)
    assert len(re.findall(r"\n    return ", s[s.index("clamp_between_fn"):s.index("piecewise_fn")])) >= 2
    # a return inside a loop, a while loop with an early return; two instances of one callee for two argument types
    idx = np.arange(10, dtype=np.int64)
    s = compiles(parpy.print_compiled(function_calls, [x, x.copy(), np.zeros(10, dtype=np.int64), idx, 10], dev({'N': parpy.threads(10)})))
    assert re.search(r"float add_any_fn\d+\(float \w+, float \w+\)", s) and re.search(r"int64_t add_any_fn\d+\(int64_t \w+, int64_t \w+\)", s)
    assert "while (" in s[s.index("halvings_fn"):s.index('extern "C" __global__')]
    with pytest.raises(RuntimeError, match="return statement inside a loop"):
        parpy.print_compiled(function_calls, [x, x.copy(), np.zeros(10, dtype=np.int64), idx, 10], opts_for({'N': parpy.threads(10)}))
    # a callee that indexes its parameter is inlined, the scalar one beside it is a function
    s = compiles(parpy.print_compiled(mixed_callees, [x, x.copy(), 10], dev({'N': parpy.threads(10)})))
    assert "second_of" not in s and re.search(r"float add_call_fn\d+\(", s)
    # statement calls are inlined in both modes
    a = np.zeros((10, 15), dtype=F)
    s = compiles(parpy.print_compiled(add_2d_inplace, [a, a.copy(), 10, 15], dev({'2d': parpy.threads(10), '1d': parpy.threads(15)})))
    assert "__device__ __forceinline__ float add" not in s
    # without the option nothing changes
    s = parpy.print_compiled(add_mul_nested, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)}))
    assert "_fn1" not in s
    with pytest.raises(TypeError, match="takes scalars"):
        @parpy.jit
        def whole(x, y, N):
            parpy.label('N')
            for i in range(N):
                y[i] = add_any(x, y[i])
        parpy.print_compiled(whole, [x, x.copy(), 10], dev({'N': parpy.threads(10)}))


def test_statement_calls_with_sub_tensors():
    a2, a3 = np.zeros((10, 15), dtype=F), np.zeros((10, 20, 30), dtype=F)
    compiles(parpy.print_compiled(add_2d_inplace, [a2, a2.copy(), 10, 15], opts_for({'2d': parpy.threads(10), '1d': parpy.threads(15)})))
    compiles(parpy.print_compiled(add_3d_inplace, [a3, a3.copy(), 10, 20, 30],
                                  opts_for({'3d': parpy.threads(10), '2d': parpy.threads(20), '1d': parpy.threads(30)})))
    z = np.zeros((10, 15), dtype=np.int32)
    compiles(parpy.print_compiled(add_2d_inplace_x2, [a2, a2.copy(), z, z.copy(), 10, 15],
                                  opts_for({'2d': parpy.threads(10), '1d': parpy.threads(15)})))


def test_unknown_and_recursive_callees_are_rejected():
    def plain(x, y, M):
        for i in range(M):
            y[i] += x[i]
    with pytest.raises(RuntimeError, match=r".*unknown function plain.*"):
        @parpy.jit
        def add_2d(x, y, N, M):
            parpy.label('N')
            for i in range(N):
                plain(x[i], y[i], M)
    with pytest.raises(RuntimeError, match=r".*unknown function reset.*"):
        @parpy.jit
        def reset(x, i):
            with parpy.gpu:
                if i > 0:
                    x[i] = 0.0
                    reset(x, i - 1)


def test_external_declarations_are_validated():
    assert "sqrt_ext" in parpy._ext_decls[HIP]
    with pytest.raises(RuntimeError, match="Unsupported parameter type annotation"):
        @parpy.external("dummy", HIP, parpy.Target.Device)
        def dummy(x: int) -> types.I32:
            return x
    with pytest.raises(RuntimeError, match="Unsupported return type annotation on external function"):
        @parpy.external("dummy", HIP, parpy.Target.Device)
        def dummy2(x: types.I32) -> int:
            return x
    with pytest.raises(RuntimeError, match="Host externals are not supported"):
        @parpy.external("dummy", HIP, parpy.Target.Host)
        def dummy3(x: types.I64) -> types.I64:
            return x


def test_external_calls_compile():
    s = compiles(parpy.print_compiled(ext_sqrt, [F(2.0), np.zeros(1, dtype=F)], opts_for({})))
    assert "sqrtf(" in s
    x = np.zeros(10, dtype=F)
    o = opts_for({'N': parpy.threads(10)})
    s = compiles(parpy.print_compiled(clamp_many, [x.copy(), x], o), o)
    assert "#include <hip_utils.h>" in s and re.search(r"clamp\((x_|parpy_at\(x_)", s)
    s = compiles(parpy.print_compiled(sum_ext_seq, [np.zeros((10, 20)), np.zeros(10), 10, 20], o), o)
    assert re.search(r"sum_row_ext\(\(&(x_|parpy_at\(x_)", s) and "const double* __restrict__ x_" not in s   # the external may write through its pointer
    s = compiles(parpy.print_compiled(sum_rows_using_ext, [x.copy(), np.zeros((10, 64), dtype=F), 10], o), o)
    # one workgroup of 64 threads per row makes the call; one thread stores the result
    assert "<<<dim3(1, 10, 1), dim3(64, 1, 1)" in s and "threadIdx.x == 0" in s


def test_external_misuse_is_rejected():
    with pytest.raises(RuntimeError, match=r"Call to unknown function zero_for_cuda.*"):
        @parpy.jit
        def f(x):
            with parpy.gpu:
                x[:] = zero_for_cuda()
        parpy.print_compiled(f, [np.zeros(10, dtype=np.int32)], opts_for({}))
    with pytest.raises(TypeError, match="incompatible types"):
        @parpy.jit
        def g(out, x, y):
            with parpy.gpu:
                out[0] = sum_row(x, 10) + sum_row(y, 20)
        parpy.print_compiled(g, [np.zeros(1), np.zeros(10), np.zeros(20)], opts_for({}))

    @parpy.external("clamp_non_existent", HIP, parpy.Target.Device, header="<hip_utils.h>")
    def clamp_missing(x: types.F32, lo: types.F32, hi: types.F32) -> types.F32:
        return x

    @parpy.jit
    def h(out, x):
        parpy.label('N')
        out[:] = clamp_missing(x[:], 0.0, 10.0)
    o = opts_for({'N': parpy.threads(10)})
    s = parpy.print_compiled(h, [np.zeros(10, dtype=F), np.zeros(10, dtype=F)], o)
    with pytest.raises(RuntimeError, match="Compilation of generated HIP code failed"):
        compiles(s, o)


# ---------------------------------------------------------------- results (GPU)
@pytest.mark.gpu
def test_calls_give_the_results_of_the_inlined_code():
    rng = np.random.default_rng(11)
    x = rng.standard_normal(10).astype(F)
    y = np.zeros_like(x)
    add_direct(x, y, 10, opts=opts_for({'N': parpy.threads(10)}))
    assert np.array_equal(x, y)
    y = np.zeros_like(x)
    add_mul_nested(x, y, 10, opts=opts_for({'N': parpy.threads(10)}))
    assert np.allclose(x ** 2, y)
    y = np.zeros_like(x)
    with_locals(x, y, 10, opts=opts_for({'N': parpy.threads(10)}))
    assert np.allclose(y, 1.5 * x * x)
    a, b = rng.standard_normal((10, 15)).astype(F), np.zeros((10, 15), dtype=F)
    add_2d_inplace(a, b, 10, 15, opts=opts_for({'2d': parpy.threads(10), '1d': parpy.threads(15)}))
    assert np.array_equal(a, b)
    z, w = rng.integers(0, 10, (10, 15)).astype(np.int32), np.zeros((10, 15), dtype=np.int32)
    b[:] = 0
    add_2d_inplace_x2(a, b, z, w, 10, 15, opts=opts_for({'2d': parpy.threads(10), '1d': parpy.threads(15)}))
    assert np.array_equal(a, b) and np.array_equal(z, w)
    a3, b3 = rng.standard_normal((10, 20, 30)).astype(F), np.zeros((10, 20, 30), dtype=F)
    add_3d_inplace(a3, b3, 10, 20, 30, opts=opts_for({'3d': parpy.threads(10), '2d': parpy.threads(20), '1d': parpy.threads(30)}))
    assert np.array_equal(a3, b3)


@pytest.mark.gpu
def test_callees_with_several_returns_give_what_python_gives():
    rng = np.random.default_rng(13)
    x = (3.0 * rng.standard_normal(500)).astype(F)
    y0 = rng.standard_normal(500).astype(F)
    y, sgn = y0.copy(), np.zeros(500, dtype=np.int64)
    early_returns(x, y, sgn, 500, opts=opts_for({'N': parpy.threads(500)}))
    t = x.astype(np.float64) * y0
    pw = np.where(t > 1.0, (t - 1.0) ** 2, np.where(t < -1.0, -t, t + 2.0))
    want = np.clip(x, -1.0, 2.0) + pw
    assert np.allclose(y, want, rtol=1e-6, atol=1e-6)
    assert np.array_equal(sgn, np.sign(x).astype(np.int64))


@pytest.mark.gpu
def test_device_functions_give_the_results_of_the_inlined_code():
    rng = np.random.default_rng(17)
    dev = lambda p: opts_for(p, device_functions=True)
    x = rng.standard_normal(10).astype(F)
    y = np.zeros_like(x)
    add_mul_nested(x, y, 10, opts=dev({'N': parpy.threads(10)}))
    assert np.allclose(x ** 2, y)
    y = np.zeros_like(x)
    with_locals(x, y, 10, opts=dev({'N': parpy.threads(10)}))
    assert np.allclose(y, 1.5 * x * x)
    x = (3.0 * rng.standard_normal(500)).astype(F)
    y0 = rng.standard_normal(500).astype(F)
    outs = []
    for o in (opts_for({'N': parpy.threads(500)}), dev({'N': parpy.threads(500)})):
        y, sgn = y0.copy(), np.zeros(500, dtype=np.int64)
        early_returns(x, y, sgn, 500, opts=o)
        outs.append((y, sgn))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][1], outs[1][1])
    # callees that exist only as functions, against the same steps in NumPy / plain Python
    idx = rng.integers(1, 5000, 500).astype(np.int64)
    idx[:12] = 2 ** np.arange(12)
    y, steps = y0.copy(), np.zeros(500, dtype=np.int64)
    function_calls(x, y, steps, idx, 500, opts=dev({'N': parpy.threads(500)}))
    first = np.where(x <= 0, 0, np.where(x <= 1, 1, np.where(x <= 2, 2, np.where(x <= 3, 3, 4))))
    assert np.allclose(y, first + (x + y0), rtol=1e-6, atol=1e-6)
    def halv(n):
        c = 0
        while n > 1:
            n2 = n // 2
            c += 1
            if n2 * 2 != n:
                return -c
            n = n2
        return c
    assert np.array_equal(steps, np.array([halv(int(n)) + 1 for n in idx]))
    y = np.zeros(10, dtype=F)
    xs = rng.standard_normal(10).astype(F)
    mixed_callees(xs, y, 10, opts=dev({'N': parpy.threads(10)}))
    assert np.allclose(y[:9], xs[1:] + (xs[:9] + 1.0))


@pytest.mark.gpu
def test_externals_run():
    rng = np.random.default_rng(12)
    y = np.zeros(1, dtype=F)
    ext_sqrt(F(2.0), y, opts=opts_for({}))
    assert np.allclose(y, np.sqrt(F(2.0)))
    x = (rng.standard_normal(10) * 10).astype(F)
    out = np.zeros_like(x)
    clamp_many(out, x, opts=opts_for({'N': parpy.threads(10)}))
    assert np.array_equal(out, np.clip(x, 0.0, 10.0))
    xd, yd = rng.standard_normal((10, 20)), np.zeros(10)
    sum_ext_seq(xd, yd, 10, 20, opts=opts_for({'N': parpy.threads(10)}))
    assert np.allclose(yd, xd.sum(axis=1))
    xf, of = rng.standard_normal((10, 64)).astype(F), np.zeros(10, dtype=F)
    sum_rows_using_ext(of, xf, 10, opts=opts_for({'N': parpy.threads(10)}))
    assert np.allclose(of, xf.sum(axis=1), atol=1e-5)


def test_device_functions_of_one_name_with_different_bodies_stay_apart():
    """A callee redefined after one of its callers was declared: the earlier caller keeps the earlier body, and both
    bodies become functions of their own."""
    @parpy.jit
    def twice(x: types.F32):
        return x + x

    @parpy.jit
    def uses_first(x: types.F32):
        return twice(x) + 1.0

    @parpy.jit
    def twice(x: types.F32):      # noqa: F811  (the redefinition is the point)
        return x * 3.0

    @parpy.jit
    def both(x, y, N):
        parpy.label('N')
        for i in range(N):
            y[i] = uses_first(x[i]) + twice(x[i])
    x = np.zeros(10, dtype=F)
    s = compiles(parpy.print_compiled(both, [x, x.copy(), 10], opts_for({'N': parpy.threads(10)}, device_functions=True)))
    bodies = re.findall(r"(?:float|double) twice_fn\d+\(float (\w+)\) \{\n\s+return \((.*?)\);", s)
    assert len(bodies) == 2 and any("+" in b[1] for b in bodies) and any("* 3.0" in b[1] for b in bodies), s[s.index("__device__ __forceinline__ float twice"):][:600]
