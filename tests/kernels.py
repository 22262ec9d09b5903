"""ParPy user functions shared by the CPU (code generation) and GPU (parity) tests.

They restate the reference's test inputs for reductions over rows, axes and
whole tensors (test/test_reduce.py:12-70), strided reductions (:285-293) and a
few element-wise / dictionary / control-flow shapes from its other tests.
"""
import parpy_amd as parpy
from parpy_amd.operators import sum, prod, max, min, exp, log, float32, int32


def sum_rows(x, out, N):
    parpy.label('outer')
    for i in range(N):
        parpy.label('inner')
        out[i] = sum(x[i, :])


def prod_rows(x, out, N):
    parpy.label('outer')
    for i in range(N):
        parpy.label('inner')
        out[i] = prod(x[i, :])


def max_rows(x, out, N):
    parpy.label('outer')
    for i in range(N):
        parpy.label('inner')
        out[i] = max(x[i, :])


def min_rows(x, out, N):
    parpy.label('outer')
    for i in range(N):
        parpy.label('inner')
        out[i] = min(x[i, :])


def sum_axis(x, out, N):
    parpy.label('outer')
    parpy.label('inner')
    out[:] = sum(x[:, :], axis=1)


def prod_axis(x, out, N):
    parpy.label('outer')
    parpy.label('inner')
    out[:] = prod(x[:, :], axis=1)


def max_axis(x, out, N):
    parpy.label('outer')
    parpy.label('inner')
    out[:] = max(x[:, :], axis=1)


def min_axis(x, out, N):
    parpy.label('outer')
    parpy.label('inner')
    out[:] = min(x[:, :], axis=1)


def sum_2d(x, out, N):
    parpy.label('outer')
    out[0] = sum(x[:, :])


def prod_2d(x, out, N):
    parpy.label('outer')
    out[0] = prod(x[:, :])


def max_2d(x, out, N):
    parpy.label('outer')
    out[0] = max(x[:, :])


def min_2d(x, out, N):
    parpy.label('outer')
    out[0] = min(x[:, :])


ROW_REDUCTIONS = [sum_rows, prod_rows, max_rows, min_rows, sum_axis, prod_axis, max_axis, min_axis]
FULL_REDUCTIONS = [sum_2d, prod_2d, max_2d, min_2d]
NUMPY_OP = {"sum": "sum", "prod": "prod", "max": "max", "min": "min"}


def odd_entries_sum(x, y, N, M):
    parpy.label('N')
    for i in range(N):
        y[i] = 0.0
        parpy.label('M')
        for j in range(1, M, 2):
            y[i] += x[i, j]


def axpy(a, x, y, out, N):
    parpy.label('N')
    for i in range(N):
        out[i] = a * x[i] + y[i]


def saxpy_slices(a, x, y, out):
    parpy.label('N')
    out[:] = a * x[:] + y[:]


def dict_scale(d, out):
    parpy.label('N')
    for i in range(d["n"]):
        out[i] = d["scale"] * d["x"][i] + d["shift"][i % 4]


def collatz_steps(x, out, N):
    parpy.label('N')
    for i in range(N):
        v = x[i]
        steps = int32(0)
        while v != 1:
            if v % 2 == 0:
                v = v // 2
            else:
                v = 3 * v + 1
            steps = steps + int32(1)
        out[i] = steps


def gpu_context_fill(out):
    with parpy.gpu:
        out[0] = float32(7.0)
        out[1] = out[0] + float32(1.0)


def column_sums(x, out, N, M):
    parpy.label('M')
    for j in range(M):
        acc = float32(0.0)
        for i in range(N):
            acc = acc + x[i, j]
        out[j] = acc


def alias_maybe_same(a, b, N, M, steps):
    """Two aliases of which one may end up naming the same array as the other."""
    parpy.label('N')
    for i in range(N):
        for t in range(steps):
            src = a
            dst = b
            if t & 1:
                dst = a
            parpy.label('M')
            for j in range(M):
                dst[i, j] = src[i, j] + float32(1.0)
