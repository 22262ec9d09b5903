"""Whole programs in the style of the reference's regression tests, compiled for gfx950 (CPU part)
and run against NumPy (GPU part): symmetric rank-k update with a triangular iteration space
(test/test_syrk.py), CSR SpMV and SpMM with data-dependent loop bounds (test/test_spmv.py,
test/test_spmm.py), nested loops with different inner thread counts (test/test_sync.py:57-92),
a Jacobi stencil on shifted slices and matrix products on slices (test/test_slicing.py)."""
import re

import numpy as np
import pytest

import parpy_amd as parpy
from parpy_amd.compile import hiprtc_compile
from parpy_amd.operators import exp, float32, sum

HIP = parpy.CompileBackend.Hip


def opts_for(p, **kw):
    o = parpy.par(p)
    o.backend = HIP
    for k, v in kw.items():
        setattr(o, k, v)
    return o


def compiles(s):
    hiprtc_compile(s[:s.index("// host side")], opts_for({}))
    return s


# ---------------------------------------------------------------- programs
def syrk(alpha, beta, C, A, N, M):
    parpy.label('i')
    for i in range(N):
        parpy.label('j')
        for j in range(i + 1):
            C[i, j] = C[i, j] * beta
            parpy.label('k')
            for k in range(M):
                C[i, j] = C[i, j] + alpha * A[i, k] * A[j, k]


def spmv(A, x, y):
    parpy.label('row')
    for row in range(A["nrows"]):
        parpy.label('i')
        for i in range(A["rows"][row], A["rows"][row + 1]):
            y[row] += A["values"][i] * x[A["cols"][i]]


def spmm(A, B, C):
    parpy.label('i')
    for i in range(A["nrows"]):
        parpy.label('j')
        for j in range(B["ncols"]):
            parpy.label('aidx')
            for aidx in range(A["rows"][i], A["rows"][i + 1]):
                C[i, j] += A["values"][aidx] * B["values"][A["cols"][aidx], j]


def exp_then_sum(x, N, M, out):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            parpy.label('K_1')
            x[i, j, :] = exp(x[i, j, :])
        parpy.label('M')
        for j in range(M):
            parpy.label('K_2')
            out[i, j] = sum(x[i, j, :])


def jacobi(nsteps, A, B):
    for t in range(1, nsteps):
        parpy.label('N')
        B[1:-1] = (A[:-2] + A[1:-1] + A[2:]) / 3.0
        parpy.label('N')
        A[1:-1] = (B[:-2] + B[1:-1] + B[2:]) / 3.0


def matmul_rows(a, b, M, N, c):
    for i in range(M):
        parpy.label('N')
        for j in range(N):
            parpy.label('K')
            c[i, j] = sum(a[i, :] * b[:, j])


def mul_planes(x, y, out):
    parpy.label('N')
    parpy.label('M')
    out[:, :] = x[:, 0, :] * y[0, :, :]


# ---------------------------------------------------------------- inputs
def axpy(a, x, y, out, N):
    """The statement of test/test_axpy.py:9-11: a labelled slice statement with a scalar taken from a tensor."""
    parpy.label('i')
    out[:] = a * x[:] + y[:]


def collatz(out, N):
    """The loop of test/test_collatz.py:9-20: a while loop of data-dependent length per element."""
    parpy.label('i')
    for i in range(1, N + 1):
        v = i
        count = 0
        while v > 1:
            if v % 2 == 0:
                v = v / 2
            else:
                v = 3 * v + 1
            count = count + 1
        out[i] = count


def syrk_data():
    M, N = 20, 30
    C = np.fromfunction(lambda i, j: ((i * j + 2) % N) / M, (N, N), dtype=np.float32).astype(np.float32)
    A = np.fromfunction(lambda i, j: ((i * j + 2) % N) / N, (N, M), dtype=np.float32).astype(np.float32)
    return 1.5, 1.2, C, A, N, M


def random_csr(n, m, density, seed):
    rng = np.random.default_rng(seed)
    nnz = int(n * m * density)
    flat = np.sort(rng.choice(n * m, size=nnz, replace=False))
    rows, cols = np.divmod(flat, m)
    crows = np.zeros(n + 1, dtype=np.int64)
    np.add.at(crows, rows + 1, 1)
    crows = np.cumsum(crows)
    vals = rng.standard_normal(nnz).astype(np.float32)
    dense = np.zeros((n, m), dtype=np.float32)
    dense[rows, cols] = vals
    return {"values": vals, "rows": crows, "cols": cols.astype(np.int64), "nrows": n}, dense


SYRK_PAR = [{'i': parpy.threads(30)}, {'i': parpy.threads(30), 'k': parpy.threads(64).reduce()},
            {'i': parpy.threads(30), 'k': parpy.threads(256).reduce()}, {'i': parpy.threads(30), 'k': parpy.threads(1024).reduce()}]
SPMV_PAR = [{"row": parpy.threads(256)}, {"row": parpy.threads(256), "i": parpy.threads(128).reduce()}]
SPMM_PAR = [{"i": parpy.threads(128)}, {"i": parpy.threads(128), "j": parpy.threads(64)},
            {"i": parpy.threads(128), "j": parpy.threads(64), "aidx": parpy.threads(64).reduce()}]
NEST_PAR = {'N': parpy.threads(10), 'M': parpy.threads(20), 'K_1': parpy.threads(64), 'K_2': parpy.threads(128)}


# ---------------------------------------------------------------- code generation (no GPU)
@pytest.mark.parametrize("p", SYRK_PAR, ids=lambda p: "+".join(p))
def test_syrk_compiles(p):
    compiles(parpy.print_compiled(syrk, list(syrk_data()), opts_for(p)))


@pytest.mark.parametrize("p", SPMV_PAR, ids=lambda p: "+".join(p))
def test_spmv_compiles(p):
    A, _ = random_csr(256, 4096, 0.01, 1)
    compiles(parpy.print_compiled(spmv, [A, np.zeros(4096, dtype=np.float32), np.zeros(256, dtype=np.float32)], opts_for(p)))


@pytest.mark.parametrize("p", SPMM_PAR, ids=lambda p: "+".join(p))
def test_spmm_compiles(p):
    A, _ = random_csr(128, 256, 0.02, 2)
    B = {"values": np.zeros((256, 64), dtype=np.float32), "ncols": 64}
    compiles(parpy.print_compiled(spmm, [A, B, np.zeros((128, 64), dtype=np.float32)], opts_for(p)))


def test_other_programs_compile():
    x = np.zeros((10, 20, 30), dtype=np.float32)
    compiles(parpy.print_compiled(exp_then_sum, [x, 10, 20, np.zeros((10, 20), dtype=np.float32)], opts_for(NEST_PAR)))
    a = np.zeros(10, dtype=np.float32)
    s = compiles(parpy.print_compiled(jacobi, [5, a, a.copy()], opts_for({'N': parpy.threads(64)})))
    host = s[s.index("// host side"):]
    assert host.count("<<<") == 2 and "for (" in host   # the time loop runs on the host: two launches per step
    compiles(parpy.print_compiled(matmul_rows, [np.zeros((10, 15), dtype=np.float32), np.zeros((15, 20), dtype=np.float32), 10, 20,
                                                np.zeros((10, 20), dtype=np.float32)], opts_for({'N': parpy.threads(64), 'K': parpy.threads(64)})))
    compiles(parpy.print_compiled(mul_planes, [np.zeros((10, 4, 15), dtype=np.float32), np.zeros((5, 10, 15), dtype=np.float32),
                                               np.zeros((10, 15), dtype=np.float32)], opts_for({'N': parpy.threads(64), 'M': parpy.threads(64)})))


def test_axpy_and_collatz_compile_and_need_parallelism():
    import torch
    N = 100
    a = torch.randn(1, dtype=torch.float32)[0]            # a 0-d tensor, as in the reference's test
    x, y = torch.randn(N), torch.randn(N)
    s = compiles(parpy.print_compiled(axpy, [a, x, y, torch.zeros_like(x), N], opts_for({'i': parpy.threads(128)})))
    assert re.search(r"<<<dim3\(1, 1, 1\), dim3\(128, 1, 1\)", s)
    with pytest.raises(RuntimeError, match="does not contain any parallelism"):
        parpy.print_compiled(axpy, [a, x, y, torch.zeros_like(x), N], opts_for({}))
    s = compiles(parpy.print_compiled(collatz, [np.zeros(1001, dtype=np.int32), 1000], opts_for({'i': parpy.threads(128)})))
    assert "while (" in s


# ---------------------------------------------------------------- results (GPU)
@pytest.mark.gpu
def test_axpy_and_collatz():
    import torch
    torch.manual_seed(1234)
    N = 100
    a = torch.randn(1, dtype=torch.float32)[0]
    x, y = torch.randn(N), torch.randn(N)
    want = torch.zeros_like(x)
    axpy(a, x, y, want, N)
    got = torch.zeros_like(x)
    parpy.jit(axpy)(a, x, y, got, N, opts=opts_for({'i': parpy.threads(128)}))
    assert torch.allclose(want, got, atol=1e-5)
    want = np.zeros(1001, dtype=np.int32)
    collatz(want, 1000)
    got = np.zeros(1001, dtype=np.int32)
    parpy.jit(collatz)(got, 1000, opts=opts_for({'i': parpy.threads(256)}))
    assert np.array_equal(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("p", SYRK_PAR, ids=lambda p: "+".join(p))
def test_syrk(p):
    alpha, beta, C, A, N, M = syrk_data()
    want = C.copy()
    tri = np.tril(np.ones((N, N), dtype=bool))
    want[tri] = (C * np.float32(beta) + np.float32(alpha) * (A @ A.T))[tri]
    got = C.copy()
    parpy.jit(syrk)(alpha, beta, got, A, N, M, opts=opts_for(p))
    assert np.allclose(got, want, atol=1e-4, rtol=1e-5)
    assert np.array_equal(got[~tri], C[~tri])     # the upper triangle is not touched


@pytest.mark.gpu
@pytest.mark.parametrize("p", SPMV_PAR, ids=lambda p: "+".join(p))
def test_spmv(p):
    A, dense = random_csr(256, 4096, 0.01, 1)
    x = np.random.default_rng(5).standard_normal(4096).astype(np.float32)
    y = np.zeros(256, dtype=np.float32)
    parpy.jit(spmv)(A, x, y, opts=opts_for(p))
    assert np.allclose(y, dense.astype(np.float64) @ x, atol=1e-4)


def test_spmv_with_one_thread_per_row_shares_rows_among_eight_lanes():
    """Bounds that are data (a CSR row): lane g of a group of eight takes the elements lo+g, lo+g+8, ...;
    the gather x[cols[i]] goes lane by lane, the partial sums meet in three cross-lane steps."""
    A, _ = random_csr(256, 4096, 0.01, 1)
    args = [A, np.zeros(4096, dtype=np.float32), np.zeros(256, dtype=np.float32)]
    s = compiles(parpy.print_compiled(spmv, args, opts_for({"row": parpy.threads(256)})))
    assert re.search(r"i_\d+ \+= 8\)", s) and "= parpy_sum8(" in s and "<<<dim3(8, 1, 1), dim3(256, 1, 1)" in s
    s = compiles(parpy.print_compiled(spmv, args, opts_for({"row": parpy.threads(256)}, opt_lane_split=False)))
    assert "= parpy_sum8(" not in s and "<<<dim3(1, 1, 1), dim3(256, 1, 1)" in s


@pytest.mark.gpu
@pytest.mark.parametrize("rows,density", [(5000, 0.002), (300, 0.05), (64, 0.3)])
def test_spmv_with_one_thread_per_row_on_ragged_rows(rows, density):
    A, dense = random_csr(rows, 2048, density, rows)
    lens = np.diff(A["rows"])
    assert lens.min() == 0 or rows < 1000          # the big case has empty rows
    x = np.random.default_rng(7).standard_normal(2048).astype(np.float32)
    want = dense.astype(np.float64) @ x
    for split in (True, False):
        y = np.zeros(rows, dtype=np.float32)
        parpy.jit(spmv)(A, x, y, opts=opts_for({"row": parpy.threads(rows)}, opt_lane_split=split))
        assert np.allclose(y, want, atol=1e-4), (rows, split)


@pytest.mark.gpu
@pytest.mark.parametrize("p", SPMM_PAR, ids=lambda p: "+".join(p))
def test_spmm(p):
    A, dense = random_csr(128, 256, 0.02, 2)
    Bv = np.random.default_rng(6).standard_normal((256, 64)).astype(np.float32)
    C = np.zeros((128, 64), dtype=np.float32)
    parpy.jit(spmm)(A, {"values": Bv, "ncols": 64}, C, opts=opts_for(p))
    assert np.allclose(C, dense.astype(np.float64) @ Bv, atol=1e-4)


@pytest.mark.gpu
def test_nested_loops_with_different_inner_thread_counts():
    x = np.random.default_rng(7).standard_normal((10, 20, 30)).astype(np.float32)
    out = np.zeros((10, 20), dtype=np.float32)
    xd = x.copy()
    parpy.jit(exp_then_sum)(xd, 10, 20, out, opts=opts_for(NEST_PAR))
    assert np.allclose(xd, np.exp(x), atol=1e-5, rtol=1e-5)
    assert np.allclose(out, np.exp(x.astype(np.float64)).sum(axis=2), atol=1e-4, rtol=1e-5)


@pytest.mark.gpu
def test_stencil_and_products_on_slices():
    rng = np.random.default_rng(8)
    A, B = rng.standard_normal(10).astype(np.float32), rng.standard_normal(10).astype(np.float32)
    wa, wb = A.copy(), B.copy()
    jacobi(5, wa, wb)                              # the function itself, run by the Python interpreter
    parpy.jit(jacobi)(5, A, B, opts=opts_for({'N': parpy.threads(64)}))
    assert np.allclose(A, wa, atol=1e-5) and np.allclose(B, wb, atol=1e-5)
    a, b = rng.standard_normal((10, 15)).astype(np.float32), rng.standard_normal((15, 20)).astype(np.float32)
    c = np.zeros((10, 20), dtype=np.float32)
    parpy.jit(matmul_rows)(a, b, 10, 20, c, opts=opts_for({'N': parpy.threads(64), 'K': parpy.threads(64)}))
    assert np.allclose(c, a @ b, atol=1e-4)
    x, y = rng.standard_normal((10, 4, 15)).astype(np.float32), rng.standard_normal((5, 10, 15)).astype(np.float32)
    out = np.zeros((10, 15), dtype=np.float32)
    parpy.jit(mul_planes)(x, y, out, opts=opts_for({'N': parpy.threads(64), 'M': parpy.threads(64)}))
    assert np.array_equal(out, x[:, 0, :] * y[0, :, :])


def shift_groups(a, b, N):
    parpy.label('i')
    for q in range(N):
        b[4 * q] = a[4 * q] + 1.0
        b[4 * q + 1] = a[4 * q + 1] * 2.0
        b[4 * q + 2] = a[4 * q + 2] - 3.0
        b[4 * q + 3] = a[4 * q + 3] * a[4 * q]


def carry_groups(a, N):
    parpy.label('i')
    for q in range(N):
        a[4 * q + 1] = a[4 * q] + 1.0
        a[4 * q + 2] = a[4 * q + 1] * 2.0
        a[4 * q + 3] = a[4 * q + 2] - 3.0
        a[4 * q] = a[4 * q + 3] * 0.5


@pytest.mark.gpu
@pytest.mark.parametrize("pack", [True, False], ids=["packed", "unpacked"])
def test_groups_of_four_adjacent_elements(pack):
    """Four neighbouring elements read and written by one lane: as one 16-byte access where nothing
    in between can touch them, element by element where each load reads what the last store wrote."""
    rng = np.random.default_rng(21)
    N = 3000
    a = rng.standard_normal(4 * N).astype(np.float32)
    b = np.zeros_like(a)
    o = opts_for({'i': parpy.threads(N)}, opt_pack_accesses=pack)
    parpy.jit(shift_groups)(a, b, N, opts=o)
    g = a.reshape(N, 4)
    want = np.stack([g[:, 0] + np.float32(1), g[:, 1] * np.float32(2), g[:, 2] - np.float32(3), g[:, 3] * g[:, 0]], axis=1)
    assert np.array_equal(b.reshape(N, 4), want)
    c = a.copy()
    parpy.jit(carry_groups)(c, N, opts=o)
    w1 = g[:, 0] + np.float32(1)
    w2 = w1 * np.float32(2)
    w3 = w2 - np.float32(3)
    assert np.array_equal(c.reshape(N, 4), np.stack([w3 * np.float32(0.5), w1, w2, w3], axis=1))


@pytest.mark.gpu
@pytest.mark.parametrize("share", [True, False], ids=["shared", "plain"])
def test_strided_iterations_of_one_thread_with_a_guarded_index(share):
    """512 iterations on 64 threads (thread g runs g, g + 64, ...): `a[i % 64]` is the same element in all of a
    thread's iterations but only exists for i % 64 < 48, `b[i // 64]` is the iteration counter's element."""
    import kernels as K
    rng = np.random.default_rng(4)
    a, b = rng.standard_normal(48).astype(np.float32), rng.standard_normal(8).astype(np.float32)
    out = np.zeros(512, dtype=np.float32)
    K.strided_guarded_pick(a, b, out, 512, opts=opts_for({'i': parpy.threads(64)}, opt_share_iterations=share))
    i = np.arange(512)
    want = np.where(i % 64 < 48, a[np.minimum(i % 64, 47)], np.float32(-1.0)) + b[i // 64]
    assert np.array_equal(out, want.astype(np.float32))
