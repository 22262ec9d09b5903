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


def sum_planes(x, out, N, M):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            parpy.label('K')
            out[i, j] = sum(x[i, j, :])


def prod_planes(x, out, N, M):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            parpy.label('K')
            out[i, j] = prod(x[i, j, :])


def max_planes(x, out, N, M):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            parpy.label('K')
            out[i, j] = max(x[i, j, :])


def min_planes(x, out, N, M):
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            parpy.label('K')
            out[i, j] = min(x[i, j, :])


def scaled_row_sums(x, y, out, N, M):
    """A reduction between two element-wise loops of the same nest: the row is scaled in place, summed (over more
    threads than a workgroup holds when the options say so) and divided by its sum."""
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        for j in range(M):
            y[i, j] = x[i, j] * 2.0 + 1.0
        parpy.label('M')
        s = sum(y[i, :])
        out[i] = s
        parpy.label('M')
        for j in range(M):
            y[i, j] = y[i, j] / s


PLANE_REDUCTIONS = [sum_planes, prod_planes, max_planes, min_planes]
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


# ---------------------------------------------------------------- HMM forward pass out of small jitted pieces
# The reference model's recurrence (test/test_forward.py:83-160, split per phase as in
# benchmarks/forward.py:94-187) written with helper functions that return values: every score is an
# expression call that the compiler inlines.  Operators are reached through a module alias.
import parpy_amd.operators as ops


@parpy.jit
def shift_score(hmm, alpha, inst, state, j):
    """Score of reaching `state` from its j-th shift predecessor (always in duration layer 0)."""
    quarter = hmm["num_states"] // 64
    kmers = hmm["num_states"] // 16
    pred = ops.int32(j * quarter + (state // 4) % quarter)
    return hmm["trans1"][pred % kmers, state % 4] + hmm["trans2"][state // kmers] + alpha[inst, pred]


@parpy.jit
def stay_score(hmm, alpha, inst, state):
    """Score of reaching `state` by staying on its k-mer: from the next duration layer, or from itself in the last."""
    kmers = hmm["num_states"] // 16
    layer = state // kmers
    pred = ops.int32(state)
    p = hmm["gamma"]
    if layer != 15:
        pred = ops.int32(state + kmers)
        p = ops.float32(0.0)
        if layer == 14:
            p = hmm["synthetic_248"]
    return p + alpha[inst, pred]


@parpy.jit
def lse5(a, b, c, d, e):
    m = ops.max(ops.max(ops.max(ops.max(a, b), c), d), e)
    s = m + ops.log(ops.exp(a - m) + ops.exp(b - m) + ops.exp(c - m) + ops.exp(d - m) + ops.exp(e - m))
    return ops.max(s, ops.float32(-ops.inf))


@parpy.jit
def pieces_init(hmm, seqs, alpha, inst):
    o = seqs["data"][inst, 0]
    parpy.label('state')
    for state in range(hmm["num_states"]):
        alpha[inst, state] = hmm["initial_prob"][state] + hmm["output_prob"][o, state % (hmm["num_states"] // 16)]


@parpy.jit
def pieces_step(hmm, seqs, alpha1, alpha2, inst, t):
    src = alpha2
    dst = alpha1
    if t & 1:
        src = alpha1
        dst = alpha2
    o = seqs["data"][inst, t]
    parpy.label('state')
    for state in range(hmm["num_states"]):
        if t < seqs["lens"][inst]:
            total = lse5(shift_score(hmm, src, inst, state, 0), shift_score(hmm, src, inst, state, 1),
                         shift_score(hmm, src, inst, state, 2), shift_score(hmm, src, inst, state, 3),
                         stay_score(hmm, src, inst, state))
            dst[inst, state] = total + hmm["output_prob"][o, state % (hmm["num_states"] // 16)]
        elif t == seqs["lens"][inst]:
            dst[inst, state] = src[inst, state]


@parpy.jit
def pieces_total(hmm, seqs, result, alpha1, alpha2, inst):
    alpha = alpha2
    if seqs["maxlen"] & 1:
        alpha = alpha1
    parpy.label('state')
    m = ops.max(alpha[inst, :], axis=0)
    parpy.label('state')
    s = ops.sum(ops.exp(alpha[inst, :] - m), axis=0)
    result[inst] = m + ops.log(s)


@parpy.jit
def forward_in_pieces(hmm, seqs, alpha1, alpha2, result):
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        pieces_init(hmm, seqs, alpha1, inst)
        for t in range(1, seqs["maxlen"]):
            pieces_step(hmm, seqs, alpha1, alpha2, inst, t)
        pieces_total(hmm, seqs, result, alpha1, alpha2, inst)


@parpy.jit
def strided_guarded_pick(a, b, out, N):
    """512 iterations on 64 threads: thread g runs i = g, g + 64, ...; `a` has 48 elements, the test guards its index."""
    parpy.label('i')
    for i in range(N):
        out[i] = (a[i % 64] if i % 64 < 48 else float32(-1.0)) + b[i // 64]


@parpy.jit
def pick_by_quotients(a, idx, out, N):
    """`i // 3` of a loop counter fits 31 bits; `idx[i] // 3` of a loaded 64-bit value does not provably."""
    parpy.label('i')
    for i in range(N):
        out[i] = a[(i // 3) % 8] + a[(idx[i] // 3) % 8]


@parpy.jit
def exchange_steps(a, b, N, M, T):
    """T steps that swap source and destination; row i reads row i + 1 of what the previous step wrote, so the
    workgroups of different rows depend on each other."""
    parpy.label('i')
    for i in range(N):
        for t in range(T):
            src = a
            dst = b
            if t & 1:
                src = b
                dst = a
            parpy.label('j')
            for j in range(M):
                dst[i, j] = src[(i + 1) % N, j] + src[i, (j + 1) % M]


@parpy.jit
def exchange_steps_within_rows(a, b, N, M, T):
    """The same with every row on its own: only the workgroups of one row exchange data."""
    parpy.label('i')
    for i in range(N):
        for t in range(T):
            src = a
            dst = b
            if t & 1:
                src = b
                dst = a
            parpy.label('j')
            for j in range(M):
                dst[i, j] = src[i, (j + 7) % M] + src[i, (j + M // 2) % M]
