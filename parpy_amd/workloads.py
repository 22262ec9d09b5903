"""The hot-path workloads as ParPy user code, plus their seeded input generators.

The kernels are written against the public surface only (`jit`, `label`,
operators) exactly as a user of the reference would write them; each cites the
reference source it restates.  Everything arithmetic in them is compiled by the
HIP backend -- nothing here calls a hand-written kernel.
"""
import numpy as np

import parpy_amd as parpy
from parpy_amd.operators import exp, float32, float64, inf, int32, int64, log, max, min, sum


# ---------------------------------------------------------------- reductions / softmax
@parpy.jit
def sum_rows(x, out, N):
    """out[i] = sum(x[i, :])  (test/test_reduce.py:12-16, benchmarks/paper-ex.py:11-16)."""
    parpy.label('outer')
    for i in range(N):
        parpy.label('inner')
        out[i] = sum(x[i, :])


@parpy.jit
def softmax(x, N, M, out):
    """Row-wise softmax in four labelled statements (test/test_softmax.py:11-26)."""
    parpy.label('N')
    for i in range(N):
        parpy.label('M')
        m = max(x[i, :])

        parpy.label('M')
        out[i, :] = exp(x[i, :] - m)

        parpy.label('M')
        s = sum(out[i, :])

        parpy.label('M')
        out[i, :] = out[i, :] / s


@parpy.jit
def copy_1d(x, out):
    """out[:] = x[:] -- a plain streaming copy (counter calibration and bandwidth reference)."""
    parpy.label('N')
    out[:] = x[:]


# ---------------------------------------------------------------- SDDMM
@parpy.jit
def sddmm_decompress_csr(C_crows, C_rows, N):
    """CSR row pointers -> per-non-zero row ids (benchmarks/sddmm.py:21-27)."""
    parpy.label('N')
    for row in range(N):
        parpy.label('M')
        for i in range(C_crows[row], C_crows[row + 1]):
            C_rows[i] = row


@parpy.jit
def sddmm_coo(A, B, C, D, alpha, beta):
    """D[i] = alpha * dot(A[rows[i], :], B[:, cols[i]]) + beta * values[i]  (benchmarks/sddmm.py:63-70)."""
    parpy.label('nnz')
    for i in range(C["nnz"]):
        row = C["rows"][i]
        col = C["cols"][i]
        t = sum(A[row, :] * B[:, col])
        D[i] = alpha * t + beta * C["values"][i]


@parpy.jit
def sddmm_csr(A, B, C, D, N, alpha, beta):
    """SDDMM on a CSR mask: the row pointers are decompressed into `C["rows"]` by a call to the kernel
    above, then the non-zeros are processed as in the COO form (benchmarks/sddmm.py:29-42)."""
    sddmm_decompress_csr(C["crows"], C["rows"], N)
    parpy.label('nnz')
    for i in range(C["nnz"]):
        row = C["rows"][i]
        col = C["cols"][i]
        t = sum(A[row, :] * B[:, col])
        D[i] = alpha * t + beta * C["values"][i]


@parpy.jit
def sddmm_coo_bt(A, BT, C, D, alpha, beta):
    """The same product for a caller that holds B transposed (BT[j, :] = B[:, j], e.g. a constant matrix turned
    round once): both operands of a non-zero are rows, nothing is staged per call."""
    parpy.label('nnz')
    for i in range(C["nnz"]):
        row = C["rows"][i]
        col = C["cols"][i]
        t = sum(A[row, :] * BT[col, :])
        D[i] = alpha * t + beta * C["values"][i]


@parpy.jit
def gather_row_sums(table, idx, out, n):
    """out[i] = sum(table[idx[i], :]): one dependent index load, then a row of contiguous 128-byte lines from a
    random place of the table, for every i -- the access pattern of SDDMM's row of B^T without the arithmetic
    (the measure of how fast random lines come out of L2)."""
    parpy.label('i')
    for i in range(n):
        r = idx[i]
        out[i] = sum(table[r, :])


# ---------------------------------------------------------------- HMM forward, reference (16-layer) model
@parpy.jit
def forward_kernel(hmm, seqs, alpha1, alpha2, result):
    """Batched HMM forward pass of the reference's test kernel (test/test_forward.py:83-160).

    The only difference is `state % (num_states // 16)` in the initial step where
    the reference test hard-codes `% 64` for its 3-mer model; the benchmark
    version of the same kernel uses this general form (benchmarks/forward.py:99-101).
    """
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        # Initialization
        o = seqs["data"][inst, 0]
        parpy.label('state')
        for state in range(hmm["num_states"]):
            alpha1[inst, state] = hmm["initial_prob"][state] + hmm["output_prob"][o, state % (hmm["num_states"] // 16)]

        # Forward steps (t = 1, .., maxlen-1)
        for t in range(1, seqs["maxlen"]):
            alpha_src = alpha2
            alpha_dst = alpha1
            if t & 1:
                alpha_src = alpha1
                alpha_dst = alpha2
            o = seqs["data"][inst, t]
            parpy.label('state')
            for state in range(hmm["num_states"]):
                if t < seqs["lens"][inst]:
                    num_kmers = hmm["num_states"] // 16

                    pred1 = int32((state // 4) % (hmm["num_states"] // 64))
                    pred2 = int32(hmm["num_states"] // 64 + (state // 4) % (hmm["num_states"] // 64))
                    pred3 = int32(2 * hmm["num_states"] // 64 + (state // 4) % (hmm["num_states"] // 64))
                    pred4 = int32(3 * hmm["num_states"] // 64 + (state // 4) % (hmm["num_states"] // 64))
                    t11 = hmm["trans1"][pred1 % num_kmers, state % 4]
                    t12 = hmm["trans1"][pred2 % num_kmers, state % 4]
                    t13 = hmm["trans1"][pred3 % num_kmers, state % 4]
                    t14 = hmm["trans1"][pred4 % num_kmers, state % 4]
                    t2 = hmm["trans2"][state // num_kmers]
                    p1 = t11 + t2 + alpha_src[inst, pred1]
                    p2 = t12 + t2 + alpha_src[inst, pred2]
                    p3 = t13 + t2 + alpha_src[inst, pred3]
                    p4 = t14 + t2 + alpha_src[inst, pred4]

                    pred5 = int32(0)
                    p5 = float32(0.0)
                    if state // num_kmers == 15:
                        pred5 = state
                        p5 = hmm["gamma"]
                    elif state // num_kmers == 14:
                        pred5 = ((state // num_kmers) + 1) * num_kmers + state % num_kmers
                        p5 = hmm["synthetic_248"]
                    else:
                        pred5 = ((state // num_kmers) + 1) * num_kmers + state % num_kmers
                        p5 = float32(0.0)
                    p5 = p5 + alpha_src[inst, pred5]

                    # Inlined version of log_sum_exp.
                    maxp = max(p1, p2)
                    maxp = max(maxp, p3)
                    maxp = max(maxp, p4)
                    maxp = max(maxp, p5)
                    lsexp = maxp + log(
                        exp(p1 - maxp) + exp(p2 - maxp) + exp(p3 - maxp) +
                        exp(p4 - maxp) + exp(p5 - maxp)
                    )
                    lsexp = max(lsexp, float32(-inf))

                    alpha_dst[inst, state] = lsexp + hmm["output_prob"][o, state % num_kmers]
                elif t == seqs["lens"][inst]:
                    alpha_dst[inst, state] = alpha_src[inst, state]

        # Summation of final alpha values
        alpha = alpha2
        if seqs["maxlen"] & 1:
            alpha = alpha1

        parpy.label('state')
        maxp = max(alpha[inst, :])

        parpy.label('state')
        psum = sum(exp(alpha[inst, :] - maxp))

        result[inst] = maxp + log(psum)


# ---------------------------------------------------------------- HMM forward, synthetic single-layer model
@parpy.jit
def forward_syn_init(hmm, seqs, alpha_src, inst):
    o = seqs["data"][inst, 0]
    parpy.label('state')
    for state in range(hmm["num_states"]):
        alpha_src[inst, state] = hmm["initial_prob"][state] + hmm["output_prob"][o, state]


@parpy.jit
def forward_syn_step(hmm, seqs, alpha1, alpha2, inst, t):
    alpha_src = alpha2
    alpha_dst = alpha1
    if t & 1:
        alpha_src = alpha1
        alpha_dst = alpha2
    o = seqs["data"][inst, t]
    parpy.label('state')
    for state in range(hmm["num_states"]):
        if t < seqs["lens"][inst]:
            q = state // 4
            pred1 = q
            pred2 = hmm["num_states"] // 4 + q
            pred3 = 2 * (hmm["num_states"] // 4) + q
            pred4 = 3 * (hmm["num_states"] // 4) + q
            p1 = hmm["trans1"][pred1, state % 4] + alpha_src[inst, pred1]
            p2 = hmm["trans1"][pred2, state % 4] + alpha_src[inst, pred2]
            p3 = hmm["trans1"][pred3, state % 4] + alpha_src[inst, pred3]
            p4 = hmm["trans1"][pred4, state % 4] + alpha_src[inst, pred4]
            p5 = hmm["stay"][state] + alpha_src[inst, state]
            maxp = max(p1, p2)
            maxp = max(maxp, p3)
            maxp = max(maxp, p4)
            maxp = max(maxp, p5)
            lsexp = maxp + log(
                exp(p1 - maxp) + exp(p2 - maxp) + exp(p3 - maxp) +
                exp(p4 - maxp) + exp(p5 - maxp)
            )
            lsexp = max(lsexp, float32(-inf))
            alpha_dst[inst, state] = lsexp + hmm["output_prob"][o, state]


@parpy.jit
def forward_syn_lse(hmm, seqs, result, alpha1, alpha2, inst):
    # after len-1 steps the newest state vector is alpha2 when len is even
    alpha = alpha1
    if seqs["lens"][inst] & 1 == 0:
        alpha = alpha2

    parpy.label('state')
    maxp = max(alpha[inst, :])

    parpy.label('state')
    psum = sum(exp(alpha[inst, :] - maxp))

    result[inst] = maxp + log(psum)


@parpy.jit
def forward_syn(hmm, seqs, result, alpha1, alpha2):
    """Synthetic single-layer HMM forward pass, structured like the reference's
    benchmark kernel (benchmarks/forward.py:94-187): init, per-step and final
    log-sum-exp helpers inlined into one labelled batch loop; nothing is written
    once t >= len and the final buffer is picked by the parity of the length."""
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        forward_syn_init(hmm, seqs, alpha1, inst)
        for t in range(1, seqs["maxlen"]):
            forward_syn_step(hmm, seqs, alpha1, alpha2, inst, t)
        forward_syn_lse(hmm, seqs, result, alpha1, alpha2, inst)


# ---------------------------------------------------------------- HMM forward, synthetic model, four states at a time
@parpy.jit
def syn4_state(e1, e2, e3, e4, t1, t2, t3, t4, w, own, m, emission):
    """New score of one state of a group whose scores do not exceed the predecessors' by more than e^80."""
    return m + log(e1 * t1 + e2 * t2 + e3 * t3 + e4 * t4 + w * exp(own - m)) + emission


@parpy.jit
def syn4_state_wide(e1, e2, e3, e4, t1, t2, t3, t4, w, own, m, emission):
    """The same for any scores: the sum is referred to the larger of `own` and `m`, so that the one exponential
    taken here never exceeds one."""
    s = e1 * t1 + e2 * t2 + e3 * t3 + e4 * t4
    e = exp(-abs(own - m))
    total = s + w * e
    base = m
    if own > m:
        total = w + s * e
        base = own
    return base + log(total) + emission


@parpy.jit
def forward_syn4_step(hmm, seqs, alpha1, alpha2, inst, t):
    alpha_src = alpha2
    alpha_dst = alpha1
    if t & 1:
        alpha_src = alpha1
        alpha_dst = alpha2
    o = seqs["data"][inst, t]
    parpy.label('state')
    for q in range(hmm["num_states"] // 4):
        if t < seqs["lens"][inst]:
            nq = hmm["num_states"] // 4
            a1 = alpha_src[inst, q]
            a2 = alpha_src[inst, nq + q]
            a3 = alpha_src[inst, 2 * nq + q]
            a4 = alpha_src[inst, 3 * nq + q]
            o0 = alpha_src[inst, 4 * q]
            o1 = alpha_src[inst, 4 * q + 1]
            o2 = alpha_src[inst, 4 * q + 2]
            o3 = alpha_src[inst, 4 * q + 3]
            b0 = hmm["output_prob"][o, 4 * q]
            b1 = hmm["output_prob"][o, 4 * q + 1]
            b2 = hmm["output_prob"][o, 4 * q + 2]
            b3 = hmm["output_prob"][o, 4 * q + 3]
            # reference point of the group: the largest predecessor score, kept finite so that a group
            # whose predecessors are all unreachable (-inf) gives exp(-inf) = 0 and not exp(nan)
            m = max(max(max(a1, a2), max(a3, a4)), float32(-3.0e38))
            e1 = exp(a1 - m)
            e2 = exp(a2 - m)
            e3 = exp(a3 - m)
            e4 = exp(a4 - m)
            if max(max(o0, o1), max(o2, o3)) - m <= float32(80.0):
                alpha_dst[inst, 4 * q] = syn4_state(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 0], hmm["ptrans1"][nq + q, 0],
                    hmm["ptrans1"][2 * nq + q, 0], hmm["ptrans1"][3 * nq + q, 0], hmm["pstay"][4 * q], o0, m, b0)
                alpha_dst[inst, 4 * q + 1] = syn4_state(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 1], hmm["ptrans1"][nq + q, 1],
                    hmm["ptrans1"][2 * nq + q, 1], hmm["ptrans1"][3 * nq + q, 1], hmm["pstay"][4 * q + 1], o1, m, b1)
                alpha_dst[inst, 4 * q + 2] = syn4_state(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 2], hmm["ptrans1"][nq + q, 2],
                    hmm["ptrans1"][2 * nq + q, 2], hmm["ptrans1"][3 * nq + q, 2], hmm["pstay"][4 * q + 2], o2, m, b2)
                alpha_dst[inst, 4 * q + 3] = syn4_state(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 3], hmm["ptrans1"][nq + q, 3],
                    hmm["ptrans1"][2 * nq + q, 3], hmm["ptrans1"][3 * nq + q, 3], hmm["pstay"][4 * q + 3], o3, m, b3)
            else:
                alpha_dst[inst, 4 * q] = syn4_state_wide(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 0], hmm["ptrans1"][nq + q, 0],
                    hmm["ptrans1"][2 * nq + q, 0], hmm["ptrans1"][3 * nq + q, 0], hmm["pstay"][4 * q], o0, m, b0)
                alpha_dst[inst, 4 * q + 1] = syn4_state_wide(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 1], hmm["ptrans1"][nq + q, 1],
                    hmm["ptrans1"][2 * nq + q, 1], hmm["ptrans1"][3 * nq + q, 1], hmm["pstay"][4 * q + 1], o1, m, b1)
                alpha_dst[inst, 4 * q + 2] = syn4_state_wide(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 2], hmm["ptrans1"][nq + q, 2],
                    hmm["ptrans1"][2 * nq + q, 2], hmm["ptrans1"][3 * nq + q, 2], hmm["pstay"][4 * q + 2], o2, m, b2)
                alpha_dst[inst, 4 * q + 3] = syn4_state_wide(
                    e1, e2, e3, e4, hmm["ptrans1"][q, 3], hmm["ptrans1"][nq + q, 3],
                    hmm["ptrans1"][2 * nq + q, 3], hmm["ptrans1"][3 * nq + q, 3], hmm["pstay"][4 * q + 3], o3, m, b3)


@parpy.jit
def forward_syn4(hmm, seqs, result, alpha1, alpha2):
    """The synthetic forward pass with the step written over groups of four states.

    States 4q .. 4q+3 have the same four shift predecessors q, S/4+q, S/2+q, 3S/4+q.  Their scores are
    referred to the largest of the four once per group, `exp(a_j - m)` is taken once per group, and the
    transition and stay probabilities enter in linear space (`ptrans1 = exp(trans1)`, `pstay = exp(stay)`):
    alpha'[4q+u] = m + log(sum_j ptrans1[pred_j, u] * e_j + pstay[4q+u] * exp(alpha[4q+u] - m)) + emission.
    A group in which some state scores more than e^80 above every predecessor takes a second branch that
    refers each state to the larger of m and its own score, so no exponential can overflow; unreachable
    states (-inf) stay -inf.  Same recurrence as `forward_syn` in real arithmetic: 3 exponentials and
    logarithms per state instead of 6."""
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        forward_syn_init(hmm, seqs, alpha1, inst)
        for t in range(1, seqs["maxlen"]):
            forward_syn4_step(hmm, seqs, alpha1, alpha2, inst, t)
        forward_syn_lse(hmm, seqs, result, alpha1, alpha2, inst)


# ---------------------------------------------------------------- probability tables of the linear-space forms
@parpy.jit
def probability(x):
    """exp of a single-precision logarithm, taken in double precision and rounded once."""
    return float32(exp(float64(x)))


@parpy.jit
def emission_probabilities(hmm, lin, rowmax):
    """`pemit` = exp(output_prob - emit_max) with `emit_max` the largest entry of the whole table (row maxima
    first, then the maximum of those), so that the largest emission probability becomes one."""
    parpy.label('obs')
    for o in range(hmm["num_obs"]):
        parpy.label('state')
        rowmax[o] = max(hmm["output_prob"][o, :])
    parpy.label('obs')
    lin["emit_max"][0] = max(rowmax[:])
    parpy.label('obs')
    for o in range(hmm["num_obs"]):
        parpy.label('state')
        for s in range(hmm["num_kmers"]):
            lin["pemit"][o, s] = float32(exp(float64(hmm["output_prob"][o, s]) - float64(lin["emit_max"][0])))


@parpy.jit
def scaled_tables(hmm, lin, rowmax):
    """The synthetic model's log-space tables (`trans1`, `stay`, `initial_prob`, `output_prob`) as the probability
    tables `forward_scaled` and `forward_syn4` read: `ptrans1`, `pstay`, `pinit`, `pemit`, `emit_max`."""
    emission_probabilities(hmm, lin, rowmax)
    parpy.label('all')
    for s in range(hmm["num_states"]):
        lin["pstay"][s] = probability(hmm["stay"][s])
        lin["pinit"][s] = probability(hmm["initial_prob"][s])
        for u in range(4):
            lin["ptrans1"][s, u] = probability(hmm["trans1"][s, u])


@parpy.jit
def scaled_reference_tables(hmm, lin, rowmax):
    """The reference's 16-layer model (tables of `load_reference_model`) as the probability tables
    `forward_kernel_scaled` reads: `ptrans1` [4^k, 4], `pdur` [16], `pnext` [16] (one for layers 0..13, 1 - tail
    for layer 14, tail for the last layer's self loop; tail = exp(gamma)), `pinit`, `pemit`, `emit_max`."""
    emission_probabilities(hmm, lin, rowmax)
    parpy.label('all')
    for s in range(hmm["num_states"]):
        lin["pinit"][s] = probability(hmm["initial_prob"][s])
    parpy.label('all')
    for q in range(hmm["num_kmers"]):
        for u in range(4):
            lin["ptrans1"][q, u] = probability(hmm["trans1"][q, u])
    parpy.label('layer')
    for l in range(16):
        lin["pdur"][l] = probability(hmm["trans2"][l])
        tail = exp(float64(hmm["gamma"]))
        nxt = float64(1.0)
        if l == 14:
            nxt = float64(1.0) - tail
        elif l == 15:
            nxt = tail
        lin["pnext"][l] = float32(nxt)


# ---------------------------------------------------------------- HMM forward, synthetic model, scaled linear space
@parpy.jit
def forward_scaled_step(hmm, seqs, beta1, beta2, inst, t, r):
    beta_src = beta2
    beta_dst = beta1
    if t & 1:
        beta_src = beta1
        beta_dst = beta2
    o = seqs["data"][inst, t]
    parpy.label('state')
    for q in range(hmm["num_states"] // 4):
        if t < seqs["lens"][inst]:
            nq = hmm["num_states"] // 4
            a1 = beta_src[inst, q]
            a2 = beta_src[inst, nq + q]
            a3 = beta_src[inst, 2 * nq + q]
            a4 = beta_src[inst, 3 * nq + q]
            for u in range(4):
                s = (a1 * hmm["ptrans1"][q, u] + a2 * hmm["ptrans1"][nq + q, u] +
                     a3 * hmm["ptrans1"][2 * nq + q, u] + a4 * hmm["ptrans1"][3 * nq + q, u] +
                     beta_src[inst, 4 * q + u] * hmm["pstay"][4 * q + u])
                beta_dst[inst, 4 * q + u] = (s * r) * hmm["pemit"][o, 4 * q + u]


@parpy.jit
def forward_scaled_top(hmm, seqs, beta1, beta2, inst, t):
    beta = beta1
    if t & 1:
        beta = beta2
    parpy.label('state')
    top = max(beta[inst, :])
    return top


@parpy.jit
def scaled_doublings(top):
    """How many times the state vector whose largest element is `top` can be doubled without passing one
    (0 .. 120; nothing has to be exact here, any power of two near 1 / top serves as the multiplier)."""
    return int64(min(max(-log(top) * float32(1.4426950408889634), float32(0.0)), float32(120.0)))


@parpy.jit
def power_of_two(k):
    """2^k in single precision for 0 <= k <= 120, exactly: the product of two shifted ones."""
    return float32(int64(1) << min(k, int64(60))) * float32(int64(1) << max(k - int64(60), int64(0)))


@parpy.jit
def forward_scaled(hmm, seqs, result, beta1, beta2):
    """The forward pass of the synthetic model in linear space with rescaling (the classical alternative to
    log space): beta[s] holds the probability alpha[s] times a running scale.  Tables are probabilities:
    `ptrans1`, `pstay`, `pinit`, and `pemit` = emission probabilities divided by the largest of them, whose
    logarithm is `emit_max[0]` (what `scaled_tables` makes of the log-space tables).  A step is one multiplication and four multiply-adds per state for the
    sum over its predecessors and itself and two multiplications (by the multiplier `r` and by the emission),
    no exponential and no logarithm.  Every eighth step the largest element of the new state vector is looked
    up; the vector itself is left alone and the next step multiplies what it produces by a power of two that
    brings that element back to just under one (the step is linear, so this is the same as scaling its input,
    without a second pass over the vector).  A power of two scales without rounding, and all that has to be
    remembered of it is its exponent: the running scale is an integer count of doublings, and the time loop
    holds no float64 arithmetic at all.  The result is float64:
    log-likelihood = log(sum of the final vector) - doublings * log(2) + len * emit_max.

    Range: between two look-ups (eight steps; the first window also carries the 1 / num_states of the start
    vector) the largest element may shrink by up to 2^100, i.e. the steps of a window may on average keep as
    little as 2^-12.5 = 1.7e-4 of the vector, measured against the most probable emission.  Within that range the
    elements that matter (within 2^-24 of the largest) stay normal single-precision numbers and the result is
    good to 1e-4.  A read that
    leaves the range (largest element positive but below 2^-100 at a look-up) gives NaN, not digits that mean
    nothing; a read of probability zero gives log(0) = -inf, as log space would."""
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        o0 = seqs["data"][inst, 0]
        parpy.label('state')
        for state in range(hmm["num_states"]):
            beta1[inst, state] = hmm["pinit"][state] * hmm["pemit"][o0, state]
        doublings = int64(0)
        r = float32(1.0)
        for t in range(1, seqs["maxlen"]):
            forward_scaled_step(hmm, seqs, beta1, beta2, inst, t, r)
            if t < seqs["lens"][inst]:
                r = float32(1.0)
                if t % 8 == 0:
                    top = forward_scaled_top(hmm, seqs, beta1, beta2, inst, t)
                    k = scaled_doublings(top)
                    r = power_of_two(k)
                    doublings = doublings + k
                    if top > float32(0.0) and top < float32(7.888609e-31):
                        r = (top - top) / (top - top)   # out of range (see the docstring): not a number, rather than digits that mean nothing
        beta = beta1
        if seqs["lens"][inst] & 1 == 0:
            beta = beta2
        parpy.label('state')
        total = sum(beta[inst, :])
        result[inst] = (log(float64(total) * float64(r)) - float64(doublings) * float64(0.6931471805599453)
                        + float64(seqs["lens"][inst]) * float64(hmm["emit_max"][0]))


# ---------------------------------------------------------------- HMM forward, reference (16-layer) model, scaled linear space
@parpy.jit
def forward_kernel_scaled_step(hmm, seqs, beta1, beta2, inst, t, r):
    beta_src = beta2
    beta_dst = beta1
    if t & 1:
        beta_src = beta1
        beta_dst = beta2
    o = seqs["data"][inst, t]
    parpy.label('state')
    for g in range(hmm["num_states"] // 16):
        if t < seqs["lens"][inst]:
            nk = hmm["num_states"] // 16
            nq = nk // 4
            q = g % nq
            lc = g // nq
            a1 = beta_src[inst, q]
            a2 = beta_src[inst, nq + q]
            a3 = beta_src[inst, 2 * nq + q]
            a4 = beta_src[inst, 3 * nq + q]
            for l in range(4):
                layer = 4 * lc + l
                up = min(layer + 1, 15)
                for u in range(4):
                    inflow = (a1 * hmm["ptrans1"][q, u] + a2 * hmm["ptrans1"][nq + q, u] +
                              a3 * hmm["ptrans1"][2 * nq + q, u] + a4 * hmm["ptrans1"][3 * nq + q, u])
                    s = hmm["pdur"][layer] * inflow + hmm["pnext"][layer] * beta_src[inst, up * nk + 4 * q + u]
                    beta_dst[inst, layer * nk + 4 * q + u] = (s * r) * hmm["pemit"][o, 4 * q + u]


@parpy.jit
def forward_kernel_scaled(hmm, seqs, result, beta1, beta2):
    """The forward pass of the reference's 16-layer model (the recurrence of test/test_forward.py:83-160) in
    linear space with rescaling.  A state is (duration layer, k-mer).  What flows into a k-mer from the four
    k-mers that precede it (always out of layer 0) is the same for all 16 layers, so one thread computes it once
    for four neighbouring k-mers and four layers; a layer then adds what comes down from the layer above (from
    itself in the last layer).  Tables are probabilities: `ptrans1` [4^k, 4], `pdur` [16] (the reference's
    `trans2`), `pnext` [16] (1 for layers 0..13, 1 - tail for layer 14, tail for the last layer's self loop),
    `pinit`, and `pemit` [101, 4^k] = emission probabilities divided by the largest of them (`emit_max` holds its
    logarithm; `scaled_reference_tables` makes all of them from the log-space tables).  The reference's
    emission tables reach down to 1e-10, so the multiplier is renewed every fourth step (in the way described at
    `forward_scaled`: the largest element is looked up, the next step multiplies by the power of two that brings
    it back to just under one, and the doublings are counted).  The result is float64, as in `forward_scaled`."""
    parpy.label('inst')
    for inst in range(seqs["num_instances"]):
        o0 = seqs["data"][inst, 0]
        parpy.label('state')
        for state in range(hmm["num_states"]):
            beta1[inst, state] = hmm["pinit"][state] * hmm["pemit"][o0, state % (hmm["num_states"] // 16)]
        doublings = int64(0)
        r = float32(1.0)
        for t in range(1, seqs["maxlen"]):
            forward_kernel_scaled_step(hmm, seqs, beta1, beta2, inst, t, r)
            if t < seqs["lens"][inst]:
                r = float32(1.0)
                if t % 4 == 0:
                    top = forward_scaled_top(hmm, seqs, beta1, beta2, inst, t)
                    k = scaled_doublings(top)
                    r = power_of_two(k)
                    doublings = doublings + k
                    if top > float32(0.0) and top < float32(7.888609e-31):
                        r = (top - top) / (top - top)   # out of range (see the docstring): not a number, rather than digits that mean nothing
        beta = beta1
        if seqs["lens"][inst] & 1 == 0:
            beta = beta2
        parpy.label('state')
        total = sum(beta[inst, :])
        result[inst] = (log(float64(total) * float64(r)) - float64(doublings) * float64(0.6931471805599453)
                        + float64(seqs["lens"][inst]) * float64(hmm["emit_max"][0]))


# ---------------------------------------------------------------- seeded inputs
SEED = 1234


def make_rowsum(n=1024, m=65536, seed=SEED):
    rng = np.random.default_rng(seed)
    return rng.uniform(-1.0, 1.0, (n, m)).astype(np.float32)


def make_softmax(n=16384, m=4096, seed=SEED):
    import torch
    g = torch.Generator().manual_seed(seed)
    return torch.randn((n, m), generator=g, dtype=torch.float32)


def make_sddmm(n=8192, k=128, density=0.01, seed=SEED):
    """A [n,k], B [k,n] normal(0,1); CSR mask with nnz = int(density*n*n) spread evenly
    over the rows, column indices drawn without replacement and sorted per row."""
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((n, k)).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    nnz = int(density * n * n)
    per_row = np.full(n, nnz // n, dtype=np.int64)
    per_row[: nnz - per_row.sum()] += 1
    crows = np.zeros(n + 1, dtype=np.int64)
    crows[1:] = np.cumsum(per_row)
    cols = np.empty(nnz, dtype=np.int64)
    for r in range(n):
        cols[crows[r]:crows[r + 1]] = np.sort(rng.choice(n, size=per_row[r], replace=False))
    vals = rng.standard_normal(nnz).astype(np.float32)
    return A, B, crows, cols, vals


def synthetic_hmm(k, n_inst=100, min_len=5000, max_len=15000, seed=SEED, emissions=None):
    """De Bruijn HMM with S = 4^k states: four shift predecessors plus a stay transition.

    Per source state r a Dirichlet(1,1,1,1,1) draw gives the probabilities of its
    four successors 4*(r mod S/4)+c (stored as trans1[r, c]) and of staying
    (stay[r]); emissions are Dirichlet(1 x 101) per state stored observation-major
    [101, S]; the initial distribution is uniform.  `emissions` overrides the
    emission table with a constant log-probability (used by closed-form tests).
    """
    rng = np.random.default_rng(seed)
    S = 4 ** k
    p = rng.dirichlet(np.ones(5), size=S)
    trans1 = np.log(p[:, :4]).astype(np.float32)
    stay = np.log(p[:, 4]).astype(np.float32)
    if emissions is None:
        e = rng.dirichlet(np.ones(101), size=S)          # [S, 101]
        out = np.ascontiguousarray(np.log(e).T.astype(np.float32))
    else:
        out = np.full((101, S), emissions, dtype=np.float32)
    init = np.full(S, np.log(1.0 / S), dtype=np.float32)
    lens = rng.integers(min_len, max_len + 1, size=n_inst).astype(np.int64)
    maxlen = int(lens.max())
    data = rng.integers(0, 101, size=(n_inst, maxlen)).astype(np.int8)
    for i, n in enumerate(lens):
        data[i, n:] = 0
    hmm = {"trans1": trans1, "stay": stay, "output_prob": out, "initial_prob": init, "num_states": S}
    seqs = {"data": data, "lens": lens, "maxlen": maxlen, "num_instances": n_inst}
    return hmm, seqs


def load_reference_model(model_npz, signals_npz):
    """Kernel inputs for `forward_kernel` from the reference's model and signal tables (as re-packed
    from its HDF5 files): the layout work of test/test_forward.py:31-77 and
    benchmarks/forward.py:232-312.

    model: `k`, `obs` [101, 4^k] emission probabilities indexed by the k-mer read in reverse base
    order, `trans` 4 x 4^k successor probabilities, `duration` [16], `tail_factor`.
    Returned tables are natural logarithms in float32: `trans1` [4^k, 4], `trans2` [16],
    `output_prob` [101, 4^k] re-indexed to forward base order, `initial_prob` uniform over the
    first duration layer and -inf elsewhere, `gamma` = log tail, `synthetic_248` = log(1 - tail).
    Signals are concatenated int levels with per-read lengths; they become a zero-padded int8 matrix.
    """
    m = np.load(model_npz)
    k = int(m["k"])
    nk = 4 ** k
    # index of each k-mer with its base-4 digits reversed
    idx = np.arange(nk)
    rev = np.zeros(nk, dtype=np.int64)
    for _ in range(k):
        rev = rev * 4 + idx % 4
        idx = idx // 4
    with np.errstate(divide="ignore"):
        # logarithms in the precision the tables are stored in, as the reference takes them
        log_obs = np.log(m["obs"])
        log_trans = np.log(m["trans"])
    tail = float(m["tail_factor"])
    init = np.full(16 * nk, -np.inf, dtype=np.float32)
    init[:nk] = np.float32(-np.log(float(nk)))
    hmm = {
        "trans1": np.ascontiguousarray(log_trans.reshape(4, nk).T, dtype=np.float32),
        "trans2": np.log(m["duration"]).astype(np.float32),
        "output_prob": np.ascontiguousarray(log_obs[:, rev], dtype=np.float32),
        "initial_prob": init,
        "gamma": np.float32(np.log(tail)),
        "synthetic_248": np.float32(np.log1p(-tail)),
        "num_states": 16 * nk,
    }
    s = np.load(signals_npz)
    lens = np.asarray(s["lens"], dtype=np.int64)
    ends = np.cumsum(lens)
    data = np.zeros((len(lens), int(lens.max())), dtype=np.int8)
    for i, (e, n) in enumerate(zip(ends, lens)):
        data[i, :n] = s["samples"][e - n:e]
    seqs = {"data": data, "lens": lens, "maxlen": int(lens.max()), "num_instances": len(lens)}
    return hmm, seqs


def random_reference_model(k, n_reads=100, min_len=500, max_len=1500, seed=SEED, tail=0.05):
    """Seeded random tables in the format of the reference's 16-layer model (`load_reference_model`) for sizes it
    ships no tables for (its 7-mer model file is absent): Dirichlet rows for the successor, duration and emission
    probabilities, uniform start over the first layer; reads of uniform random levels and lengths."""
    rng = np.random.default_rng(seed)
    nk = 4 ** k
    hmm = {
        "trans1": np.log(rng.dirichlet(np.ones(4), size=nk)).astype(np.float32),
        "trans2": np.log(rng.dirichlet(np.ones(16))).astype(np.float32),
        "output_prob": np.ascontiguousarray(np.log(rng.dirichlet(np.ones(101), size=nk)).T.astype(np.float32)),
        "initial_prob": np.concatenate([np.full(nk, -np.log(float(nk))), np.full(15 * nk, -np.inf)]).astype(np.float32),
        "gamma": np.float32(np.log(tail)),
        "synthetic_248": np.float32(np.log1p(-tail)),
        "num_states": 16 * nk,
    }
    lens = rng.integers(min_len, max_len + 1, size=n_reads).astype(np.int64)
    data = rng.integers(0, 101, size=(n_reads, int(lens.max()))).astype(np.int8)
    seqs = {"data": data, "lens": lens, "maxlen": int(lens.max()), "num_instances": n_reads}
    return hmm, seqs


def _table_outputs(hmm, names, new):
    """Empty result arrays of the table kernels: `new(shape)` allocates float32 (NumPy or torch)."""
    S = hmm["num_states"]
    nk = hmm["output_prob"].shape[1]
    shapes = {"emit_max": (1,), "pemit": (hmm["output_prob"].shape[0], nk), "pstay": (S,), "pinit": (S,), "ptrans1": (nk, 4),
              "pdur": (16,), "pnext": (16,)}
    return {k: new(shapes[k]) for k in names}


def table_kernel_call(hmm, new, reference_format=False):
    """(jitted function, its arguments, its options) of the table kernel for a log-space model whose arrays are
    NumPy arrays or torch tensors; `new(shape)` allocates a float32 array of the same kind for a result."""
    names = ("emit_max", "pemit", "pinit", "ptrans1", "pdur", "pnext") if reference_format else ("emit_max", "pemit", "pstay", "pinit", "ptrans1")
    lin = _table_outputs(hmm, names, new)
    src = dict(hmm)
    src["num_obs"], src["num_kmers"] = int(hmm["output_prob"].shape[0]), int(hmm["output_prob"].shape[1])
    rowmax = new((src["num_obs"],))
    fn = scaled_reference_tables if reference_format else scaled_tables
    opts = parpy.par({"obs": parpy.threads(src["num_obs"]), "state": parpy.threads(256), "all": parpy.threads(src["num_states"]),
                      "layer": parpy.threads(16)})
    return fn, [src, lin, rowmax], opts


def scaled_tables_on_device(hd, reference_format=False, time_it=False):
    """Run the table kernel for a model whose log-space tables are torch tensors on the GPU and return the model
    dict that the linear-space forward passes take (the log-space tables stay in it).  With `time_it` the device
    time of the call in milliseconds is returned as well."""
    import torch
    dev = hd["output_prob"].device
    fn, args, opts = table_kernel_call(hd, lambda shape: torch.empty(shape, dtype=torch.float32, device=dev), reference_format)
    fn(*args, opts=opts)
    ms = parpy.time_call(fn, *args, opts=opts) if time_it else None
    out = dict(hd)
    out.update(args[1])
    return (out, ms) if time_it else out


def with_linear_tables(hmm):
    """The model with its transition tables also in linear space (`ptrans1`, `pstay`), as `forward_syn4` reads them.
    Host-side statement of what `scaled_tables` computes on the device: used where no GPU is there (code generation
    tests) and as the checker of the device tables."""
    out = dict(hmm)
    out["ptrans1"] = np.exp(hmm["trans1"].astype(np.float64)).astype(np.float32)
    out["pstay"] = np.exp(hmm["stay"].astype(np.float64)).astype(np.float32)
    return out


def with_scaled_tables(hmm):
    """Host-side statement of `scaled_tables` (see `with_linear_tables`): `ptrans1`, `pstay`, `pinit`, `emit_max` =
    the largest entry of the log-space emission table (one float32 element) and `pemit` = exp(output_prob - emit_max)."""
    out = with_linear_tables(hmm)
    out["pinit"] = np.exp(hmm["initial_prob"].astype(np.float64)).astype(np.float32)
    e = hmm["output_prob"].astype(np.float64)
    out["emit_max"] = np.array([e.max()], dtype=np.float32)
    out["pemit"] = np.exp(e - float(out["emit_max"][0])).astype(np.float32)
    return out


def with_scaled_reference_tables(hmm):
    """Host-side statement of `scaled_reference_tables` (see `with_linear_tables`)."""
    out = dict(hmm)
    out["ptrans1"] = np.exp(hmm["trans1"].astype(np.float64)).astype(np.float32)
    out["pdur"] = np.exp(hmm["trans2"].astype(np.float64)).astype(np.float32)
    tail = float(np.exp(np.float64(hmm["gamma"])))
    out["pnext"] = np.array([1.0] * 14 + [1.0 - tail, tail], dtype=np.float32)
    out["pinit"] = np.exp(hmm["initial_prob"].astype(np.float64)).astype(np.float32)
    e = hmm["output_prob"].astype(np.float64)
    out["emit_max"] = np.array([e.max()], dtype=np.float32)
    out["pemit"] = np.exp(e - float(out["emit_max"][0])).astype(np.float32)
    return out


def to_device(d, device="cuda"):
    """Move the arrays of a workload dict to torch tensors on `device`; ints stay Python ints."""
    import torch
    out = {}
    for key, v in d.items():
        if isinstance(v, np.ndarray):
            out[key] = torch.from_numpy(np.ascontiguousarray(v)).to(device)
        elif isinstance(v, (np.floating, float)):
            out[key] = torch.tensor(float(v), dtype=torch.float32, device=device)
        else:
            out[key] = v
    return out
