"""Pins the CPU oracle: golden vectors of the reference, closed forms, brute force.

The oracle is the checker for every GPU parity test, so it is itself checked
here against (i) the reference's golden files for the 3-mer and 5-mer models
(test/data/{3,5}mer-expected.txt, tolerance of test/test_forward.py:176-178),
(ii) identities the mathematics fixes, chosen so that a dropped term, a wrong
predecessor index or a transposed table breaks at least one of them, and
(iii) library routines (scipy / torch) for the plain numeric workloads.
"""
import itertools
import os

import numpy as np
import pytest
import scipy.special

import oracle
from parpy_amd import workloads as W


def _golden(golden_dir, k):
    hmm, seqs = oracle.reference_model_tables(os.path.join(golden_dir, f"hmm_{k}mer_model.npz"),
                                              os.path.join(golden_dir, "hmm_signals.npz"))
    exp = np.loadtxt(os.path.join(golden_dir, f"hmm_{k}mer_expected.txt"), dtype=np.float32)
    return hmm, seqs, exp


def test_fixture_layout(golden_dir):
    hmm, seqs, exp = _golden(golden_dir, 3)
    assert hmm["num_states"] == 16 * 64
    assert hmm["trans1"].shape == (64, 4) and hmm["output_prob"].shape == (101, 64)
    assert seqs["data"].shape == (100, 8885) and int(seqs["lens"].sum()) == 597998
    assert int(seqs["lens"].min()) == 2779 and exp.shape == (100,)
    # layer 0 starts uniform, every other layer is impossible
    assert np.allclose(hmm["initial_prob"][:64], np.log(1 / 64)) and np.all(np.isneginf(hmm["initial_prob"][64:]))


def test_reference_model_3mer_golden_f32(golden_dir):
    hmm, seqs, exp = _golden(golden_dir, 3)
    got = oracle.hmm_ref_forward(hmm, seqs, np.float32)
    assert np.allclose(got, exp, atol=1e-5, rtol=1e-5), np.abs(got - exp).max()


def test_reference_model_3mer_f64_agrees_within_fp32_drift(golden_dir):
    hmm, seqs, exp = _golden(golden_dir, 3)
    got = oracle.hmm_ref_forward(hmm, seqs, np.float64)
    # fp32 accumulates about 1e-4 relative drift over ~9000 steps; a wrong term is orders of magnitude away
    assert np.abs((got - exp) / exp).max() < 2e-4


def test_reference_model_5mer_golden_subset(golden_dir):
    hmm, seqs, exp = _golden(golden_dir, 5)
    sub = np.argsort(seqs["lens"])[:4]
    got = oracle.hmm_ref_forward(hmm, seqs, np.float32, subset=sub)
    assert np.allclose(got, exp[sub], atol=1e-5, rtol=1e-5), np.abs(got - exp[sub]).max()


def test_reverse_kmer_index():
    assert [oracle.reverse_kmer_index(i, 2) for i in range(16)] == [0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15]
    for k in (1, 3, 4):
        idx = [oracle.reverse_kmer_index(i, k) for i in range(4 ** k)]
        assert sorted(idx) == list(range(4 ** k))
        assert all(oracle.reverse_kmer_index(j, k) == i for i, j in enumerate(idx))


@pytest.mark.parametrize("k", [1, 2, 3])
def test_synthetic_predecessor_structure(k):
    S = 4 ** k
    pred = oracle.syn_predecessors(S)
    # four distinct predecessors per state; every state is the predecessor of exactly four states
    assert all(len(set(pred[:, s])) == 4 for s in range(S))
    assert np.array_equal(np.bincount(pred.reshape(-1), minlength=S), np.full(S, 4))
    # shifting in one base: the predecessor's low k-1 digits are the state's high k-1 digits
    for s in range(S):
        for j in range(4):
            assert pred[j, s] % (S // 4) == s // 4 and pred[j, s] // (S // 4) == j


def test_synthetic_zero_emissions_conserve_mass():
    # outgoing transitions of every state sum to one, so without emissions the total mass stays 1
    hmm, seqs = W.synthetic_hmm(3, n_inst=6, min_len=50, max_len=400, emissions=0.0)
    got = oracle.hmm_syn_forward(hmm, seqs, np.float64)
    # the tables hold float32 logarithms, so each row sums to one only to ~1e-7 per step
    assert np.abs(got).max() < 1e-4
    got32 = oracle.hmm_syn_forward(hmm, seqs, np.float32)
    assert np.abs(got32).max() < 1e-3


def test_synthetic_constant_emissions_give_len_times_c():
    c = np.float32(np.log(0.25))
    hmm, seqs = W.synthetic_hmm(2, n_inst=5, min_len=10, max_len=60, emissions=c)
    got = oracle.hmm_syn_forward(hmm, seqs, np.float64)
    # + log(1/S) from the uniform start folded in: sum_s init[s] = 1, so LL = len * c exactly in real arithmetic
    assert np.allclose(got, seqs["lens"] * float(c), rtol=0, atol=1e-4)


def test_synthetic_single_step_is_logsumexp():
    hmm, seqs = W.synthetic_hmm(3, n_inst=4, min_len=1, max_len=1)
    got = oracle.hmm_syn_forward(hmm, seqs, np.float64)
    want = [scipy.special.logsumexp(hmm["initial_prob"].astype(np.float64) +
                                    hmm["output_prob"][seqs["data"][i, 0]].astype(np.float64)) for i in range(4)]
    assert np.allclose(got, want, atol=1e-12)


@pytest.mark.parametrize("k,length", [(1, 6), (2, 4)])
def test_synthetic_bruteforce_path_enumeration(k, length):
    hmm, seqs = W.synthetic_hmm(k, n_inst=3, min_len=length, max_len=length)
    got = oracle.hmm_syn_forward(hmm, seqs, np.float64)
    for i in range(3):
        want = oracle.hmm_syn_bruteforce(hmm, seqs["data"][i], length)
        assert abs(got[i] - want) < 1e-9


def test_synthetic_c_and_numpy_restatements_agree():
    hmm, seqs = W.synthetic_hmm(3, n_inst=3, min_len=20, max_len=40)
    got = oracle.hmm_syn_forward(hmm, seqs, np.float64)
    for i in range(3):
        assert abs(got[i] - oracle.hmm_syn_forward_numpy(hmm, seqs["data"][i], int(seqs["lens"][i]))) < 1e-9


def test_synthetic_all_neg_inf_stays_neg_inf():
    # fmax(NaN, -inf) = -inf repairs log(0) - (-inf): unreachable states stay at -inf
    hmm, seqs = W.synthetic_hmm(2, n_inst=2, min_len=3, max_len=5)
    hmm["initial_prob"][:] = -np.inf
    got, alpha = oracle.hmm_syn_forward(hmm, seqs, np.float32, return_alpha=True)
    assert np.all(np.isneginf(alpha))


def test_max_steps_truncates_like_shorter_reads():
    hmm, seqs = W.synthetic_hmm(2, n_inst=4, min_len=30, max_len=50)
    short = dict(seqs, lens=np.minimum(seqs["lens"], 12))
    assert np.array_equal(oracle.hmm_syn_forward(hmm, seqs, np.float32, max_steps=12),
                          oracle.hmm_syn_forward(hmm, short, np.float32))


def test_row_reduce_and_softmax_against_library():
    import torch
    rng = np.random.default_rng(0)
    x = rng.standard_normal((7, 33)).astype(np.float32)
    assert np.allclose(oracle.row_reduce(x, "sum"), x.astype(np.float64).sum(1))
    assert np.allclose(oracle.row_reduce(x, "max"), x.max(1)) and np.allclose(oracle.row_reduce(x, "min"), x.min(1))
    assert np.allclose(oracle.row_reduce(np.ones((3, 4)) * 2, "prod"), 16.0)
    sm = oracle.softmax_rows(x)
    assert np.allclose(sm, torch.softmax(torch.from_numpy(x).double(), 1).numpy(), atol=1e-14)
    assert np.allclose(oracle.softmax_rows(np.full((2, 8), 3.0)), 1 / 8)


def test_sddmm_against_dense_product():
    A, B, crows, cols, vals = W.make_sddmm(64, 8, 0.1)
    rows = oracle.csr_rows(crows)
    assert len(rows) == len(cols) == int(0.1 * 64 * 64)
    assert all(np.all(np.diff(cols[crows[r]:crows[r + 1]]) > 0) for r in range(64))   # sorted, no duplicates
    dense = A.astype(np.float64) @ B.astype(np.float64)
    got = oracle.sddmm(A, B, rows, cols, vals, alpha=1.5, beta=2.0)
    assert np.allclose(got, 1.5 * dense[rows, cols] + 2.0 * vals, atol=1e-12)
    eye = np.eye(8, dtype=np.float32)
    assert np.allclose(oracle.sddmm(eye, eye, np.arange(8), np.arange(8)), 1.0)
    assert np.allclose(oracle.sddmm(eye, eye, np.arange(8), (np.arange(8) + 1) % 8), 0.0)


def test_product_side_model_loader_agrees_with_the_oracle(golden_dir):
    """Two independent restatements of the reference's table layout (test/test_forward.py:31-77)."""
    import os
    from parpy_amd import workloads as W
    for k in (3, 5):
        paths = (os.path.join(golden_dir, f"hmm_{k}mer_model.npz"), os.path.join(golden_dir, "hmm_signals.npz"))
        a, b = oracle.reference_model_tables(*paths), W.load_reference_model(*paths)
        for da, db in zip(a, b):
            assert sorted(da) == sorted(db)
            for key in da:
                assert np.array_equal(np.asarray(da[key]), np.asarray(db[key])), (k, key)


def test_synthetic_forward_with_state_independent_emissions_and_an_impossible_observation():
    """Emissions that do not depend on the state: the transitions conserve the total probability, so the
    log-likelihood is the sum of the emission logarithms of the read.  An observation of probability zero in every
    state makes every score -inf; the closing log-sum-exp of the reference's kernel then computes -inf - (-inf) and
    ends in NaN (test/test_forward.py:155-160 has no repair there, unlike the step), which the oracle reproduces."""
    from parpy_amd import workloads as W
    hmm, seqs = W.synthetic_hmm(3, n_inst=3, min_len=40, max_len=40, seed=5)
    S = hmm["num_states"]
    table = np.full((101, S), -np.inf, dtype=np.float32)
    table[0, :] = np.log(0.5)
    table[1, :] = np.log(0.5) - 7.0
    hmm["output_prob"] = table
    rng = np.random.default_rng(5)
    seqs["data"] = rng.integers(0, 2, size=seqs["data"].shape).astype(np.int8)
    closed = np.array([table[seqs["data"][i].astype(int), 0].astype(np.float64).sum() for i in range(3)])
    for prec, tol in ((np.float64, 1e-9), (np.float32, 1e-3)):
        got = oracle.hmm_syn_forward(hmm, seqs, prec)
        assert np.abs(got - closed).max() < tol * np.abs(closed).max()
    seqs["data"][2, 17] = 2
    for prec in (np.float64, np.float32):
        got = oracle.hmm_syn_forward(hmm, seqs, prec)
        assert np.isnan(got[2]) and np.all(np.isfinite(got[:2]))
