"""TEST INFRASTRUCTURE ONLY: CPU oracle for the five hot-path workloads.

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this package.  It restates on the CPU what the
reference computes on the GPU for each workload, each function citing the
reference lines it follows (paths relative to /root/reference):

* row reductions  -- test/test_reduce.py:12-70 (sum/prod/max/min over rows),
  neutral elements src/utils/reduce.rs:75-88.
* softmax         -- test/test_softmax.py:11-26 (oracle there: torch.softmax).
* SDDMM           -- benchmarks/sddmm.py:18-19,63-70.
* HMM forward     -- test/test_forward.py:11-160 (table layout + recurrence);
  heavy lifting in hmm_oracle.c (built into liboracle.so by build()).

Pinning status: the reference-model HMM path is pinned by the golden files
test/data/{3mer,5mer}-expected.txt; the synthetic HMM by closed forms and
path-enumeration brute force (tests/test_oracle.py); reductions, softmax and
SDDMM by NumPy / PyTorch library routines.  7-mer *reference-model* parity is
unpinned: test/data/7mer-model.hdf5 is absent from the reference checkout.
"""
import ctypes
import hashlib
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


_GCC = ["gcc", "-O2", "-fopenmp", "-shared", "-fPIC"]


def _source_stamp(src):
    h = hashlib.sha256(" ".join(_GCC).encode())
    with open(src, "rb") as f:
        h.update(f.read())
    return h.hexdigest()


def build(force=False):
    """Compile hmm_oracle.c into liboracle.so (gcc, OpenMP); rebuilt when the source's content changed."""
    src = os.path.join(_HERE, "hmm_oracle.c")
    stamp = _LIB_PATH + ".srchash"
    current = False
    if os.path.exists(_LIB_PATH) and os.path.exists(stamp):
        with open(stamp) as f:
            current = f.read().strip() == _source_stamp(src)
    if force or not current:
        subprocess.run(_GCC + ["-o", _LIB_PATH, src, "-lm"], check=True)
        with open(stamp, "w") as f:
            f.write(_source_stamp(src))
    return _LIB_PATH


def _load():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


# --------------------------------------------------------------------------
# Reductions / softmax / SDDMM (library routines are the oracle)
# --------------------------------------------------------------------------

def row_reduce(x, op="sum", dtype=np.float64):
    """test/test_reduce.py:12-34 -- out[i] = op(x[i, :]); accumulates in `dtype`."""
    f = {"sum": np.sum, "prod": np.prod, "max": np.max, "min": np.min}[op]
    return f(x.astype(dtype), axis=1)


def softmax_rows(x):
    """test/test_softmax.py:11-26 in float64 (max-shift, exp, sum, divide)."""
    x = np.asarray(x, dtype=np.float64)
    e = np.exp(x - x.max(axis=1, keepdims=True))
    return e / e.sum(axis=1, keepdims=True)


def sddmm(A, B, rows, cols, vals=None, alpha=1.0, beta=0.0, chunk=1 << 16):
    """benchmarks/sddmm.py:63-70 -- D[i] = alpha * dot(A[rows[i],:], B[:,cols[i]]) + beta*vals[i], fp64."""
    A = np.asarray(A, dtype=np.float64)
    Bt = np.ascontiguousarray(np.asarray(B, dtype=np.float64).T)
    out = np.empty(len(rows), dtype=np.float64)
    for s in range(0, len(rows), chunk):
        e = min(len(rows), s + chunk)
        out[s:e] = np.einsum("ik,ik->i", A[rows[s:e]], Bt[cols[s:e]])
    out *= alpha
    if vals is not None:
        out += beta * np.asarray(vals, dtype=np.float64)
    return out


def csr_rows(crows):
    """benchmarks/sddmm.py:21-27 -- decompress CSR row pointers to per-nnz row ids."""
    crows = np.asarray(crows)
    return np.repeat(np.arange(len(crows) - 1, dtype=np.int64), np.diff(crows))


# --------------------------------------------------------------------------
# HMM: reference (16-layer) model
# --------------------------------------------------------------------------

def reverse_kmer_index(i, k):
    """test/test_forward.py:20-21 -- reverse the base-4 digits of a k-mer index."""
    r = 0
    for x in range(k):
        r += (i // 4 ** x) % 4 * 4 ** (k - x - 1)
    return r


def reference_model_tables(model_npz, signals_npz):
    """Build the kernel's input tables from the raw fixture tables.

    Follows test/test_forward.py:31-77: log of the stored probabilities,
    trans1 = log(T).reshape(4, 4^k).T, output_prob[j, i] = log(obs)[j, rev(i)],
    initial_prob = log(1/4^k) in layer 0 and -inf elsewhere,
    synthetic_248 = log(1 - tail), num_states = 16 * 4^k; signals zero-padded
    to the longest read as int8.
    """
    m = np.load(model_npz)
    k = int(m["k"])
    K = 4 ** k
    with np.errstate(divide="ignore"):
        obs = np.log(m["obs"])
    trans1 = np.log(m["trans"]).reshape(4, K).transpose(1, 0)
    duration = np.log(m["duration"])
    tail = np.log(m["tail_factor"])
    rev = np.array([reverse_kmer_index(i, k) for i in range(K)])
    out_prob = obs[:, rev]                      # [101, K]; == transform_output_probs(...).T.T
    init = np.full((16, K), -np.inf, dtype=np.float32)
    init[0, :] = np.log(1.0 / float(K))
    syn248 = np.log(np.exp(0.0) - np.exp(tail))
    hmm = {
        "gamma": np.float32(tail),
        "trans1": np.ascontiguousarray(trans1, dtype=np.float32),
        "trans2": duration.astype(np.float32),
        "output_prob": np.ascontiguousarray(out_prob, dtype=np.float32),
        "initial_prob": init.reshape(-1),
        "synthetic_248": np.float32(syn248),
        "num_states": 16 * K,
    }
    s = np.load(signals_npz)
    lens = s["lens"].astype(np.int64)
    maxlen = int(lens.max())
    data = np.zeros((len(lens), maxlen), dtype=np.int8)
    ofs = 0
    for i, n in enumerate(lens):
        data[i, :n] = s["samples"][ofs:ofs + n].astype(np.int8)
        ofs += n
    seqs = {"data": data, "lens": lens, "maxlen": maxlen, "num_instances": len(lens)}
    return hmm, seqs


def hmm_ref_forward(hmm, seqs, dtype=np.float32, subset=None, return_alpha=False):
    """Reference-model forward pass (test/test_forward.py:83-160) via hmm_oracle.c."""
    lib = _load()
    T = np.dtype(dtype)
    fn = lib.hmm_ref_forward_f32 if T == np.float32 else lib.hmm_ref_forward_f64
    cT = ctypes.c_float if T == np.float32 else ctypes.c_double
    data, lens = seqs["data"], seqs["lens"]
    if subset is not None:
        data = np.ascontiguousarray(data[subset])
        lens = np.ascontiguousarray(lens[subset])
    n, maxlen = data.shape
    S = int(hmm["num_states"])
    t1 = np.ascontiguousarray(hmm["trans1"], dtype=T)
    t2 = np.ascontiguousarray(hmm["trans2"], dtype=T)
    em = np.ascontiguousarray(hmm["output_prob"], dtype=T)
    ini = np.ascontiguousarray(hmm["initial_prob"], dtype=T)
    out = np.empty(n, dtype=T)
    alpha = np.empty((n, S), dtype=T) if return_alpha else None
    fn.argtypes = [ctypes.c_int64] + [ctypes.c_void_p] * 4 + [cT, cT] + \
        [ctypes.c_void_p] * 2 + [ctypes.c_int64] * 2 + [ctypes.c_void_p] * 2
    fn.restype = None
    fn(S, _ptr(t1), _ptr(t2), _ptr(em), _ptr(ini), cT(float(hmm["gamma"])),
       cT(float(hmm["synthetic_248"])), _ptr(data), _ptr(lens), n, maxlen,
       _ptr(out), _ptr(alpha))
    return (out, alpha) if return_alpha else out


# --------------------------------------------------------------------------
# HMM: synthetic single-layer model
# --------------------------------------------------------------------------

def syn_predecessors(S):
    """pred[j, s] = j*S/4 + s//4 -- the four de Bruijn shift predecessors of state s."""
    s = np.arange(S, dtype=np.int64)
    return np.stack([j * (S // 4) + s // 4 for j in range(4)])


def hmm_syn_forward(hmm, seqs, dtype=np.float32, max_steps=0, subset=None,
                    return_alpha=False):
    """Synthetic-model forward pass via hmm_oracle.c (max_steps>0 truncates every read)."""
    lib = _load()
    T = np.dtype(dtype)
    fn = lib.hmm_syn_forward_f32 if T == np.float32 else lib.hmm_syn_forward_f64
    data, lens = seqs["data"], seqs["lens"]
    if subset is not None:
        data = np.ascontiguousarray(data[subset])
        lens = np.ascontiguousarray(lens[subset])
    n, maxlen = data.shape
    S = int(hmm["num_states"])
    t1 = np.ascontiguousarray(hmm["trans1"], dtype=T)
    st = np.ascontiguousarray(hmm["stay"], dtype=T)
    em = np.ascontiguousarray(hmm["output_prob"], dtype=T)
    ini = np.ascontiguousarray(hmm["initial_prob"], dtype=T)
    out = np.empty(n, dtype=T)
    alpha = np.empty((n, S), dtype=T) if return_alpha else None
    fn.argtypes = [ctypes.c_int64] + [ctypes.c_void_p] * 6 + [ctypes.c_int64] * 3 + \
        [ctypes.c_void_p] * 2
    fn.restype = None
    fn(S, _ptr(t1), _ptr(st), _ptr(em), _ptr(ini), _ptr(data),
       _ptr(np.ascontiguousarray(lens, dtype=np.int64)), n, maxlen, int(max_steps),
       _ptr(out), _ptr(alpha))
    return (out, alpha) if return_alpha else out


def hmm_syn_forward_numpy(hmm, data, length, dtype=np.float64):
    """Plain NumPy statement of the synthetic recurrence for ONE sequence (small cases)."""
    S = int(hmm["num_states"])
    t1 = hmm["trans1"].astype(dtype)
    st = hmm["stay"].astype(dtype)
    em = hmm["output_prob"].astype(dtype)
    pred = syn_predecessors(S)
    s = np.arange(S)
    a = hmm["initial_prob"].astype(dtype) + em[data[0]]
    for t in range(1, length):
        p = np.stack([t1[pred[j], s % 4] + a[pred[j]] for j in range(4)] + [st + a])
        m = np.fmax.reduce(p, axis=0)
        with np.errstate(invalid="ignore"):
            l = m + np.log(np.exp(p - m).sum(axis=0))
        a = np.fmax(l, -np.inf) + em[data[t]]
    m = a.max()
    return m + np.log(np.exp(a - m).sum())


def hmm_syn_bruteforce(hmm, data, length):
    """Sum over every state path (fp64, linear space).  Only for S**length small."""
    import itertools
    S = int(hmm["num_states"])
    t1 = np.exp(hmm["trans1"].astype(np.float64))
    st = np.exp(hmm["stay"].astype(np.float64))
    em = np.exp(hmm["output_prob"].astype(np.float64))
    ini = np.exp(hmm["initial_prob"].astype(np.float64))
    A = np.zeros((S, S))                       # A[r, s] = P(r -> s)
    for s in range(S):
        for j in range(4):
            r = j * (S // 4) + s // 4
            A[r, s] += t1[r, s % 4]
        A[s, s] += st[s]
    total = 0.0
    for path in itertools.product(range(S), repeat=length):
        p = ini[path[0]] * em[data[0], path[0]]
        for t in range(1, length):
            p *= A[path[t - 1], path[t]] * em[data[t], path[t]]
        total += p
    return np.log(total)
