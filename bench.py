"""Benchmark of the compiled hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload hmm7|hmm5|hmm5ref|rowsum|softmax|sddmm|copy]

A step is one pass of the compiled function over one batch of seeded synthetic
input that is already resident in HBM.  The default workload is the headline
one: the 7-mer HMM forward batch (4^7 = 16384 states, 100 reads of 5000..15000
samples).  One JSON line is printed; it carries the roofline of the dominant
kernel (algorithmic bytes / measured kernel time against the 8 TB/s HBM peak)
and a CPU baseline (the C oracle on the host cores, bounded sample).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


def _events_ms(fn, timed, steps, warmup, torch):
    """Run fn warmup+steps times between synchronisations -> wall ms per step; then
    `steps` more runs bracketed by HIP events on the launch stream -> device ms list."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) * 1e3 / steps
    return wall, [timed() for _ in range(steps)]


def bench_hmm(k, args, torch, parpy, W):
    import numpy as np
    hmm, seqs = W.synthetic_hmm(k)
    S, n = hmm["num_states"], seqs["num_instances"]
    hd, sd = W.to_device(hmm), W.to_device(seqs)
    a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
    a2 = torch.zeros_like(a1)
    res = torch.zeros(n, dtype=torch.float32, device="cuda")
    nthreads = min(S, args.state_threads)
    opts = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(nthreads)})
    _apply_opt_flags(opts, args)
    opts.use_cuda_graphs = bool(args.use_graphs)
    fn = lambda: W.forward_syn(hd, sd, res, a1, a2, opts=opts)
    timed = lambda: parpy.time_call(W.forward_syn, hd, sd, res, a1, a2, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    steps_total = int((seqs["lens"] - 1).sum())
    # per (sequence, step): read alpha (4S) + write alpha (4S) + emission row (4S) + the observation byte
    alg_bytes = (12 * S + 1) * steps_total
    kernel_ms = float(np.median(dev))
    cpu = None
    if not args.no_cpu:
        import oracle
        sample_steps = args.cpu_steps or (15000 if k <= 5 else 5000)   # about 2 s (5-mer) and 10 s (7-mer) on 16 cores
        t0 = time.perf_counter()
        oracle.hmm_syn_forward(hmm, seqs, np.float32, max_steps=sample_steps)
        dt = time.perf_counter() - t0
        done = int((np.minimum(seqs["lens"], sample_steps) - 1).sum())
        cpu = {"value": dt * 1e3 * steps_total / done, "unit": "ms/batch", "cores": os.cpu_count(), "kind": "port",
               "sample": f"first {sample_steps} samples of each of the {n} reads with the C oracle "
                         f"(OpenMP over reads), {dt:.1f} s measured, scaled by total steps {steps_total}/{done}"}
    ll = res.cpu().numpy()
    return {
        "metric": f"HMM-forward {k}-mer ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": wall, "unit": "ms/batch", "ms_per_step": wall, "higher_is_better": False,
        "dtype": "f32",
        "config": {"workload": f"hmm_forward_{k}mer_synthetic", "states": S, "reads": n, "min_len": 5000,
                   "max_len": 15000, "total_steps": steps_total, "state_threads": nthreads, "graph_replay": bool(args.use_graphs),
                   "mean_loglik": float(ll.mean())},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg_bytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "kernel_ms": kernel_ms, "algorithmic_bytes": alg_bytes},
        "cpu_baseline": cpu,
    }


def bench_hmm_ref(args, torch, parpy, W):
    """The reference's own 5-mer model (16 duration layers x 1024 k-mers = 16384 states) on its 100
    recorded reads, tables from tests/golden: the configuration its benchmark validates
    (benchmarks/forward.py:481-518).  Results are checked against the expected log-likelihoods."""
    import numpy as np
    g = os.path.join(ROOT, "tests", "golden")
    hmm, seqs = W.load_reference_model(os.path.join(g, "hmm_5mer_model.npz"), os.path.join(g, "hmm_signals.npz"))
    want = np.loadtxt(os.path.join(g, "hmm_5mer_expected.txt"), dtype=np.float32)
    S, n = hmm["num_states"], seqs["num_instances"]
    hd, sd = W.to_device(hmm), W.to_device(seqs)
    a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
    a2 = torch.zeros_like(a1)
    res = torch.zeros(n, dtype=torch.float32, device="cuda")
    nthreads = min(S, args.state_threads)
    opts = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(nthreads)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.forward_kernel(hd, sd, a1, a2, res, opts=opts)
    timed = lambda: parpy.time_call(W.forward_kernel, hd, sd, a1, a2, res, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    got = res.cpu().numpy()
    assert np.allclose(got, want, atol=1e-5, rtol=1e-5), float(np.abs(got - want).max())
    steps_total = int((seqs["lens"] - 1).sum())
    # per (read, step): alpha read + alpha write (4S each), one emission row of S/16 k-mers, the observation byte
    alg_bytes = (8 * S + 4 * (S // 16) + 1) * steps_total
    kernel_ms = float(np.median(dev))
    return {
        "metric": "HMM-forward reference 5-mer model ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": wall, "unit": "ms/batch", "ms_per_step": wall, "higher_is_better": False, "dtype": "f32",
        "config": {"workload": "hmm_forward_reference_5mer_model", "states": S, "reads": n, "min_len": int(seqs["lens"].min()),
                   "max_len": int(seqs["lens"].max()), "total_steps": steps_total, "state_threads": nthreads,
                   "mean_loglik": float(got.mean())},
        "roofline": {"bound": "hbm", "achieved": alg_bytes / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": alg_bytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None,
                     "kernel_ms": kernel_ms, "algorithmic_bytes": alg_bytes},
        "cpu_baseline": None,
    }


def bench_rowsum(args, torch, parpy, W):
    import numpy as np
    N, M = 1024, 65536
    args.inner_threads = args.inner_threads or 1024  # one full workgroup per row (any choice from 64 up measures within 5 %)
    x = W.make_rowsum(N, M)
    xd = torch.from_numpy(x).cuda()
    out = torch.zeros(N, dtype=torch.float32, device="cuda")
    opts = parpy.par({"outer": parpy.threads(N), "inner": parpy.threads(args.inner_threads)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.sum_rows(xd, out, N, opts=opts)
    timed = lambda: parpy.time_call(W.sum_rows, xd, out, N, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    alg = N * M * 4 + N * 4
    kernel_ms = float(np.median(dev))
    cpu = None
    if not args.no_cpu:
        t0 = time.perf_counter()
        for _ in range(3):
            np.sum(x, axis=1, dtype=np.float32)
        cpu = {"value": (time.perf_counter() - t0) / 3 * 1e3, "unit": "ms/batch", "cores": 1, "kind": "port",
               "sample": "np.sum(x, axis=1) on the full 1024x65536 matrix, mean of 3"}
    return {"metric": "row-sum 1024x65536 f32 ms + achieved HBM GB/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "rowsum_1024x65536", "inner_threads": args.inner_threads},
            "roofline": {"bound": "hbm", "achieved": alg / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": alg / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel_ms": kernel_ms,
                         "algorithmic_bytes": alg},
            "cpu_baseline": cpu}


def bench_softmax(args, torch, parpy, W):
    import numpy as np
    N, M = 16384, 4096
    args.inner_threads = args.inner_threads or 512   # 8 elements (two dwordx4) per thread, 4 workgroups per CU
    x = W.make_softmax(N, M)
    xd = x.cuda()
    out = torch.zeros_like(xd)
    opts = parpy.par({"N": parpy.threads(N), "M": parpy.threads(args.inner_threads)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.softmax(xd, N, M, out, opts=opts)
    timed = lambda: parpy.time_call(W.softmax, xd, N, M, out, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    alg = 2 * N * M * 4
    kernel_ms = float(np.median(dev))
    cpu = None
    if not args.no_cpu:
        t0 = time.perf_counter()
        for _ in range(3):
            torch.softmax(x, 1)
        cpu = {"value": (time.perf_counter() - t0) / 3 * 1e3, "unit": "ms/batch", "cores": torch.get_num_threads(),
               "kind": "port", "sample": "torch.softmax(x, 1) on the full 16384x4096 matrix, mean of 3"}
    return {"metric": "softmax 16384x4096 f32 ms + achieved HBM GB/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "softmax_16384x4096", "inner_threads": args.inner_threads},
            "roofline": {"bound": "hbm", "achieved": alg / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": alg / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel_ms": kernel_ms,
                         "algorithmic_bytes": alg},
            "cpu_baseline": cpu}


def bench_sddmm(args, torch, parpy, W):
    import numpy as np
    A, B, crows, cols, vals = W.make_sddmm()
    nnz = len(cols)
    Ad, Bd = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    # per-non-zero row ids from the CSR row pointers, with the compiled decompression kernel
    # (benchmarks/sddmm.py:21-27,108-114 of the reference), outside the timed region
    rows_d = torch.zeros(nnz, dtype=torch.int64, device="cuda")
    W.sddmm_decompress_csr(torch.from_numpy(crows).cuda(), rows_d, A.shape[0],
                           opts=parpy.par({"N": parpy.threads(A.shape[0]), "M": parpy.threads(64)}))
    C = {"rows": rows_d, "cols": torch.from_numpy(cols).cuda(), "values": torch.from_numpy(vals).cuda(), "nnz": nnz}
    D = torch.zeros(nnz, dtype=torch.float32, device="cuda")
    one = torch.tensor(1.0, dtype=torch.float32)
    zero = torch.tensor(0.0, dtype=torch.float32)
    opts = parpy.par({"nnz": parpy.threads(nnz).tpb(args.tpb)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.sddmm_coo(Ad, Bd, C, D, one, zero, opts=opts)
    timed = lambda: parpy.time_call(W.sddmm_coo, Ad, Bd, C, D, one, zero, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    kernel_ms = float(np.median(dev))
    flops = 2 * A.shape[1] * nnz
    alg = A.nbytes + B.nbytes + cols.nbytes + nnz * 8 + vals.nbytes + nnz * 4
    cpu = None
    if not args.no_cpu:
        import oracle
        rows = rows_d.cpu().numpy()
        t0 = time.perf_counter()
        oracle.sddmm(A.astype(np.float32), B.astype(np.float32), rows, cols)
        cpu = {"value": (time.perf_counter() - t0) * 1e3, "unit": "ms/batch", "cores": 1, "kind": "port",
               "sample": "chunked NumPy einsum over all non-zeros"}
    return {"metric": "SDDMM 8192x128x8192 1% ms + GFLOP/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32", "config": {"workload": "sddmm_8192_k128_1pct", "nnz": nnz, "tpb": args.tpb},
            "roofline": {"bound": "hbm", "achieved": alg / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": alg / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel_ms": kernel_ms,
                         "algorithmic_bytes": alg, "gflops": flops / (kernel_ms * 1e-3) / 1e9},
            "cpu_baseline": cpu}


def bench_copy(args, torch, parpy, W):
    """Plain device copy of 256 MiB compiled from `out[:] = x[:]`: the calibration kernel for the HBM counters."""
    import numpy as np
    n = 64 * 1024 * 1024
    x = torch.arange(n, dtype=torch.float32, device="cuda")
    out = torch.zeros_like(x)
    opts = parpy.par({"N": parpy.threads(n // 16).tpb(256)})
    fn = lambda: W.copy_1d(x, out, opts=opts)
    timed = lambda: parpy.time_call(W.copy_1d, x, out, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    assert torch.equal(x, out)
    alg = 2 * n * 4
    kernel_ms = float(np.median(dev))
    return {"metric": "device copy 256 MiB ms + achieved HBM GB/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32", "config": {"workload": "copy_256MiB"},
            "roofline": {"bound": "hbm", "achieved": alg / (kernel_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": alg / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, "traffic": None, "kernel_ms": kernel_ms,
                         "algorithmic_bytes": alg},
            "cpu_baseline": None}


def _profiled_traffic(name):
    """HBM bytes per launch from the committed rocprofv3 counter summary of this kernel, or None."""
    import re
    path = os.path.join(ROOT, "profiles", f"{name}_kernel.md")
    try:
        m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", open(path).read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def _apply_opt_flags(opts, args):
    for name in ("opt_vectorize", "opt_lds_rows", "opt_reg_cache", "opt_hoist_invariant", "opt_narrow_index", "opt_unswitch", "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_unswitch_uniform", "opt_offset32", "opt_if_convert", "opt_noalias_scopes", "opt_mfma_sddmm"):
        v = getattr(args, name)
        if v is not None:
            setattr(opts, name, bool(v))
    if args.reg_budget:
        opts.reg_budget = args.reg_budget


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="hmm7", choices=["hmm7", "hmm5", "hmm5ref", "rowsum", "softmax", "sddmm", "copy"])
    ap.add_argument("--state-threads", type=int, default=1024)
    ap.add_argument("--use-graphs", type=int, default=0, help="replay the launches of a run from a HIP graph (host-hoisted time loops)")
    ap.add_argument("--inner-threads", type=int, default=None)
    ap.add_argument("--tpb", type=int, default=256)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-steps", type=int, default=0, help="samples per read for the HMM CPU baseline")
    for name in ("opt_vectorize", "opt_lds_rows", "opt_reg_cache", "opt_hoist_invariant", "opt_narrow_index", "opt_unswitch", "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_unswitch_uniform", "opt_offset32", "opt_if_convert", "opt_noalias_scopes", "opt_mfma_sddmm"):
        ap.add_argument("--" + name.replace("_", "-"), dest=name, type=int, default=None)
    ap.add_argument("--reg-budget", type=int, default=0)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the batch would shard by reads "
              "with no exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no ROCm device is visible", file=sys.stderr)
        sys.exit(1)
    import parpy_amd as parpy
    from parpy_amd import workloads as W

    if args.workload == "hmm7":
        r = bench_hmm(7, args, torch, parpy, W)
    elif args.workload == "hmm5":
        r = bench_hmm(5, args, torch, parpy, W)
    elif args.workload == "hmm5ref":
        r = bench_hmm_ref(args, torch, parpy, W)
    elif args.workload == "rowsum":
        r = bench_rowsum(args, torch, parpy, W)
    elif args.workload == "softmax":
        r = bench_softmax(args, torch, parpy, W)
    elif args.workload == "copy":
        r = bench_copy(args, torch, parpy, W)
    else:
        r = bench_sddmm(args, torch, parpy, W)
    default_cfg = not any(getattr(args, n) is not None for n in ("opt_vectorize", "opt_lds_rows", "opt_reg_cache",
                                                                 "opt_hoist_invariant", "opt_narrow_index", "opt_unswitch", "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_unswitch_uniform", "opt_offset32", "opt_if_convert", "opt_noalias_scopes", "opt_mfma_sddmm"))
    if default_cfg and not args.reg_budget:
        r["roofline"]["traffic"] = _profiled_traffic(args.workload)
    r.update({"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "scaling": "weak", "vs_baseline": None,
              "data": "reference fixtures (tests/golden)" if args.workload == "hmm5ref" else "synthetic"})
    print(json.dumps(r))


if __name__ == "__main__":
    main()
