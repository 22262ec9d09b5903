"""Benchmark of the compiled hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload all|hmm7|hmm5|hmm5ref|hmm7ref|rowsum|softmax|sddmm|copy|ldsrates|valurates] [--form scaled|grouped|reference]

A step is one pass of the compiled function over one batch of seeded synthetic
input that is already resident in HBM.  The default run (`all`) times the
headline workload -- the 7-mer HMM forward batch (4^7 = 16384 states, 100 reads
of 5000..15000 samples) -- and then the other configurations, whose records go
under `secondary` of the same JSON line.  Every record carries the roofline of
its dominant kernel (algorithmic bytes or flops / measured kernel time against
the published peak) and a CPU baseline timed on the host cores (bounded sample).

The HMM forward pass is timed in three statements of the same recurrence, all
written as ParPy user code in parpy_amd/workloads.py: `scaled` (forward_scaled:
linear space with rescaling, float64 result, the one that meets the 1e-4
tolerance against the fp64 oracle and the `value` of the headline), `grouped`
(forward_syn4: log space, the four states that share their predecessors updated
together) and `reference` (forward_syn: log space, one state at a time, the
structure of the reference's kernel).  The figures of the other forms are in
the record too.  The reference's own 16-layer model (`hmm5ref`) is timed as its
kernel (forward_kernel) and in the scaled form (forward_kernel_scaled).  Results
are checked against the oracle outside the timed region.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
FP32_MATRIX_PEAK_TFLOPS = 157.3

OPT_FLAGS = ("opt_vectorize", "opt_lds_rows", "opt_reg_cache", "opt_hoist_invariant", "opt_narrow_index", "opt_unswitch",
             "opt_gather_transpose", "opt_nontemporal", "opt_lane_split", "opt_drop_barriers", "opt_unswitch_uniform",
             "opt_offset32", "opt_if_convert", "opt_noalias_scopes", "opt_mfma_sddmm", "opt_expand_short_loops",
             "opt_guard_bounds", "opt_prefetch_steps", "opt_pack_accesses", "opt_share_iterations", "opt_fence_iterations")

# Vector-ALU instructions per state and step in the time loop of the generated HMM kernels (counted in the ISA of
# the kernels as compiled for these shapes: full-rate instructions, and v_exp_f32 / v_log_f32), and the issue times
# of the two classes measured with register-only microkernels on this part (4 waves per SIMD; `--workload valurates`).  One workgroup of 16
# waves per read puts S / 256 rows of 64 states on each SIMD.
VALU_NS = {"full": 1.02, "trans": 3.63}   # with 100 compute units busy, as in the HMM launches (1.15 / 3.77 with all 256)
HMM_VALU_MIX = {
    "reference": {"full": 24.0, "trans": 6.0},
    "grouped": {"full": 14.2, "trans": 3.0},
    "scaled": {"full": 8.4, "trans": 0.0},
}
HMM_FORMS = {"scaled": "forward_scaled", "grouped": "forward_syn4", "reference": "forward_syn"}
# LDS bytes per clock and compute unit measured with LDS-only microkernels on this part (1024 threads, 2.4 GHz):
# 4-byte reads 102, 8- and 16-byte reads 193, 4-byte writes 61, 16-byte writes 75.  Per state and step the grouped
# and scaled forms read one predecessor word (4-byte reads) and their own state (16-byte reads) and write their
# state (16-byte writes); the reference form reads five words and writes one with 4-byte accesses.
LDS_BYTES_PER_CLK = {"read32": 102.0, "read128": 193.0, "write32": 61.0, "write128": 75.0}
LDS_CLK_GHZ = 2.4
HMM_LDS_MIX = {
    "reference": {"read32": 20, "write32": 4},
    "grouped": {"read32": 4, "read128": 4, "write128": 4},
    "scaled": {"read32": 4, "read128": 4, "write128": 4},
}


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


LDS_RESIDENT_NOTE = ("one workgroup per read keeps both state vectors in LDS for the whole read: the algorithmic bytes of the "
                     "state vectors are LDS traffic, not HBM traffic (`traffic` is what HBM saw), so `frac` can exceed 1")


def _hbm_roofline(alg_bytes, kernel_ms, workload, default_cfg, note=None):
    gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    traffic, source = _profiled_traffic(workload) if default_cfg else (None, None)
    r = {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
         "traffic": traffic, "traffic_source": source, "kernel_ms": kernel_ms, "algorithmic_bytes": alg_bytes}
    if note:
        r["note"] = note
    return r


def _time_hmm_form(form, hd, sd, n, S, nthreads, args, torch, parpy, W):
    a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
    a2 = torch.zeros_like(a1)
    res = torch.zeros(n, dtype=torch.float64 if form == "scaled" else torch.float32, device="cuda")
    f = getattr(W, HMM_FORMS[form])
    threads = min(nthreads, S) if form == "reference" else min(nthreads, S // 4)
    opts = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(threads)})
    _apply_opt_flags(opts, args)
    opts.use_cuda_graphs = bool(args.use_graphs)
    opts.persistent_loops = bool(args.persistent)
    fn = lambda: f(hd, sd, res, a1, a2, opts=opts)
    timed = lambda: parpy.time_call(f, hd, sd, res, a1, a2, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    dev.sort()
    return wall, dev[len(dev) // 2], res.cpu().numpy(), threads


def bench_hmm(k, args, torch, parpy, W, default_cfg=True):
    import numpy as np
    import oracle
    hmm, seqs = W.synthetic_hmm(k)
    S, n = hmm["num_states"], seqs["num_instances"]
    # the probability tables of the linear-space forms are made on the device from the log-space tables of the
    # workload's definition by a compiled kernel (once per model; its time is reported, not part of a step)
    (hd, table_prep_ms), sd = W.scaled_tables_on_device(W.to_device(hmm), time_it=True), W.to_device(seqs)
    steps_total = int((seqs["lens"] - 1).sum())
    longest = int(seqs["lens"].max()) - 1
    # per (sequence, step): read alpha (4S) + write alpha (4S) + emission row (4S) + the observation byte
    alg_bytes = (12 * S + 1) * steps_total
    others = [] if args.single_form else [f for f in ("scaled", "grouped", "reference") if f != args.form]
    forms = {}
    for form in [args.form] + others:
        wall, kernel_ms, ll, threads = _time_hmm_form(form, hd, sd, n, S, args.state_threads, args, torch, parpy, W)
        mix = HMM_VALU_MIX[form]
        rows_per_simd = S / 256.0
        bound_ms = longest * rows_per_simd * (mix["full"] * VALU_NS["full"] + mix["trans"] * VALU_NS["trans"]) * 1e-6
        clk_per_state = sum(b / LDS_BYTES_PER_CLK[kind] for kind, b in HMM_LDS_MIX[form].items())
        lds_ms = longest * S * clk_per_state / (LDS_CLK_GHZ * 1e9) * 1e3
        forms[form] = {"wall": wall, "kernel_ms": kernel_ms, "ll": ll, "threads": threads,
                       "valu_bound": {"ms": bound_ms, "frac": bound_ms / kernel_ms,
                                      "model": f"{longest} steps of the longest read x {rows_per_simd:g} rows of 64 states per SIMD x "
                                               f"({mix['full']} full-rate x {VALU_NS['full']} ns + {mix['trans']} exp/log x {VALU_NS['trans']} ns)"},
                       "lds_bound": {"ms": lds_ms, "frac": lds_ms / kernel_ms,
                                     "model": f"{longest} steps of the longest read x {S} states x "
                                              + " + ".join(f"{b} B {kind} at {LDS_BYTES_PER_CLK[kind]:g} B/clk" for kind, b in HMM_LDS_MIX[form].items())
                                              + f" on one compute unit at {LDS_CLK_GHZ} GHz (measured LDS rates)"}}
    # outside the timed region: the shortest reads at full length against the fp64 oracle (what the GPU tests do for all)
    sub = np.argsort(seqs["lens"])[:6]
    want = oracle.hmm_syn_forward(hmm, seqs, np.float64, subset=sub)
    checked = {}
    for form, r in forms.items():
        err = float(np.abs(r["ll"][sub].astype(np.float64) - want).max())
        # the scaled form is held to the 1e-4 of the workload's definition, the fp32 log-space forms to their measured drift
        limit = 1e-4 if form == "scaled" else 0.2
        assert np.all(np.isfinite(r["ll"])) and err < limit, f"{form} form of the {k}-mer forward pass is off by {err}"
        checked[form] = err
    cpu = None
    if not args.no_cpu:
        sample_steps = args.cpu_steps or (15000 if k <= 5 else 5000)   # about 2 s (5-mer) and 10 s (7-mer) on 16 cores
        t0 = time.perf_counter()
        oracle.hmm_syn_forward(hmm, seqs, np.float32, max_steps=sample_steps)
        dt = time.perf_counter() - t0
        done = int((np.minimum(seqs["lens"], sample_steps) - 1).sum())
        cpu = {"value": dt * 1e3 * steps_total / done, "unit": "ms/batch", "cores": os.cpu_count(), "kind": "port",
               "sample": f"first {sample_steps} samples of each of the {n} reads with the C oracle "
                         f"(OpenMP over reads), {dt:.1f} s measured, scaled by total steps {steps_total}/{done}"}
    main = forms[args.form]
    name = HMM_FORMS
    suffix = {"scaled": "_scaled", "grouped": "_grouped", "reference": ""}
    resident = LDS_RESIDENT_NOTE if main["threads"] <= 1024 and 8 * S <= 156 * 1024 else None
    roof = _hbm_roofline(alg_bytes, main["kernel_ms"], f"hmm{k}{suffix[args.form]}", default_cfg, resident)
    roof["valu_bound"] = main["valu_bound"]
    if resident:
        roof["lds_bound"] = main["lds_bound"]
    other_forms = []
    for other in others:
        alt = forms[other]
        alt_roof = _hbm_roofline(alg_bytes, alt["kernel_ms"], f"hmm{k}{suffix[other]}", default_cfg,
                                 LDS_RESIDENT_NOTE if alt["threads"] <= 1024 and 8 * S <= 156 * 1024 else None)
        alt_roof["valu_bound"] = alt["valu_bound"]
        if "note" in alt_roof:
            alt_roof["lds_bound"] = alt["lds_bound"]
        other_forms.append({"form": f"{other} ({name[other]})", "ms_per_step": alt["wall"], "state_threads": alt["threads"],
                            "dtype": "f32 state vectors, " + ("f64 result" if other == "scaled" else "f32 result"),
                            "roofline": alt_roof, "checked_max_abs_error": checked[other]})
    return {
        "metric": f"HMM-forward {k}-mer ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": main["wall"], "unit": "ms/batch", "ms_per_step": main["wall"], "higher_is_better": False,
        "dtype": "f32",
        "config": {"workload": f"hmm_forward_{k}mer_synthetic", "form": f"{args.form} ({name[args.form]})",
                   "result_dtype": "f64" if args.form == "scaled" else "f32", "states": S, "reads": n,
                   "min_len": 5000, "max_len": 15000, "total_steps": steps_total, "state_threads": main["threads"],
                   "graph_replay": bool(args.use_graphs), "mean_loglik": float(main["ll"].mean()), "table_prep_ms": table_prep_ms,
                   "checked": f"6 shortest reads at full length against the fp64 oracle, max abs error {checked[args.form]:.3g}"},
        "roofline": roof,
        "other_forms": other_forms,
        "cpu_baseline": cpu,
    }


def bench_hmm_ref(args, torch, parpy, W, default_cfg=True):
    """The reference's own 5-mer model (16 duration layers x 1024 k-mers = 16384 states) on its 100
    recorded reads, tables from tests/golden: the configuration its benchmark validates
    (benchmarks/forward.py:481-518).  Two statements of the recurrence: the reference's kernel
    (forward_kernel, log space, checked against the recorded log-likelihoods) and the scaled
    linear-space form (forward_kernel_scaled, checked against the fp64 oracle)."""
    import numpy as np
    import oracle
    g = os.path.join(ROOT, "tests", "golden")
    hmm, seqs = W.load_reference_model(os.path.join(g, "hmm_5mer_model.npz"), os.path.join(g, "hmm_signals.npz"))
    want = np.loadtxt(os.path.join(g, "hmm_5mer_expected.txt"), dtype=np.float32)
    S, n = hmm["num_states"], seqs["num_instances"]
    (hd, table_prep_ms), sd = W.scaled_tables_on_device(W.to_device(hmm), reference_format=True, time_it=True), W.to_device(seqs)
    steps_total = int((seqs["lens"] - 1).sum())
    # per (read, step): alpha read + alpha write (4S each), one emission row of S/16 k-mers, the observation byte
    alg_bytes = (8 * S + 4 * (S // 16) + 1) * steps_total
    form = "reference" if args.form == "reference" else "scaled"
    others = [] if args.single_form else [f for f in ("scaled", "reference") if f != form]
    sub = np.argsort(seqs["lens"])[:6]
    want64 = oracle.hmm_ref_forward(hmm, seqs, np.float64, subset=sub)
    runs = {}
    for f in [form] + others:
        a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
        a2 = torch.zeros_like(a1)
        if f == "scaled":
            res = torch.zeros(n, dtype=torch.float64, device="cuda")
            nthreads = min(S // 16, args.state_threads)
            call = lambda o, res=res, a1=a1, a2=a2: (W.forward_kernel_scaled, (hd, sd, res, a1, a2))
        else:
            res = torch.zeros(n, dtype=torch.float32, device="cuda")
            nthreads = min(S, args.state_threads)
            call = lambda o, res=res, a1=a1, a2=a2: (W.forward_kernel, (hd, sd, a1, a2, res))
        opts = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(nthreads)})
        _apply_opt_flags(opts, args)
        fun, fargs = call(opts)
        fn = lambda: fun(*fargs, opts=opts)
        timed = lambda: parpy.time_call(fun, *fargs, opts=opts)
        wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
        got = res.cpu().numpy()
        if f == "scaled":
            err = float(np.abs(got[sub] - want64).max())
            assert np.all(np.isfinite(got)) and err < 1e-4, f"scaled form of the reference model is off by {err}"
            checked = f"6 shortest reads against the fp64 oracle, max abs error {err:.3g}"
        else:
            assert np.allclose(got, want, atol=1e-5, rtol=1e-5), float(np.abs(got - want).max())
            checked = (f"all {n} reads against the reference's recorded log-likelihoods (atol = rtol = 1e-5), "
                       f"max abs error {float(np.abs(got - want).max()):.3g}")
        runs[f] = {"wall": wall, "kernel_ms": float(np.median(dev)), "threads": nthreads, "checked": checked,
                   "mean": float(got.mean()), "recorded": float(np.abs(got - want).max())}
    names = {"scaled": "scaled (forward_kernel_scaled)", "reference": "reference (forward_kernel)"}
    tag = {"scaled": "hmm5ref_scaled", "reference": "hmm5ref"}
    main = runs[form]
    return {
        "metric": "HMM-forward reference 5-mer model ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": main["wall"], "unit": "ms/batch", "ms_per_step": main["wall"], "higher_is_better": False, "dtype": "f32",
        "config": {"workload": "hmm_forward_reference_5mer_model", "form": names[form],
                   "result_dtype": "f64" if form == "scaled" else "f32", "states": S, "reads": n,
                   "min_len": int(seqs["lens"].min()), "max_len": int(seqs["lens"].max()), "total_steps": steps_total,
                   "state_threads": main["threads"], "mean_loglik": main["mean"], "checked": main["checked"], "table_prep_ms": table_prep_ms,
                   "max_abs_distance_to_recorded_f32_values": main["recorded"]},
        "roofline": _hbm_roofline(alg_bytes, main["kernel_ms"], tag[form], default_cfg, LDS_RESIDENT_NOTE),
        "other_forms": [{"form": names[o], "ms_per_step": runs[o]["wall"], "state_threads": runs[o]["threads"],
                         "roofline": _hbm_roofline(alg_bytes, runs[o]["kernel_ms"], tag[o], default_cfg, LDS_RESIDENT_NOTE),
                         "checked": runs[o]["checked"]} for o in others],
        "cpu_baseline": None,
        "data": "reference fixtures (tests/golden)",
    }


def bench_hmm_ref7(args, torch, parpy, W, default_cfg=True):
    """The reference's kernel (forward_kernel, test/test_forward.py:83-160) on a model of its 7-mer size: 16 layers x
    16384 k-mers = 262144 states, a state vector of 1 MiB per read that cannot stay in LDS, so every step is one
    launch over all reads with the state vectors in global memory (time loop on the host).  The reference ships no
    7-mer tables; tables and reads are seeded random data in its format (100 reads of 500..1500 samples).  One
    thread per k-mer: the 16 layers of a k-mer are the iterations of one thread."""
    import numpy as np
    import oracle
    hmm, seqs = W.random_reference_model(7)
    S, n = hmm["num_states"], seqs["num_instances"]
    hd, sd = W.to_device(hmm), W.to_device(seqs)
    a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
    a2 = torch.zeros_like(a1)
    res = torch.zeros(n, dtype=torch.float32, device="cuda")
    nthreads = args.state_threads if args.state_threads > 1024 else S // 16
    # workgroups of 256 threads: 64 per read instead of 16 fill the last round of workgroups of a step more evenly
    # (36.9 ms per batch against 42.0 ms with 1024 threads per workgroup, 37.2 with 512, 38.1 with 128)
    opts = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(nthreads).tpb(args.tpb)})
    _apply_opt_flags(opts, args)
    opts.use_cuda_graphs = bool(args.use_graphs)
    opts.persistent_loops = bool(args.persistent)
    fn = lambda: W.forward_kernel(hd, sd, a1, a2, res, opts=opts)
    timed = lambda: parpy.time_call(W.forward_kernel, hd, sd, a1, a2, res, opts=opts)
    steps = max(2, args.steps // 3)
    wall, dev = _events_ms(fn, timed, steps, min(args.warmup, 2), torch)
    got = res.cpu().numpy()
    sub = np.argsort(seqs["lens"])[:4]
    want = oracle.hmm_ref_forward(hmm, seqs, np.float32, subset=list(sub))
    err = float(np.abs(got[sub] - want).max())
    assert np.all(np.isfinite(got)) and np.allclose(got[sub], want, atol=1e-5, rtol=1e-5), err
    steps_total = int((seqs["lens"] - 1).sum())
    longest = int(seqs["lens"].max()) - 1
    # per (read, step): alpha read + alpha write (4S each), one emission row of S/16 k-mers, the observation byte
    alg_bytes = (8 * S + 4 * (S // 16) + 1) * steps_total
    kernel_ms = float(np.median(dev))
    roof = _hbm_roofline(alg_bytes, kernel_ms, "hmm7ref", default_cfg)
    if roof["traffic"]:
        roof["traffic"] *= longest   # the profile holds the mean over the step launches; a call makes one per step
    roof["note"] = ("kernel_ms is the whole call: one launch per step over all reads that are still running "
                    f"({longest} steps, {kernel_ms * 1e3 / longest:.1f} us per step)")
    return {
        "metric": "HMM-forward, model of the reference's 7-mer size (262144 states) ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": wall, "unit": "ms/batch", "ms_per_step": wall, "higher_is_better": False, "dtype": "f32",
        "config": {"workload": "hmm_forward_reference_format_7mer_random_tables", "form": "reference (forward_kernel)", "states": S,
                   "reads": n, "min_len": int(seqs["lens"].min()), "max_len": int(seqs["lens"].max()), "total_steps": steps_total,
                   "state_threads": nthreads, "threads_per_workgroup": args.tpb, "steps_of_the_longest_read": longest, "graph_replay": bool(args.use_graphs),
                   "checked": f"4 shortest reads against the fp32 oracle (atol = rtol = 1e-5), max abs error {err:.3g}"},
        "roofline": roof,
        "cpu_baseline": None,
        "data": "seeded random tables in the reference's model format",
    }


LDS_RATE_KERNELS = r'''
typedef float f4 __attribute__((ext_vector_type(4)));
extern "C" __global__ void __launch_bounds__(1024) lds_read128(float* out, int iters) {
  __shared__ f4 buf[4096];
  for (int i = threadIdx.x; i < 4096; i += 1024) buf[i] = f4{(float)i, 1.0f, 2.0f, 3.0f};
  __syncthreads();
  f4 acc = {0, 0, 0, 0};
  volatile __attribute__((address_space(3))) f4* vb = (__attribute__((address_space(3))) f4*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    f4 a = vb[0], b = vb[1024], c = vb[2048], d = vb[3072];
    acc += (a + b) + (c + d);
  }
  out[blockIdx.x * 1024 + threadIdx.x] = acc.x + acc.y + acc.z + acc.w;
}
extern "C" __global__ void __launch_bounds__(1024) lds_read32(float* out, int iters) {
  __shared__ float buf[16384];
  for (int i = threadIdx.x; i < 16384; i += 1024) buf[i] = (float)i;
  __syncthreads();
  float acc = 0;
  volatile __attribute__((address_space(3))) float* vb = (__attribute__((address_space(3))) float*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    float s = 0;
    #pragma unroll
    for (int k = 0; k < 16; ++k) s += vb[k * 1024];
    acc += s;
  }
  out[blockIdx.x * 1024 + threadIdx.x] = acc;
}
extern "C" __global__ void __launch_bounds__(1024) lds_write128(float* out, int iters) {
  __shared__ f4 buf[4096];
  f4 v = {1.0f, 2.0f, 3.0f, (float)threadIdx.x};
  volatile __attribute__((address_space(3))) f4* vb = (__attribute__((address_space(3))) f4*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    vb[0] = v; vb[1024] = v; vb[2048] = v; vb[3072] = v;
    v.x += 1.0f;
  }
  __syncthreads();
  out[blockIdx.x * 1024 + threadIdx.x] = buf[threadIdx.x].x;
}

typedef float f2 __attribute__((ext_vector_type(2)));
extern "C" __global__ void __launch_bounds__(1024) lds_write32(float* out, int iters) {
  __shared__ float buf[16384];
  float v = (float)threadIdx.x;
  volatile __attribute__((address_space(3))) float* vb = (__attribute__((address_space(3))) float*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    #pragma unroll
    for (int k = 0; k < 16; ++k) vb[k * 1024] = v;
    v += 1.0f;
  }
  __syncthreads();
  out[blockIdx.x * 1024 + threadIdx.x] = buf[threadIdx.x];
}
extern "C" __global__ void __launch_bounds__(1024) lds_write64(float* out, int iters) {
  __shared__ f2 buf[8192];
  f2 v = {1.0f, (float)threadIdx.x};
  volatile __attribute__((address_space(3))) f2* vb = (__attribute__((address_space(3))) f2*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    #pragma unroll
    for (int k = 0; k < 8; ++k) vb[k * 1024] = v;
    v.x += 1.0f;
  }
  __syncthreads();
  out[blockIdx.x * 1024 + threadIdx.x] = buf[threadIdx.x].x;
}
extern "C" __global__ void __launch_bounds__(1024) lds_read64(float* out, int iters) {
  __shared__ f2 buf[8192];
  for (int i = threadIdx.x; i < 8192; i += 1024) buf[i] = f2{(float)i, 1.0f};
  __syncthreads();
  f2 acc = {0, 0};
  volatile __attribute__((address_space(3))) f2* vb = (__attribute__((address_space(3))) f2*)buf + threadIdx.x;
  for (int it = 0; it < iters; ++it) {
    f2 s = {0, 0};
    #pragma unroll
    for (int k = 0; k < 8; ++k) s += vb[k * 1024];
    acc += s;
  }
  out[blockIdx.x * 1024 + threadIdx.x] = acc.x + acc.y;
}
'''


def bench_lds_rates(args, torch, parpy, W, default_cfg=True):
    """LDS bytes per clock and compute unit for 4-, 8- and 16-byte reads and writes: hand-written microkernels (the
    only ones in this file; everything else is compiled from ParPy user code) whose loops touch nothing but
    registers and LDS, 1024 threads per workgroup, one workgroup per compute unit.  These are the rates behind
    `lds_bound` of the HMM records."""
    o = parpy.CompileOptions()
    o.backend = parpy.CompileBackend.Hip
    iters, blocks = 20000, 100
    out = torch.zeros(blocks * 1024, dtype=torch.float32, device="cuda")
    rates = {}
    for name in ("lds_read32", "lds_read64", "lds_read128", "lds_write32", "lds_write64", "lds_write128"):
        f = parpy.compile_string(name, LDS_RATE_KERNELS, o, grid=(blocks, 1, 1), block=(1024, 1, 1))
        f(out, 10)
        parpy.sync(o.backend)
        ts = []
        for _ in range(5):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            f(out, iters)
            parpy.sync(o.backend)
            ts.append(time.perf_counter() - t0)
        per_cu = 1024 * 64 * iters / sorted(ts)[2]        # every thread moves 64 bytes per iteration
        rates[name] = {"GB/s per CU": per_cu / 1e9, "B/clk at 2.4 GHz": per_cu / (LDS_CLK_GHZ * 1e9)}
    return {"metric": "LDS bytes per clock and compute unit, 1xMI355X", "value": rates["lds_read128"]["B/clk at 2.4 GHz"], "unit": "B/clk/CU",
            "ms_per_step": None, "higher_is_better": True, "dtype": "f32", "config": {"workload": "lds_rates", "rates": rates},
            "roofline": None, "cpu_baseline": None}


def _valu_rate_kernel(name, adds, exps):
    """A loop whose body is `adds` independent v_add_f32 (eight accumulators) and `exps` independent v_exp_f32, registers only."""
    lines = [f"v_add_f32 v{16 + i % 8}, v{16 + i % 8}, v{41 + i % 8}" for i in range(adds)]
    lines += [f"v_exp_f32 v{24 + i % 8}, v{24 + i % 8}" for i in range(exps)]
    body = "\\n".join(lines)
    init = "\\n".join([f"v_mov_b32 v{r}, 0x3f000000" for r in range(40, 52)] + [f"v_mov_b32 v{r}, 0" for r in range(16, 32)])
    clob = ", ".join(f'"v{r}"' for r in range(16, 32))
    clob_all = ", ".join(f'"v{r}"' for r in list(range(16, 32)) + list(range(40, 52)))
    return f'''
extern "C" __global__ void __launch_bounds__(1024) {name}(float* out, int iters) {{
  asm volatile("{init}" ::: {clob_all});
  for (int i = 0; i < iters; ++i) {{
    asm volatile("{body}" ::: {clob});
  }}
  float r, r2;
  asm volatile("v_mov_b32 %0, v16\\nv_mov_b32 %1, v24" : "=v"(r), "=v"(r2));
  out[blockIdx.x * 1024 + threadIdx.x] = r + r2;
}}'''


def bench_valu_rates(args, torch, parpy, W, default_cfg=True):
    """Issue time of a full-rate vector instruction and of v_exp_f32 per wave with four waves on a SIMD (a
    1024-thread workgroup on its compute unit): register-only microkernels.  These are `VALU_NS`, the times behind
    `valu_bound` of the HMM records."""
    o = parpy.CompileOptions()
    o.backend = parpy.CompileBackend.Hip
    iters, blocks = 20000, 100
    out = torch.zeros(blocks * 1024, dtype=torch.float32, device="cuda")
    res = {}
    for name, adds, exps in (("valu_add32", 32, 0), ("valu_exp8", 0, 8)):
        f = parpy.compile_string(name, _valu_rate_kernel(name, adds, exps), o, grid=(blocks, 1, 1), block=(1024, 1, 1))
        f(out, 10)
        parpy.sync(o.backend)
        ts = []
        for _ in range(5):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            f(out, iters)
            parpy.sync(o.backend)
            ts.append(time.perf_counter() - t0)
        # four waves per SIMD take turns: the time of one instruction of one wave is the loop time over 4 x count
        res[name] = sorted(ts)[2] * 1e9 / (iters * 4 * (adds + exps))
    return {"metric": "vector-ALU issue time per wave instruction with 4 waves per SIMD, 1xMI355X", "value": res["valu_add32"], "unit": "ns",
            "ms_per_step": None, "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "valu_rates", "v_add_f32_ns": res["valu_add32"], "v_exp_f32_ns": res["valu_exp8"]},
            "roofline": None, "cpu_baseline": None}


def bench_rowsum(args, torch, parpy, W, default_cfg=True):
    import numpy as np
    N, M = 1024, 65536
    inner = args.inner_threads or 1024  # one full workgroup per row (any choice from 64 up measures within 5 %)
    x = W.make_rowsum(N, M)
    xd = torch.from_numpy(x).cuda()
    out = torch.zeros(N, dtype=torch.float32, device="cuda")
    opts = parpy.par({"outer": parpy.threads(N), "inner": parpy.threads(inner)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.sum_rows(xd, out, N, opts=opts)
    timed = lambda: parpy.time_call(W.sum_rows, xd, out, N, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    want = x.sum(axis=1, dtype=np.float64)
    err = float(np.abs(out.cpu().numpy() - want).max())
    assert err < 1e-2, err
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
            "config": {"workload": "rowsum_1024x65536", "inner_threads": inner,
                       "checked": f"all rows against the fp64 sum, max abs error {err:.3g}"},
            "roofline": _hbm_roofline(alg, kernel_ms, "rowsum", default_cfg),
            "cpu_baseline": cpu}


def bench_softmax(args, torch, parpy, W, default_cfg=True):
    import numpy as np
    N, M = 16384, 4096
    inner = args.inner_threads or 512   # 8 elements (two dwordx4) per thread, 4 workgroups per CU
    x = W.make_softmax(N, M)
    xd = x.cuda()
    out = torch.zeros_like(xd)
    opts = parpy.par({"N": parpy.threads(N), "M": parpy.threads(inner)})
    _apply_opt_flags(opts, args)
    fn = lambda: W.softmax(xd, N, M, out, opts=opts)
    timed = lambda: parpy.time_call(W.softmax, xd, N, M, out, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    alg = 2 * N * M * 4
    kernel_ms = float(np.median(dev))
    t0 = time.perf_counter()
    want = torch.softmax(x, 1)
    cpu_ms = (time.perf_counter() - t0) * 1e3
    got = out.cpu()
    rel = float(((got - want).abs() / want).max())
    assert torch.allclose(got, want, atol=1e-5, rtol=1e-5), rel
    cpu = None
    if not args.no_cpu:
        cpu = {"value": cpu_ms, "unit": "ms/batch", "cores": torch.get_num_threads(),
               "kind": "port", "sample": "torch.softmax(x, 1) on the full 16384x4096 matrix, one run"}
    return {"metric": "softmax 16384x4096 f32 ms + achieved HBM GB/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "softmax_16384x4096", "inner_threads": inner,
                       "checked": f"every element against torch.softmax on the CPU, max relative error {rel:.3g}"},
            "roofline": _hbm_roofline(alg, kernel_ms, "softmax", default_cfg),
            "cpu_baseline": cpu}


def bench_sddmm(args, torch, parpy, W, default_cfg=True):
    import numpy as np
    import oracle
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
    opts.use_cuda_graphs = bool(args.use_graphs)
    fn = lambda: W.sddmm_coo(Ad, Bd, C, D, one, zero, opts=opts)
    timed = lambda: parpy.time_call(W.sddmm_coo, Ad, Bd, C, D, one, zero, opts=opts)
    wall, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    kernel_ms = float(np.median(dev))
    flops = 2 * A.shape[1] * nnz
    # what any SDDMM on this mask must move once: A, B, the CSR mask (column indices + row pointers), the result
    compulsory = A.nbytes + B.nbytes + cols.nbytes + crows.nbytes + nnz * 4
    # what the COO kernel of the reference's benchmark is handed on top of that: a row index and a value per non-zero
    coo_bytes = A.nbytes + B.nbytes + cols.nbytes + nnz * 8 + vals.nbytes + nnz * 4
    rows = rows_d.cpu().numpy()
    t0 = time.perf_counter()
    want = oracle.sddmm(A, B, rows, cols)
    cpu_ms = (time.perf_counter() - t0) * 1e3
    got = D.cpu().numpy()
    bad = np.abs(got - want) > 1e-5 + 1e-5 * np.abs(want)
    assert bad.mean() < 1e-3 and np.abs(got - want).max() < 5e-4, (float(bad.mean()), float(np.abs(got - want).max()))
    cpu = None
    if not args.no_cpu:
        cpu = {"value": cpu_ms, "unit": "ms/batch", "cores": 1, "kind": "port", "sample": "chunked NumPy einsum over all non-zeros, one run"}
    tflops = flops / (kernel_ms * 1e-3) / 1e12
    l2 = _profiled_field("sddmm", "l2_bytes_per_call") if default_cfg else None
    traffic, source = _profiled_traffic("sddmm") if default_cfg else (None, None)
    return {"metric": "SDDMM 8192x128x8192 1% ms + TFLOP/s", "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "sddmm_8192_k128_1pct", "nnz": nnz, "tpb": args.tpb,
                       "checked": f"every non-zero against the fp64 oracle: {float(bad.mean()) * 100:.4f} % outside atol = rtol = 1e-5, "
                                  f"max abs error {float(np.abs(got - want).max()):.3g}"},
            # the contraction is 0.17 GFLOP of gathered dot products: priced against the fp32 matrix peak as the
            # workload's definition asks, although the time goes to L2 requests of the row gathers
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": FP32_MATRIX_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tflops / FP32_MATRIX_PEAK_TFLOPS, "traffic": traffic, "traffic_source": source,
                         "kernel_ms": kernel_ms, "flops": flops,
                         "hbm_compulsory_bytes": compulsory, "hbm_compulsory_gbs": compulsory / (kernel_ms * 1e-3) / 1e9,
                         "coo_argument_bytes": coo_bytes,
                         "l2_bytes_per_call": l2, "l2_gbs": (l2 / (kernel_ms * 1e-3) / 1e9) if l2 else None,
                         "l2_source": "profiles/sddmm_kernel.md (TCC_REQ_sum x 128 B)" if l2 else None},
            "cpu_baseline": cpu}


def bench_copy(args, torch, parpy, W, default_cfg=True):
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
            "roofline": _hbm_roofline(alg, kernel_ms, "copy", default_cfg),
            "cpu_baseline": None}


def _profiled_field(name, field):
    """A figure from the committed rocprofv3 counter summary of this kernel (profiles/<name>_kernel.md), or None."""
    import re
    path = os.path.join(ROOT, "profiles", f"{name}_kernel.md")
    try:
        m = re.search(r"^%s:\s*(\d+)" % re.escape(field), open(path).read(), re.M)
        return int(m.group(1)) if m else None
    except OSError:
        return None


def _profiled_traffic(name):
    """(HBM bytes per launch, where the figure comes from): FETCH_SIZE + WRITE_SIZE of the committed counter runs of
    the same kernel (the file gives their commands), not measured in this run."""
    v = _profiled_field(name, "traffic_bytes_per_launch")
    return (v, f"profiles/{name}_kernel.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of the same kernel, commands in that file)") if v else (None, None)


def _apply_opt_flags(opts, args):
    for name in OPT_FLAGS:
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
    ap.add_argument("--workload", default="all", choices=["all", "hmm7", "hmm5", "hmm5ref", "hmm7ref", "rowsum", "softmax", "sddmm", "copy", "ldsrates", "valurates"])
    ap.add_argument("--form", default="scaled", choices=["scaled", "grouped", "reference"],
                    help="which statement of the HMM step is the record's value (the others are timed beside it)")
    ap.add_argument("--single-form", action="store_true", help="time only the chosen form of the HMM step (profiling runs)")
    ap.add_argument("--state-threads", type=int, default=1024)
    ap.add_argument("--use-graphs", type=int, default=0, help="replay the launches of a run from a HIP graph (host-hoisted time loops)")
    ap.add_argument("--persistent", type=int, default=0, help="run host-hoisted time loops inside one kernel when the grid fits the device")
    ap.add_argument("--inner-threads", type=int, default=None)
    ap.add_argument("--tpb", type=int, default=256)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-steps", type=int, default=0, help="samples per read for the HMM CPU baseline")
    for name in OPT_FLAGS:
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

    default_cfg = not any(getattr(args, n) is not None for n in OPT_FLAGS) and not args.reg_budget
    runners = {
        "hmm7": lambda: bench_hmm(7, args, torch, parpy, W, default_cfg),
        "hmm5": lambda: bench_hmm(5, args, torch, parpy, W, default_cfg),
        "hmm5ref": lambda: bench_hmm_ref(args, torch, parpy, W, default_cfg),
        "hmm7ref": lambda: bench_hmm_ref7(args, torch, parpy, W, default_cfg),
        "rowsum": lambda: bench_rowsum(args, torch, parpy, W, default_cfg),
        "softmax": lambda: bench_softmax(args, torch, parpy, W, default_cfg),
        "sddmm": lambda: bench_sddmm(args, torch, parpy, W, default_cfg),
        "copy": lambda: bench_copy(args, torch, parpy, W, default_cfg),
        "ldsrates": lambda: bench_lds_rates(args, torch, parpy, W, default_cfg),
        "valurates": lambda: bench_valu_rates(args, torch, parpy, W, default_cfg),
    }
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "scaling": "weak", "vs_baseline": None}
    if args.workload == "all":
        r = runners["hmm7"]()
        r.update(common)
        r.setdefault("data", "synthetic")
        r["secondary"] = []
        for w in ("hmm5", "hmm5ref", "hmm7ref", "rowsum", "softmax", "sddmm"):
            s = runners[w]()
            s.setdefault("data", "synthetic")
            r["secondary"].append(s)
    else:
        r = runners[args.workload]()
        r.update(common)
        r.setdefault("data", "synthetic")
    print(json.dumps(r))


if __name__ == "__main__":
    main()
