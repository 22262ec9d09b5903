"""Benchmark of the compiled hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]
                    [--workload all|hmm7|hmm5|hmm5ref|hmm7ref|rowsum|softmax|sddmm|sddmm_bt|copy|ldsrates|valurates|stepmodes] [--form scaled|grouped|reference]

A step is one pass of the compiled function over one batch of seeded synthetic
input that is already resident in HBM.  The default run (`all`) first measures
the machine rates that the bound models use (LDS, vector ALU, the latency of a
dependent step: hand-written microkernels, about two seconds), then times the
headline workload -- the 7-mer HMM forward batch (4^7 = 16384 states, 100 reads
of 5000..15000 samples) -- and then the other configurations, whose records go
under `secondary` of the same JSON line and, as scalars, into `config`
(`forms_ms`, `secondary_ms`, `secondary_frac`, `measured_rates`).  Every record
carries the roofline of its dominant kernel (algorithmic bytes or flops /
measured kernel time against the published peak) and a CPU baseline timed on
the host cores (bounded sample).

The HMM forward pass is timed in three statements of the same recurrence, all
written as ParPy user code in parpy_amd/workloads.py: `scaled` (forward_scaled:
linear space with rescaling by powers of two, float64 result, the one that
meets the 1e-4 tolerance against the fp64 oracle and the `value` of the
headline; a kernel the user rewrites, not the reference's), `grouped`
(forward_syn4: log space, the four states that share their predecessors updated
together) and `reference` (forward_syn: log space, one state at a time, the
structure of the reference's kernel, unchanged user code).  All start from the
log-space tables of the workload's definition; the probability tables of the
linear-space forms are made from them on the device by a compiled kernel
(`config.table_prep_ms`).  The reference's own 16-layer model (`hmm5ref`) is
timed as its kernel (forward_kernel) and in the scaled form
(forward_kernel_scaled).  Results are checked against the oracle outside the
timed region.
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
             "opt_guard_bounds", "opt_prefetch_steps", "opt_pack_accesses", "opt_share_iterations", "opt_fence_iterations", "opt_keep_stored", "opt_keep_own")

# Vector-ALU instructions per state and step in the time loop of the generated HMM kernels (counted in the ISA of
# the kernels as compiled for these shapes: full-rate instructions, and v_exp_f32 / v_log_f32).  One workgroup of 16
# waves per read puts S / 256 rows of 64 states on each SIMD.  The issue times of the two classes and the LDS rates
# are measured by microkernels in the same run (`measure_rates`); the figures below are what those measured when the
# committed profiles were taken (profiles/valu_rates.md, profiles/lds_rates.md) and serve as a cross-check only.
COMMITTED_VALU_NS = {"fast": 1.02, "normal": 2.03, "trans": 3.63}
COMMITTED_LDS_GBS_PER_CU = {"read32": 245.5, "read64": 463.0, "read128": 465.9, "write32": 147.5, "write64": 197.7, "write128": 178.9}
# Per state and step: instructions of the double-rate class (v_add / v_sub / v_mul / v_fma_f32), of the single-rate
# class (v_max / v_min, integer and address arithmetic, selects) and transcendentals (SQ_INSTS_VALU_* counters of the
# 7-mer kernels, profiles/hmm7_valu_classes.md).
HMM_VALU_MIX = {
    "reference": {"fast": 21.0, "normal": 3.57, "trans": 6.0},
    "grouped": {"fast": 11.25, "normal": 2.5, "trans": 3.0},
    "scaled": {"fast": 7.04, "normal": 1.91, "trans": 0.0},
}
HMM_FORMS = {"scaled": "forward_scaled", "grouped": "forward_syn4", "reference": "forward_syn"}
# LDS bytes per state and step: the grouped and scaled forms read one predecessor word (4-byte reads, issued two to
# an instruction) and their own state (16-byte reads) and write their state (16-byte writes); the reference form
# reads five words and writes one with 4-byte accesses.
HMM_LDS_MIX = {
    "reference": {"read32": 20, "write32": 4},
    "grouped": {"read32": 4, "read128": 4, "write128": 4},
    "scaled": {"read32": 4, "read128": 4, "write128": 4},
}
# The vendor's LDS width for this part (AMD CDNA 4 architecture white paper: 160 KB of LDS per compute unit, read
# bandwidth doubled over CDNA 3 to 256 bytes per clock; the write path is not stated separately and is taken as
# CDNA 3's 128 bytes per clock) at the 2.4 GHz peak engine clock.
VENDOR_LDS_BYTES_PER_CLK = {"read": 256.0, "write": 128.0}
PEAK_CLOCK_GHZ = 2.4


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


def _hmm_bounds(form, S, longest, kernel_ms, rates):
    """Vector-ALU and LDS time of the longest read of a batch under the rates measured in this run, as fractions
    of the kernel's time; the LDS time also under the vendor's LDS width at the peak clock."""
    mix = HMM_VALU_MIX[form]
    rows_per_simd = S / 256.0
    ns = rates["valu_ns"]
    parts_ns = mix["fast"] * ns["fast"] + mix["normal"] * ns["normal"] + mix["trans"] * ns["trans"]
    replay_ns = ns["replay_ns_per_state"][form]
    valu_ms = longest * rows_per_simd * replay_ns * 1e-6
    parts_ms = longest * rows_per_simd * parts_ns * 1e-6
    gbs = rates["lds_gbs_per_cu"]
    lds_ms = longest * S * sum(b / (gbs[kind] * 1e9) for kind, b in HMM_LDS_MIX[form].items()) * 1e3
    clk = sum(b / VENDOR_LDS_BYTES_PER_CLK["read" if kind.startswith("read") else "write"] for kind, b in HMM_LDS_MIX[form].items())
    vendor_ms = longest * S * clk / (PEAK_CLOCK_GHZ * 1e9) * 1e3
    return {
        "valu_bound": {"ms": valu_ms, "frac": valu_ms / kernel_ms, "rates": rates["source"],
                       "model": f"{longest} steps of the longest read x {rows_per_simd:g} rows of 64 states per SIMD x {replay_ns:.3g} ns: a "
                                f"register-only replay of the step's instruction classes per state ({mix['fast']} double-rate, "
                                f"{mix['normal']} single-rate, {mix['trans']} exp/log), four waves per SIMD",
                       "sum_of_parts_ms": parts_ms, "sum_of_parts_frac": parts_ms / kernel_ms,
                       "sum_of_parts": f"{mix['fast']} x {ns['fast']:.3g} ns + {mix['normal']} x {ns['normal']:.3g} ns + {mix['trans']} x {ns['trans']:.3g} ns "
                                       "per state (each class measured alone)"},
        "lds_bound": {"ms": lds_ms, "frac": lds_ms / kernel_ms, "rates": rates["source"],
                      "model": f"{longest} steps of the longest read x {S} states x "
                               + " + ".join(f"{b} B {kind} at {gbs[kind]:.4g} GB/s" for kind, b in HMM_LDS_MIX[form].items())
                               + " on one compute unit (LDS-only microkernels of this run)",
                      "vendor_width_ms": vendor_ms, "vendor_width_frac": vendor_ms / kernel_ms,
                      "vendor_width": f"reads {VENDOR_LDS_BYTES_PER_CLK['read']:g} B/clk, writes {VENDOR_LDS_BYTES_PER_CLK['write']:g} B/clk per "
                                      f"compute unit at {PEAK_CLOCK_GHZ} GHz (CDNA 4 white paper; write width taken as CDNA 3's)"},
    }


def bench_hmm(k, args, torch, parpy, W, default_cfg=True, rates=None):
    import numpy as np
    import oracle
    rates = rates or measure_rates(args, torch, parpy)
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
        forms[form] = {"wall": wall, "kernel_ms": kernel_ms, "ll": ll, "threads": threads}
        forms[form].update(_hmm_bounds(form, S, longest, kernel_ms, rates))
    # outside the timed region: the three shortest and the three longest reads (where the running scale has
    # gathered the most) at full length against the fp64 oracle (the GPU tests do this for every read)
    order = np.argsort(seqs["lens"])
    sub = np.concatenate([order[:3], order[-3:]])
    want = oracle.hmm_syn_forward(hmm, seqs, np.float64, subset=sub)
    checked = {}
    for form, r in forms.items():
        err = float(np.abs(r["ll"][sub].astype(np.float64) - want).max())
        # the scaled form is held to the 1e-4 of the workload's definition, the fp32 log-space forms to their measured drift
        limit = 1e-4 if form == "scaled" else 0.6
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
               "sample": f"first {sample_steps} samples of each of the {n} reads with the C oracle of the reference's log-space kernel "
                         f"(OpenMP over reads), {dt:.1f} s measured, scaled by total steps {steps_total}/{done}"}
    main = forms[args.form]
    name = HMM_FORMS
    suffix = {"scaled": "_scaled", "grouped": "_grouped", "reference": ""}
    is_resident = lambda r: r["threads"] <= 1024 and 8 * S <= 156 * 1024
    roof = _hbm_roofline(alg_bytes, main["kernel_ms"], f"hmm{k}{suffix[args.form]}", default_cfg, LDS_RESIDENT_NOTE if is_resident(main) else None)
    roof["valu_bound"] = main["valu_bound"]
    if is_resident(main):
        roof["lds_bound"] = main["lds_bound"]
    if k <= 5 and "step_floor_ns" in rates:
        floor_ms = longest * rates["step_floor_ns"] * 1e-6
        roof["latency_bound"] = {"ms": floor_ms, "frac": floor_ms / main["kernel_ms"],
                                 "model": f"{longest} dependent steps of the longest read x {rates['step_floor_ns']:.0f} ns: one 16-byte LDS store, "
                                          "the workgroup barrier and one dependent 16-byte LDS load of a 256-thread workgroup "
                                          "(register-only body, microkernel of this run)"}
    other_forms = []
    for other in others:
        alt = forms[other]
        alt_roof = _hbm_roofline(alg_bytes, alt["kernel_ms"], f"hmm{k}{suffix[other]}", default_cfg, LDS_RESIDENT_NOTE if is_resident(alt) else None)
        alt_roof["valu_bound"] = alt["valu_bound"]
        if is_resident(alt):
            alt_roof["lds_bound"] = alt["lds_bound"]
        other_forms.append({"form": f"{other} ({name[other]})", "ms_per_step": alt["wall"], "state_threads": alt["threads"],
                            "dtype": "f32 state vectors, " + ("f64 result" if other == "scaled" else "f32 result"),
                            "roofline": alt_roof, "checked_max_abs_error": checked[other]})
    config = {"workload": f"hmm_forward_{k}mer_synthetic", "form": f"{args.form} ({name[args.form]})",
              "result_dtype": "f64" if args.form == "scaled" else "f32", "states": S, "reads": n,
              "min_len": 5000, "max_len": 15000, "total_steps": steps_total, "state_threads": main["threads"],
              "graph_replay": bool(args.use_graphs), "mean_loglik": float(main["ll"].mean()), "table_prep_ms": table_prep_ms,
              "checked": f"3 shortest and 3 longest reads at full length against the fp64 oracle, max abs error {checked[args.form]:.3g}",
              # every statement of the step that was timed, in scalars (nested records may not survive a parser)
              "forms_ms": {f: forms[f]["wall"] for f in forms},
              "forms_kernel_ms": {f: forms[f]["kernel_ms"] for f in forms},
              "forms_max_abs_error": checked,
              "forms_valu_bound_frac": {f: forms[f]["valu_bound"]["frac"] for f in forms},
              "forms_lds_bound_frac": {f: forms[f]["lds_bound"]["frac"] for f in forms if is_resident(forms[f])},
              "lds_bound_frac": main["lds_bound"]["frac"] if is_resident(main) else None,
              "lds_bound_frac_vendor_width": main["lds_bound"]["vendor_width_frac"] if is_resident(main) else None,
              "valu_bound_frac": main["valu_bound"]["frac"]}
    return {
        "metric": f"HMM-forward {k}-mer ms/batch + achieved HBM GB/s (% of peak), 1xMI355X",
        "value": main["wall"], "unit": "ms/batch", "ms_per_step": main["wall"], "higher_is_better": False,
        "dtype": "f32",
        "config": config,
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
    order = np.argsort(seqs["lens"])
    sub = np.concatenate([order[:3], order[-3:]])
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
            checked = f"3 shortest and 3 longest reads against the fp64 oracle, max abs error {err:.3g}"
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
                   "max_abs_distance_to_recorded_f32_values": main["recorded"],
                   "forms_ms": {f: runs[f]["wall"] for f in runs}, "forms_kernel_ms": {f: runs[f]["kernel_ms"] for f in runs}},
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


STEP_FLOOR_KERNELS = r'''
typedef float f4 __attribute__((ext_vector_type(4)));
// What one dependent step of a 256-thread workgroup costs at the least: a 16-byte LDS load of what another thread
// stored in the step before, two multiply-adds, a 16-byte LDS store, the workgroup barrier.
extern "C" __global__ void __launch_bounds__(256) step_floor(float* out, int iters) {
  __shared__ f4 buf[2][256];
  const int tid = threadIdx.x;
  f4 v = {1.0f, 2.0f, 3.0f, (float)tid};
  buf[0][tid] = v;
  __syncthreads();
  for (int it = 1; it <= iters; ++it) {
    f4 a = buf[(it + 1) & 1][(tid + 67) & 255];
    v = a * 0.999f + v * 0.001f;
    buf[it & 1][tid] = v;
    __syncthreads();
  }
  out[blockIdx.x * 256 + tid] = v.x + v.w;
}
// Shader clock against the constant 100 MHz counter over a loop of dependent multiply-adds, 1024 threads.
extern "C" __global__ void __launch_bounds__(1024) clock_probe(unsigned long long* out, int iters) {
  const unsigned long long c0 = __builtin_readcyclecounter(), w0 = __builtin_amdgcn_s_memrealtime();
  float a = (float)threadIdx.x;
  for (int i = 0; i < iters; ++i) a = a * 1.0001f + 0.5f;
  const unsigned long long c1 = __builtin_readcyclecounter(), w1 = __builtin_amdgcn_s_memrealtime();
  if (threadIdx.x == 0) { out[2 * blockIdx.x] = c1 - c0; out[2 * blockIdx.x + 1] = w1 - w0; }
  if (a == 12345.678f) out[0] = 0;
}
'''


def _median_wall(f, args_small, args_full, parpy, torch, backend):
    f(*args_small)
    parpy.sync(backend)
    ts = []
    for _ in range(5):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        f(*args_full)
        parpy.sync(backend)
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[2]


def _lds_rates(torch, parpy):
    """GB/s per compute unit of 4-, 8- and 16-byte LDS reads and writes: hand-written microkernels (with the other
    rate kernels the only ones in this file; everything else is compiled from ParPy user code) whose loops touch
    nothing but registers and LDS, 1024 threads per workgroup, one workgroup on each of 100 compute units."""
    o = parpy.CompileOptions()
    o.backend = parpy.CompileBackend.Hip
    iters, blocks = 20000, 100
    out = torch.zeros(blocks * 1024, dtype=torch.float32, device="cuda")
    rates = {}
    for name in ("lds_read32", "lds_read64", "lds_read128", "lds_write32", "lds_write64", "lds_write128"):
        f = parpy.compile_string(name, LDS_RATE_KERNELS, o, grid=(blocks, 1, 1), block=(1024, 1, 1))
        t = _median_wall(f, (out, 10), (out, iters), parpy, torch, o.backend)
        rates[name[4:]] = 1024 * 64 * iters / t / 1e9        # every thread moves 64 bytes per iteration
    return rates


def _valu_rates(torch, parpy):
    """Issue times per wave instruction with four waves on a SIMD (a 1024-thread workgroup on its compute unit, 100
    compute units busy), register-only microkernels: the double-rate class, the single-rate class, transcendentals,
    and -- per statement of the HMM step -- a replay of the instruction classes of 16 states in the proportions the
    hardware counters report for the kernel (`replay_ns_per_state`): mixing transcendentals with other
    instructions costs more than the sum of the parts, however they are ordered, and the replay includes that."""
    o = parpy.CompileOptions()
    o.backend = parpy.CompileBackend.Hip
    iters, blocks = 20000, 100
    out = torch.zeros(blocks * 1024, dtype=torch.float32, device="cuda")
    res = {"replay_ns_per_state": {}}
    jobs = [("fast", "valu_add32", "a" * 32, 32), ("normal", "valu_max32", "m" * 32, 32), ("trans", "valu_exp8", "e" * 8, 8)]
    jobs += [("replay:" + form, "valu_replay_" + form, _replay_pattern(mix), 16) for form, mix in HMM_VALU_MIX.items()]
    for key, name, pattern, per in jobs:
        f = parpy.compile_string(name, _valu_rate_kernel(name, pattern), o, grid=(blocks, 1, 1), block=(1024, 1, 1))
        t = _median_wall(f, (out, 10), (out, iters), parpy, torch, o.backend)
        # four waves per SIMD take turns: the time of one instruction (or state) of one wave is the loop time over 4 x count
        v = t * 1e9 / (iters * 4 * per)
        if key.startswith("replay:"):
            res["replay_ns_per_state"][key[7:]] = v
        else:
            res[key] = v
    return res


def _step_floor_and_clock(torch, parpy):
    o = parpy.CompileOptions()
    o.backend = parpy.CompileBackend.Hip
    blocks, iters = 100, 200000
    out = torch.zeros(blocks * 256, dtype=torch.float32, device="cuda")
    f = parpy.compile_string("step_floor", STEP_FLOOR_KERNELS, o, grid=(blocks, 1, 1), block=(256, 1, 1))
    floor_ns = _median_wall(f, (out, 10), (out, iters), parpy, torch, o.backend) * 1e9 / iters
    ticks = torch.zeros(2 * blocks, dtype=torch.int64, device="cuda")
    g = parpy.compile_string("clock_probe", STEP_FLOOR_KERNELS, o, grid=(blocks, 1, 1), block=(1024, 1, 1))
    g(ticks, 1000)
    g(ticks, 2000000)
    parpy.sync(o.backend)
    t = ticks.cpu().numpy().reshape(blocks, 2).astype("float64")
    ratio = float((t[:, 0] / t[:, 1]).mean())
    # (the second counter runs at 100 MHz; a ratio of one means both read the same constant clock on this part)
    ghz = ratio * 0.1 if ratio > 1.5 else None
    return floor_ns, ghz


_RATES = {}


def measure_rates(args, torch, parpy):
    """The machine rates behind the bound models of the HMM records, measured in this run (about two seconds)."""
    if "r" not in _RATES:
        lds = _lds_rates(torch, parpy)
        floor_ns, ghz = _step_floor_and_clock(torch, parpy)
        _RATES["r"] = {"lds_gbs_per_cu": lds, "valu_ns": _valu_rates(torch, parpy), "step_floor_ns": floor_ns,
                       "shader_clock_ghz_under_valu_load": ghz,
                       "source": "microkernels of this run: 100 workgroups of 1024 threads, one per compute unit",
                       "committed_cross_check": {"valu_ns": COMMITTED_VALU_NS, "lds_gbs_per_cu": COMMITTED_LDS_GBS_PER_CU}}
    return _RATES["r"]


def bench_lds_rates(args, torch, parpy, W, default_cfg=True):
    """LDS rates per compute unit for 4-, 8- and 16-byte reads and writes (the rates behind `lds_bound` of the HMM records)."""
    r = measure_rates(args, torch, parpy)
    ghz = r["shader_clock_ghz_under_valu_load"]
    table = {k: {"GB/s per CU": v, "B/clk at 2.4 GHz": v / PEAK_CLOCK_GHZ, "B/clk at the measured clock": (v / ghz) if ghz else None}
             for k, v in r["lds_gbs_per_cu"].items()}
    return {"metric": "LDS bytes per clock and compute unit, 1xMI355X", "value": table["read128"]["B/clk at 2.4 GHz"], "unit": "B/clk/CU",
            "ms_per_step": None, "higher_is_better": True, "dtype": "f32",
            "config": {"workload": "lds_rates", "rates": table, "shader_clock_ghz_under_valu_load": ghz, "step_floor_ns_256_threads": r["step_floor_ns"]},
            "roofline": None, "cpu_baseline": None}


def _valu_rate_kernel(name, pattern):
    """A loop whose body is the instruction string `pattern` on registers only: 'a' an independent v_add_f32 (eight
    accumulators; the double-rate class), 'm' a v_max_f32 (the single-rate class), 'e' a v_exp_f32."""
    lines, na, ne = [], 0, 0
    for ch in pattern:
        if ch == "a":
            lines.append(f"v_add_f32 v{16 + na % 8}, v{16 + na % 8}, v{41 + na % 8}")
            na += 1
        elif ch == "m":
            lines.append(f"v_max_f32 v{16 + na % 8}, v{16 + na % 8}, v{41 + na % 8}")
            na += 1
        else:
            lines.append(f"v_exp_f32 v{24 + ne % 8}, v{24 + ne % 8}")
            ne += 1
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


def _replay_pattern(mix, states=16):
    """The instruction classes of `states` states of a step, state by state: double-rate, single-rate, transcendental."""
    out, done = [], {"fast": 0, "normal": 0, "trans": 0}
    for k in range(1, states + 1):
        for cls, ch in (("fast", "a"), ("normal", "m"), ("trans", "e")):
            n = int(round(mix[cls] * k)) - done[cls]
            out.append(ch * n)
            done[cls] += n
    return "".join(out)


def bench_valu_rates(args, torch, parpy, W, default_cfg=True):
    """Vector-ALU issue times (the times behind `valu_bound` of the HMM records)."""
    r = measure_rates(args, torch, parpy)
    v = r["valu_ns"]
    return {"metric": "vector-ALU issue time per wave instruction with 4 waves per SIMD, 1xMI355X", "value": v["fast"], "unit": "ns",
            "ms_per_step": None, "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "valu_rates", "v_add_f32_ns": v["fast"], "v_max_f32_ns": v["normal"], "v_exp_f32_ns": v["trans"],
                       "replay_ns_per_state": v["replay_ns_per_state"], "instruction_classes_per_state": HMM_VALU_MIX,
                       "shader_clock_ghz_under_valu_load": r["shader_clock_ghz_under_valu_load"]},
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


def _l2_line_rate(nnz, rows, K, tpb, args, torch, parpy, W):
    """128-byte lines per microsecond that come out of L2 / the memory-side cache when every lane group fetches a
    row of K floats from a random place of an 8192 x K table (4 MiB, as B^T): the compiled `gather_row_sums` with
    the launch shape and occupancy of the SDDMM kernel, one dependent index load in front of the lines."""
    import numpy as np
    rng = np.random.default_rng(W.SEED)
    table = torch.from_numpy(rng.standard_normal((rows, K)).astype(np.float32)).cuda()
    idx = torch.from_numpy(rng.integers(0, rows, size=nnz).astype(np.int64)).cuda()
    out = torch.zeros(nnz, dtype=torch.float32, device="cuda")
    opts = parpy.par({"i": parpy.threads(nnz).tpb(tpb)})
    fn = lambda: W.gather_row_sums(table, idx, out, nnz, opts=opts)
    timed = lambda: parpy.time_call(W.gather_row_sums, table, idx, out, nnz, opts=opts)
    _, dev = _events_ms(fn, timed, args.steps, args.warmup, torch)
    want = table[idx[:4096]].sum(dim=1)
    assert torch.allclose(out[:4096], want, atol=1e-4, rtol=1e-5)
    ms = float(np.median(dev))
    lines = nnz * (K * 4 // 128)
    return lines / (ms * 1e3), ms


def bench_sddmm(args, torch, parpy, W, default_cfg=True, transposed_operand=False):
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
    if transposed_operand:
        # the caller holds B transposed (a constant operand turned round once, outside the timed region)
        BTd = Bd.t().contiguous()
        fun, fargs = W.sddmm_coo_bt, (Ad, BTd, C, D, one, zero)
    else:
        fun, fargs = W.sddmm_coo, (Ad, Bd, C, D, one, zero)
    fn = lambda: fun(*fargs, opts=opts)
    timed = lambda: parpy.time_call(fun, *fargs, opts=opts)
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
    # the bound the kernel is against: a non-zero costs two dependent gathers, the index and then the four 128-byte
    # lines of its row of B^T (its row of A is shared with its neighbours through L1); the rate at which such lines
    # arrive is measured with the same launch shape, and the dot products cannot come faster than their lines
    line_rate, gather_ms = _l2_line_rate(nnz, B.shape[1], A.shape[1], args.tpb, args, torch, parpy, W)
    lines = nnz * (A.shape[1] * 4 // 128)
    l2_bound_ms = lines / line_rate * 1e-3
    name = "sddmm_8192_k128_1pct" + ("_transposed_operand" if transposed_operand else "")
    return {"metric": "SDDMM 8192x128x8192 1% ms + TFLOP/s" + (", B passed transposed" if transposed_operand else ""),
            "value": wall, "unit": "ms/batch", "ms_per_step": wall,
            "higher_is_better": False, "dtype": "f32",
            "config": {"workload": name, "nnz": nnz, "tpb": args.tpb,
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
                         "l2_source": "profiles/sddmm_kernel.md (TCC_REQ_sum x 128 B)" if l2 else None,
                         "l2_latency_bound": {"ms": l2_bound_ms, "frac": l2_bound_ms / kernel_ms, "lines_per_us": line_rate,
                                              "model": f"{lines} random 128-byte lines of B^T (four per non-zero) at the rate of the compiled "
                                                       f"gather of this run ({gather_ms * 1e3:.1f} us for the same launch shape: index load, then the "
                                                       "lines of a random row of a 4 MiB table)"}},
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


def bench_step_modes(args, torch, parpy, W, default_cfg=True):
    """A host-hoisted time loop three ways -- a launch per step, the launches of a run replayed from a HIP graph, the
    whole loop inside one kernel with a barrier per read -- on the synthetic 7-mer with 16 workgroups per read and on
    a model of the reference's 7-mer size with 64 per read, for 1, 4, 8 and 32 reads of 300 steps.  Microseconds per
    step (best of three timed calls); the three modes must give bit-equal results."""
    import numpy as np
    L = 300
    table = {}

    def run(fn, hmm, seqs, threads, reference_order, **kw):
        hd, sd = W.to_device(hmm), W.to_device(seqs)
        n, S = seqs["num_instances"], hmm["num_states"]
        a1 = torch.zeros((n, S), dtype=torch.float32, device="cuda")
        a2 = torch.zeros_like(a1)
        res = torch.zeros(n, dtype=torch.float32, device="cuda")
        o = parpy.par({"inst": parpy.threads(n), "state": parpy.threads(threads)})
        for k_, v in kw.items():
            setattr(o, k_, v)
        fargs = [hd, sd, a1, a2, res] if reference_order else [hd, sd, res, a1, a2]
        for _ in range(3):
            fn(*fargs, opts=o)
        parpy.sync(parpy.CompileBackend.Hip)
        t = min(parpy.time_call(fn, *fargs, opts=o) for _ in range(3))
        return res.cpu().numpy(), t * 1e3 / (L - 1)

    cases = [("synthetic_7mer_16_workgroups_per_read", W.forward_syn, False, lambda n: W.synthetic_hmm(7, n_inst=n, min_len=L, max_len=L), 16384),
             ("reference_format_7mer_64_workgroups_per_read", W.forward_kernel, True,
              lambda n: W.random_reference_model(7, n_reads=n, min_len=L, max_len=L), 65536)]
    for label, fn, ref_order, make, threads in cases:
        table[label] = {}
        for n in (1, 4, 8, 32):
            hmm, seqs = make(n)
            base, row = None, {}
            for mode, kw in (("launches", {}), ("graph", {"use_cuda_graphs": True}), ("one_kernel", {"persistent_loops": True})):
                got, us = run(fn, hmm, seqs, threads, ref_order, **kw)
                base = got if base is None else base
                assert np.array_equal(got, base), (label, n, mode)
                row[mode] = round(us, 2)
            table[label][f"reads_{n}"] = row
    first = table["synthetic_7mer_16_workgroups_per_read"]["reads_8"]
    return {"metric": "host-hoisted time loop: microseconds per step as launches, graph replay, one kernel", "value": first["one_kernel"],
            "unit": "us/step", "ms_per_step": first["one_kernel"] * 1e-3, "higher_is_better": False, "dtype": "f32",
            "config": {"workload": "step_modes", "steps_per_run": L - 1, "us_per_step": table},
            "roofline": {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": None, "traffic": None,
                         "note": "a comparison of launch mechanisms, not a bandwidth measurement"},
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
    ap.add_argument("--workload", default="all", choices=["all", "hmm7", "hmm5", "hmm5ref", "hmm7ref", "rowsum", "softmax", "sddmm", "sddmm_bt", "copy", "ldsrates", "valurates", "stepmodes"])
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
        "stepmodes": lambda: bench_step_modes(args, torch, parpy, W, default_cfg),
    }
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "scaling": "weak", "vs_baseline": None}
    runners["sddmm_bt"] = lambda: bench_sddmm(args, torch, parpy, W, default_cfg, transposed_operand=True)
    if args.workload == "all":
        rates = measure_rates(args, torch, parpy)       # LDS, vector-ALU and step-latency microkernels: about two seconds
        r = bench_hmm(7, args, torch, parpy, W, default_cfg, rates)
        r.update(common)
        r.setdefault("data", "synthetic")
        r["secondary"] = []
        sec_ms, sec_frac, sec_bound = {}, {}, {}
        for w in ("hmm5", "hmm5ref", "hmm7ref", "rowsum", "softmax", "sddmm", "sddmm_bt"):
            s = bench_hmm(5, args, torch, parpy, W, default_cfg, rates) if w == "hmm5" else runners[w]()
            s.setdefault("data", "synthetic")
            r["secondary"].append(s)
            sec_ms[w] = s["value"]
            sec_frac[w] = s["roofline"]["frac"]
            sec_bound[w] = s["roofline"]["bound"]
            for o in s.get("other_forms", []):
                sec_ms[w + ":" + o["form"].split(" ")[0]] = o["ms_per_step"]
                sec_frac[w + ":" + o["form"].split(" ")[0]] = o["roofline"]["frac"]
            for extra in ("latency_bound", "l2_latency_bound", "lds_bound", "valu_bound"):
                if extra in s["roofline"]:
                    sec_frac[w + ":" + extra] = s["roofline"][extra]["frac"]
        # the same figures as scalars inside `config`, for readers that keep only the contract's keys
        r["config"]["secondary_ms"] = sec_ms
        r["config"]["secondary_frac"] = sec_frac
        r["config"]["secondary_bound"] = sec_bound
        r["config"]["measured_rates"] = {"lds_gbs_per_cu": rates["lds_gbs_per_cu"], "valu_ns": rates["valu_ns"],
                                         "step_floor_ns_256_threads": rates["step_floor_ns"],
                                         "shader_clock_ghz_under_valu_load": rates["shader_clock_ghz_under_valu_load"]}
    else:
        r = runners[args.workload]()
        r.update(common)
        r.setdefault("data", "synthetic")
    print(json.dumps(r))


if __name__ == "__main__":
    main()
