"""parpy_hip_plan_run_noalloc: temporaries from the library's scratch array, results identical to parpy_hip_plan_run."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _ptr_args(arrays):
    ptrs = [a.data_ptr() for a in arrays]
    return (ctypes.c_void_p * len(ptrs))(*ptrs), len(ptrs)


def _compiled(fn, args, opts):
    """The wrapper of the specialisation for `args` (compiles on first use; runs it once)."""
    import parpy_amd as parpy
    from parpy_amd.validate import check_arguments
    fn(*args, opts=opts)
    parpy.sync(parpy.CompileBackend.Hip)
    opts = parpy.backend._resolve_backend(opts, True)
    return parpy._compile_function(parpy._ir_asts[fn], check_arguments(args, opts, True), opts)


def _rowsum_pair(lib, n, m, tpb_total, seed):
    """Multi-block row sums (per-block partial sums in a device temporary, then a second kernel)."""
    import torch
    import parpy_amd as parpy
    from parpy_amd import workloads as W
    g = torch.Generator().manual_seed(seed)
    x = (torch.rand((n, m), generator=g) * 2 - 1).cuda()
    out = torch.zeros(n, dtype=torch.float32, device="cuda")
    opts = parpy.par({"outer": parpy.threads(n), "inner": parpy.threads(tpb_total).tpb(128)})
    w = _compiled(W.sum_rows, [x, out, n], opts)
    assert w.launch_count() == 2, "expected the two-kernel multi-block reduction"
    want = out.clone()
    got = torch.full_like(out, float("nan"))
    arr, k = _ptr_args([x, got])
    rc = lib.parpy_hip_plan_run_noalloc(w.plan, arr, k)
    assert rc == 0, lib.parpy_get_error_message()
    torch.cuda.synchronize()
    ref = x.double().sum(1).cpu().numpy()
    assert np.allclose(want.cpu().numpy(), ref, atol=1e-3)
    return got.cpu().numpy(), want.cpu().numpy()


def test_noalloc_matches_plan_run_twice_second_smaller():
    import torch
    from parpy_amd import runtime
    import parpy_amd as parpy
    lib = runtime._compile_runtime_lib(parpy.CompileBackend.Hip)
    print("case: row sums 100 x 65536 on 1024 threads per row (8 blocks per row)", flush=True)
    got, want = _rowsum_pair(lib, 100, 65536, 1024, 1)
    assert np.array_equal(got, want)
    print("case: row sums 37 x 3000 on 256 threads per row (2 blocks per row)", flush=True)
    got, want = _rowsum_pair(lib, 37, 3000, 256, 2)
    assert np.array_equal(got, want)


def _sddmm_case(lib, nrows, ncols, k, nnz_per_row, seed):
    """(plan wrapper, pointer arguments with a fresh output last, result of the allocating entry point, fresh output)."""
    import torch
    import parpy_amd as parpy
    from parpy_amd import workloads as W
    rng = np.random.default_rng(seed)
    A = torch.from_numpy(rng.standard_normal((nrows, k)).astype(np.float32)).cuda()
    B = torch.from_numpy(rng.standard_normal((k, ncols)).astype(np.float32)).cuda()
    rows = np.repeat(np.arange(nrows, dtype=np.int64), nnz_per_row)
    cols = np.concatenate([np.sort(rng.choice(ncols, size=nnz_per_row, replace=False)) for _ in range(nrows)]).astype(np.int64)
    nnz = len(rows)
    C = {"rows": torch.from_numpy(rows).cuda(), "cols": torch.from_numpy(cols).cuda(),
         "values": torch.from_numpy(rng.standard_normal(nnz).astype(np.float32)).cuda(), "nnz": nnz}
    D = torch.zeros(nnz, dtype=torch.float32, device="cuda")
    opts = parpy.par({"nnz": parpy.threads(nnz).tpb(256)})
    w = _compiled(W.sddmm_coo, [A, B, C, D, 1.5, 2.0], opts)
    assert w.launch_count() == 2, "expected a transposition kernel in front of the main kernel"
    got = torch.full_like(D, 7.0)
    # flattened pointer arguments in call order, dictionary fields sorted by key
    flat = [A, B, C["cols"], C["rows"], C["values"], got]
    return w, flat, D, got


def test_noalloc_sddmm_transposed_temporary_then_smaller():
    """SDDMM keeps the transposed B in a temporary (4 MiB, then 64 KiB): same bits as the allocating entry point."""
    import torch
    import parpy_amd as parpy
    from parpy_amd import runtime
    lib = runtime._compile_runtime_lib(parpy.CompileBackend.Hip)
    for (n, k, per_row, seed) in [(8192, 128, 16, 3), (256, 64, 12, 4)]:
        print(f"case: sddmm n={n} k={k} nnz per row={per_row}", flush=True)
        w, flat, want, got = _sddmm_case(lib, n, n, k, per_row, seed)
        arr, cnt = _ptr_args(flat)
        rc = lib.parpy_hip_plan_run_noalloc(w.plan, arr, cnt)
        assert rc == 0, lib.parpy_get_error_message()
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want.cpu().numpy())


def test_noalloc_rejects_temporaries_beyond_the_scratch_size():
    """B of 128 x 65536 floats needs a 32 MiB transposed temporary: more than the 16 MiB the library holds."""
    import torch
    import parpy_amd as parpy
    from parpy_amd import runtime
    lib = runtime._compile_runtime_lib(parpy.CompileBackend.Hip)
    print("case: sddmm with a 32 MiB temporary is refused", flush=True)
    w, flat, want, got = _sddmm_case(lib, 64, 65536, 128, 32, 5)
    arr, cnt = _ptr_args(flat)
    rc = lib.parpy_hip_plan_run_noalloc(w.plan, arr, cnt)
    assert rc != 0
    assert b"scratch memory" in lib.parpy_get_error_message()
    torch.cuda.synchronize()
    assert bool((got == 7.0).all()), "a refused call must not have run anything"
    # the allocating entry point still serves the same plan
    assert lib.parpy_hip_plan_run(w.plan, arr, cnt) == 0
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want.cpu().numpy())
