"""mx_spmv_static -- the entry point that allocates nothing -- against mx_spmv, through the C ABI.

Its kernels put the sums of the virtual rows into a fixed device array of the library instead
of the plan's own buffer; everything else is shared with mx_spmv, so y must be the same bit
for bit.  Two calls in a row, the second on a smaller matrix (the array then still holds the
first call's sums beyond what the second writes), both precisions, a hybrid plan with strips,
a plan without slices (nothing to put into the array), and the refusal of a plan whose sums do
not fit.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(mx, torch, A, x, tau, flags):
    part = mx.Partition(A, *tau)
    plan = mx.Plan(part, flags)
    xd = torch.from_numpy(x).cuda()
    y_ref = plan.spmv(xd)
    torch.cuda.synchronize()
    y = torch.full_like(y_ref, float("nan"))
    plan.spmv_static(xd, y)                  # (the first call on a device looks the array's address up)
    torch.cuda.synchronize()
    # the property the entry point exists for: the device's free memory is the same before and after a call
    y.fill_(float("nan"))
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    plan.spmv_static(xd, y)
    free1 = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    assert free1 == free0 == torch.cuda.mem_get_info()[0], (free0, free1)
    info = dict(plan.info)
    plan.close()
    part.close()
    return y_ref.cpu().numpy(), y.cpu().numpy(), info


def test_static_entry_point_equals_mx_spmv(mx, ora):
    import torch
    lib = mx._lib.load()
    assert lib.mx_static_scratch_bytes() == 32 << 20
    calls = [
        # (workload, scale, tau, flags): larger first, then smaller
        (2, 1.0, (0.0, 0.0), mx.MX_PLAN_CSR_SLICES),
        (2, 0.5, (0.0, 0.0), mx.MX_PLAN_CSR_SLICES),   # a plan in the one-launch form: its two launches run here
        (2, 1 / 16, (0.0, 0.0), mx.MX_PLAN_CSR_SLICES),
        (4, 1.0, (0.0, 0.0), mx.MX_PLAN_CSR_SLICES),
        (5, 1 / 64, (1.0, 1.0), mx.MX_PLAN_CSR_SLICES | mx.MX_PLAN_KEEP_TILES),
        (2, 1 / 16, (1.0, 1.0), mx.MX_PLAN_ALL_TILES | mx.MX_PLAN_CSR_SLICES),
        (1, 1.0, (0.0, 0.0), mx.MX_PLAN_CSR_ROWS),
    ]
    used = []
    for cfg, scale, tau, flags in calls:
        print("static entry point: workload=%d scale=%g tau=%s flags=%d" % (cfg, scale, tau, flags), flush=True)
        A, x = mx.gen_config(cfg, scale=scale)
        y_ref, y, info = _both(mx, torch, A, x, tau, flags)
        assert np.array_equal(y_ref.view(np.uint16 if y.dtype == np.float16 else np.uint64),
                              y.view(np.uint16 if y.dtype == np.float16 else np.uint64)), (cfg, scale, tau, flags)
        # and it is the product: against the oracle, to the bar of the other parity tests
        if A.dtype == mx.MX_F64:
            ref, tol = ora.spmv_f64(A.val, A.rowPtr, A.colInd, x), 1e-12
        else:
            ref, tol = ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0].astype(np.float64), 1e-2
        err = np.linalg.norm(y.astype(np.float64) - ref) / np.linalg.norm(ref)
        assert err <= tol, (cfg, scale, tau, flags, err)
        if tau == (0.0, 0.0) and flags & mx.MX_PLAN_CSR_SLICES:
            assert info["csr_variant"] == 1  # the slice kernels, the ones that use the array
        used.append(info["csr_variant"])
    assert used.count(1) >= 4, used


def test_static_entry_point_holds_the_largest_workload(mx, ora):
    """The mixed workload at full size (27 MB of sums) fits the array: the hybrid plan of the benchmark's point,
    made on the device, through both entry points."""
    import torch
    A, x = mx.gen_config(5)
    plan = mx.Plan.from_device(torch.from_numpy(A.rowPtr).cuda(), torch.from_numpy(A.colInd).cuda(), torch.from_numpy(A.val).cuda(),
                               A.cols, 1.0, 1.0)
    assert plan.info["csr_variant"] == 1 and plan.info["tile_strip_nnz"] > 0
    xd = torch.from_numpy(x).cuda()
    y_ref = plan.spmv(xd)
    y = torch.full_like(y_ref, float("nan"))
    plan.spmv_static(xd, y)
    torch.cuda.synchronize()
    assert torch.equal(y, y_ref)
    ref = ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0].astype(np.float64)
    assert np.linalg.norm(y.cpu().numpy().astype(np.float64) - ref) / np.linalg.norm(ref) <= 1e-2
    plan.close()


def test_static_entry_point_refuses_what_does_not_fit(mx):
    import torch
    # 4.4 M rows of one entry each: one virtual row per row, 8 bytes of sum each -> more than 32 MiB
    rows = 4400000
    cols = 65536
    rng = np.random.default_rng(5)
    A = mx.Csr(rows, cols, np.arange(rows + 1, dtype=np.int32), rng.integers(0, cols, rows).astype(np.int32),
               rng.uniform(-1, 1, rows))
    x = rng.uniform(-1, 1, cols)
    part = mx.Partition(A, 0.0, 0.0)
    plan = mx.Plan(part, mx.MX_PLAN_CSR_SLICES)
    assert plan.info["csr_variant"] == 1
    xd = torch.from_numpy(x).cuda()
    y = torch.zeros(rows, dtype=torch.float64, device="cuda")
    with pytest.raises(mx.MxError) as e:
        plan.spmv_static(xd, y)
    assert e.value.code == 1 and "fixed array" in str(e.value)
    y_ref = plan.spmv(xd)  # the plan itself is fine
    torch.cuda.synchronize()
    ref = A.val * x[A.colInd]
    assert np.allclose(y_ref.cpu().numpy(), ref, rtol=1e-15, atol=0)
    plan.close()
    part.close()
