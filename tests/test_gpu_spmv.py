"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F64_TOL = 1e-12  # relative L2, binary64
F16_TOL = 1e-2   # relative L2, binary16 values with binary32 accumulation


def rel_l2(got, ref):
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    d = np.linalg.norm(ref)
    return np.linalg.norm(got - ref) / (d if d > 0 else 1.0)


def oracle_y(ora, mx, A, x):
    if A.dtype == mx.MX_F64:
        return ora.spmv_f64(A.val, A.rowPtr, A.colInd, x)
    return ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0]


def test_mfma_operand_layout_f64(mx):
    """v_mfma_f64_16x16x4_f64: A[i][k] in lane 16k+i, B[k][j] in lane 16k+j, D[i][j] in
    accumulator register i//4 of lane 16*(i%4)+j -- the mapping tile_f64_kernel relies on."""
    from matxtract_amd import _lib
    rng = np.random.default_rng(5)
    A = rng.integers(-4, 5, (16, 4)).astype(np.float64)
    B = rng.integers(-4, 5, (4, 16)).astype(np.float64)
    a = np.zeros(64)
    b = np.zeros(64)
    for lane in range(64):
        a[lane] = A[lane % 16, lane // 16]
        b[lane] = B[lane // 16, lane % 16]
    raw = np.zeros((64, 4))
    _lib.check(_lib.load().mx_probe_mfma_f64(a.ctypes.data, b.ctypes.data, raw.ctypes.data))
    D = np.zeros((16, 16))
    for i in range(16):
        for j in range(16):
            D[i, j] = raw[16 * (i % 4) + j, i // 4]
    assert np.array_equal(D, A @ B)


def test_mfma_operand_layout_f16(mx):
    """v_mfma_f32_16x16x32_f16: A[i][8g+e] is element e of lane 16g+i, B[8g+e][j] element e of
    lane 16g+j, D[i][j] accumulator register i%4 of lane 16*(i//4)+j (tile_f16_kernel)."""
    from matxtract_amd import _lib
    rng = np.random.default_rng(6)
    A = rng.integers(-4, 5, (16, 32)).astype(np.float16)
    B = rng.integers(-4, 5, (32, 16)).astype(np.float16)
    a = np.zeros((64, 8), np.float16)
    b = np.zeros((64, 8), np.float16)
    for lane in range(64):
        for e in range(8):
            a[lane, e] = A[lane % 16, 8 * (lane // 16) + e]
            b[lane, e] = B[8 * (lane // 16) + e, lane % 16]
    raw = np.zeros((64, 4), np.float32)
    _lib.check(_lib.load().mx_probe_mfma_f16(a.ctypes.data, b.ctypes.data, raw.ctypes.data))
    D = np.zeros((16, 16), np.float32)
    for i in range(16):
        for j in range(16):
            D[i, j] = raw[16 * (i // 4) + j, i % 4]
    assert np.array_equal(D, A.astype(np.float32) @ B.astype(np.float32))


CASES = [
    # (workload, scale)
    (1, 1.0), (2, 1 / 16), (3, 0.02), (4, 1 / 32), (5, 1 / 128),
]
TAUS = [(0.0, 0.0), (0.5, 0.25), (1.0, 1.0), (0.75, 0.0), (0.25, 0.25), (1.0, 0.5)]


@pytest.mark.parametrize("cfg,scale", CASES)
@pytest.mark.parametrize("flags", ["default", "no_tiles", "all_tiles"])
def test_hybrid_spmv_matches_oracle(mx, ora, cfg, scale, flags):
    import torch
    A, x = mx.gen_config(cfg, scale=scale)
    ref = oracle_y(ora, mx, A, x)
    tol = F64_TOL if A.dtype == mx.MX_F64 else F16_TOL
    fl = {"default": mx.MX_PLAN_DEFAULT, "no_tiles": mx.MX_PLAN_NO_TILES, "all_tiles": mx.MX_PLAN_ALL_TILES}[flags]
    xd = torch.from_numpy(x).cuda()
    for tau in TAUS:
        print("case workload=%d scale=%g flags=%s tau=%s" % (cfg, scale, flags, tau), flush=True)
        part = mx.Partition(A, *tau)
        plan = mx.Plan(part, fl)
        y = plan.spmv(xd)
        torch.cuda.synchronize()
        err = rel_l2(y.cpu().numpy(), ref)
        assert err <= tol, (tau, err)
        # a second call must give the same answer (no state carried in y)
        y2 = plan.spmv(xd, y)
        torch.cuda.synchronize()
        assert rel_l2(y2.cpu().numpy(), ref) <= tol
        plan.close()
        part.close()
