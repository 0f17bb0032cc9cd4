"""The reference's C++ surface (include/MatXtract.h, mmio.h, csr2csc.h of this repository).

CPU: the reference's own driver source, where it is at hand, must pass the compiler's syntax
and type checks against this include directory in both precisions, except for its one direct
CUDA call; and the in-repo driver tests/cxx/surface_driver.cpp, which uses the same calls with
the same argument shapes, must build.  GPU: that driver runs and everything it computes is
compared with the oracle.
"""
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DRIVER = "/root/reference/test/test_autotc_spmv.cpp"
CXX_DIR = os.path.join(ROOT, "tests", "cxx")


def _gxx():
    if shutil.which("g++") is None:
        pytest.skip("no g++")


@pytest.mark.parametrize("precision", ["fp64", "fp16"])
def test_reference_driver_passes_the_syntax_check(precision):
    """g++ -fsyntax-only on the reference's driver, as it lies in the reference's tree (nothing
    of it is copied or kept), with this repository's include/ in place of the reference's: every
    name it uses from MatXtract.h, csr2csc.h, mmio.h and common.h must resolve, with the
    reference's argument types.  The one thing that may not: cudaDeviceSynchronize() (:1529),
    which a maintainer deletes (the wrappers are synchronous)."""
    _gxx()
    if not os.path.exists(REF_DRIVER):
        pytest.skip("the reference's source is not on this machine")
    cmd = ["g++", "-std=c++17", "-fopenmp", "-fsyntax-only", "-I" + os.path.join(ROOT, "include"), REF_DRIVER]
    if precision == "fp64":
        cmd.insert(1, "-Dfp64")
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    errors = [l for l in r.stderr.splitlines() if re.search(r"\berror\b", l)]
    assert len(errors) == 1 and "cudaDeviceSynchronize" in errors[0], "\n".join(errors[:20])


def _build_drivers():
    _gxx()
    r = subprocess.run(["make", "-C", CXX_DIR, "all"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "warning" not in r.stderr, r.stderr[-2000:]
    return {p: os.path.join(CXX_DIR, "build", "surface_driver_" + p) for p in ("fp64", "fp16")}


def test_surface_driver_builds_in_both_precisions(mx):
    """cdspmv, du_tcspmv_fp64 / du_tcspmv_fp16_v2 with vectors by value, se_tcspmv_*, csr2csc /
    csc2csr, exclusive_scan, initVec, divup through the three headers the reference's driver
    includes, -Wall -Wextra clean, linked against the library."""
    exes = _build_drivers()
    assert all(os.path.exists(e) for e in exes.values())


def _read_arrays(path, dtypes):
    buf = open(path, "rb").read()
    out, at = [], 0
    for dt in dtypes:
        n = int(np.frombuffer(buf, np.int64, 1, at)[0])
        at += 8
        out.append(np.frombuffer(buf, dt, n, at).copy())
        at += n * np.dtype(dt).itemsize
    assert at == len(buf)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("precision,workload,scale,tau", [
    ("fp64", 2, 1 / 16, (0.5, 0.25)), ("fp64", 2, 1 / 16, (1.0, 1.0)), ("fp64", 3, 0.02, (0.75, 0.5)),
    ("fp16", 5, 1 / 128, (0.5, 0.25)), ("fp16", 5, 1 / 128, (1.0, 1.0)), ("fp16", 4, 1 / 32, (0.75, 0.25)),
])
def test_surface_driver_against_the_oracle(mx, ora, tmp_path, precision, workload, scale, tau):
    exes = {p: os.path.join(CXX_DIR, "build", "surface_driver_" + p) for p in ("fp64", "fp16")}
    if not all(os.path.exists(e) for e in exes.values()):
        exes = _build_drivers()
    out = str(tmp_path / "out.bin")
    print("surface driver: %s workload=%d scale=%g tau=%s" % (precision, workload, scale, tau), flush=True)
    env = dict(os.environ, MATXTRACT_WARM="1", MATXTRACT_ITERS="2")
    r = subprocess.run([exes[precision], str(workload), repr(scale), repr(tau[0]), repr(tau[1]), out],
                       capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout[-500:], r.stderr[-2000:])
    vt = np.float64 if precision == "fp64" else np.float16
    i32 = np.int32
    (cscPtr, cscInd, cscVal, backPtr, backInd, backVal, y_cd, y_du, order, y_se, scan, iv, du) = _read_arrays(
        out, [i32, i32, vt, i32, i32, vt, vt, vt, i32, vt, i32, vt, i32])
    A, x = mx.gen_config(workload, scale=scale)
    f64 = precision == "fp64"
    tol = 1e-12 if f64 else 1e-2

    def rel(got, ref):
        got, ref = got.astype(np.float64), ref.astype(np.float64)
        return np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-300)

    # transposes: the oracle's csr2csc, and back again (rows come back stably sorted by column)
    tp, ti, tv = ora.transpose(A.rowPtr, A.colInd, A.val, A.cols)
    assert np.array_equal(cscPtr, tp) and np.array_equal(cscInd, ti) and np.array_equal(cscVal.view(np.uint8), tv.view(np.uint8))
    bp, bi, bv = ora.transpose(tp, ti, tv, A.rows)
    assert np.array_equal(backPtr, bp) and np.array_equal(backInd, bi) and np.array_equal(backVal.view(np.uint8), bv.view(np.uint8))
    # products
    if f64:
        ref = ora.spmv_f64(A.val, A.rowPtr, A.colInd, x)
    else:
        ref = ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0].astype(np.float64)
    y0 = (np.arange(A.rows) % 3).astype(np.float64)
    assert rel(y_cd, ref + y0) <= tol                      # cdspmv adds to the Y it is given
    assert rel(y_du, ref) <= tol, rel(y_du, ref)            # du_tcspmv_* + scatter through rId + cdspmv on top
    assert rel(y_se, ref) <= tol, rel(y_se, ref)            # se_tcspmv_* + scatter through rId[order_rid] + cdspmv
    P = ora.partition(A.rowPtr, A.colInd, A.val, A.cols, *tau)
    assert sorted(order.tolist()) == list(range(P.dRows))  # a permutation of [0, dRows)
    assert scan.tolist() == [0, 3, 3, 8, 9, 9] and du[0] == 3
    assert np.array_equal(iv.astype(np.float64), (np.arange(20) % 15).astype(np.float64))
