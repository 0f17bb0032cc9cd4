"""Known-answer fixtures of the canonical partition (tests/golden/partition_*.json, written by
tests/golden/make_golden.py: a naive pure-Python restatement that shares no code with the C oracle
or the library).  The oracle and the library's host partitioner must both reproduce every array;
on a GPU the plans built from them must give the fixtures' y exactly (small integers: no rounding
in either precision)."""
import glob
import json
import os

import numpy as np
import pytest

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "partition_*.json")))
SCALARS = ("dCols", "sCols", "nnzColD", "dRows", "sRows", "nnzRowD", "chunkNum", "totalTcFrags", "nnzCD")
INT_ARRAYS = ("newArray", "rId", "newArray_", "ddRowPtr", "ddColInd", "chunkPtr", "sparse_AToX_index", "fragPtr",
              "cdRowPtr", "cdColInd")
VAL_ARRAYS = ("ddVal", "tcVal", "cdVal")


def load(path):
    with open(path) as f:
        return json.load(f)


def check_partition(P, want, dtype, who):
    for k in SCALARS:
        assert getattr(P, k) == want[k], (who, k)
    assert np.array_equal(np.asarray(P.descColId), np.array(want["descColId"], np.int32)), (who, "descColId")
    for k in INT_ARRAYS:
        assert np.array_equal(np.asarray(getattr(P, k)), np.array(want[k], np.int32)), (who, k)
    for k in VAL_ARRAYS:
        assert np.array_equal(np.asarray(getattr(P, k)).astype(np.float64), np.array(want[k], np.float64)), (who, k)
    bits = np.array([int(b, 16) for b in want["fragBit"]], dtype=np.uint32 if dtype == np.float64 else np.uint64)
    assert np.array_equal(np.asarray(P.fragBit), bits), (who, "fragBit")


def test_fixtures_are_there():
    assert len(GOLDEN) >= 6


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[10:-5] for p in GOLDEN])
@pytest.mark.parametrize("dtype", [np.float64, np.float16], ids=["f64", "f16"])
def test_oracle_and_library_reproduce_the_fixture(ora, mx, path, dtype):
    fx = load(path)
    want = fx["f64" if dtype == np.float64 else "f16"]
    rp, ci = np.array(fx["rowPtr"], np.int32), np.array(fx["colInd"], np.int32)
    va = np.array(fx["val"], dtype)
    x = np.array(fx["x"], dtype)
    y = np.array(fx["y"], np.float64)
    # the oracle
    Po = ora.partition(rp, ci, va, fx["cols"], fx["tau_c"], fx["tau_r"])
    check_partition(Po, want, dtype, "oracle")
    assert np.array_equal(np.asarray(Po.hybrid(x), np.float64), _hybrid_expectation(fx, want)), "oracle hybrid y"
    spmv = ora.spmv_f64(va, rp, ci, x) if dtype == np.float64 else ora.spmv_f16_f32acc(va, rp, ci, x)[0]
    assert np.array_equal(np.asarray(spmv, np.float64), y), "oracle spmv y"
    # the library's host partitioner
    A = mx.Csr(fx["rows"], fx["cols"], rp, ci, va)
    Pl = mx.Partition(A, fx["tau_c"], fx["tau_r"])
    check_partition(Pl, want, dtype, "library")
    Pl.close()


def _hybrid_expectation(fx, want):
    """y as the reference's hybrid computes it: the tiles hold one value per (row, column) -- of a
    column named twice the last -- plus the residual product."""
    x = np.array(fx["x"], np.float64)
    y = np.zeros(fx["rows"])
    x_cd = np.concatenate([x[want["descColId"][:want["dCols"]]], x[want["newArray"]]]) if want["dCols"] else x
    for i in range(fx["rows"]):
        for p in range(want["cdRowPtr"][i], want["cdRowPtr"][i + 1]):
            y[i] += want["cdVal"][p] * x_cd[want["cdColInd"][p]]
    fragK = len(want["sparse_AToX_index"]) // max(want["totalTcFrags"], 1)
    for w in range(want["chunkNum"]):
        for f in range(want["chunkPtr"][w], want["chunkPtr"][w + 1]):
            bits, k = int(want["fragBit"][f], 16), want["fragPtr"][f]
            for b in range(8 * fragK):
                if (bits >> b) & 1:
                    col = want["descColId"][want["sparse_AToX_index"][f * fragK + b % fragK]]
                    y[want["rId"][8 * w + b // fragK]] += want["tcVal"][k] * x[col]
                    k += 1
    return y


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float16], ids=["f64", "f16"])
def test_plans_give_the_fixtures_y(mx, dtype):
    import torch
    for path in GOLDEN:
        fx = load(path)
        A = mx.Csr(fx["rows"], fx["cols"], np.array(fx["rowPtr"], np.int32), np.array(fx["colInd"], np.int32),
                   np.array(fx["val"], dtype))
        xd = torch.from_numpy(np.array(fx["x"], dtype)).cuda()
        for tau in ((fx["tau_c"], fx["tau_r"]), (0.0, 0.0)):
            for flags in (mx.MX_PLAN_DEFAULT, mx.MX_PLAN_KEEP_TILES, mx.MX_PLAN_ALL_TILES):
                print("golden", fx["name"], np.dtype(dtype).name, tau, flags, flush=True)
                P = mx.Partition(A, *tau)
                plan = mx.Plan(P, flags)
                y = plan.spmv(xd)
                torch.cuda.synchronize()
                assert np.array_equal(y.cpu().numpy().astype(np.float64), np.array(fx["y"], np.float64)), (fx["name"], tau, flags)
                plan.close()
                P.close()
