"""Host side of the product (no GPU): the partitioner against the oracle, bit for bit; the
generators; Matrix-Market ingest; the C ABI's symbols and error behaviour."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest
import scipy.sparse as sp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

INT_ARRAYS = ("newArray", "rId", "newArray_", "ddRowPtr", "ddColInd", "chunkPtr", "sparse_AToX_index",
              "fragPtr", "fragBit", "cdRowPtr", "cdColInd")
VAL_ARRAYS = ("ddVal", "tcVal", "cdVal")
SCALARS = ("dCols", "sCols", "nnzColD", "nnzColS", "dRows", "sRows", "nnzRowD", "nnzRowS", "chunkNum",
           "totalTcFrags", "tcValCount", "nnzCD", "fragM", "fragK")


def assert_same_partition(P, O):
    """P: product partition, O: oracle partition; every canonical array must be identical."""
    for name in SCALARS:
        assert getattr(P, name) == getattr(O, name), name
    for name in INT_ARRAYS:
        assert np.array_equal(getattr(P, name), getattr(O, name)), name
    for name in VAL_ARRAYS:  # compare bit patterns, not values
        a, b = getattr(P, name), getattr(O, name)
        assert a.dtype.itemsize == b.dtype.itemsize and np.array_equal(a.view(np.uint8), b.view(np.uint8)), name
    if P.dCols or P.dRows:
        assert np.array_equal(P.descColId, O.descColId), "descColId"
        assert P.cols_ratio == O.cols_ratio
        # 0 extracted entries over 0 fragments is 0/0 = NaN on both sides, as in the reference
        assert P.tc_nnz_ratio == O.tc_nnz_ratio or (np.isnan(P.tc_nnz_ratio) and np.isnan(O.tc_nnz_ratio))


TAUS = [(0.0, 0.0), (0.25, 0.0), (0.25, 0.25), (0.5, 0.25), (0.5, 0.5), (0.75, 0.5), (1.0, 0.0), (1.0, 0.75),
        (1.0, 1.0), (0.37, 0.11)]


@pytest.mark.parametrize("cfg,scale", [(1, 0.25), (2, 1 / 32), (3, 0.004), (4, 1 / 128), (5, 1 / 512)])
def test_partition_bit_exact_on_synthetic_workloads(mx, ora, cfg, scale):
    A, _ = mx.gen_config(cfg, scale=scale)
    for tau in TAUS:
        P = mx.Partition(A, *tau)
        O = ora.partition(A.rowPtr, A.colInd, A.val, A.cols, *tau)
        assert_same_partition(P, O)
        h = P.hash
        assert h == mx.Partition(A, *tau).hash  # deterministic (the partitioner is multi-threaded)
        P.close()


@pytest.mark.parametrize("cfg,taus", [(3, [(0.75, 0.5), (1.0, 1.0)]), (4, [(0.5, 0.25), (1.0, 1.0)]),
                                      (5, [(1.0, 1.0), (0.5, 0.25), (0.37, 0.11)])])
def test_partition_bit_exact_at_full_size(mx, ora, cfg, taus):
    """The partition at the sizes the benchmark runs, array for array against the oracle: above 2^24 entries
    (workloads 3 and 5) the reference's `int dColsNnz = nnzA * colProp` is a binary32 product that rounds
    (test/test_autotc_spmv.cpp:1131, :1249), and at tau = 1 on workload 5 the rounded target lies beyond the
    matrix, where every line with an entry is taken (63.3 M entries in tiles)."""
    A, _ = mx.gen_config(cfg)
    for tau in taus:
        P = mx.Partition(A, *tau)
        O = ora.partition(A.rowPtr, A.colInd, A.val, A.cols, *tau)
        assert_same_partition(P, O)
        assert P.nnzRowD + P.nnzCD == A.nnz
        if tau == (1.0, 1.0):
            assert P.nnzRowD == A.nnz and P.nnzCD == 0
        P.close()
        del O


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("dtype", [np.float64, np.float16])
def test_partition_bit_exact_on_hostile_inputs(mx, ora, seed, dtype):
    """Unsorted rows, repeated (row, col) pairs, empty rows and columns, non-square shapes, a
    ragged last chunk."""
    rng = np.random.default_rng(1000 + seed)
    rows, cols = int(rng.integers(1, 90)), int(rng.integers(1, 90))
    lens = rng.integers(0, min(cols, 12) + 1, rows)
    lens[rng.random(rows) < 0.2] = 0
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = rng.integers(0, cols, rp[-1]).astype(np.int32)      # with replacement: duplicates, any order
    va = (rng.integers(-8, 9, rp[-1]) / 8.0).astype(dtype)
    A = mx.Csr(rows, cols, rp, ci, va)
    for tau in TAUS:
        P = mx.Partition(A, *tau)
        O = ora.partition(rp, ci, va, cols, *tau)
        assert_same_partition(P, O)
        P.close()


def test_partition_rejects_bad_arguments(mx):
    A, _ = mx.gen_config(1, scale=0.05)
    with pytest.raises(mx.MxError) as e:
        mx.Partition(A, 0.25, 0.5)  # col_frac < hot_frac, as the reference CLI refuses
    assert e.value.code == 1 and "col_frac must be greater than hot_frac" in str(e.value)
    with pytest.raises(mx.MxError):
        mx.Partition(A, 1.5, 0.5)
    bad = mx.Csr(A.rows, A.cols, A.rowPtr, A.colInd.copy(), A.val)
    bad.colInd[3] = A.cols  # out of range
    with pytest.raises(mx.MxError):
        mx.Partition(bad, 0.5, 0.25)
    bad = mx.Csr(A.rows, A.cols, A.rowPtr.copy(), A.colInd, A.val)
    bad.rowPtr[2] = bad.rowPtr[3] + 1  # not monotone
    with pytest.raises(mx.MxError):
        mx.Partition(bad, 0.5, 0.25)


def test_empty_matrix(mx, ora):
    A = mx.Csr(5, 7, np.zeros(6, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float64))
    for tau in [(0.0, 0.0), (1.0, 1.0)]:
        P = mx.Partition(A, *tau)
        O = ora.partition(A.rowPtr, A.colInd, A.val, 7, *tau)
        assert P.nnzCD == 0 and P.totalTcFrags == 0
        assert_same_partition(P, O)


def test_transpose_matches_oracle_and_scipy(mx, ora):
    rng = np.random.default_rng(4)
    A = sp.random(80, 60, 0.1, format="csr", random_state=rng)
    A.sort_indices()
    for dtype in (np.float64, np.float16):
        val = A.data.astype(dtype)
        got = mx.transpose(A.indptr, A.indices, val, 60)
        ref = ora.transpose(A.indptr, A.indices, val, 60)
        for g, r in zip(got, ref):
            assert np.array_equal(g.view(np.uint8), r.view(np.uint8))
    C_ = A.tocsc()
    C_.sort_indices()
    tp, ti, tv = mx.transpose(A.indptr, A.indices, A.data, 60)
    assert np.array_equal(tp, C_.indptr) and np.array_equal(ti, C_.indices) and np.array_equal(tv, C_.data)


# ---------------------------------------------------------------- generators
def test_generators_are_seeded_and_well_formed(mx):
    for cfg, scale in [(1, 0.5), (2, 1 / 16), (3, 0.008), (4, 1 / 64), (5, 1 / 256)]:
        A, x = mx.gen_config(cfg, scale=scale)
        B, x2 = mx.gen_config(cfg, scale=scale)
        assert np.array_equal(A.colInd, B.colInd) and np.array_equal(A.val.view(np.uint8), B.val.view(np.uint8))
        assert np.array_equal(x.view(np.uint8), x2.view(np.uint8))
        C_, _ = mx.gen_config(cfg, seed=12345, scale=scale)
        if cfg != 3:  # the stencil has no random part in the matrix
            assert not np.array_equal(A.colInd, C_.colInd)
        assert A.rows == A.cols and A.rowPtr[0] == 0 and A.rowPtr[-1] == A.nnz
        for r in range(0, A.rows, max(1, A.rows // 200)):  # sorted, distinct columns in each row
            c = A.colInd[A.rowPtr[r]:A.rowPtr[r + 1]]
            assert np.all(np.diff(c) > 0) and (len(c) == 0 or (c[0] >= 0 and c[-1] < A.cols))
        assert A.val.dtype == (np.float64 if cfg <= 3 else np.float16)
        v = A.val.astype(np.float64)
        assert np.all(np.abs(v) <= 26.0) and np.all(np.isfinite(v))


def test_generator_shapes(mx):
    A, _ = mx.gen_config(1)
    assert A.rows == 4096 and A.nnz == 65536 and np.all(np.diff(A.rowPtr) == 16)
    A, _ = mx.gen_config(2, scale=1 / 8)
    assert A.rows == 8192 and np.all(np.diff(A.rowPtr) == 64)
    # 40% of the entries sit in dense, 8-aligned 8x8 blocks
    dense = 0
    for br in range(0, A.rows, 8):
        cols = [set(A.colInd[A.rowPtr[r]:A.rowPtr[r + 1]] // 8 * 8) for r in range(br, br + 8)]
        for c0 in set.intersection(*cols):
            if all(np.isin(np.arange(c0, c0 + 8), A.colInd[A.rowPtr[r]:A.rowPtr[r + 1]]).all() for r in range(br, br + 8)):
                dense += 64
    assert 0.38 <= dense / A.nnz <= 0.45
    A, x = mx.gen_config(3, scale=0.008)  # 20^3
    assert A.rows == 8000 and A.nnz == (3 * 20 - 2) ** 3 and x.min() >= 0 and x.max() <= 1
    A, _ = mx.gen_config(4, scale=1 / 16)
    lens = np.diff(A.rowPtr)
    assert lens.min() == 1 and lens.max() <= 4096 and 6 <= lens.mean() <= 16 and (lens == 1).mean() > 0.8
    A, _ = mx.gen_config(5, scale=1 / 64)
    lens = np.diff(A.rowPtr)
    strip = [r for r in range(0, A.rows, 8) if np.all(lens[r:r + 8] == 32) and
             np.all(np.diff(A.colInd[A.rowPtr[r]:A.rowPtr[r + 1]]) == 1)]
    assert 0.12 <= 8 * len(strip) / A.rows <= 0.28


def test_generator_families(mx):
    """mx_gen_config_family: the share of dense structure of workloads 2 and 5 as a parameter.  The benchmark's own
    share gives the benchmark's matrix; more share gives more dense structure, everything else as before; other
    workloads take no share."""
    for cfg, scale, default in ((2, 1 / 8, 0.4), (5, 1 / 64, 0.2)):
        A, x = mx.gen_config(cfg, scale=scale)
        B, xb = mx.gen_config(cfg, scale=scale, dense_share=default)
        assert np.array_equal(A.rowPtr, B.rowPtr) and np.array_equal(A.colInd, B.colInd) and np.array_equal(A.val, B.val)
        assert np.array_equal(x, xb)
        dense = []
        for share in (0.1, 0.4, 0.7) if cfg == 2 else (0.05, 0.2, 0.4):
            F, _ = mx.gen_config(cfg, scale=scale, dense_share=share)
            assert F.rows == A.rows and F.cols == A.cols
            rowOf = np.repeat(np.arange(F.rows), np.diff(F.rowPtr))
            assert np.all((np.diff(F.colInd) > 0) | (np.diff(rowOf) != 0))
            brk = np.ones(F.nnz, bool)
            brk[1:] = (np.diff(F.colInd) != 1) | (np.diff(rowOf) != 0)
            runs = np.diff(np.append(np.nonzero(brk)[0], F.nnz))
            dense.append(runs[runs >= 8].sum() / F.nnz)      # entries in runs of eight consecutive columns or more
            if cfg == 2:
                assert np.all(np.diff(F.rowPtr) == 64)
                assert abs(dense[-1] - share) < 0.05, (share, dense[-1])
        assert dense[0] < dense[1] < dense[2], dense
    with pytest.raises(mx.MxError):
        mx.gen_config(3, scale=1 / 64, dense_share=0.3)
    with pytest.raises(mx.MxError):
        mx.gen_config(2, scale=1 / 64, dense_share=1.5)


def test_generators_with_structure_off_the_grid(mx, ora):
    """MX_GEN_UNALIGNED: the 8 x 8 blocks of workload 2 start at any column of their band and the strips of workload
    5 at a column that is not a multiple of eight; everything else about the matrices stays as it was (sizes, row
    lengths, sorted distinct columns), and the partition of such a matrix equals the oracle's."""
    for cfg, scale in ((2, 1 / 8), (5, 1 / 64)):
        A, _ = mx.gen_config(cfg, scale=scale)
        U, x = mx.gen_config(cfg, scale=scale, unaligned=True)
        assert U.rows == A.rows and U.cols == A.cols and U.dtype == A.dtype
        assert U.colInd.min() >= 0 and U.colInd.max() < U.cols
        rowOf = np.repeat(np.arange(U.rows), np.diff(U.rowPtr))
        assert np.all((np.diff(U.colInd) > 0) | (np.diff(rowOf) != 0))
        # runs of at least eight consecutive columns, and where they start
        brk = np.ones(U.nnz, bool)
        brk[1:] = (np.diff(U.colInd) != 1) | (np.diff(rowOf) != 0)
        starts = np.nonzero(brk)[0]
        big = np.diff(np.append(starts, U.nnz)) >= 8
        off = np.bincount(U.colInd[starts[big]] % 8, minlength=8) / big.sum()
        if cfg == 2:
            assert np.all(np.diff(U.rowPtr) == 64) and U.nnz == A.nnz
            assert off.min() > 0.08                    # every offset about as often as any other
            # the dense blocks are still there: eight rows from a multiple of eight share the run
            r = int(rowOf[starts[big][len(starts[big]) // 2]]) // 8 * 8
            c0 = int(U.colInd[starts[big][len(starts[big]) // 2]])
            for rr in range(r, r + 8):
                assert np.isin(np.arange(c0, c0 + 8), U.colInd[U.rowPtr[rr]:U.rowPtr[rr + 1]]).all()
        else:
            lens = np.diff(U.rowPtr)
            strip = [r for r in range(0, U.rows, 8) if np.all(lens[r:r + 8] == 32) and
                     np.all(np.diff(U.colInd[U.rowPtr[r]:U.rowPtr[r + 1]]) == 1)]
            assert 0.12 <= 8 * len(strip) / U.rows <= 0.28
            at = np.array([U.colInd[U.rowPtr[r]] % 8 for r in strip])
            assert (at == 0).mean() < 0.05              # (a strip pushed back from the last columns may land on the grid)
        for tau in ((1.0, 1.0), (0.5, 0.25)):
            P = mx.Partition(U, *tau)
            assert_same_partition(P, ora.partition(U.rowPtr, U.colInd, U.val, U.cols, *tau))
            P.close()


# ---------------------------------------------------------------- Matrix-Market ingest
def write_mtx(path, header, size, lines):
    with open(path, "w") as f:
        f.write("%%MatrixMarket matrix coordinate " + header + "\n% a comment\n" + size + "\n" + "\n".join(lines) + "\n")


def test_mmio_general_keeps_file_order(mx, tmp_path):
    p = tmp_path / "g.mtx"
    write_mtx(p, "real general", "3 4 5", ["2 3 1.5", "1 4 -2", "2 1 3", "1 1 4", "2 3 7"])
    A, sym = mx.mmio_read(p)
    assert not sym and (A.rows, A.cols, A.nnz) == (3, 4, 5)
    assert A.rowPtr.tolist() == [0, 2, 5, 5]
    assert A.colInd.tolist() == [3, 0, 2, 0, 2]           # file order inside each row, duplicates kept
    assert A.val.tolist() == [-2.0, 4.0, 1.5, 3.0, 7.0]


def test_mmio_symmetric_expansion_and_pattern(mx, tmp_path):
    p = tmp_path / "s.mtx"
    write_mtx(p, "pattern symmetric", "3 3 3", ["2 1", "3 3", "3 1"])
    A, sym = mx.mmio_read(p)
    assert sym and A.nnz == 5
    D = sp.csr_matrix((A.val, A.colInd, A.rowPtr), shape=(3, 3)).toarray()
    assert np.array_equal(D, np.array([[0, 1, 1], [1, 0, 0], [1, 0, 1.0]]))
    # the mirrored entry directly follows the stored one: row 0 gets (0,1) from "2 1" then (0,2) from "3 1"
    assert A.colInd[A.rowPtr[0]:A.rowPtr[1]].tolist() == [1, 2]
    p = tmp_path / "k.mtx"
    write_mtx(p, "real skew-symmetric", "2 2 1", ["2 1 5"])
    A, sym = mx.mmio_read(p)
    assert not sym and A.nnz == 1                          # not expanded, as in the reference
    p = tmp_path / "i.mtx"
    write_mtx(p, "integer general", "2 2 2", ["1 1 3", "2 2 -4"])
    A, _ = mx.mmio_read(p, mx.MX_F16)
    assert A.val.dtype == np.float16 and A.val.tolist() == [3.0, -4.0]
    with pytest.raises(mx.MxError) as e:
        mx.mmio_read(tmp_path / "missing.mtx")
    assert e.value.code == 4


def _read_reference_head(path, fragbit_dtype, val_dtype):
    """The read sequence of the reference's tile-file reader (test/tckernel.cpp:586-638)."""
    with open(path, "rb") as f:
        def arr(dtype, n):
            return np.frombuffer(f.read(np.dtype(dtype).itemsize * n), dtype=dtype)
        chunkNum = int(arr(np.int32, 1)[0])
        chunkPtr = arr(np.int32, chunkNum + 1)
        totalTcFrags, fragK = (int(v) for v in arr(np.int32, 2))
        atox = arr(np.int32, totalTcFrags * fragK)
        fragPtr = arr(np.int32, int(arr(np.uint64, 1)[0]))
        fragBit = arr(fragbit_dtype, int(arr(np.uint64, 1)[0]))
        tcVal = arr(val_dtype, int(arr(np.uint64, 1)[0]))
        return chunkPtr, fragK, atox, fragPtr, fragBit, tcVal, f.tell()


@pytest.mark.parametrize("cfg,scale", [(1, 1.0), (2, 1 / 16), (5, 1 / 256)])
def test_partition_file_round_trip(mx, cfg, scale, tmp_path):
    """save -> load gives the same partition, array for array; the head of the file is laid out
    as the reference's tile file, so a reader written after the reference's finds its arrays."""
    A, _ = mx.gen_config(cfg, scale=scale)
    f64 = A.dtype == mx.MX_F64
    for tau in ((0.0, 0.0), (0.5, 0.25), (1.0, 1.0)):
        P = mx.Partition(A, *tau)
        path = str(tmp_path / ("p_%d_%g_%g.dat" % (cfg, tau[0], tau[1])))
        P.save(path)
        Q = mx.Partition.load(path, A.dtype)
        assert Q.hash == P.hash
        assert (Q.tau_c, Q.tau_r) == (P.tau_c, P.tau_r) == (np.float32(tau[0]), np.float32(tau[1]))
        for name in mx.Partition.ARRAYS:
            assert np.array_equal(getattr(P, name), getattr(Q, name)), name
        for name in ("rows", "cols", "nnz", "dCols", "sCols", "dRows", "sRows", "nnzRowD", "nnzCD", "chunkNum",
                     "totalTcFrags", "tcValCount", "cols_ratio", "tc_nnz_ratio"):
            assert getattr(P, name) == getattr(Q, name), name
        chunkPtr, fragK, atox, fragPtr, fragBit, tcVal, _ = _read_reference_head(
            path, np.uint32 if f64 else np.uint64, np.float64 if f64 else np.float16)
        assert fragK == P.fragK
        assert np.array_equal(chunkPtr, P.chunkPtr) and np.array_equal(atox, P.sparse_AToX_index)
        assert np.array_equal(fragPtr, P.fragPtr) and np.array_equal(fragBit, P.fragBit)
        assert np.array_equal(tcVal.view(np.uint8), np.asarray(P.tcVal).view(np.uint8))
        P.close()
        Q.close()


def test_partition_file_is_checked_on_load(mx, tmp_path):
    A, _ = mx.gen_config(2, scale=1 / 32)
    P = mx.Partition(A, 0.5, 0.25)
    good = str(tmp_path / "good.dat")
    P.save(good)
    blob = open(good, "rb").read()
    _, _, _, _, _, _, head_end = _read_reference_head(good, np.uint32, np.float64)

    def load(data, dtype=mx.MX_F64):
        path = str(tmp_path / "case.dat")
        with open(path, "wb") as f:
            f.write(data)
        return mx.Partition.load(path, dtype)

    # a value changed in the residual: the checksum catches it
    bad = bytearray(blob)
    bad[-64] ^= 0x40
    with pytest.raises(mx.MxError, match="checksum|range|inconsistent"):
        load(bytes(bad))
    # cut short, in the head and in the extension
    for n in (10, head_end - 3, head_end + 40, len(blob) - 1):
        with pytest.raises(mx.MxError):
            load(blob[:n])
    # the tile part alone is what the reference's tool writes: refused, with a message that says why
    with pytest.raises(mx.MxError, match="tile part only"):
        load(blob[:head_end])
    # read with the other precision
    with pytest.raises(mx.MxError):
        load(blob, mx.MX_F16)
    # a column index pushed out of range (inside the reference's part of the file)
    bad = bytearray(blob)
    off = 4 + 4 * (P.chunkNum + 1) + 8  # first entry of sparse_AToX_index
    bad[off:off + 4] = np.int32(P.dCols + 5).tobytes()
    with pytest.raises(mx.MxError):
        load(bytes(bad))
    with pytest.raises(mx.MxError):
        mx.Partition.load(str(tmp_path / "missing.dat"))
    P.close()


def _walk_slice_layout(L, x, f64, subset=False):
    """y from the slice kernel's layout, walked the way the kernel walks it (workgroup, wave,
    batch, step, lane), every index checked on the way.  Accumulates in float64."""
    BE, W, SW = L["batchEntries"], L["waves"], L["sliceCols"]
    assert L["stepEntries"] == 1   # chunks may end after any entry
    ecol, ev = L["ecol"], L["eval"].astype(np.float64)
    if L.get("use_dict"):
        # the value dictionary form: a byte per entry at the place of its column offset names the value
        assert 0 < L["nDict"] <= 255 and len(L["ecode"]) == len(ecol) and np.all(L["dict"][L["nDict"]:] == 0)
        assert np.all((L["ecode"] < L["nDict"]) | (L["ecode"] == 255))
    partial = np.full(L["chunks"] * 64, np.nan)
    assert len(ecol) >= L["batches"] * 64 * BE
    lane = np.arange(64)
    seen_chunks = 0
    for b in range(L["nWG"]):
        q, wgChunk0, wgChunks, _ = L["wgDesc"][b]
        assert 0 <= q < L["S"] and wgChunk0 == seen_chunks and (0 if L.get("fused") else 1) <= wgChunks <= 4096
        xs = np.zeros(SW)
        n = max(0, min(SW, len(x) - q * SW))
        xs[:n] = x[q * SW:q * SW + n]
        inside = 0
        for w in range(W):
            batch0, nb, chunk0, nChunks = L["waveDesc"][b * W + w]
            assert chunk0 == inside and 0 <= batch0 and batch0 + nb <= L["batches"]
            inside += nChunks
            ends = L["chunkEnd"][wgChunk0 + chunk0:wgChunk0 + chunk0 + nChunks]
            assert np.all(np.diff(np.concatenate(([0], ends))) > 0) and (nChunks == 0 or ends[-1] <= nb * BE)
            assert nChunks == 0 or ends[-1] > (nb - 1) * BE, "a wave's stream has no spare batch"
            acc, ci = np.zeros(64), 0
            for t in range(nb):
                bt = batch0 + t
                c = ecol[bt * 64 * BE:(bt + 1) * 64 * BE].reshape(64, BE).astype(np.int64)
                if L.get("use_dict"):
                    v = L["dict"].astype(np.float64)[L["ecode"][bt * 64 * BE:(bt + 1) * 64 * BE]].reshape(64, BE)
                elif f64:   # sub-blocks of two values per lane
                    v = ev[bt * 64 * BE:(bt + 1) * 64 * BE].reshape(BE // 2, 64, 2).transpose(1, 0, 2).reshape(64, BE)
                else:
                    v = ev[bt * 64 * BE:(bt + 1) * 64 * BE].reshape(64, BE)
                assert c.max() < SW
                for k in range(BE):
                    acc += v[:, k] * xs[c[:, k]]
                    if ci < nChunks and t * BE + k + 1 == ends[ci]:
                        partial[(wgChunk0 + chunk0 + ci) * 64 + lane] = acc
                        acc, ci = np.zeros(64), ci + 1
            assert ci == nChunks
        assert inside == wgChunks
        seen_chunks += wgChunks
    assert seen_chunks == L["chunks"] and not np.isnan(partial).any()
    segPtr, segIdx = L["segPtr"], L["segIdx"]
    assert segPtr[0] == 0 and segPtr[-1] == L["vrows"] == len(segIdx) and np.all(np.diff(segPtr) >= 0)
    assert len(np.unique(segIdx)) == len(segIdx) and (len(segIdx) == 0 or (segIdx.min() >= 0 and segIdx.max() < len(partial)))
    # y as the combine kernel forms it: rows with one virtual row through rowInfo, the others through the lists
    nv = np.diff(segPtr)
    info = L["rowInfo"]
    assert np.array_equal(info[nv == 0], np.full((nv == 0).sum(), -1)) and np.all(info[nv > 1] == -2)
    single = nv == 1
    assert np.array_equal(info[single], segIdx[segPtr[:-1][single]])
    y = np.zeros(len(nv))      # rows without entries: zero (all rows) or not written (subset)
    y[single] = partial[info[single]]
    y[nv > 1] = np.nan
    for lst, lo, hi in ((L["lightInfo"], 2, L["lightSegs"]), (L["heavyInfo"], L["lightSegs"] + 1, 1 << 30)):
        for r, a, n, _ in lst:
            assert n == nv[r] and a == segPtr[r] and lo <= n <= hi and np.isnan(y[r])
            y[r] = partial[segIdx[a:a + n]].sum()
    assert not np.isnan(y).any()
    return y, partial


@pytest.mark.parametrize("dtype", [np.float64, np.float16])
def test_slice_layout_walk_with_a_value_dictionary(mx, ora, dtype):
    """A matrix with few distinct values: the layout also holds one byte per entry and the values
    they name; walked through those instead of the values it gives the same sums, bit for bit, and
    its padding names the zero.  A matrix with more than 255 values has no such form."""
    rng = np.random.default_rng(12)
    A, _ = mx.gen_config(5 if dtype == np.float16 else 2, scale=1 / 256 if dtype == np.float16 else 1 / 32)
    assert A.nnz >= 65536
    few = mx.Csr(A.rows, A.cols, A.rowPtr, A.colInd, rng.choice(np.array([-2.0, -0.5, 0.25, 1.0, 3.0]), A.nnz).astype(dtype))
    x = rng.integers(-2, 3, A.cols).astype(np.float64)
    L = mx.slice_layout(few, nCU=8)
    assert L["nDict"] == 5
    y_plain, p_plain = _walk_slice_layout(L, x, dtype == np.float64)
    L["use_dict"] = True
    y_dict, p_dict = _walk_slice_layout(L, x, dtype == np.float64)
    assert np.array_equal(p_plain, p_dict) and np.array_equal(y_plain, y_dict)
    M = sp.csr_matrix((few.val.astype(np.float64), few.colInd, few.rowPtr), shape=(few.rows, few.cols))
    assert np.array_equal(y_dict, M @ x)
    assert mx.slice_layout(A, nCU=8)["nDict"] == 0   # the generator's values: thousands of them


@pytest.mark.parametrize("case", ["block", "powerlaw", "mixed", "unsorted", "tiny", "wide_f64", "subset"])
def test_slice_layout_walk(mx, ora, case):
    """The column-slice layout, walked on the CPU exactly as the kernel reads it, gives A x; the
    padding it stores is zero; rows cut into several virtual rows add up; a subset of the rows
    leaves the others without virtual rows."""
    rng = np.random.default_rng(5)
    sel = None
    nCU = 8
    if case == "block":
        A, x = mx.gen_config(2, scale=1 / 32)
    elif case == "powerlaw":
        A, x = mx.gen_config(4, scale=1 / 64)
    elif case == "mixed":
        A, x = mx.gen_config(5, scale=1 / 128)
        nCU = 3
    elif case == "wide_f64":   # five binary64 slices, one of them empty, ragged last slice
        rows, cols = 700, 4 * 16384 + 77
        lens = rng.integers(0, 90, rows)
        lens[5] = 3000
        rp = np.zeros(rows + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        ci = np.concatenate([np.sort(rng.choice(cols, n, replace=False)) for n in lens]).astype(np.int32)
        ci[(ci >= 16384) & (ci < 32768)] += 16384
        A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)))
        x = rng.uniform(-1, 1, cols)
    elif case == "unsorted":   # columns in any order inside a row, duplicates allowed
        rows, cols = 300, 70000
        lens = rng.integers(0, 200, rows)
        rp = np.zeros(rows + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        ci = rng.integers(0, cols, rp[-1]).astype(np.int32)
        A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)).astype(np.float16))
        x = rng.uniform(-1, 1, cols).astype(np.float16)
    elif case == "tiny":
        A = mx.Csr(3, 5, np.array([0, 2, 2, 3], np.int32), np.array([4, 0, 2], np.int32), np.array([1.0, 2.0, 3.0]))
        x = np.arange(1.0, 6.0)
    else:
        A, x = mx.gen_config(4, scale=1 / 64)
        sel = (np.diff(A.rowPtr) >= 32).astype(np.uint8)
    f64 = A.dtype == mx.MX_F64
    L = mx.slice_layout(A, nCU=nCU, sel=sel)
    assert L["S"] == -(-A.cols // L["sliceCols"])
    y, _ = _walk_slice_layout(L, np.asarray(x, np.float64), f64, subset=sel is not None)
    lens = np.diff(A.rowPtr)
    keep = np.ones(A.rows, bool) if sel is None else sel.astype(bool)
    ref = np.zeros(A.rows)
    rowOf = np.repeat(np.arange(A.rows), lens)
    np.add.at(ref, rowOf, A.val.astype(np.float64) * np.asarray(x, np.float64)[A.colInd])
    ref[~keep] = 0.0
    assert np.allclose(y, ref, rtol=1e-12, atol=1e-12 * max(1.0, np.abs(ref).max()))
    # every stored value is an entry of the matrix or a zero: the sums of absolute values agree
    held = np.abs(A.val.astype(np.float64))[np.repeat(keep, lens)].sum()
    assert np.isclose(np.abs(L["eval"].astype(np.float64)).sum(), held, rtol=1e-12)
    # rows outside the subset own nothing; no virtual row is longer than the cap
    nv = np.diff(L["segPtr"])
    assert np.all(nv[~keep] == 0) and np.all(nv[keep & (lens > 0)] >= 1) and np.all(nv[lens == 0] == 0)
    assert np.all(nv <= -(-lens // 1) ) and L["cap"] % L["batchEntries"] == 0


def _xcd_of_logical_workgroup(b, nWG):
    """Logical workgroups [k * nWG / 8, (k + 1) * nWG / 8) are taken by workgroups that run on XCD k."""
    assert nWG % 8 == 0
    return b // (nWG // 8)


@pytest.mark.parametrize("case", ["block", "stencil", "wide_f64", "unsorted_f16", "empty_rows"])
def test_fused_slice_layout_walk(mx, case):
    """The layout of the one-launch form, walked on the CPU: the streams give the same sums as ever; every
    workgroup's sums belong to rows of the groups it counts off; all workgroups that count a group off
    sit on one XCD and are as many as the group expects; every group is counted off by someone; and the
    places of a row name exactly its virtual rows, so that adding them up gives A x."""
    rng = np.random.default_rng(9)
    nCU = 16
    if case == "block":
        A, x = mx.gen_config(2, scale=1 / 8)
        nCU = 64
    elif case == "stencil":
        A, x = mx.gen_config(3, scale=0.03)
        nCU = 32
    elif case == "wide_f64":
        nCU = 64
        rows, cols = 5000, 4 * 16384 + 77
        lens = rng.integers(0, 40, rows)
        rp = np.zeros(rows + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        ci = np.concatenate([np.sort(rng.choice(cols, n, replace=False)) for n in lens]).astype(np.int32)
        A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)))
        x = rng.uniform(-1, 1, cols)
    elif case == "unsorted_f16":
        nCU = 40
        rows, cols = 4100, 3 * 65536 + 5
        lens = rng.integers(0, 30, rows)
        rp = np.zeros(rows + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        ci = rng.integers(0, cols, rp[-1]).astype(np.int32)
        A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)).astype(np.float16))
        x = rng.uniform(-1, 1, cols).astype(np.float16)
    else:   # long stretches of rows without entries: their groups must still be counted off and written as zero
        nCU = 32
        rows, cols = 6000, 40000
        lens = rng.integers(1, 50, rows)
        lens[300:1700] = 0
        lens[4000:4600] = 0
        rp = np.zeros(rows + 1, np.int32)
        rp[1:] = np.cumsum(lens)
        ci = np.concatenate([np.sort(rng.choice(cols, n, replace=False)) for n in lens]).astype(np.int32)
        A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)))
        x = rng.uniform(-1, 1, cols)
    f64 = A.dtype == mx.MX_F64
    L = mx.slice_layout(A, nCU=nCU, fused=True)
    assert L["fused"] == 1 and L["nWG"] == nCU and L["groupRows"] == 256 and L["nGroups"] == -(-A.rows // 256)
    xf = np.asarray(x, np.float64)
    y2, partial = _walk_slice_layout(L, xf, f64)          # the arrays of the two-launch form stay valid
    GR, P = L["groupRows"], L["placesPerRow"]
    segPtr, segIdx = L["segPtr"], L["segIdx"]
    rowOfV = np.full(L["chunks"] * 64, -1)
    rowOfV[segIdx] = np.repeat(np.arange(A.rows), np.diff(segPtr))
    need = np.zeros(L["nGroups"], np.int64)
    xcdOfGroup = np.full(L["nGroups"], -1)
    for b in range(L["nWG"]):
        g0, ng = L["wgGroups"][b]
        _, c0, nc, _ = L["wgDesc"][b]
        k = _xcd_of_logical_workgroup(b, L["nWG"])
        assert 0 <= g0 and g0 + ng <= L["nGroups"] and (ng > 0 or nc == 0)
        need[g0:g0 + ng] += 1
        assert np.all((xcdOfGroup[g0:g0 + ng] == -1) | (xcdOfGroup[g0:g0 + ng] == k)), "a group is counted off from two XCDs"
        xcdOfGroup[g0:g0 + ng] = k
        mine = rowOfV[c0 * 64:(c0 + nc) * 64]
        mine = mine[mine >= 0]
        assert mine.size == 0 or (mine.min() // GR >= g0 and mine.max() // GR < g0 + ng), "sums outside the workgroup's groups"
    assert np.array_equal(need, L["groupNeed"]) and need.min() >= 1
    # the sums as the one-launch kernel stores them: virtual row v at fusedTarget[v]; the k-th virtual row of
    # row r sits at ((r // GR) * P + k) * GR + r % GR, padding lanes at the spare places behind the last group
    nv = np.diff(segPtr)
    assert nv.max() == P and 1 <= P <= 8 and np.array_equal(L["rowVrows"][:A.rows], nv) and np.all(L["rowVrows"][A.rows:] == 0)
    tgt = L["fusedTarget"]
    spare = L["nGroups"] * P * GR
    assert tgt.shape == (L["chunks"] * 64,)
    pad = rowOfV < 0
    assert np.array_equal(tgt[pad], spare + (np.nonzero(pad)[0] & 63))
    real = tgt[~pad]
    assert len(np.unique(real)) == len(real) and real.max() < spare
    sums = np.zeros(spare + 64)
    sums[tgt] = partial
    y = np.zeros(A.rows)
    rows = np.arange(A.rows)
    for k in range(P):
        has = nv > k
        at = ((rows // GR) * P + k) * GR + rows % GR
        assert np.array_equal(at[has], tgt[segIdx[segPtr[:-1][has] + k]])
        y[has] += sums[at[has]]
    assert L["wgDesc"][:, 2].max() <= 96     # the targets of a workgroup's chunks fit the LDS beside x
    ref = np.zeros(A.rows)
    np.add.at(ref, np.repeat(np.arange(A.rows), np.diff(A.rowPtr)), A.val.astype(np.float64) * xf[A.colInd])
    assert np.allclose(y, ref, rtol=1e-12, atol=1e-12 * max(1.0, np.abs(ref).max()))
    assert np.allclose(y2, ref, rtol=1e-12, atol=1e-12 * max(1.0, np.abs(ref).max()))


def test_fused_slice_layout_is_refused_where_it_does_not_fit(mx):
    """A row with more than eight virtual rows, or fewer workgroups per XCD than slices: the ordinary layout."""
    A, _ = mx.gen_config(4, scale=1 / 32)     # power-law rows reach every slice
    L = mx.slice_layout(A, nCU=64, fused=True)
    assert np.diff(L["segPtr"]).max() > 8 and L["fused"] == 0
    plain = mx.slice_layout(A, nCU=64)
    for k in ("wgDesc", "waveDesc", "chunkEnd", "segIdx", "ecol", "eval", "rowInfo"):
        assert np.array_equal(L[k], plain[k]), k
    B, _ = mx.gen_config(2, scale=1 / 2)      # two slices everywhere, one workgroup per XCD
    assert mx.slice_layout(B, nCU=8, fused=True)["fused"] == 0


def test_slice_layout_rejects_bad_matrices(mx):
    rp = np.array([0, 2, 3], np.int32)
    good = mx.Csr(2, 4, rp, np.array([0, 3, 1], np.int32), np.ones(3))
    assert mx.slice_layout(good, nCU=4)["vrows"] == 2          # both rows lie in one slice: one virtual row each
    for bad_cols in (np.array([0, 4, 1], np.int32), np.array([0, -1, 1], np.int32)):
        A = mx.Csr.__new__(mx.Csr)
        A.__dict__.update(good.__dict__)
        A.colInd = bad_cols
        with pytest.raises(mx.MxError, match="column index"):
            mx.slice_layout(A, nCU=4)
    A = mx.Csr.__new__(mx.Csr)
    A.__dict__.update(good.__dict__)
    A.rowPtr = np.array([0, 3, 2], np.int32)
    with pytest.raises(mx.MxError, match="rowPtr"):
        mx.slice_layout(A, nCU=4)
    with pytest.raises(mx.MxError):
        mx.slice_layout(good, nCU=0)


@pytest.mark.parametrize("seed", range(6))
def test_slice_layout_walk_random_shapes(mx, seed):
    """Random shapes, precisions, machine sizes and row subsets through the same walk."""
    rng = np.random.default_rng(100 + seed)
    f64 = bool(seed % 2)
    rows = int(rng.integers(1, 3000))
    cols = int(rng.integers(1, 5 * (16384 if f64 else 65536)))
    kind = seed % 3
    if kind == 0:
        lens = rng.integers(0, 60, rows)
    elif kind == 1:
        lens = np.minimum(cols, np.floor(1.5 * rng.uniform(1e-4, 1, rows) ** (-1 / 0.6)).astype(np.int64))
    else:
        lens = (rng.uniform(size=rows) < 0.3).astype(np.int64)
        lens[rng.integers(0, rows)] = min(cols, 20000)
    lens = np.minimum(lens, cols)
    rp = np.zeros(rows + 1, np.int32)
    rp[1:] = np.cumsum(lens)
    ci = np.concatenate([rng.choice(cols, n, replace=False) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int32)
    dt = np.float64 if f64 else np.float16
    A = mx.Csr(rows, cols, rp, ci, rng.uniform(-1, 1, len(ci)).astype(dt))
    x = rng.uniform(-1, 1, cols).astype(dt).astype(np.float64)
    sel = (rng.uniform(size=rows) < 0.5).astype(np.uint8) if seed >= 3 else None
    L = mx.slice_layout(A, nCU=int(rng.integers(1, 40)), sel=sel)
    y, _ = _walk_slice_layout(L, x, f64, subset=sel is not None)
    keep = np.ones(rows, bool) if sel is None else sel.astype(bool)
    ref = np.zeros(rows)
    np.add.at(ref, np.repeat(np.arange(rows), lens), A.val.astype(np.float64) * x[A.colInd])
    ref[~keep] = 0.0
    assert np.allclose(y, ref, rtol=1e-12, atol=1e-12 * max(1.0, np.abs(ref).max(initial=0.0)))


def test_init_vec(mx):
    v = mx.init_vec(40)
    assert np.array_equal(v, np.arange(40) % 15)
    h = mx.init_vec(40, mx.MX_F16)
    assert h.dtype == np.float16 and np.array_equal(h.astype(np.float64), np.arange(40) % 15)


def test_f16_conversions_match_numpy(mx):
    from matxtractt_amd import _lib
    L = _lib.load()
    rng = np.random.default_rng(2)
    vals = np.concatenate([rng.uniform(-70000, 70000, 3000), rng.uniform(-1e-4, 1e-4, 3000),
                           [0.0, 65504.0, 65520.0, 2.9802322e-08, 1e-9, np.inf]]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.mx_f32_to_f16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, ref)
    h = np.arange(0, 65536, 7, dtype=np.uint16)
    back = np.array([L.mx_f16_to_f32(int(b)) for b in h], np.float32)
    ref = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(back[ok], ref[ok])


def test_algorithmic_bytes(mx):
    # nnz*(sizeof(valT)+4) + (rows+1)*4 + cols*sizeof(valT) + rows*sizeof(valT)
    assert mx.algorithmic_bytes(mx.MX_F64, 4096, 4096, 65536) == 868356
    assert mx.algorithmic_bytes(mx.MX_F64, 1000000, 1000000, 26463592) == 337563108
    assert mx.algorithmic_bytes(mx.MX_F16, 10, 20, 100) == 100 * 6 + 11 * 4 + 20 * 2 + 10 * 2


# ---------------------------------------------------------------- ABI
def declared_symbols():
    text = open(os.path.join(ROOT, "include", "matxtract_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(mx):
    from matxtractt_amd import _lib
    L = _lib.load()
    names = declared_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(L, n), "libmatxtract_hip.so does not export " + n
    assert sorted(_lib.SIGNATURES) == names  # the Python binding covers exactly the header


def test_device_entry_points_fail_loudly_without_a_gpu(mx):
    if mx.device_count() > 0:
        pytest.skip("a GPU is present")
    A, x = mx.gen_config(1, scale=0.05)
    P = mx.Partition(A, 0.5, 0.25)
    with pytest.raises(mx.MxError) as e:
        mx.Plan(P)
    assert e.value.code == 3 and "no CPU fallback" in str(e.value)
    with pytest.raises(mx.MxError):
        mx.cdspmv(A, x, np.zeros(A.rows))
    # the device route of the extraction has no host fallback either
    with pytest.raises(mx.MxError) as e:
        mx.Partition(A, 0.5, 0.25, device=True)
    assert e.value.code == 3 and "no HIP device" in str(e.value)
    with pytest.raises(mx.MxError) as e:  # arguments are checked before anything touches the device
        mx.Partition(A, 0.25, 0.5, device=True)
    assert e.value.code == 1
    # tau = (0, 0) extracts nothing: handed to the host routine, device or not
    mx.Partition(A, 0.0, 0.0, device=True).close()


def test_product_does_not_reach_into_the_oracle():
    """Nothing under the package, the headers or bench-independent entry points names the oracle."""
    pkg = os.path.join(ROOT, "matxtractt_amd")
    for base, _, files in os.walk(pkg):
        if os.path.basename(base) == "build":
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h", "Makefile")):
                text = open(os.path.join(base, f), errors="replace").read()
                assert "mx_oracle" not in text and "oracle/" not in text, os.path.join(base, f)


# ---------------------------------------------------------------- CLI argument handling (no GPU needed)
def cli(*args):
    exe = os.path.join(ROOT, "matxtractt_amd", "bin", "matxtract_perftest")
    if not os.path.exists(exe):
        pytest.skip("CLI not built")
    return subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)


def test_cli_argument_errors_match_the_reference():
    r = cli()
    assert r.returncode == 1 and "Run the code by './matxtract_perftest (col_frac) (hot_frac) matrix.mtx'." in r.stdout
    r = cli("0.2", "0.5", "x.mtx")
    assert r.returncode == 1 and "Error: col_frac must be greater than hot_frac." in r.stdout
    r = cli("0.5", "0.2", "0.1", "x.mtx")
    assert r.returncode == 1 and "Error: Too many arguments provided." in r.stdout


# ---------------------------------------------------------------- the host half of a plan, walked on the CPU
def _walk_plan_layout(L, x, dtype):
    """y as the kernels would compute it from a plan's host layout: the CSR part row by row, the
    tile layouts step by step -- slot j of half h multiplies its fragM x fragK block with the x at
    the step's column ids (general layout) or at first column + 0..fragK-1 (strip layout); a
    half's rows collect until a step with flag 1, then the sums go to y (added in the general
    layout, stored in the strip layout, whose rows nothing else may write; the binary64 form of the
    second layout -- blocks of 8 x 8, four slots per half -- shares its rows with the CSR part and is
    added once)."""
    fragM, slots = L["fragM"], L["slots"]
    x = np.asarray(x, np.float64)
    y = np.zeros(L["rows"])
    rp, ci, va = L["csrRowPtr"], L["csrColInd"], L["csrVal"].astype(np.float64)
    for r in range(L["rows"]):
        y[r] = np.dot(va[rp[r]:rp[r + 1]], x[ci[rp[r]:rp[r + 1]]])
    touched = np.zeros(L["rows"], bool)
    entries = 0
    for t, T in enumerate(L["tiles"]):
        fragK = 8 if t == 1 else L["fragK"]        # the plan's own chunks are made of 8-column blocks
        half = 4 if t == 1 else slots // 2
        val = T["val"].astype(np.float64)
        seen_steps = 0
        for w in range(T["nWaves"]):
            s0, s1 = T["waveDesc"][w][:2]
            assert s0 == seen_steps and s1 > s0, "waves cover the steps in order"
            seen_steps = s1
            acc = np.zeros((2, fragM))
            for s in range(s0, s1):
                hdr = T["hdr"][s]
                flags, n = hdr[16], (hdr[17], hdr[18])
                assert 0 <= n[0] <= half and 0 <= n[1] <= half and n[0] + n[1] > 0
                vo = T["valOffset"][s]
                for h in range(2):
                    for j in range(n[h]):
                        slot = 2 * j + h if (t == 0 and fragK == 4) else half * h + j   # the general binary64 step interleaves its halves
                        blk = val[vo + ((n[0] if h else 0) + j) * fragM * fragK:][:fragM * fragK].reshape(fragM, fragK)
                        if t == 1:
                            c0 = hdr[21 + slot]
                            assert c0 >= 0 and c0 % fragK == 0 and c0 + fragK <= L["cols"]
                            cols = np.arange(c0, c0 + fragK)
                            assert np.array_equal(T["atox"][s][slot * fragK:(slot + 1) * fragK], cols), "both forms of a strip step agree"
                        else:
                            cols = T["atox"][s][slot * fragK:(slot + 1) * fragK]
                        used = cols >= 0
                        assert np.all(blk[:, ~used] == 0) and np.all(cols[used] < L["cols"])
                        acc[h] += blk[:, used] @ x[cols[used]]
                        entries += int(np.count_nonzero(blk))
                if flags & 1:
                    for h in range(2):
                        rows = hdr[8 * h:8 * h + fragM] if (flags & 2) or h == 0 else None
                        if rows is None:
                            continue
                        sums = acc[h] if (flags & 2) else acc[0] + acc[1]
                        for i, r in enumerate(rows):
                            if r < 0:
                                assert sums[i] == 0
                                continue
                            if t == 1 and L["fragK"] == 4:
                                assert L["stripRows"][r] == 2 and not touched[r], "a row of a block chunk is finished once"
                                touched[r] = True
                                y[r] += sums[i]
                            elif t == 1:
                                assert L["stripRows"][r] == 1 and not touched[r] and y[r] == 0, "a strip row is written once, by the strips alone"
                                touched[r] = True
                                y[r] = sums[i]
                            else:
                                assert L["stripRows"][r] == 0
                                y[r] += sums[i]
                    acc[:] = 0
            assert not acc.any(), "a wave ends on a stored step"
        assert seen_steps == T["steps"]
    assert np.array_equal(touched, L["stripRows"].astype(bool)), "every strip row is written"
    return y, entries


def _strip_matrix(mx, rng, rows=1024, cols=6000):
    """binary16: runs of rows that are one aligned run of 32 columns, among short random rows, one of
    them as long as a strip row."""
    rp, ci = [0], []
    for r in range(rows):
        if r == 70:
            c = sorted(rng.choice(cols, 32, replace=False).tolist())
        elif (r // 64) % 3 == 0:
            base = 8 * ((r // 8) % 600)
            c = list(range(base, base + 32))
        else:
            c = sorted(rng.choice(cols, 1 + int(rng.integers(0, 3)), replace=False).tolist())
        ci += c
        rp.append(len(ci))
    va = rng.integers(-3, 4, len(ci)).astype(np.float16)
    return mx.Csr(rows, cols, np.array(rp, np.int32), np.array(ci, np.int32), va)


def _block_rows_matrix(mx, rng, rows=768, cols=4003):
    """binary16: groups of rows that share two or three aligned blocks of eight columns, far apart,
    each row holding five to eight of a block's columns; runs of 20 columns off the grid of eight;
    short random rows between."""
    rp, ci = [0], []
    for r in range(rows):
        grp = r // 16
        if grp % 3 == 0:
            blocks = [(7 * grp) % 400, 100 + (11 * grp) % 300, 450 + grp % 40][:2 + grp % 2]
            c = sorted(int(8 * b + k) for b in set(blocks) for k in rng.choice(8, int(rng.integers(5, 9)), replace=False))
        elif grp % 3 == 1:
            base = 8 * ((5 * grp) % 450) + 3
            c = list(range(base, base + 20))
        elif grp == 5:
            c = list(range(3992, 4003))    # reaches into the last, partial block of x: never a strip row
        else:
            c = sorted(rng.choice(cols, 1 + int(rng.integers(0, 3)), replace=False).tolist())
        ci += c
        rp.append(len(ci))
    va = rng.integers(-3, 4, len(ci)).astype(np.float16)
    return mx.Csr(rows, cols, np.array(rp, np.int32), np.array(ci, np.int32), va)


@pytest.mark.parametrize("case", ["block_f64", "mixed_f16", "strips_f16", "blocks_f16", "twice_f64", "twice_f16", "stencil_f64"])
def test_plan_layout_walk(mx, ora, case):
    """The host half of a plan -- fragment gate, strip rows, the CSR part, both tile layouts --
    reproduces A x exactly (integer data) for every combination of plan flags, without a GPU."""
    rng = np.random.default_rng(sum(map(ord, case)))
    if case == "strips_f16":
        A = _strip_matrix(mx, rng)
    elif case == "blocks_f16":
        A = _block_rows_matrix(mx, rng)
    elif case.startswith("twice"):
        dtype = np.float64 if case.endswith("f64") else np.float16
        lens = rng.integers(0, 50, 300)
        rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        A = mx.Csr(300, 80, rp, rng.integers(0, 80, rp[-1]).astype(np.int32), rng.integers(-3, 4, rp[-1]).astype(dtype))
    else:
        cfg, scale = {"block_f64": (2, 1 / 64), "mixed_f16": (5, 1 / 512), "stencil_f64": (3, 1 / 512)}[case]
        A, _ = mx.gen_config(cfg, scale=scale)
        A = mx.Csr(A.rows, A.cols, A.rowPtr, A.colInd, rng.integers(-3, 4, A.nnz).astype(A.val.dtype))
    x = rng.integers(-2, 3, A.cols).astype(A.val.dtype)
    ref = (ora.spmv_f64(A.val, A.rowPtr, A.colInd, x) if A.dtype == mx.MX_F64
           else ora.spmv_f16_f32acc(A.val, A.rowPtr, A.colInd, x)[0]).astype(np.float64)
    strips_seen = 0
    for tau in ((1.0, 1.0), (0.75, 0.5), (0.5, 0.0), (0.0, 0.0)):
        P = mx.Partition(A, *tau)
        for flags in (mx.MX_PLAN_DEFAULT, mx.MX_PLAN_KEEP_TILES, mx.MX_PLAN_ALL_TILES, mx.MX_PLAN_NO_TILES):
            L = mx.plan_layout(P, flags, nCU=4)
            y, entries = _walk_plan_layout(L, x, A.val.dtype)
            assert np.array_equal(y, ref), (case, tau, flags)
            if flags == mx.MX_PLAN_NO_TILES or tau == (0.0, 0.0):
                assert L["tiles"][0]["steps"] == 0 and L["tiles"][1]["steps"] == 0 and L["csr_nnz"] == A.nnz
            if flags == mx.MX_PLAN_ALL_TILES:
                assert L["tiles"][1]["steps"] == 0, "strip chunks are a matter of the default selection"
            strips_seen += L["tiles"][1]["steps"]
        P.close()
    assert (strips_seen > 0) == (case in ("strips_f16", "blocks_f16", "mixed_f16", "block_f64")), strips_seen



def _chunks_of_steps(hdr):
    """The block counts of a tile layout's chunks, read back from its step headers: a step whose
    halves are different chunks (flag 2) holds two (or one, waiting for a partner that never came), a
    chunk larger than half a step runs over steps without that flag up to one with flag 1."""
    chunks, run = [], 0
    for h in hdr:
        flags, n0, n1 = int(h[16]), int(h[17]), int(h[18])
        if flags & 2:
            chunks.append(n0)
            if n1 > 0:
                chunks.append(n1)
        else:
            run += n0 + n1
            if flags & 1:
                chunks.append(run)
                run = 0
    assert run == 0
    return chunks


@pytest.mark.parametrize("case", ["block_f64", "mixed_f16", "strips_f16", "blocks_f16", "twice_f64"])
def test_tile_steps_from_block_counts_alone(mx, case):
    """mx_tile_steps -- the host's share of laying tiles out on the device: steps and waves from the
    chunks' block counts -- gives the steps, value offsets, look-ahead fields and waves that
    mx_plan_layout gives the same chunks (general tiles, binary16 strips, binary64 blocks)."""
    rng = np.random.default_rng(sum(map(ord, case)))
    if case == "strips_f16":
        A = _strip_matrix(mx, rng)
    elif case == "blocks_f16":
        A = _block_rows_matrix(mx, rng)
    elif case == "twice_f64":
        lens = rng.integers(0, 50, 300)
        rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        A = mx.Csr(300, 80, rp, rng.integers(0, 80, rp[-1]).astype(np.int32), rng.integers(-3, 4, rp[-1]).astype(np.float64))
    else:
        cfg, scale = {"block_f64": (2, 1 / 64), "mixed_f16": (5, 1 / 512)}[case]
        A, _ = mx.gen_config(cfg, scale=scale)
    seen = 0
    for tau in ((1.0, 1.0), (0.75, 0.5)):
        P = mx.Partition(A, *tau)
        for flags in (mx.MX_PLAN_KEEP_TILES, mx.MX_PLAN_ALL_TILES):
            for nCU in (1, 4):
                L = mx.plan_layout(P, flags, nCU=nCU)
                f64 = A.dtype == mx.MX_F64
                for t, T in enumerate(L["tiles"]):
                    if T["steps"] == 0:
                        continue
                    # the plan's own chunks are made of blocks of 8 columns, four to a half, in both precisions
                    slots, values, per_min = (8, 64, 1 if f64 else 2) if t == 1 else (L["slots"], 8 * L["fragK"], 2)
                    chunks = _chunks_of_steps(T["hdr"])
                    S = mx.tile_steps(chunks, slots, values, per_min, nCU)
                    assert S["steps"] == T["steps"] and S["nWaves"] == T["nWaves"], (case, tau, flags, t)
                    assert np.array_equal(S["stepDesc"][:, 2:5], T["hdr"][:, 16:19])          # flags, blocks per half
                    assert np.array_equal(S["stepDesc"][:, 5], T["valOffset"])
                    assert np.array_equal(S["stepDesc"][:, 6:8], T["hdr"][:, 19:21])          # the step four further on
                    assert np.array_equal(S["waveDesc"], T["waveDesc"])
                    assert S["totalBlocks"] * values == T["val"].size
                    assert len(chunks) == T["chunks"]
                    seen += 1
        P.close()
    assert seen > 0, case
    with pytest.raises(mx.MxError):
        mx.tile_steps([0, 3], 8, 64, 2, 4)


def test_host_code_under_sanitizers(tmp_path):
    """The library's host code (generators, partition, slice layout, the host half of a plan) built
    with -fsanitize=address,undefined and run on the five workloads at small scale: no report."""
    import shutil
    import subprocess
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    src = os.path.join(ROOT, "matxtractt_amd", "csrc")
    exe = str(tmp_path / "host_driver")
    cmd = ["g++", "-O1", "-g", "-std=c++17", "-fopenmp", "-fsanitize=address,undefined", "-fno-omit-frame-pointer",
           "-fno-sanitize-recover=undefined", "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROOT, "include"), "-I" + src,
           "-I/opt/rocm/include", os.path.join(ROOT, "tests", "sanitize", "host_driver.cpp"),
           os.path.join(ROOT, "tests", "sanitize", "launch_stubs.cpp")] + \
          [os.path.join(src, f) for f in ("mx_util.cpp", "mx_partition.cpp", "mx_gen.cpp", "mx_mmio.cpp", "mx_host_layout.cpp",
                                          "mx_plan.cpp", "mx_plan_device.cpp", "mx_plan_view.cpp", "mx_run.cpp", "mx_tune.cpp",
                                          "mx_oneshot.cpp")] + \
          ["-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib", "-o", exe]
    b = subprocess.run(cmd, capture_output=True, text=True)
    if b.returncode != 0 and ("asan" in b.stderr or "ubsan" in b.stderr) and "cannot find" in b.stderr:
        pytest.skip("sanitizer runtimes not installed")
    assert b.returncode == 0, b.stderr[-2000:]
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", OMP_NUM_THREADS="4")
    r = subprocess.run([exe], capture_output=True, text=True, env=env, timeout=600)
    assert r.returncode == 0 and r.stdout.strip().endswith("ok"), (r.stdout[-500:], r.stderr[-3000:])
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]


@pytest.mark.parametrize("cfg,scale,tau,variant", [
    (1, 1.0, (0.0, 0.0), 0),      # 65 k entries: one launch of the row kernel beats two of the slice form
    (2, 1.0, (0.0, 0.0), 1),      # scattered columns, 4.2 M entries: x in LDS
    (2, 0.25, (0.0, 0.0), 0),     # the same matrix at a quarter of the size: too small for two launches
    (3, 0.1, (0.0, 0.0), 0),      # stencil: neighbouring entries share lines of x
    (3, 1.0, (0.0, 0.0), 1),      # ... at full size its two distinct values make the one-byte form of the slices win
    (4, 1.0, (0.0, 0.0), 1),
    (5, 0.1, (0.0, 0.0), 1),
    (5, 1.0, (1.0, 1.0), 1),      # the hybrid point the benchmark reports: strips + slices
])
def test_plan_form_is_decided_from_the_matrix(mx, cfg, scale, tau, variant):
    """The form of the CSR part comes from counts over the matrix and fixed rates, not from a timed
    trial: the same matrix gets the same plan on every run (and under a profiler).  Checked here
    against what the five workloads measured fastest on MI355X."""
    A, _ = mx.gen_config(cfg, scale=scale)
    part = mx.Partition(A, *tau)
    seen = []
    for _ in range(2):
        L = mx.plan_layout(part, mx.MX_PLAN_DEFAULT, nCU=256)
        seen.append((L["csr_variant"], round(L["est_rows_us"], 6), round(L["est_slices_us"], 6)))
    part.close()
    assert seen[0] == seen[1]
    assert seen[0][0] == variant, seen[0]
    assert seen[0][1] > 0 and seen[0][2] > 0
    # pinned forms leave no choice and say so
    part = mx.Partition(A, *tau)
    L = mx.plan_layout(part, mx.MX_PLAN_CSR_ROWS, nCU=256)
    assert L["csr_variant"] == 0 and L["est_rows_us"] == 0.0
    part.close()
