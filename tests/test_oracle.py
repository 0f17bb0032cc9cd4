"""Pins the CPU oracle (oracle/mx_oracle.c) against things it does not share code with:
library routines (scipy, numpy), brute force on tiny inputs, closed forms and invariants.
None of these tests re-types the oracle's own formula."""
import numpy as np
import pytest
import scipy.sparse as sp


def random_csr(rng, rows, cols, density, dtype=np.float64, sort=True):
    A = sp.random(rows, cols, density, format="csr", random_state=rng, dtype=np.float64)
    A.data[:] = rng.uniform(-1, 1, A.nnz)
    if sort:
        A.sort_indices()
    return A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(dtype), A


# ---------------------------------------------------------------- binary16 conversions
def test_h2f_all_bit_patterns(ora):
    h = np.arange(65536, dtype=np.uint16)
    got = np.array([ora.lib().ora_h2f(int(v)) for v in h], dtype=np.float32)
    ref = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(ref)], ref.view(np.uint32)[~np.isnan(ref)])
    assert np.all(np.isnan(got[np.isnan(ref)]))


def test_f2h_matches_numpy_round_to_nearest_even(ora):
    rng = np.random.default_rng(0)
    vals = [0.0, -0.0, 1.0, -1.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-08, 2.9802322e-08,
            2.98023224e-08 * 1.0000001, 6.1035156e-05, 6.0975552e-05, np.inf, -np.inf, 1e10, -1e10,
            1.0009765625, 1.00048828125, 1.00146484375, 0.333251953125]
    vals += list(rng.uniform(-70000, 70000, 4000)) + list(rng.uniform(-1, 1, 4000))
    vals += list(rng.uniform(-1e-4, 1e-4, 4000)) + list(rng.uniform(-1e-7, 1e-7, 2000))
    # exact ties between neighbouring binary16 values
    h = rng.integers(0, 0x7bff, 3000).astype(np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    vals += list((lo + hi) / 2)
    vals = np.array(vals, dtype=np.float32)
    with np.errstate(over="ignore"):
        ref = vals.astype(np.float16).view(np.uint16)
    got = np.array([ora.lib().ora_f2h(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, ref)


# ---------------------------------------------------------------- spmv_serial
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_spmv_f64_matches_scipy(ora, seed):
    rng = np.random.default_rng(seed)
    rp, ci, va, A = random_csr(rng, 300, 257, 0.05)
    x = rng.uniform(-1, 1, 257)
    y = ora.spmv_f64(va, rp, ci, x)
    ref = A @ x
    assert np.linalg.norm(y - ref) <= 1e-14 * np.linalg.norm(ref)


def test_spmv_f64_dense_brute_force_and_accumulate(ora):
    rng = np.random.default_rng(7)
    n = 48
    D = np.where(rng.random((n, n)) < 0.3, rng.integers(-5, 6, (n, n)), 0).astype(np.float64)
    A = sp.csr_matrix(D)
    x = rng.integers(-7, 8, n).astype(np.float64)
    y0 = rng.integers(-3, 4, n).astype(np.float64)
    # integer data: every partial sum is exact, so equality is bit-exact; y is added to (Y += A x)
    y = ora.spmv_f64(A.data, A.indptr, A.indices, x, y0=y0)
    assert np.array_equal(y, y0 + D @ x)


def test_spmv_f64_identity_and_unsorted_duplicates(ora):
    n = 17
    rp = np.arange(n + 1, dtype=np.int32)
    ci = np.arange(n, dtype=np.int32)
    x = np.linspace(-1, 1, n)
    assert np.array_equal(ora.spmv_f64(np.ones(n), rp, ci, x), x)
    # columns out of order and repeated inside a row are legal input
    rp = np.array([0, 4], np.int32)
    ci = np.array([2, 0, 2, 1], np.int32)
    va = np.array([1.0, 2.0, 3.0, 4.0])
    assert ora.spmv_f64(va, rp, ci, np.array([10.0, 100.0, 1000.0]))[0] == 2 * 10 + 4 * 100 + 4 * 1000


def test_spmv_f64_stencil_closed_form(ora, mx):
    # 27-point stencil (centre 26, neighbours -1) applied to the all-ones vector gives
    # 26 - (#neighbours): 0 inside, 9 on faces, 15 on edges, 19 at corners.
    A, _ = mx.gen_config(3, scale=0.001)  # 10^3 grid
    g = round(A.rows ** (1 / 3))
    assert g ** 3 == A.rows
    y = ora.spmv_f64(A.val, A.rowPtr, A.colInd, np.ones(A.cols)).reshape(g, g, g)
    on_border = lambda i: (i == 0) | (i == g - 1)
    z, yy, xx = np.meshgrid(np.arange(g), np.arange(g), np.arange(g), indexing="ij")
    nb = on_border(z).astype(int) + on_border(yy) + on_border(xx)
    expect = np.choose(nb, [0.0, 9.0, 15.0, 19.0])
    assert np.array_equal(y, expect)


def test_spmv_f16_f32acc_matches_numpy_cumsum(ora):
    rng = np.random.default_rng(11)
    rp, ci, va, _ = random_csr(rng, 200, 190, 0.1, dtype=np.float16)
    x = rng.uniform(-1, 1, 190).astype(np.float16)
    y32, y16 = ora.spmv_f16_f32acc(va, rp, ci, x)
    for r in range(200):
        prods = va[rp[r]:rp[r + 1]].astype(np.float32) * x[ci[rp[r]:rp[r + 1]]].astype(np.float32)
        acc = np.float32(0)
        for p in prods:  # sequential binary32 accumulation in CSR order
            acc = np.float32(acc + p)
        assert y32[r] == acc
        assert y16[r] == np.float16(acc)


def test_spmv_f16_halfacc_matches_numpy_float16_loop(ora):
    rng = np.random.default_rng(12)
    rp, ci, va, _ = random_csr(rng, 60, 50, 0.2, dtype=np.float16)
    x = rng.uniform(-1, 1, 50).astype(np.float16)
    y = ora.spmv_f16_halfacc(va, rp, ci, x)
    for r in range(60):
        t = np.float16(0)
        for p in range(rp[r], rp[r + 1]):
            prod = np.float16(np.float32(va[p]) * np.float32(x[ci[p]]))
            t = np.float16(np.float32(t) + np.float32(prod))
        assert y[r] == t


def test_eqcheck_semantics(ora):
    a = np.array([1.0, 2.0, 0.0, 4.0])
    assert ora.eqcheck(a, a.copy(), 1e-8) == -1
    b = a.copy()
    b[3] *= 1 + 1e-6
    assert ora.eqcheck(a, b, 1e-8) == 3
    # 0 against 0 is 0/0 = NaN, which the reference's check lets pass
    assert ora.eqcheck(np.zeros(3), np.zeros(3), 1e-8) == -1


# ---------------------------------------------------------------- transposes
def test_transpose_matches_scipy_and_round_trips(ora):
    rng = np.random.default_rng(3)
    rp, ci, va, A = random_csr(rng, 120, 90, 0.07)
    tp, ti, tv = ora.transpose(rp, ci, va, 90)
    C = A.tocsc()
    C.sort_indices()
    assert np.array_equal(tp, C.indptr) and np.array_equal(ti, C.indices) and np.array_equal(tv, C.data)
    bp, bi, bv = ora.transpose(tp, ti, tv, 120)
    assert np.array_equal(bp, rp) and np.array_equal(bi, ci) and np.array_equal(bv, va)


def test_transpose_is_stable_on_duplicates(ora):
    # row 0 lists column 1 twice, column 0 once, in this order: (1,a) (0,b) (1,c)
    rp = np.array([0, 3, 5], np.int32)
    ci = np.array([1, 0, 1, 1, 1], np.int32)
    va = np.array([1.0, 2.0, 3.0, 4.0, 5.0])
    tp, ti, tv = ora.transpose(rp, ci, va, 2)
    assert tp.tolist() == [0, 1, 5]
    assert ti.tolist() == [0, 0, 0, 1, 1]          # ascending source row
    assert tv.tolist() == [2.0, 1.0, 3.0, 4.0, 5.0]  # equal (row, col) pairs keep source order


# ---------------------------------------------------------------- thresholds
def test_threshold_is_float_product_truncated(ora):
    f32 = np.float32
    cases = [(100, 0.5), (26463592, 0.25), (26463592, 1.0), (2 ** 24, 1.0), (2 ** 24 + 1, 1.0),
             (2 ** 24 + 3, 1.0), (63290371, 0.5), (63290371, 1.0), (64000001, 0.75), (11257094, 0.25), (7, 0.0)]
    for nnz, tau in cases:
        expect = int(f32(nnz) * f32(tau))  # numpy float32 arithmetic, then truncation
        assert ora.threshold(nnz, tau) == expect
    # above 2^24 the int->float conversion rounds: 2^24+1 -> 2^24, 2^24+3 -> 2^24+4 (unreachable total)
    assert ora.threshold(2 ** 24 + 1, 1.0) == 2 ** 24
    assert ora.threshold(2 ** 24 + 3, 1.0) == 2 ** 24 + 4


# ---------------------------------------------------------------- cascaded extraction
def brute_force_selection(D, tau_c, tau_r):
    """The selection rule restated with numpy on a small dense matrix pattern."""
    f32 = np.float32
    nnz = int((D != 0).sum())
    ccnt = (D != 0).sum(axis=0)
    order = np.lexsort((np.arange(len(ccnt)), -ccnt))  # count desc, ties by ascending id
    T = int(f32(nnz) * f32(tau_c))
    k = int(np.searchsorted(np.cumsum(ccnt[order]), T, side="left")) + 1
    dense_cols = order[:k]
    rcnt = (D[:, dense_cols] != 0).sum(axis=1)
    rorder = np.lexsort((np.arange(len(rcnt)), -rcnt))
    U = int(f32(nnz) * f32(tau_r))
    kr = int(np.searchsorted(np.cumsum(rcnt[rorder]), U, side="left")) + 1
    return order, k, rorder[:kr]


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("tau", [(0.5, 0.25), (0.3, 0.3), (1.0, 0.5), (0.75, 0.0), (0.9, 0.6)])
def test_partition_selection_matches_brute_force(ora, seed, tau):
    rng = np.random.default_rng(100 + seed)
    n = 40
    D = np.where(rng.random((n, n)) < rng.uniform(0.05, 0.4), rng.uniform(-1, 1, (n, n)), 0.0)
    D[rng.integers(0, n), :] = rng.uniform(-1, 1, n)  # one heavy row, one heavy column
    D[:, rng.integers(0, n)] = rng.uniform(-1, 1, n)
    A = sp.csr_matrix(D)
    A.sort_indices()
    P = ora.partition(A.indptr, A.indices, A.data, n, *tau)
    order, k, rid = brute_force_selection(D, *tau)
    assert P.dCols == k
    assert np.array_equal(P.descColId, order)
    assert np.array_equal(P.rId, rid)
    assert np.array_equal(P.newArray, np.sort(order[k:]))
    assert np.array_equal(P.newArray_, np.setdiff1d(np.arange(n), rid))
    # A_dd is exactly D[rId][:, dense cols] with columns renumbered by rank
    Add = sp.csr_matrix((P.ddVal, P.ddColInd, P.ddRowPtr), shape=(P.dRows, P.dCols)).toarray()
    assert np.array_equal(Add, D[np.ix_(rid, order[:k])])


def rebuild_from_partition(P, n_rows, n_cols):
    """Dense matrix re-assembled from tiles + residual through the index maps."""
    M = np.zeros((n_rows, n_cols))
    K, Mf = P.fragK, P.fragM
    colOrig = np.concatenate([P.descColId[:P.dCols], P.newArray]).astype(np.int64)
    for w in range(P.chunkNum):
        for f in range(P.chunkPtr[w], P.chunkPtr[w + 1]):
            bits = int(P.fragBit[f])
            v = P.fragPtr[f]
            for b in range(Mf * K):
                if (bits >> b) & 1:
                    r, c = divmod(b, K)
                    row = P.rId[w * Mf + r]
                    col = colOrig[P.sparse_AToX_index[f * K + c]]
                    M[row, col] += P.tcVal[v]
                    v += 1
            assert v == P.fragPtr[f + 1]
    for r in range(n_rows):
        for p in range(P.cdRowPtr[r], P.cdRowPtr[r + 1]):
            M[r, colOrig[P.cdColInd[p]]] += P.cdVal[p]
    return M


@pytest.mark.parametrize("dtype", [np.float64, np.float16])
@pytest.mark.parametrize("tau", [(0.5, 0.25), (1.0, 1.0), (1.0, 0.0), (0.25, 0.25), (0.6, 0.1)])
def test_partition_conserves_every_entry(ora, dtype, tau):
    rng = np.random.default_rng(5)
    n = 70
    D = np.where(rng.random((n, n)) < 0.15, rng.integers(1, 9, (n, n)) / 8.0, 0.0)  # exact in binary16
    A = sp.csr_matrix(D)
    A.sort_indices()
    P = ora.partition(A.indptr, A.indices, A.data.astype(dtype), n, *tau)
    M = rebuild_from_partition(P, n, n)
    assert np.array_equal(M, D)
    # bookkeeping identities
    assert P.nnzCD == A.nnz - P.nnzRowD
    assert P.fragPtr[-1] == P.nnzRowD == sum(bin(int(b)).count("1") for b in P.fragBit)
    assert np.all(np.diff(P.chunkPtr) >= 0)
    for w in range(P.chunkNum):  # used prefix of each chunk's column list is strictly increasing
        lst = P.sparse_AToX_index[P.chunkPtr[w] * P.fragK:P.chunkPtr[w + 1] * P.fragK]
        used = len(np.unique(P.ddColInd[P.ddRowPtr[w * 8]:P.ddRowPtr[min(w * 8 + 8, P.dRows)]]))
        assert np.all(np.diff(lst[:used]) > 0) and np.all(lst[used:] == 0) and np.all(lst < P.dCols)
    expected_ratio = P.nnzRowD / (P.totalTcFrags * P.fragM * P.fragK)
    assert P.tc_nnz_ratio == pytest.approx(expected_ratio, rel=1e-15)


def test_partition_special_cases(ora):
    rng = np.random.default_rng(9)
    rp, ci, va, A = random_csr(rng, 64, 64, 0.12)
    n = 64
    # tau = (0,0): nothing extracted, the residual is A itself
    P = ora.partition(rp, ci, va, n, 0.0, 0.0)
    assert P.dCols == 0 and P.dRows == 0 and P.totalTcFrags == 0
    assert np.array_equal(P.cdRowPtr, rp) and np.array_equal(P.cdColInd, ci) and np.array_equal(P.cdVal, va)
    # tau = (1,1): every non-empty column and row extracted, residual empty
    P = ora.partition(rp, ci, va, n, 1.0, 1.0)
    assert P.dCols == int((np.bincount(ci, minlength=n) > 0).sum())
    assert P.dRows == int((np.diff(rp) > 0).sum())
    assert P.nnzCD == 0 and P.nnzRowD == A.nnz
    # tau_r = 0: the threshold 0 is met by the first row, so exactly one row is extracted
    P = ora.partition(rp, ci, va, n, 0.5, 0.0)
    assert P.dRows == 1
    # all columns tie -> identity order (stable sort); all rows tie likewise
    I = sp.identity(16, format="csr")
    P = ora.partition(I.indptr, I.indices, I.data, 16, 1.0, 1.0)
    assert np.array_equal(P.descColId, np.arange(16)) and np.array_equal(P.rId, np.arange(16))


def test_partition_duplicate_entries_last_one_wins_in_tiles(ora):
    # row 0 holds column 3 twice (values 5 then 7): the tile keeps 7, counted once
    rp = np.array([0, 3, 4], np.int32)
    ci = np.array([3, 1, 3, 2], np.int32)
    va = np.array([5.0, 1.0, 7.0, 2.0])
    P = ora.partition(rp, ci, va, 4, 1.0, 1.0)
    assert P.nnzRowD == 4 and P.fragPtr[-1] == 3
    M = rebuild_from_partition(P, 2, 4)
    assert M[0, 3] == 7.0 and M[0, 1] == 1.0 and M[1, 2] == 2.0


@pytest.mark.parametrize("dtype", [np.float64, np.float16])
def test_tile_product_equals_csr_product_of_extracted_block(ora, dtype):
    rng = np.random.default_rng(21)
    n = 96
    D = np.where(rng.random((n, n)) < 0.2, rng.integers(-4, 5, (n, n)), 0).astype(np.float64)
    A = sp.csr_matrix(D)
    A.sort_indices()
    P = ora.partition(A.indptr, A.indices, A.data.astype(dtype), n, 0.7, 0.4)
    x_d = rng.integers(-3, 4, P.dCols).astype(dtype)
    y_tile = ora.tcspmv(P, x_d)
    # small integers: all sums exact in either precision, so the comparison is bit-exact
    Add = sp.csr_matrix((P.ddVal.astype(np.float64), P.ddColInd, P.ddRowPtr), shape=(P.dRows, P.dCols))
    assert np.array_equal(y_tile.astype(np.float64), Add @ x_d.astype(np.float64))


@pytest.mark.parametrize("tau", [(0.5, 0.25), (1.0, 1.0), (0.8, 0.0)])
def test_hybrid_equals_plain_spmv(ora, tau):
    # the 4-block identity y = S x_s + A_ds x_d + A_dd x_d of the reference driver
    rng = np.random.default_rng(33)
    rp, ci, va, A = random_csr(rng, 150, 150, 0.08)
    x = rng.uniform(-1, 1, 150)
    P = ora.partition(rp, ci, va, 150, *tau)
    y = P.hybrid(x)
    ref = A @ x
    assert np.linalg.norm(y - ref) <= 1e-13 * np.linalg.norm(ref)


def test_eqcheck_binary16(ora):
    """ora_eqcheck_f16 (the reference's FP16 eQcheck, test/test_autotc_spmv.cpp:276-292: values
    widened to float, relative to the larger magnitude, 0/0 passes) against a numpy restatement on
    hand-picked pairs."""
    a = np.array([0.0, 1.0, 1.0, -2.0, 100.0, 1e-4, 0.5, 65504.0, 6e-8], np.float16)
    b = np.array([0.0, 1.0, 1.125, -2.25, 89.0, 1.2e-4, -0.5, 60000.0, 0.0], np.float16)
    af, bf = a.astype(np.float32), b.astype(np.float32)
    with np.errstate(invalid="ignore", divide="ignore"):
        rel = np.abs(af - bf) / np.maximum(np.abs(af), np.abs(bf))
    for tol in (1e-1, 0.12, 1e-3, 0.5, 2.5):
        bad = np.nonzero(rel > np.float32(tol))[0]  # NaN (0/0) compares false: passes
        assert ora.eqcheck(a, b, tol) == (int(bad[0]) if len(bad) else -1), tol
    assert ora.eqcheck(a, a.copy(), 1e-1) == -1
    # known answers: |1 - 1.125| / 1.125 = 1/9 is the first failure at 0.1; 11/100 passes 0.12, 0.2/1.2 does not; a sign flip is 2
    assert ora.eqcheck(a, b, 1e-1) == 2 and ora.eqcheck(a, b, 0.12) == 5 and ora.eqcheck(a, b, 0.5) == 6
    assert ora.eqcheck(a[:2], b[:2], 0.0) == -1


def test_hash_is_fnv1a_64(ora, mx):
    """ora_hash against the published FNV-1a 64-bit test vectors, chained calls against one call,
    and the library's mx_partition_hash (same function over the canonical arrays in the
    documented order)."""
    vec = {b"": 0xcbf29ce484222325, b"a": 0xaf63dc4c8601ec8c, b"b": 0xaf63df4c8601f1a5, b"foobar": 0x85944171f73967e8,
           b"chongo was here!\n": 0x46810940eff5f915}
    for s, h in vec.items():
        assert ora.hash_arrays(np.frombuffer(s, np.uint8)) == h, s
    parts = [np.frombuffer(b"foo", np.uint8), np.frombuffer(b"bar", np.uint8)]
    assert ora.hash_arrays(*parts) == vec[b"foobar"]
    A, _ = mx.gen_config(2, scale=1 / 64)
    for tau in ((0.5, 0.25), (1.0, 1.0)):
        P = mx.Partition(A, *tau)
        Q = ora.partition(A.rowPtr, A.colInd, A.val, A.cols, *tau)
        arrays = [np.array([Q.dCols], np.int32), np.array([Q.dRows], np.int32), Q.descColId[:Q.dCols], Q.newArray, Q.rId,
                  Q.newArray_, Q.chunkPtr, Q.sparse_AToX_index, Q.fragPtr, Q.fragBit, Q.tcVal, Q.cdRowPtr, Q.cdColInd, Q.cdVal]
        assert ora.hash_arrays(*arrays) == P.hash
        P.close()
