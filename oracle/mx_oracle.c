/*
 * mx_oracle.c -- CPU restatement of the reference's hybrid-SpMV path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker, never the product:
 * nothing in the shipped library links, loads or calls it.  It is used by the
 * test-suite, by the smoke check and by the benchmark's CPU-baseline leg.
 *
 * Every function restates one piece of the reference in plain, single-threaded
 * C and cites the reference lines it follows (paths are relative to the
 * reference repository root).  It deliberately keeps the reference's own
 * algorithmic route (transpose -> qsort -> split -> transpose back -> qsort ->
 * split -> per-window tiles -> row-merge) so that the product's faster,
 * differently-organised partitioner is checked against an independent
 * derivation.
 *
 * Value type: `elem` is the byte size of one matrix value, 8 (IEEE binary64)
 * or 2 (IEEE binary16, carried as uint16_t bits).  The partition only moves
 * values, so it is generic in `elem`; the arithmetic routines come in an f64
 * and an f16 flavour.  Tile shape follows include/common.h:53-70:
 * 8x4 with a 32-bit bitmap for f64, 8x8 with a 64-bit bitmap for f16.
 *
 * How each function is pinned (none of it by re-typing its own formula):
 *   ora_spmv_f64            scipy.sparse product, dense brute force, closed
 *                           forms (identity, 27-point stencil row sums)
 *   ora_f2h / ora_h2f       numpy.float16 over all 65536 bit patterns and a
 *                           sweep of floats incl. ties, subnormals, overflow
 *   ora_spmv_f16_f32acc     numpy float32 cumulative sums in CSR order
 *   ora_spmv_f16_halfacc    numpy float16 step-by-step loop on small cases
 *   ora_transpose           scipy tocsc() on duplicate-free input; stability on
 *                           duplicates by brute force; double transpose
 *   ora_partition           numpy brute-force restatement of the selection
 *                           rule on tiny matrices, conservation of the entry
 *                           multiset, tau = 1 / tau_r = 0 special cases,
 *                           (int)((float)nnz * tau) table, tile -> triple
 *                           reconstruction
 *   ora_tcspmv_*            equals ora_spmv on A_dd, bit-exact on small-integer
 *                           data
 * PARITY UNPINNED (no reference test, fixture or build can pin them here):
 *   - the within-row entry order cuSPARSE's csr2csc emits on the reference
 *     authors' machine (utilities/csr2csc.cpp:52-83); the documented behaviour
 *     (ascending, stable) is what ora_transpose implements;
 *   - qsort's order of equal counts on the authors' C library; glibc's
 *     merge-sort (stable) is what this file gets by calling qsort itself.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#include <stdio.h>

#include "mx_oracle.h"

/* ------------------------------------------------------------------------ */
/* binary16 <-> binary32 (the reference relies on CUDA's `half`, a plain IEEE
 * binary16 with round-to-nearest-even conversions; include/common.h:60-68). */

float ora_h2f(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t ex = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (ex == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: renormalise */
            int sh = 0;
            while (!(man & 0x400u)) { man <<= 1; ++sh; }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - sh + 1) << 23) | (man << 13);
        }
    } else if (ex == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((ex + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t ora_f2h(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        if (ax == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7e00u | ((ax >> 13) & 0x3ffu));
    }
    int e = (int)(ax >> 23) - 127;
    uint32_t m = ax & 0x7fffffu;
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    if (e >= -14) {
        uint32_t h = ((uint32_t)(e + 15) << 10) | (m >> 13);
        uint32_t rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h; /* may carry to inf */
        return (uint16_t)(sign | h);
    }
    if (e < -25) return sign;
    m |= 0x800000u;
    int shift = (-14 - e) + 13; /* 14..24 */
    uint32_t hm = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1u);
    uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (hm & 1u))) ++hm;
    return (uint16_t)(sign | hm);
}

/* ------------------------------------------------------------------------ */
/* spmv_serial: test/test_autotc_spmv.cpp:300-316.  One thread, row loop,
 * running sum in CSR order, result ADDED to what Y already holds. */

void ora_spmv_f64(const double *val, const int *rowPtr, const int *colInd,
                  const double *x, double *y, int rows)
{
    for (int i = 0; i < rows; ++i) {
        double t = 0.0;
        for (int p = rowPtr[i]; p < rowPtr[i + 1]; ++p)
            t = t + val[p] * x[colInd[p]];
        y[i] = y[i] + t;
    }
}

/* The synthetic FP16 workloads specify binary16 inputs with binary32
 * accumulation; the product of two binary16 numbers is exact in binary32.
 * y is delivered in binary32 (y32) and, rounded once, in binary16 (y16). */
void ora_spmv_f16_f32acc(const uint16_t *val, const int *rowPtr, const int *colInd,
                         const uint16_t *x, float *y32, uint16_t *y16, int rows)
{
    for (int i = 0; i < rows; ++i) {
        float t = 0.0f;
        for (int p = rowPtr[i]; p < rowPtr[i + 1]; ++p) {
            float prod = ora_h2f(val[p]) * ora_h2f(x[colInd[p]]);
            t = t + prod;
        }
        if (y32) y32[i] = t;
        if (y16) y16[i] = ora_f2h(t);
    }
}

/* The reference's own FP16 arithmetic (valT = half in spmv_serial,
 * test/test_autotc_spmv.cpp:303-314): every product and every partial sum is
 * rounded to binary16.  Kept to report its distance from the f32-accumulate
 * result; it is not the parity target. */
void ora_spmv_f16_halfacc(const uint16_t *val, const int *rowPtr, const int *colInd,
                          const uint16_t *x, uint16_t *y, int rows)
{
    for (int i = 0; i < rows; ++i) {
        uint16_t t = 0;
        for (int p = rowPtr[i]; p < rowPtr[i + 1]; ++p) {
            uint16_t prod = ora_f2h(ora_h2f(val[p]) * ora_h2f(x[colInd[p]]));
            t = ora_f2h(ora_h2f(t) + ora_h2f(prod));
        }
        y[i] = ora_f2h(ora_h2f(y[i]) + ora_h2f(t));
    }
}

/* eQcheck: test/test_autotc_spmv.cpp:257-293.  Element-wise relative error
 * against max(|a|,|b|); 0/0 gives NaN, which compares false and passes, as in
 * the reference.  Returns the first failing index, or -1 if all pass. */
int ora_eqcheck_f64(const double *a, const double *b, int n, double tol)
{
    for (int i = 0; i < n; ++i)
        if (fabs(a[i] - b[i]) / fmax(fabs(a[i]), fabs(b[i])) > tol) return i;
    return -1;
}

int ora_eqcheck_f16(const uint16_t *a, const uint16_t *b, int n, float tol)
{
    for (int i = 0; i < n; ++i) {
        float v1 = ora_h2f(a[i]), v2 = ora_h2f(b[i]);
        if (fabs(v1 - v2) / fmax(fabs(v1), fabs(v2)) > tol) return i;
    }
    return -1;
}

/* ------------------------------------------------------------------------ */
/* csr2csc / csc2csr: utilities/csr2csc.cpp:4-203 hand the matrix to
 * cusparseCsr2cscEx2(ALG_DEFAULT); the documented result lists every output
 * column with its source rows ascending, equal (row,col) pairs in source
 * order.  That is a counting-sort transpose.  `outer` is the number of source
 * rows, `inner` the number of source columns. */

int ora_transpose(int elem, int outer, int inner, int nnz,
                  const int *ptr, const int *ind, const void *val,
                  int **tPtr, int **tInd, void **tVal)
{
    int *cp = (int *)calloc((size_t)inner + 1, sizeof(int));
    int *ri = (int *)malloc((size_t)(nnz > 0 ? nnz : 1) * sizeof(int));
    char *tv = (char *)malloc((size_t)(nnz > 0 ? nnz : 1) * (size_t)elem);
    int *cursor = (int *)malloc(((size_t)inner + 1) * sizeof(int));
    if (!cp || !ri || !tv || !cursor) return -1;
    for (int p = 0; p < nnz; ++p) cp[ind[p] + 1]++;
    for (int c = 0; c < inner; ++c) cp[c + 1] += cp[c];
    memcpy(cursor, cp, ((size_t)inner + 1) * sizeof(int));
    const char *sv = (const char *)val;
    for (int r = 0; r < outer; ++r)
        for (int p = ptr[r]; p < ptr[r + 1]; ++p) {
            int q = cursor[ind[p]]++;
            ri[q] = r;
            memcpy(tv + (size_t)q * elem, sv + (size_t)p * elem, (size_t)elem);
        }
    free(cursor);
    *tPtr = cp;
    *tInd = ri;
    *tVal = tv;
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Cascaded extraction: test/test_autotc_spmv.cpp:1106-1427 and 1486-1492. */

typedef struct {
    int count;
    int index;
} count_index; /* CountWithIndex, test/test_autotc_spmv.cpp:10-14 */

/* compare_desc_structure, test/test_autotc_spmv.cpp:252-255: count only. */
static int cmp_count_desc(const void *a, const void *b)
{
    return ((const count_index *)b)->count - ((const count_index *)a)->count;
}

/* `int dColsNnz = nnzA * colProp;` (test/test_autotc_spmv.cpp:1131,1249):
 * int times float is evaluated in float, then truncated. */
int ora_threshold(int nnz, float frac)
{
    float t = (float)nnz * frac;
    return (int)t;
}

/* Shortest prefix of the sorted counts whose sum reaches `target`
 * (test/test_autotc_spmv.cpp:1133-1141, 1251-1259).  The reference scans
 * `rowA` entries and leaves the size at 0 when the target is out of reach
 * (undefined behaviour downstream); here the scan covers all `n` entries and
 * an unreachable target selects every entry with a non-zero count, which is
 * what a reachable target equal to the total would select. */
static int prefix_reach(const count_index *s, int n, int target, int *sum_out)
{
    int sum = 0;
    for (int i = 0; i < n; ++i) {
        sum += s[i].count;
        if (sum >= target) {
            *sum_out = sum;
            return i + 1;
        }
    }
    int k = 0;
    sum = 0;
    while (k < n && s[k].count > 0) sum += s[k++].count;
    *sum_out = sum;
    return k;
}

static void *xmalloc(size_t n)
{
    void *p = malloc(n ? n : 1);
    if (!p) {
        fprintf(stderr, "mx_oracle: out of memory\n");
        abort();
    }
    return p;
}

static void *xcalloc(size_t n, size_t sz)
{
    void *p = calloc(n ? n : 1, sz);
    if (!p) {
        fprintf(stderr, "mx_oracle: out of memory\n");
        abort();
    }
    return p;
}

static int cmp_int_asc(const void *a, const void *b)
{
    int x = *(const int *)a, y = *(const int *)b;
    return (x > y) - (x < y);
}

/* Gather the listed columns (or rows) of a compressed matrix, in list order
 * (test/test_autotc_spmv.cpp:1162-1176, 1203-1221, 1286-1300, 1328-1345). */
static void gather_lines(int elem, const int *ptr, const int *ind, const void *val,
                         const int *list, int nlist, int **oPtr, int **oInd, void **oVal)
{
    int total = 0;
    for (int i = 0; i < nlist; ++i) total += ptr[list[i] + 1] - ptr[list[i]];
    int *p = (int *)xmalloc(((size_t)nlist + 1) * sizeof(int));
    int *x = (int *)xmalloc((size_t)total * sizeof(int));
    char *v = (char *)xmalloc((size_t)total * elem);
    int w = 0;
    p[0] = 0;
    for (int i = 0; i < nlist; ++i) {
        int a = ptr[list[i]], b = ptr[list[i] + 1];
        memcpy(x + w, ind + a, (size_t)(b - a) * sizeof(int));
        memcpy(v + (size_t)w * elem, (const char *)val + (size_t)a * elem, (size_t)(b - a) * elem);
        w += b - a;
        p[i + 1] = w;
    }
    *oPtr = p;
    *oInd = x;
    *oVal = v;
}

/* Indices of [0,n) not in `sel`, ascending (the byte-bitmap scans at
 * test/test_autotc_spmv.cpp:1178-1201 and 1302-1326). */
static int *complement(const int *sel, int nsel, int n)
{
    char *mark = (char *)xcalloc((size_t)n, 1);
    for (int i = 0; i < nsel; ++i) mark[sel[i]] = 1;
    int *out = (int *)xmalloc((size_t)(n - nsel) * sizeof(int));
    int w = 0;
    for (int i = 0; i < n; ++i)
        if (!mark[i]) out[w++] = i;
    free(mark);
    return out;
}

void ora_partition_free(ora_partition *P)
{
    if (!P) return;
    free(P->descColId);
    free(P->newArray);
    free(P->rId);
    free(P->newArray_);
    free(P->ddRowPtr);
    free(P->ddColInd);
    free(P->ddVal);
    free(P->chunkPtr);
    free(P->sparse_AToX_index);
    free(P->fragPtr);
    free(P->fragBit);
    free(P->tcVal);
    free(P->cdRowPtr);
    free(P->cdColInd);
    free(P->cdVal);
    free(P);
}

ora_partition *ora_partition_create(int elem, int rows, int cols, int nnz,
                                    const int *rowPtr, const int *colInd, const void *val,
                                    float colProp, float rowProp)
{
    ora_partition *P = (ora_partition *)xcalloc(1, sizeof(*P));
    P->elem = elem;
    P->rows = rows;
    P->cols = cols;
    P->nnz = nnz;
    P->fragM = 8;
    P->fragK = (elem == 8) ? 4 : 8; /* include/common.h:56-67 */
    const int fragM = P->fragM, fragK = P->fragK;

    /* tau = (0,0): no extraction, the residual kernel runs on A itself
     * (test/test_autotc_spmv.cpp:1106,1638-1658). */
    if (rowProp == 0.0f && colProp == 0.0f) {
        P->sCols = cols;
        P->sRows = rows;
        P->nnzColS = nnz;
        P->descColId = (int *)xmalloc(sizeof(int));
        P->newArray = (int *)xmalloc((size_t)cols * sizeof(int));
        for (int i = 0; i < cols; ++i) P->newArray[i] = i;
        P->rId = (int *)xmalloc(sizeof(int));
        P->newArray_ = (int *)xmalloc((size_t)rows * sizeof(int));
        for (int i = 0; i < rows; ++i) P->newArray_[i] = i;
        P->ddRowPtr = (int *)xcalloc(1, sizeof(int));
        P->ddColInd = (int *)xmalloc(sizeof(int));
        P->ddVal = xmalloc(1);
        P->chunkPtr = (int *)xcalloc(1, sizeof(int));
        P->sparse_AToX_index = (int *)xmalloc(sizeof(int));
        P->fragPtr = (int *)xcalloc(1, sizeof(int));
        P->fragBit = xmalloc(8);
        P->tcVal = xmalloc(1);
        P->nnzCD = nnz;
        P->cdRowPtr = (int *)xmalloc(((size_t)rows + 1) * sizeof(int));
        memcpy(P->cdRowPtr, rowPtr, ((size_t)rows + 1) * sizeof(int));
        P->cdColInd = (int *)xmalloc((size_t)nnz * sizeof(int));
        memcpy(P->cdColInd, colInd, (size_t)nnz * sizeof(int));
        P->cdVal = xmalloc((size_t)nnz * elem);
        memcpy(P->cdVal, val, (size_t)nnz * elem);
        return P;
    }

    /* 1.1 column pass: :1119-1141 */
    int *cscPtr, *cscInd;
    void *cscVal;
    ora_transpose(elem, rows, cols, nnz, rowPtr, colInd, val, &cscPtr, &cscInd, &cscVal);

    count_index *dc = (count_index *)xmalloc((size_t)cols * sizeof(count_index));
    for (int i = 0; i < cols; ++i) {
        dc[i].count = cscPtr[i + 1] - cscPtr[i];
        dc[i].index = i;
    }
    qsort(dc, (size_t)cols, sizeof(count_index), cmp_count_desc);
    int dColsNnz = ora_threshold(nnz, colProp);
    int nnzColD = 0;
    int dCols = prefix_reach(dc, cols, dColsNnz, &nnzColD);
    int sCols = cols - dCols;
    int nnzColS = nnz - nnzColD;
    P->dCols = dCols;
    P->sCols = sCols;
    P->nnzColD = nnzColD;
    P->nnzColS = nnzColS;
    P->cols_ratio = (float)dCols / (float)cols; /* :1142 */

    P->descColId = (int *)xmalloc((size_t)cols * sizeof(int));
    for (int i = 0; i < cols; ++i) P->descColId[i] = dc[i].index;
    free(dc);
    P->newArray = complement(P->descColId, dCols, cols); /* :1178-1201 */

    int *dcscPtr, *dcscInd, *scscPtr, *scscInd;
    void *dcscVal, *scscVal;
    gather_lines(elem, cscPtr, cscInd, cscVal, P->descColId, dCols, &dcscPtr, &dcscInd, &dcscVal);
    gather_lines(elem, cscPtr, cscInd, cscVal, P->newArray, sCols, &scscPtr, &scscInd, &scscVal);
    free(cscPtr);
    free(cscInd);
    free(cscVal);

    /* 1.2 back to row-major: :1234-1238 */
    int *dcsrPtr, *dcsrInd, *scsrPtr, *scsrInd;
    void *dcsrVal, *scsrVal;
    ora_transpose(elem, dCols, rows, nnzColD, dcscPtr, dcscInd, dcscVal, &dcsrPtr, &dcsrInd, &dcsrVal);
    ora_transpose(elem, sCols, rows, nnzColS, scscPtr, scscInd, scscVal, &scsrPtr, &scsrInd, &scsrVal);
    free(dcscPtr);
    free(dcscInd);
    free(dcscVal);
    free(scscPtr);
    free(scscInd);
    free(scscVal);

    /* row pass on the dense-column block: :1240-1267 */
    count_index *dr = (count_index *)xmalloc((size_t)rows * sizeof(count_index));
    for (int i = 0; i < rows; ++i) {
        dr[i].count = dcsrPtr[i + 1] - dcsrPtr[i];
        dr[i].index = i;
    }
    qsort(dr, (size_t)rows, sizeof(count_index), cmp_count_desc);
    int dRowsNnz = ora_threshold(nnz, rowProp); /* fraction of the TOTAL nnz */
    int nnzRowD = 0;
    int dRows = prefix_reach(dr, rows, dRowsNnz, &nnzRowD);
    int sRows = rows - dRows;
    int nnzRowS = nnzColD - nnzRowD;
    P->dRows = dRows;
    P->sRows = sRows;
    P->nnzRowD = nnzRowD;
    P->nnzRowS = nnzRowS;
    P->rId = (int *)xmalloc((size_t)dRows * sizeof(int));
    for (int i = 0; i < dRows; ++i) P->rId[i] = dr[i].index;
    free(dr);
    P->newArray_ = complement(P->rId, dRows, rows); /* :1302-1326 */

    int *dsPtr, *dsInd;
    void *dsVal;
    gather_lines(elem, dcsrPtr, dcsrInd, dcsrVal, P->rId, dRows, &P->ddRowPtr, &P->ddColInd, &P->ddVal);
    gather_lines(elem, dcsrPtr, dcsrInd, dcsrVal, P->newArray_, sRows, &dsPtr, &dsInd, &dsVal);
    free(dcsrPtr);
    free(dcsrInd);
    free(dcsrVal);

    /* 2. tile format over A_dd.
     * ecrPreprocess_opt1 (:502-585): per window of fragM rows, the sorted
     * set of distinct columns; every entry gets its rank in that set. */
    const int *ddPtr = P->ddRowPtr, *ddInd = P->ddColInd;
    int chunkNum = (dRows + fragM - 1) / fragM; /* :1354 */
    P->chunkNum = chunkNum;
    int *ecrId = (int *)xmalloc((size_t)nnzRowD * sizeof(int));
    int **use_x = (int **)xcalloc((size_t)chunkNum + 1, sizeof(int *));
    int *nec = (int *)xcalloc((size_t)chunkNum + 1, sizeof(int));
    P->chunkPtr = (int *)xcalloc((size_t)chunkNum + 1, sizeof(int));
    for (int w = 0; w < chunkNum; ++w) {
        int r0 = w * fragM, r1 = r0 + fragM < dRows ? r0 + fragM : dRows;
        int a = ddPtr[r0], b = ddPtr[r1], n = b - a;
        int blocks = 0;
        if (n > 0) {
            int *win = (int *)xmalloc((size_t)n * sizeof(int));
            memcpy(win, ddInd + a, (size_t)n * sizeof(int));
            qsort(win, (size_t)n, sizeof(int), cmp_int_asc);
            int u = 0;
            for (int i = 0; i < n; ++i)
                if (i == 0 || win[i] != win[i - 1]) win[u++] = win[i];
            use_x[w] = win;
            nec[w] = u;
            blocks = (u + fragK - 1) / fragK;
            for (int e = a; e < b; ++e) { /* rank by binary search */
                int lo = 0, hi = u - 1, key = ddInd[e];
                while (lo < hi) {
                    int mid = (lo + hi) >> 1;
                    if (win[mid] < key) lo = mid + 1; else hi = mid;
                }
                ecrId[e] = lo;
            }
        }
        P->chunkPtr[w + 1] = P->chunkPtr[w] + blocks; /* :1369-1374 */
    }
    int totalTcFrags = P->chunkPtr[chunkNum];
    P->totalTcFrags = totalTcFrags;
    P->tc_nnz_ratio = (double)nnzRowD / ((double)totalTcFrags * fragM * fragK); /* :1376 */

    /* sparse_AToX_index (:1380-1404): the window's column list, zero padded. */
    P->sparse_AToX_index = (int *)xcalloc((size_t)totalTcFrags * fragK, sizeof(int));
    for (int w = 0; w < chunkNum; ++w)
        if (nec[w] > 0)
            memcpy(P->sparse_AToX_index + (size_t)P->chunkPtr[w] * fragK, use_x[w],
                   (size_t)nec[w] * sizeof(int));

    /* generateFormat_opt / _fp16 (:718-978): per fragment a bitmap with bit
     * (localRow*fragK + localCol); values listed in ascending bit order; a
     * repeated (row,col) keeps the value met last and is counted once. */
    size_t slots = (size_t)fragM * fragK;
    P->fragBit = xcalloc((size_t)totalTcFrags + 1, 8);
    uint64_t *bits = (uint64_t *)P->fragBit;
    P->fragPtr = (int *)xcalloc((size_t)totalTcFrags + 1, sizeof(int));
    P->tcVal = xmalloc((size_t)nnzRowD * elem);
    char *tcv = (char *)P->tcVal;
    int tcCount = 0;
    for (int w = 0; w < chunkNum; ++w) {
        int nf = P->chunkPtr[w + 1] - P->chunkPtr[w];
        if (nf == 0) continue;
        int r0 = w * fragM, r1 = r0 + fragM < dRows ? r0 + fragM : dRows;
        char *grid = (char *)xcalloc((size_t)nf * slots, (size_t)elem);
        char *has = (char *)xcalloc((size_t)nf * slots, 1);
        for (int r = r0; r < r1; ++r)
            for (int e = ddPtr[r]; e < ddPtr[r + 1]; ++e) {
                int fr = ecrId[e] / fragK, c = ecrId[e] % fragK;
                int bit = (r - r0) * fragK + c;
                size_t pos = (size_t)fr * slots + (size_t)bit;
                memcpy(grid + pos * elem, (const char *)P->ddVal + (size_t)e * elem, (size_t)elem);
                has[pos] = 1;
                bits[P->chunkPtr[w] + fr] |= (uint64_t)1 << bit;
            }
        for (int fr = 0; fr < nf; ++fr) {
            int f = P->chunkPtr[w] + fr;
            int cnt = 0;
            for (size_t s = 0; s < slots; ++s)
                if (has[(size_t)fr * slots + s]) {
                    memcpy(tcv + (size_t)tcCount * elem, grid + ((size_t)fr * slots + s) * elem, (size_t)elem);
                    ++tcCount;
                    ++cnt;
                }
            P->fragPtr[f + 1] = cnt;
        }
        free(grid);
        free(has);
    }
    for (int f = 0; f < totalTcFrags; ++f) P->fragPtr[f + 1] += P->fragPtr[f];
    P->tcValCount = tcCount;
    if (elem == 8) { /* FP64 bitmaps are 32 bits wide: narrow in place */
        uint32_t *b32 = (uint32_t *)P->fragBit;
        for (int f = 0; f < totalTcFrags; ++f) b32[f] = (uint32_t)bits[f];
    }
    for (int w = 0; w < chunkNum; ++w) free(use_x[w]);
    free(use_x);
    free(nec);
    free(ecrId);

    /* residual: merge2CSR_opt (:129-250).  Row i = sparse-column entries of
     * row i (column + dCols) followed by the dense-column entries of row i if
     * that row was not extracted. */
    int nnzCD = nnzColS + nnzRowS;
    P->nnzCD = nnzCD;
    P->cdRowPtr = (int *)xcalloc((size_t)rows + 1, sizeof(int));
    for (int i = 0; i < rows; ++i) P->cdRowPtr[i + 1] = scsrPtr[i + 1] - scsrPtr[i];
    for (int k = 0; k < sRows; ++k) P->cdRowPtr[P->newArray_[k] + 1] += dsPtr[k + 1] - dsPtr[k];
    for (int i = 0; i < rows; ++i) P->cdRowPtr[i + 1] += P->cdRowPtr[i];
    P->cdColInd = (int *)xmalloc((size_t)nnzCD * sizeof(int));
    P->cdVal = xmalloc((size_t)nnzCD * elem);
    int *cur = (int *)xmalloc((size_t)rows * sizeof(int));
    memcpy(cur, P->cdRowPtr, (size_t)rows * sizeof(int));
    for (int i = 0; i < rows; ++i)
        for (int k = scsrPtr[i]; k < scsrPtr[i + 1]; ++k) {
            int q = cur[i]++;
            P->cdColInd[q] = dCols + scsrInd[k];
            memcpy((char *)P->cdVal + (size_t)q * elem, (const char *)scsrVal + (size_t)k * elem, (size_t)elem);
        }
    for (int k = 0; k < sRows; ++k) {
        int i = P->newArray_[k];
        for (int e = dsPtr[k]; e < dsPtr[k + 1]; ++e) {
            int q = cur[i]++;
            P->cdColInd[q] = dsInd[e];
            memcpy((char *)P->cdVal + (size_t)q * elem, (const char *)dsVal + (size_t)e * elem, (size_t)elem);
        }
    }
    free(cur);
    free(scsrPtr);
    free(scsrInd);
    free(scsrVal);
    free(dsPtr);
    free(dsInd);
    free(dsVal);
    return P;
}

/* ------------------------------------------------------------------------ */
/* tcspmv_serial: test/test_autotc_spmv.cpp:981-1048 (FP64) and
 * test/test_tcspmv.cpp:1051-1118 (FP16).  Walks the fragments of each row
 * chunk; bit (m*fragK + k) of the bitmap consumes the next packed value and
 * multiplies it by x_d[sparse_AToX_index[f*fragK + k]]. */

void ora_tcspmv_f64(const double *x_d, double *y_d, const int *chunkPtr, const int *fragPtr,
                    const uint32_t *fragBit, const double *tcVal, const int *atox, int dRows)
{
    const int fragM = 8, fragK = 4;
    int chunkNum = (dRows + fragM - 1) / fragM;
    for (int i = 0; i < dRows; ++i) y_d[i] = 0.0;
    for (int w = 0; w < chunkNum; ++w)
        for (int f = chunkPtr[w]; f < chunkPtr[w + 1]; ++f) {
            const double *v = tcVal + fragPtr[f];
            int used = 0;
            for (int m = 0; m < fragM; ++m) {
                int row = w * fragM + m;
                if (row >= dRows) continue;
                for (int k = 0; k < fragK; ++k)
                    if ((fragBit[f] >> (m * fragK + k)) & 1u)
                        y_d[row] = y_d[row] + v[used++] * x_d[atox[f * fragK + k]];
            }
        }
}

/* FP16 tiles with binary32 accumulation per row (the synthetic workloads'
 * arithmetic); y returned in binary32. */
void ora_tcspmv_f16(const uint16_t *x_d, float *y_d, const int *chunkPtr, const int *fragPtr,
                    const uint64_t *fragBit, const uint16_t *tcVal, const int *atox, int dRows)
{
    const int fragM = 8, fragK = 8;
    int chunkNum = (dRows + fragM - 1) / fragM;
    for (int i = 0; i < dRows; ++i) y_d[i] = 0.0f;
    for (int w = 0; w < chunkNum; ++w)
        for (int f = chunkPtr[w]; f < chunkPtr[w + 1]; ++f) {
            const uint16_t *v = tcVal + fragPtr[f];
            int used = 0;
            for (int m = 0; m < fragM; ++m) {
                int row = w * fragM + m;
                if (row >= dRows) continue;
                for (int k = 0; k < fragK; ++k)
                    if ((fragBit[f] >> (m * fragK + k)) & 1ull) {
                        float prod = ora_h2f(v[used++]) * ora_h2f(x_d[atox[f * fragK + k]]);
                        y_d[row] = y_d[row] + prod;
                    }
            }
        }
}

/* Whole hybrid product on the CPU from a partition, as the driver assembles
 * it (test/test_autotc_spmv.cpp:1454-1463, 1531-1559): x_d/x_s from the column
 * maps, tile result scattered through rId, residual accumulated on top. */
void ora_hybrid_f64(const ora_partition *P, const double *x, double *y)
{
    int rows = P->rows, cols = P->cols, dCols = P->dCols;
    double *xcd = (double *)xmalloc((size_t)cols * sizeof(double));
    for (int j = 0; j < dCols; ++j) xcd[j] = x[P->descColId[j]];
    for (int j = 0; j < P->sCols; ++j) xcd[dCols + j] = x[P->newArray[j]];
    for (int i = 0; i < rows; ++i) y[i] = 0.0;
    if (P->dRows > 0) {
        double *hot = (double *)xmalloc((size_t)P->dRows * sizeof(double));
        ora_tcspmv_f64(xcd, hot, P->chunkPtr, P->fragPtr, (const uint32_t *)P->fragBit,
                       (const double *)P->tcVal, P->sparse_AToX_index, P->dRows);
        for (int i = 0; i < P->dRows; ++i) y[P->rId[i]] = hot[i];
        free(hot);
    }
    ora_spmv_f64((const double *)P->cdVal, P->cdRowPtr, P->cdColInd, xcd, y, rows);
    free(xcd);
}

void ora_hybrid_f16(const ora_partition *P, const uint16_t *x, float *y)
{
    int rows = P->rows, cols = P->cols, dCols = P->dCols;
    uint16_t *xcd = (uint16_t *)xmalloc((size_t)cols * sizeof(uint16_t));
    for (int j = 0; j < dCols; ++j) xcd[j] = x[P->descColId[j]];
    for (int j = 0; j < P->sCols; ++j) xcd[dCols + j] = x[P->newArray[j]];
    float *res = (float *)xmalloc((size_t)rows * sizeof(float));
    ora_spmv_f16_f32acc((const uint16_t *)P->cdVal, P->cdRowPtr, P->cdColInd, xcd, res, NULL, rows);
    for (int i = 0; i < rows; ++i) y[i] = 0.0f;
    if (P->dRows > 0) {
        float *hot = (float *)xmalloc((size_t)P->dRows * sizeof(float));
        ora_tcspmv_f16(xcd, hot, P->chunkPtr, P->fragPtr, (const uint64_t *)P->fragBit,
                       (const uint16_t *)P->tcVal, P->sparse_AToX_index, P->dRows);
        for (int i = 0; i < P->dRows; ++i) y[P->rId[i]] = hot[i];
        free(hot);
    }
    for (int i = 0; i < rows; ++i) y[i] += res[i];
    free(res);
    free(xcd);
}

/* FNV-1a over a byte range: used to compare large canonical arrays cheaply. */
uint64_t ora_hash(const void *p, size_t n, uint64_t h)
{
    const unsigned char *b = (const unsigned char *)p;
    if (h == 0) h = 14695981039346656037ull;
    for (size_t i = 0; i < n; ++i) {
        h ^= b[i];
        h *= 1099511628211ull;
    }
    return h;
}

void ora_free(void *p) { free(p); }
