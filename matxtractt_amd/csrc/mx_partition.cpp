// Host side of the hybrid SpMV: the cascaded compute-density extraction.
//
// Produces exactly the arrays the reference driver derives inline in its main()
// (test/test_autotc_spmv.cpp:1106-1427, 1486-1492) but by a different route: where the
// reference transposes the matrix three times through cuSPARSE and sorts with qsort, this
// builds every output directly from the row-major input:
//   * counts are histogrammed, and "sort by count descending, ties by ascending id"
//     (qsort with compare_desc_structure, :252-255, :1130, :1248) is a counting sort;
//   * a row of the dense-column block D, of A_dd, of A_ds or of the sparse-column block S
//     is the row's own entries filtered by column class and stably sorted by their new
//     column id -- which is what csr2csc -> gather columns -> csc2csr (:1119-1238) yields;
//   * tiles are built per 8-row chunk from those sorted rows (:502-585, :718-978).
// Rows are independent, so steps run under OpenMP.
#include <algorithm>
#include <mutex>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <utility>

#include "mx_internal.h"

namespace {

using mx::set_error;

// Order of [0,n) by cnt descending, ties by ascending index.
void order_by_count_desc(const std::vector<int> &cnt, std::vector<int> &order)
{
    const int n = (int)cnt.size();
    order.resize(n);
    if (n == 0) return;
    int maxc = *std::max_element(cnt.begin(), cnt.end());
    std::vector<int> start((size_t)maxc + 2, 0);
    for (int i = 0; i < n; ++i) start[cnt[i]]++;
    // start[c] := number of items with count > c
    int acc = 0;
    for (int c = maxc; c >= 0; --c) {
        int h = start[c];
        start[c] = acc;
        acc += h;
    }
    for (int i = 0; i < n; ++i) order[start[cnt[i]]++] = i;
}

using mx::threshold;

// Shortest prefix of `order` whose counts sum to >= target (:1133-1141, :1251-1259).  An
// unreachable target (possible only through float rounding of nnz) selects every line with
// a non-zero count, the same set a reachable target equal to the total selects.
int prefix_reach(const std::vector<int> &cnt, const std::vector<int> &order, int target, int *sum_out)
{
    const int n = (int)order.size();
    long long sum = 0;
    for (int i = 0; i < n; ++i) {
        sum += cnt[order[i]];
        if (sum >= target) {
            *sum_out = (int)sum;
            return i + 1;
        }
    }
    int k = 0;
    sum = 0;
    while (k < n && cnt[order[k]] > 0) sum += cnt[order[k++]];
    *sum_out = (int)sum;
    return k;
}

template <typename V>
struct Entry {
    int key;
    V val;
};

template <typename V>
void sort_entries(std::vector<Entry<V>> &v)
{
    bool sorted = true;
    for (size_t i = 1; i < v.size(); ++i)
        if (v[i].key < v[i - 1].key) {
            sorted = false;
            break;
        }
    if (!sorted)
        std::stable_sort(v.begin(), v.end(), [](const Entry<V> &a, const Entry<V> &b) { return a.key < b.key; });
}

template <typename V>
int build(const mx_csr *A, float tau_c, float tau_r, mx_partition *P)
{
    const int rows = A->rows, cols = A->cols, nnz = A->nnz;
    const int *rp = A->rowPtr, *ci = A->colInd;
    const V *av = (const V *)A->val;
    const int fragM = P->fragM, fragK = P->fragK;

    if (tau_c == 0.0f && tau_r == 0.0f) {  // no extraction (:1106, :1638-1658)
        P->extracted = false;
        P->sCols = cols;
        P->sRows = rows;
        P->nnzColS = nnz;
        P->newArray.resize(cols);
        std::iota(P->newArray.begin(), P->newArray.end(), 0);
        P->newArray_.resize(rows);
        std::iota(P->newArray_.begin(), P->newArray_.end(), 0);
        P->ddRowPtr.assign(1, 0);
        P->chunkPtr.assign(1, 0);
        P->fragPtr.assign(1, 0);
        P->nnzCD = nnz;
        P->cdRowPtr.assign(rp, rp + rows + 1);
        P->cdColInd.assign(ci, ci + nnz);
        P->cdVal.resize(nnz, sizeof(V));
        if (nnz) std::memcpy(P->cdVal.data(), av, (size_t)nnz * sizeof(V));
        return MX_OK;
    }
    P->extracted = true;

    // ---- column pass (:1122-1141)
    std::vector<int> ccnt(cols, 0);
    for (int p = 0; p < nnz; ++p) ccnt[ci[p]]++;
    order_by_count_desc(ccnt, P->descColId);
    int nnzColD = 0;
    const int dCols = prefix_reach(ccnt, P->descColId, threshold(nnz, tau_c), &nnzColD);
    const int sCols = cols - dCols;
    P->dCols = dCols;
    P->sCols = sCols;
    P->nnzColD = nnzColD;
    P->nnzColS = nnz - nnzColD;
    P->cols_ratio = (float)dCols / (float)cols;

    // new column id: rank for an extracted column, dCols + position in newArray otherwise --
    // which is also the column space of the residual A_CD (:129-250).
    std::vector<int> newCol(cols, -1);
    for (int i = 0; i < dCols; ++i) newCol[P->descColId[i]] = i;
    P->newArray.resize(sCols);
    for (int c = 0, s = 0; c < cols; ++c)
        if (newCol[c] < 0) {
            P->newArray[s] = c;
            newCol[c] = dCols + s;
            ++s;
        }

    // ---- row pass on the dense-column block (:1240-1267)
    std::vector<int> rcnt(rows, 0);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        int c = 0;
        for (int p = rp[r]; p < rp[r + 1]; ++p) c += newCol[ci[p]] < dCols;
        rcnt[r] = c;
    }
    std::vector<int> descRowId;
    order_by_count_desc(rcnt, descRowId);
    int nnzRowD = 0;
    const int dRows = prefix_reach(rcnt, descRowId, threshold(nnz, tau_r), &nnzRowD);
    const int sRows = rows - dRows;
    P->dRows = dRows;
    P->sRows = sRows;
    P->nnzRowD = nnzRowD;
    P->nnzRowS = nnzColD - nnzRowD;
    P->rId.assign(descRowId.begin(), descRowId.begin() + dRows);
    std::vector<int> rowRank(rows, -1);
    for (int i = 0; i < dRows; ++i) rowRank[P->rId[i]] = i;
    P->newArray_.resize(sRows);
    for (int r = 0, s = 0; r < rows; ++r)
        if (rowRank[r] < 0) P->newArray_[s++] = r;

    // ---- A_dd (:1286-1300) and residual A_CD (:129-250) row by row
    P->ddRowPtr.assign((size_t)dRows + 1, 0);
    for (int i = 0; i < dRows; ++i) P->ddRowPtr[i + 1] = P->ddRowPtr[i] + rcnt[P->rId[i]];
    P->ddColInd.resize(nnzRowD);
    P->ddVal.resize(nnzRowD, sizeof(V));
    V *ddv = (V *)P->ddVal.data();

    P->cdRowPtr.assign((size_t)rows + 1, 0);
    for (int r = 0; r < rows; ++r) {
        int len = rp[r + 1] - rp[r];
        P->cdRowPtr[r + 1] = P->cdRowPtr[r] + (len - rcnt[r]) + (rowRank[r] < 0 ? rcnt[r] : 0);
    }
    const int nnzCD = P->cdRowPtr[rows];
    P->nnzCD = nnzCD;
    P->cdColInd.resize(nnzCD);
    P->cdVal.resize(nnzCD, sizeof(V));
    V *cdv = (V *)P->cdVal.data();

#pragma omp parallel
    {
        std::vector<Entry<V>> dense, sparse;
#pragma omp for schedule(dynamic, 256)
        for (int r = 0; r < rows; ++r) {
            dense.clear();
            sparse.clear();
            for (int p = rp[r]; p < rp[r + 1]; ++p) {
                int nc = newCol[ci[p]];
                (nc < dCols ? dense : sparse).push_back({nc, av[p]});
            }
            sort_entries(dense);
            sort_entries(sparse);
            int q = P->cdRowPtr[r];
            for (const auto &e : sparse) {  // S row, columns offset by dCols (already in nc)
                P->cdColInd[q] = e.key;
                cdv[q] = e.val;
                ++q;
            }
            if (rowRank[r] < 0) {  // A_ds row appended
                for (const auto &e : dense) {
                    P->cdColInd[q] = e.key;
                    cdv[q] = e.val;
                    ++q;
                }
            } else {
                int d = P->ddRowPtr[rowRank[r]];
                for (const auto &e : dense) {
                    P->ddColInd[d] = e.key;
                    ddv[d] = e.val;
                    ++d;
                }
            }
        }
    }

    // ---- tile format over A_dd
    const int chunkNum = (dRows + fragM - 1) / fragM;  // :1354
    P->chunkNum = chunkNum;
    const int *ddp = P->ddRowPtr.data();
    const int *ddc = P->ddColInd.data();
    std::vector<int> ecr(nnzRowD);     // rank of each entry's column inside its chunk (:502-585)
    std::vector<int> uniq(nnzRowD);    // per chunk, its sorted distinct columns, stored at ddp[8w]
    std::vector<int> ucount(chunkNum, 0);
    P->chunkPtr.assign((size_t)chunkNum + 1, 0);
#pragma omp parallel for schedule(dynamic, 64)
    for (int w = 0; w < chunkNum; ++w) {
        int r0 = w * fragM, r1 = std::min(r0 + fragM, dRows);
        int a = ddp[r0], b = ddp[r1];
        if (b <= a) continue;
        int *u = uniq.data() + a;
        std::copy(ddc + a, ddc + b, u);
        std::sort(u, u + (b - a));
        int n = (int)(std::unique(u, u + (b - a)) - u);
        ucount[w] = n;
        for (int e = a; e < b; ++e) ecr[e] = (int)(std::lower_bound(u, u + n, ddc[e]) - u);
    }
    for (int w = 0; w < chunkNum; ++w)
        P->chunkPtr[w + 1] = P->chunkPtr[w] + (ucount[w] + fragK - 1) / fragK;  // :1369-1374
    const int totalTcFrags = P->chunkPtr[chunkNum];
    P->totalTcFrags = totalTcFrags;
    P->tc_nnz_ratio = (double)nnzRowD / ((double)totalTcFrags * fragM * fragK);  // :1376

    P->sparse_AToX_index.assign((size_t)totalTcFrags * fragK, 0);  // :1380-1404
    std::vector<uint64_t> bits((size_t)totalTcFrags, 0);
    P->fragPtr.assign((size_t)totalTcFrags + 1, 0);
#pragma omp parallel for schedule(dynamic, 64)
    for (int w = 0; w < chunkNum; ++w) {
        int r0 = w * fragM, r1 = std::min(r0 + fragM, dRows);
        int f0 = P->chunkPtr[w];
        std::copy(uniq.data() + ddp[r0], uniq.data() + ddp[r0] + ucount[w],
                  P->sparse_AToX_index.data() + (size_t)f0 * fragK);
        for (int r = r0; r < r1; ++r)
            for (int e = ddp[r]; e < ddp[r + 1]; ++e)
                bits[f0 + ecr[e] / fragK] |= (uint64_t)1 << ((r - r0) * fragK + ecr[e] % fragK);
        for (int f = f0; f < P->chunkPtr[w + 1]; ++f) P->fragPtr[f + 1] = __builtin_popcountll(bits[f]);
    }
    for (int f = 0; f < totalTcFrags; ++f) P->fragPtr[f + 1] += P->fragPtr[f];
    const int tcValCount = P->fragPtr[totalTcFrags];
    P->tcValCount = tcValCount;
    P->tcVal.resize(tcValCount, sizeof(V));
    V *tcv = (V *)P->tcVal.data();
    // Values per fragment in ascending bit order (:718-847).  Walking a chunk row by row and
    // each sorted row left to right meets the bits of any one fragment in ascending order; a
    // repeated (row, column) sits next to its twin and replaces it (last one wins, :803-807).
#pragma omp parallel
    {
        std::vector<int> cursor;
#pragma omp for schedule(dynamic, 64)
        for (int w = 0; w < chunkNum; ++w) {
            int r0 = w * fragM, r1 = std::min(r0 + fragM, dRows);
            int f0 = P->chunkPtr[w], nf = P->chunkPtr[w + 1] - f0;
            if (nf == 0) continue;
            cursor.assign(P->fragPtr.begin() + f0, P->fragPtr.begin() + f0 + nf);
            for (int r = r0; r < r1; ++r)
                for (int e = ddp[r]; e < ddp[r + 1]; ++e) {
                    int fr = ecr[e] / fragK;
                    if (e > ddp[r] && ecr[e] == ecr[e - 1])
                        tcv[cursor[fr] - 1] = ddv[e];
                    else
                        tcv[cursor[fr]++] = ddv[e];
                }
        }
    }
    if (P->dtype == MX_F64) {
        P->fragBit32.resize(totalTcFrags);
        for (int f = 0; f < totalTcFrags; ++f) P->fragBit32[f] = (uint32_t)bits[f];
    } else {
        P->fragBit64.swap(bits);
    }
    return MX_OK;
}

uint64_t fnv(const void *p, size_t n, uint64_t h)
{
    const unsigned char *b = (const unsigned char *)p;
    for (size_t i = 0; i < n; ++i) {
        h ^= b[i];
        h *= 1099511628211ull;
    }
    return h;
}

}  // namespace

// The argument checks of mx_partition_create, shared with the device route.
int mx::check_partition_args(const mx_csr *A, float tau_c, float tau_r, mx_partition **out)
{
    if (!A || !out) {
        set_error("mx_partition_create: null argument");
        return MX_ERR_ARG;
    }
    *out = nullptr;
    if (A->rows < 0 || A->cols < 0 || A->nnz < 0 || !A->rowPtr || (A->nnz > 0 && (!A->colInd || !A->val))) {
        set_error("mx_partition_create: bad matrix description");
        return MX_ERR_ARG;
    }
    if (A->dtype != MX_F64 && A->dtype != MX_F16) {
        set_error("mx_partition_create: unknown dtype");
        return MX_ERR_ARG;
    }
    if (!(tau_c >= 0.0f && tau_c <= 1.0f && tau_r >= 0.0f && tau_r <= 1.0f)) {
        set_error("mx_partition_create: tau_c and tau_r must lie in [0,1]");
        return MX_ERR_ARG;
    }
    if (tau_c < tau_r) {  // test/test_autotc_spmv.cpp:1064-1069
        set_error("mx_partition_create: col_frac must be greater than hot_frac");
        return MX_ERR_ARG;
    }
    if (A->rowPtr[0] != 0 || A->rowPtr[A->rows] != A->nnz) {
        set_error("mx_partition_create: rowPtr does not span [0, nnz]");
        return MX_ERR_ARG;
    }
    for (int r = 0; r < A->rows; ++r)
        if (A->rowPtr[r + 1] < A->rowPtr[r]) {
            set_error("mx_partition_create: rowPtr not monotone");
            return MX_ERR_ARG;
        }
    for (int p = 0; p < A->nnz; ++p)
        if ((unsigned)A->colInd[p] >= (unsigned)A->cols) {
            set_error("mx_partition_create: column index out of range");
            return MX_ERR_ARG;
        }
    return MX_OK;
}

extern "C" int mx_partition_create(const mx_csr *A, float tau_c, float tau_r, mx_partition **out)
{
    const int ok = mx::check_partition_args(A, tau_c, tau_r, out);
    if (ok != MX_OK) return ok;
    mx_partition *P = new (std::nothrow) mx_partition();
    if (!P) {
        set_error("mx_partition_create: out of memory");
        return MX_ERR_ALLOC;
    }
    P->dtype = A->dtype;
    P->rows = A->rows;
    P->cols = A->cols;
    P->nnz = A->nnz;
    P->fragM = mx::kFragM;
    P->fragK = mx::frag_k(A->dtype);
    P->tau_c = tau_c;
    P->tau_r = tau_r;
    int rc;
    try {
        rc = A->dtype == MX_F64 ? build<double>(A, tau_c, tau_r, P) : build<uint16_t>(A, tau_c, tau_r, P);
    } catch (const std::bad_alloc &) {
        set_error("mx_partition_create: out of memory");
        rc = MX_ERR_ALLOC;
    }
    if (rc != MX_OK) {
        delete P;
        return rc;
    }
    *out = P;
    return MX_OK;
}

extern "C" void mx_partition_destroy(mx_partition *p) { delete p; }

int mx::partition_host(const mx_partition *p)
{
    static std::mutex lock;
    std::lock_guard<std::mutex> hold(lock);
    if (p->host_ready) return MX_OK;
    if (!p->twin || !p->twin_download) {
        set_error("partition: its arrays are nowhere");
        return MX_ERR_ARG;
    }
    return p->twin_download(const_cast<mx_partition *>(p));
}

static int partition_view(const mx_partition *p, mx_partition_view *v, bool arrays);
extern "C" int mx_partition_get(const mx_partition *p, mx_partition_view *v)
{
    if (!p || !v) {
        set_error("mx_partition_get: null argument");
        return MX_ERR_ARG;
    }
    const int rc = mx::partition_host(p);
    if (rc) return rc;
    return partition_view(p, v, true);
}
extern "C" int mx_partition_counts(const mx_partition *p, mx_partition_view *v)
{
    if (!p || !v) {
        set_error("mx_partition_counts: null argument");
        return MX_ERR_ARG;
    }
    return partition_view(p, v, p->host_ready);
}
static int partition_view(const mx_partition *p, mx_partition_view *v, bool arrays)
{
    std::memset(v, 0, sizeof(*v));
    v->dtype = p->dtype;
    v->rows = p->rows;
    v->cols = p->cols;
    v->nnz = p->nnz;
    v->fragM = p->fragM;
    v->fragK = p->fragK;
    v->dCols = p->dCols;
    v->sCols = p->sCols;
    v->nnzColD = p->nnzColD;
    v->nnzColS = p->nnzColS;
    v->dRows = p->dRows;
    v->sRows = p->sRows;
    v->nnzRowD = p->nnzRowD;
    v->nnzRowS = p->nnzRowS;
    v->cols_ratio = p->cols_ratio;
    v->tc_nnz_ratio = p->tc_nnz_ratio;
    v->descColId = p->extracted ? p->descColId.data() : nullptr;
    v->newArray = p->newArray.data();
    v->rId = p->rId.data();
    v->newArray_ = p->newArray_.data();
    v->ddRowPtr = p->ddRowPtr.data();
    v->ddColInd = p->ddColInd.data();
    v->ddVal = p->ddVal.data();
    v->chunkNum = p->chunkNum;
    v->totalTcFrags = p->totalTcFrags;
    v->tcValCount = p->tcValCount;
    v->chunkPtr = p->chunkPtr.data();
    v->sparse_AToX_index = p->sparse_AToX_index.data();
    v->fragPtr = p->fragPtr.data();
    v->fragBit = p->dtype == MX_F64 ? (const void *)p->fragBit32.data() : (const void *)p->fragBit64.data();
    v->tcVal = p->tcVal.data();
    v->nnzCD = p->nnzCD;
    v->cdRowPtr = p->cdRowPtr.data();
    v->cdColInd = p->cdColInd.data();
    v->cdVal = p->cdVal.data();
    v->tau_c = p->tau_c;
    v->tau_r = p->tau_r;
    if (!arrays) {  // the counts alone: the arrays are still on the device
        v->descColId = v->newArray = v->rId = v->newArray_ = v->ddRowPtr = v->ddColInd = nullptr;
        v->chunkPtr = v->sparse_AToX_index = v->fragPtr = v->cdRowPtr = v->cdColInd = nullptr;
        v->ddVal = v->fragBit = v->tcVal = v->cdVal = nullptr;
    }
    return MX_OK;
}

extern "C" uint64_t mx_partition_hash(const mx_partition *p)
{
    if (!p || mx::partition_host(p) != MX_OK) return 0;
    uint64_t h = 14695981039346656037ull;
    const int es = mx::elem_size(p->dtype);
    h = fnv(&p->dCols, 4, h);
    h = fnv(&p->dRows, 4, h);
    h = fnv(p->descColId.data(), (size_t)p->dCols * 4, h);
    h = fnv(p->newArray.data(), p->newArray.size() * 4, h);
    h = fnv(p->rId.data(), p->rId.size() * 4, h);
    h = fnv(p->newArray_.data(), p->newArray_.size() * 4, h);
    h = fnv(p->chunkPtr.data(), p->chunkPtr.size() * 4, h);
    h = fnv(p->sparse_AToX_index.data(), p->sparse_AToX_index.size() * 4, h);
    h = fnv(p->fragPtr.data(), p->fragPtr.size() * 4, h);
    if (p->dtype == MX_F64)
        h = fnv(p->fragBit32.data(), p->fragBit32.size() * 4, h);
    else
        h = fnv(p->fragBit64.data(), p->fragBit64.size() * 8, h);
    h = fnv(p->tcVal.data(), (size_t)p->tcValCount * es, h);
    h = fnv(p->cdRowPtr.data(), p->cdRowPtr.size() * 4, h);
    h = fnv(p->cdColInd.data(), p->cdColInd.size() * 4, h);
    h = fnv(p->cdVal.data(), (size_t)p->nnzCD * es, h);
    return h;
}

// ---- partition file -------------------------------------------------------------------
// The head of the file is the reference's "_preprocessed.dat" (written by
// test/tcpreprocess.cpp:1208-1255, read back by test/tckernel.cpp:586-638), field for field:
//   int chunkNum; int chunkPtr[chunkNum+1]; int totalTcFrags; int fragK;
//   int sparse_AToX_index[totalTcFrags*fragK]; size_t n; int fragPtr[n];
//   size_t n; bitmap fragBit[n]; size_t n; valT tcVal[n]
// (bitmaps are uint32_t for binary64 as there, uint64_t for binary16), so that tool's reader
// takes the tile part of a binary64 file as it is.  The reference stores nothing else; the
// rest of the partition (sizes, thresholds, the four index maps, A_dd and the residual A_CD)
// follows in an extension that starts with a magic word.
namespace {

const uint64_t kFileMagic = 0x3154524150584d00ull;  // "\0MXPART1", little-endian

struct Writer {
    FILE *f;
    bool ok = true;
    void raw(const void *p, size_t n)
    {
        if (n && fwrite(p, 1, n, f) != n) ok = false;
    }
    template <typename T>
    void pod(const T &v) { raw(&v, sizeof(T)); }
    template <typename T>
    void vec(const std::vector<T> &v)
    {
        pod<uint64_t>((uint64_t)v.size());
        raw(v.data(), v.size() * sizeof(T));
    }
};

struct Reader {
    FILE *f;
    bool ok = true;
    void raw(void *p, size_t n)
    {
        if (n && fread(p, 1, n, f) != n) ok = false;
    }
    template <typename T>
    void pod(T &v) { raw(&v, sizeof(T)); }
    template <typename T>
    void vec(std::vector<T> &v, uint64_t limit)
    {
        uint64_t n = 0;
        pod(n);
        if (!ok || n > limit) {
            ok = false;
            return;
        }
        v.resize((size_t)n);
        raw(v.data(), (size_t)n * sizeof(T));
    }
};

}  // namespace

extern "C" int mx_partition_save(const mx_partition *p, const char *path)
{
    if (!p || !path) {
        set_error("mx_partition_save: null argument");
        return MX_ERR_ARG;
    }
    if (int rc = mx::partition_host(p)) return rc;
    FILE *f = fopen(path, "wb");
    if (!f) {
        set_error(std::string("mx_partition_save: cannot open ") + path);
        return MX_ERR_IO;
    }
    Writer w{f};
    const int es = mx::elem_size(p->dtype);
    // the reference's fields
    w.pod<int>(p->chunkNum);
    std::vector<int> cp(p->chunkPtr);
    cp.resize((size_t)p->chunkNum + 1, 0);
    w.raw(cp.data(), cp.size() * sizeof(int));
    w.pod<int>(p->totalTcFrags);
    w.pod<int>(p->fragK);
    w.raw(p->sparse_AToX_index.data(), (size_t)p->totalTcFrags * p->fragK * sizeof(int));
    std::vector<int> fp(p->fragPtr);
    fp.resize((size_t)p->totalTcFrags + 1, 0);
    w.pod<size_t>(fp.size());
    w.raw(fp.data(), fp.size() * sizeof(int));
    w.pod<size_t>((size_t)p->totalTcFrags);
    if (p->dtype == MX_F64) w.raw(p->fragBit32.data(), (size_t)p->totalTcFrags * 4);
    else w.raw(p->fragBit64.data(), (size_t)p->totalTcFrags * 8);
    w.pod<size_t>((size_t)p->tcValCount);
    w.raw(p->tcVal.data(), (size_t)p->tcValCount * es);
    // the extension
    w.pod(kFileMagic);
    const int head[8] = {(int)p->dtype, p->rows, p->cols, p->nnz, p->fragM, p->fragK, p->extracted ? 1 : 0, 0};
    w.raw(head, sizeof(head));
    w.pod(p->tau_c);
    w.pod(p->tau_r);
    const int counts[10] = {p->dCols, p->sCols, p->nnzColD, p->nnzColS, p->dRows, p->sRows, p->nnzRowD, p->nnzRowS,
                            p->nnzCD, p->tcValCount};
    w.raw(counts, sizeof(counts));
    w.pod(p->cols_ratio);
    w.pod(p->tc_nnz_ratio);
    w.vec(p->descColId);
    w.vec(p->newArray);
    w.vec(p->rId);
    w.vec(p->newArray_);
    w.vec(p->ddRowPtr);
    w.vec(p->ddColInd);
    w.vec(p->ddVal.bytes);
    w.vec(p->cdRowPtr);
    w.vec(p->cdColInd);
    w.vec(p->cdVal.bytes);
    w.pod<uint64_t>(mx_partition_hash(p));
    const bool ok = w.ok && fclose(f) == 0;
    if (!ok) {
        set_error(std::string("mx_partition_save: write failed: ") + path);
        return MX_ERR_IO;
    }
    return MX_OK;
}

extern "C" int mx_partition_load(const char *path, mx_dtype dtype, mx_partition **out)
{
    if (!path || !out) {
        set_error("mx_partition_load: null argument");
        return MX_ERR_ARG;
    }
    *out = nullptr;
    FILE *f = fopen(path, "rb");
    if (!f) {
        set_error(std::string("mx_partition_load: cannot open ") + path);
        return MX_ERR_IO;
    }
    fseek(f, 0, SEEK_END);
    const uint64_t fileSize = (uint64_t)ftell(f);  // no array can be longer than the file
    fseek(f, 0, SEEK_SET);
    mx_partition *p = new (std::nothrow) mx_partition();
    if (!p) {
        fclose(f);
        set_error("mx_partition_load: out of memory");
        return MX_ERR_ALLOC;
    }
    auto fail = [&](const char *what) {
        fclose(f);
        delete p;
        set_error(std::string("mx_partition_load: ") + what + ": " + path);
        return MX_ERR_IO;
    };
    try {
        Reader r{f};
        const int es = mx::elem_size(dtype);
        r.pod(p->chunkNum);
        if (!r.ok || p->chunkNum < 0 || (uint64_t)p->chunkNum * 4 > fileSize) return fail("bad chunk count");
        p->chunkPtr.resize((size_t)p->chunkNum + 1);
        r.raw(p->chunkPtr.data(), p->chunkPtr.size() * sizeof(int));
        r.pod(p->totalTcFrags);
        r.pod(p->fragK);
        if (!r.ok || p->totalTcFrags < 0 || p->fragK != mx::frag_k(dtype) ||
            (uint64_t)p->totalTcFrags * p->fragK * 4 > fileSize)
            return fail("tile header does not fit the requested precision");
        p->sparse_AToX_index.resize((size_t)p->totalTcFrags * p->fragK);
        r.raw(p->sparse_AToX_index.data(), p->sparse_AToX_index.size() * sizeof(int));
        size_t n = 0;
        r.pod(n);
        if (!r.ok || n != (size_t)p->totalTcFrags + 1) return fail("bad fragPtr length");
        p->fragPtr.resize(n);
        r.raw(p->fragPtr.data(), n * sizeof(int));
        r.pod(n);
        if (!r.ok || n != (size_t)p->totalTcFrags) return fail("bad fragBit length");
        if (dtype == MX_F64) {
            p->fragBit32.resize(n);
            r.raw(p->fragBit32.data(), n * 4);
        } else {
            p->fragBit64.resize(n);
            r.raw(p->fragBit64.data(), n * 8);
        }
        r.pod(n);
        if (!r.ok || (uint64_t)n * es > fileSize) return fail("bad tcVal length");
        p->tcValCount = (int)n;
        p->tcVal.resize(n, es);
        r.raw(p->tcVal.data(), n * es);
        uint64_t magic = 0;
        r.pod(magic);
        if (!r.ok || magic != kFileMagic)
            return fail("the file holds the tile part only (written by the reference tool): the residual is missing");
        int head[8], counts[10];
        r.raw(head, sizeof(head));
        r.pod(p->tau_c);
        r.pod(p->tau_r);
        r.raw(counts, sizeof(counts));
        r.pod(p->cols_ratio);
        r.pod(p->tc_nnz_ratio);
        if (!r.ok || head[0] != (int)dtype || head[4] != mx::kFragM || head[5] != p->fragK)
            return fail("written for the other precision");
        p->dtype = dtype;
        p->rows = head[1];
        p->cols = head[2];
        p->nnz = head[3];
        p->fragM = head[4];
        p->extracted = head[6] != 0;
        p->dCols = counts[0];
        p->sCols = counts[1];
        p->nnzColD = counts[2];
        p->nnzColS = counts[3];
        p->dRows = counts[4];
        p->sRows = counts[5];
        p->nnzRowD = counts[6];
        p->nnzRowS = counts[7];
        p->nnzCD = counts[8];
        if (counts[9] != p->tcValCount) return fail("inconsistent value count");
        r.vec(p->descColId, fileSize);
        r.vec(p->newArray, fileSize);
        r.vec(p->rId, fileSize);
        r.vec(p->newArray_, fileSize);
        r.vec(p->ddRowPtr, fileSize);
        r.vec(p->ddColInd, fileSize);
        r.vec(p->ddVal.bytes, fileSize);
        r.vec(p->cdRowPtr, fileSize);
        r.vec(p->cdColInd, fileSize);
        r.vec(p->cdVal.bytes, fileSize);
        uint64_t hash = 0;
        r.pod(hash);
        if (!r.ok) return fail("truncated");
        // sizes the rest of the library relies on
        if (p->rows < 0 || p->cols < 0 || p->dRows < 0 || p->dCols < 0 || p->dCols > p->cols || p->dRows > p->rows ||
            (int)p->cdRowPtr.size() != p->rows + 1 || (int)p->cdColInd.size() != p->nnzCD ||
            p->cdVal.bytes.size() != (size_t)p->nnzCD * es || (int)p->rId.size() != p->dRows ||
            (int)p->ddRowPtr.size() != (p->extracted ? p->dRows + 1 : (int)p->ddRowPtr.size()) ||
            (p->extracted && (int)p->descColId.size() != p->cols) ||
            p->chunkNum != (p->extracted ? (p->dRows + p->fragM - 1) / p->fragM : p->chunkNum) ||
            p->chunkPtr.back() != p->totalTcFrags || p->fragPtr.back() != p->tcValCount)
            return fail("inconsistent sizes");
        for (int c : p->cdColInd)
            if ((unsigned)c >= (unsigned)std::max(p->cols, 1)) return fail("column index out of range");
        for (int c : p->sparse_AToX_index)
            if ((unsigned)c >= (unsigned)std::max(p->dCols, 1)) return fail("tile column out of range");
        for (int c : p->rId)
            if ((unsigned)c >= (unsigned)std::max(p->rows, 1)) return fail("row index out of range");
        if (hash != mx_partition_hash(p)) return fail("checksum mismatch");
    } catch (const std::bad_alloc &) {
        fclose(f);
        delete p;
        set_error("mx_partition_load: out of memory");
        return MX_ERR_ALLOC;
    }
    fclose(f);
    *out = p;
    return MX_OK;
}

// csr2csc / csc2csr (utilities/csr2csc.cpp:4-203) as a stable counting-sort transpose.
extern "C" int mx_transpose(mx_dtype dtype, int outer, int inner, int nnz, const int *ptr, const int *ind,
                            const void *val, int **tPtr, int **tInd, void **tVal)
{
    if (outer < 0 || inner < 0 || nnz < 0 || !ptr || !tPtr || !tInd || !tVal || (nnz > 0 && (!ind || !val))) {
        set_error("mx_transpose: bad argument");
        return MX_ERR_ARG;
    }
    const size_t es = (size_t)mx::elem_size(dtype);
    int *cp = (int *)calloc((size_t)inner + 1, sizeof(int));
    int *ri = (int *)malloc((size_t)std::max(nnz, 1) * sizeof(int));
    unsigned char *tv = (unsigned char *)malloc((size_t)std::max(nnz, 1) * es);
    std::vector<int> cursor;
    try {
        cursor.resize((size_t)inner + 1);
    } catch (const std::bad_alloc &) {
        free(cp);
        cp = nullptr;
    }
    if (!cp || !ri || !tv) {
        free(cp);
        free(ri);
        free(tv);
        set_error("mx_transpose: out of memory");
        return MX_ERR_ALLOC;
    }
    for (int p = 0; p < nnz; ++p) {
        if ((unsigned)ind[p] >= (unsigned)inner) {
            free(cp);
            free(ri);
            free(tv);
            set_error("mx_transpose: index out of range");
            return MX_ERR_ARG;
        }
        cp[ind[p] + 1]++;
    }
    for (int c = 0; c < inner; ++c) cp[c + 1] += cp[c];
    std::copy(cp, cp + inner + 1, cursor.begin());
    const unsigned char *sv = (const unsigned char *)val;
    for (int r = 0; r < outer; ++r)
        for (int p = ptr[r]; p < ptr[r + 1]; ++p) {
            int q = cursor[ind[p]]++;
            ri[q] = r;
            std::memcpy(tv + (size_t)q * es, sv + (size_t)p * es, es);
        }
    *tPtr = cp;
    *tInd = ri;
    *tVal = tv;
    return MX_OK;
}

extern "C" void mx_free(void *p) { free(p); }

extern "C" double mx_algorithmic_bytes(mx_dtype dtype, int rows, int cols, int nnz)
{
    const double s = mx::elem_size(dtype);
    return (double)nnz * (s + 4.0) + ((double)rows + 1.0) * 4.0 + (double)cols * s + (double)rows * s;
}

extern "C" void mx_init_vec(mx_dtype dtype, void *v, int n)
{
    if (!v) return;
    if (dtype == MX_F64) {
        double *d = (double *)v;
        for (int i = 0; i < n; ++i) d[i] = (double)(float)(i % 15);
    } else {
        uint16_t *h = (uint16_t *)v;
        for (int i = 0; i < n; ++i) h[i] = mx::f64_to_f16_bits((double)(i % 15));
    }
}
