// Device side of the preprocessing: the transposes, and the two selections of the cascaded
// extraction (which columns, then which rows, are dense).
//
// The reference transposes on the GPU as well -- csr2csc / csc2csr copy the matrix to the
// device, call cusparseCsr2cscEx2 and copy the result back (utilities/csr2csc.cpp:4-203), three
// times per run (test/test_autotc_spmv.cpp:1119-1238).  Here the matrix stays where it is: the
// entry point takes device arrays and leaves device arrays, so a caller that already holds the
// matrix in HBM pays no PCIe traffic.  The order inside every output line is the one the host
// transpose (mx_transpose) produces -- ascending source line, equal pairs in source order -- so
// the two are interchangeable bit for bit.
//
// Route: a transpose is a stable sort of the entries by their index.  Entry e of source line r
// gets the key ind[e] and the payload e; source order is ascending (r, e), so a stable sort by
// key alone gives ascending (ind, r, e).  rocPRIM's radix sort is stable and sorts only the
// ceil(log2(inner)) bits the keys can have.  Three small kernels around it: the source line of
// every entry (binary search in ptr), the output line pointers from the sorted keys (every
// thread writes the pointers of the lines that start at its position), and the gather of
// source lines and values through the sorted payload.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "mx_device.h"
#include "mx_internal.h"

namespace mxp {

constexpr int kBlock = 256;
// Entry numbers are formed as blockIdx.x * kBlock + threadIdx.x in 32 bits: the last block must not pass 2^31.
constexpr int kMaxCount = 2147483647 - 2 * kBlock;

// line[e] = r with ptr[r] <= e < ptr[r+1]; bad |= 1 where ind[e] lies outside [0, inner).
__global__ __launch_bounds__(kBlock) void entry_lines_kernel(const int *__restrict__ ptr, const int *__restrict__ ind,
                                                             int outer, int inner, int nnz, int *__restrict__ line,
                                                             int *__restrict__ payload, int *__restrict__ bad)
{
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= nnz) return;
    // last r in [0, outer) with ptr[r] <= e  (empty lines repeat a pointer: the last one wins,
    // and it is the only one whose range holds e)
    int lo = 0, hi = outer - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (ptr[mid] <= e) lo = mid;
        else hi = mid - 1;
    }
    line[e] = lo;
    payload[e] = e;
    if ((unsigned)ind[e] >= (unsigned)inner) atomicOr(bad, 1);
}

// tPtr[c] = number of sorted keys below c, for c in [0, inner].  Thread k owns the lines
// (key[k-1], key[k]]; the thread behind the last key owns what is left, inner included.
__global__ __launch_bounds__(kBlock) void line_pointers_kernel(const int *__restrict__ key, int nnz, int inner,
                                                               int *__restrict__ tPtr)
{
    const long long k = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (k > nnz) return;
    const int first = k == 0 ? 0 : key[k - 1] + 1;
    const int last = k == nnz ? inner : key[k];
    for (int c = first; c <= last; ++c) tPtr[c] = (int)k;
}

template <typename V>
__global__ __launch_bounds__(kBlock) void gather_kernel(const int *__restrict__ payload, const int *__restrict__ line,
                                                        const V *__restrict__ val, int nnz, int *__restrict__ tInd,
                                                        V *__restrict__ tVal)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    const int e = payload[k];
    tInd[k] = line[e];
    tVal[k] = val[e];
}

// ---- selection ---------------------------------------------------------------------------
// The line of entry e, as in entry_lines_kernel.
__device__ __forceinline__ int line_of(const int *__restrict__ ptr, int outer, int e)
{
    int lo = 0, hi = outer - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (ptr[mid] <= e) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

// cnt[ind[e]] += 1 for every entry (integer atomics: the result does not depend on the order).
__global__ __launch_bounds__(kBlock) void index_histogram_kernel(const int *__restrict__ ind, int nnz, int inner,
                                                                 int *__restrict__ cnt, int *__restrict__ bad)
{
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= nnz) return;
    const int c = ind[e];
    if ((unsigned)c >= (unsigned)inner) atomicOr(bad, 1);
    else atomicAdd(&cnt[c], 1);
}

// bad |= bit where v[i] lies outside [0, lim): the index arrays of a caller are looked at before a
// kernel uses them as addresses.
__global__ __launch_bounds__(kBlock) void range_check_kernel(const int *__restrict__ v, int n, int lim, int bit,
                                                             int *__restrict__ bad)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n && (unsigned)v[i] >= (unsigned)lim) atomicOr(bad, bit);
}
// bad |= bit unless ptr[0] == 0, ptr[n] == total and ptr never falls.
__global__ __launch_bounds__(kBlock) void pointer_check_kernel(const int *__restrict__ ptr, int n, int total, int bit,
                                                               int *__restrict__ bad)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i > n) return;
    const int p = ptr[i];
    if ((i == 0 && p != 0) || (i == n && p != total) || (i < n && ptr[i + 1] < p) || p < 0 || p > total) atomicOr(bad, bit);
}

__global__ __launch_bounds__(kBlock) void iota_kernel(int *__restrict__ v, int n)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) v[i] = i;
}

// The shortest prefix of the sorted counts whose sum reaches `target`, from their running sums:
// res[0] = its length (stays -1 when the target is out of reach), res[1] = its sum; res[2], res[3]
// = number and sum of the counts that are not zero (what an unreachable target selects).
__global__ __launch_bounds__(kBlock) void prefix_reach_kernel(const int *__restrict__ sortedCnt, const int *__restrict__ run,
                                                              int n, int target, int *__restrict__ res)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const int s = run[i], prev = i ? run[i - 1] : 0;
    if (s >= target && (i == 0 || prev < target)) {
        res[0] = i + 1;
        res[1] = s;
    }
    if (sortedCnt[i] > 0 && (i == n - 1 || sortedCnt[i + 1] == 0)) {
        res[2] = i + 1;
        res[3] = s;
    }
}

// dense[order[i]] = 1 for the first k lines of the order
__global__ __launch_bounds__(kBlock) void mark_selected_kernel(const int *__restrict__ order, int k, unsigned char *__restrict__ dense)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < k) dense[order[i]] = 1;
}

// rcnt[r] = entries of row r in selected columns
__global__ __launch_bounds__(kBlock) void dense_row_counts_kernel(const int *__restrict__ rowPtr, const int *__restrict__ col,
                                                                  const unsigned char *__restrict__ dense, int rows, int nnz,
                                                                  int *__restrict__ rcnt)
{
    // The lanes of a wave hold consecutive entries, so their rows ascend: the first lane of every run
    // of equal rows adds the run's count in one atomic (a row of thousands of entries would otherwise
    // take thousands of atomics on one address).
    const int e = blockIdx.x * kBlock + threadIdx.x;
    const bool in = e < nnz;
    const int r = in ? line_of(rowPtr, rows, e) : -1;
    const bool d = in && dense[col[e]];
    const int lane = threadIdx.x & 63;
    const int rPrev = __shfl_up(r, 1);
    const unsigned long long heads = __ballot(lane == 0 || r != rPrev), hits = __ballot(d);
    if (!in || !((heads >> lane) & 1)) return;
    const unsigned long long above = lane == 63 ? 0ull : heads >> (lane + 1);
    const int next = above ? lane + 1 + __builtin_ctzll(above) : 64;
    const unsigned long long run = (next == 64 ? ~0ull : (1ull << next) - 1) & ~((1ull << lane) - 1);
    const int c = __popcll(hits & run);
    if (c) atomicAdd(&rcnt[r], c);
}

// ---- split --------------------------------------------------------------------------------
// rank[order[i]] = i for the first k lines of the order
__global__ __launch_bounds__(kBlock) void scatter_rank_kernel(const int *__restrict__ order, int k, int *__restrict__ rank)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < k) rank[order[i]] = i;
}

// notSel[c] = 1 where the column was not selected (input of the running count that numbers them)
__global__ __launch_bounds__(kBlock) void not_selected_kernel(const unsigned char *__restrict__ dense, int cols, int *__restrict__ notSel)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c <= cols) notSel[c] = c < cols ? !dense[c] : 0;
}

// new column id of an unselected column: dCols + its position among the unselected, ascending
__global__ __launch_bounds__(kBlock) void sparse_columns_kernel(const unsigned char *__restrict__ dense, const int *__restrict__ pos,
                                                                int cols, int dCols, int *__restrict__ newCol)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c < cols && !dense[c]) newCol[c] = dCols + pos[c];
}

// lengths of the residual's rows (entries in unselected columns, plus those in selected columns
// when the row itself was not selected) and of A_dd's rows (rank order); one more element, zero,
// so that a running count over n + 1 elements ends with the total
__global__ __launch_bounds__(kBlock) void split_lengths_kernel(const int *__restrict__ rowPtr, const int *__restrict__ rcnt,
                                                               const int *__restrict__ rowRank, const int *__restrict__ rowOrder,
                                                               int rows, int dRows, int *__restrict__ cdLen, int *__restrict__ ddLen)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r <= rows) cdLen[r] = r < rows ? (rowPtr[r + 1] - rowPtr[r] - rcnt[r]) + (rowRank[r] < 0 ? rcnt[r] : 0) : 0;
    if (r <= dRows) ddLen[r] = r < dRows ? rcnt[rowOrder[r]] : 0;
}

// Sort key of an entry: [which matrix][its row there][residual only: selected column?][new column].
// A_dd (matrix 0) sorts in front of the residual (matrix 1); inside a residual row the entries in
// unselected columns come first, then those in selected ones; equal keys keep source order.
__global__ __launch_bounds__(kBlock) void split_keys_kernel(const int *__restrict__ rowPtr, const int *__restrict__ col,
                                                            const int *__restrict__ newCol, const int *__restrict__ rowRank,
                                                            int rows, int nnz, int dCols, int colBits, int rowBits,
                                                            unsigned long long *__restrict__ key, int *__restrict__ payload)
{
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= nnz) return;
    const int r = line_of(rowPtr, rows, e), nc = newCol[col[e]], rank = rowRank[r];
    const bool sel = nc < dCols;
    unsigned long long k;
    if (sel && rank >= 0) k = ((unsigned long long)rank << (colBits + 1)) | (unsigned long long)nc;
    else
        k = (1ull << (rowBits + colBits + 1)) | ((unsigned long long)r << (colBits + 1)) |
            ((unsigned long long)sel << colBits) | (unsigned long long)nc;
    key[e] = k;
    payload[e] = e;
}

template <typename V>
__global__ __launch_bounds__(kBlock) void split_gather_kernel(const unsigned long long *__restrict__ key, const int *__restrict__ payload,
                                                              const V *__restrict__ val, int nnz, int nDD, int colBits,
                                                              int *__restrict__ ddInd, V *__restrict__ ddVal,
                                                              int *__restrict__ cdInd, V *__restrict__ cdVal)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    const int nc = (int)(key[k] & ((1ull << colBits) - 1));
    const V v = val[payload[k]];
    if (k < nDD) {
        ddInd[k] = nc;
        ddVal[k] = v;
    } else {
        cdInd[k - nDD] = nc;
        cdVal[k - nDD] = v;
    }
}

// ---- tile encoding ------------------------------------------------------------------------
// key = [chunk of the entry's row][column] for every entry of A_dd; payload = the entry
__global__ __launch_bounds__(kBlock) void tile_keys_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                           int dRows, int n, int colBits, unsigned long long *__restrict__ key,
                                                           int *__restrict__ payload)
{
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= n) return;
    const int w = line_of(ddRowPtr, dRows, e) / mx::kFragM;
    key[e] = ((unsigned long long)w << colBits) | (unsigned long long)ddCol[e];
    payload[e] = e;
}

// head[k] = 1 where sorted position k holds the first occurrence of its (chunk, column)
__global__ __launch_bounds__(kBlock) void tile_heads_kernel(const unsigned long long *__restrict__ key, int n, int *__restrict__ head)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < n) head[k] = k == 0 || key[k] != key[k - 1];
}

// frags[w] = ceil(distinct columns of chunk w / fragK); one more element, zero.  The entries of
// chunk w sit at sorted positions [a, b) = ddRowPtr[8w] .. ddRowPtr[min(8w + 8, dRows)], and `run`
// is the inclusive running count of the heads.
__global__ __launch_bounds__(kBlock) void tile_chunk_frags_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ run,
                                                                  int dRows, int chunkNum, int fragK, int *__restrict__ frags)
{
    const int w = blockIdx.x * kBlock + threadIdx.x;
    if (w > chunkNum) return;
    int f = 0;
    if (w < chunkNum) {
        const int a = ddRowPtr[w * mx::kFragM], b = ddRowPtr[min(w * mx::kFragM + mx::kFragM, dRows)];
        if (b > a) f = (run[b - 1] - run[a] + 1 + fragK - 1) / fragK;
    }
    frags[w] = f;
}

// Per sorted position: the rank of its column inside its chunk (ecr) goes back to the entry; a
// head also writes its column into the chunk's list; every entry sets its bit.
__global__ __launch_bounds__(kBlock) void tile_rank_kernel(const unsigned long long *__restrict__ key, const int *__restrict__ payload,
                                                           const int *__restrict__ head, const int *__restrict__ run,
                                                           const int *__restrict__ ddRowPtr, const int *__restrict__ chunkPtr, int dRows,
                                                           int n, int colBits, int fragK, int *__restrict__ ecr, int *__restrict__ atox,
                                                           unsigned long long *__restrict__ bits)
{
    const int k = blockIdx.x * kBlock + threadIdx.x, lane = threadIdx.x & 63;
    int f = -1;
    unsigned long long v = 0;
    if (k < n) {
        const int w = (int)(key[k] >> colBits), c = (int)(key[k] & ((1ull << colBits) - 1));
        const int rank = run[k] - run[ddRowPtr[w * mx::kFragM]];
        const int e = payload[k];
        ecr[e] = rank;
        const int f0 = chunkPtr[w];
        if (head[k]) atox[(size_t)f0 * fragK + rank] = c;
        const int r = line_of(ddRowPtr, dRows, e) - w * mx::kFragM;
        f = f0 + rank / fragK;
        v = 1ull << (r * fragK + rank % fragK);
    }
    // Sorted positions ascend by (chunk, column), so the fragments of a wave's lanes ascend too: the
    // bits of every run of equal fragments are gathered at its first lane, which issues one atomic.
    const int fPrev = __shfl_up(f, 1);
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long o = __shfl_down(v, off);
        const int fo = __shfl_down(f, off);
        if (lane + off < 64 && fo == f) v |= o;
    }
    if (f >= 0 && (lane == 0 || f != fPrev)) atomicOr(&bits[f], v);
}

// count[f] = set bits of fragment f; one more element, zero
__global__ __launch_bounds__(kBlock) void tile_popcount_kernel(const unsigned long long *__restrict__ bits, int nf, int *__restrict__ count)
{
    const int f = blockIdx.x * kBlock + threadIdx.x;
    if (f <= nf) count[f] = f < nf ? __popcll(bits[f]) : 0;
}

// Values of a fragment in ascending bit order: an entry's place is the number of set bits below
// its own.  Of entries that name the same row and column (neighbours in the sorted row) the last
// one is kept.
template <typename V>
__global__ __launch_bounds__(kBlock) void tile_values_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                             const V *__restrict__ ddVal, const int *__restrict__ ecr,
                                                             const int *__restrict__ chunkPtr, const int *__restrict__ fragPtr,
                                                             const unsigned long long *__restrict__ bits, int dRows, int n, int fragK,
                                                             V *__restrict__ tcVal)
{
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= n) return;
    const int i = line_of(ddRowPtr, dRows, e);
    if (e + 1 < ddRowPtr[i + 1] && ddCol[e + 1] == ddCol[e]) return;  // a later twin wins
    const int w = i / mx::kFragM, rank = ecr[e], f = chunkPtr[w] + rank / fragK;
    const int bit = (i - w * mx::kFragM) * fragK + rank % fragK;
    tcVal[fragPtr[f] + __popcll(bits[f] & ((1ull << bit) - 1))] = ddVal[e];
}

__global__ __launch_bounds__(kBlock) void narrow_bits_kernel(const unsigned long long *__restrict__ bits, int nf, unsigned *__restrict__ out)
{
    const int f = blockIdx.x * kBlock + threadIdx.x;
    if (f < nf) out[f] = (unsigned)bits[f];
}

struct Scratch {
    void *p = nullptr;
    ~Scratch()
    {
        if (p) (void)hipFree(p);
    }
};

}  // namespace mxp

// `who` is the name of the entry point the enclosing function works for
#define MXP_TRY(call)                                                                       \
    do {                                                                                    \
        hipError_t e_ = (call);                                                             \
        if (e_ != hipSuccess) {                                                             \
            mx::set_error(std::string(who) + ": " + #call + ": " + hipGetErrorString(e_)); \
            return e_ == hipErrorOutOfMemory ? MX_ERR_ALLOC : MX_ERR_DEVICE;                \
        }                                                                                   \
    } while (0)

extern "C" int mx_transpose_device(mx_dtype dtype, int outer, int inner, int nnz, const int *ptr_dev, const int *ind_dev,
                                   const void *val_dev, int *tPtr_dev, int *tInd_dev, void *tVal_dev, void *stream)
{
    static const char who[] = "mx_transpose_device";
    using namespace mxp;
    if ((dtype != MX_F64 && dtype != MX_F16) || outer < 0 || inner < 0 || nnz < 0 || !ptr_dev || !tPtr_dev ||
        (nnz > 0 && (!ind_dev || !val_dev || !tInd_dev || !tVal_dev || outer == 0))) {
        mx::set_error("mx_transpose_device: bad argument");
        return MX_ERR_ARG;
    }
    if (nnz > kMaxCount || inner > kMaxCount || outer > kMaxCount) {
        mx::set_error("mx_transpose_device: more than 2^31 - 513 entries or lines");
        return MX_ERR_ARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int pblocks = (int)(((long long)nnz + 1 + kBlock - 1) / kBlock);
    if (nnz == 0) {
        hipLaunchKernelGGL(line_pointers_kernel, dim3(pblocks), dim3(kBlock), 0, s, (const int *)nullptr, 0, inner, tPtr_dev);
        MXP_TRY(hipGetLastError());
        MXP_TRY(hipStreamSynchronize(s));
        return MX_OK;
    }
    int bits = 1;
    while (bits < 31 && (1ll << bits) < (long long)inner) ++bits;
    // one allocation: line[nnz], payload in/out [nnz] each, keys out [nnz], flag, sort storage
    size_t sortBytes = 0;
    MXP_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const int *)nullptr, (int *)nullptr, (const int *)nullptr,
                                      (int *)nullptr, (size_t)nnz, 0u, (unsigned)bits, s));
    const size_t n4 = ((size_t)nnz * sizeof(int) + 255) & ~(size_t)255;
    Scratch scratch;
    MXP_TRY(hipMalloc(&scratch.p, 4 * n4 + 256 + sortBytes));
    unsigned char *base = (unsigned char *)scratch.p;
    int *line = (int *)base, *payIn = (int *)(base + n4), *payOut = (int *)(base + 2 * n4), *keyOut = (int *)(base + 3 * n4);
    int *bad = (int *)(base + 4 * n4);
    void *sortTmp = base + 4 * n4 + 256;
    const int eblocks = (nnz + kBlock - 1) / kBlock;
    MXP_TRY(hipMemsetAsync(bad, 0, sizeof(int), s));
    hipLaunchKernelGGL(entry_lines_kernel, dim3(eblocks), dim3(kBlock), 0, s, ptr_dev, ind_dev, outer, inner, nnz, line,
                       payIn, bad);
    MXP_TRY(hipGetLastError());
    // an index outside [0, inner) must not reach the pointer kernel: look before going on
    int badHost = 0;
    MXP_TRY(hipMemcpyAsync(&badHost, bad, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));
    if (badHost) {
        mx::set_error("mx_transpose_device: index out of range");
        return MX_ERR_ARG;
    }
    MXP_TRY(rocprim::radix_sort_pairs(sortTmp, sortBytes, ind_dev, keyOut, (const int *)payIn, payOut, (size_t)nnz, 0u,
                                      (unsigned)bits, s));
    hipLaunchKernelGGL(line_pointers_kernel, dim3(pblocks), dim3(kBlock), 0, s, (const int *)keyOut, nnz, inner, tPtr_dev);
    MXP_TRY(hipGetLastError());
    if (dtype == MX_F64)
        hipLaunchKernelGGL(gather_kernel<double>, dim3(eblocks), dim3(kBlock), 0, s, (const int *)payOut, (const int *)line,
                           (const double *)val_dev, nnz, tInd_dev, (double *)tVal_dev);
    else
        hipLaunchKernelGGL(gather_kernel<uint16_t>, dim3(eblocks), dim3(kBlock), 0, s, (const int *)payOut,
                           (const int *)line, (const uint16_t *)val_dev, nnz, tInd_dev, (uint16_t *)tVal_dev);
    MXP_TRY(hipGetLastError());
    MXP_TRY(hipStreamSynchronize(s));  // the scratch is released on return
    return MX_OK;
}


namespace mxp {

// order[0..n) = the lines by count descending, ties by ascending line (a stable descending sort
// of the counts with the line numbers as payload); then the prefix that reaches `target`.
// cnt, order: device arrays of n; work: 3 n ints + 4; returns the prefix length and its sum.
static int order_and_reach(const int *cnt, int n, int target, int *order, int *work, void *sortTmp, size_t sortBytes,
                           void *scanTmp, size_t scanBytes, hipStream_t s, int *len, int *sum)
{
    static const char who[] = "mx_select_device";
    *len = 0;
    *sum = 0;
    if (n == 0) return MX_OK;
    int *ids = work, *sortedCnt = work + n, *run = work + 2 * (size_t)n, *res = work + 3 * (size_t)n;
    const int blocks = (n + kBlock - 1) / kBlock;
    hipLaunchKernelGGL(iota_kernel, dim3(blocks), dim3(kBlock), 0, s, ids, n);
    MXP_TRY(hipGetLastError());
    MXP_TRY(rocprim::radix_sort_pairs_desc(sortTmp, sortBytes, cnt, sortedCnt, (const int *)ids, order, (size_t)n, 0u, 32u, s));
    MXP_TRY(rocprim::inclusive_scan(scanTmp, scanBytes, (const int *)sortedCnt, run, (size_t)n, rocprim::plus<int>(), s));
    const int init[4] = {-1, 0, 0, 0};
    MXP_TRY(hipMemcpyAsync(res, init, sizeof(init), hipMemcpyHostToDevice, s));
    hipLaunchKernelGGL(prefix_reach_kernel, dim3(blocks), dim3(kBlock), 0, s, (const int *)sortedCnt, (const int *)run, n,
                       target, res);
    MXP_TRY(hipGetLastError());
    int got[4];
    MXP_TRY(hipMemcpyAsync(got, res, sizeof(got), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));
    *len = got[0] >= 0 ? got[0] : got[2];
    *sum = got[0] >= 0 ? got[1] : got[3];
    return MX_OK;
}

}  // namespace mxp

extern "C" int mx_select_device(int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, float tau_c,
                                float tau_r, int *descColId_dev, int *descRowId_dev, mx_selection *out, void *stream)
{
    static const char who[] = "mx_select_device";
    using namespace mxp;
    if (rows < 0 || cols < 0 || nnz < 0 || !rowPtr_dev || !out || (cols > 0 && !descColId_dev) ||
        (rows > 0 && !descRowId_dev) || (nnz > 0 && (!colInd_dev || rows == 0 || cols == 0)) || !(tau_c >= 0.f) ||
        !(tau_c <= 1.f) || !(tau_r >= 0.f) || !(tau_r <= tau_c)) {
        mx::set_error("mx_select_device: bad argument");
        return MX_ERR_ARG;
    }
    if (nnz > kMaxCount || rows > kMaxCount || cols > kMaxCount) {
        mx::set_error("mx_select_device: more than 2^31 - 513 entries, rows or columns");
        return MX_ERR_ARG;
    }
    hipStream_t s = (hipStream_t)stream;
    *out = mx_selection{0, 0, 0, 0};
    const size_t n = (size_t)std::max(rows, cols);
    size_t sortBytes = 0, scanBytes = 0;
    if (n > 0) {
        MXP_TRY(rocprim::radix_sort_pairs_desc(nullptr, sortBytes, (const int *)nullptr, (int *)nullptr, (const int *)nullptr,
                                               (int *)nullptr, n, 0u, 32u, s));
        MXP_TRY(rocprim::inclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, n, rocprim::plus<int>(), s));
    }
    sortBytes = (sortBytes + 255) & ~(size_t)255;
    // counts [n], work [3 n + 4], flag, dense flags [cols], the library's storage
    const size_t cntB = (n * sizeof(int) + 255) & ~(size_t)255, workB = ((3 * n + 4) * sizeof(int) + 255) & ~(size_t)255;
    const size_t denseB = ((size_t)cols + 255) & ~(size_t)255;
    Scratch scratch;
    MXP_TRY(hipMalloc(&scratch.p, cntB + workB + 256 + denseB + sortBytes + scanBytes + 256));
    unsigned char *base = (unsigned char *)scratch.p;
    int *cnt = (int *)base, *work = (int *)(base + cntB), *bad = (int *)(base + cntB + workB);
    unsigned char *dense = base + cntB + workB + 256;
    void *sortTmp = dense + denseB, *scanTmp = dense + denseB + sortBytes;
    const int eblocks = (nnz + kBlock - 1) / kBlock;

    // ---- column pass (test/test_autotc_spmv.cpp:1122-1141)
    MXP_TRY(hipMemsetAsync(base, 0, cntB + workB + 256 + denseB, s));
    if (nnz > 0) {
        hipLaunchKernelGGL(index_histogram_kernel, dim3(eblocks), dim3(kBlock), 0, s, colInd_dev, nnz, cols, cnt, bad);
        MXP_TRY(hipGetLastError());
    }
    int badHost = 0;
    MXP_TRY(hipMemcpyAsync(&badHost, bad, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));
    if (badHost) {
        mx::set_error("mx_select_device: column index out of range");
        return MX_ERR_ARG;
    }
    int rc = order_and_reach(cnt, cols, mx::threshold(nnz, tau_c), descColId_dev, work, sortTmp, sortBytes, scanTmp, scanBytes,
                             s, &out->dCols, &out->nnzColD);
    if (rc != MX_OK) return rc;

    // ---- row pass on the selected columns (:1240-1267)
    MXP_TRY(hipMemsetAsync(cnt, 0, cntB, s));
    if (out->dCols > 0) {
        hipLaunchKernelGGL(mark_selected_kernel, dim3((out->dCols + kBlock - 1) / kBlock), dim3(kBlock), 0, s,
                           (const int *)descColId_dev, out->dCols, dense);
        MXP_TRY(hipGetLastError());
    }
    if (nnz > 0) {
        hipLaunchKernelGGL(dense_row_counts_kernel, dim3(eblocks), dim3(kBlock), 0, s, rowPtr_dev, colInd_dev,
                           (const unsigned char *)dense, rows, nnz, cnt);
        MXP_TRY(hipGetLastError());
    }
    rc = order_and_reach(cnt, rows, mx::threshold(nnz, tau_r), descRowId_dev, work, sortTmp, sortBytes, scanTmp, scanBytes, s,
                         &out->dRows, &out->nnzRowD);
    return rc;
}


extern "C" int mx_split_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                               const void *val_dev, const mx_selection *sel, const int *descColId_dev,
                               const int *descRowId_dev, int *ddRowPtr_dev, int *ddColInd_dev, void *ddVal_dev,
                               int *cdRowPtr_dev, int *cdColInd_dev, void *cdVal_dev, void *stream)
{
    static const char who[] = "mx_split_device";
    using namespace mxp;
    if ((dtype != MX_F64 && dtype != MX_F16) || rows < 0 || cols < 0 || nnz < 0 || !sel || !rowPtr_dev || !ddRowPtr_dev ||
        !cdRowPtr_dev || sel->dCols < 0 || sel->dCols > cols || sel->dRows < 0 || sel->dRows > rows || sel->nnzRowD < 0 ||
        sel->nnzRowD > nnz || (sel->dCols > 0 && !descColId_dev) || (sel->dRows > 0 && !descRowId_dev) ||
        (nnz > 0 && (!colInd_dev || !val_dev || rows == 0 || cols == 0)) || (sel->nnzRowD > 0 && (!ddColInd_dev || !ddVal_dev)) ||
        (nnz - sel->nnzRowD > 0 && (!cdColInd_dev || !cdVal_dev))) {
        mx::set_error("mx_split_device: bad argument");
        return MX_ERR_ARG;
    }
    if (nnz > kMaxCount || rows > kMaxCount || cols > kMaxCount) {
        mx::set_error("mx_split_device: more than 2^31 - 513 entries, rows or columns");
        return MX_ERR_ARG;
    }
    hipStream_t s = (hipStream_t)stream;
    const int dCols = sel->dCols, dRows = sel->dRows, nDD = sel->nnzRowD;
    int colBits = 1, rowBits = 1;
    while (colBits < 31 && (1ll << colBits) < (long long)cols) ++colBits;
    while (rowBits < 31 && (1ll << rowBits) < (long long)rows) ++rowBits;
    const unsigned keyBits = (unsigned)(colBits + rowBits + 2);
    const size_t nScan = (size_t)std::max(rows, cols) + 1;
    size_t sortBytes = 0, scanBytes = 0;
    if (nnz > 0)
        MXP_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                          (const int *)nullptr, (int *)nullptr, (size_t)nnz, 0u, keyBits, s));
    MXP_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, nScan, rocprim::plus<int>(), s));
    sortBytes = (sortBytes + 255) & ~(size_t)255;
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    const size_t colB = al(((size_t)cols + 1) * sizeof(int)), rowB = al(((size_t)rows + 1) * sizeof(int));
    const size_t denseB = al((size_t)cols + 1), keyB = al((size_t)nnz * 8), payB = al((size_t)nnz * 4);
    // newCol, notSel, pos [cols+1]; rowRank, rcnt, cdLen, ddLen [rows+1]; dense; keys and payloads in and out
    Scratch scratch;
    MXP_TRY(hipMalloc(&scratch.p, 3 * colB + 4 * rowB + denseB + 2 * keyB + 2 * payB + sortBytes + scanBytes + 256));
    unsigned char *b = (unsigned char *)scratch.p;
    int *newCol = (int *)b, *notSel = (int *)(b + colB), *pos = (int *)(b + 2 * colB);
    b += 3 * colB;
    int *rowRank = (int *)b, *rcnt = (int *)(b + rowB), *cdLen = (int *)(b + 2 * rowB), *ddLen = (int *)(b + 3 * rowB);
    b += 4 * rowB;
    unsigned char *dense = b;
    b += denseB;
    unsigned long long *keyIn = (unsigned long long *)b, *keyOut = (unsigned long long *)(b + keyB);
    b += 2 * keyB;
    int *payIn = (int *)b, *payOut = (int *)(b + payB);
    b += 2 * payB;
    void *sortTmp = b, *scanTmp = b + sortBytes;
    int *bad = (int *)((unsigned char *)sortTmp + sortBytes + scanBytes);  // in the 256 spare bytes at the end
    auto grid = [](long long n) { return dim3((unsigned)((n + kBlock - 1) / kBlock)); };

    // the caller's arrays become addresses below: row pointers, column ids and both orders are
    // looked at first (1 = rowPtr, 2 = colInd, 4 = descColId, 8 = descRowId)
    MXP_TRY(hipMemsetAsync(bad, 0, sizeof(int), s));
    hipLaunchKernelGGL(pointer_check_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, rowPtr_dev, rows, nnz, 1, bad);
    if (nnz > 0) hipLaunchKernelGGL(range_check_kernel, grid(nnz), dim3(kBlock), 0, s, colInd_dev, nnz, cols, 2, bad);
    if (dCols > 0) hipLaunchKernelGGL(range_check_kernel, grid(dCols), dim3(kBlock), 0, s, descColId_dev, dCols, cols, 4, bad);
    if (dRows > 0) hipLaunchKernelGGL(range_check_kernel, grid(dRows), dim3(kBlock), 0, s, descRowId_dev, dRows, rows, 8, bad);
    MXP_TRY(hipGetLastError());
    {
        int badHost = 0;
        MXP_TRY(hipMemcpyAsync(&badHost, bad, sizeof(int), hipMemcpyDeviceToHost, s));
        MXP_TRY(hipStreamSynchronize(s));
        if (badHost) {
            mx::set_error(std::string("mx_split_device: ") + ((badHost & 1) ? "rowPtr does not rise from 0 to nnz" :
                          (badHost & 2) ? "column index out of range" : (badHost & 4) ? "descColId entry out of range" :
                          "descRowId entry out of range"));
            return MX_ERR_ARG;
        }
    }

    // new column ids: rank for a selected column, dCols + position among the others otherwise
    MXP_TRY(hipMemsetAsync(dense, 0, denseB, s));
    MXP_TRY(hipMemsetAsync(rowRank, 0xff, rowB, s));  // -1
    MXP_TRY(hipMemsetAsync(rcnt, 0, rowB, s));
    if (dCols > 0) {
        hipLaunchKernelGGL(mark_selected_kernel, grid(dCols), dim3(kBlock), 0, s, descColId_dev, dCols, dense);
        hipLaunchKernelGGL(scatter_rank_kernel, grid(dCols), dim3(kBlock), 0, s, descColId_dev, dCols, newCol);
    }
    hipLaunchKernelGGL(not_selected_kernel, grid((long long)cols + 1), dim3(kBlock), 0, s, (const unsigned char *)dense, cols, notSel);
    MXP_TRY(hipGetLastError());
    MXP_TRY(rocprim::exclusive_scan(scanTmp, scanBytes, (const int *)notSel, pos, 0, (size_t)cols + 1, rocprim::plus<int>(), s));
    if (cols > 0)
        hipLaunchKernelGGL(sparse_columns_kernel, grid(cols), dim3(kBlock), 0, s, (const unsigned char *)dense, (const int *)pos, cols,
                           dCols, newCol);
    // rows: rank of the selected ones, counts inside the selected columns, lengths, pointers
    if (dRows > 0) hipLaunchKernelGGL(scatter_rank_kernel, grid(dRows), dim3(kBlock), 0, s, descRowId_dev, dRows, rowRank);
    if (nnz > 0)
        hipLaunchKernelGGL(dense_row_counts_kernel, grid(nnz), dim3(kBlock), 0, s, rowPtr_dev, colInd_dev,
                           (const unsigned char *)dense, rows, nnz, rcnt);
    hipLaunchKernelGGL(split_lengths_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, rowPtr_dev, (const int *)rcnt,
                       (const int *)rowRank, descRowId_dev, rows, dRows, cdLen, ddLen);
    MXP_TRY(hipGetLastError());
    MXP_TRY(rocprim::exclusive_scan(scanTmp, scanBytes, (const int *)cdLen, cdRowPtr_dev, 0, (size_t)rows + 1, rocprim::plus<int>(), s));
    MXP_TRY(rocprim::exclusive_scan(scanTmp, scanBytes, (const int *)ddLen, ddRowPtr_dev, 0, (size_t)dRows + 1, rocprim::plus<int>(), s));
    if (nnz > 0) {
        hipLaunchKernelGGL(split_keys_kernel, grid(nnz), dim3(kBlock), 0, s, rowPtr_dev, colInd_dev, (const int *)newCol,
                           (const int *)rowRank, rows, nnz, dCols, colBits, rowBits, keyIn, payIn);
        MXP_TRY(hipGetLastError());
        MXP_TRY(rocprim::radix_sort_pairs(sortTmp, sortBytes, (const unsigned long long *)keyIn, keyOut, (const int *)payIn, payOut,
                                          (size_t)nnz, 0u, keyBits, s));
        if (dtype == MX_F64)
            hipLaunchKernelGGL(split_gather_kernel<double>, grid(nnz), dim3(kBlock), 0, s, (const unsigned long long *)keyOut,
                               (const int *)payOut, (const double *)val_dev, nnz, nDD, colBits, ddColInd_dev, (double *)ddVal_dev,
                               cdColInd_dev, (double *)cdVal_dev);
        else
            hipLaunchKernelGGL(split_gather_kernel<uint16_t>, grid(nnz), dim3(kBlock), 0, s, (const unsigned long long *)keyOut,
                               (const int *)payOut, (const uint16_t *)val_dev, nnz, nDD, colBits, ddColInd_dev,
                               (uint16_t *)ddVal_dev, cdColInd_dev, (uint16_t *)cdVal_dev);
        MXP_TRY(hipGetLastError());
    }
    // the totals must be what the caller sized the outputs for
    int totals[2] = {0, 0};
    MXP_TRY(hipMemcpyAsync(&totals[0], ddRowPtr_dev + dRows, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipMemcpyAsync(&totals[1], cdRowPtr_dev + rows, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));
    if (totals[0] != nDD || totals[1] != nnz - nDD) {
        mx::set_error("mx_split_device: the selection does not belong to this matrix (entry totals differ)");
        return MX_ERR_ARG;
    }
    return MX_OK;
}


extern "C" void mx_tiles_device_free(mx_device_tiles *t)
{
    if (!t) return;
    if (t->base) (void)hipFree(t->base);
    *t = mx_device_tiles{};
}

extern "C" int mx_tiles_device(mx_dtype dtype, int dRows, int dCols, int nnzRowD, const int *ddRowPtr_dev,
                               const int *ddColInd_dev, const void *ddVal_dev, mx_device_tiles *out, void *stream)
{
    static const char who[] = "mx_tiles_device";
    using namespace mxp;
    if ((dtype != MX_F64 && dtype != MX_F16) || dRows < 0 || dCols < 0 || nnzRowD < 0 || !out || !ddRowPtr_dev ||
        (nnzRowD > 0 && (!ddColInd_dev || !ddVal_dev || dRows == 0 || dCols == 0))) {
        mx::set_error("mx_tiles_device: bad argument");
        return MX_ERR_ARG;
    }
    if (nnzRowD > kMaxCount || dRows > kMaxCount || dCols > kMaxCount) {
        mx::set_error("mx_tiles_device: more than 2^31 - 513 entries, rows or columns");
        return MX_ERR_ARG;
    }
    hipStream_t s = (hipStream_t)stream;
    *out = mx_device_tiles{};
    const int fragK = mx::frag_k(dtype), n = nnzRowD, chunkNum = (dRows + mx::kFragM - 1) / mx::kFragM;
    const size_t es = (size_t)mx::elem_size(dtype);
    int colBits = 1, chunkBits = 1;
    while (colBits < 31 && (1ll << colBits) < (long long)dCols) ++colBits;
    while (chunkBits < 31 && (1ll << chunkBits) < (long long)chunkNum) ++chunkBits;
    const unsigned keyBits = (unsigned)(colBits + chunkBits);
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    auto grid = [](long long m) { return dim3((unsigned)((m + kBlock - 1) / kBlock)); };
    size_t sortBytes = 0, scanBytes = 0;
    if (n > 0)
        MXP_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                          (const int *)nullptr, (int *)nullptr, (size_t)n, 0u, keyBits, s));
    MXP_TRY(rocprim::inclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr,
                                    (size_t)std::max(n, chunkNum) + 1, rocprim::plus<int>(), s));
    {   // the exclusive form may ask for a different amount: take the larger
        size_t b2 = 0;
        MXP_TRY(rocprim::exclusive_scan(nullptr, b2, (const int *)nullptr, (int *)nullptr, 0, (size_t)std::max(n, chunkNum) + 1,
                                        rocprim::plus<int>(), s));
        scanBytes = std::max(scanBytes, b2);
    }
    sortBytes = al(sortBytes);
    scanBytes = al(scanBytes);
    // scratch: keys and payloads in and out, heads, their running count, ecr, per-chunk fragments
    const size_t keyB = al((size_t)n * 8), intB = al(((size_t)n + 1) * 4), chB = al(((size_t)chunkNum + 1) * 4);
    Scratch scratch;
    MXP_TRY(hipMalloc(&scratch.p, 2 * keyB + 5 * intB + 2 * chB + sortBytes + scanBytes + 256));
    unsigned char *b = (unsigned char *)scratch.p;
    unsigned long long *keyIn = (unsigned long long *)b, *keyOut = (unsigned long long *)(b + keyB);
    b += 2 * keyB;
    int *payIn = (int *)b, *payOut = (int *)(b + intB), *head = (int *)(b + 2 * intB), *run = (int *)(b + 3 * intB),
        *ecr = (int *)(b + 4 * intB);
    b += 5 * intB;
    int *frags = (int *)b, *chunkPtrTmp = (int *)(b + chB);
    b += 2 * chB;
    void *sortTmp = b, *scanTmp = b + sortBytes;
    {
        // the caller's A_dd is about to be used for addressing: pointers and column ids are looked at first
        int *bad = (int *)((unsigned char *)sortTmp + sortBytes + scanBytes);  // in the 256 spare bytes at the end
        MXP_TRY(hipMemsetAsync(bad, 0, sizeof(int), s));
        hipLaunchKernelGGL(pointer_check_kernel, grid((long long)dRows + 1), dim3(kBlock), 0, s, ddRowPtr_dev, dRows, n, 1, bad);
        if (n > 0) hipLaunchKernelGGL(range_check_kernel, grid(n), dim3(kBlock), 0, s, ddColInd_dev, n, dCols, 2, bad);
        MXP_TRY(hipGetLastError());
        int badHost = 0;
        MXP_TRY(hipMemcpyAsync(&badHost, bad, sizeof(int), hipMemcpyDeviceToHost, s));
        MXP_TRY(hipStreamSynchronize(s));
        if (badHost) {
            mx::set_error((badHost & 1) ? "mx_tiles_device: ddRowPtr does not rise from 0 to nnzRowD"
                                        : "mx_tiles_device: column index out of range");
            return MX_ERR_ARG;
        }
    }

    // distinct columns per chunk: sort by (chunk, column), mark first occurrences, count them
    if (n > 0) {
        hipLaunchKernelGGL(tile_keys_kernel, grid(n), dim3(kBlock), 0, s, ddRowPtr_dev, ddColInd_dev, dRows, n, colBits, keyIn, payIn);
        MXP_TRY(hipGetLastError());
        MXP_TRY(rocprim::radix_sort_pairs(sortTmp, sortBytes, (const unsigned long long *)keyIn, keyOut, (const int *)payIn, payOut,
                                          (size_t)n, 0u, keyBits, s));
        hipLaunchKernelGGL(tile_heads_kernel, grid(n), dim3(kBlock), 0, s, (const unsigned long long *)keyOut, n, head);
        MXP_TRY(hipGetLastError());
        MXP_TRY(rocprim::inclusive_scan(scanTmp, scanBytes, (const int *)head, run, (size_t)n, rocprim::plus<int>(), s));
    }
    hipLaunchKernelGGL(tile_chunk_frags_kernel, grid((long long)chunkNum + 1), dim3(kBlock), 0, s, ddRowPtr_dev, (const int *)run,
                       dRows, chunkNum, fragK, frags);
    MXP_TRY(hipGetLastError());
    // chunkPtr lives in the output block, whose size needs the total first
    MXP_TRY(rocprim::exclusive_scan(scanTmp, scanBytes, (const int *)frags, chunkPtrTmp, 0, (size_t)chunkNum + 1, rocprim::plus<int>(), s));
    int totalTcFrags = 0;
    MXP_TRY(hipMemcpyAsync(&totalTcFrags, chunkPtrTmp + chunkNum, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));

    // output block: chunkPtr, sparse_AToX_index, fragPtr, fragBit (64-bit while it is built), tcVal (at most n)
    const size_t cpB = al(((size_t)chunkNum + 1) * 4), axB = al((size_t)totalTcFrags * fragK * 4 + 4),
                 fpB = al(((size_t)totalTcFrags + 1) * 4), fbB = al((size_t)totalTcFrags * 8 + 8), tvB = al((size_t)n * es + 8);
    Scratch outBlock;
    MXP_TRY(hipMalloc(&outBlock.p, cpB + axB + fpB + fbB + tvB));
    unsigned char *o = (unsigned char *)outBlock.p;
    int *chunkPtr = (int *)o, *atox = (int *)(o + cpB), *fragPtr = (int *)(o + cpB + axB);
    unsigned long long *bits = (unsigned long long *)(o + cpB + axB + fpB);
    void *tcVal = o + cpB + axB + fpB + fbB;
    MXP_TRY(hipMemcpyAsync(chunkPtr, chunkPtrTmp, ((size_t)chunkNum + 1) * 4, hipMemcpyDeviceToDevice, s));
    MXP_TRY(hipMemsetAsync(atox, 0, axB + fpB + fbB, s));  // padding of the column lists is zero (:1380-1404)
    if (n > 0) {
        hipLaunchKernelGGL(tile_rank_kernel, grid(n), dim3(kBlock), 0, s, (const unsigned long long *)keyOut, (const int *)payOut,
                           (const int *)head, (const int *)run, ddRowPtr_dev, (const int *)chunkPtr, dRows, n, colBits, fragK, ecr,
                           atox, bits);
        MXP_TRY(hipGetLastError());
    }
    // fragPtr: running count of the set bits.  head[] is free again and long enough only when
    // totalTcFrags <= n, which holds (every fragment has an entry) -- but take no chances:
    if (totalTcFrags > n) {
        mx::set_error("mx_tiles_device: more fragments than entries (ddRowPtr is not A_dd's)");
        return MX_ERR_ARG;
    }
    hipLaunchKernelGGL(tile_popcount_kernel, grid((long long)totalTcFrags + 1), dim3(kBlock), 0, s, (const unsigned long long *)bits,
                       totalTcFrags, head);
    MXP_TRY(hipGetLastError());
    MXP_TRY(rocprim::exclusive_scan(scanTmp, scanBytes, (const int *)head, fragPtr, 0, (size_t)totalTcFrags + 1, rocprim::plus<int>(), s));
    if (n > 0) {
        if (dtype == MX_F64)
            hipLaunchKernelGGL(tile_values_kernel<double>, grid(n), dim3(kBlock), 0, s, ddRowPtr_dev, ddColInd_dev,
                               (const double *)ddVal_dev, (const int *)ecr, (const int *)chunkPtr, (const int *)fragPtr,
                               (const unsigned long long *)bits, dRows, n, fragK, (double *)tcVal);
        else
            hipLaunchKernelGGL(tile_values_kernel<uint16_t>, grid(n), dim3(kBlock), 0, s, ddRowPtr_dev, ddColInd_dev,
                               (const uint16_t *)ddVal_dev, (const int *)ecr, (const int *)chunkPtr, (const int *)fragPtr,
                               (const unsigned long long *)bits, dRows, n, fragK, (uint16_t *)tcVal);
        MXP_TRY(hipGetLastError());
    }
    if (dtype == MX_F64 && totalTcFrags > 0) {  // 8 x 4 bits: the reference keeps them in 32-bit words
        // narrowed in place, front to back: word f of the narrow form lies below word f of the wide one,
        // but another thread may still need it -- go through the free scratch instead
        hipLaunchKernelGGL(narrow_bits_kernel, grid(totalTcFrags), dim3(kBlock), 0, s, (const unsigned long long *)bits, totalTcFrags,
                           (unsigned *)run);
        MXP_TRY(hipGetLastError());
        MXP_TRY(hipMemcpyAsync(bits, run, (size_t)totalTcFrags * 4, hipMemcpyDeviceToDevice, s));
    }
    int tcValCount = 0;
    MXP_TRY(hipMemcpyAsync(&tcValCount, fragPtr + totalTcFrags, sizeof(int), hipMemcpyDeviceToHost, s));
    MXP_TRY(hipStreamSynchronize(s));
    out->chunkNum = chunkNum;
    out->totalTcFrags = totalTcFrags;
    out->fragK = fragK;
    out->tcValCount = tcValCount;
    out->chunkPtr = chunkPtr;
    out->sparse_AToX_index = atox;
    out->fragPtr = fragPtr;
    out->fragBit = bits;
    out->tcVal = tcVal;
    out->base = outBlock.p;
    outBlock.p = nullptr;  // the caller's now
    return MX_OK;
}


// mx_partition_create with the extraction done on the device: the matrix is uploaded, selected,
// split and encoded there (mx_select_device, mx_split_device, mx_tiles_device) and the arrays come
// back into the same host structure, so that everything downstream (plans, files, the checksum)
// cannot tell the two routes apart.
// The device arrays of a partition made here (mx_partition::twin) and their way down.
namespace {
void twin_free(void *w)
{
    mx::PartitionTwin *W = (mx::PartitionTwin *)w;
    if (!W) return;
    (void)hipFree(W->order);
    (void)hipFree(W->split);
    mx_tiles_device_free(&W->T);
    delete W;
}
// fills the host vectors of P from its twin
int twin_download(mx_partition *P)
{
    using namespace mxp;
    static const char who[] = "mx_partition_create_device (arrays to the host)";
    const mx::PartitionTwin &W = *(const mx::PartitionTwin *)P->twin;
    const int rows = W.rows, cols = W.cols, nDD = W.nDD, nCD = W.nCD, dRows = W.dRows, dCols = W.dCols;
    const size_t es = (size_t)mx::elem_size(W.dtype);
    const mx_device_tiles &T = W.T;
    try {
        P->descColId.resize(cols);
        P->rId.resize(dRows);
        P->ddRowPtr.resize((size_t)dRows + 1);
        P->ddColInd.resize(nDD);
        P->ddVal.resize(nDD, (int)es);
        P->cdRowPtr.resize((size_t)rows + 1);
        P->cdColInd.resize(nCD);
        P->cdVal.resize(nCD, (int)es);
        P->chunkPtr.resize((size_t)T.chunkNum + 1);
        P->sparse_AToX_index.resize((size_t)T.totalTcFrags * T.fragK);
        P->fragPtr.resize((size_t)T.totalTcFrags + 1);
        if (W.dtype == MX_F64) P->fragBit32.resize(T.totalTcFrags);
        else P->fragBit64.resize(T.totalTcFrags);
        P->tcVal.resize(T.tcValCount, (int)es);
    } catch (const std::bad_alloc &) {
        mx::set_error("mx_partition_create_device: out of memory");
        return MX_ERR_ALLOC;
    }
    auto down = [](void *dst, const void *src, size_t bytes) {
        return bytes ? hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost) : hipSuccess;
    };
    MXP_TRY(down(P->descColId.data(), W.dc, (size_t)cols * 4));
    MXP_TRY(down(P->rId.data(), W.dr, (size_t)dRows * 4));
    MXP_TRY(down(P->ddRowPtr.data(), W.ddp, ((size_t)dRows + 1) * 4));
    MXP_TRY(down(P->ddColInd.data(), W.ddc, (size_t)nDD * 4));
    MXP_TRY(down(P->ddVal.data(), W.ddv, (size_t)nDD * es));
    MXP_TRY(down(P->cdRowPtr.data(), W.cdp, ((size_t)rows + 1) * 4));
    MXP_TRY(down(P->cdColInd.data(), W.cdc, (size_t)nCD * 4));
    MXP_TRY(down(P->cdVal.data(), W.cdv, (size_t)nCD * es));
    MXP_TRY(down(P->chunkPtr.data(), T.chunkPtr, ((size_t)T.chunkNum + 1) * 4));
    MXP_TRY(down(P->sparse_AToX_index.data(), T.sparse_AToX_index, (size_t)T.totalTcFrags * T.fragK * 4));
    MXP_TRY(down(P->fragPtr.data(), T.fragPtr, ((size_t)T.totalTcFrags + 1) * 4));
    if (W.dtype == MX_F64) MXP_TRY(down(P->fragBit32.data(), T.fragBit, (size_t)T.totalTcFrags * 4));
    else MXP_TRY(down(P->fragBit64.data(), T.fragBit, (size_t)T.totalTcFrags * 8));
    MXP_TRY(down(P->tcVal.data(), T.tcVal, (size_t)T.tcValCount * es));
    // the lists of what was not selected, ascending (test/test_autotc_spmv.cpp:1143-1160, :1261-1277)
    std::vector<unsigned char> taken((size_t)std::max(rows, cols), 0);
    for (int i = 0; i < dCols; ++i) taken[P->descColId[i]] = 1;
    P->newArray.clear();
    P->newArray.reserve(P->sCols);
    for (int c = 0; c < cols; ++c)
        if (!taken[c]) P->newArray.push_back(c);
    std::fill(taken.begin(), taken.end(), 0);
    for (int i = 0; i < dRows; ++i) taken[P->rId[i]] = 1;
    P->newArray_.clear();
    P->newArray_.reserve(P->sRows);
    for (int r = 0; r < rows; ++r)
        if (!taken[r]) P->newArray_.push_back(r);
    P->host_ready = true;
    return MX_OK;
}
}  // namespace

extern "C" int mx_partition_create_device(const mx_csr *A, float tau_c, float tau_r, mx_partition **out)
{
    static const char who[] = "mx_partition_create_device";
    using namespace mxp;
    const int ok = mx::check_partition_args(A, tau_c, tau_r, out);
    if (ok != MX_OK) return ok;
    if (tau_c == 0.0f && tau_r == 0.0f) return mx_partition_create(A, tau_c, tau_r, out);  // nothing to extract
    int ndev = 0;
    if (hipGetDeviceCount(&ndev) != hipSuccess || ndev < 1) {
        mx::set_error("mx_partition_create_device: no HIP device");
        return MX_ERR_DEVICE;
    }
    (void)who;
    const int rows = A->rows, cols = A->cols, nnz = A->nnz;
    const size_t es = (size_t)mx::elem_size(A->dtype);
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    mx::PartitionTwin *W = new (std::nothrow) mx::PartitionTwin();
    if (!W) {
        mx::set_error("mx_partition_create_device: out of memory");
        return MX_ERR_ALLOC;
    }
    struct TwinGuard {
        mx::PartitionTwin *w;
        ~TwinGuard() { twin_free(w); }
    } wg{W};
    W->dtype = A->dtype;
    W->rows = rows;
    W->cols = cols;
    W->nnz = nnz;
    // the matrix (released when the extraction is done) and the two orders (kept)
    const size_t rpB = al(((size_t)rows + 1) * 4), ciB = al((size_t)nnz * 4 + 4), vaB = al((size_t)nnz * es + 8),
                 dcB = al((size_t)cols * 4 + 4), drB = al((size_t)rows * 4 + 4);
    Scratch in;
    MXP_TRY(hipMalloc(&in.p, rpB + ciB + vaB));
    unsigned char *b = (unsigned char *)in.p;
    int *rp = (int *)b, *ci = (int *)(b + rpB);
    void *va = b + rpB + ciB;
    MXP_TRY(hipMalloc(&W->order, dcB + drB));
    W->dc = (int *)W->order;
    W->dr = (int *)((unsigned char *)W->order + dcB);
    int *dc = W->dc, *dr = W->dr;
    MXP_TRY(hipMemcpy(rp, A->rowPtr, ((size_t)rows + 1) * 4, hipMemcpyHostToDevice));
    if (nnz > 0) {
        MXP_TRY(hipMemcpy(ci, A->colInd, (size_t)nnz * 4, hipMemcpyHostToDevice));
        MXP_TRY(hipMemcpy(va, A->val, (size_t)nnz * es, hipMemcpyHostToDevice));
    }
    mx_selection sel{};
    int rc = mx_select_device(rows, cols, nnz, rp, ci, tau_c, tau_r, dc, dr, &sel, nullptr);
    if (rc != MX_OK) return rc;
    const int nDD = sel.nnzRowD, nCD = nnz - nDD;
    const size_t ddpB = al(((size_t)sel.dRows + 1) * 4), ddcB = al((size_t)nDD * 4 + 4), ddvB = al((size_t)nDD * es + 8),
                 cdpB = al(((size_t)rows + 1) * 4), cdcB = al((size_t)nCD * 4 + 4), cdvB = al((size_t)nCD * es + 8);
    MXP_TRY(hipMalloc(&W->split, ddpB + ddcB + ddvB + cdpB + cdcB + cdvB));
    b = (unsigned char *)W->split;
    W->ddp = (int *)b;
    W->ddc = (int *)(b + ddpB);
    W->ddv = b + ddpB + ddcB;
    W->cdp = (int *)(b + ddpB + ddcB + ddvB);
    W->cdc = (int *)(b + ddpB + ddcB + ddvB + cdpB);
    W->cdv = b + ddpB + ddcB + ddvB + cdpB + cdcB;
    rc = mx_split_device(A->dtype, rows, cols, nnz, rp, ci, va, &sel, dc, dr, W->ddp, W->ddc, W->ddv, W->cdp, W->cdc, W->cdv, nullptr);
    if (rc != MX_OK) return rc;
    rc = mx_tiles_device(A->dtype, sel.dRows, sel.dCols, nDD, W->ddp, W->ddc, W->ddv, &W->T, nullptr);
    if (rc != MX_OK) return rc;
    W->dRows = sel.dRows;
    W->dCols = sel.dCols;
    W->nDD = nDD;
    W->nCD = nCD;
    const mx_device_tiles &T = W->T;

    mx_partition *P = new (std::nothrow) mx_partition();
    if (!P) {
        mx::set_error("mx_partition_create_device: out of memory");
        return MX_ERR_ALLOC;
    }
    // the counts; the arrays stay on the device until somebody asks for them (mx::partition_host)
    P->dtype = A->dtype;
    P->rows = rows;
    P->cols = cols;
    P->nnz = nnz;
    P->fragM = mx::kFragM;
    P->fragK = mx::frag_k(A->dtype);
    P->tau_c = tau_c;
    P->tau_r = tau_r;
    P->extracted = true;
    P->dCols = sel.dCols;
    P->sCols = cols - sel.dCols;
    P->nnzColD = sel.nnzColD;
    P->nnzColS = nnz - sel.nnzColD;
    P->cols_ratio = (float)sel.dCols / (float)cols;
    P->dRows = sel.dRows;
    P->sRows = rows - sel.dRows;
    P->nnzRowD = nDD;
    P->nnzRowS = sel.nnzColD - nDD;
    P->nnzCD = nCD;
    P->chunkNum = T.chunkNum;
    P->totalTcFrags = T.totalTcFrags;
    P->tcValCount = T.tcValCount;
    P->tc_nnz_ratio = (double)nDD / ((double)T.totalTcFrags * mx::kFragM * P->fragK);
    P->host_ready = false;
    P->twin = W;
    P->twin_download = twin_download;
    P->twin_free = twin_free;
    wg.w = nullptr;  // the partition owns the twin now
    *out = P;
    return MX_OK;
}
