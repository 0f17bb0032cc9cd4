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

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/device/device_scan.hpp>

#include "mx_internal.h"

namespace mxp {

constexpr int kBlock = 256;

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
    const int e = blockIdx.x * kBlock + threadIdx.x;
    if (e >= nnz) return;
    if (dense[col[e]]) atomicAdd(&rcnt[line_of(rowPtr, rows, e)], 1);
}

struct Scratch {
    void *p = nullptr;
    ~Scratch()
    {
        if (p) (void)hipFree(p);
    }
};

}  // namespace mxp

#define MXP_TRY(call)                                                                                      \
    do {                                                                                                   \
        hipError_t e_ = (call);                                                                            \
        if (e_ != hipSuccess) {                                                                            \
            mx::set_error(std::string("mx_transpose_device: ") + #call + ": " + hipGetErrorString(e_));   \
            return e_ == hipErrorOutOfMemory ? MX_ERR_ALLOC : MX_ERR_DEVICE;                                  \
        }                                                                                                  \
    } while (0)

extern "C" int mx_transpose_device(mx_dtype dtype, int outer, int inner, int nnz, const int *ptr_dev, const int *ind_dev,
                                   const void *val_dev, int *tPtr_dev, int *tInd_dev, void *tVal_dev, void *stream)
{
    using namespace mxp;
    if ((dtype != MX_F64 && dtype != MX_F16) || outer < 0 || inner < 0 || nnz < 0 || !ptr_dev || !tPtr_dev ||
        (nnz > 0 && (!ind_dev || !val_dev || !tInd_dev || !tVal_dev || outer == 0))) {
        mx::set_error("mx_transpose_device: bad argument");
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

#undef MXP_TRY
#define MXP_TRY(call)                                                                                    \
    do {                                                                                                 \
        hipError_t e_ = (call);                                                                          \
        if (e_ != hipSuccess) {                                                                          \
            mx::set_error(std::string("mx_select_device: ") + #call + ": " + hipGetErrorString(e_));    \
            return e_ == hipErrorOutOfMemory ? MX_ERR_ALLOC : MX_ERR_DEVICE;                             \
        }                                                                                                \
    } while (0)

namespace mxp {

// order[0..n) = the lines by count descending, ties by ascending line (a stable descending sort
// of the counts with the line numbers as payload); then the prefix that reaches `target`.
// cnt, order: device arrays of n; work: 3 n ints + 4; returns the prefix length and its sum.
static int order_and_reach(const int *cnt, int n, int target, int *order, int *work, void *sortTmp, size_t sortBytes,
                           void *scanTmp, size_t scanBytes, hipStream_t s, int *len, int *sum)
{
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
    using namespace mxp;
    if (rows < 0 || cols < 0 || nnz < 0 || !rowPtr_dev || !out || (cols > 0 && !descColId_dev) ||
        (rows > 0 && !descRowId_dev) || (nnz > 0 && (!colInd_dev || rows == 0 || cols == 0)) || !(tau_c >= 0.f) ||
        !(tau_c <= 1.f) || !(tau_r >= 0.f) || !(tau_r <= tau_c)) {
        mx::set_error("mx_select_device: bad argument");
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
