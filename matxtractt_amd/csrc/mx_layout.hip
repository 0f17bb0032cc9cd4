// The slice layout of the CSR part (see DeviceSlices) built on the device from a CSR matrix that
// lives in device memory: the same arrays, byte for byte, as the host route (build_slices in
// mx_host_layout.cpp), for matrices that are already in HBM and for plans of large matrices, whose
// layout the host cores take a second to make.  The reference has no counterpart: its CSR
// kernel reads the CSR arrays as they are (src/spmv_kernel/cdSpMV.cu:407-418).
//
// What depends on every entry or every virtual row runs here: rows put in ascending column
// order (a stable sort by (row, column) when some row is not), virtual rows cut at slice borders
// and at the cap, their stable sort by (slice, length descending, kind of row), the entries
// placed into the lanes' streams, the lists the combine kernel walks.  What depends on chunks
// only (64 virtual rows each) -- which workgroup and wave streams which chunk -- is decided on the
// host by the routine both routes share (plan_slice_chunks), from the chunks' lengths.
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

namespace mxl {

constexpr int kBlock = 256;

struct Buf {  // device memory released at scope exit unless taken
    void *p = nullptr;
    Buf() = default;
    Buf(const Buf &) = delete;
    Buf &operator=(const Buf &) = delete;
    ~Buf() { release(); }
    void release()
    {
        if (p) (void)hipFree(p);
        p = nullptr;
    }
    template <typename T>
    T *as() const
    {
        return (T *)p;
    }
    void *take()
    {
        void *q = p;
        p = nullptr;
        return q;
    }
};

// The row of every entry, in two steps: every row that has entries writes its number at the place of
// its first entry (all other places hold 0), and a running maximum carries it to the rest of the row.
__global__ __launch_bounds__(kBlock) void row_heads_kernel(const int *__restrict__ rowPtr, int rows, int *__restrict__ head)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r < rows && rowPtr[r + 1] > rowPtr[r]) head[rowPtr[r]] = r;
}
// flag |= 1 when some row's columns are not ascending
__global__ __launch_bounds__(kBlock) void row_order_kernel(const int *__restrict__ rowPtr, const int *__restrict__ col,
                                                           const int *__restrict__ row, int nnz, int *__restrict__ flag)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    const bool descends = k < nnz && k > rowPtr[row[k]] && col[k] < col[k - 1];
    // (one atomic per wave at most, and none once the flag is up: a matrix whose rows are all out of order would
    // put one per entry on the same word, and half a million of them take four milliseconds)
    if (__any(descends) && (threadIdx.x & 63) == 0 && *(volatile int *)flag == 0) atomicOr(flag, 1);
}

__global__ __launch_bounds__(kBlock) void sort_keys_kernel(const int *__restrict__ row, const int *__restrict__ col, int nnz,
                                                           int colBits, unsigned long long *__restrict__ key, int *__restrict__ pay)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    key[k] = ((unsigned long long)(unsigned)row[k] << colBits) | (unsigned)col[k];
    pay[k] = k;
}

__global__ __launch_bounds__(kBlock) void iota_kernel(int *__restrict__ v, int n)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < n) v[k] = k;
}

// runHead[k] = k where a run of one (row, slice) starts at position k of the ordered entries, 0 elsewhere
__global__ __launch_bounds__(kBlock) void run_heads_kernel(const int *__restrict__ rowPtr, const int *__restrict__ row,
                                                           const int *__restrict__ col, const int *__restrict__ ord, int nnz,
                                                           int SW, int *__restrict__ runHead)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    const bool head = k == rowPtr[row[k]] || col[ord[k]] / SW != col[ord[k - 1]] / SW;
    runHead[k] = head ? k : 0;
}

struct MaxOp {
    __device__ __host__ int operator()(int a, int b) const { return a > b ? a : b; }
};

// start[k] = 1 where a virtual row starts: every cap-th position of a run
__global__ __launch_bounds__(kBlock) void vrow_starts_kernel(const int *__restrict__ runStart, int nnz, int cap, int *__restrict__ start)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < nnz) start[k] = ((k - runStart[k]) % cap == 0) ? 1 : 0;
}

// per virtual row: where it starts, its row and slice
__global__ __launch_bounds__(kBlock) void vrow_records_kernel(const int *__restrict__ start, const int *__restrict__ vid,
                                                              const int *__restrict__ row, const int *__restrict__ col,
                                                              const int *__restrict__ ord, int nnz, int SW, int *__restrict__ vStart,
                                                              int *__restrict__ vRow, int *__restrict__ vSlice)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz || !start[k]) return;
    const int t = vid[k];
    vStart[t] = k;
    vRow[t] = row[k];
    vSlice[t] = col[ord[k]] / SW;
}

// segPtr[r] = virtual rows before row r
__global__ __launch_bounds__(kBlock) void seg_ptr_kernel(const int *__restrict__ rowPtr, const int *__restrict__ vid, int rows, int nnz,
                                                         int nV, int *__restrict__ segPtr)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r > rows) return;
    const int p = r < rows ? rowPtr[r] : nnz;
    segPtr[r] = p < nnz ? vid[p] : nV;
}

// the sort key of every virtual row: (slice, cap - length, kind of its row)
__global__ __launch_bounds__(kBlock) void vrow_keys_kernel(const int *__restrict__ vStart, const int *__restrict__ vRow,
                                                           const int *__restrict__ vSlice, const int *__restrict__ segPtr, int nV,
                                                           int nnz, int cap, int lightSegs, unsigned *__restrict__ key,
                                                           int *__restrict__ pay, int *__restrict__ vLen)
{
    const int t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= nV) return;
    const int len = (t + 1 < nV ? vStart[t + 1] : nnz) - vStart[t];
    const int r = vRow[t], nv = segPtr[r + 1] - segPtr[r];
    const int kind = nv <= 1 ? 0 : nv <= lightSegs ? 1 : 2;
    key[t] = ((unsigned)vSlice[t] * (unsigned)(cap + 1) + (unsigned)(cap - len)) * 3u + (unsigned)kind;
    pay[t] = t;
    vLen[t] = len;
}

// sliceStart[q] = number of sorted keys that belong to slices before q, for q in [0, S]
__global__ __launch_bounds__(kBlock) void slice_starts_kernel(const unsigned *__restrict__ sortedKey, int nV, int S, unsigned perSlice,
                                                              int *__restrict__ sliceStart)
{
    const int q = blockIdx.x * kBlock + threadIdx.x;
    if (q > S) return;
    const unsigned long long want = (unsigned long long)q * perSlice;
    int lo = 0, hi = nV;
    while (lo < hi) {  // first position whose key is not below `want`
        const int mid = (lo + hi) >> 1;
        if ((unsigned long long)sortedKey[mid] < want) lo = mid + 1;
        else hi = mid;
    }
    sliceStart[q] = lo;
}

__global__ __launch_bounds__(kBlock) void gather_len_kernel(const int *__restrict__ sorted, const int *__restrict__ vLen,
                                                            const int *__restrict__ first, int n, int *__restrict__ out)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = vLen[sorted[first[i]]];
}

// segIdx[t] = 64 * chunk + lane of every virtual row
__global__ __launch_bounds__(kBlock) void vrow_places_kernel(const int *__restrict__ sorted, const int *__restrict__ chunkFirst,
                                                             const int *__restrict__ chunkN, long long chunks, int *__restrict__ segIdx)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    const long long c = i >> 6;
    const int l = (int)(i & 63);
    if (c >= chunks || l >= chunkN[c]) return;
    segIdx[sorted[chunkFirst[c] + l]] = (int)(c * 64 + l);
}

// every entry to its place in the streams (see DeviceSlices: lanes' column offsets of a batch
// contiguous, binary16 values likewise, binary64 values in sub-blocks of two per lane)
template <typename V>
__global__ __launch_bounds__(kBlock) void place_entries_kernel(const int *__restrict__ start, const int *__restrict__ vid,
                                                               const int *__restrict__ vStart, const int *__restrict__ vSlice,
                                                               const int *__restrict__ segIdx, const long long *__restrict__ chunkStep0,
                                                               const int *__restrict__ ord, const int *__restrict__ col,
                                                               const V *__restrict__ val, const unsigned char *__restrict__ code,
                                                               int nnz, int SW, unsigned short *__restrict__ ecol, V *__restrict__ eval,
                                                               unsigned char *__restrict__ ecode)
{
    constexpr int BE = mx::kSliceBatchEntries;
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    const int t = vid[k] + start[k] - 1;  // vid counts the starts before k
    const int place = segIdx[t], l = place & 63;
    const size_t st = (size_t)chunkStep0[place >> 6] + (size_t)(k - vStart[t]), batch = st / BE, j = st % BE;
    const size_t atc = (batch * 64 + l) * BE + j;
    const size_t atv = sizeof(V) == 8 ? batch * 64 * BE + (j / 2) * 128 + (size_t)l * 2 + j % 2 : atc;
    const int p = ord[k];
    ecol[atc] = (unsigned short)(col[p] - vSlice[t] * SW);
    eval[atv] = val[p];
    if (ecode) ecode[atc] = code[p];
}

// the padding of every virtual row up to its chunk's longest member names the row's own last column
__global__ __launch_bounds__(kBlock) void pad_columns_kernel(const int *__restrict__ vStart, const int *__restrict__ vLen,
                                                             const int *__restrict__ vSlice, const int *__restrict__ segIdx,
                                                             const long long *__restrict__ chunkStep0, const int *__restrict__ chunkSteps,
                                                             const int *__restrict__ ord, const int *__restrict__ col, int nV, int SW,
                                                             unsigned short *__restrict__ ecol)
{
    constexpr int BE = mx::kSliceBatchEntries;
    const int t = blockIdx.x * kBlock + threadIdx.x;
    if (t >= nV) return;
    const int len = vLen[t], place = segIdx[t], l = place & 63, c = place >> 6;
    if (len <= 0) return;
    const unsigned short last = (unsigned short)(col[ord[vStart[t] + len - 1]] - vSlice[t] * SW);
    for (int n = len; n < chunkSteps[c]; ++n) {
        const size_t st = (size_t)chunkStep0[c] + n, batch = st / BE, j = st % BE;
        ecol[(batch * 64 + l) * BE + j] = last;
    }
}

// rowInfo and the marks of the two lists (rows with 2..lightSegs virtual rows, rows with more)
__global__ __launch_bounds__(kBlock) void row_info_kernel(const int *__restrict__ segPtr, const int *__restrict__ segIdx,
                                                          const char *__restrict__ elsewhere, int rows, int lightSegs,
                                                          int *__restrict__ rowInfo, int *__restrict__ isLight, int *__restrict__ isHeavy,
                                                          int *__restrict__ over4, int *__restrict__ most)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    int n = 0;
    if (r < rows) {
        const int a = segPtr[r];
        n = segPtr[r + 1] - a;
        const int e = elsewhere ? elsewhere[r] : 0;
        const bool fetched = e == 2;
        rowInfo[r] = fetched ? -2 : n == 0 ? (e ? -2 : -1) : n == 1 ? segIdx[a] : -2;
        const bool listed = n > 1 && !fetched;
        isLight[r] = listed && n <= lightSegs;
        isHeavy[r] = listed && n > lightSegs;
        if (listed && n <= lightSegs && n > 4) atomicOr(over4, 1);
    } else if (r == rows) {  // the scans run over rows + 1 elements
        isLight[r] = isHeavy[r] = 0;
    }
    // the most virtual rows of any row: one atomic per wave
    int m = n;
    for (int off = 32; off > 0; off >>= 1) m = max(m, __shfl_xor(m, off));
    if ((threadIdx.x & 63) == 0 && m > 1) atomicMax(most, m);
}

__global__ __launch_bounds__(kBlock) void row_lists_kernel(const int *__restrict__ segPtr, const int *__restrict__ segIdx,
                                                           const int *__restrict__ isLight, const int *__restrict__ isHeavy,
                                                           const int *__restrict__ lightPos, const int *__restrict__ heavyPos, int rows,
                                                           int places, int *__restrict__ lightRow, int *__restrict__ lightIdx,
                                                           int *__restrict__ heavyInfo)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r >= rows) return;
    const int a = segPtr[r], n = segPtr[r + 1] - a;
    if (isLight[r]) {
        const int i = lightPos[r];
        lightRow[i] = r;
        for (int k = 0; k < n; ++k) lightIdx[(size_t)i * places + k] = segIdx[a + k];
    }
    if (isHeavy[r]) {
        const int i = heavyPos[r];
        heavyInfo[4 * (size_t)i] = r;
        heavyInfo[4 * (size_t)i + 1] = a;
        heavyInfo[4 * (size_t)i + 2] = n;
        heavyInfo[4 * (size_t)i + 3] = 0;
    }
}

// ---- value dictionary ----
template <typename V>
__global__ __launch_bounds__(kBlock) void value_keys_kernel(const V *__restrict__ val, int nnz, unsigned long long *__restrict__ key,
                                                            int *__restrict__ pay)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    unsigned long long b = 0;
    if constexpr (sizeof(V) == 8) b = __builtin_bit_cast(unsigned long long, val[k]);
    else b = __builtin_bit_cast(unsigned short, val[k]);
    key[k] = b;
    pay[k] = k;
}
__global__ __launch_bounds__(kBlock) void value_heads_kernel(const unsigned long long *__restrict__ key, int nnz, int *__restrict__ head)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < nnz) head[k] = (k == 0 || key[k] != key[k - 1]) ? 1 : 0;
}
// the distinct values (at most `most`) with the position of their first entry
__global__ __launch_bounds__(kBlock) void value_table_kernel(const unsigned long long *__restrict__ key, const int *__restrict__ pay,
                                                             const int *__restrict__ head, const int *__restrict__ rank, int nnz, int most,
                                                             unsigned long long *__restrict__ tabVal, int *__restrict__ tabFirst)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz || !head[k]) return;
    const int i = rank[k];
    if (i < most) {
        tabVal[i] = key[k];
        tabFirst[i] = pay[k];  // the sort is stable: the first of a run is the earliest entry with that value
    }
}
// code of every entry: the place of its value among the sorted distinct values, through codeOf
template <typename V>
__global__ __launch_bounds__(kBlock) void value_codes_kernel(const V *__restrict__ val, int nnz, const unsigned long long *__restrict__ tabVal,
                                                             const unsigned char *__restrict__ codeOf, int nd, unsigned char *__restrict__ code)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k >= nnz) return;
    unsigned long long b = 0;
    if constexpr (sizeof(V) == 8) b = __builtin_bit_cast(unsigned long long, val[k]);
    else b = __builtin_bit_cast(unsigned short, val[k]);
    int lo = 0, hi = nd - 1;
    while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if (tabVal[mid] < b) lo = mid + 1;
        else hi = mid;
    }
    code[k] = codeOf[lo];
}

// ---- statistics and the row-tile form from device arrays ----
// bad |= 1 unless rowPtr rises from 0 to nnz; bad |= 2 for a column outside [0, cols)
__global__ __launch_bounds__(kBlock) void check_csr_kernel(const int *__restrict__ rowPtr, const int *__restrict__ col, int rows, int cols,
                                                           int nnz, int *__restrict__ bad)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (i <= rows) {
        const int p = rowPtr[i];
        if ((i == 0 && p != 0) || (i == rows && p != nnz) || (i < rows && rowPtr[i + 1] < p) || p < 0 || p > nnz) atomicOr(bad, 1);
    }
    if (i < nnz && (unsigned)col[i] >= (unsigned)cols) atomicOr(bad, 2);
}
// sum += distinct 64-byte lines of x that the 64 entries of every stride-th window name (one thread per window)
__global__ __launch_bounds__(kBlock) void window_lines_kernel(const int *__restrict__ col, long long sampled, long long stride, int perLine,
                                                              unsigned long long *__restrict__ sum)
{
    const long long i = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (i >= sampled) return;
    const int *c = col + i * stride * 64;
    int d = 0;
    for (int a = 0; a < 64; ++a) {
        const int la = c[a] / perLine;
        bool seen = false;
        for (int b = 0; b < a && !seen; ++b) seen = c[b] / perLine == la;
        d += !seen;
    }
    atomicAdd(sum, (unsigned long long)d);
}
// one wave per workgroup of the row kernel: the lowest and the highest column of its entries
__global__ __launch_bounds__(kBlock) void block_ranges_kernel(const int4 *__restrict__ desc, const int *__restrict__ col, int nBlocks,
                                                              int *__restrict__ lo, int *__restrict__ wide)
{
    const int b = (blockIdx.x * kBlock + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (b >= nBlocks) return;
    const int4 d = desc[b];
    int mn = 0x7fffffff, mx_ = 0;
    for (int p = d.z + lane; p < d.w; p += 64) {
        mn = min(mn, col[p]);
        mx_ = max(mx_, col[p]);
    }
    for (int o = 32; o > 0; o >>= 1) {
        mn = min(mn, __shfl_xor(mn, o, 64));
        mx_ = max(mx_, __shfl_xor(mx_, o, 64));
    }
    if (lane == 0) {
        lo[b] = d.w > d.z ? mn : 0;
        if (d.w > d.z && mx_ - mn > 65535) atomicOr(wide, 1);
    }
}
__global__ __launch_bounds__(kBlock) void narrow_columns_kernel(const int4 *__restrict__ desc, const int *__restrict__ col,
                                                                const int *__restrict__ lo, int nBlocks, unsigned short *__restrict__ c16)
{
    const int b = (blockIdx.x * kBlock + threadIdx.x) >> 6, lane = threadIdx.x & 63;
    if (b >= nBlocks) return;
    const int4 d = desc[b];
    const int base = lo[b];
    for (int p = d.z + lane; p < d.w; p += 64) c16[p] = (unsigned short)(col[p] - base);
}

inline dim3 grid(long long n) { return dim3((unsigned)((std::max<long long>(n, 1) + kBlock - 1) / kBlock)); }

}  // namespace mxl

#define MXL_TRY(call)                                                                                 \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            mx::set_error(std::string("slice layout on the device: ") + #call + ": " + hipGetErrorString(e_)); \
            return e_ == hipErrorOutOfMemory ? MX_ERR_ALLOC : MX_ERR_DEVICE;                          \
        }                                                                                             \
    } while (0)

namespace mx {

// The value dictionary of a matrix in device memory, as make_value_dict gives it on the host: at
// most 255 distinct bit patterns, numbered in the order of their first entry; codes[nnz] (device)
// and dict (256 values, host, zero-padded).  *nDict = 0 when the matrix has more.
template <typename V>
static int device_value_dict(const V *val, int nnz, mxl::Buf &codes, std::vector<unsigned char> &dict, int *nDict, hipStream_t s,
                             int most = 255, size_t codePad = 0)
{
    using namespace mxl;
    *nDict = 0;
    {
        // most matrices have thousands of distinct values among their first entries: look there first
        const int sample = std::min(nnz, 16384);
        std::vector<V> h((size_t)sample);
        MXL_TRY(hipMemcpyAsync(h.data(), val, (size_t)sample * sizeof(V), hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        std::vector<unsigned long long> b((size_t)sample);
        for (int i = 0; i < sample; ++i) {
            if constexpr (sizeof(V) == 8) std::memcpy(&b[i], &h[i], 8);
            else {
                unsigned short u;
                std::memcpy(&u, &h[i], 2);
                b[i] = u;
            }
        }
        std::sort(b.begin(), b.end());
        if (std::unique(b.begin(), b.end()) - b.begin() > most) return MX_OK;
    }
    Buf keyIn, keyOut, payIn, payOut, head, rank, tabVal, tabFirst, tmp;
    size_t sortBytes = 0, scanBytes = 0;
    const unsigned bits = sizeof(V) == 8 ? 64u : 16u;
    MXL_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                      (const int *)nullptr, (int *)nullptr, (size_t)nnz, 0u, bits, s));
    MXL_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, (size_t)nnz, rocprim::plus<int>(), s));
    MXL_TRY(hipMalloc(&keyIn.p, (size_t)nnz * 8));
    MXL_TRY(hipMalloc(&keyOut.p, (size_t)nnz * 8));
    MXL_TRY(hipMalloc(&payIn.p, (size_t)nnz * 4));
    MXL_TRY(hipMalloc(&payOut.p, (size_t)nnz * 4));
    MXL_TRY(hipMalloc(&head.p, (size_t)nnz * 4));
    MXL_TRY(hipMalloc(&rank.p, (size_t)nnz * 4));
    MXL_TRY(hipMalloc(&tabVal.p, 256 * 8));
    MXL_TRY(hipMalloc(&tabFirst.p, 256 * 4));
    MXL_TRY(hipMalloc(&tmp.p, std::max(sortBytes, scanBytes) + 256));
    hipLaunchKernelGGL(value_keys_kernel<V>, grid(nnz), dim3(kBlock), 0, s, val, nnz, keyIn.as<unsigned long long>(), payIn.as<int>());
    MXL_TRY(hipGetLastError());
    MXL_TRY(rocprim::radix_sort_pairs(tmp.p, sortBytes, (const unsigned long long *)keyIn.p, keyOut.as<unsigned long long>(),
                                      (const int *)payIn.p, payOut.as<int>(), (size_t)nnz, 0u, bits, s));
    hipLaunchKernelGGL(value_heads_kernel, grid(nnz), dim3(kBlock), 0, s, (const unsigned long long *)keyOut.p, nnz, head.as<int>());
    MXL_TRY(hipGetLastError());
    MXL_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)head.p, rank.as<int>(), 0, (size_t)nnz, rocprim::plus<int>(), s));
    int lastRank = 0, lastHead = 0;
    MXL_TRY(hipMemcpyAsync(&lastRank, rank.as<int>() + (nnz - 1), 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipMemcpyAsync(&lastHead, head.as<int>() + (nnz - 1), 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    const int nd = lastRank + lastHead;
    if (nd > most) return MX_OK;
    hipLaunchKernelGGL(value_table_kernel, grid(nnz), dim3(kBlock), 0, s, (const unsigned long long *)keyOut.p, (const int *)payOut.p,
                       (const int *)head.p, (const int *)rank.p, nnz, most, tabVal.as<unsigned long long>(), tabFirst.as<int>());
    MXL_TRY(hipGetLastError());
    std::vector<unsigned long long> tv((size_t)nd);
    std::vector<int> tf((size_t)nd);
    MXL_TRY(hipMemcpyAsync(tv.data(), tabVal.p, (size_t)nd * 8, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipMemcpyAsync(tf.data(), tabFirst.p, (size_t)nd * 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    // codes in the order of first appearance, as the host's scan over the entries numbers them
    std::vector<int> order((size_t)nd);
    for (int i = 0; i < nd; ++i) order[i] = i;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return tf[a] < tf[b]; });
    std::vector<unsigned char> codeOf(256, 0);
    dict.assign((size_t)256 * sizeof(V), 0);
    for (int c = 0; c < nd; ++c) {
        codeOf[order[c]] = (unsigned char)c;
        std::memcpy(&dict[(size_t)c * sizeof(V)], &tv[order[c]], sizeof(V));  // little-endian: the low bytes are the value
    }
    Buf dCodeOf;
    MXL_TRY(hipMalloc(&dCodeOf.p, 256));
    MXL_TRY(hipMemcpyAsync(dCodeOf.p, codeOf.data(), 256, hipMemcpyHostToDevice, s));
    MXL_TRY(hipMalloc(&codes.p, (size_t)nnz + codePad));
    if (codePad) MXL_TRY(hipMemsetAsync((unsigned char *)codes.p + nnz, 0, codePad, s));
    hipLaunchKernelGGL(value_codes_kernel<V>, grid(nnz), dim3(kBlock), 0, s, val, nnz, (const unsigned long long *)tabVal.p,
                       (const unsigned char *)dCodeOf.p, nd, codes.as<unsigned char>());
    MXL_TRY(hipGetLastError());
    MXL_TRY(hipStreamSynchronize(s));
    *nDict = nd;
    return MX_OK;
}

template <typename V>
static int build_slices_device_t(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr, const int *col, const V *val, int nCU,
                                 int S, const char *elsewhere, DeviceSlices &D, hipStream_t s, std::vector<int> *segPtrOut,
                                 std::vector<int> *segIdxOut, int fused)
{
    using namespace mxl;
    const int E = slice_step_entries(dtype), BE = kSliceBatchEntries, SW = slice_cols(dtype), W = kSliceWaves;
    const int budget = std::max(nCU, 1);
    const long long fair = (long long)nnz / ((long long)budget * W * 64);
    int cap = (int)std::min<long long>(512, std::max<long long>(16, (fair + BE - 1) / BE * BE));
    if (const int v = mx::opt().slice_cap)
        if (v >= BE && v <= 4096) cap = v / BE * BE;
    D = DeviceSlices();
    D.S = S;
    D.rows = rows;
    D.cols = cols;
    D.sliceCols = SW;
    D.nnz = nnz;
    // ---- rows in ascending column order
    Buf row, ord, flag;
    MXL_TRY(hipMalloc(&row.p, std::max<size_t>((size_t)nnz, 1) * 4));
    MXL_TRY(hipMalloc(&ord.p, std::max<size_t>((size_t)nnz, 1) * 4));
    MXL_TRY(hipMalloc(&flag.p, 256));
    MXL_TRY(hipMemsetAsync(flag.p, 0, 256, s));
    int *over4 = flag.as<int>() + 1;
    Buf tmp;
    size_t scanBytes = 0, b2 = 0;
    const size_t nScan = (size_t)std::max(nnz, rows + 1) + 1;
    MXL_TRY(rocprim::inclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, nScan, MaxOp(), s));
    MXL_TRY(rocprim::exclusive_scan(nullptr, b2, (const int *)nullptr, (int *)nullptr, 0, nScan, rocprim::plus<int>(), s));
    scanBytes = std::max(scanBytes, b2);
    MXL_TRY(hipMalloc(&tmp.p, scanBytes + 256));
    if (nnz > 0) {
        // (`ord` is free until the order of the entries is known: it holds the row heads meanwhile)
        MXL_TRY(hipMemsetAsync(ord.p, 0, (size_t)nnz * 4, s));
        hipLaunchKernelGGL(row_heads_kernel, grid(rows), dim3(kBlock), 0, s, rowPtr, rows, ord.as<int>());
        MXL_TRY(hipGetLastError());
        MXL_TRY(rocprim::inclusive_scan(tmp.p, scanBytes, (const int *)ord.p, row.as<int>(), (size_t)nnz, MaxOp(), s));
        hipLaunchKernelGGL(row_order_kernel, grid(nnz), dim3(kBlock), 0, s, rowPtr, col, (const int *)row.p, nnz, flag.as<int>());
        MXL_TRY(hipGetLastError());
    }
    int unsorted = 0;
    MXL_TRY(hipMemcpyAsync(&unsorted, flag.p, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    if (unsorted) {
        int colBits = 1, rowBits = 1;
        while (colBits < 31 && (1ll << colBits) < (long long)cols) ++colBits;
        while (rowBits < 31 && (1ll << rowBits) < (long long)rows) ++rowBits;
        Buf keyIn, keyOut, payIn, tmp;
        size_t sortBytes = 0;
        MXL_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                          (const int *)nullptr, (int *)nullptr, (size_t)nnz, 0u, (unsigned)(colBits + rowBits), s));
        MXL_TRY(hipMalloc(&keyIn.p, (size_t)nnz * 8));
        MXL_TRY(hipMalloc(&keyOut.p, (size_t)nnz * 8));
        MXL_TRY(hipMalloc(&payIn.p, (size_t)nnz * 4));
        MXL_TRY(hipMalloc(&tmp.p, sortBytes + 256));
        hipLaunchKernelGGL(sort_keys_kernel, grid(nnz), dim3(kBlock), 0, s, (const int *)row.p, col, nnz, colBits,
                           keyIn.as<unsigned long long>(), payIn.as<int>());
        MXL_TRY(hipGetLastError());
        MXL_TRY(rocprim::radix_sort_pairs(tmp.p, sortBytes, (const unsigned long long *)keyIn.p, keyOut.as<unsigned long long>(),
                                          (const int *)payIn.p, ord.as<int>(), (size_t)nnz, 0u, (unsigned)(colBits + rowBits), s));
        MXL_TRY(hipStreamSynchronize(s));
    } else if (nnz > 0) {
        hipLaunchKernelGGL(iota_kernel, grid(nnz), dim3(kBlock), 0, s, ord.as<int>(), nnz);
        MXL_TRY(hipGetLastError());
    }
    // ---- virtual rows
    Buf runHead, runStart, start, vid;
    MXL_TRY(hipMalloc(&runHead.p, ((size_t)nnz + 1) * 4));
    MXL_TRY(hipMalloc(&runStart.p, ((size_t)nnz + 1) * 4));
    MXL_TRY(hipMalloc(&start.p, ((size_t)nnz + 1) * 4));
    MXL_TRY(hipMalloc(&vid.p, ((size_t)nnz + 1) * 4));
    int nV = 0;
    if (nnz > 0) {
        hipLaunchKernelGGL(run_heads_kernel, grid(nnz), dim3(kBlock), 0, s, rowPtr, (const int *)row.p, col, (const int *)ord.p, nnz, SW,
                           runHead.as<int>());
        MXL_TRY(hipGetLastError());
        MXL_TRY(rocprim::inclusive_scan(tmp.p, scanBytes, (const int *)runHead.p, runStart.as<int>(), (size_t)nnz, MaxOp(), s));
        hipLaunchKernelGGL(vrow_starts_kernel, grid(nnz), dim3(kBlock), 0, s, (const int *)runStart.p, nnz, cap, start.as<int>());
        MXL_TRY(hipGetLastError());
        MXL_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)start.p, vid.as<int>(), 0, (size_t)nnz, rocprim::plus<int>(), s));
        int lastVid = 0, lastStart = 0;
        MXL_TRY(hipMemcpyAsync(&lastVid, vid.as<int>() + (nnz - 1), 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipMemcpyAsync(&lastStart, start.as<int>() + (nnz - 1), 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        nV = lastVid + lastStart;
    }
    runHead.release();
    D.vrows = nV;
    Buf vStart, vRow, vSlice, vLen, segPtr, key, keyOut, pay, sorted, sliceCount;
    const size_t nv1 = (size_t)nV + 1;
    MXL_TRY(hipMalloc(&vStart.p, nv1 * 4));
    MXL_TRY(hipMalloc(&vRow.p, nv1 * 4));
    MXL_TRY(hipMalloc(&vSlice.p, nv1 * 4));
    MXL_TRY(hipMalloc(&vLen.p, nv1 * 4));
    MXL_TRY(hipMalloc(&segPtr.p, ((size_t)rows + 2) * 4));
    MXL_TRY(hipMalloc(&key.p, nv1 * 4));
    MXL_TRY(hipMalloc(&keyOut.p, nv1 * 4));
    MXL_TRY(hipMalloc(&pay.p, nv1 * 4));
    MXL_TRY(hipMalloc(&sorted.p, nv1 * 4));
    MXL_TRY(hipMalloc(&sliceCount.p, ((size_t)S + 2) * 4));
    if (nnz > 0) {
        hipLaunchKernelGGL(vrow_records_kernel, grid(nnz), dim3(kBlock), 0, s, (const int *)start.p, (const int *)vid.p, (const int *)row.p,
                           col, (const int *)ord.p, nnz, SW, vStart.as<int>(), vRow.as<int>(), vSlice.as<int>());
        MXL_TRY(hipGetLastError());
    }
    hipLaunchKernelGGL(seg_ptr_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, rowPtr, (const int *)vid.p, rows, nnz, nV,
                       segPtr.as<int>());
    MXL_TRY(hipGetLastError());
    std::vector<int> sliceCnt((size_t)S, 0);
    if (nV > 0) {
        hipLaunchKernelGGL(vrow_keys_kernel, grid(nV), dim3(kBlock), 0, s, (const int *)vStart.p, (const int *)vRow.p, (const int *)vSlice.p,
                           (const int *)segPtr.p, nV, nnz, cap, kSliceLightSegs, key.as<unsigned>(), pay.as<int>(), vLen.as<int>());
        MXL_TRY(hipGetLastError());
    }
    // ---- the one-launch form, where it is wanted and the matrix suits it: the records of the virtual rows come
    // down, the host plans (plan_fused_records: the same plan as the host route's), the order goes up
    SlicePlan SP;
    int fusedPlaces = 0;
    bool fusedTaken = false;
    std::vector<int> hSegPtr;
    if (fused && nV > 0 && !elsewhere) {
        std::vector<int> hRowPtr((size_t)rows + 1), hSlice((size_t)nV), hLen((size_t)nV), hSorted;
        hSegPtr.resize((size_t)rows + 1);
        MXL_TRY(hipMemcpyAsync(hRowPtr.data(), rowPtr, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipMemcpyAsync(hSegPtr.data(), segPtr.p, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipMemcpyAsync(hSlice.data(), vSlice.p, (size_t)nV * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipMemcpyAsync(hLen.data(), vLen.p, (size_t)nV * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        const int rc = plan_fused_records(dtype, budget, S, rows, cap, hRowPtr.data(), hSegPtr.data(), hSlice.data(), hLen.data(), nV, fused,
                                          hSorted, SP, &fusedPlaces);
        if (rc < 0) return rc;
        fusedTaken = rc == 1;
        if (fusedTaken) {
            MXL_TRY(hipMemcpyAsync(sorted.p, hSorted.data(), (size_t)nV * 4, hipMemcpyHostToDevice, s));
            MXL_TRY(hipStreamSynchronize(s));  // `hSorted` leaves scope
        }
    }
    if (nV > 0 && !fusedTaken) {
        unsigned keyBits = 1;
        while (keyBits < 32 && (1ull << keyBits) < (unsigned long long)S * (unsigned long long)(cap + 1) * 3ull) ++keyBits;
        size_t sortBytes = 0;
        MXL_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned *)nullptr, (unsigned *)nullptr, (const int *)nullptr,
                                          (int *)nullptr, (size_t)nV, 0u, keyBits, s));
        Buf sortTmp;
        MXL_TRY(hipMalloc(&sortTmp.p, sortBytes + 256));
        MXL_TRY(rocprim::radix_sort_pairs(sortTmp.p, sortBytes, (const unsigned *)key.p, keyOut.as<unsigned>(), (const int *)pay.p,
                                          sorted.as<int>(), (size_t)nV, 0u, keyBits, s));
        hipLaunchKernelGGL(slice_starts_kernel, grid((long long)S + 1), dim3(kBlock), 0, s, (const unsigned *)keyOut.p, nV, S,
                           (unsigned)(cap + 1) * 3u, sliceCount.as<int>());
        MXL_TRY(hipGetLastError());
        std::vector<int> sliceStart((size_t)S + 1, 0);
        MXL_TRY(hipMemcpyAsync(sliceStart.data(), sliceCount.p, ((size_t)S + 1) * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        for (int q = 0; q < S; ++q) sliceCnt[q] = sliceStart[q + 1] - sliceStart[q];
    }
    // ---- chunks: their lengths come down, the plan of the streams goes up
    std::vector<std::vector<SliceChunk>> sliceChunks((size_t)S);
    std::vector<int> firstIdx;
    if (!fusedTaken) {
        int at = 0;
        for (int q = 0; q < S; ++q) {
            for (int f = at; f < at + sliceCnt[q]; f += 64) {
                sliceChunks[q].push_back({f, std::min(64, at + sliceCnt[q] - f), 0});
                firstIdx.push_back(f);
            }
            at += sliceCnt[q];
        }
    }
    const int nChunk = (int)firstIdx.size();
    if (nChunk > 0 && !fusedTaken) {
        Buf dFirst, dLen;
        std::vector<int> len((size_t)nChunk);
        MXL_TRY(hipMalloc(&dFirst.p, (size_t)nChunk * 4));
        MXL_TRY(hipMalloc(&dLen.p, (size_t)nChunk * 4));
        MXL_TRY(hipMemcpyAsync(dFirst.p, firstIdx.data(), (size_t)nChunk * 4, hipMemcpyHostToDevice, s));
        hipLaunchKernelGGL(gather_len_kernel, grid(nChunk), dim3(kBlock), 0, s, (const int *)sorted.p, (const int *)vLen.p,
                           (const int *)dFirst.p, nChunk, dLen.as<int>());
        MXL_TRY(hipGetLastError());
        MXL_TRY(hipMemcpyAsync(len.data(), dLen.p, (size_t)nChunk * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        int i = 0;
        for (int q = 0; q < S; ++q)
            for (SliceChunk &c : sliceChunks[q]) c.steps = (len[i++] + E - 1) / E;
    }
    if (!fusedTaken) {
        const int rc = plan_slice_chunks(dtype, budget, S, sliceChunks, SP);
        if (rc) return rc;
    }
    D.nWG = SP.nWG;
    D.maxWgChunks = SP.maxWgChunks;
    D.steps = SP.totalSteps;
    D.chunks = SP.totalChunks;
    auto up = [&](void **dst, const void *src, size_t bytes) -> int {
        MXL_TRY(hipMalloc(dst, std::max<size_t>(bytes, 4)));
        if (bytes) MXL_TRY(hipMemcpyAsync(*dst, src, bytes, hipMemcpyHostToDevice, s));
        return MX_OK;
    };
    int rc;
    if ((rc = up((void **)&D.wgDesc, SP.wgDesc.data(), SP.wgDesc.size() * 4))) return rc;
    if ((rc = up((void **)&D.waveDesc, SP.waveDesc.data(), SP.waveDesc.size() * 4))) return rc;
    if ((rc = up((void **)&D.chunkEnd, SP.chunkEnd.data(), SP.chunkEnd.size() * 4))) return rc;
    Buf chunkFirst, chunkN, chunkSteps, chunkStep0;
    if ((rc = up(&chunkFirst.p, SP.chunkFirst.data(), SP.chunkFirst.size() * 4))) return rc;
    if ((rc = up(&chunkN.p, SP.chunkN.data(), SP.chunkN.size() * 4))) return rc;
    if ((rc = up(&chunkSteps.p, SP.chunkSteps.data(), SP.chunkSteps.size() * 4))) return rc;
    if ((rc = up(&chunkStep0.p, SP.chunkStep0.data(), SP.chunkStep0.size() * 8))) return rc;
    // ---- the streams
    const size_t nEcol = ((size_t)SP.totalSteps + kSlicePadSteps) * 64 * E;
    MXL_TRY(hipMalloc((void **)&D.ecol, nEcol * 2));
    MXL_TRY(hipMemsetAsync(D.ecol, 0, nEcol * 2, s));
    MXL_TRY(hipMalloc(&D.eval, nEcol * sizeof(V)));
    MXL_TRY(hipMemsetAsync(D.eval, 0, nEcol * sizeof(V), s));
    Buf codes;
    std::vector<unsigned char> dict;
    int nDict = 0;
    {
        if (nnz >= 65536 && mx::opt().csr_dict != 0) {
            if ((rc = device_value_dict<V>(val, nnz, codes, dict, &nDict, s))) return rc;
        }
        if (nDict > 0) {
            MXL_TRY(hipMalloc((void **)&D.ecode, nEcol));
            MXL_TRY(hipMemsetAsync(D.ecode, 255, nEcol, s));
            if ((rc = up(&D.dict, dict.data(), dict.size()))) return rc;
            D.nDict = nDict;
        }
    }
    MXL_TRY(hipMalloc((void **)&D.segIdx, nv1 * 4));
    MXL_TRY(hipMemsetAsync(D.segIdx, 0, nv1 * 4, s));
    if (SP.totalChunks > 0) {
        hipLaunchKernelGGL(vrow_places_kernel, grid(SP.totalChunks * 64), dim3(kBlock), 0, s, (const int *)sorted.p, (const int *)chunkFirst.p,
                           (const int *)chunkN.p, SP.totalChunks, D.segIdx);
        MXL_TRY(hipGetLastError());
    }
    if (nnz > 0) {
        hipLaunchKernelGGL(place_entries_kernel<V>, grid(nnz), dim3(kBlock), 0, s, (const int *)start.p, (const int *)vid.p,
                           (const int *)vStart.p, (const int *)vSlice.p, (const int *)D.segIdx, (const long long *)chunkStep0.p,
                           (const int *)ord.p, col, val, (const unsigned char *)codes.p, nnz, SW, D.ecol, (V *)D.eval,
                           nDict > 0 ? D.ecode : nullptr);
        MXL_TRY(hipGetLastError());
        hipLaunchKernelGGL(pad_columns_kernel, grid(nV), dim3(kBlock), 0, s, (const int *)vStart.p, (const int *)vLen.p, (const int *)vSlice.p,
                           (const int *)D.segIdx, (const long long *)chunkStep0.p, (const int *)chunkSteps.p, (const int *)ord.p, col, nV, SW,
                           D.ecol);
        MXL_TRY(hipGetLastError());
    }
    // ---- how the sums become y
    const size_t nInfo = ((size_t)rows + 3) / 4 * 4 + 4;
    MXL_TRY(hipMalloc((void **)&D.rowInfo, nInfo * 4));
    MXL_TRY(hipMemsetAsync(D.rowInfo, 0xfe, nInfo * 4, s));  // (overwritten below for the rows; the padding must read -2)
    {
        std::vector<int> fill(nInfo - (size_t)rows, -2);
        MXL_TRY(hipMemcpyAsync(D.rowInfo + rows, fill.data(), fill.size() * 4, hipMemcpyHostToDevice, s));
        MXL_TRY(hipStreamSynchronize(s));  // `fill` leaves scope
    }
    Buf isLight, isHeavy, lightPos, heavyPos;
    const size_t r1 = (size_t)rows + 1;
    MXL_TRY(hipMalloc(&isLight.p, r1 * 4));
    MXL_TRY(hipMalloc(&isHeavy.p, r1 * 4));
    MXL_TRY(hipMalloc(&lightPos.p, r1 * 4));
    MXL_TRY(hipMalloc(&heavyPos.p, r1 * 4));
    hipLaunchKernelGGL(row_info_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, (const int *)segPtr.p, (const int *)D.segIdx, elsewhere,
                       rows, kSliceLightSegs, D.rowInfo, isLight.as<int>(), isHeavy.as<int>(), over4, over4 + 1);
    MXL_TRY(hipGetLastError());
    MXL_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)isLight.p, lightPos.as<int>(), 0, r1, rocprim::plus<int>(), s));
    MXL_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)isHeavy.p, heavyPos.as<int>(), 0, r1, rocprim::plus<int>(), s));
    int nLight = 0, nHeavy = 0, anyOver4 = 0, mostVrows = 0;
    MXL_TRY(hipMemcpyAsync(&mostVrows, over4 + 1, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipMemcpyAsync(&nLight, lightPos.as<int>() + rows, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipMemcpyAsync(&nHeavy, heavyPos.as<int>() + rows, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipMemcpyAsync(&anyOver4, over4, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    D.nLight = nLight;
    D.nHeavy = nHeavy;
    D.mostVrows = std::max(mostVrows, nV > 0 ? 1 : 0);
    const int places = anyOver4 ? kSliceLightSegs : 4;
    D.lightQuads = places / 4;
    MXL_TRY(hipMalloc((void **)&D.lightRow, ((size_t)nLight + 1) * 4));
    MXL_TRY(hipMemsetAsync(D.lightRow, 0, ((size_t)nLight + 1) * 4, s));
    MXL_TRY(hipMalloc((void **)&D.lightIdx, ((size_t)nLight * places + 8) * 4));
    MXL_TRY(hipMemsetAsync(D.lightIdx, 0xff, (size_t)nLight * places * 4, s));                    // -1 = no virtual row
    MXL_TRY(hipMemsetAsync(D.lightIdx + (size_t)nLight * places, 0, 8 * 4, s));                   // the spare entries read 0
    MXL_TRY(hipMalloc((void **)&D.heavyInfo, ((size_t)nHeavy * 4 + 4) * 4));
    MXL_TRY(hipMemsetAsync(D.heavyInfo, 0, ((size_t)nHeavy * 4 + 4) * 4, s));
    hipLaunchKernelGGL(row_lists_kernel, grid(rows), dim3(kBlock), 0, s, (const int *)segPtr.p, (const int *)D.segIdx, (const int *)isLight.p,
                       (const int *)isHeavy.p, (const int *)lightPos.p, (const int *)heavyPos.p, rows, places, D.lightRow, D.lightIdx,
                       D.heavyInfo);
    MXL_TRY(hipGetLastError());
    const size_t accBytes = dtype == MX_F64 ? 8 : 4;
    MXL_TRY(hipMalloc(&D.partial, ((size_t)SP.totalChunks * 64 + 64) * accBytes));
    MXL_TRY(hipMemsetAsync(D.partial, 0, ((size_t)SP.totalChunks * 64 + 64) * accBytes, s));
    if (fusedTaken) {
        // what the one-launch kernel needs beyond the two-launch arrays (which stay valid: the plan falls back on them)
        std::vector<int> hSegIdx(nv1, 0), target;
        MXL_TRY(hipMemcpyAsync(hSegIdx.data(), D.segIdx, nv1 * 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        fused_targets(rows, SP.nGroups, fusedPlaces, SP.totalChunks, hSegPtr.data(), hSegIdx.data(), target);
        D.nGroups = SP.nGroups;
        D.maxWgGroups = SP.maxWgGroups;
        D.placesPerRow = fusedPlaces;
        if ((rc = up((void **)&D.wgGroups, SP.wgGroups.data(), SP.wgGroups.size() * 4))) return rc;
        if ((rc = up((void **)&D.groupNeed, SP.groupNeed.data(), SP.groupNeed.size() * 4))) return rc;
        const size_t nTarget = target.size() + 64;  // (64 spare entries, zero)
        MXL_TRY(hipMalloc((void **)&D.fusedTarget, nTarget * 4));
        MXL_TRY(hipMemsetAsync(D.fusedTarget, 0, nTarget * 4, s));
        MXL_TRY(hipMemcpyAsync(D.fusedTarget, target.data(), target.size() * 4, hipMemcpyHostToDevice, s));
        const size_t nCount = (size_t)SP.nGroups + 1, nClaim = (size_t)SP.nWG + 1;
        const size_t sumBytes = ((size_t)SP.nGroups * fusedPlaces * kFusedGroupRows + 64) * accBytes;
        MXL_TRY(hipMalloc((void **)&D.groupCount, nCount * 4));
        MXL_TRY(hipMemsetAsync(D.groupCount, 0, nCount * 4, s));
        MXL_TRY(hipMalloc((void **)&D.claim, nClaim * 4));
        MXL_TRY(hipMemsetAsync(D.claim, 0, nClaim * 4, s));
        MXL_TRY(hipMalloc(&D.fusedSums, sumBytes));
        MXL_TRY(hipMemsetAsync(D.fusedSums, 0, sumBytes, s));
        MXL_TRY(hipStreamSynchronize(s));  // `target` leaves scope
        D.fused = true;
    }
    if (segPtrOut) {
        segPtrOut->assign((size_t)rows + 1, 0);
        MXL_TRY(hipMemcpyAsync(segPtrOut->data(), segPtr.p, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost, s));
    }
    if (segIdxOut) {
        segIdxOut->assign(nv1, 0);
        MXL_TRY(hipMemcpyAsync(segIdxOut->data(), D.segIdx, nv1 * 4, hipMemcpyDeviceToHost, s));
    }
    MXL_TRY(hipStreamSynchronize(s));
    return MX_OK;
}

int check_csr_device(int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, hipStream_t s, const char *who)
{
    using namespace mxl;
    // (the kernels number entries and rows with 32-bit thread indices, rounded up to whole workgroups)
    constexpr int most = 2147483647 - 2 * kBlock;
    if (rows > most || cols > most || nnz > most) {
        set_error(std::string(who) + ": more rows, columns or entries than the device route can number");
        return MX_ERR_ARG;
    }
    Buf bad;
    MXL_TRY(hipMalloc(&bad.p, 256));
    MXL_TRY(hipMemsetAsync(bad.p, 0, 256, s));
    hipLaunchKernelGGL(check_csr_kernel, grid(std::max<long long>((long long)rows + 1, nnz)), dim3(kBlock), 0, s, rowPtr_dev, col_dev, rows,
                       cols, nnz, bad.as<int>());
    MXL_TRY(hipGetLastError());
    int h = 0;
    MXL_TRY(hipMemcpyAsync(&h, bad.p, 4, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    if (h) {
        set_error(std::string(who) + ((h & 1) ? ": rowPtr does not rise from 0 to nnz" : ": column index out of range"));
        return MX_ERR_ARG;
    }
    return MX_OK;
}

int lines_per_gather_device(mx_dtype dtype, int nnz, const int *col_dev, hipStream_t s, double *out)
{
    using namespace mxl;
    const long long windows = nnz / 64, stride = std::max<long long>(1, windows / 65536), sampled = windows / stride;
    *out = 1.0;
    if (sampled <= 0) return MX_OK;
    Buf sum;
    MXL_TRY(hipMalloc(&sum.p, 256));
    MXL_TRY(hipMemsetAsync(sum.p, 0, 256, s));
    hipLaunchKernelGGL(window_lines_kernel, grid(sampled), dim3(kBlock), 0, s, col_dev, sampled, stride, 64 / elem_size(dtype),
                       sum.as<unsigned long long>());
    MXL_TRY(hipGetLastError());
    unsigned long long h = 0;
    MXL_TRY(hipMemcpyAsync(&h, sum.p, 8, hipMemcpyDeviceToHost, s));
    MXL_TRY(hipStreamSynchronize(s));
    *out = (double)h / (double)sampled;
    return MX_OK;
}

// The row-tile form (DeviceCsr) of a CSR matrix in device memory: what upload_csr makes from host
// arrays.  `desc` = the workgroups' row ranges (pack_rows, made on the host from the row pointers).
int upload_csr_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev,
                      const std::vector<int> &desc, bool scan, DeviceCsr &A, hipStream_t s)
{
    using namespace mxl;
    const size_t es = (size_t)elem_size(dtype);
    A = DeviceCsr();
    A.rows = rows;
    A.cols = cols;
    A.nnz = nnz;
    A.npt = csr_entries_per_lane(dtype);
    A.scan = scan;
    A.nBlocks = (int)desc.size() / 4;
    MXL_TRY(hipMalloc((void **)&A.rowPtr, ((size_t)rows + 1) * 4));
    MXL_TRY(hipMemcpyAsync(A.rowPtr, rowPtr_dev, ((size_t)rows + 1) * 4, hipMemcpyDeviceToDevice, s));
    MXL_TRY(hipMalloc(&A.val, ((size_t)nnz + kCsrPad) * es));
    MXL_TRY(hipMemsetAsync((unsigned char *)A.val + (size_t)nnz * es, 0, (size_t)kCsrPad * es, s));
    if (nnz) MXL_TRY(hipMemcpyAsync(A.val, val_dev, (size_t)nnz * es, hipMemcpyDeviceToDevice, s));
    MXL_TRY(hipMalloc((void **)&A.blockDesc, std::max<size_t>(desc.size(), 4) * 4));
    if (!desc.empty()) MXL_TRY(hipMemcpyAsync(A.blockDesc, desc.data(), desc.size() * 4, hipMemcpyHostToDevice, s));
    bool narrow = mx::opt().csr_col16 && nnz > 0;
    Buf lo, wide;
    if (narrow) {
        MXL_TRY(hipMalloc(&lo.p, std::max<size_t>((size_t)A.nBlocks, 1) * 4));
        MXL_TRY(hipMalloc(&wide.p, 256));
        MXL_TRY(hipMemsetAsync(wide.p, 0, 256, s));
        hipLaunchKernelGGL(block_ranges_kernel, grid((long long)A.nBlocks * 64), dim3(kBlock), 0, s, (const int4 *)A.blockDesc, col_dev,
                           A.nBlocks, lo.as<int>(), wide.as<int>());
        MXL_TRY(hipGetLastError());
        int w = 0;
        MXL_TRY(hipMemcpyAsync(&w, wide.p, 4, hipMemcpyDeviceToHost, s));
        MXL_TRY(hipStreamSynchronize(s));
        narrow = w == 0;
    }
    if (narrow) {
        MXL_TRY(hipMalloc((void **)&A.col16, ((size_t)nnz + kCsrPad) * 2));
        MXL_TRY(hipMemsetAsync(A.col16 + nnz, 0, (size_t)kCsrPad * 2, s));
        hipLaunchKernelGGL(narrow_columns_kernel, grid((long long)A.nBlocks * 64), dim3(kBlock), 0, s, (const int4 *)A.blockDesc, col_dev,
                           (const int *)lo.p, A.nBlocks, A.col16);
        MXL_TRY(hipGetLastError());
        A.colBase = (int *)lo.take();
        if (nnz >= 65536 && mx::opt().csr_dict != 0) {
            Buf codes;
            std::vector<unsigned char> dict;
            int nd = 0, rc;
            if (dtype == MX_F64) rc = device_value_dict<double>((const double *)val_dev, nnz, codes, dict, &nd, s, 256, kCsrPad);
            else rc = device_value_dict<_Float16>((const _Float16 *)val_dev, nnz, codes, dict, &nd, s, 256, kCsrPad);
            if (rc) return rc;
            if (nd > 0) {
                A.codes = (unsigned char *)codes.take();
                MXL_TRY(hipMalloc(&A.dict, dict.size()));
                MXL_TRY(hipMemcpyAsync(A.dict, dict.data(), dict.size(), hipMemcpyHostToDevice, s));
                MXL_TRY(hipStreamSynchronize(s));
                A.nDict = nd;
            }
        }
    } else {
        MXL_TRY(hipMalloc((void **)&A.col, ((size_t)nnz + kCsrPad) * 4));
        MXL_TRY(hipMemsetAsync(A.col + nnz, 0, (size_t)kCsrPad * 4, s));
        if (nnz) MXL_TRY(hipMemcpyAsync(A.col, col_dev, (size_t)nnz * 4, hipMemcpyDeviceToDevice, s));
    }
    MXL_TRY(hipStreamSynchronize(s));
    return MX_OK;
}

int build_slices_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev,
                        int nCU, int S, const char *elsewhere_dev, DeviceSlices &D, hipStream_t s, std::vector<int> *segPtrOut,
                        std::vector<int> *segIdxOut, int fused)
{
    if (rows < 1 || cols < 1 || nnz < 0 || S < 1 || !rowPtr_dev || (nnz > 0 && (!col_dev || !val_dev))) {
        set_error("slice layout on the device: bad argument");
        return MX_ERR_ARG;
    }
    MXL_TRY(prepare_slice_kernels(dtype));
    if (dtype == MX_F64)
        return build_slices_device_t<double>(dtype, rows, cols, nnz, rowPtr_dev, col_dev, (const double *)val_dev, nCU, S, elsewhere_dev, D,
                                             s, segPtrOut, segIdxOut, fused);
    return build_slices_device_t<_Float16>(dtype, rows, cols, nnz, rowPtr_dev, col_dev, (const _Float16 *)val_dev, nCU, S, elsewhere_dev,
                                           D, s, segPtrOut, segIdxOut, fused);
}

}  // namespace mx
