// Device side of the preprocessing: the transposes.
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

#include <cstdint>
#include <cstring>
#include <string>

#include <rocprim/device/device_radix_sort.hpp>

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
