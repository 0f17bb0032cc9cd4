// The reference's one-shot calls (host pointers in, host pointers out) and the MFMA layout probes.
#include <algorithm>
#include <atomic>
#include <chrono>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <numeric>
#include <omp.h>
#include <parallel/algorithm>
#include <queue>
#include <vector>

#include "mx_plan_parts.h"

using namespace mxp;

// ---- reference surface: host pointers in, host pointers out ------------------------------

static int cdspmv_any(mx_dtype dtype, const void *csrVal, const int *csrRowPtr, const int *csrColInd, const void *x,
                      void *y, int rows, int cols, int nnz, int warm, int iters, double *cdTime, double *cdPre)
{
    if (!csrRowPtr || !x || !y || rows < 0 || cols < 0 || nnz < 0 || (nnz > 0 && (!csrVal || !csrColInd))) {
        set_error("cdspmv: bad argument");
        return MX_ERR_ARG;
    }
    mx::refresh_options();
    int rc = need_device();
    if (rc) return rc;
    for (int p = 0; p < nnz; ++p)
        if ((unsigned)csrColInd[p] >= (unsigned)cols) {
            set_error("cdspmv: column index out of range");
            return MX_ERR_ARG;
        }
    if (csrRowPtr[0] != 0 || csrRowPtr[rows] != nnz) {
        set_error("cdspmv: rowPtr does not span [0, nnz]");
        return MX_ERR_ARG;
    }
    mx_plan plan;
    plan.dtype = dtype;
    plan.rows = rows;
    plan.cols = cols;
    plan.nnz = nnz;
    const size_t es = (size_t)mx::elem_size(dtype);
    void *dx = nullptr, *dy = nullptr, *dscratch = nullptr;
    auto body = [&]() -> int {
        double pre = 0.0;
        int r = upload_csr(dtype, rows, cols, nnz, csrRowPtr, csrColInd, csrVal, plan.csr, &pre);
        if (r) return r;
        if (cdPre) *cdPre = pre;
        if ((r = upload_bytes(&dx, x, cols * es))) return r;
        if ((r = upload_bytes(&dy, y, rows * es))) return r;
        if ((r = upload_bytes(&dscratch, nullptr, 0, rows * es))) return r;
        MX_HIP(hipStreamCreate(&plan.stream));
        MX_HIP(hipEventCreate(&plan.ev0));
        MX_HIP(hipEventCreate(&plan.ev1));
        double ms = 0.0;
        if (iters > 0) {
            r = time_loop(&plan, warm, iters, [&]() -> int {
                MX_HIP(mx::launch_csr(dtype, plan.csr, dx, dscratch, 0, plan.stream));
                return MX_OK;
            }, &ms);
            if (r) return r;
        }
        if (cdTime) *cdTime = ms;
        MX_HIP(mx::launch_csr(dtype, plan.csr, dx, dy, 1, plan.stream));  // y += A*x
        MX_HIP(hipStreamSynchronize(plan.stream));
        MX_HIP(hipMemcpy(y, dy, rows * es, hipMemcpyDeviceToHost));
        return MX_OK;
    };
    rc = body();
    free_csr(plan.csr);
    (void)hipFree(dx);
    (void)hipFree(dy);
    (void)hipFree(dscratch);
    if (plan.ev0) (void)hipEventDestroy(plan.ev0);
    if (plan.ev1) (void)hipEventDestroy(plan.ev1);
    if (plan.stream) (void)hipStreamDestroy(plan.stream);
    return rc;
}

extern "C" int mx_cdspmv_f64(const double *csrVal, const int *csrRowPtr, const int *csrColInd, const double *x, double *y,
                             int rows, int cols, int nnz, int warm, int iters, double *cdTime, double *cdPre)
{
    return cdspmv_any(MX_F64, csrVal, csrRowPtr, csrColInd, x, y, rows, cols, nnz, warm, iters, cdTime, cdPre);
}

extern "C" int mx_cdspmv_f16(const uint16_t *csrVal, const int *csrRowPtr, const int *csrColInd, const uint16_t *x,
                             uint16_t *y, int rows, int cols, int nnz, int warm, int iters, double *cdTime, double *cdPre)
{
    return cdspmv_any(MX_F16, csrVal, csrRowPtr, csrColInd, x, y, rows, cols, nnz, warm, iters, cdTime, cdPre);
}

static int du_any(mx_dtype dtype, const int *chunkPtr, const int *fragPtr, const void *fragBit, const void *tcVal,
                  const int *atox, const void *x_d, void *y_d, int dRows, int dCols, int warm, int iters, double *tcTime)
{
    if (!chunkPtr || !fragPtr || !x_d || !y_d || dRows < 0 || dCols < 0) {
        set_error("du_tcspmv: bad argument");
        return MX_ERR_ARG;
    }
    mx::refresh_options();
    int rc = need_device();
    if (rc) return rc;
    const int fragK = mx::frag_k(dtype), fragM = mx::kFragM;
    const size_t es = (size_t)mx::elem_size(dtype);
    const int chunkNum = (dRows + fragM - 1) / fragM;
    const int frags = chunkPtr[chunkNum];
    const int vals = fragPtr[frags];
    if (frags > 0 && (!fragBit || !atox || (vals > 0 && !tcVal))) {
        set_error("du_tcspmv: missing tile arrays");
        return MX_ERR_ARG;
    }
    for (size_t i = 0; i < (size_t)frags * fragK; ++i)
        if ((unsigned)atox[i] >= (unsigned)std::max(dCols, 1)) {
            set_error("du_tcspmv: sparse_AToX_index out of range");
            return MX_ERR_ARG;
        }
    mx_plan plan;
    plan.dtype = dtype;
    mx::DeviceTiles &T = plan.tiles;
    void *dx = nullptr, *dy = nullptr, *dscratch = nullptr;
    auto body = [&]() -> int {
        int r;
        if ((r = upload_tiles(dtype, chunkNum, nullptr, dRows, chunkPtr, fragPtr, fragBit, tcVal, atox, nullptr, nullptr, T,
                              nullptr)))
            return r;
        if ((r = upload_bytes(&dx, x_d, dCols * es))) return r;
        // FP64 uploads the caller's y and adds to it; FP16 starts from zero
        // (du_tcSpMV_fp64.cu:296-297 vs du_tcSpMV_fp16_v2.cu:146-147)
        if (dtype == MX_F64) {
            if ((r = upload_bytes(&dy, y_d, dRows * es))) return r;
        } else {
            if ((r = upload_bytes(&dy, nullptr, 0, dRows * es))) return r;
        }
        if ((r = upload_bytes(&dscratch, nullptr, 0, dRows * es))) return r;
        MX_HIP(hipStreamCreate(&plan.stream));
        MX_HIP(hipEventCreate(&plan.ev0));
        MX_HIP(hipEventCreate(&plan.ev1));
        double ms = 0.0;
        if (iters > 0 && chunkNum > 0) {
            r = time_loop(&plan, warm, iters, [&]() -> int {
                MX_HIP(mx::launch_tiles(dtype, T, dx, dscratch, 0, plan.stream));
                return MX_OK;
            }, &ms);
            if (r) return r;
        }
        if (tcTime) *tcTime = ms;
        MX_HIP(mx::launch_tiles(dtype, T, dx, dy, dtype == MX_F64 ? 1 : 0, plan.stream));
        MX_HIP(hipStreamSynchronize(plan.stream));
        MX_HIP(hipMemcpy(y_d, dy, dRows * es, hipMemcpyDeviceToHost));
        return MX_OK;
    };
    rc = body();
    free_tiles(T);
    (void)hipFree(dx);
    (void)hipFree(dy);
    (void)hipFree(dscratch);
    if (plan.ev0) (void)hipEventDestroy(plan.ev0);
    if (plan.ev1) (void)hipEventDestroy(plan.ev1);
    if (plan.stream) (void)hipStreamDestroy(plan.stream);
    return rc;
}

extern "C" int mx_du_tcspmv_f64(const int *chunkPtr, const int *fragPtr, const uint32_t *fragBit, const double *tcVal,
                                const int *sparse_AToX_index, const double *x_d, double *y_d, int dRows, int dCols,
                                int warm, int iters, double *tcTime)
{
    return du_any(MX_F64, chunkPtr, fragPtr, fragBit, tcVal, sparse_AToX_index, x_d, y_d, dRows, dCols, warm, iters, tcTime);
}

extern "C" int mx_du_tcspmv_f16(const int *chunkPtr, const int *fragPtr, const uint64_t *fragBit, const uint16_t *tcVal,
                                const int *sparse_AToX_index, const uint16_t *x_d, uint16_t *y_d, int dRows, int dCols,
                                int warm, int iters, double *tcTime)
{
    return du_any(MX_F16, chunkPtr, fragPtr, fragBit, tcVal, sparse_AToX_index, x_d, y_d, dRows, dCols, warm, iters, tcTime);
}

// MFMA layout probes (used by the GPU tests): D(16x16) = A*B on one wave.
extern "C" int mx_probe_mfma_f64(const double *A, const double *B, double *D)
{
    int rc = need_device();
    if (rc) return rc;
    double *dA = nullptr, *dB = nullptr, *dD = nullptr;
    auto body = [&]() -> int {
        int r;
        if ((r = upload(&dA, A, 64))) return r;
        if ((r = upload(&dB, B, 64))) return r;
        if ((r = upload<double>(&dD, nullptr, 0, 256))) return r;
        MX_HIP(mx::launch_probe_f64(dA, dB, dD, nullptr));
        MX_HIP(hipDeviceSynchronize());
        MX_HIP(hipMemcpy(D, dD, 256 * sizeof(double), hipMemcpyDeviceToHost));
        return MX_OK;
    };
    rc = body();
    (void)hipFree(dA);
    (void)hipFree(dB);
    (void)hipFree(dD);
    return rc;
}

extern "C" int mx_probe_mfma_f16(const uint16_t *A, const uint16_t *B, float *D)
{
    int rc = need_device();
    if (rc) return rc;
    uint16_t *dA = nullptr, *dB = nullptr;
    float *dD = nullptr;
    auto body = [&]() -> int {
        int r;
        if ((r = upload(&dA, A, 512))) return r;
        if ((r = upload(&dB, B, 512))) return r;
        if ((r = upload<float>(&dD, nullptr, 0, 256))) return r;
        MX_HIP(mx::launch_probe_f16(dA, dB, dD, nullptr));
        MX_HIP(hipDeviceSynchronize());
        MX_HIP(hipMemcpy(D, dD, 256 * sizeof(float), hipMemcpyDeviceToHost));
        return MX_OK;
    };
    rc = body();
    (void)hipFree(dA);
    (void)hipFree(dB);
    (void)hipFree(dD);
    return rc;
}

