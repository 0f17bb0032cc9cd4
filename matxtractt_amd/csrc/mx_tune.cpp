// The extraction fractions for a matrix: timed over a grid (mx_tune_tau) or estimated from counts
// (mx_estimate_tau).
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

extern "C" int mx_tune_tau(const mx_csr *A, int levels, int flags, int warm, int iters, float *tau_c, float *tau_r,
                           mx_tau_point *table, int cap, int *n_points)
{
    mx::refresh_options();
    if (!A || levels < 2 || levels > 65 || warm < 0 || iters <= 0 || !tau_c || !tau_r || (table && cap < 0)) {
        set_error("mx_tune_tau: bad argument");
        return MX_ERR_ARG;
    }
    int rc = need_device();
    if (rc) return rc;
    const size_t es = (size_t)mx::elem_size(A->dtype);
    void *dx = nullptr, *dy = nullptr;
    {
        // x as the reference's driver fills it (initVec, include/common.h:237-245)
        std::vector<unsigned char> hx(std::max<size_t>((size_t)A->cols * es, 16));
        mx_init_vec(A->dtype, hx.data(), A->cols);
        if ((rc = upload_bytes(&dx, hx.data(), hx.size()))) return rc;
        if ((rc = upload_bytes(&dy, nullptr, 0, std::max<size_t>((size_t)A->rows * es, 16)))) {
            (void)hipFree(dx);
            return rc;
        }
    }
    // The tuner needs the device anyway: a large matrix goes up once and every candidate's extraction
    // and plan are made there (mx_plan_create_device: the same plans, a fraction of the time); below
    // about two million entries the host route is as fast.
    const bool onDevice = A->nnz >= (1 << 21) && A->rows > 0 && A->cols > 0;
    int *dRowPtr = nullptr, *dColInd = nullptr;
    void *dVal = nullptr;
    auto release = [&]() {
        (void)hipFree(dx);
        (void)hipFree(dy);
        (void)hipFree(dRowPtr);
        (void)hipFree(dColInd);
        (void)hipFree(dVal);
    };
    if (onDevice) {
        rc = upload(&dRowPtr, A->rowPtr, (size_t)A->rows + 1);
        if (!rc) rc = upload(&dColInd, A->colInd, (size_t)A->nnz);
        if (!rc) rc = upload_bytes(&dVal, A->val, (size_t)A->nnz * es);
        if (rc) {
            release();
            return rc;
        }
    }
    double best = 0.0, csrOnly = -1.0;
    bool have = false;
    int n = 0;
    rc = MX_OK;
    for (int ic = 0; ic < levels && !rc; ++ic)
        for (int ir = 0; ir <= ic && !rc; ++ir) {
            const float c = (float)ic / (float)(levels - 1), r = (float)ir / (float)(levels - 1);
            mx_partition *P = nullptr;
            mx_plan *plan = nullptr;
            double ms = 0.0;
            int tileNnz = 0;
            bool anyTile = false;  // does the candidate hand anything to a tile kernel?
            if (onDevice) {
                if ((rc = mx_plan_create_device(A->dtype, A->rows, A->cols, A->nnz, dRowPtr, dColInd, dVal, c, r, flags, &plan))) break;
                anyTile = plan->tile_nnz > 0;
            } else {
                if ((rc = mx_partition_create(A, c, r, &P))) break;
                if (P->extracted && !(flags & MX_PLAN_NO_TILES)) {
                    const double gate = tile_gate(P->dtype) * P->fragM * P->fragK;
                    const int nFrags = P->chunkPtr[P->chunkNum];
                    for (int f = 0; f < nFrags && !anyTile; ++f) {
                        const int vals = P->fragPtr[f + 1] - P->fragPtr[f];
                        anyTile = (flags & MX_PLAN_ALL_TILES) ? vals > 0 : (vals > 0 && (double)vals >= gate);
                    }
                }
            }
            if (!anyTile && csrOnly >= 0.0) {
                ms = csrOnly;  // the same plan as an earlier candidate
            } else {
                if (!plan) rc = mx_plan_create(P, flags, &plan);
                if (!rc) rc = mx_time(plan, dx, dy, warm, iters, &ms, nullptr, nullptr);
                if (!rc) {
                    tileNnz = plan->tile_nnz;
                    if (!anyTile) csrOnly = ms;
                }
            }
            mx_plan_destroy(plan);
            mx_partition_destroy(P);
            if (rc) break;
            if (table && n < cap) table[n] = mx_tau_point{c, r, ms, tileNnz};
            ++n;
            // a candidate without tiles never displaces an equally fast earlier one: ties go to (0, 0)
            if (!have || ms < best) {
                best = ms;
                *tau_c = anyTile ? c : 0.0f;
                *tau_r = anyTile ? r : 0.0f;
                have = true;
            }
        }
    release();
    if (n_points) *n_points = n;
    return rc;
}

// The two fractions from counts alone: for every point of the grid the extraction runs on the device
// (HybridDevice::analyse) and the plan's own estimate of what its tiles save per product is read off;
// the point with the largest saving wins, (0, 0) when none saves anything.  Nothing is planned or
// timed.  (The reference's counterpart is the regression model of ML/train_*.py over the count
// features of ML/extract_features.cpp:31-95, queried through ML/bayes_opt.py.)
extern "C" int mx_estimate_tau(const mx_csr *A, int levels, float *tau_c, float *tau_r, mx_tau_estimate *table, int cap, int *n_points)
{
    mx::refresh_options();
    if (!A || levels < 2 || levels > 65 || !tau_c || !tau_r || (table && cap < 0) || A->rows < 1 || A->cols < 1 || A->nnz < 0 ||
        !A->rowPtr || (A->nnz > 0 && (!A->colInd || !A->val)) || (A->dtype != MX_F64 && A->dtype != MX_F16)) {
        set_error("mx_estimate_tau: bad argument");
        return MX_ERR_ARG;
    }
    int rc = need_device();
    if (rc) return rc;
    const size_t es = (size_t)mx::elem_size(A->dtype);
    int *dRowPtr = nullptr, *dColInd = nullptr;
    void *dVal = nullptr;
    auto release = [&]() {
        (void)hipFree(dRowPtr);
        (void)hipFree(dColInd);
        (void)hipFree(dVal);
    };
    rc = upload(&dRowPtr, A->rowPtr, (size_t)A->rows + 1);
    if (!rc) rc = upload(&dColInd, A->colInd, (size_t)A->nnz);
    if (!rc) rc = upload_bytes(&dVal, A->val, (size_t)A->nnz * es);
    if (!rc) rc = mx::check_csr_device(A->rows, A->cols, A->nnz, dRowPtr, dColInd, nullptr, "mx_estimate_tau");
    if (rc) {
        release();
        return rc;
    }
    const int fragM = mx::kFragM, fragK = mx::frag_k(A->dtype);
    const double need = tile_gate(A->dtype) * fragM * fragK;
    int minVals = (int)need;
    while ((double)minVals < need) ++minVals;
    const bool wantStrips = A->dtype == MX_F16 && !mx::opt().no_strips;
    const bool wantBlocks = A->dtype == MX_F64 && !mx::opt().no_blocks;
    double best = 0.0;
    *tau_c = *tau_r = 0.0f;
    int n = 0;
    try {
        for (int ic = 0; ic < levels && !rc; ++ic)
            for (int ir = 0; ir <= ic && !rc; ++ir) {
                const float c = (float)ic / (float)(levels - 1), r = (float)ir / (float)(levels - 1);
                mx_tau_estimate e{c, r, 0.0, 0};
                if (ic > 0 && A->nnz > 0) {  // (tau_c = 0 selects nothing)
                    mx::HybridDevice H;
                    mx::HybridCounts cnt;
                    if ((rc = H.analyse(A->dtype, A->rows, A->cols, A->nnz, dRowPtr, dColInd, dVal, c, r, minVals, true, wantStrips, wantBlocks,
                                        &cnt, nullptr)))
                        break;
                    if (cnt.blocks64) cnt.generalFrags = cnt.generalEntries = 0;
                    double netNs = 0.0;
                    const int worth = tiles_worth(A->dtype, fragM, fragK, cnt.blocks64, (double)cnt.generalEntries, (double)cnt.generalFrags,
                                                  (double)cnt.stripEntries, (double)cnt.stripBlocks, (double)cnt.stripBlocksOff, (double)A->nnz,
                                                  &netNs);
                    e.saved_us = netNs * 1e-3;
                    e.tile_entries = worth == 0 ? 0 : (worth == 2 ? cnt.generalEntries : 0) + cnt.stripEntries;
                }
                if (table && n < cap) table[n] = e;
                ++n;
                if (e.saved_us > best) {
                    best = e.saved_us;
                    *tau_c = c;
                    *tau_r = r;
                }
            }
    } catch (const std::bad_alloc &) {
        set_error("mx_estimate_tau: out of memory");
        rc = MX_ERR_ALLOC;
    }
    release();
    if (n_points) *n_points = n;
    return rc;
}

