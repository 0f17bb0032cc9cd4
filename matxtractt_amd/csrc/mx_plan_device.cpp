// Plans made where the matrix already is: from CSR arrays in device memory, with or without an
// extraction, and from a partition that was made on the device.  Only counts cross to the host.
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

// The CSR part of a plan from arrays in device memory: the form is chosen as setup_csr_part chooses
// it -- the same counts, taken on the device -- and only that form is built, there.  Nothing of the
// matrix crosses to the host but its row pointers (for the row-tile form) or the lengths of its
// chunks (for the slice form).  `elsewhere_dev` (optional): marks of rows that another kernel writes.
static int setup_csr_part_device(mx_plan *plan, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev, int flags,
                                 const char *elsewhere_dev, std::pair<std::vector<int>, std::vector<int>> *segOut = nullptr)
{
    const mx_dtype dtype = plan->dtype;
    const int rows = plan->rows, cols = plan->cols;
    int rc;
    plan->csr_nnz = nnz;
    hipDeviceProp_t prop;
    int dev = 0;
    MX_HIP(hipGetDevice(&dev));
    MX_HIP(hipGetDeviceProperties(&prop, dev));
    const int nCU = std::max(1, prop.multiProcessorCount);
    const int S = rows > 0 ? slice_count(dtype, rows, cols, nnz, nCU) : 0;
    bool want[2] = {true, S > 0};
    const int env = mx::opt().csr_kernel;
    if (env == 3 || plan_autotune()) {
        // The split form and the timed choice exist on the host route only: the part comes down and takes that
        // route, so that the plan is the one mx_plan_create makes under the same settings.
        const size_t es = (size_t)mx::elem_size(dtype);
        std::vector<int> rp((size_t)rows + 1), ci((size_t)std::max(nnz, 1));
        std::vector<unsigned char> va(std::max<size_t>((size_t)nnz * es, 1));
        std::vector<char> marks;
        MX_HIP(hipMemcpy(rp.data(), rowPtr_dev, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost));
        if (nnz) MX_HIP(hipMemcpy(ci.data(), colInd_dev, (size_t)nnz * 4, hipMemcpyDeviceToHost));
        if (nnz) MX_HIP(hipMemcpy(va.data(), val_dev, (size_t)nnz * es, hipMemcpyDeviceToHost));
        if (elsewhere_dev) {
            marks.resize((size_t)rows);
            MX_HIP(hipMemcpy(marks.data(), elsewhere_dev, (size_t)rows, hipMemcpyDeviceToHost));
        }
        return setup_csr_part(plan, rp.data(), ci.data(), va.data(), flags, elsewhere_dev ? marks.data() : nullptr, segOut);
    }
    if (flags & MX_PLAN_CSR_ROWS) want[1] = false;
    if ((flags & MX_PLAN_CSR_SLICES) && S > 0) want[0] = false;
    if (env == 1) want[0] = true, want[1] = false;
    if (env == 2 && S > 0) want[1] = true, want[0] = false;
    if (want[1]) {
        // (the one-launch form where the matrix suits it and the device deals its workgroups as the form assumes:
        // the layout is made for it in the same pass -- the records of the virtual rows go to the host, its plan
        // comes back, the entries stay)
        int wantFused = !elsewhere_dev ? fused_wanted(flags, dtype, rows, S, -1, nCU) : 0;
        if (wantFused) {
            int ok = 0;
            MX_HIP(mx::fused_placement_ok(nCU, &ok));
            if (!ok) wantFused = 0;
        }
        rc = mx::build_slices_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, nCU, S, elsewhere_dev, plan->slices, nullptr,
                                     segOut ? &segOut->first : nullptr, segOut ? &segOut->second : nullptr, wantFused);
        if (rc) return rc;
        if (plan->slices.ecode) plan->slices.useDict = true;
    }
    if (want[0] && want[1]) {
        // the estimates of csr_estimates from what the device counted: the virtual rows are those of
        // the layout just made, the one-byte form exists when the layout has it
        CsrStats st;
        st.vrows = plan->slices.vrows;
        st.fewValues = plan->slices.ecode != nullptr;
        if ((rc = mx::lines_per_gather_device(dtype, nnz, colInd_dev, nullptr, &st.linesPerGather))) return rc;
        csr_estimates(dtype, cols, nnz, st, &plan->est_rows_us, &plan->est_slices_us);
        // (as the host route, which estimates before it has a layout: by the average of the sums under a workgroup)
        if (!elsewhere_dev && fused_wanted(flags, dtype, rows, S, plan->slices.mostVrows, nCU)) plan->est_slices_us -= kFusedSavesUs;
        want[plan->est_slices_us < plan->est_rows_us ? 0 : 1] = false;
    }
    if (want[1]) {
        plan->csr_variant = 1;
        plan->fused = plan->slices.fused;
        decide_keep(plan, flags);
        return MX_OK;
    }
    free_slices(plan->slices);
    plan->csr_variant = 0;
    std::vector<int> rp((size_t)rows + 1, 0), desc;
    MX_HIP(hipMemcpy(rp.data(), rowPtr_dev, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost));
    const int npt = mx::csr_entries_per_lane(dtype);
    pack_rows(rp.data(), rows, npt, desc);
    double sum = 0.0, sq = 0.0;
    for (int r = 0; r < rows; ++r) {
        const double n = rp[r + 1] - rp[r];
        sum += n;
        sq += n * n;
    }
    const double mean = rows > 0 ? sum / rows : 0.0, var = rows > 0 ? sq / rows - mean * mean : 0.0;
    bool scan = mean > 0.0 && var > 0.25 * mean * mean;
    if (mx::opt().csr_reduce == 1) scan = false;
    if (mx::opt().csr_reduce == 2) scan = true;
    rc = mx::upload_csr_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, desc, scan, plan->csr, nullptr);
    if (rc) return rc;
    if (plan->csr.codes) plan->csr.useDict = true;
    return MX_OK;
}

// A plan for y = A x from a CSR matrix that lives in device memory: nothing of the matrix crosses
// to the host but its row pointers (for the row-tile form) or the lengths of its chunks (for the
// slice form).  The form is chosen as in mx_plan_create -- the same counts, taken on the device --
// so the plan equals the one mx_plan_create makes from a partition of the same matrix with
// tau = (0, 0).
extern "C" int mx_plan_create_device_csr(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                                         const void *val_dev, int flags, mx_plan **out)
{
    mx::refresh_options();
    if (!out || (dtype != MX_F64 && dtype != MX_F16) || rows < 0 || cols < 0 || nnz < 0 || !rowPtr_dev ||
        (nnz > 0 && (!colInd_dev || !val_dev || rows == 0 || cols == 0))) {
        set_error("mx_plan_create_device_csr: bad argument");
        return MX_ERR_ARG;
    }
    *out = nullptr;
    int rc = need_device();
    if (rc) return rc;
    if ((rc = mx::check_csr_device(rows, cols, nnz, rowPtr_dev, colInd_dev, nullptr, "mx_plan_create_device_csr"))) return rc;
    mx_plan *plan = new (std::nothrow) mx_plan();
    if (!plan) {
        set_error("mx_plan_create_device_csr: out of memory");
        return MX_ERR_ALLOC;
    }
    plan->dtype = dtype;
    plan->rows = rows;
    plan->cols = cols;
    plan->nnz = nnz;
    plan->csr_nnz = nnz;
    plan->prep_route = 1;
    auto fail = [&](int code) {
        mx_plan_destroy(plan);
        return code;
    };
    if (hipStreamCreate(&plan->stream) != hipSuccess || hipEventCreate(&plan->ev0) != hipSuccess ||
        hipEventCreate(&plan->ev1) != hipSuccess) {
        set_error("mx_plan_create_device_csr: could not create stream/events");
        return fail(MX_ERR_DEVICE);
    }
    {
        void *fixed = nullptr;
        if (mx::static_scratch(&fixed) != hipSuccess) {
            (void)hipGetLastError();
            set_error("mx_plan_create_device_csr: hipGetSymbolAddress failed for the fixed array of sums");
            return fail(MX_ERR_DEVICE);
        }
    }
    try {
        rc = setup_csr_part_device(plan, nnz, rowPtr_dev, colInd_dev, val_dev, flags, nullptr);
        if (rc) return fail(rc);
    } catch (const std::bad_alloc &) {
        set_error("mx_plan_create_device_csr: out of memory");
        return fail(MX_ERR_ALLOC);
    }
    *out = plan;
    return MX_OK;
}

// The steps of a tile layout from the block counts of its chunks alone, as build_tiles lays them out:
// a chunk of up to half a step's blocks shares a step with the next such chunk (half 0 and half 1), a
// larger one takes whole steps of its own, half 0 filled first.  SF: block slots of a step; BS: values
// per block.  stepDesc: `stride` (8 or 10) ints per step {chunk of half 0, chunk of half 1 (-1 none, -2
// the first goes on), flags, blocks in half 0, blocks in half 1, first value, first value and blocks in
// half 0 of the step four further on[, first block of half 0 inside its chunk, 0]}; chunkBlock0: the first
// block of every chunk in the stored values.
static int plan_tile_steps(const std::vector<int> &chunkBlocks, int SF, int BS, int perMin, int nCU, int stride, std::vector<int> &stepDesc,
                           std::vector<int> &chunkBlock0, std::vector<int> &waveDesc, long long *totalBlocks)
{
    const int HF = SF / 2, n = (int)chunkBlocks.size();
    std::vector<int> stepVo, stepA, stepEnd, who;  // who: {chunk of half 0, of half 1, flags, blocks, blocks, first block} per step
    chunkBlock0.assign((size_t)n, 0);
    long long blocks = 0;
    int pending = -1;
    auto emit = [&](int a, int b, int flags, int n0, int n1, int i0) {
        const int d[6] = {a, b, flags, n0, n1, i0};
        who.insert(who.end(), d, d + 6);
        stepVo.push_back((int)(blocks * BS));
        stepA.push_back(n0);
        stepEnd.push_back(flags & 1);
        blocks += n0 + n1;
    };
    for (int k = 0; k < n; ++k) {
        const int nb = chunkBlocks[k];
        if (nb < 1 || (stride == 8 && nb > SF)) {
            set_error("tile layout: a chunk with an impossible number of blocks");
            return MX_ERR_DEVICE;
        }
        if (nb <= HF) {
            if (pending >= 0) {
                chunkBlock0[pending] = (int)blocks;
                chunkBlock0[k] = (int)blocks + chunkBlocks[pending];
                emit(pending, k, 3, chunkBlocks[pending], nb, 0);
                pending = -1;
            } else {
                pending = k;
            }
        } else {
            chunkBlock0[k] = (int)blocks;
            for (int i0 = 0; i0 < nb; i0 += SF) {
                const int m = std::min(nb - i0, SF), n0 = std::min(m, HF);
                emit(k, -2, i0 + SF >= nb ? 1 : 0, n0, m - n0, i0);
            }
        }
        if (blocks * BS > 2000000000LL) {
            set_error("tile layout: too many values for 32-bit offsets");
            return MX_ERR_ARG;
        }
    }
    if (pending >= 0) {
        chunkBlock0[pending] = (int)blocks;
        emit(pending, -1, 3, chunkBlocks[pending], 0, 0);
    }
    const int steps = (int)stepVo.size();
    std::vector<int> ahead;
    tile_waves(steps, nCU, perMin, stepVo, stepA, stepEnd, waveDesc, ahead);
    stepDesc.assign((size_t)steps * stride, 0);
    for (int st = 0; st < steps; ++st) {
        int *d = &stepDesc[(size_t)st * stride];
        for (int k = 0; k < 5; ++k) d[k] = who[(size_t)st * 6 + k];
        d[5] = stepVo[st];
        d[6] = ahead[2 * (size_t)st];
        d[7] = ahead[2 * (size_t)st + 1];
        if (stride > 8) d[8] = who[(size_t)st * 6 + 5];
    }
    *totalBlocks = blocks;
    return MX_OK;
}

// plan_tile_steps for inspection (tests hold it against the layouts build_tiles makes, without a GPU)
extern "C" void mx_tile_steps_free(mx_tile_steps_view *v)
{
    if (!v) return;
    free(v->stepDesc);
    free(v->chunkBlock0);
    free(v->waveDesc);
    std::memset(v, 0, sizeof(*v));
}
extern "C" int mx_tile_steps(const int *chunkBlocks, int nChunks, int slots, int blockValues, int perMin, int nCU, mx_tile_steps_view *out)
{
    if (!out || nChunks < 0 || (nChunks > 0 && !chunkBlocks) || slots < 2 || (slots & 1) || blockValues < 1 || perMin < 1 || nCU < 1) {
        set_error("mx_tile_steps: bad argument");
        return MX_ERR_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    try {
        std::vector<int> blocks(chunkBlocks, chunkBlocks + nChunks), stepDesc, chunkBlock0, waveDesc;
        long long total = 0;
        const int rc = plan_tile_steps(blocks, slots, blockValues, perMin, nCU, 10, stepDesc, chunkBlock0, waveDesc, &total);
        if (rc) return rc;
        auto give = [](const std::vector<int> &v) {
            int *q = (int *)malloc(std::max<size_t>(v.size(), 1) * sizeof(int));
            if (q && !v.empty()) std::memcpy(q, v.data(), v.size() * sizeof(int));
            return q;
        };
        out->steps = (int)(stepDesc.size() / 10);
        out->nWaves = (int)(waveDesc.size() / 8);
        out->totalBlocks = total;
        out->stepDesc = give(stepDesc);
        out->chunkBlock0 = give(chunkBlock0);
        out->waveDesc = give(waveDesc);
        if (!out->stepDesc || !out->chunkBlock0 || !out->waveDesc) {
            mx_tile_steps_free(out);
            set_error("mx_tile_steps: out of memory");
            return MX_ERR_ALLOC;
        }
    } catch (const std::bad_alloc &) {
        mx_tile_steps_free(out);
        set_error("mx_tile_steps: out of memory");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}

// A hybrid plan from a CSR matrix in device memory and the two extraction fractions: the
// extraction, the plan's decisions, the CSR part with its layout and the strips' layout are all
// made on the device (mx_hybrid.hip, mx_layout.hip); what a decision needs comes to the host as
// counts.  The plan equals the one mx_plan_create makes from mx_partition_create(_device) of the
// same matrix, whatever tile forms it keeps.
extern "C" int mx_plan_create_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                                     const void *val_dev, float tau_c, float tau_r, int flags, mx_plan **out)
{
    mx::refresh_options();
    return create_plan_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, tau_c, tau_r, flags, out, false);
}

// `noBlocks`: a binary64 plan without the 8 x 8 block form (the second attempt, when a row of a block
// chunk turned out to have more virtual rows than the block layout has places for).
// `twin`: the extraction is there already, in the device arrays of a partition that was made on the
// device (mx_plan_create hands it in; the matrix arguments are not looked at then).
int mxp::create_plan_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev,
                            float tau_c, float tau_r, int flags, mx_plan **out, bool noBlocks, const mx::PartitionTwin *twin)
{
    const char *who = twin ? "mx_plan_create" : "mx_plan_create_device";
    int rc;
    if (!twin) {
        if (!out || (dtype != MX_F64 && dtype != MX_F16) || rows < 1 || cols < 1 || nnz < 0 || !rowPtr_dev ||
            (nnz > 0 && (!colInd_dev || !val_dev)) || !(tau_c >= 0.0f && tau_c <= 1.0f) || !(tau_r >= 0.0f && tau_r <= 1.0f)) {
            set_error(std::string(who) + ": bad argument");
            return MX_ERR_ARG;
        }
        *out = nullptr;
        if (tau_c == 0.0f && tau_r == 0.0f)  // nothing to extract
            return mx_plan_create_device_csr(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, flags, out);
        if ((rc = need_device())) return rc;
        if ((rc = mx::check_csr_device(rows, cols, nnz, rowPtr_dev, colInd_dev, nullptr, who))) return rc;
    } else {
        *out = nullptr;
        if ((rc = need_device())) return rc;
    }
    // (what a failure has to release, also one that arrives as an exception)
    mx_plan *plan = nullptr;
    int *partPtr = nullptr, *partCol = nullptr;
    void *partVal = nullptr;
    char *stripRows = nullptr;
    auto fail = [&](int code) {
        (void)hipFree(partPtr);
        (void)hipFree(partCol);
        (void)hipFree(partVal);
        (void)hipFree(stripRows);
        partPtr = partCol = nullptr;
        partVal = nullptr;
        stripRows = nullptr;
        mx_plan_destroy(plan);
        plan = nullptr;
        return code;
    };
    try {
        hipDeviceProp_t prop;
        int dev = 0;
        MX_HIP(hipGetDevice(&dev));
        MX_HIP(hipGetDeviceProperties(&prop, dev));
        const int nCU = std::max(1, prop.multiProcessorCount);
        const int fragM = mx::kFragM, fragK = mx::frag_k(dtype);
        const bool noTiles = (flags & MX_PLAN_NO_TILES) != 0, allTiles = !noTiles && (flags & MX_PLAN_ALL_TILES) != 0;
        const bool wantStrips = dtype == MX_F16 && !noTiles && !allTiles && !mx::opt().no_strips;
        const bool wantBlocks = dtype == MX_F64 && !noTiles && !allTiles && !noBlocks && !mx::opt().no_blocks;
        // (the smallest count that passes `(double)vals >= gate * fragM * fragK`; every fragment that holds anything
        // with MX_PLAN_ALL_TILES)
        const double need = tile_gate(dtype) * fragM * fragK;
        int minVals = (int)need;
        while ((double)minVals < need) ++minVals;
        if (allTiles) minVals = 1;
        mx::HybridDevice H;
        mx::HybridCounts cnt;
        PhaseLog phase;
        if (twin) rc = H.adopt(*twin, minVals, !noTiles, wantStrips, wantBlocks, &cnt, nullptr);
        else
            rc = H.analyse(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, tau_c, tau_r, minVals, !noTiles, wantStrips, wantBlocks, &cnt,
                           nullptr);
        if (rc) return rc;
        phase(twin ? "gate, strip rows (device, on the partition's device arrays)" : "extraction, gate, strip rows (device)");
        if (cnt.blocks64) cnt.generalFrags = cnt.generalEntries = 0;  // the general tiles are not used beside blocks
        int worth = 2;
        if (noTiles) worth = 0;
        else if (!(flags & (MX_PLAN_KEEP_TILES | MX_PLAN_ALL_TILES)))
            worth = tiles_worth(dtype, fragM, fragK, cnt.blocks64, (double)cnt.generalEntries, (double)cnt.generalFrags,
                                (double)cnt.stripEntries, (double)cnt.stripBlocks, (double)cnt.stripBlocksOff, (double)nnz);
        const bool keepBlocks = worth >= 1 && cnt.blocks64 && cnt.stripBlocks > 0;
        const bool keepStrips = worth >= 1 && !cnt.blocks64 && cnt.stripBlocks > 0;
        const bool keepGeneral = worth == 2 && cnt.generalFrags > 0;

        plan = new (std::nothrow) mx_plan();
        if (!plan) {
            set_error(std::string(who) + ": out of memory");
            return MX_ERR_ALLOC;
        }
        plan->dtype = dtype;
        plan->rows = rows;
        plan->cols = cols;
        plan->nnz = nnz;
        plan->prep_route = 1;
        plan->ext_dCols = cnt.dCols;
        plan->ext_dRows = cnt.dRows;
        plan->ext_nnzRowD = cnt.nnzRowD;
        plan->ext_frags = cnt.frags;
        if (hipStreamCreate(&plan->stream) != hipSuccess || hipEventCreate(&plan->ev0) != hipSuccess ||
            hipEventCreate(&plan->ev1) != hipSuccess) {
            set_error(std::string(who) + ": could not create stream/events");
            return fail(MX_ERR_DEVICE);
        }
        {
            void *fixed = nullptr;
            if (mx::static_scratch(&fixed) != hipSuccess) {
                (void)hipGetLastError();
                set_error(std::string(who) + ": hipGetSymbolAddress failed for the fixed array of sums");
                return fail(MX_ERR_DEVICE);
            }
        }
        if (keepGeneral) {
            // the general tile form first: the walk over A_dd that assembles the CSR part also fills its values
            std::vector<int> chunkBlocks, stepDesc, chunkBlock0, waveDesc;
            long long totalBlocks = 0;
            if ((rc = H.tile_chunks(keepStrips, chunkBlocks))) return fail(rc);
            if (!chunkBlocks.empty()) {
                const int BS = fragM * fragK;
                if ((rc = plan_tile_steps(chunkBlocks, mx::tile_slots(dtype), BS, 2, nCU, 10, stepDesc, chunkBlock0, waveDesc, &totalBlocks)))
                    return fail(rc);
                mx::DeviceTiles &T = plan->tiles;
                T.chunkNum = (int)chunkBlocks.size();
                T.frags = (int)cnt.generalFrags;
                T.vals = (int)cnt.generalEntries;
                T.stored = totalBlocks * BS;
                T.steps = (int)(stepDesc.size() / 10);
                T.dense = false;
                T.nWaves = (int)(waveDesc.size() / 8);
                if ((rc = H.tile_layout(keepStrips, stepDesc, chunkBlock0, waveDesc, totalBlocks, T))) return fail(rc);
                plan->tile_nnz += T.vals;
                phase("tile steps (device)");
            }
        }
        std::vector<int> blockStepDesc, blockRows;  // binary64 blocks: their steps and the block row of every chunk
        if (keepBlocks) {
            std::vector<int> chunkBlocks, chunkBlock0, waveDesc;
            long long totalBlocks = 0;
            if ((rc = H.block_chunks(chunkBlocks, blockRows))) return fail(rc);
            if ((rc = plan_tile_steps(chunkBlocks, 8, 64, 1, nCU, 10, blockStepDesc, chunkBlock0, waveDesc, &totalBlocks))) return fail(rc);
            mx::DeviceTiles &T = plan->strips;
            T.chunkNum = (int)chunkBlocks.size();
            T.frags = (int)cnt.stripBlocks;
            T.vals = (int)cnt.stripEntries;
            T.stored = totalBlocks * 64;
            T.steps = (int)(blockStepDesc.size() / 10);
            T.dense = T.steps > 0;
            T.nWaves = (int)(waveDesc.size() / 8);
            if ((rc = H.block_layout(blockStepDesc, chunkBlock0, waveDesc, totalBlocks, T))) return fail(rc);
            plan->tile_nnz += T.vals;
            phase("block steps (device)");
        }
        int partNnz = 0;
        if ((rc = H.csr_part(keepStrips, keepGeneral, keepBlocks, &partPtr, &partCol, &partVal, &partNnz, &stripRows))) return fail(rc);
        phase("CSR part assembled (device)");
        std::pair<std::vector<int>, std::vector<int>> seg;  // virtual rows of every row (slice form), for the blocks
        if ((rc = setup_csr_part_device(plan, partNnz, partPtr, partCol, partVal, flags, stripRows, keepBlocks ? &seg : nullptr)))
            return fail(rc);
        phase("CSR part layout (device)");
        if (keepBlocks && plan->csr_variant == 1) {
            // the blocks ride in the combine kernel's launch: where each of their rows finds the sums of its
            // virtual rows (eight places per row; a row with more sends the whole plan back to be made without blocks)
            const int steps = plan->strips.steps;
            std::vector<int> vidx((size_t)steps * 128, -1);
            bool fits = true;
            for (int st = 0; st < steps && fits; ++st) {
                const int *d = &blockStepDesc[(size_t)st * 10];
                if (!(d[2] & 1)) continue;
                for (int half = 0; half < 2; ++half) {
                    const int chunk = half == 0 ? d[0] : d[1];
                    if (chunk < 0) continue;
                    for (int i = 0; i < 8; ++i) {
                        const int r = blockRows[chunk] * 8 + i;
                        if (r >= rows) continue;
                        const int a = seg.first[r], n = seg.first[r + 1] - a;
                        if (n > 8) fits = false;
                        for (int j = 0; j < std::min(n, 8); ++j) vidx[(size_t)st * 128 + half * 64 + i * 8 + j] = seg.second[a + j];
                    }
                }
            }
            if (!fits) {
                fail(MX_OK);
                return create_plan_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, tau_c, tau_r, flags, out, true, twin);
            }
            if ((rc = upload(&plan->strips.vidx, vidx.data(), vidx.size(), 128))) return fail(rc);
        }
        if (keepStrips) {
            std::vector<int> stepDesc, chunkBlock0, waveDesc;
            long long totalBlocks = 0;
            if ((rc = plan_tile_steps(cnt.stripChunkBlocks, 8, 64, 2, nCU, 8, stepDesc, chunkBlock0, waveDesc, &totalBlocks))) return fail(rc);
            mx::DeviceTiles &T = plan->strips;
            T.chunkNum = (int)cnt.stripChunkBlocks.size();
            T.frags = (int)cnt.stripBlocks;
            T.vals = (int)cnt.stripEntries;
            T.stored = totalBlocks * 64;
            T.steps = (int)(stepDesc.size() / 8);
            T.dense = T.steps > 0;
            T.nWaves = (int)(waveDesc.size() / 8);
            if ((rc = H.strip_layout(stepDesc, chunkBlock0, waveDesc, totalBlocks, T))) return fail(rc);
            T.ownedRows = true;  // strip rows have nothing in the CSR part, which leaves zeros there
            plan->tile_nnz += T.vals;
            phase("strip steps (device)");
        }
        if (dtype == MX_F16 && plan->tiles.nWaves > 0) {
            // (general tiles share rows with the CSR part: its sums stay binary32 until the tile kernel has added its own)
            if ((rc = upload_bytes(&plan->ywide, nullptr, 0, (size_t)std::max(rows, 1) * sizeof(float)))) return fail(rc);
        }
        (void)hipFree(partPtr);
        (void)hipFree(partCol);
        (void)hipFree(partVal);
        (void)hipFree(stripRows);
        decide_keep(plan, flags);  // (again, now that the tile part is known: it counts towards what a product touches)
        *out = plan;
        return MX_OK;
    } catch (const std::bad_alloc &) {
        set_error(std::string(who) + ": out of memory");
        return fail(MX_ERR_ALLOC);
    }
}

