// The layouts the kernels run on, made on the host: the row tiles and the column slices of the CSR part
// (with the one-launch form of the slices), the tile part in its three forms, and their upload; the views
// of the slice layout that tests walk.
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

namespace mxp {


int need_device()
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        (void)hipGetLastError();
        set_error("no HIP device available (this library has no CPU fallback)");
        return MX_ERR_DEVICE;
    }
    return MX_OK;
}


int upload_bytes(void **dst, const void *src, size_t n, size_t pad)
{
    return upload<unsigned char>((unsigned char **)dst, (const unsigned char *)src, n, pad);
}

// Rows of each CSR-kernel workgroup (the role of pre_startRowPerBlock,
// src/spmv_kernel/cdSpMV.cu:4-27, but row-aligned): greedily pack whole rows while their
// entries, counted from the tile's aligned start, fit one tile; a longer row stands alone.
// One descriptor {first row, end row, first entry, end entry} per workgroup.
void pack_rows(const int *rowPtr, int rows, int npt, std::vector<int> &desc)
{
    const int tile = 256 * npt;
    desc.clear();
    int r = 0;
    while (r < rows) {
        const int base = rowPtr[r] & ~(npt - 1);
        int r1 = r + 1;
        while (r1 < rows && rowPtr[r1 + 1] - base <= tile && r1 - r < tile) ++r1;
        desc.push_back(r);
        desc.push_back(r1);
        desc.push_back(rowPtr[r]);
        desc.push_back(rowPtr[r1]);
        r = r1;
    }
}

void free_csr(mx::DeviceCsr &A)
{
    (void)hipFree(A.rowPtr);
    (void)hipFree(A.col);
    (void)hipFree(A.col16);
    (void)hipFree(A.colBase);
    (void)hipFree(A.val);
    (void)hipFree(A.codes);
    (void)hipFree(A.dict);
    (void)hipFree(A.blockDesc);
    A = mx::DeviceCsr();
}

void free_tiles(mx::DeviceTiles &T)
{
    (void)hipFree(T.waveDesc);
    (void)hipFree(T.hdr);
    (void)hipFree(T.atox);
    (void)hipFree(T.tcVal);
    (void)hipFree(T.vidx);
    T = mx::DeviceTiles();
}

void free_slices(mx::DeviceSlices &P)
{
    (void)hipFree(P.waveDesc);
    (void)hipFree(P.chunkEnd);
    (void)hipFree(P.wgDesc);
    (void)hipFree(P.ecol);
    (void)hipFree(P.eval);
    (void)hipFree(P.ecode);
    (void)hipFree(P.dict);
    (void)hipFree(P.partial);
    (void)hipFree(P.rowInfo);
    (void)hipFree(P.lightRow);
    (void)hipFree(P.lightIdx);
    (void)hipFree(P.heavyInfo);
    (void)hipFree(P.segIdx);
    (void)hipFree(P.wgGroups);
    (void)hipFree(P.groupNeed);
    (void)hipFree(P.groupCount);
    (void)hipFree(P.fusedTarget);
    (void)hipFree(P.fusedSums);
    (void)hipFree(P.claim);
    P = mx::DeviceSlices();
}

// Number of column slices csr_slice_kernel would cut x into, or 0 when the matrix does not suit
// it: every slice costs at least one workgroup that copies 128 KB of x, which has to stay small
// next to the matrix itself.
int slice_count(mx_dtype dtype, int rows, int cols, int nnz, int nCU)
{
    if (cols < 1 || rows < 1 || nnz < 4096) return 0;
    const int S = (cols + mx::slice_cols(dtype) - 1) / mx::slice_cols(dtype);
    if (S > 2 * nCU) return 0;
    if ((double)S * mx::kSliceBytes > 2.0 * (double)nnz * (mx::elem_size(dtype) + 2)) return 0;
    return S;
}

// The distinct values (bit patterns) of a matrix, when there are at most `most` (<= 256):
// codes[p] names the value of entry p, dict holds the values padded with zeros to 256.  False when
// there are more.
bool make_value_dict(int es, const void *val, int nnz, std::vector<unsigned char> &codes, std::vector<unsigned char> &dict,
                     int *nDict, int most)
{
    codes.assign((size_t)nnz, 0);
    dict.assign((size_t)256 * es, 0);
    int nd = 0;
    if (es == 8) {
        const uint64_t *v = (const uint64_t *)val;
        uint64_t seen[256];
        for (int p = 0; p < nnz; ++p) {
            int k = 0;
            while (k < nd && seen[k] != v[p]) ++k;  // few values: a short scan, most hits early
            if (k == nd) {
                if (nd == most) return false;
                seen[nd++] = v[p];
            }
            codes[p] = (unsigned char)k;
        }
        std::memcpy(dict.data(), seen, (size_t)nd * 8);
    } else {
        const uint16_t *v = (const uint16_t *)val;
        std::vector<int> codeOf(65536, -1);
        uint16_t seen[256];
        for (int p = 0; p < nnz; ++p) {
            int k = codeOf[v[p]];
            if (k < 0) {
                if (nd == most) return false;
                k = nd;
                codeOf[v[p]] = nd;
                seen[nd++] = v[p];
            }
            codes[p] = (unsigned char)k;
        }
        std::memcpy(dict.data(), seen, (size_t)nd * 2);
    }
    *nDict = nd;
    return true;
}


// A workgroup of the slice layout on its way into the descriptors: its slice and, per wave, the
// chunks (indices into the slice's list) in the order the wave streams them.
struct SliceWg {
    int slice = 0;
    std::vector<int> chunk[mx::kSliceWaves];
    int waveSteps[mx::kSliceWaves] = {};
    int waveCost[mx::kSliceWaves] = {};  // steps plus what the chunk ends cost: what the dealing evens out
    long long steps = 0;  // stored steps (every wave's stream rounded up to whole batches)
    int chunks = 0;
};

// `mine` (chunks of slice q, in the order they are to be dealt) to the waves of `w`: each to the wave
// with the fewest steps so far.
void deal_to_waves(SliceWg &w, int q, const std::vector<int> &mine, const std::vector<mx::SliceChunk> &ch, int SPB)
{
    const int W = mx::kSliceWaves;
    w.slice = q;
    w.steps = 0;
    for (int k = 0; k < W; ++k) {
        w.waveSteps[k] = w.waveCost[k] = 0;
        w.chunk[k].clear();
    }
    // (a wave that ends a chunk stores 64 sums and starts over: measured, that costs it as much as about two
    // steps of its stream, and thirty short chunks take a wave far longer than one long chunk of as many steps)
    for (int c : mine) {
        int best = 0;
        for (int k = 1; k < W; ++k)
            if (w.waveCost[k] < w.waveCost[best]) best = k;
        w.chunk[best].push_back(c);
        w.waveSteps[best] += ch[c].steps;
        w.waveCost[best] += ch[c].steps + mx::kSliceChunkCost;
    }
    w.chunks = (int)mine.size();
    for (int k = 0; k < W; ++k) w.steps += (w.waveSteps[k] + SPB - 1) / SPB * SPB;
}

// The descriptors the kernels read and the place of every chunk in the streams, from the workgroups
// and their waves' chunks.
int emit_slice_plan(const std::vector<SliceWg> &wgs, const std::vector<std::vector<mx::SliceChunk>> &sliceChunks, int SPB, int E,
                           mx::SlicePlan &P)
{
    const int W = mx::kSliceWaves;
    const int nWG = (int)wgs.size();
    long long totalSteps = 0, totalChunks = 0;
    std::vector<long long> wgStep((size_t)nWG + 1, 0), wgChunk((size_t)nWG + 1, 0);
    int maxWgChunks = 0;
    for (int b = 0; b < nWG; ++b) {
        wgStep[b] = totalSteps;
        wgChunk[b] = totalChunks;
        totalSteps += wgs[b].steps;
        totalChunks += wgs[b].chunks;
        maxWgChunks = std::max(maxWgChunks, wgs[b].chunks);
    }
    if (totalSteps * 64 * E > 2000000000LL || totalChunks * 64 > 2000000000LL) {
        set_error("slice layout: too many entries for 32-bit offsets");
        return MX_ERR_ARG;
    }
    P.nWG = nWG;
    P.maxWgChunks = maxWgChunks;
    P.totalSteps = totalSteps;
    P.totalChunks = totalChunks;
    P.wgDesc.assign((size_t)nWG * 4 + 4, 0);
    P.waveDesc.assign((size_t)nWG * W * 4 + 4, 0);
    P.chunkEnd.assign((size_t)totalChunks + 64, 0);
    P.chunkSlice.assign((size_t)totalChunks, 0);
    P.chunkFirst.assign((size_t)totalChunks, 0);
    P.chunkN.assign((size_t)totalChunks, 0);
    P.chunkSteps.assign((size_t)totalChunks, 0);
    P.chunkStep0.assign((size_t)totalChunks, 0);
    for (int b = 0; b < nWG; ++b) {
        const SliceWg &G = wgs[b];
        const int q = G.slice;
        const auto &ch = sliceChunks[q];
        long long step = wgStep[b], chunk = wgChunk[b];
        P.wgDesc[(size_t)b * 4 + 0] = q;
        P.wgDesc[(size_t)b * 4 + 1] = (int)chunk;
        P.wgDesc[(size_t)b * 4 + 2] = G.chunks;
        for (int w = 0; w < W; ++w) {
            int *d = &P.waveDesc[((size_t)b * W + w) * 4];
            d[0] = (int)(step / SPB);                   // first batch
            d[1] = (G.waveSteps[w] + SPB - 1) / SPB;    // batches
            d[2] = (int)(chunk - wgChunk[b]);           // first chunk, counted inside the workgroup
            d[3] = (int)G.chunk[w].size();
            int rel = 0;
            for (int c : G.chunk[w]) {
                P.chunkSlice[chunk] = q;
                P.chunkFirst[chunk] = ch[c].first;
                P.chunkN[chunk] = ch[c].n;
                P.chunkSteps[chunk] = ch[c].steps;
                P.chunkStep0[chunk] = step;
                step += ch[c].steps;
                rel += ch[c].steps;
                P.chunkEnd[chunk++] = rel;
            }
            step = (step + SPB - 1) / SPB * SPB;
        }
    }
    return MX_OK;
}

// A virtual row on its way into the slice layout.
struct VRow {
    int start, len, slice;  // start: into the entries in (row, column) order
    int kind;               // of its row: 0 = this is its only virtual row, 1 = light, 2 = heavy
};

// The decisions of the one-launch form (see DeviceSlices).  Every XCD gets a contiguous range of whole
// groups of rows with an eighth of the entries, and budget / 8 logical workgroups; a slice with
// entries in those rows gets workgroups in proportion to its entries there, and each of them a
// contiguous run of the slice's virtual rows (in row order) with an even share of the entries.  A
// workgroup's virtual rows are then ordered by length and cut into chunks of 64, which go to its waves
// longest first.  The groups a workgroup counts off are those of its rows, stretched so that the
// workgroups of one (XCD, slice) cover all groups of the XCD between them: every group is counted off by
// at least one workgroup, also one whose rows have no entries.  Fills `sorted`, `sliceChunks` and SP and
// returns true; false (nothing filled) when the matrix does not suit the form: a budget that is not a
// multiple of eight, fewer workgroups per XCD than slices with entries in its rows, an XCD without
// entries.  (SP.nWG = -1: an error, which is set.)
static bool plan_fused(mx_dtype dtype, int budget, int S, int rows, int nGroups, int cap, const std::vector<int> &rowStart,
                       const std::vector<int> &segPtr, const std::vector<VRow> &vr, std::vector<int> &sorted,
                       std::vector<std::vector<mx::SliceChunk>> &sliceChunks, mx::SlicePlan &SP)
{
    const int E = mx::slice_step_entries(dtype), SPB = mx::kSliceBatchEntries / E, X = mx::kFusedXcds, GR = mx::kFusedGroupRows;
    const int nV = (int)vr.size(), nk = budget / X;
    const long long nnz = rowStart[rows];
    if (budget < X || budget % X || nGroups < X || nnz == 0) return false;
    // the groups of every XCD
    std::vector<int> xg((size_t)X + 1, 0);
    {
        int g = 0;
        for (int k = 1; k < X; ++k) {
            const long long target = nnz * k / X;
            while (g < nGroups && (long long)rowStart[std::min(rows, g * GR)] < target) ++g;
            xg[k] = std::min(std::max(g, xg[k - 1] + 1), nGroups - (X - k));
            g = xg[k];
        }
        xg[X] = nGroups;
    }
    std::vector<int> xcdOfGroup((size_t)nGroups);
    for (int k = 0; k < X; ++k)
        for (int g = xg[k]; g < xg[k + 1]; ++g) xcdOfGroup[g] = k;
    std::vector<int> rowOf((size_t)nV);
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int t = segPtr[r]; t < segPtr[r + 1]; ++t) rowOf[t] = r;
    // entries and virtual rows of every (XCD, slice)
    std::vector<long long> partEntries((size_t)X * S, 0);
    std::vector<int> partVrows((size_t)X * S, 0);
    for (int t = 0; t < nV; ++t) {
        const size_t p = (size_t)xcdOfGroup[rowOf[t] / GR] * S + vr[t].slice;
        partEntries[p] += vr[t].len;
        ++partVrows[p];
    }
    // workgroups of every part, and the first logical workgroup of each
    std::vector<int> partWgs((size_t)X * S, 0), partBase((size_t)X * S, 0);
    for (int k = 0; k < X; ++k) {
        long long xcdEntries = 0;
        int busy = 0;
        for (int q = 0; q < S; ++q) {
            xcdEntries += partEntries[(size_t)k * S + q];
            busy += partVrows[(size_t)k * S + q] > 0;
        }
        if (busy == 0 || busy > nk) return false;
        std::vector<double> want((size_t)S, 0.0);
        int used = 0;
        for (int q = 0; q < S; ++q) {
            const size_t p = (size_t)k * S + q;
            if (partVrows[p] == 0) continue;
            want[q] = (double)partEntries[p] * nk / (double)xcdEntries;
            partWgs[p] = std::min(std::max(1, (int)want[q]), partVrows[p]);
            used += partWgs[p];
        }
        while (used > nk) {  // rounding small parts up took more than there is: from the part furthest above its share
            int best = -1;
            for (int q = 0; q < S; ++q) {
                const size_t p = (size_t)k * S + q;
                if (partWgs[p] > 1 && (best < 0 || partWgs[p] - want[q] > partWgs[(size_t)k * S + best] - want[best])) best = q;
            }
            if (best < 0) return false;
            --partWgs[(size_t)k * S + best];
            --used;
        }
        while (used < nk) {  // what rounding down left over goes where most is missing
            int best = -1;
            for (int q = 0; q < S; ++q) {
                const size_t p = (size_t)k * S + q;
                if (partVrows[p] > partWgs[p] && (best < 0 || want[q] - partWgs[p] > want[best] - partWgs[(size_t)k * S + best])) best = q;
            }
            if (best < 0) break;  // fewer virtual rows than workgroups: the rest stay empty
            ++partWgs[(size_t)k * S + best];
            ++used;
        }
        int b = k * nk;
        for (int q = 0; q < S; ++q) {
            partBase[(size_t)k * S + q] = b;
            b += partWgs[(size_t)k * S + q];
        }
    }
    // every virtual row to its workgroup: inside a part in row order, cut where the running entries pass
    // the next share
    std::vector<int> wgOf((size_t)nV), wgCount((size_t)budget + 1, 0), rowLo((size_t)budget, INT_MAX), rowHi((size_t)budget, -1);
    {
        std::vector<long long> run((size_t)X * S, 0);
        std::vector<int> seen((size_t)X * S, 0);
        for (int t = 0; t < nV; ++t) {
            const size_t p = (size_t)xcdOfGroup[rowOf[t] / GR] * S + vr[t].slice;
            const int w = partWgs[p];
            // (at least one virtual row per workgroup: the j-th workgroup starts no later than at the part's
            // (vrows - w + j)-th virtual row and no earlier than at its j-th)
            int j = partEntries[p] > 0 ? (int)(((run[p] + vr[t].len / 2) * w) / partEntries[p]) : 0;
            j = std::min(std::min(j, w - 1), seen[p]);
            j = std::max(j, w - (partVrows[p] - seen[p]));
            run[p] += vr[t].len;
            ++seen[p];
            const int b = partBase[p] + j;
            wgOf[t] = b;
            ++wgCount[b + 1];
            rowLo[b] = std::min(rowLo[b], rowOf[t]);
            rowHi[b] = std::max(rowHi[b], rowOf[t]);
        }
    }
    // (wgOf rises with t inside a part, so j never skips a workgroup downwards; a skipped one upwards stays empty)
    for (int b = 0; b < budget; ++b) wgCount[b + 1] += wgCount[b];
    // virtual rows by (workgroup, length descending), row order kept among equals: two counting sorts
    {
        std::vector<int> byLen((size_t)nV), at((size_t)cap + 2, 0);
        for (int t = 0; t < nV; ++t) at[(size_t)(cap - vr[t].len) + 1]++;
        for (int k = 0; k <= cap; ++k) at[k + 1] += at[k];
        for (int t = 0; t < nV; ++t) byLen[at[cap - vr[t].len]++] = t;
        std::vector<int> cur(wgCount.begin(), wgCount.end() - 1);
        for (int i = 0; i < nV; ++i) sorted[cur[wgOf[byLen[i]]]++] = byLen[i];
    }
    // chunks, waves, groups
    std::vector<SliceWg> wgs((size_t)budget);
    SP.wgGroups.assign((size_t)budget * 2 + 2, 0);
    SP.groupNeed.assign((size_t)nGroups + 1, 0);
    SP.nGroups = nGroups;
    SP.maxWgGroups = 0;
    for (int k = 0; k < X; ++k)
        for (int q = 0; q < S; ++q) {
            const size_t p = (size_t)k * S + q;
            const int w = partWgs[p];
            // the workgroups of the part that hold anything, in order
            std::vector<int> live;
            for (int j = 0; j < w; ++j)
                if (wgCount[partBase[p] + j + 1] > wgCount[partBase[p] + j]) live.push_back(partBase[p] + j);
            for (size_t i = 0; i < live.size(); ++i) {
                const int b = live[i];
                if ((wgCount[b + 1] - wgCount[b] + 63) / 64 > mx::kFusedWgChunks) return false;  // (its targets would not fit the LDS)
                std::vector<int> mine;
                for (int f = wgCount[b]; f < wgCount[b + 1]; f += 64) {
                    mine.push_back((int)sliceChunks[q].size());
                    sliceChunks[q].push_back({f, std::min(64, wgCount[b + 1] - f), (vr[sorted[f]].len + E - 1) / E});
                }
                deal_to_waves(wgs[b], q, mine, sliceChunks[q], SPB);
                const int ga = i == 0 ? xg[k] : rowLo[b] / GR;
                const int gb = i + 1 == live.size() ? xg[k + 1] - 1 : std::max(rowHi[b] / GR, rowLo[live[i + 1]] / GR - 1);
                SP.wgGroups[(size_t)b * 2] = ga;
                SP.wgGroups[(size_t)b * 2 + 1] = gb - ga + 1;
                if (gb - ga + 1 > mx::kFusedWgGroups) return false;  // (a lane per group counts it off)
                SP.maxWgGroups = std::max(SP.maxWgGroups, gb - ga + 1);
                for (int g = ga; g <= gb; ++g) ++SP.groupNeed[g];
            }
        }
    for (int b = 0; b < budget; ++b)
        if (wgs[b].chunks == 0) {  // a workgroup without virtual rows: nothing to stream, no group to count off
            int q = 0;
            while (q < S - 1 && partVrows[(size_t)(b / nk) * S + q] == 0) ++q;
            deal_to_waves(wgs[b], q, std::vector<int>(), sliceChunks[q], SPB);
            SP.wgGroups[(size_t)b * 2] = xg[b / nk];
        }
    if (emit_slice_plan(wgs, sliceChunks, SPB, E, SP)) SP.nWG = -1;
    return true;
}

}  // namespace mxp

int mx::plan_fused_records(mx_dtype dtype, int budget, int S, int rows, int cap, const int *rowPtr, const int *segPtrIn, const int *vSlice,
                           const int *vLen, int nV, int mode, std::vector<int> &sorted, SlicePlan &SP, int *places)
{
    const int GR = mx::kFusedGroupRows, nGroups = (rows + GR - 1) / GR;
    int most = 0;
    for (int r = 0; r < rows; ++r) most = std::max(most, segPtrIn[r + 1] - segPtrIn[r]);
    // the form needs every row's sums in at most eight places
    if (most > mx::kSliceLightSegs || (long long)nGroups * mx::kSliceLightSegs * GR > 2000000000LL) return 0;
    std::vector<mxp::VRow> vr((size_t)nV);
    for (int t = 0; t < nV; ++t) vr[t] = {0, vLen[t], vSlice[t], 0};
    const std::vector<int> rowStart(rowPtr, rowPtr + rows + 1), segPtr(segPtrIn, segPtrIn + rows + 1);
    std::vector<std::vector<mx::SliceChunk>> sliceChunks((size_t)S);
    sorted.assign((size_t)nV, 0);
    SP = mx::SlicePlan();
    const bool suits = mxp::plan_fused(dtype, budget, S, rows, nGroups, cap, rowStart, segPtr, vr, sorted, sliceChunks, SP);
    if (SP.nWG < 0) return MX_ERR_ARG;  // (the error is set)
    // the slowest workgroup reads the sums of every group it covers after its last chunk: beyond kFusedAddBytes
    // of them that tail outweighs the launch saved, and the form is left unless it was asked for
    const long long addBytes = (long long)SP.maxWgGroups * std::max(most, 1) * GR * (dtype == MX_F64 ? 8 : 4);
    if (!suits || (mode != 1 && addBytes > mx::kFusedAddBytes)) {
        SP = mx::SlicePlan();
        sorted.clear();
        return 0;
    }
    // (as many places as the longest list of virtual rows has: the one who adds reads every place of a row)
    *places = std::max(most, 1);
    return 1;
}

void mx::fused_targets(int rows, int nGroups, int places, long long totalChunks, const int *segPtr, const int *segIdx, std::vector<int> &target)
{
    // the k-th virtual row of row r at ((r / GR) * places + k) * GR + r % GR; the padding lanes of a chunk at the
    // spare places behind the last group
    const int GR = mx::kFusedGroupRows;
    const size_t spare = (size_t)nGroups * places * GR;
    target.assign((size_t)totalChunks * 64, 0);
    for (size_t v = 0; v < target.size(); ++v) target[v] = (int)(spare + (v & 63));
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r)
        for (int t = segPtr[r]; t < segPtr[r + 1]; ++t) target[segIdx[t]] = (int)(((size_t)(r / GR) * places + (t - segPtr[r])) * GR + r % GR);
}

namespace mxp {

// `elsewhere` (optional) marks rows whose result another kernel writes: 1 = the strips of a binary16
// plan (the row has nothing here), 2 = the 8 x 8 blocks of a binary64 plan, whose waves fetch the sums
// of the row's virtual rows themselves.  Such rows get rowInfo -2 and appear in no list, so that the
// combine kernel's own kinds neither zero them nor add to them.
// `fused`: lay the virtual rows out for the one-launch form (ordered by group of rows before length,
// workgroups dealt per XCD); D.fused tells whether the matrix suited it -- when it does not (a row
// with more than eight virtual rows, more slices than workgroups in an XCD's rows, row subsets or
// rows written elsewhere) the ordinary layout is made.
int build_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                 const char *sel, HostSlices &D, const char *elsewhere, int fused)
{
    const int es = mx::elem_size(dtype), E = mx::slice_step_entries(dtype);
    const int BE = mx::kSliceBatchEntries;
    const int SW = mx::slice_cols(dtype), W = mx::kSliceWaves;
    // entries of the selected rows, row by row, ascending by column (stable)
    std::vector<int> selPtr((size_t)rows + 1, 0);
    for (int r = 0; r < rows; ++r) selPtr[r + 1] = selPtr[r] + ((!sel || sel[r]) ? rowPtr[r + 1] - rowPtr[r] : 0);
    const int nnz = selPtr[rows];
    std::vector<int> ord((size_t)nnz);
    // a lane's fair share of the entries; virtual rows are cut to that, so that no chunk is more
    // than a wave's share and the chunks can be dealt evenly (measured: half of it costs more
    // in extra virtual rows than it gains in balance)
    const int budget = std::max(nCU, 1);
    const long long fair = (long long)nnz / ((long long)budget * W * 64);
    int cap = (int)std::min<long long>(512, std::max<long long>(16, (fair + BE - 1) / BE * BE));
    if (const int v = mx::opt().slice_cap)  // for tuning runs
        if (v >= BE && v <= 4096) cap = v / BE * BE;
    std::vector<int> segPtr((size_t)rows + 1, 0);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int r = 0; r < rows; ++r) {
        const int n = selPtr[r + 1] - selPtr[r];
        if (n == 0) continue;
        int *o = &ord[selPtr[r]];
        std::iota(o, o + n, rowPtr[r]);
        bool sorted = true;
        for (int k = 1; k < n && sorted; ++k) sorted = col[o[k - 1]] <= col[o[k]];
        if (!sorted) std::stable_sort(o, o + n, [&](int a, int b) { return col[a] < col[b]; });
        int nv = 0;
        for (int k = 0; k < n;) {
            const int q = col[o[k]] / SW;
            int e = k;
            while (e < n && e - k < cap && col[o[e]] / SW == q) ++e;
            ++nv;
            k = e;
        }
        segPtr[r + 1] = nv;
    }
    for (int r = 0; r < rows; ++r) segPtr[r + 1] += segPtr[r];
    const int nV = segPtr[rows];
    std::vector<VRow> vr((size_t)nV);
#pragma omp parallel for schedule(dynamic, 1024)
    for (int r = 0; r < rows; ++r) {
        const int n = selPtr[r + 1] - selPtr[r];
        const int *o = n ? &ord[selPtr[r]] : nullptr;
        int t = segPtr[r];
        const int nv = segPtr[r + 1] - segPtr[r], kind = nv <= 1 ? 0 : nv <= mx::kSliceLightSegs ? 1 : 2;
        for (int k = 0; k < n;) {
            const int q = col[o[k]] / SW;
            int e = k;
            while (e < n && e - k < cap && col[o[e]] / SW == q) ++e;
            vr[t++] = {selPtr[r] + k, e - k, q, kind};
            k = e;
        }
    }
    // the one-launch form needs every row's sums in at most eight places
    const int GR = mx::kFusedGroupRows, nGroups = (rows + GR - 1) / GR;
    int most = 0;
    if (fused) {
        for (int r = 0; r < rows; ++r) most = std::max(most, segPtr[r + 1] - segPtr[r]);
        if (sel || elsewhere || most > mx::kSliceLightSegs || (long long)nGroups * mx::kSliceLightSegs * GR > 2000000000LL) fused = false;
    }
    std::vector<int> keyStart, sorted((size_t)nV);
    std::vector<std::vector<mx::SliceChunk>> sliceChunks(S);
    mx::SlicePlan SP;
    const size_t perSlice = (size_t)(cap + 1) * 3;
    if (fused) {
        const bool suits = plan_fused(dtype, budget, S, rows, nGroups, cap, selPtr, segPtr, vr, sorted, sliceChunks, SP);
        // the slowest workgroup reads the sums of every group it covers after its last chunk: beyond kFusedAddBytes
        // of them that tail outweighs the launch saved, and the form is left unless it was asked for
        const long long addBytes = (long long)SP.maxWgGroups * std::max(most, 1) * GR * (dtype == MX_F64 ? 8 : 4);
        fused = suits && (fused == 1 || addBytes <= mx::kFusedAddBytes) ? fused : 0;
        if (SP.nWG < 0) return MX_ERR_ARG;  // (the error is set)
        if (!fused) {  // the matrix does not suit the form: the ordinary layout, from a clean slate
            for (auto &v : sliceChunks) v.clear();
            SP = mx::SlicePlan();
        }
    }
    if (!fused) {
        // virtual rows by (slice, length descending, kind of row), row order kept among equals: a
        // counting sort.  The kind keeps the sums that one workgroup of the combine kernel gathers
        // close together: consecutive heavy rows have virtual rows of the same slice and length more
        // often than a heavy row and its neighbours of other kinds do.
        const size_t nKeys = (size_t)S * perSlice;
        keyStart.assign(nKeys + 1, 0);
        auto key_of = [&](const VRow &v) { return (size_t)v.slice * perSlice + (size_t)(cap - v.len) * 3 + (size_t)v.kind; };
        for (int t = 0; t < nV; ++t) keyStart[key_of(vr[t]) + 1]++;
        for (size_t k = 0; k < nKeys; ++k) keyStart[k + 1] += keyStart[k];
        {
            std::vector<int> cur(keyStart.begin(), keyStart.end() - 1);
            for (int t = 0; t < nV; ++t) sorted[cur[key_of(vr[t])]++] = t;
        }
        // chunks of every slice: 64 virtual rows of the sorted order each, as long as their first member
        for (int q = 0; q < S; ++q) {
            const int a = keyStart[(size_t)q * perSlice], b = keyStart[(size_t)(q + 1) * perSlice];
            for (int f = a; f < b; f += 64) sliceChunks[q].push_back({f, std::min(64, b - f), (vr[sorted[f]].len + E - 1) / E});
        }
        const int rc = mx::plan_slice_chunks(dtype, budget, S, sliceChunks, SP);
        if (rc) return rc;
    }
    const int nWG = SP.nWG, maxWgChunks = SP.maxWgChunks;
    const long long totalSteps = SP.totalSteps, totalChunks = SP.totalChunks;
    const size_t padSteps = mx::kSlicePadSteps;  // spare zero steps after the last
    std::vector<unsigned short> ecol(((size_t)totalSteps + padSteps) * 64 * E, 0);
    std::vector<unsigned char> ev(((size_t)totalSteps + padSteps) * 64 * E * es, 0);
    // one byte per entry instead of its value when the selected rows hold at most 256 distinct
    // values (MX_CSR_DICT=0: never)
    std::vector<unsigned char> codeOfEntry, dictv, ecode;
    int nDict = 0;
    bool haveDict = false;
    {
        // (255 values at most: code 255 names the zero that the padding of the layout multiplies x with)
        if (!sel && nnz >= 65536 && mx::opt().csr_dict != 0)
            haveDict = make_value_dict(es, val, rowPtr[rows], codeOfEntry, dictv, &nDict, 255);
        if (haveDict) ecode.assign(ecol.size(), 255);
    }
    std::vector<int> &wgDesc = SP.wgDesc, &waveDesc = SP.waveDesc, &chunkEnd = SP.chunkEnd;
    std::vector<int> segIdx((size_t)nV + 1, 0);
    const unsigned char *sv = (const unsigned char *)val;
#pragma omp parallel for schedule(dynamic, 64)
    for (long long c = 0; c < totalChunks; ++c) {
        const int q = SP.chunkSlice[c], steps = SP.chunkSteps[c];
        const long long step = SP.chunkStep0[c];
        for (int l = 0; l < SP.chunkN[c]; ++l) {
            const int t = sorted[SP.chunkFirst[c] + l];
            const VRow &v = vr[t];
            segIdx[t] = (int)(c * 64 + l);
            for (int n = 0; n < v.len; ++n) {
                const int p = ord[v.start + n];
                const size_t st = (size_t)step + n, batch = st / BE, k = st % BE;
                // a lane's column offsets of a batch are contiguous; so are its binary16
                // values; binary64 values go in sub-blocks of two per lane
                const size_t atc = (batch * 64 + l) * BE + k;
                const size_t atv = dtype == MX_F64 ? batch * 64 * BE + (k / 2) * 128 + (size_t)l * 2 + k % 2 : atc;
                ecol[atc] = (unsigned short)(col[p] - q * SW);
                if (haveDict) ecode[atc] = codeOfEntry[p];
                std::memcpy(&ev[atv * es], sv + (size_t)p * es, es);
            }
            // the padding up to the chunk's longest member multiplies zero with the x of the
            // virtual row's own last column: a non-finite x then reaches the rows that name its
            // column, as in a plain CSR product, and no others
            if (v.len > 0) {
                const unsigned short lastCol = (unsigned short)(col[ord[v.start + v.len - 1]] - q * SW);
                for (int n = v.len; n < steps * E; ++n) {
                    const size_t st = (size_t)step + n, batch = st / BE, k = st % BE;
                    ecol[(batch * 64 + l) * BE + k] = lastCol;
                }
            }
        }
    }
    // how the sums become y: rows with one virtual row are named at that virtual row, the others
    // are listed
    std::vector<int> rowInfo(((size_t)rows + 3) / 4 * 4 + 4, -2), lightInfo, heavyInfo;
    for (int r = 0; r < rows; ++r) {
        const int a = segPtr[r], n = segPtr[r + 1] - a;
        // (elsewhere 2: the row's sums are fetched by the block layout of a binary64 plan, which writes its y)
        const bool fetched = elsewhere && elsewhere[r] == 2;
        rowInfo[r] = fetched ? -2 : n == 0 ? ((elsewhere && elsewhere[r]) ? -2 : -1) : n == 1 ? segIdx[a] : -2;
        if (n > 1 && !fetched) {
            std::vector<int> &L = n > mx::kSliceLightSegs ? heavyInfo : lightInfo;
            L.insert(L.end(), {r, a, n, 0});
        }
    }
    D.nWG = nWG;
    D.S = S;
    D.rows = rows;
    D.cols = cols;
    D.sliceCols = SW;
    D.maxWgChunks = maxWgChunks;
    D.steps = totalSteps;
    D.chunks = totalChunks;
    D.nnz = nnz;
    D.vrows = nV;
    D.cap = cap;
    D.subset = sel != nullptr;
    D.wgDesc.swap(wgDesc);
    D.waveDesc.swap(waveDesc);
    D.chunkEnd.swap(chunkEnd);
    D.segPtr.swap(segPtr);
    D.segIdx.swap(segIdx);
    D.rowInfo.swap(rowInfo);
    D.lightInfo.swap(lightInfo);
    D.heavyInfo.swap(heavyInfo);
    D.ecol.swap(ecol);
    D.eval.swap(ev);
    if (haveDict) {
        D.ecode.swap(ecode);
        D.dict.swap(dictv);
        D.nDict = nDict;
    }
    D.fused = fused != 0;
    if (fused) {
        int most = 0;
        for (int r = 0; r < rows; ++r) most = std::max(most, D.segPtr[r + 1] - D.segPtr[r]);
        // (as many places as the longest list of virtual rows has: the one who adds reads every place of a row)
        const int places = std::max(most, 1);
        D.placesPerRow = places;
        D.nGroups = SP.nGroups;
        D.maxWgGroups = SP.maxWgGroups;
        D.wgGroups.swap(SP.wgGroups);
        D.groupNeed.swap(SP.groupNeed);
        mx::fused_targets(rows, nGroups, places, totalChunks, D.segPtr.data(), D.segIdx.data(), D.fusedTarget);
        D.rowVrows.assign((size_t)nGroups * GR, 0);
        for (int r = 0; r < rows; ++r) D.rowVrows[r] = (unsigned char)(D.segPtr[r + 1] - D.segPtr[r]);
    }
    return MX_OK;
}

// `segOut` (optional): receives segPtr and segIdx (the virtual rows of every matrix row).
// `fused`: the layout of the one-launch form where the matrix suits it (D.fused says whether it did).
int upload_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                  const char *sel, mx::DeviceSlices &D, const char *elsewhere,
                  std::pair<std::vector<int>, std::vector<int>> *segOut, int fused)
{
    // The whole matrix: the layout is made on the device (the same arrays, in a fraction of the
    // time for a large matrix); MX_LAYOUT=host keeps the host route, which also serves row subsets.
    if (!sel && !mx::opt().layout_host) {
        const size_t es = (size_t)mx::elem_size(dtype);
        const int nnz = rowPtr[rows];
        int *dRowPtr = nullptr, *dCol = nullptr;
        void *dVal = nullptr, *dElse = nullptr;
        int rc = upload(&dRowPtr, rowPtr, (size_t)rows + 1);
        if (!rc) rc = upload(&dCol, col, (size_t)nnz);
        if (!rc) rc = upload_bytes(&dVal, val, (size_t)nnz * es);
        if (!rc && elsewhere) rc = upload_bytes(&dElse, elsewhere, (size_t)rows);
        if (!rc)
            rc = mx::build_slices_device(dtype, rows, cols, nnz, dRowPtr, dCol, dVal, nCU, S, (const char *)dElse, D, nullptr,
                                         segOut ? &segOut->first : nullptr, segOut ? &segOut->second : nullptr, fused);
        (void)hipFree(dRowPtr);
        (void)hipFree(dCol);
        (void)hipFree(dVal);
        (void)hipFree(dElse);
        return rc;
    }
    HostSlices H;
    int rc = build_slices(dtype, rows, cols, rowPtr, col, val, nCU, S, sel, H, elsewhere, fused);
    if (rc) return rc;
    MX_HIP(mx::prepare_slice_kernels(dtype));
    if (segOut) {
        segOut->first = H.segPtr;
        segOut->second = H.segIdx;
    }
    D.nWG = H.nWG;
    D.S = H.S;
    D.rows = H.rows;
    D.cols = H.cols;
    D.sliceCols = H.sliceCols;
    D.maxWgChunks = H.maxWgChunks;
    D.steps = H.steps;
    D.chunks = H.chunks;
    D.nnz = H.nnz;
    D.vrows = H.vrows;
    D.subset = H.subset;
    D.nLight = (int)H.lightInfo.size() / 4;
    D.nHeavy = (int)H.heavyInfo.size() / 4;
    for (int r = 0; r < rows; ++r) D.mostVrows = std::max(D.mostVrows, H.segPtr[r + 1] - H.segPtr[r]);
    if ((rc = upload(&D.wgDesc, H.wgDesc.data(), H.wgDesc.size()))) return rc;
    if ((rc = upload(&D.waveDesc, H.waveDesc.data(), H.waveDesc.size()))) return rc;
    if ((rc = upload(&D.chunkEnd, H.chunkEnd.data(), H.chunkEnd.size()))) return rc;
    if ((rc = upload(&D.ecol, H.ecol.data(), H.ecol.size()))) return rc;
    if ((rc = upload_bytes(&D.eval, H.eval.data(), H.eval.size()))) return rc;
    if (!H.ecode.empty()) {
        void *dc = nullptr;
        if ((rc = upload_bytes(&dc, H.ecode.data(), H.ecode.size()))) return rc;
        D.ecode = (unsigned char *)dc;
        if ((rc = upload_bytes(&D.dict, H.dict.data(), H.dict.size()))) return rc;
        D.nDict = H.nDict;
    }
    if ((rc = upload_bytes(&D.partial, nullptr, 0, ((size_t)H.chunks * 64 + 64) * (dtype == MX_F64 ? 8 : 4)))) return rc;
    if ((rc = upload(&D.rowInfo, H.rowInfo.data(), H.rowInfo.size()))) return rc;
    if ((rc = upload(&D.segIdx, H.segIdx.data(), H.segIdx.size()))) return rc;
    {
        // the light rows' virtual rows, eight places per row
        const int nL = (int)H.lightInfo.size() / 4;
        int most = 0;
        for (int i = 0; i < nL; ++i) most = std::max(most, H.lightInfo[4 * (size_t)i + 2]);
        const int places = most <= 4 ? 4 : mx::kSliceLightSegs;  // four places per row where that is enough
        D.lightQuads = places / 4;
        std::vector<int> lr((size_t)nL), li((size_t)nL * places, -1);
        for (int i = 0; i < nL; ++i) {
            lr[i] = H.lightInfo[4 * (size_t)i];
            const int a = H.lightInfo[4 * (size_t)i + 1], n = H.lightInfo[4 * (size_t)i + 2];
            for (int k = 0; k < n; ++k) li[(size_t)i * places + k] = H.segIdx[a + k];
        }
        if ((rc = upload(&D.lightRow, lr.data(), lr.size(), 1))) return rc;
        if ((rc = upload(&D.lightIdx, li.data(), li.size(), 8))) return rc;
    }
    if ((rc = upload(&D.heavyInfo, H.heavyInfo.data(), H.heavyInfo.size(), 4))) return rc;
    if (H.fused) {
        D.nGroups = H.nGroups;
        D.maxWgGroups = H.maxWgGroups;
        D.placesPerRow = H.placesPerRow;
        if ((rc = upload(&D.wgGroups, H.wgGroups.data(), H.wgGroups.size()))) return rc;
        if ((rc = upload(&D.groupNeed, H.groupNeed.data(), H.groupNeed.size()))) return rc;
        if ((rc = upload(&D.groupCount, (const int *)nullptr, 0, (size_t)H.nGroups + 1))) return rc;
        if ((rc = upload(&D.fusedTarget, H.fusedTarget.data(), H.fusedTarget.size(), 64))) return rc;
        if ((rc = upload_bytes(&D.fusedSums, nullptr, 0, ((size_t)H.nGroups * H.placesPerRow * mx::kFusedGroupRows + 64) * (dtype == MX_F64 ? 8 : 4))))
            return rc;
        if ((rc = upload(&D.claim, (const unsigned *)nullptr, 0, (size_t)H.nWG + 1))) return rc;
        D.fused = true;
    }
    return MX_OK;
}



// The waves of a tile layout: whole chunks, about `per` steps each; few enough waves that all of
// them are resident at once (24 per CU), so that none has to wait for a second round.
// stepVo / stepA / stepChunkEnd: first value, blocks in half 0 and "a wave may end here" of every
// step.  waveDesc: 8 ints per wave (see DeviceTiles); ahead: per step the first value and the
// blocks in half 0 of the step four further on (the wave's last when past it).
void tile_waves(int steps, int nCU, int perMin, const std::vector<int> &stepVo, const std::vector<int> &stepA,
                       const std::vector<int> &stepChunkEnd, std::vector<int> &waveDesc, std::vector<int> &ahead)
{
    nCU = std::max(1, nCU);
    const int tper = mx::opt().tile_per;
    // (binary64 block waves keep two steps in registers and live on the number of waves: a step each)
    const int per = tper > 0 ? tper : std::max(perMin, (steps + nCU * 24 - 1) / (nCU * 24));
    waveDesc.clear();
    ahead.assign((size_t)steps * 2, 0);
    for (int s0 = 0; s0 < steps;) {
        int s1 = std::min(steps, s0 + per);
        while (s1 < steps && !stepChunkEnd[s1 - 1]) ++s1;
        int d[8] = {s0, s1, 0, 0, 0, 0, 0, 0};
        for (int k = 0; k < 4; ++k) {
            const int sk = std::min(s0 + k, s1 - 1);
            d[2 + k] = stepVo[sk];
            d[6] |= stepA[sk] << (8 * k);
        }
        waveDesc.insert(waveDesc.end(), d, d + 8);
        for (int s = s0; s < s1; ++s) {
            const int s4 = std::min(s + 4, s1 - 1);
            ahead[2 * (size_t)s] = stepVo[s4];
            ahead[2 * (size_t)s + 1] = stepA[s4];
        }
        s0 = s1;
    }
}

int build_tiles(mx_dtype dtype, int chunkNum, const char *selFrag, int dRows, const int *chunkPtr, const int *fragPtr,
                const void *fragBit, const void *tcVal, const int *atox, const int *colMap, const int *rowMap, int nCU,
                HostTiles &T, const char *rowTaken, const std::vector<StripChunk> *stripChunks)
{
    const int es = mx::elem_size(dtype), fragM = mx::kFragM;
    // (the plan's own chunks -- binary16 strips, binary64 blocks -- are made of blocks of 8 columns, four
    // to a half, in both precisions; the reference's fragments are fragK wide)
    const int fragK = stripChunks ? 8 : mx::frag_k(dtype);
    const int SF = stripChunks ? 8 : mx::tile_slots(dtype), HF = SF / 2, H = mx::kTileHdr, BS = fragM * fragK;  // BS: values per block
    const bool f64 = dtype == MX_F64;
    auto slot_of = [&](int half, int i) { return stripChunks ? 4 * half + i : mx::tile_slot(dtype, half, i); };
    const uint32_t *bit32 = (const uint32_t *)fragBit;
    const uint64_t *bit64 = (const uint64_t *)fragBit;
    const unsigned char *tv = (const unsigned char *)tcVal;
    std::vector<int> hdr, dAtox, stepVo, stepA, stepChunkEnd;  // stepChunkEnd: 1 when a wave may end after the step
    std::vector<unsigned char> dVal;
    size_t voff = 0;  // values stored so far; always a multiple of BS, so every block is 16-byte aligned
    int nsel = 0, nnz = 0, nfr = 0;

    // The blocks of a chunk, rebuilt from its selected fragments: their columns (in the caller's
    // numbering) in ascending order, fragK per block.  The reference orders a chunk's columns by
    // their rank among the dense columns, which scatters neighbouring columns over the fragments;
    // in ascending order a dense strip becomes blocks of consecutive columns, and the gathers of
    // any chunk touch fewer lines.
    typedef TileBlock Block;
    std::vector<Block> blocks;
    struct ColRef {
        int col, f, pos;
    };
    std::vector<ColRef> refs;
    int chunkVals = 0;  // entries build_blocks put into `blocks`
    std::vector<int> chunkOfFrag;  // only needed to find a fragment's rows
    if (rowTaken) {
        chunkOfFrag.resize((size_t)chunkPtr[chunkNum]);
        for (int w = 0; w < chunkNum; ++w)
            for (int f = chunkPtr[w]; f < chunkPtr[w + 1]; ++f) chunkOfFrag[f] = w;
    }
    auto gone = [&](int f, int r) {  // row r of fragment f was taken into a strip chunk
        if (!rowTaken) return false;
        const int i = chunkOfFrag[f] * fragM + r;
        return i < dRows && rowTaken[i] != 0;
    };
    auto build_blocks = [&](const std::vector<int> &fsel) {
        refs.clear();
        for (int f : fsel) {
            const uint64_t bm = f64 ? (uint64_t)bit32[f] : bit64[f];
            for (int c = 0; c < fragK; ++c) {
                bool used = false;
                for (int r = 0; r < fragM && !used; ++r) used = ((bm >> (r * fragK + c)) & 1ull) && !gone(f, r);
                if (!used) continue;  // a padding position of the chunk's last fragment, or only rows that went elsewhere
                const int col = atox[(size_t)f * fragK + c];
                refs.push_back({colMap ? colMap[col] : col, f, c});
            }
        }
        std::sort(refs.begin(), refs.end(), [](const ColRef &a, const ColRef &b) { return a.col < b.col; });
        chunkVals = 0;
        const int nb = ((int)refs.size() + fragK - 1) / fragK;
        blocks.assign(nb, Block());
        for (Block &B : blocks) {
            B.vals.assign((size_t)BS * es, 0);
            for (int c = 0; c < 8; ++c) B.cols[c] = -1;
        }
        // where each fragment's values start for every (row, position): walk its bits in order
        for (int i = 0; i < (int)refs.size(); ++i) blocks[i / fragK].cols[i % fragK] = refs[i].col;
        std::vector<int> where((size_t)fsel.size() * fragK, -1);  // (fragment in fsel, pos) -> index in refs
        for (int i = 0; i < (int)refs.size(); ++i) {
            const int fi = (int)(std::find(fsel.begin(), fsel.end(), refs[i].f) - fsel.begin());
            where[(size_t)fi * fragK + refs[i].pos] = i;
        }
        for (int fi = 0; fi < (int)fsel.size(); ++fi) {
            const int f = fsel[fi];
            const uint64_t bm = f64 ? (uint64_t)bit32[f] : bit64[f];
            int k = 0;
            for (int bit = 0; bit < BS; ++bit)
                if ((bm >> bit) & 1ull) {
                    const int r = bit / fragK, i = where[(size_t)fi * fragK + bit % fragK];
                    if (!gone(f, r)) {
                        std::memcpy(&blocks[i / fragK].vals[((size_t)r * fragK + i % fragK) * es], tv + (size_t)(fragPtr[f] + k) * es, es);
                        ++chunkVals;
                    }
                    ++k;
                }
        }
    };
    auto put_block = [&](size_t s, int slot, const Block &B) {  // the next block of step s
        dVal.insert(dVal.end(), B.vals.begin(), B.vals.end());
        voff += BS;
        for (int c = 0; c < fragK; ++c) dAtox[s * 64 + (size_t)slot * fragK + c] = B.cols[c];
        if (SF == 8) hdr[s * H + 21 + slot] = B.cols[0];
    };
    // a step with the blocks a0[0..n0) (half 0) and a1[0..n1) (half 1) of two chunks, given by
    // their fragM output rows r0 and r1 (r1 null: none; with flags & 2 clear both halves are r0's)
    auto emit = [&](const Block *a0, int n0, const int *r0, const Block *a1, int n1, const int *r1, int flags) {
        const size_t s = stepVo.size();
        hdr.resize((s + 1) * H, 0);
        dAtox.resize((s + 1) * 64, -1);
        stepVo.push_back((int)voff);
        stepA.push_back(n0);
        stepChunkEnd.push_back(flags & 1);
        for (int i = 0; i < 16; ++i) hdr[s * H + i] = -1;
        for (int half = 0; half < 2; ++half) {
            const int *rr = half ? r1 : r0;
            if (!rr || (half && !(flags & 2))) continue;
            for (int i = 0; i < fragM; ++i) hdr[s * H + half * 8 + i] = rr[i];
        }
        hdr[s * H + 16] = flags;
        hdr[s * H + 17] = n0;
        hdr[s * H + 18] = n1;
        for (int i = 21; i < 29; ++i) hdr[s * H + i] = -1;
        for (int i = 0; i < n0; ++i) put_block(s, slot_of(0, i), a0[i]);
        for (int i = 0; i < n1; ++i) put_block(s, slot_of(1, i), a1[i]);
    };
    std::vector<int> fsel;
    std::vector<Block> pending;
    int pendingRows[8], curRows[8];
    bool havePending = false;  // a small chunk waiting for a partner
    // a chunk's blocks into steps: up to half a step shares one with the next such chunk, more
    // takes whole steps of its own
    auto place = [&](const std::vector<Block> &bl, const int *rows) {
        if ((int)bl.size() <= HF) {
            if (havePending) {
                emit(pending.data(), (int)pending.size(), pendingRows, bl.data(), (int)bl.size(), rows, 3);
                havePending = false;
            } else {
                havePending = true;
                pending = bl;
                std::copy(rows, rows + 8, pendingRows);
            }
        } else {
            for (size_t i0 = 0; i0 < bl.size(); i0 += SF) {
                const int n = (int)std::min(bl.size() - i0, (size_t)SF), n0 = std::min(n, HF);
                emit(&bl[i0], n0, rows, &bl[i0 + n0], n - n0, rows, i0 + SF >= bl.size() ? 1 : 0);
            }
        }
    };
    if (stripChunks) {
        for (const StripChunk &C : *stripChunks) {
            ++nsel;
            nnz += C.nnz;
            nfr += (int)C.blocks.size();
            place(C.blocks, C.rows);
            if (voff > 2000000000u) {
                set_error("tile layout: too many values for 32-bit offsets");
                return MX_ERR_ARG;
            }
        }
    } else {
        for (int w = 0; w < chunkNum; ++w) {
            fsel.clear();
            for (int f = chunkPtr[w]; f < chunkPtr[w + 1]; ++f)
                if (fragPtr[f + 1] > fragPtr[f] && (!selFrag || selFrag[f])) fsel.push_back(f);
            if (fsel.empty()) continue;
            build_blocks(fsel);
            if (blocks.empty()) continue;  // all its rows went into strip chunks
            ++nsel;
            nnz += chunkVals;
            nfr += (int)fsel.size();
            for (int i = 0; i < 8; ++i) {
                const int local = w * fragM + i;
                // (a row that went into a strip chunk has nothing here and is not written from here)
                const bool here = i < fragM && local < dRows && !(rowTaken && rowTaken[local]);
                curRows[i] = here ? (rowMap ? rowMap[local] : local) : -1;
            }
            place(blocks, curRows);
            if (voff > 2000000000u) {
                set_error("tile layout: too many values for 32-bit offsets");
                return MX_ERR_ARG;
            }
        }
    }
    if (havePending) emit(pending.data(), (int)pending.size(), pendingRows, nullptr, 0, nullptr, 3);
    const int steps = (int)stepVo.size();
    T.chunkNum = nsel;
    T.frags = nfr;
    T.vals = nnz;
    T.stored = (long long)voff;
    T.steps = steps;
    T.dense = stripChunks != nullptr && steps > 0;
    if (steps == 0) return MX_OK;
    std::vector<int> waveDesc, ahead;
    tile_waves(steps, nCU, (stripChunks && f64) ? 1 : 2, stepVo, stepA, stepChunkEnd, waveDesc, ahead);
    for (int s = 0; s < steps; ++s) {
        hdr[(size_t)s * H + 19] = ahead[2 * (size_t)s];
        hdr[(size_t)s * H + 20] = ahead[2 * (size_t)s + 1];
    }
    T.nWaves = (int)waveDesc.size() / 8;
    T.waveDesc.swap(waveDesc);
    T.hdr.swap(hdr);
    T.atox.swap(dAtox);
    T.valOffset.swap(stepVo);
    T.val.swap(dVal);
    return MX_OK;
}

int upload_tiles(mx_dtype dtype, int chunkNum, const char *selFrag, int dRows, const int *chunkPtr, const int *fragPtr,
                 const void *fragBit, const void *tcVal, const int *atox, const int *colMap, const int *rowMap,
                 mx::DeviceTiles &T, int *tile_nnz, const char *rowTaken,
                 const std::vector<StripChunk> *stripChunks, std::vector<int> *hdrOut)
{
    int nCU = 256;
    {
        hipDeviceProp_t prop;
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            nCU = std::max(1, prop.multiProcessorCount);
    }
    HostTiles H;
    int rc = build_tiles(dtype, chunkNum, selFrag, dRows, chunkPtr, fragPtr, fragBit, tcVal, atox, colMap, rowMap, nCU, H,
                         rowTaken, stripChunks);
    if (rc) return rc;
    T.chunkNum = H.chunkNum;
    T.frags = H.frags;
    T.vals = H.vals;
    T.stored = H.stored;
    T.steps = H.steps;
    T.dense = H.dense;
    T.nWaves = H.nWaves;
    if (tile_nnz) *tile_nnz = H.vals;
    if (hdrOut) *hdrOut = H.hdr;
    if (H.steps == 0) return MX_OK;
    if ((rc = upload(&T.waveDesc, H.waveDesc.data(), H.waveDesc.size(), 64))) return rc;
    if ((rc = upload(&T.hdr, H.hdr.data(), H.hdr.size(), 256))) return rc;
    if ((rc = upload(&T.atox, H.atox.data(), H.atox.size(), 256))) return rc;
    // a lane of a step with few blocks reads where an absent block would be: 4 KB of slack
    if ((rc = upload_bytes(&T.tcVal, H.val.data(), H.val.size(), 8192))) return rc;
    return MX_OK;
}

int upload_csr(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr, const int *col, const void *val,
               mx::DeviceCsr &A, double *pack_ms)
{
    const int es = mx::elem_size(dtype), npt = mx::csr_entries_per_lane(dtype);
    A.rows = rows;
    A.cols = cols;
    A.npt = npt;
    A.nnz = nnz;
    int rc;
    auto t0 = std::chrono::steady_clock::now();
    std::vector<int> desc;
    pack_rows(rowPtr, rows, npt, desc);
    if ((rc = upload(&A.rowPtr, rowPtr, (size_t)rows + 1))) return rc;
    if ((rc = upload_bytes(&A.val, val, (size_t)nnz * es, (size_t)mx::kCsrPad * es))) return rc;
    A.nBlocks = (int)desc.size() / 4;
    if ((rc = upload(&A.blockDesc, desc.data(), desc.size()))) return rc;
    {
        // rows of very different lengths: sum tiles by a segmented scan (MX_CSR_REDUCE=rows|scan overrides)
        double sum = 0.0, sq = 0.0;
        for (int r = 0; r < rows; ++r) {
            const double n = rowPtr[r + 1] - rowPtr[r];
            sum += n;
            sq += n * n;
        }
        const double mean = rows > 0 ? sum / rows : 0.0, var = rows > 0 ? sq / rows - mean * mean : 0.0;
        A.scan = mean > 0.0 && var > 0.25 * mean * mean;
        if (mx::opt().csr_reduce == 1) A.scan = false;
        if (mx::opt().csr_reduce == 2) A.scan = true;
    }
    // 16-bit column offsets when every workgroup's columns span fewer than 65536
    // (MX_CSR_COL16=0 keeps 32-bit ids)
    bool narrow = mx::opt().csr_col16 && nnz > 0;
    std::vector<int> cbase((size_t)A.nBlocks, 0);
    if (narrow) {
        int wide = 0;
#pragma omp parallel for schedule(static) reduction(+ : wide)
        for (int b = 0; b < A.nBlocks; ++b) {
            const int p0 = desc[4 * (size_t)b + 2], p1 = desc[4 * (size_t)b + 3];
            int lo = INT_MAX, hi = 0;
            for (int p = p0; p < p1; ++p) {
                lo = std::min(lo, col[p]);
                hi = std::max(hi, col[p]);
            }
            if (p1 > p0) {
                cbase[b] = lo;
                wide += hi - lo > 65535;
            }
        }
        narrow = wide == 0;
    }
    if (narrow) {
        std::vector<unsigned short> c16((size_t)nnz);
#pragma omp parallel for schedule(static)
        for (int b = 0; b < A.nBlocks; ++b)
            for (int p = desc[4 * (size_t)b + 2]; p < desc[4 * (size_t)b + 3]; ++p)
                c16[p] = (unsigned short)(col[p] - cbase[b]);
        void *d16 = nullptr;
        if ((rc = upload_bytes(&d16, c16.data(), (size_t)nnz * 2, (size_t)mx::kCsrPad * 2))) return rc;
        A.col16 = (unsigned short *)d16;
        if ((rc = upload(&A.colBase, cbase.data(), cbase.size()))) return rc;
        // at most 256 distinct values (bit patterns): a byte per entry and a dictionary beside the
        // values; the plan times both forms (MX_CSR_DICT=0: never)
        if (nnz >= 65536 && mx::opt().csr_dict != 0) {
            std::vector<unsigned char> codes, dict;
            int nd = 0;
            const bool few = make_value_dict(es, val, nnz, codes, dict, &nd);
            if (few) {
                void *dc = nullptr;
                if ((rc = upload_bytes(&dc, codes.data(), (size_t)nnz, (size_t)mx::kCsrPad))) return rc;
                A.codes = (unsigned char *)dc;
                if ((rc = upload_bytes(&A.dict, dict.data(), dict.size()))) return rc;
                A.nDict = nd;
            }
        }
    } else {
        if ((rc = upload(&A.col, col, (size_t)nnz, mx::kCsrPad))) return rc;
    }
    auto t1 = std::chrono::steady_clock::now();
    if (pack_ms) *pack_ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    return MX_OK;
}

}  // namespace mxp

using namespace mxp;

// The part of the slice layout that looks at chunks only (64 virtual rows each; a few per thousand
// entries): which workgroup and wave streams which chunk, and where.  Shared by the host route and
// the device route of the layout, which hand in the chunks of every slice (longest first, as the
// sort leaves them) and fill the streams from what comes back.
int mx::plan_slice_chunks(mx_dtype dtype, int budget, int S, const std::vector<std::vector<mx::SliceChunk>> &sliceChunks,
                          mx::SlicePlan &P)
{
    const int E = mx::slice_step_entries(dtype), SPB = mx::kSliceBatchEntries / E;
    // the slice's share of the workgroups (in proportion to its steps, largest remainders, at
    // least one when it holds anything)
    std::vector<long long> sliceSteps(S, 0);
    long long allSteps = 0;
    int busy = 0;
    for (int q = 0; q < S; ++q) {
        for (const mx::SliceChunk &c : sliceChunks[q]) sliceSteps[q] += c.steps + mx::kSliceChunkCost;
        allSteps += sliceSteps[q];
        busy += !sliceChunks[q].empty();
    }
    std::vector<int> Gq(S, 0);
    {
        const int total = std::max(budget, busy);
        std::vector<double> want(S, 0.0);
        int used = 0;
        for (int q = 0; q < S; ++q) {
            if (sliceChunks[q].empty()) continue;
            want[q] = allSteps > 0 ? (double)sliceSteps[q] * total / (double)allSteps : 1.0;
            Gq[q] = std::max(1, (int)want[q]);
            used += Gq[q];
        }
        while (used < total && busy > 0) {  // hand out what rounding down left over
            int best = -1;
            for (int q = 0; q < S; ++q)
                if (!sliceChunks[q].empty() && (best < 0 || want[q] - Gq[q] > want[best] - Gq[best])) best = q;
            ++Gq[best];
            ++used;
        }
        for (int q = 0; q < S; ++q) {
            const int nc = (int)sliceChunks[q].size();
            Gq[q] = std::min(std::max(Gq[q], (nc + mx::kSliceWgChunks - 1) / mx::kSliceWgChunks), std::max(nc, 1));
            if (nc == 0) Gq[q] = 0;
        }
    }
    // workgroups: a slice's chunks, longest first, each to the workgroup of the slice with the
    // fewest steps so far; then the same inside the workgroup for its waves
    std::vector<mxp::SliceWg> wgs;
    for (int q = 0; q < S; ++q) {
        const int g0 = (int)wgs.size(), G = Gq[q];
        if (G == 0) continue;
        wgs.resize(wgs.size() + G);
        std::vector<std::vector<int>> mine(G);
        typedef std::pair<long long, int> Load;
        std::priority_queue<Load, std::vector<Load>, std::greater<Load>> heap;
        for (int g = 0; g < G; ++g) heap.push({0, g});
        const auto &ch = sliceChunks[q];
        for (int c = 0; c < (int)ch.size(); ++c) {
            Load top = heap.top();
            heap.pop();
            mine[top.second].push_back(c);
            top.first += ch[c].steps + mx::kSliceChunkCost;
            if ((int)mine[top.second].size() < mx::kSliceWgChunks) heap.push(top);
        }
        for (int g = 0; g < G; ++g) deal_to_waves(wgs[g0 + g], q, mine[g], ch, SPB);
    }
    return emit_slice_plan(wgs, sliceChunks, SPB, E, P);
}

static int slice_layout_view(const mx_csr *A, int nCU, const unsigned char *sel, bool fused, mx_slice_layout_view *out);
extern "C" int mx_slice_layout(const mx_csr *A, int nCU, const unsigned char *sel, mx_slice_layout_view *out)
{
    return slice_layout_view(A, nCU, sel, false, out);
}
extern "C" int mx_slice_layout_fused(const mx_csr *A, int nCU, mx_slice_layout_view *out)
{
    return slice_layout_view(A, nCU, nullptr, true, out);
}
static int slice_layout_view(const mx_csr *A, int nCU, const unsigned char *sel, bool fused, mx_slice_layout_view *out)
{
    mx::refresh_options();
    if (!A || !out || nCU < 1 || A->rows < 0 || A->cols < 1 || !A->rowPtr || (A->nnz > 0 && (!A->colInd || !A->val))) {
        set_error("mx_slice_layout: bad argument");
        return MX_ERR_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    if (A->rowPtr[0] != 0 || A->rowPtr[A->rows] != A->nnz) {
        set_error("mx_slice_layout: rowPtr does not span [0, nnz]");
        return MX_ERR_ARG;
    }
    for (int r = 0; r < A->rows; ++r)
        if (A->rowPtr[r + 1] < A->rowPtr[r]) {
            set_error("mx_slice_layout: rowPtr is not ascending");
            return MX_ERR_ARG;
        }
    for (int p = 0; p < A->nnz; ++p)
        if ((unsigned)A->colInd[p] >= (unsigned)A->cols) {
            set_error("mx_slice_layout: column index out of range");
            return MX_ERR_ARG;
        }
    const int S = (A->cols + mx::slice_cols(A->dtype) - 1) / mx::slice_cols(A->dtype);
    HostSlices H;
    try {
        int rc = build_slices(A->dtype, A->rows, A->cols, A->rowPtr, A->colInd, A->val, nCU, S, (const char *)sel, H, nullptr, fused);
        if (rc) return rc;
    } catch (const std::bad_alloc &) {
        set_error("mx_slice_layout: out of memory");
        return MX_ERR_ALLOC;
    }
    auto give = [](const auto &v) {
        typedef typename std::decay<decltype(v)>::type::value_type T;
        T *p = (T *)malloc(std::max<size_t>(v.size(), 1) * sizeof(T));
        if (p && !v.empty()) std::memcpy(p, v.data(), v.size() * sizeof(T));
        return p;
    };
    out->nWG = H.nWG;
    out->S = H.S;
    out->sliceCols = H.sliceCols;
    out->waves = mx::kSliceWaves;
    out->stepEntries = mx::slice_step_entries(A->dtype);
    out->batchEntries = mx::kSliceBatchEntries;
    out->cap = H.cap;
    out->chunks = (int)H.chunks;
    out->batches = (int)(H.steps / (mx::kSliceBatchEntries / mx::slice_step_entries(A->dtype)));
    out->vrows = H.vrows;
    out->nLight = (int)H.lightInfo.size() / 4;
    out->nHeavy = (int)H.heavyInfo.size() / 4;
    out->lightSegs = mx::kSliceLightSegs;
    out->nEcol = (long long)H.ecol.size();
    out->wgDesc = give(H.wgDesc);
    out->waveDesc = give(H.waveDesc);
    out->chunkEnd = give(H.chunkEnd);
    out->segPtr = give(H.segPtr);
    out->segIdx = give(H.segIdx);
    out->rowInfo = give(H.rowInfo);
    out->lightInfo = give(H.lightInfo);
    out->heavyInfo = give(H.heavyInfo);
    out->ecol = give(H.ecol);
    out->eval = give(H.eval);
    out->nDict = H.ecode.empty() ? 0 : H.nDict;
    out->ecode = give(H.ecode);
    out->dict = give(H.dict);
    out->fused = H.fused ? 1 : 0;
    if (H.fused) {
        out->groupRows = mx::kFusedGroupRows;
        out->nGroups = H.nGroups;
        out->placesPerRow = H.placesPerRow;
        out->wgGroups = give(H.wgGroups);
        out->groupNeed = give(H.groupNeed);
        out->fusedTarget = give(H.fusedTarget);
        out->rowVrows = give(H.rowVrows);
        if (!out->wgGroups || !out->groupNeed || !out->fusedTarget || !out->rowVrows) {
            mx_slice_layout_free(out);
            set_error("mx_slice_layout: out of memory");
            return MX_ERR_ALLOC;
        }
    }
    if (!out->wgDesc || !out->waveDesc || !out->chunkEnd || !out->segPtr || !out->segIdx || !out->rowInfo || !out->lightInfo ||
        !out->heavyInfo || !out->ecol || !out->ecode || !out->dict ||
        !out->eval) {
        mx_slice_layout_free(out);
        set_error("mx_slice_layout: out of memory");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}

extern "C" void mx_slice_layout_free(mx_slice_layout_view *v)
{
    if (!v) return;
    free(v->wgDesc);
    free(v->waveDesc);
    free(v->chunkEnd);
    free(v->segPtr);
    free(v->segIdx);
    free(v->rowInfo);
    free(v->lightInfo);
    free(v->heavyInfo);
    free(v->ecol);
    free(v->eval);
    free(v->ecode);
    free(v->dict);
    free(v->wgGroups);
    free(v->groupNeed);
    free(v->fusedTarget);
    free(v->rowVrows);
    std::memset(v, 0, sizeof(*v));
}

// The same view from the device route of the layout: the matrix goes up, the layout is built
// there (mx_layout.hip) and comes down.  For tests: every array must equal mx_slice_layout's.
extern "C" int mx_slice_layout_device(const mx_csr *A, int nCU, mx_slice_layout_view *out)
{
    mx::refresh_options();
    if (!A || !out || nCU < 1 || A->rows < 1 || A->cols < 1 || !A->rowPtr || (A->nnz > 0 && (!A->colInd || !A->val))) {
        set_error("mx_slice_layout_device: bad argument");
        return MX_ERR_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    int rc = need_device();
    if (rc) return rc;
    if (A->rowPtr[0] != 0 || A->rowPtr[A->rows] != A->nnz) {
        set_error("mx_slice_layout_device: rowPtr does not span [0, nnz]");
        return MX_ERR_ARG;
    }
    for (int p = 0; p < A->nnz; ++p)
        if ((unsigned)A->colInd[p] >= (unsigned)A->cols) {
            set_error("mx_slice_layout_device: column index out of range");
            return MX_ERR_ARG;
        }
    const int S = (A->cols + mx::slice_cols(A->dtype) - 1) / mx::slice_cols(A->dtype);
    const size_t es = (size_t)mx::elem_size(A->dtype);
    int *dRowPtr = nullptr, *dCol = nullptr;
    void *dVal = nullptr;
    mx::DeviceSlices D;
    std::vector<int> segPtr, segIdx;
    rc = upload(&dRowPtr, A->rowPtr, (size_t)A->rows + 1);
    if (!rc) rc = upload(&dCol, A->colInd, (size_t)A->nnz);
    if (!rc) rc = upload_bytes(&dVal, A->val, (size_t)A->nnz * es);
    if (!rc) rc = mx::build_slices_device(A->dtype, A->rows, A->cols, A->nnz, dRowPtr, dCol, dVal, nCU, S, nullptr, D, nullptr, &segPtr, &segIdx);
    (void)hipFree(dRowPtr);
    (void)hipFree(dCol);
    (void)hipFree(dVal);
    if (rc) {
        free_slices(D);
        return rc;
    }
    auto down = [&](const void *src, size_t bytes) -> void * {
        void *p = malloc(std::max<size_t>(bytes, 1));
        if (p && bytes && hipMemcpy(p, src, bytes, hipMemcpyDeviceToHost) != hipSuccess) {
            free(p);
            p = nullptr;
        }
        return p;
    };
    const int E = mx::slice_step_entries(A->dtype);
    out->nWG = D.nWG;
    out->S = D.S;
    out->sliceCols = D.sliceCols;
    out->waves = mx::kSliceWaves;
    out->stepEntries = E;
    out->batchEntries = mx::kSliceBatchEntries;
    out->chunks = (int)D.chunks;
    out->batches = (int)(D.steps / (mx::kSliceBatchEntries / E));
    out->vrows = D.vrows;
    out->nLight = D.nLight;
    out->nHeavy = D.nHeavy;
    out->lightSegs = mx::kSliceLightSegs;
    out->nEcol = (long long)(((size_t)D.steps + mx::kSlicePadSteps) * 64 * E);
    {
        // (the cap is a function of the size alone, as in the host route)
        const long long fair = (long long)A->nnz / ((long long)nCU * mx::kSliceWaves * 64);
        const int BE = mx::kSliceBatchEntries;
        out->cap = (int)std::min<long long>(512, std::max<long long>(16, (fair + BE - 1) / BE * BE));
        if (const int v = mx::opt().slice_cap)
            if (v >= BE && v <= 4096) out->cap = v / BE * BE;
    }
    out->wgDesc = (int *)down(D.wgDesc, ((size_t)D.nWG * 4 + 4) * 4);
    out->waveDesc = (int *)down(D.waveDesc, ((size_t)D.nWG * mx::kSliceWaves * 4 + 4) * 4);
    out->chunkEnd = (int *)down(D.chunkEnd, ((size_t)D.chunks + 64) * 4);
    out->segPtr = (int *)malloc(std::max<size_t>(segPtr.size(), 1) * 4);
    if (out->segPtr) std::memcpy(out->segPtr, segPtr.data(), segPtr.size() * 4);
    out->segIdx = (int *)down(D.segIdx, ((size_t)D.vrows + 1) * 4);
    out->rowInfo = (int *)down(D.rowInfo, (((size_t)A->rows + 3) / 4 * 4 + 4) * 4);
    out->heavyInfo = (int *)down(D.heavyInfo, ((size_t)D.nHeavy * 4 + 4) * 4);
    out->ecol = (unsigned short *)down(D.ecol, (size_t)out->nEcol * 2);
    out->eval = (unsigned char *)down(D.eval, (size_t)out->nEcol * es);
    out->nDict = D.ecode ? D.nDict : 0;
    out->ecode = (unsigned char *)(D.ecode ? down(D.ecode, (size_t)out->nEcol) : malloc(1));
    out->dict = (unsigned char *)(D.ecode ? down(D.dict, 256 * es) : malloc(1));
    // the light rows in the form of the host view: {row, first virtual row in segIdx, count, 0}
    {
        std::vector<int> lr((size_t)D.nLight + 1, 0);
        bool ok = D.nLight == 0 || hipMemcpy(lr.data(), D.lightRow, (size_t)D.nLight * 4, hipMemcpyDeviceToHost) == hipSuccess;
        out->lightInfo = ok ? (int *)malloc(std::max<size_t>((size_t)D.nLight * 16, 1)) : nullptr;
        if (out->lightInfo)
            for (int i = 0; i < D.nLight; ++i) {
                const int r = lr[i];
                out->lightInfo[4 * i] = r;
                out->lightInfo[4 * i + 1] = segPtr[r];
                out->lightInfo[4 * i + 2] = segPtr[r + 1] - segPtr[r];
                out->lightInfo[4 * i + 3] = 0;
            }
    }
    free_slices(D);
    if (!out->wgDesc || !out->waveDesc || !out->chunkEnd || !out->segPtr || !out->segIdx || !out->rowInfo || !out->lightInfo ||
        !out->heavyInfo || !out->ecol || !out->ecode || !out->dict || !out->eval) {
        mx_slice_layout_free(out);
        set_error("mx_slice_layout_device: out of memory or copy failed");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}

// MX_CSR_NPT overrides the default (for tuning runs); only values with a compiled kernel count.
int mx::csr_entries_per_lane(mx_dtype dtype)
{
    const int v = mx::opt().csr_npt;
    if (dtype == MX_F64) return (v == 4 || v == 8) ? v : 4;
    return (v == 8 || v == 16) ? v : 8;
}

