// Device plans: persistent device copies of a partition and the launch sequence of one
// hybrid SpMV; plus the reference's one-shot host-pointer entry points built on top.
#include <algorithm>
#include <mutex>
#include <atomic>
#include <chrono>
#include <climits>
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <omp.h>
#include <parallel/algorithm>
#include <queue>
#include <vector>

#include "mx_device.h"
#include "mx_internal.h"

namespace {

using mx::set_error;

#define MX_HIP(call)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            set_error(std::string(#call) + ": " + hipGetErrorString(e_));                             \
            return MX_ERR_DEVICE;                                                                     \
        }                                                                                             \
    } while (0)

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

template <typename T>
int upload(T **dst, const T *src, size_t n, size_t pad = 0)
{
    *dst = nullptr;
    const size_t total = std::max<size_t>(n + pad, 1);
    MX_HIP(hipMalloc((void **)dst, total * sizeof(T)));
    if (pad || n == 0) MX_HIP(hipMemset(*dst, 0, total * sizeof(T)));
    if (n) MX_HIP(hipMemcpy(*dst, src, n * sizeof(T), hipMemcpyHostToDevice));
    return MX_OK;
}

int upload_bytes(void **dst, const void *src, size_t n, size_t pad = 0)
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
    (void)hipFree(P.rowVrows);
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
                     int *nDict, int most = 256)
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

// Re-lays the rows `sel` marks (all rows when null) of a CSR matrix for csr_slice_kernel (see
// DeviceSlices).
struct HostSlices {
    int nWG = 0, S = 0, rows = 0, cols = 0, sliceCols = 0, maxWgChunks = 0, nnz = 0, vrows = 0, cap = 0;
    long long steps = 0, chunks = 0;
    bool subset = false;
    std::vector<int> wgDesc, waveDesc, chunkEnd, segPtr, segIdx, rowInfo, lightInfo, heavyInfo;
    std::vector<unsigned short> ecol;
    std::vector<unsigned char> eval;
    std::vector<unsigned char> ecode, dict;  // value dictionary form (empty when the rows hold more than 256 values)
    int nDict = 0;
    // one-launch form (see DeviceSlices): set when it was asked for and the matrix suits it
    bool fused = false;
    int nGroups = 0, maxWgGroups = 0, placesPerRow = 0;
    std::vector<int> wgGroups, groupNeed, fusedTarget;
    std::vector<unsigned char> rowVrows;
};

// A workgroup of the slice layout on its way into the descriptors: its slice and, per wave, the
// chunks (indices into the slice's list) in the order the wave streams them.
struct SliceWg {
    int slice = 0;
    std::vector<int> chunk[mx::kSliceWaves];
    int waveSteps[mx::kSliceWaves] = {};
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
        w.waveSteps[k] = 0;
        w.chunk[k].clear();
    }
    for (int c : mine) {
        int best = 0;
        for (int k = 1; k < W; ++k)
            if (w.waveSteps[k] < w.waveSteps[best]) best = k;
        w.chunk[best].push_back(c);
        w.waveSteps[best] += ch[c].steps;
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

// `elsewhere` (optional) marks rows whose result another kernel writes: 1 = the strips of a binary16
// plan (the row has nothing here), 2 = the 8 x 8 blocks of a binary64 plan, whose waves fetch the sums
// of the row's virtual rows themselves.  Such rows get rowInfo -2 and appear in no list, so that the
// combine kernel's own kinds neither zero them nor add to them.
// `fused`: lay the virtual rows out for the one-launch form (ordered by group of rows before length,
// workgroups dealt per XCD); D.fused tells whether the matrix suited it -- when it does not (a row
// with more than eight virtual rows, more slices than workgroups in an XCD's rows, row subsets or
// rows written elsewhere) the ordinary layout is made.
int build_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                 const char *sel, HostSlices &D, const char *elsewhere = nullptr, bool fused = false)
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
    if (const char *e = std::getenv("MX_SLICE_CAP")) {  // for tuning runs
        const int v = std::atoi(e);
        if (v >= BE && v <= 4096) cap = v / BE * BE;
    }
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
    if (fused) {
        int most = 0;
        for (int r = 0; r < rows; ++r) most = std::max(most, segPtr[r + 1] - segPtr[r]);
        if (sel || elsewhere || most > mx::kSliceLightSegs || (long long)nGroups * mx::kSliceLightSegs * GR > 2000000000LL) fused = false;
    }
    std::vector<int> keyStart, sorted((size_t)nV);
    std::vector<std::vector<mx::SliceChunk>> sliceChunks(S);
    mx::SlicePlan SP;
    const size_t perSlice = (size_t)(cap + 1) * 3;
    if (fused) {
        fused = plan_fused(dtype, budget, S, rows, nGroups, cap, selPtr, segPtr, vr, sorted, sliceChunks, SP);
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
        const char *ed = std::getenv("MX_CSR_DICT");
        // (255 values at most: code 255 names the zero that the padding of the layout multiplies x with)
        if (!sel && nnz >= 65536 && !(ed && !std::atoi(ed)))
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
    D.fused = fused;
    if (fused) {
        int most = 0;
        for (int r = 0; r < rows; ++r) most = std::max(most, D.segPtr[r + 1] - D.segPtr[r]);
        const int places = most <= 4 ? 4 : mx::kSliceLightSegs;
        D.placesPerRow = places;
        D.nGroups = SP.nGroups;
        D.maxWgGroups = SP.maxWgGroups;
        D.wgGroups.swap(SP.wgGroups);
        D.groupNeed.swap(SP.groupNeed);
        // where every virtual row puts its sum: the k-th of row r at ((r / GR) * places + k) * GR + r % GR; the
        // padding lanes of a chunk at the spare places behind the last group
        const size_t spare = (size_t)nGroups * places * GR;
        D.fusedTarget.assign((size_t)totalChunks * 64, 0);
        for (size_t v = 0; v < D.fusedTarget.size(); ++v) D.fusedTarget[v] = (int)(spare + (v & 63));
        D.rowVrows.assign((size_t)nGroups * GR, 0);
#pragma omp parallel for schedule(static)
        for (int r = 0; r < rows; ++r) {
            D.rowVrows[r] = (unsigned char)(D.segPtr[r + 1] - D.segPtr[r]);
            for (int t = D.segPtr[r]; t < D.segPtr[r + 1]; ++t)
                D.fusedTarget[D.segIdx[t]] = (int)(((size_t)(r / GR) * places + (t - D.segPtr[r])) * GR + r % GR);
        }
    }
    return MX_OK;
}

// `segOut` (optional): receives segPtr and segIdx (the virtual rows of every matrix row).
// `fused`: the layout of the one-launch form where the matrix suits it (D.fused says whether it did);
// made on the host.
int upload_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                  const char *sel, mx::DeviceSlices &D, const char *elsewhere = nullptr,
                  std::pair<std::vector<int>, std::vector<int>> *segOut = nullptr, bool fused = false)
{
    // The whole matrix: the layout is made on the device (the same arrays, in a fraction of the
    // time for a large matrix); MX_LAYOUT=host keeps the host route, which also serves row subsets.
    const char *lay = std::getenv("MX_LAYOUT");
    if (!sel && !fused && !(lay && !std::strcmp(lay, "host"))) {
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
                                         segOut ? &segOut->first : nullptr, segOut ? &segOut->second : nullptr);
        (void)hipFree(dRowPtr);
        (void)hipFree(dCol);
        (void)hipFree(dVal);
        (void)hipFree(dElse);
        return rc;
    }
    HostSlices H;
    int rc = build_slices(dtype, rows, cols, rowPtr, col, val, nCU, S, sel, H, elsewhere, fused);
    if (rc) return rc;
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
        if ((rc = upload(&D.rowVrows, H.rowVrows.data(), H.rowVrows.size(), 64))) return rc;
        if ((rc = upload_bytes(&D.fusedSums, nullptr, 0, ((size_t)H.nGroups * H.placesPerRow * mx::kFusedGroupRows + 64) * (dtype == MX_F64 ? 8 : 4))))
            return rc;
        if ((rc = upload(&D.claim, (const unsigned *)nullptr, 0, (size_t)H.nWG + 1))) return rc;
        D.fused = true;
    }
    return MX_OK;
}

// Puts tiles on the device for the tile kernels (see DeviceTiles): the fragments named by
// `selFrag` (all when null), expanded to full blocks.  Column ids go through `colMap` and
// output rows through `rowMap` when given.
// One block of the tile kernels: fragM x fragK values, row-major, zeros included, and the column
// of each of its fragK positions (-1 = unused).
struct TileBlock {
    std::vector<unsigned char> vals;
    int cols[8];
};
// A chunk the plan forms itself for tile_dense_kernel: up to fragM rows (caller's numbering, -1 =
// none) with one and the same set of columns -- whole runs of fragK from a multiple of fragK --
// and that set as blocks.
struct StripChunk {
    int rows[8];
    std::vector<TileBlock> blocks;
    int nnz;
};

// `rowTaken` (optional, per row of A_dd) marks rows whose entries the plan has put into strip
// chunks: they are left out of the fragments here.  With `stripChunks` the canonical chunks are
// not used at all: the given chunks are laid out, for tile_dense_kernel.
// (The layout is made on the host alone -- build_tiles; `nCU` only sizes the waves -- and
// upload_tiles puts it on the device.)
struct HostTiles {
    int chunkNum = 0, frags = 0, vals = 0, steps = 0, nWaves = 0;
    long long stored = 0;
    bool dense = false;
    std::vector<int> waveDesc, hdr, atox, valOffset;  // valOffset: first value of every step (the kernels get it from the headers)
    std::vector<unsigned char> val;
};

// The waves of a tile layout: whole chunks, about `per` steps each; few enough waves that all of
// them are resident at once (24 per CU), so that none has to wait for a second round.
// stepVo / stepA / stepChunkEnd: first value, blocks in half 0 and "a wave may end here" of every
// step.  waveDesc: 8 ints per wave (see DeviceTiles); ahead: per step the first value and the
// blocks in half 0 of the step four further on (the wave's last when past it).
static void tile_waves(int steps, int nCU, int perMin, const std::vector<int> &stepVo, const std::vector<int> &stepA,
                       const std::vector<int> &stepChunkEnd, std::vector<int> &waveDesc, std::vector<int> &ahead)
{
    nCU = std::max(1, nCU);
    const int tper = std::getenv("MX_TILE_PER") ? std::atoi(std::getenv("MX_TILE_PER")) : 0;
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
                HostTiles &T, const char *rowTaken = nullptr, const std::vector<StripChunk> *stripChunks = nullptr)
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
                 mx::DeviceTiles &T, int *tile_nnz, const char *rowTaken = nullptr,
                 const std::vector<StripChunk> *stripChunks = nullptr, std::vector<int> *hdrOut = nullptr)
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
        const char *envr = std::getenv("MX_CSR_REDUCE");
        if (envr && !std::strcmp(envr, "rows")) A.scan = false;
        if (envr && !std::strcmp(envr, "scan")) A.scan = true;
    }
    // 16-bit column offsets when every workgroup's columns span fewer than 65536
    // (MX_CSR_COL16=0 keeps 32-bit ids)
    const char *env16 = std::getenv("MX_CSR_COL16");
    bool narrow = !(env16 && std::atoi(env16) == 0) && nnz > 0;
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
        const char *ed = std::getenv("MX_CSR_DICT");
        if (nnz >= 65536 && !(ed && !std::atoi(ed))) {
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

}  // namespace

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
        for (const mx::SliceChunk &c : sliceChunks[q]) sliceSteps[q] += c.steps;
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
    std::vector<SliceWg> wgs;
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
            top.first += ch[c].steps;
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
        if (const char *e = std::getenv("MX_SLICE_CAP")) {
            const int v = std::atoi(e);
            if (v >= BE && v <= 4096) out->cap = v / BE * BE;
        }
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
    const char *e = std::getenv("MX_CSR_NPT");
    const int v = e ? std::atoi(e) : 0;
    if (dtype == MX_F64) return (v == 4 || v == 8) ? v : 4;
    return (v == 8 || v == 16) ? v : 8;
}

struct mx_plan {
    mx_dtype dtype = MX_F64;
    int rows = 0, cols = 0, nnz = 0;
    mx::DeviceCsr csr;        // CSR part (or its short rows), row-tile form (csr_rows_kernel)
    mx::DeviceSlices slices;  // CSR part (or its long rows), x-resident-in-LDS form (csr_slice_kernel)
    int csr_variant = 0;      // 0 = row tiles, 1 = slices, 2 = row tiles for the short rows, then slices for the long ones
    bool fused = false;       // slices in the one-launch form (slices.fused), until a misplaced workgroup is reported
    unsigned fused_seq = 0;   // one-launch products queued so far
    int csr_nnz = 0;
    double est_rows_us = 0, est_slices_us = 0;  // what the choice of the form was made from (0: no choice was made)
    mx::DeviceTiles tiles;    // tile part, general form (tile_kernel)
    mx::DeviceTiles strips;   // tile part, binary16 strips on rows of their own (tile_dense_kernel)
    int tile_nnz = 0;
    // binary16 plans whose general tiles share rows with the CSR part: the CSR part's sums as
    // binary32, one per row, which the tile kernel adds to (y is then rounded once)
    void *ywide = nullptr;
    int ext_dCols = 0, ext_dRows = 0, ext_nnzRowD = 0, ext_frags = 0;  // what the extraction behind the plan selected
    int prep_route = 0;  // 0 = laid out on the host from host arrays, 1 = on the device from device arrays
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

extern "C" int mx_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

extern "C" void mx_plan_destroy(mx_plan *plan)
{
    if (!plan) return;
    free_csr(plan->csr);
    free_slices(plan->slices);
    free_tiles(plan->tiles);
    free_tiles(plan->strips);
    (void)hipFree(plan->ywide);
    if (plan->ev0) (void)hipEventDestroy(plan->ev0);
    if (plan->ev1) (void)hipEventDestroy(plan->ev1);
    if (plan->stream) (void)hipStreamDestroy(plan->stream);
    delete plan;
}

// Mean milliseconds per iteration of `body` over `iters` back-to-back runs after `warm`
// untimed ones, by events on the stream the kernels run on.
template <typename F>
static int time_loop(mx_plan *plan, int warm, int iters, F body, double *ms)
{
    for (int i = 0; i < warm; ++i) {
        int rc = body();
        if (rc) return rc;
    }
    MX_HIP(hipStreamSynchronize(plan->stream));
    MX_HIP(hipEventRecord(plan->ev0, plan->stream));
    for (int i = 0; i < iters; ++i) {
        int rc = body();
        if (rc) return rc;
    }
    MX_HIP(hipEventRecord(plan->ev1, plan->stream));
    MX_HIP(hipEventSynchronize(plan->ev1));
    float t = 0.f;
    MX_HIP(hipEventElapsedTime(&t, plan->ev0, plan->ev1));
    *ms = (double)t / (double)std::max(iters, 1);
    return MX_OK;
}

// The word in host memory that the one-launch kernels write when a workgroup is misplaced: one per
// process, pinned and mapped, allocated at the first use (null when that fails).
static std::atomic<bool> g_fused_off{false};
static unsigned *misplaced_word()
{
    static std::once_flag once;
    static unsigned *word = nullptr;
    std::call_once(once, []() {
        void *p = nullptr;
        if (hipHostMalloc(&p, 64, hipHostMallocMapped) == hipSuccess && p) {
            std::memset(p, 0, 64);
            word = (unsigned *)p;
        } else {
            (void)hipGetLastError();
        }
    });
    return word;
}

extern "C" int mx_debug_fused_misplaced(int set)
{
    unsigned *word = misplaced_word();
    if (!word) return MX_ERR_DEVICE;
    *(volatile unsigned *)word = set ? 1u : 0u;
    if (!set) g_fused_off.store(false);
    return MX_OK;
}

// `partial` (optional): where the slice kernel puts the sums of the virtual rows, in place of the
// plan's own buffer.
static int launch_csr_part(mx_plan *plan, const void *x, void *y, int accumulate, hipStream_t s,
                           const mx::DeviceTiles *strips = nullptr, void *partial = nullptr, void *ywide = nullptr)
{
    if (plan->csr_variant != 0 && ((uintptr_t)x & 15)) {
        set_error("mx_spmv: x must be 16-byte aligned for this plan");
        return MX_ERR_ARG;
    }
    if (plan->csr_variant != 1) MX_HIP(mx::launch_csr(plan->dtype, plan->csr, x, y, accumulate, s, ywide));
    if (plan->csr_variant == 1 && plan->fused && !strips && !partial) {  // (sums in a caller's buffer: the two launches)
        // one launch.  A workgroup that found its share of the work taken already has said so in the
        // host-visible word: the products since the last look cannot be trusted, and from here on every
        // plan takes the two launches.
        unsigned *word = misplaced_word();
        // (a one-launch product carries the number of its launch: under stream capture, where the same
        // arguments would be replayed, the two launches are recorded)
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &cap) != hipSuccess) {
            (void)hipGetLastError();
            cap = hipStreamCaptureStatusNone;
        }
        if (cap != hipStreamCaptureStatusNone) {
            // fall through to the two launches below
        } else if (!word || g_fused_off.load()) {
            plan->fused = false;
        } else if (*(volatile unsigned *)word) {
            g_fused_off.store(true);
            plan->fused = false;
            set_error("mx_spmv: two workgroups of an earlier one-launch product took the same share of the work; "
                      "products since the previous call may be wrong; plans use the two-launch form from now on");
            return MX_ERR_DEVICE;
        } else {
            MX_HIP(mx::launch_fused(plan->dtype, plan->slices, x, y, accumulate, s, ywide, word, plan->fused_seq++));
            return MX_OK;
        }
    }
    if (plan->csr_variant != 0) {
        if (partial) {
            mx::DeviceSlices L = plan->slices;  // a view: same arrays, other sums
            L.partial = partial;
            MX_HIP(mx::launch_slices(plan->dtype, L, x, y, accumulate, s, 0, strips, ywide));
        } else {
            MX_HIP(mx::launch_slices(plan->dtype, plan->slices, x, y, accumulate, s, 0, strips, ywide));
        }
    }
    return MX_OK;
}

// Bytes of the sums of a plan's virtual rows (what upload_slices allocates for them).
static size_t partial_bytes(const mx_plan *plan)
{
    if (plan->csr_variant == 0) return 0;
    return ((size_t)plan->slices.chunks * 64 + 64) * (plan->dtype == MX_F64 ? 8 : 4);
}

// Row length from which a row of a split plan goes to the slice kernel (MX_SPLIT_LEN overrides).
static int split_length()
{
    const char *e = std::getenv("MX_SPLIT_LEN");
    const int v = e ? std::atoi(e) : 0;
    return v > 0 ? v : 32;
}

// What the choice between the forms of the CSR part looks at: all of it is counted from the
// matrix, none of it is timed, so the same matrix gets the same plan on every run.
struct CsrStats {
    double linesPerGather = 0;  // mean number of distinct 64-byte lines of x that 64 consecutive entries name
    double vrows = 0;           // virtual rows the slice layout would have (distinct slices per row, long ones cut)
    bool fewValues = false;     // at most 255 distinct values: the one-byte-per-value forms exist
    int mostVrows = 0;          // most virtual rows of any row
};

static CsrStats csr_stats(mx_dtype dtype, int rows, const int *rowPtr, const int *col, const void *val, int nCU)
{
    CsrStats st;
    const int nnz = rowPtr[rows], es = mx::elem_size(dtype), perLine = 64 / es, SW = mx::slice_cols(dtype);
    // (a mean: every stride-th window of 64 entries is enough, at most 65536 of them)
    const long long windows = nnz / 64, stride = std::max<long long>(1, windows / 65536);
    const long long sampled = windows / stride;
    double lines = 0;
#pragma omp parallel for schedule(static) reduction(+ : lines)
    for (long long i = 0; i < sampled; ++i) {
        const long long w = i * stride;
        int l[64];
        for (int k = 0; k < 64; ++k) l[k] = col[w * 64 + k] / perLine;
        std::sort(l, l + 64);
        int d = 1;
        for (int k = 1; k < 64; ++k) d += l[k] != l[k - 1];
        lines += d;
    }
    st.linesPerGather = sampled > 0 ? lines / (double)sampled : 1.0;
    const long long fair = (long long)nnz / ((long long)std::max(nCU, 1) * mx::kSliceWaves * 64);
    const int BE = mx::kSliceBatchEntries;
    const int cap = (int)std::min<long long>(512, std::max<long long>(16, (fair + BE - 1) / BE * BE));
    double vrows = 0;
    int mostVrows = 0;
#pragma omp parallel for schedule(dynamic, 4096) reduction(+ : vrows) reduction(max : mostVrows)
    for (int r = 0; r < rows; ++r) {
        const int a = rowPtr[r], b = rowPtr[r + 1];
        if (b <= a) continue;
        // distinct slices of the row, and what the cap adds for a long run inside one slice (rows come
        // sorted by column from most callers; the residual of an extracted partition does not)
        int n = 0, run = 0, last = -1;
        bool ascending = true;
        for (int p = a; p < b && ascending; ++p) {
            const int q = col[p] / SW;
            ascending = q >= last;
            if (q != last || run == cap) {
                ++n;
                run = 0;
                last = q;
            }
            ++run;
        }
        if (!ascending) {
            int local[64];
            std::vector<int> big;
            int *sl = local;
            if (b - a > 64) {
                big.resize((size_t)(b - a));
                sl = big.data();
            }
            for (int p = a; p < b; ++p) sl[p - a] = col[p] / SW;
            std::sort(sl, sl + (b - a));
            n = 0, run = 0, last = -1;
            for (int p = 0; p < b - a; ++p) {
                if (sl[p] != last || run == cap) {
                    ++n;
                    run = 0;
                    last = sl[p];
                }
                ++run;
            }
        }
        vrows += n;
        mostVrows = std::max(mostVrows, n);
    }
    st.vrows = vrows;
    st.mostVrows = mostVrows;
    const char *ed = std::getenv("MX_CSR_DICT");
    if (nnz >= 65536 && !(ed && !std::atoi(ed))) {
        std::vector<unsigned char> codes, dict;
        int nd = 0;
        st.fewValues = make_value_dict(es, val, nnz, codes, dict, &nd, 255);
    }
    return st;
}

// Estimated time of a product through the row-tile form and through the slice form, in
// microseconds, from rates measured on MI355X (back-to-back products, five synthetic workloads at
// three sizes each; the estimates are within 20 % of every one of them):
//  * row tiles: one launch (2.5), then the entries at a cost that grows with the number of
//    distinct lines of x a wave-wide gather names -- 1.2 + 0.065 * lines microseconds per million
//    entries -- times up to 1.6 when x does not fit one L2 (4 MB) and the gathers are scattered,
//    times 0.85 with one byte per value;
//  * slices: two dependent launches and the copy of x into LDS (9.5), the stream of stored
//    bytes (column offset 2 + value sizeof(valT) or 1, padded by about 8 %) at 9 bytes per ns
//    while it stays inside the memory-side cache from one product to the next (up to 64 MB),
//    5.8 beyond, and 2 microseconds per million virtual rows in the combine kernel.
static void csr_estimates(mx_dtype dtype, int cols, int nnz, const CsrStats &st, double *usRows, double *usSlices)
{
    const double es = mx::elem_size(dtype), M = 1e-6 * (double)nnz;
    double perM = 1.2 + 0.065 * st.linesPerGather;
    // (scattered gathers that miss the L2: nothing for a stencil's dozen lines, all of it from two dozen on)
    if ((double)cols * es > 4.0e6) perM *= 1.0 + 0.6 * std::min(1.0, std::max(0.0, (st.linesPerGather - 12.0) / 12.0));
    if (st.fewValues) perM *= 0.85;
    *usRows = 2.5 + M * perM;
    const double bytes = (double)nnz * 1.08 * (2.0 + (st.fewValues ? 1.0 : es));
    *usSlices = 9.5 + bytes / (bytes <= 64.0e6 ? 9.0e6 : 5.8e6) + 2.0e-6 * st.vrows;
}

// Which forms of the CSR part a plan may take (want[0] row tiles, [1] slices, [2] split) after the
// caller's flags, MX_CSR_KERNEL and -- when both of the first two are still open and nothing is to be
// timed -- the estimates.  S = slice_count() of the matrix.
struct CsrChoice {
    bool want[3] = {true, true, false};
    double usRows = 0, usSlices = 0;  // the estimates, when they decided
    bool fewValues = false;
    int mostVrows = -1;  // most virtual rows of a row (-1: not counted)
};
static bool plan_autotune()
{
    static const bool on = std::getenv("MX_PLAN_AUTOTUNE") && std::atoi(std::getenv("MX_PLAN_AUTOTUNE"));
    return on;
}
// Whether a plan asks for the one-launch form of the slices.  Never with MX_PLAN_NO_FUSE or
// MX_CSR_FUSED=0, after a misplaced workgroup was reported, or for a matrix with a row of more than
// eight virtual rows (mostVrows < 0: not counted, the layout will see).  Otherwise where it pays:
// the workgroup that comes last to a group of rows adds that group up alone, and the slowest
// workgroup comes last to all of its groups, so the form wins while a workgroup's rows are few --
// measured on the block-clustered workload at 256 workgroups: 9.5 against 11.3 us at 32 768 rows, a
// tie at 49 152 and at 65 536 -- and is taken up to 160 rows per workgroup.  MX_PLAN_FUSE (or
// MX_CSR_FUSED=1) takes it wherever the matrix suits it.
static bool fused_wanted(int flags, int rows, int mostVrows, int nCU)
{
    static const char *env = std::getenv("MX_CSR_FUSED");
    if ((flags & MX_PLAN_NO_FUSE) || (env && !std::atoi(env)) || g_fused_off.load()) return false;
    if (mostVrows > mx::kSliceLightSegs || nCU % mx::kFusedXcds) return false;
    if ((flags & MX_PLAN_FUSE) || (env && std::atoi(env))) return true;
    return (long long)rows <= 160LL * nCU;
}
// What the one-launch form saves of the slice form's estimate where it is taken (microseconds): the second
// launch and its wait, less the adding at the end of the first.
constexpr double kFusedSavesUs = 1.8;

static CsrChoice choose_csr_form(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val,
                                 int flags, int nCU, int S, bool mayFuse = false)
{
    CsrChoice c;
    const char *env = std::getenv("MX_CSR_KERNEL");
    if (flags & MX_PLAN_CSR_ROWS) c.want[1] = c.want[2] = false;
    if (flags & MX_PLAN_CSR_SLICES) c.want[0] = c.want[2] = false;
    if (env && !std::strcmp(env, "rows")) c.want[0] = true, c.want[1] = c.want[2] = false;
    if (env && !std::strcmp(env, "slices")) c.want[1] = true, c.want[0] = c.want[2] = false;
    if (env && !std::strcmp(env, "split")) c.want[2] = true, c.want[0] = c.want[1] = false;
    if (S == 0) c.want[1] = c.want[2] = false;
    if (c.want[0] && c.want[1] && !plan_autotune()) {
        const CsrStats st = csr_stats(dtype, rows, rowPtr, col, val, nCU);
        csr_estimates(dtype, cols, rowPtr[rows], st, &c.usRows, &c.usSlices);
        c.fewValues = st.fewValues;
        c.mostVrows = st.mostVrows;
        // (the one-launch form of the slices, where the plan would take it: the device's placement is looked at
        // later, and a plan whose strips ride in the second launch keeps both launches)
        if (mayFuse && fused_wanted(flags, rows, st.mostVrows, nCU)) c.usSlices -= kFusedSavesUs;
        c.want[c.usSlices < c.usRows ? 0 : 1] = false;
    }
    return c;
}

// Puts the CSR part on the device.  Three executable forms exist: row tiles with direct x
// gathers; column slices with x resident in LDS; and a split in which the long rows (most of
// the entries of a matrix with a heavy tail of row lengths) take the slices and the many short
// ones the row tiles.  Unless a flag or MX_CSR_KERNEL=rows|slices|split forces one, the choice
// between the first two is made from counts over the matrix (csr_stats, csr_estimates): the form
// with the lower estimate is built, and the one-byte-per-value form of it wherever the matrix has
// at most 255 distinct values.  Nothing is timed, so a matrix gets the same plan on every run, with
// or without a profiler attached.  MX_PLAN_AUTOTUNE=1 brings the timed choice back: both forms
// (and both value forms) are built and run a few times on the spot and the fastest is kept.
// The split runs only when asked for: it has not won on any matrix measured so far.
// `stripRows` (optional): rows that the strip form of the tile kernel writes (and the CSR part has
// nothing for).
// `segOut` (optional): receives the virtual rows of every matrix row when the slice form is taken.
static int setup_csr_part(mx_plan *plan, const int *rowPtr, const int *col, const void *val, int flags,
                          const char *stripRows = nullptr,
                          std::pair<std::vector<int>, std::vector<int>> *segOut = nullptr)
{
    const int rows = plan->rows, cols = plan->cols;
    const int nnz = rowPtr[rows];
    const size_t es = (size_t)mx::elem_size(plan->dtype);
    plan->csr_nnz = nnz;
    hipDeviceProp_t prop;
    int dev = 0;
    MX_HIP(hipGetDevice(&dev));
    MX_HIP(hipGetDeviceProperties(&prop, dev));
    const int nCU = std::max(1, prop.multiProcessorCount);
    const int S = slice_count(plan->dtype, rows, cols, nnz, nCU);
    CsrChoice pick = choose_csr_form(plan->dtype, rows, cols, rowPtr, col, val, flags, nCU, S, stripRows == nullptr);
    bool(&want)[3] = pick.want;
    plan->est_rows_us = pick.usRows;
    plan->est_slices_us = pick.usSlices;
    const bool autotune = plan_autotune();
    // the split: rows of at least split_length() entries, when they hold a good part of the matrix
    std::vector<char> longRow;
    int longNnz = 0, longRows = 0;
    if (S > 0 && want[2]) {
        const int T = split_length();
        longRow.assign((size_t)rows, 0);
        for (int r = 0; r < rows; ++r)
            if (rowPtr[r + 1] - rowPtr[r] >= T) {
                longRow[r] = 1;
                longNnz += rowPtr[r + 1] - rowPtr[r];
                ++longRows;
            }
        if (longNnz < 4096 || longRows == rows || (double)longNnz < 0.1 * (double)nnz) want[2] = false;
    }
    if (!want[0] && !want[1] && !want[2]) want[0] = true;  // a matrix the slice kernel cannot take runs on row tiles whatever was asked
    const int nWant = (int)want[0] + (int)want[1] + (int)want[2];
    int rc;
    void *tx = nullptr, *ty = nullptr;  // an x and a y to time candidates with, when there is a choice
    auto scratch = [&]() -> int {
        if (tx) return MX_OK;
        int e = upload_bytes(&tx, nullptr, 0, std::max<size_t>(cols * es, 16));
        if (e) return e;
        if ((e = upload_bytes(&ty, nullptr, 0, std::max<size_t>(rows * es, 16)))) {
            (void)hipFree(tx);
            tx = nullptr;
        }
        return e;
    };
    // the one-launch form of the slices, for a CSR part that is the whole product on a device whose
    // workgroups land where the layout assumes
    bool wantFused = want[1] && fused_wanted(flags, rows, pick.mostVrows, nCU) && !stripRows;
    if (wantFused) {
        int ok = 0;
        MX_HIP(mx::fused_placement_ok(nCU, &ok));
        wantFused = ok != 0;
    }
    auto build = [&](int v, mx::DeviceCsr &C, mx::DeviceSlices &L) -> int {
        if (v == 0) return upload_csr(plan->dtype, rows, cols, nnz, rowPtr, col, val, C, nullptr);
        if (v == 1) return upload_slices(plan->dtype, rows, cols, rowPtr, col, val, nCU, S, nullptr, L, stripRows, segOut, wantFused);
        // the short rows as a CSR matrix of their own (the long rows empty), the long ones as slices
        std::vector<int> rp((size_t)rows + 1, 0);
        for (int r = 0; r < rows; ++r) rp[r + 1] = rp[r] + (longRow[r] ? 0 : rowPtr[r + 1] - rowPtr[r]);
        std::vector<int> c2((size_t)rp[rows]);
        std::vector<unsigned char> v2((size_t)rp[rows] * es);
#pragma omp parallel for schedule(static)
        for (int r = 0; r < rows; ++r) {
            if (longRow[r]) continue;
            const int n = rowPtr[r + 1] - rowPtr[r];
            if (n == 0) continue;
            std::memcpy(&c2[rp[r]], col + rowPtr[r], (size_t)n * sizeof(int));
            std::memcpy(&v2[(size_t)rp[r] * es], (const unsigned char *)val + (size_t)rowPtr[r] * es, (size_t)n * es);
        }
        int r1 = upload_csr(plan->dtype, rows, cols, rp[rows], rp.data(), c2.data(), v2.data(), C, nullptr);
        if (r1) return r1;
        // (binary64 blocks do not ride with the split form: their rows stay with the combine kernel's own
        // kinds and the blocks add to y afterwards)
        return upload_slices(plan->dtype, rows, cols, rowPtr, col, val, nCU, S, longRow.data(), L,
                             plan->dtype == MX_F64 ? nullptr : stripRows);
    };
    double best = 0.0;
    bool have = false;
    rc = MX_OK;
    for (int v = 0; v < 3 && !rc; ++v) {
        if (!want[v]) continue;
        mx::DeviceCsr C;
        mx::DeviceSlices L;
        rc = build(v, C, L);
        double ms = 0.0;
        // (the one-byte-per-value form is taken wherever it exists; MX_CSR_DICT=0 keeps it from being built)
        if (!rc && !autotune) {
            if (v == 0 && C.codes) C.useDict = true;
            if (v != 0 && L.ecode) L.useDict = true;
        }
        const bool choice = autotune && (nWant > 1 || (v == 0 && C.codes) || (v == 1 && L.ecode));
        if (!rc && choice) rc = scratch();
        if (!rc && choice) {
            std::swap(plan->csr, C);
            std::swap(plan->slices, L);
            const int keepVariant = plan->csr_variant;
            plan->csr_variant = v;
            rc = time_loop(plan, 3, 10, [&]() { return launch_csr_part(plan, tx, ty, 0, plan->stream); }, &ms);
            if (!rc && v == 1 && plan->slices.ecode) {  // the same slices with one byte per value
                double msDict = 0.0;
                plan->slices.useDict = true;
                rc = time_loop(plan, 3, 10, [&]() { return launch_csr_part(plan, tx, ty, 0, plan->stream); }, &msDict);
                const char *ed = std::getenv("MX_CSR_DICT");
                if (!rc && (msDict < ms || (ed && std::atoi(ed) == 2))) ms = msDict;
                else plan->slices.useDict = false;
            }
            if (!rc && v == 0 && plan->csr.codes) {  // the same rows with one byte per value (MX_CSR_DICT=2: whatever the timing)
                double msDict = 0.0;
                plan->csr.useDict = true;
                rc = time_loop(plan, 3, 10, [&]() { return launch_csr_part(plan, tx, ty, 0, plan->stream); }, &msDict);
                const char *ed = std::getenv("MX_CSR_DICT");
                if (!rc && (msDict < ms || (ed && std::atoi(ed) == 2))) ms = msDict;
                else plan->csr.useDict = false;
            }
            plan->csr_variant = keepVariant;
            std::swap(plan->csr, C);
            std::swap(plan->slices, L);
        }
        if (!rc && (!have || ms < best)) {
            std::swap(plan->csr, C);
            std::swap(plan->slices, L);
            plan->csr_variant = v;
            plan->fused = v == 1 && plan->slices.fused;
            best = ms;
            have = true;
        }
        free_csr(C);
        free_slices(L);
    }
    (void)hipFree(tx);
    (void)hipFree(ty);
    return rc;
}

// Minimum fill of a fragment for the MFMA tile kernel to take it (default plans;
// MX_TILE_GATE=<fraction> overrides).  A fragment costs its bitmap, its value offset and fragK
// column ids whatever it holds, and the decode work of a whole tile; below about half full the
// same entries are cheaper in the CSR part.
static double tile_gate(mx_dtype)
{
    const char *e = std::getenv("MX_TILE_GATE");
    if (e) {
        const double v = std::atof(e);
        if (v >= 0.0 && v <= 1.0) return v;
    }
    return 0.5;
}

// Do the tiles pay for their launch?  (The reference gates its tile kernel on the size of the
// matrix and its fill, test/test_autotc_spmv.cpp:1507,1518.)  What they take off the CSR part
// saves es + 2 bytes per entry of its stream; what they cost is one more dependent launch and
// their own stream.  Rates as measured on MI355X: the CSR part and the strip form of the tile
// kernel move about 5000 bytes per ns (5 TB/s), the general tile kernel, bound by instruction
// issue, about 2200; a further launch in the sequence costs about 5 us with its ramp and tail
// (the strips of the mixed workload break even at about 15 M entries when launched apart);
// strips usually ride in the launch of the combine kernel, where they came out ahead at every
// size tried (1.7 M entries and up): they are charged little.
// general*: the reference's fragments that pass the fill gate; strip*: the chunks of the plan's
// own (binary16 strips, or binary64 8 x 8 blocks with `blocks64`).
// 0 = nothing pays, 1 = only the plan's own chunks do, 2 = keep both.
// `netNs` (optional): what the forms that are kept save per product by this estimate, in ns.
static int tiles_worth(mx_dtype dtype, int fragM, int fragK, bool blocks64, double generalEntries, double generalFrags,
                       double stripEntries, double stripBlocks, double *netNs = nullptr)
{
    const int es = mx::elem_size(dtype);
    const double blockBytes = (double)fragM * (blocks64 ? 8 : fragK) * es, slots = mx::tile_slots(dtype);
    const double generalBytes = generalFrags * blockBytes + generalFrags / slots * (mx::kTileHdr * 4.0 + 256.0);
    const double stripBytes = stripBlocks * blockBytes + stripBlocks / slots * (mx::kTileHdr * 4.0);
    const double launchNs = 5000.0, stripLaunchNs = 1000.0, fastRate = 5000.0, generalRate = 2200.0;  // bytes per ns
    const double savedNs = (generalEntries + stripEntries) * (es + 2) / fastRate;
    const double generalCost = generalFrags > 0 ? launchNs + generalBytes / generalRate : 0.0;
    const double stripCost = stripBlocks > 0 ? stripLaunchNs + stripBytes / fastRate : 0.0;
    if (netNs) *netNs = 0.0;
    if (savedNs <= generalCost + stripCost) return 0;
    if (generalFrags > 0 && generalEntries * (es + 2) / fastRate <= generalCost) {
        if (netNs) *netNs = stripEntries * (es + 2) / fastRate - stripCost;
        return 1;
    }
    if (netNs) *netNs = savedNs - generalCost - stripCost;
    return 2;
}

// MX_PLAN_LOG=1: the phases of mx_plan_create with their host time, on stderr
struct PhaseLog {
    bool on = std::getenv("MX_PLAN_LOG") && std::atoi(std::getenv("MX_PLAN_LOG"));
    std::chrono::steady_clock::time_point t = std::chrono::steady_clock::now();
    void operator()(const char *what)
    {
        if (!on) return;
        const auto now = std::chrono::steady_clock::now();
        std::fprintf(stderr, "mx_plan_create: %-38s %8.1f ms\n", what, std::chrono::duration<double, std::milli>(now - t).count());
        t = now;
    }
};

// The host half of a plan for an extracted partition: which fragments the tile kernels take
// (`sel`), which rows of A_dd go into strip chunks of the plan's own (`taken`, `stripChunks`,
// `stripRows` = the same rows in the caller's numbering), and the CSR part -- the residual plus
// every entry of A_dd that the tiles leave -- in the caller's numbering.
struct HostPlanParts {
    std::vector<char> sel, taken, stripRows;  // stripRows: 1 = written by the strips alone, 2 = shared with binary64 blocks
    std::vector<char> inBlock;                // binary64: A_dd entries that went into 8 x 8 blocks
    std::vector<StripChunk> stripChunks;
    std::vector<int> rowPtr, col;
    std::vector<unsigned char> val;
};

static int plan_host_parts(const mx_partition *P, int flags, HostPlanParts &H, PhaseLog &phase, bool noBlocks = false)
{
    const int es = mx::elem_size(P->dtype), fragK = P->fragK, fragM = P->fragM;
    const int rows = P->rows, cols = P->cols;
    // residual column space -> the caller's column ids, so x needs no permutation
    std::vector<int> colOrig(cols);
    for (int c = 0; c < P->dCols; ++c) colOrig[c] = P->descColId[c];
    for (int c = P->dCols; c < cols; ++c) colOrig[c] = P->newArray[c - P->dCols];
    // which fragments go to the tile kernel
    const int chunkNum = P->chunkNum, nFrags = P->chunkPtr[chunkNum];
    std::vector<char> &sel = H.sel;
    sel.assign((size_t)nFrags, 0);
    const double gate = tile_gate(P->dtype);
    if (!(flags & MX_PLAN_NO_TILES)) {
        for (int f = 0; f < nFrags; ++f) {
            const int vals = P->fragPtr[f + 1] - P->fragPtr[f];
            sel[f] = (flags & MX_PLAN_ALL_TILES) ? vals > 0 : (vals > 0 && (double)vals >= gate * fragM * fragK);
        }
    }
    // binary16 rows of A_dd whose columns, in the caller's numbering, fall into at most a
    // step's worth of blocks of fragK consecutive columns and fill them at least half -- a row
    // of a dense strip in the simplest case -- with nothing in the residual and no column
    // named twice.  The blocks of a row start at multiples of fragK, or, where that takes fewer
    // blocks, at the row's own first column plus multiples of fragK (a strip that starts off
    // the grid of eight is four blocks then, not five: two chunks share a step again).  Rows
    // with the same set of blocks are put together, fragM at a time, into chunks of the plan's
    // own (the canonical chunks follow the row order, where rows of other shapes fall between
    // them and one chunk straddles two strips).  A chunk of at least fragM/2 rows goes to
    // tile_dense_kernel; its rows leave the fragments.
    std::vector<char> &taken = H.taken;
    std::vector<StripChunk> &stripChunks = H.stripChunks;
    taken.clear();
    stripChunks.clear();
    if (P->dtype == MX_F16 && fragM == 8 && fragK == 8 && !(flags & (MX_PLAN_NO_TILES | MX_PLAN_ALL_TILES)) &&
        !(std::getenv("MX_NO_STRIPS") && std::atoi(std::getenv("MX_NO_STRIPS")))) {
        constexpr int kMaxBlocks = 8;  // block slots of a binary16 step
        struct Cand {
            int nb, b[kMaxBlocks], n, i;  // first column of every block (ascending), entries, row of A_dd
        };
        std::vector<Cand> cand;
        const int nThreads = std::max(1, omp_get_max_threads());
        std::vector<std::vector<Cand>> found((size_t)nThreads);
#pragma omp parallel num_threads(nThreads)
        {
            std::vector<Cand> &mine = found[(size_t)omp_get_thread_num()];
            std::vector<int> cols;
            // the blocks of the sorted columns for blocks that start at shift + multiples of fragK; false
            // when they are too many or one would reach past the end of x
            auto blocks_at = [&](int shift, Cand &c) {
                c.nb = 0;
                for (int col : cols) {
                    const int first = (col - shift) / fragK * fragK + shift;
                    if (first + fragK > P->cols) return false;
                    if (c.nb == 0 || c.b[c.nb - 1] != first) {
                        if (c.nb == kMaxBlocks) return false;
                        c.b[c.nb++] = first;
                    }
                }
                return true;
            };
#pragma omp for schedule(static)
            for (int i = 0; i < P->dRows; ++i) {
                const int p0 = P->ddRowPtr[i], n = P->ddRowPtr[i + 1] - p0, r = P->rId[i];
                if (n < fragK / 2 || n > kMaxBlocks * fragK || P->cdRowPtr[r + 1] != P->cdRowPtr[r]) continue;
                cols.resize((size_t)n);
                for (int k = 0; k < n; ++k) cols[k] = P->descColId[P->ddColInd[p0 + k]];
                std::sort(cols.begin(), cols.end());
                bool twice = false;
                for (int k = 1; k < n; ++k) twice = twice || cols[k] == cols[k - 1];
                if (twice) continue;  // named twice: stays with the fragments, where the last counts
                Cand c, own;
                c.n = own.n = n;
                c.i = own.i = i;
                bool ok = blocks_at(0, c);
                const int shift = cols[0] % fragK;
                if (shift && blocks_at(shift, own) && (!ok || own.nb < c.nb)) {
                    c = own;
                    ok = true;
                }
                if (!ok || 2 * n < c.nb * fragK) continue;
                for (int k = c.nb; k < kMaxBlocks; ++k) c.b[k] = -1;
                mine.push_back(c);
            }
        }
        for (const std::vector<Cand> &f : found) cand.insert(cand.end(), f.begin(), f.end());
        found.clear();
        auto same = [](const Cand &x, const Cand &y) { return x.nb == y.nb && std::equal(x.b, x.b + kMaxBlocks, y.b); };
        // (a total order -- no two candidates share a row -- so the result does not depend on how the sort splits its work)
        __gnu_parallel::sort(cand.begin(), cand.end(), [](const Cand &x, const Cand &y) {
            if (!std::equal(x.b, x.b + kMaxBlocks, y.b)) return std::lexicographical_compare(x.b, x.b + kMaxBlocks, y.b, y.b + kMaxBlocks);
            return x.i < y.i;
        });
        taken.assign((size_t)P->dRows, 0);
        const uint16_t *ddv16 = (const uint16_t *)P->ddVal.data();  // binary16 bit patterns
        // runs of candidates with the same blocks, and the first chunk of each
        std::vector<size_t> runStart;
        std::vector<size_t> runChunk0;
        size_t nStripChunks = 0;
        for (size_t a = 0; a < cand.size();) {
            size_t b = a;
            while (b < cand.size() && same(cand[b], cand[a])) ++b;
            const size_t full = (b - a) / fragM, rest = (b - a) % fragM;
            const size_t n = full + (2 * rest >= (size_t)fragM ? 1 : 0);
            if (n) {
                runStart.push_back(a);
                runChunk0.push_back(nStripChunks);
                nStripChunks += n;
            }
            a = b;
        }
        runStart.push_back(cand.size());
        runChunk0.push_back(nStripChunks);
        stripChunks.resize(nStripChunks);
        const long nRuns = (long)runChunk0.size() - 1;
#pragma omp parallel for schedule(dynamic, 16)
        for (long run = 0; run < nRuns; ++run) {
            const size_t a = runStart[run];
            const int nb = cand[a].nb;
            size_t b = a;
            while (b < cand.size() && same(cand[b], cand[a])) ++b;
            for (size_t q = 0; q < runChunk0[run + 1] - runChunk0[run]; ++q) {
                const size_t g = a + q * fragM;
                const int nr = (int)std::min(b - g, (size_t)fragM);
                StripChunk &C = stripChunks[runChunk0[run] + q];
                C.nnz = 0;
                C.blocks.resize(nb);
                for (int k = 0; k < nb; ++k) {
                    C.blocks[k].vals.assign((size_t)fragM * fragK * es, 0);
                    for (int c = 0; c < fragK; ++c) C.blocks[k].cols[c] = cand[a].b[k] + c;
                }
                for (int j = 0; j < 8; ++j) C.rows[j] = -1;
                for (int j = 0; j < nr; ++j) {
                    const int i = cand[g + j].i;
                    taken[i] = 1;
                    C.rows[j] = P->rId[i];
                    C.nnz += cand[g + j].n;
                    for (int p = P->ddRowPtr[i]; p < P->ddRowPtr[i + 1]; ++p) {
                        const int c = P->descColId[P->ddColInd[p]];
                        const int k = (int)(std::upper_bound(cand[a].b, cand[a].b + nb, c) - cand[a].b) - 1;
                        ((uint16_t *)C.blocks[k].vals.data())[j * fragK + (c - cand[a].b[k])] = ddv16[p];
                    }
                }
            }
        }
        if (stripChunks.empty()) taken.clear();
    }
    // binary64: aligned 8 x 8 blocks (eight consecutive rows from a multiple of eight, eight consecutive
    // columns from a multiple of eight, both in the caller's numbering) that the extracted block fills
    // at least three quarters -- the dense blocks of a block-structured matrix.  Their entries leave the
    // CSR part (and the reference's fragments, which are not used beside them: the general tile kernel
    // is bound by instruction issue and has not paid on any matrix measured); each row of eight rows with
    // such blocks becomes one chunk for tile_block_wave.  A column named twice keeps its last value in
    // the block; the earlier ones stay in the CSR part, so that y is the sum of all of them.
    std::vector<char> &inBlock = H.inBlock;
    inBlock.clear();
    const char *envNoBlocks = std::getenv("MX_NO_BLOCKS");
    if (P->dtype == MX_F64 && !noBlocks && !(flags & (MX_PLAN_NO_TILES | MX_PLAN_ALL_TILES)) &&
        !(envNoBlocks && std::atoi(envNoBlocks)) && P->dRows > 0) {
        const int need = 48;  // of 64
        std::vector<int> ddRowOf((size_t)rows, -1);
        for (int i = 0; i < P->dRows; ++i) ddRowOf[P->rId[i]] = i;
        const int nbr = (rows + 7) / 8;
        std::vector<std::vector<int>> blocksOf((size_t)nbr);  // block columns taken, ascending, per block row
#pragma omp parallel
        {
            std::vector<int> bc;
#pragma omp for schedule(dynamic, 64)
            for (int br = 0; br < nbr; ++br) {
                bc.clear();
                for (int r = 8 * br; r < std::min(rows, 8 * br + 8); ++r) {
                    const int i = ddRowOf[r];
                    if (i < 0) continue;
                    for (int p = P->ddRowPtr[i]; p < P->ddRowPtr[i + 1]; ++p) {
                        if (p + 1 < P->ddRowPtr[i + 1] && P->ddColInd[p + 1] == P->ddColInd[p]) continue;  // an earlier twin
                        bc.push_back(P->descColId[P->ddColInd[p]] / 8);
                    }
                }
                if ((int)bc.size() < need) continue;
                std::sort(bc.begin(), bc.end());
                for (size_t a = 0; a < bc.size();) {
                    size_t b = a;
                    while (b < bc.size() && bc[b] == bc[a]) ++b;
                    if ((int)(b - a) >= need && (bc[a] + 1) * 8 <= cols) blocksOf[br].push_back(bc[a]);
                    a = b;
                }
            }
        }
        size_t nChunks = 0;
        for (int br = 0; br < nbr; ++br) nChunks += !blocksOf[br].empty();
        if (nChunks > 0) {
            inBlock.assign((size_t)P->ddRowPtr[P->dRows], 0);
            H.stripRows.assign((size_t)rows, 0);
            std::vector<int> chunkOf((size_t)nbr, -1);
            for (int br = 0; br < nbr; ++br)
                if (!blocksOf[br].empty()) {
                    chunkOf[br] = (int)stripChunks.size();
                    stripChunks.emplace_back();
                }
            const double *ddv = (const double *)P->ddVal.data();
#pragma omp parallel for schedule(dynamic, 64)
            for (int br = 0; br < nbr; ++br) {
                if (chunkOf[br] < 0) continue;
                const std::vector<int> &bcs = blocksOf[br];
                StripChunk &C = stripChunks[chunkOf[br]];
                C.nnz = 0;
                C.blocks.resize(bcs.size());
                for (size_t b = 0; b < bcs.size(); ++b) {
                    C.blocks[b].vals.assign((size_t)64 * es, 0);
                    for (int c = 0; c < 8; ++c) C.blocks[b].cols[c] = bcs[b] * 8 + c;
                }
                for (int j = 0; j < 8; ++j) {
                    const int r = 8 * br + j;
                    C.rows[j] = r < rows ? r : -1;
                    if (r >= rows) continue;
                    H.stripRows[r] = 2;
                    const int i = ddRowOf[r];
                    if (i < 0) continue;
                    for (int p = P->ddRowPtr[i]; p < P->ddRowPtr[i + 1]; ++p) {
                        if (p + 1 < P->ddRowPtr[i + 1] && P->ddColInd[p + 1] == P->ddColInd[p]) continue;
                        const int c = P->descColId[P->ddColInd[p]];
                        const auto it = std::lower_bound(bcs.begin(), bcs.end(), c / 8);
                        if (it == bcs.end() || *it != c / 8) continue;
                        ((double *)C.blocks[it - bcs.begin()].vals.data())[j * 8 + c % 8] = ddv[p];
                        inBlock[p] = 1;
                        ++C.nnz;
                    }
                }
            }
            std::fill(sel.begin(), sel.end(), 0);
        }
    }
    phase("fragment gate, strip rows");
    if (!taken.empty()) {
        // the gate again, on what the taken rows leave of each fragment
#pragma omp parallel for schedule(static)
        for (int w = 0; w < chunkNum; ++w) {
            uint64_t rowsLeft = 0;  // bits of the rows that stay
            for (int r = 0; r < fragM; ++r) {
                const int i = w * fragM + r;
                if (i < P->dRows && !taken[i]) rowsLeft |= 0xffull << (r * fragK);
            }
            for (int f = P->chunkPtr[w]; f < P->chunkPtr[w + 1]; ++f) {
                const int vals = __builtin_popcountll(P->fragBit64[f] & rowsLeft);
                sel[f] = sel[f] && vals > 0 && (double)vals >= gate * fragM * fragK;
            }
        }
    }
    // do the tiles pay for their launch (tiles_worth)?  MX_PLAN_KEEP_TILES skips the question.
    if (!(flags & (MX_PLAN_NO_TILES | MX_PLAN_ALL_TILES | MX_PLAN_KEEP_TILES))) {
        double generalEntries = 0, generalFrags = 0, stripEntries = 0, stripBlocks = 0;
        for (int w = 0; w < chunkNum; ++w) {
            uint64_t rowsLeft = ~0ull;
            if (!taken.empty())
                for (int r = 0; r < fragM; ++r) {
                    const int i = w * fragM + r;
                    if (i < P->dRows && taken[i]) rowsLeft &= ~(0xffull << (r * fragK));
                }
            for (int f = P->chunkPtr[w]; f < P->chunkPtr[w + 1]; ++f) {
                if (!sel[f]) continue;
                generalFrags += 1;
                generalEntries += taken.empty() ? P->fragPtr[f + 1] - P->fragPtr[f]
                                                : __builtin_popcountll(P->fragBit64[f] & rowsLeft);
            }
        }
        for (const StripChunk &C : stripChunks) {
            stripEntries += C.nnz;
            stripBlocks += (double)C.blocks.size();
        }
        const int worth = tiles_worth(P->dtype, fragM, fragK, !inBlock.empty(), generalEntries, generalFrags, stripEntries, stripBlocks);
        if (worth == 0) {
            std::fill(sel.begin(), sel.end(), 0);
            stripChunks.clear();
            taken.clear();
            inBlock.clear();
            H.stripRows.clear();
        } else if (worth == 1) {
            std::fill(sel.begin(), sel.end(), 0);  // the strips pay, the general tiles do not
        }
    }
    // fragment of every A_dd entry: the rank of its column among the chunk's columns, / fragK.
    // The used prefix of a chunk's column list is ascending (the zero padding after it is
    // not), and so are the columns of a row of A_dd: one walk over both.
    std::vector<int> usedCols((size_t)chunkNum, 0);
#pragma omp parallel for schedule(static)
    for (int w = 0; w < chunkNum; ++w) {
        const int f0 = P->chunkPtr[w], f1 = P->chunkPtr[w + 1];
        const int *a = &P->sparse_AToX_index[(size_t)f0 * fragK];
        int n = (f1 - f0) * fragK;
        while (n > 1 && a[n - 1] == 0) --n;
        usedCols[w] = n;
    }
    // CSR part = residual rows + the A_dd entries whose fragment stays out of the tile kernel
    std::vector<int> &rowPtr = H.rowPtr;
    rowPtr.assign((size_t)rows + 1, 0);
    for (int r = 0; r < rows; ++r) rowPtr[r + 1] = P->cdRowPtr[r + 1] - P->cdRowPtr[r];
    std::vector<char> keep((size_t)P->ddRowPtr[P->dRows], 0);  // A_dd entry goes to the CSR part
    // (rows of A_dd come longest first: small dynamic pieces, not one static range per thread)
#pragma omp parallel for schedule(dynamic, 512)
    for (int i = 0; i < P->dRows; ++i) {
        const int w = i / fragM, f0 = P->chunkPtr[w];
        const int *a = &P->sparse_AToX_index[(size_t)f0 * fragK];
        const int na = usedCols[w];
        const bool rowTaken = !taken.empty() && taken[i];
        int n = 0, rank = 0;
        for (int p = P->ddRowPtr[i]; p < P->ddRowPtr[i + 1]; ++p) {
            const int c = P->ddColInd[p];
            while (rank < na && a[rank] < c) ++rank;
            // Of entries that name the same column twice the tile format holds the last
            // (generateFormat_opt overwrites, test/test_autotc_spmv.cpp:718-847); the
            // earlier ones go to the CSR part, so that y is the sum of all of them.
            const bool earlierTwin = p + 1 < P->ddRowPtr[i + 1] && P->ddColInd[p + 1] == c;
            keep[p] = rowTaken ? 0 : (!inBlock.empty() && inBlock[p]) ? 0 : (earlierTwin || !sel[f0 + rank / fragK]);
            n += keep[p];
        }
        rowPtr[P->rId[i] + 1] += n;
    }
    for (int r = 0; r < rows; ++r) rowPtr[r + 1] += rowPtr[r];
    const int csrNnz = rowPtr[rows];
    std::vector<int> &col = H.col;
    std::vector<unsigned char> &val = H.val;
    col.assign((size_t)csrNnz, 0);
    val.assign((size_t)csrNnz * es, 0);
    const unsigned char *cdv = (const unsigned char *)P->cdVal.data();
    const unsigned char *ddv = (const unsigned char *)P->ddVal.data();
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        int q = rowPtr[r];
        for (int p = P->cdRowPtr[r]; p < P->cdRowPtr[r + 1]; ++p, ++q) {
            col[q] = colOrig[P->cdColInd[p]];
            std::memcpy(&val[(size_t)q * es], cdv + (size_t)p * es, es);
        }
    }
#pragma omp parallel for schedule(dynamic, 512)
    for (int i = 0; i < P->dRows; ++i) {
        const int r = P->rId[i];
        int q = rowPtr[r] + (P->cdRowPtr[r + 1] - P->cdRowPtr[r]);
        for (int p = P->ddRowPtr[i]; p < P->ddRowPtr[i + 1]; ++p) {
            if (!keep[p]) continue;
            col[q] = P->descColId[P->ddColInd[p]];
            std::memcpy(&val[(size_t)q * es], ddv + (size_t)p * es, es);
            ++q;
        }
    }
    std::vector<char> &stripRows = H.stripRows;
    if (inBlock.empty()) stripRows.clear();
    if (!taken.empty()) {
        stripRows.assign((size_t)rows, 0);
        for (int i = 0; i < P->dRows; ++i)
            if (taken[i]) stripRows[P->rId[i]] = 1;
    }
    return MX_OK;
}

static int create_plan(const mx_partition *P, int flags, mx_plan **out, bool noBlocks);
static int create_plan_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev,
                              float tau_c, float tau_r, int flags, mx_plan **out, bool noBlocks, const mx::PartitionTwin *twin);
extern "C" int mx_plan_create(const mx_partition *P, int flags, mx_plan **out)
{
    // A partition that was made on the device still has its arrays there: the plan is made from them where they
    // are -- the same plan, array for array, as from the host arrays (MX_LAYOUT=host, MX_CSR_KERNEL=split and
    // MX_PLAN_AUTOTUNE=1 keep the host route, which brings the arrays down first).
    if (P && out && P->twin && P->extracted) {
        const char *lay = std::getenv("MX_LAYOUT"), *ker = std::getenv("MX_CSR_KERNEL");
        if (!(lay && !std::strcmp(lay, "host")) && !(ker && !std::strcmp(ker, "split")) && !plan_autotune())
            return create_plan_device(P->dtype, P->rows, P->cols, P->nnz, nullptr, nullptr, nullptr, P->tau_c, P->tau_r, flags, out, false,
                                      (const mx::PartitionTwin *)P->twin);
    }
    if (P) {
        const int rc = mx::partition_host(P);
        if (rc) return rc;
    }
    return create_plan(P, flags, out, false);
}

// `noBlocks`: a binary64 plan without the 8 x 8 block form (the second attempt, when a row of a block
// chunk turned out to have more virtual rows than the block layout has places for).
static int create_plan(const mx_partition *P, int flags, mx_plan **out, bool noBlocks)
{
    if (!P || !out) {
        set_error("mx_plan_create: null argument");
        return MX_ERR_ARG;
    }
    *out = nullptr;
    int rc = need_device();
    if (rc) return rc;
    mx_plan *plan = new (std::nothrow) mx_plan();
    if (!plan) {
        set_error("mx_plan_create: out of memory");
        return MX_ERR_ALLOC;
    }
    plan->dtype = P->dtype;
    plan->rows = P->rows;
    plan->cols = P->cols;
    plan->nnz = P->nnz;
    if (P->extracted) {
        plan->ext_dCols = P->dCols;
        plan->ext_dRows = P->dRows;
        plan->ext_nnzRowD = P->nnzRowD;
        plan->ext_frags = P->totalTcFrags;
    }
    auto fail = [&](int code) {
        mx_plan_destroy(plan);
        return code;
    };
    if (hipStreamCreate(&plan->stream) != hipSuccess || hipEventCreate(&plan->ev0) != hipSuccess ||
        hipEventCreate(&plan->ev1) != hipSuccess) {
        set_error("mx_plan_create: could not create stream/events");
        return fail(MX_ERR_DEVICE);
    }
    {
        // set-up: the address of the fixed array of mx_spmv_static on this device (kept per device)
        void *fixed = nullptr;
        if (mx::static_scratch(&fixed) != hipSuccess) {
            (void)hipGetLastError();
            set_error("mx_plan_create: hipGetSymbolAddress failed for the fixed array of sums");
            return fail(MX_ERR_DEVICE);
        }
    }
    PhaseLog phase;
    try {
        if (!P->extracted) {
            rc = setup_csr_part(plan, P->cdRowPtr.data(), P->cdColInd.data(), P->cdVal.data(), flags);
            if (rc) return fail(rc);
            phase("CSR part (layouts, trial)");
        } else {
            HostPlanParts H;
            rc = plan_host_parts(P, flags, H, phase, noBlocks);
            if (rc) return fail(rc);
            const int chunkNum = P->chunkNum;
            std::vector<char> &sel = H.sel, &taken = H.taken, &stripRows = H.stripRows;
            std::vector<StripChunk> &stripChunks = H.stripChunks;
            std::vector<int> &rowPtr = H.rowPtr, &col = H.col;
            std::vector<unsigned char> &val = H.val;
            phase("CSR part assembled");
            const bool blocks64 = P->dtype == MX_F64 && !stripChunks.empty();
            std::pair<std::vector<int>, std::vector<int>> seg;  // virtual rows of every row (slice form)
            rc = setup_csr_part(plan, rowPtr.data(), col.data(), val.data(), flags, stripRows.empty() ? nullptr : stripRows.data(),
                                blocks64 ? &seg : nullptr);
            if (rc) return fail(rc);
            phase("CSR part (layouts, trial)");

            // tile part: the selected chunks; columns and rows back in the caller's numbering
            const void *bits = P->dtype == MX_F64 ? (const void *)P->fragBit32.data() : (const void *)P->fragBit64.data();
            int nnzGeneral = 0, nnzStrips = 0;
            rc = upload_tiles(P->dtype, chunkNum, sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                              P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(),
                              plan->tiles, &nnzGeneral, taken.empty() ? nullptr : taken.data());
            if (rc) return fail(rc);
            if (!stripChunks.empty()) {
                std::vector<int> stepHdr;  // the layout's headers, for the places of the virtual-row sums
                rc = upload_tiles(P->dtype, chunkNum, sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                                  P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(),
                                  plan->strips, &nnzStrips, nullptr, &stripChunks, blocks64 ? &stepHdr : nullptr);
                if (rc) return fail(rc);
                if (!blocks64) {
                    // strip rows have nothing in the residual and left the fragments: the CSR part,
                    // which runs first, writes zeros there and the strip kernel may overwrite
                    plan->strips.ownedRows = true;
                } else if (plan->csr_variant == 1) {
                    // the blocks ride in the combine kernel's launch: where each of their rows finds the
                    // sums of its virtual rows (eight places per row; a row with more sends the whole plan
                    // back to be made without blocks)
                    const int steps = plan->strips.steps;
                    std::vector<int> vidx((size_t)steps * 128, -1);
                    bool fits = true;
                    for (int st = 0; st < steps && fits; ++st) {
                        const int *h = &stepHdr[(size_t)st * mx::kTileHdr];
                        if (!(h[16] & 1)) continue;
                        for (int half = 0; half < 2; ++half)
                            for (int i = 0; i < 8; ++i) {
                                const int r = h[half * 8 + i];
                                if (r < 0) continue;
                                const int a = seg.first[r], n = seg.first[r + 1] - a;
                                if (n > 8) fits = false;
                                for (int j = 0; j < std::min(n, 8); ++j) vidx[(size_t)st * 128 + half * 64 + i * 8 + j] = seg.second[a + j];
                            }
                    }
                    if (!fits) {
                        mx_plan_destroy(plan);
                        return create_plan(P, flags, out, true);
                    }
                    if ((rc = upload(&plan->strips.vidx, vidx.data(), vidx.size(), 128))) return fail(rc);
                }
            }
            plan->tile_nnz = nnzGeneral + nnzStrips;
            if (P->dtype == MX_F16 && plan->tiles.nWaves > 0) {
                rc = upload_bytes(&plan->ywide, nullptr, 0, (size_t)std::max(P->rows, 1) * sizeof(float));
                if (rc) return fail(rc);
            }
            phase("tile layouts");
        }
    } catch (const std::bad_alloc &) {
        set_error("mx_plan_create: out of memory");
        return fail(MX_ERR_ALLOC);
    }
    *out = plan;
    return MX_OK;
}

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
    const char *env = std::getenv("MX_CSR_KERNEL");
    if ((env && !std::strcmp(env, "split")) || plan_autotune()) {
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
    if (env && !std::strcmp(env, "rows")) want[0] = true, want[1] = false;
    if (env && !std::strcmp(env, "slices") && S > 0) want[1] = true, want[0] = false;
    if (want[1]) {
        rc = mx::build_slices_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, nCU, S, elsewhere_dev, plan->slices, nullptr,
                                     segOut ? &segOut->first : nullptr, segOut ? &segOut->second : nullptr);
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
        if (!elsewhere_dev && plan->slices.nHeavy == 0 && fused_wanted(flags, rows, -1, nCU)) plan->est_slices_us -= kFusedSavesUs;
        want[plan->est_slices_us < plan->est_rows_us ? 0 : 1] = false;
    }
    if (want[1]) {
        plan->csr_variant = 1;
        // The one-launch form where the host route would take it (no row with more than eight virtual rows: the
        // layout just made has no heavy rows).  Its layout is made on the host, from a copy of the part: the
        // matrices it is taken for are small (160 rows per workgroup at most, unless it is forced).
        bool wantFused = !elsewhere_dev && plan->slices.nHeavy == 0 && fused_wanted(flags, rows, -1, nCU);
        if (wantFused) {
            int ok = 0;
            MX_HIP(mx::fused_placement_ok(nCU, &ok));
            wantFused = ok != 0;
        }
        if (wantFused) {
            const size_t es = (size_t)mx::elem_size(dtype);
            std::vector<int> rp((size_t)rows + 1), ci((size_t)std::max(nnz, 1));
            std::vector<unsigned char> va(std::max<size_t>((size_t)nnz * es, 1));
            MX_HIP(hipMemcpy(rp.data(), rowPtr_dev, ((size_t)rows + 1) * 4, hipMemcpyDeviceToHost));
            if (nnz) MX_HIP(hipMemcpy(ci.data(), colInd_dev, (size_t)nnz * 4, hipMemcpyDeviceToHost));
            if (nnz) MX_HIP(hipMemcpy(va.data(), val_dev, (size_t)nnz * es, hipMemcpyDeviceToHost));
            mx::DeviceSlices L;
            rc = upload_slices(dtype, rows, cols, rp.data(), ci.data(), va.data(), nCU, S, nullptr, L, nullptr, segOut, true);
            if (rc) {
                free_slices(L);
                return rc;
            }
            if (L.fused) {
                free_slices(plan->slices);
                plan->slices = L;
                if (plan->slices.ecode) plan->slices.useDict = true;
                plan->fused = true;
            } else {
                free_slices(L);
            }
        }
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
    const char *envr = std::getenv("MX_CSR_REDUCE");
    if (envr && !std::strcmp(envr, "rows")) scan = false;
    if (envr && !std::strcmp(envr, "scan")) scan = true;
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
static int create_plan_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev,
                              float tau_c, float tau_r, int flags, mx_plan **out, bool noBlocks, const mx::PartitionTwin *twin = nullptr);
extern "C" int mx_plan_create_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev,
                                     const void *val_dev, float tau_c, float tau_r, int flags, mx_plan **out)
{
    return create_plan_device(dtype, rows, cols, nnz, rowPtr_dev, colInd_dev, val_dev, tau_c, tau_r, flags, out, false);
}

// `noBlocks`: a binary64 plan without the 8 x 8 block form (the second attempt, when a row of a block
// chunk turned out to have more virtual rows than the block layout has places for).
// `twin`: the extraction is there already, in the device arrays of a partition that was made on the
// device (mx_plan_create hands it in; the matrix arguments are not looked at then).
static int create_plan_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev,
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
        const char *envNoStrips = std::getenv("MX_NO_STRIPS"), *envNoBlocks = std::getenv("MX_NO_BLOCKS");
        const bool wantStrips = dtype == MX_F16 && !noTiles && !allTiles && !(envNoStrips && std::atoi(envNoStrips));
        const bool wantBlocks = dtype == MX_F64 && !noTiles && !allTiles && !noBlocks && !(envNoBlocks && std::atoi(envNoBlocks));
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
                                (double)cnt.stripEntries, (double)cnt.stripBlocks);
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
        *out = plan;
        return MX_OK;
    } catch (const std::bad_alloc &) {
        set_error(std::string(who) + ": out of memory");
        return fail(MX_ERR_ALLOC);
    }
}

// Every device array of a plan copied to host memory, with a name: for tests that hold the routes
// of making a plan against each other.
extern "C" void mx_plan_arrays_free(mx_plan_array *a, int n)
{
    if (!a) return;
    for (int i = 0; i < n; ++i) {
        free(a[i].data);
        a[i].data = nullptr;
    }
}
extern "C" int mx_plan_arrays(const mx_plan *plan, mx_plan_array *out, int cap, int *n)
{
    if (!plan || !out || !n || cap < 1) {
        set_error("mx_plan_arrays: bad argument");
        return MX_ERR_ARG;
    }
    *n = 0;
    const size_t es = (size_t)mx::elem_size(plan->dtype);
    int rc = MX_OK;
    auto add = [&](const char *name, const void *dev, size_t bytes) {
        if (rc || !dev) return;
        if (*n >= cap) {
            set_error("mx_plan_arrays: more arrays than the caller has room for");
            rc = MX_ERR_ARG;
            return;
        }
        void *p = malloc(std::max<size_t>(bytes, 1));
        if (!p || (bytes && hipMemcpy(p, dev, bytes, hipMemcpyDeviceToHost) != hipSuccess)) {
            free(p);
            set_error("mx_plan_arrays: out of memory or copy failed");
            rc = MX_ERR_ALLOC;
            return;
        }
        out[*n].name = name;
        out[*n].bytes = bytes;
        out[*n].data = p;
        ++*n;
    };
    if (plan->csr_variant != 1) {
        const mx::DeviceCsr &A = plan->csr;
        add("csr.rowPtr", A.rowPtr, ((size_t)A.rows + 1) * 4);
        add("csr.col", A.col, (size_t)A.nnz * 4);
        add("csr.col16", A.col16, (size_t)A.nnz * 2);
        add("csr.colBase", A.colBase, (size_t)A.nBlocks * 4);
        add("csr.val", A.val, (size_t)A.nnz * es);
        add("csr.blockDesc", A.blockDesc, (size_t)A.nBlocks * 16);
        add("csr.codes", A.codes, (size_t)A.nnz);
        add("csr.dict", A.dict, 256 * es);
    }
    if (plan->csr_variant != 0) {
        const mx::DeviceSlices &D = plan->slices;
        const size_t nEcol = ((size_t)D.steps + mx::kSlicePadSteps) * 64 * mx::slice_step_entries(plan->dtype);
        add("slices.wgDesc", D.wgDesc, ((size_t)D.nWG * 4 + 4) * 4);
        add("slices.waveDesc", D.waveDesc, ((size_t)D.nWG * mx::kSliceWaves * 4 + 4) * 4);
        add("slices.chunkEnd", D.chunkEnd, ((size_t)D.chunks + 64) * 4);
        add("slices.ecol", D.ecol, nEcol * 2);
        add("slices.eval", D.eval, nEcol * es);
        add("slices.ecode", D.ecode, nEcol);
        add("slices.dict", D.dict, 256 * es);
        add("slices.rowInfo", D.rowInfo, (((size_t)D.rows + 3) / 4 * 4 + 4) * 4);
        add("slices.segIdx", D.segIdx, ((size_t)D.vrows + 1) * 4);
        add("slices.lightRow", D.lightRow, (size_t)D.nLight * 4);
        add("slices.lightIdx", D.lightIdx, (size_t)D.nLight * 4 * D.lightQuads * 4);
        add("slices.heavyInfo", D.heavyInfo, ((size_t)D.nHeavy * 4 + 4) * 4);
        if (D.fused) {
            add("slices.wgGroups", D.wgGroups, ((size_t)D.nWG * 2 + 2) * 4);
            add("slices.groupNeed", D.groupNeed, ((size_t)D.nGroups + 1) * 4);
            add("slices.fusedTarget", D.fusedTarget, (size_t)D.chunks * 64 * 4);
            add("slices.rowVrows", D.rowVrows, (size_t)D.nGroups * mx::kFusedGroupRows);
        }
    }
    const mx::DeviceTiles *two[2] = {&plan->tiles, &plan->strips};
    static const char *const names[2][5] = {{"tiles.waveDesc", "tiles.hdr", "tiles.atox", "tiles.tcVal", "tiles.vidx"},
                                            {"strips.waveDesc", "strips.hdr", "strips.atox", "strips.tcVal", "strips.vidx"}};
    for (int t = 0; t < 2; ++t) {
        const mx::DeviceTiles &T = *two[t];
        if (T.nWaves <= 0) continue;
        add(names[t][0], T.waveDesc, (size_t)T.nWaves * 8 * 4);
        add(names[t][1], T.hdr, (size_t)T.steps * mx::kTileHdr * 4);
        add(names[t][2], T.atox, (size_t)T.steps * 64 * 4);
        add(names[t][3], T.tcVal, (size_t)T.stored * es);
        add(names[t][4], T.vidx, (size_t)T.steps * 128 * 4);
    }
    if (rc) {
        mx_plan_arrays_free(out, *n);
        *n = 0;
    }
    return rc;
}

extern "C" void mx_plan_layout_free(mx_plan_layout_view *v)
{
    if (!v) return;
    free(v->csrRowPtr);
    free(v->csrColInd);
    free(v->csrVal);
    free(v->stripRows);
    for (int t = 0; t < 2; ++t) {
        free(v->tiles[t].hdr);
        free(v->tiles[t].atox);
        free(v->tiles[t].waveDesc);
        free(v->tiles[t].valOffset);
        free(v->tiles[t].val);
    }
    std::memset(v, 0, sizeof(*v));
}

extern "C" int mx_plan_layout(const mx_partition *P, int flags, int nCU, mx_plan_layout_view *out)
{
    if (!P || !out || nCU < 1) {
        set_error("mx_plan_layout: bad argument");
        return MX_ERR_ARG;
    }
    std::memset(out, 0, sizeof(*out));
    if (int rc = mx::partition_host(P)) return rc;
    const int es = mx::elem_size(P->dtype);
    auto give = [](const auto *p, size_t n) {
        typedef typename std::remove_cv<typename std::remove_pointer<decltype(p)>::type>::type T;
        T *q = (T *)malloc(std::max<size_t>(n, 1) * sizeof(T));
        if (q && n) std::memcpy(q, p, n * sizeof(T));
        return q;
    };
    try {
        out->rows = P->rows;
        out->cols = P->cols;
        out->fragM = P->fragM;
        out->fragK = P->fragK;
        out->slots = mx::tile_slots(P->dtype);
        HostPlanParts H;
        HostTiles T[2];
        if (!P->extracted) {
            out->csr_nnz = P->cdRowPtr[P->rows];
            out->csrRowPtr = give(P->cdRowPtr.data(), (size_t)P->rows + 1);
            out->csrColInd = give(P->cdColInd.data(), (size_t)out->csr_nnz);
            out->csrVal = give((const unsigned char *)P->cdVal.data(), (size_t)out->csr_nnz * es);
        } else {
            PhaseLog quiet;
            quiet.on = false;
            int rc = plan_host_parts(P, flags, H, quiet);
            if (rc) return rc;
            out->csr_nnz = H.rowPtr[P->rows];
            out->csrRowPtr = give(H.rowPtr.data(), H.rowPtr.size());
            out->csrColInd = give(H.col.data(), H.col.size());
            out->csrVal = give(H.val.data(), H.val.size());
            const void *bits = P->dtype == MX_F64 ? (const void *)P->fragBit32.data() : (const void *)P->fragBit64.data();
            rc = build_tiles(P->dtype, P->chunkNum, H.sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                             P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(), nCU, T[0],
                             H.taken.empty() ? nullptr : H.taken.data());
            if (rc) return rc;
            if (!H.stripChunks.empty()) {
                rc = build_tiles(P->dtype, P->chunkNum, H.sel.data(), P->dRows, P->chunkPtr.data(), P->fragPtr.data(), bits,
                                 P->tcVal.data(), P->sparse_AToX_index.data(), P->descColId.data(), P->rId.data(), nCU, T[1],
                                 nullptr, &H.stripChunks);
                if (rc) return rc;
            }
        }
        {
            // the form of the CSR part a plan on a device with nCU compute units takes for it
            const int *rp = P->extracted ? H.rowPtr.data() : P->cdRowPtr.data();
            const int *ci = P->extracted ? H.col.data() : P->cdColInd.data();
            const void *va = P->extracted ? (const void *)H.val.data() : P->cdVal.data();
            const int S = slice_count(P->dtype, P->rows, P->cols, rp[P->rows], nCU);
            const CsrChoice pick = choose_csr_form(P->dtype, P->rows, P->cols, rp, ci, va, flags, nCU, S, H.stripRows.empty());
            out->csr_variant = pick.want[2] ? 2 : pick.want[0] && pick.want[1] ? -1 : pick.want[1] ? 1 : 0;
            out->est_rows_us = pick.usRows;
            out->est_slices_us = pick.usSlices;
        }
        std::vector<unsigned char> sr((size_t)P->rows, 0);
        if (!H.stripRows.empty()) std::memcpy(sr.data(), H.stripRows.data(), sr.size());
        out->stripRows = give(sr.data(), sr.size());
        bool ok = out->csrRowPtr && out->csrColInd && out->csrVal && out->stripRows;
        for (int t = 0; t < 2; ++t) {
            mx_tile_layout_view &V = out->tiles[t];
            V.steps = T[t].steps;
            V.nWaves = T[t].nWaves;
            V.chunks = T[t].chunkNum;
            V.nnz = T[t].vals;
            V.dense = T[t].dense ? 1 : 0;
            V.nVal = (long long)(T[t].val.size() / (size_t)es);
            V.hdr = give(T[t].hdr.data(), T[t].hdr.size());
            V.atox = give(T[t].atox.data(), T[t].atox.size());
            V.waveDesc = give(T[t].waveDesc.data(), T[t].waveDesc.size());
            V.valOffset = give(T[t].valOffset.data(), T[t].valOffset.size());
            V.val = give(T[t].val.data(), T[t].val.size());
            ok = ok && V.hdr && V.atox && V.waveDesc && V.valOffset && V.val;
        }
        if (!ok) {
            mx_plan_layout_free(out);
            set_error("mx_plan_layout: out of memory");
            return MX_ERR_ALLOC;
        }
    } catch (const std::bad_alloc &) {
        mx_plan_layout_free(out);
        set_error("mx_plan_layout: out of memory");
        return MX_ERR_ALLOC;
    }
    return MX_OK;
}

extern "C" int mx_plan_get_info(const mx_plan *plan, mx_plan_info *info)
{
    if (!plan || !info) {
        set_error("mx_plan_get_info: null argument");
        return MX_ERR_ARG;
    }
    const double es = mx::elem_size(plan->dtype);
    const int fragK = mx::frag_k(plan->dtype);
    const double bitBytes = plan->dtype == MX_F64 ? 4 : 8;
    info->dtype = plan->dtype;
    info->rows = plan->rows;
    info->cols = plan->cols;
    info->nnz = plan->nnz;
    info->tile_chunks = plan->tiles.chunkNum + plan->strips.chunkNum;
    info->tile_frags = plan->tiles.frags + plan->strips.frags;
    info->tile_nnz = plan->tile_nnz;
    info->csr_nnz = plan->csr_nnz;
    info->csr_blocks = plan->csr_variant == 1 ? plan->slices.nWG : plan->csr.nBlocks;
    info->csr_variant = plan->csr_variant;
    // what each kernel has to move at least once: its arrays, x once, its y rows
    info->csr_bytes = (double)plan->csr_nnz * (es + 4) + ((double)plan->rows + 1) * 4 + (double)plan->cols * es +
                      (double)plan->rows * es;
    // what the tile kernel reads and writes per launch: headers, column ids, values, x once per
    // column id, y once per row
    info->tile_bytes = 0.0;
    if (plan->tiles.steps)
        info->tile_bytes += (double)plan->tiles.steps * (mx::kTileHdr * 4.0 + 64 * 4.0) + (double)plan->tiles.stored * es +
                            (double)plan->tiles.frags * fragK * es + (double)plan->tiles.chunkNum * 8 * 2 * es;
    if (plan->strips.steps)  // no column ids, no old y
        info->tile_bytes += (double)plan->strips.steps * (mx::kTileHdr * 4.0) + (double)plan->strips.stored * es +
                            (double)plan->strips.frags * 8 * es + (double)plan->strips.chunkNum * 8 * es;
    (void)bitBytes;
    const bool sliceMain = plan->csr_variant == 1 || (plan->csr_variant == 2 && plan->slices.nnz > plan->csr.nnz);
    info->csr_main_kernel = sliceMain ? 1 : 0;
    info->csr_main_nnz = plan->csr_variant == 2 ? (sliceMain ? plan->slices.nnz : plan->csr.nnz) : plan->csr_nnz;
    info->tile_variant = plan->strips.steps > 0 ? (plan->dtype == MX_F64 ? 2 : 1) : 0;
    info->tile_strip_nnz = plan->strips.vals;
    info->csr_value_dict = plan->csr_variant == 1 ? (plan->slices.useDict ? plan->slices.nDict : 0)
                                                  : (plan->csr.useDict ? plan->csr.nDict : 0);
    info->est_rows_us = plan->est_rows_us;
    info->est_slices_us = plan->est_slices_us;
    info->prep_route = plan->prep_route;
    info->ext_dCols = plan->ext_dCols;
    info->ext_dRows = plan->ext_dRows;
    info->ext_nnzRowD = plan->ext_nnzRowD;
    info->ext_frags = plan->ext_frags;
    info->csr_fused = plan->csr_variant == 1 && plan->fused ? 1 : 0;
    return MX_OK;
}

// What a plan asks of x before anything is launched: 16-byte alignment where a kernel copies x in 16-byte
// vectors (the slice forms of the CSR part) or reads it in aligned 16-byte pieces with no other way to run
// (the binary64 8 x 8 blocks; the binary16 strips read at any alignment).
static int check_x(const mx_plan *plan, const void *x, const char *who)
{
    if (!((uintptr_t)x & 15)) return MX_OK;
    if (plan->csr_variant != 0) {
        set_error(std::string(who) + ": x must be 16-byte aligned for this plan (its CSR part keeps x in LDS)");
        return MX_ERR_ARG;
    }
    if (plan->dtype == MX_F64 && plan->strips.dense && plan->strips.nWaves > 0) {
        set_error(std::string(who) + ": x must be 16-byte aligned for this plan (its 8 x 8 blocks read x in aligned 16-byte pieces)");
        return MX_ERR_ARG;
    }
    return MX_OK;
}

static int spmv_on(mx_plan *plan, const void *x, void *y, hipStream_t s, void *partial = nullptr)
{
    if (int bad = check_x(plan, x, "mx_spmv")) return bad;
    // the strips ride in the launch of the combine kernel when the CSR part has one (MX_STRIPS_APART=1:
    // a launch of their own, as with the row-tile form of the CSR part)
    static const bool apart = std::getenv("MX_STRIPS_APART") && std::atoi(std::getenv("MX_STRIPS_APART"));
    const bool ride = plan->dtype == MX_F64 ? (plan->csr_variant == 1 && plan->strips.vidx != nullptr)
                                            : (!apart && plan->csr_variant == 1 && mx::strips_can_ride(plan->dtype, plan->strips, x));
    // (a binary16 row that gets sums from both parts: the CSR part leaves its sum in binary32 as
    // well and the tile kernel adds to that, so that y is rounded once, not twice)
    void *wide = plan->tiles.nWaves > 0 ? plan->ywide : nullptr;
    int rc = launch_csr_part(plan, x, y, 0, s, ride ? &plan->strips : nullptr, partial, wide);
    if (rc) return rc;
    MX_HIP(mx::launch_tiles(plan->dtype, plan->tiles, x, y, 1, s, wide));
    if (!ride) MX_HIP(mx::launch_tiles(plan->dtype, plan->strips, x, y, 1, s));
    return MX_OK;
}

extern "C" int mx_spmv(mx_plan *plan, const void *x_dev, void *y_dev, void *stream)
{
    if (!plan || !x_dev || !y_dev) {
        set_error("mx_spmv: null argument");
        return MX_ERR_ARG;
    }
    return spmv_on(plan, x_dev, y_dev, (hipStream_t)stream);
}

extern "C" int mx_spmv_static(mx_plan *plan, const void *x_dev, void *y_dev, void *stream)
{
    if (!plan || !x_dev || !y_dev) {
        set_error("mx_spmv_static: null argument");
        return MX_ERR_ARG;
    }
    const size_t need = partial_bytes(plan);
    if (need > mx::kStaticScratchBytes) {
        set_error("mx_spmv_static: the plan's virtual rows need " + std::to_string(need) +
                  " bytes of sums, the fixed array holds " + std::to_string(mx::kStaticScratchBytes) +
                  " (use mx_spmv, which keeps them in the plan's own buffer)");
        return MX_ERR_ARG;
    }
    void *fixed = nullptr;
    MX_HIP(mx::static_scratch(&fixed));  // the address on the current device; looked up once per device
    return spmv_on(plan, x_dev, y_dev, (hipStream_t)stream, need ? fixed : nullptr);
}

extern "C" int mx_static_scratch_bytes(void) { return (int)mx::kStaticScratchBytes; }

extern "C" int mx_spmv_repeat(mx_plan *plan, const void *x_dev, void *y_dev, int n, void *stream)
{
    if (!plan || !x_dev || !y_dev || n < 0) {
        set_error("mx_spmv_repeat: bad argument");
        return MX_ERR_ARG;
    }
    for (int i = 0; i < n; ++i) {
        int rc = spmv_on(plan, x_dev, y_dev, (hipStream_t)stream);
        if (rc) return rc;
    }
    return MX_OK;
}

extern "C" int mx_spmv_host(mx_plan *plan, const void *x_host, void *y_host)
{
    if (!plan || !x_host || !y_host) {
        set_error("mx_spmv_host: null argument");
        return MX_ERR_ARG;
    }
    const size_t es = (size_t)mx::elem_size(plan->dtype);
    void *dx = nullptr, *dy = nullptr;
    MX_HIP(hipMalloc(&dx, std::max<size_t>(plan->cols * es, 1)));
    if (hipMalloc(&dy, std::max<size_t>(plan->rows * es, 1)) != hipSuccess) {
        (void)hipFree(dx);
        set_error("mx_spmv_host: hipMalloc failed");
        return MX_ERR_DEVICE;
    }
    int rc = MX_OK;
    auto body = [&]() -> int {
        MX_HIP(hipMemcpyAsync(dx, x_host, plan->cols * es, hipMemcpyHostToDevice, plan->stream));
        int r = spmv_on(plan, dx, dy, plan->stream);
        if (r) return r;
        MX_HIP(hipMemcpyAsync(y_host, dy, plan->rows * es, hipMemcpyDeviceToHost, plan->stream));
        MX_HIP(hipStreamSynchronize(plan->stream));
        return MX_OK;
    };
    rc = body();
    (void)hipFree(dx);
    (void)hipFree(dy);
    return rc;
}

extern "C" int mx_time_csr_main(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters, double *ms)
{
    if (!plan || !x_dev || !y_dev || warm < 0 || iters <= 0 || !ms) {
        set_error("mx_time_csr_main: bad argument");
        return MX_ERR_ARG;
    }
    hipStream_t s = plan->stream;
    if (int bad = check_x(plan, x_dev, "mx_time_csr_main")) return bad;
    int rc = time_loop(plan, warm, iters, [&]() -> int {
        // the kernel that holds most of the entries
        if (plan->csr_variant == 1 && plan->fused)
            return launch_csr_part(plan, x_dev, y_dev, 0, s);
        if (plan->csr_variant == 1 || (plan->csr_variant == 2 && plan->slices.nnz > plan->csr.nnz))
            MX_HIP(mx::launch_slices(plan->dtype, plan->slices, x_dev, y_dev, 0, s, 1));
        else
            MX_HIP(mx::launch_csr(plan->dtype, plan->csr, x_dev, y_dev, 0, s));
        return MX_OK;
    }, ms);
    if (rc) return rc;
    rc = spmv_on(plan, x_dev, y_dev, s);  // leave y holding the product
    if (rc) return rc;
    MX_HIP(hipStreamSynchronize(s));
    return MX_OK;
}

extern "C" int mx_time(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters, double *ms_total,
                       double *ms_tile, double *ms_csr)
{
    if (!plan || !x_dev || !y_dev || warm < 0 || iters <= 0) {
        set_error("mx_time: bad argument");
        return MX_ERR_ARG;
    }
    hipStream_t s = plan->stream;
    int rc;
    double t = 0.0;
    if ((rc = check_x(plan, x_dev, "mx_time"))) return rc;
    if (ms_total) {
        rc = time_loop(plan, warm, iters, [&]() { return spmv_on(plan, x_dev, y_dev, s); }, &t);
        if (rc) return rc;
        *ms_total = t;
    }
    // The reference adds up two numbers, tile part and residual part, each timed alone
    // (test/test_autotc_spmv.cpp:1561-1572).  A plan whose strips or blocks ride in the combine kernel's
    // launch has no tile kernel of its own: ms_csr is then the CSR part as the product runs it, riders
    // included, and ms_tile what they add to that launch (the same launches without them taken off).
    static const bool apart = std::getenv("MX_STRIPS_APART") && std::atoi(std::getenv("MX_STRIPS_APART"));
    const bool ride = plan->dtype == MX_F64 ? (plan->csr_variant == 1 && plan->strips.vidx != nullptr)
                                            : (!apart && plan->csr_variant == 1 && mx::strips_can_ride(plan->dtype, plan->strips, x_dev));
    void *wide = plan->tiles.nWaves > 0 ? plan->ywide : nullptr;
    const bool blocksApart = !ride && plan->dtype == MX_F64 && plan->strips.nWaves > 0;  // binary64 blocks in a launch of their own
    double tBare = 0.0;
    if (ms_csr || (ms_tile && (ride || blocksApart))) {
        rc = time_loop(plan, warm, iters, [&]() { return launch_csr_part(plan, x_dev, y_dev, 0, s, ride ? &plan->strips : nullptr, nullptr, wide); }, &t);
        if (rc) return rc;
        if (ms_csr) *ms_csr = t;
        if (ms_tile && ride) {
            // (the rows of riders are left alone by the bare launch: nothing is added to them, y stays bounded)
            rc = time_loop(plan, warm, iters, [&]() { return launch_csr_part(plan, x_dev, y_dev, 0, s, nullptr, nullptr, wide); }, &tBare);
            if (rc) return rc;
        }
    }
    if (ms_tile) {
        *ms_tile = ride ? std::max(0.0, t - tBare) : 0.0;
        if (plan->tiles.chunkNum > 0 || (!ride && !blocksApart && plan->strips.chunkNum > 0)) {
            // overwrite mode: the timed loop must not grow y without bound
            double tt = 0.0;
            rc = time_loop(plan, warm, iters, [&]() -> int {
                MX_HIP(mx::launch_tiles(plan->dtype, plan->tiles, x_dev, y_dev, 0, s));
                if (!ride && !blocksApart) MX_HIP(mx::launch_tiles(plan->dtype, plan->strips, x_dev, y_dev, 0, s));
                return MX_OK;
            }, &tt);
            if (rc) return rc;
            *ms_tile += tt;
        }
        if (blocksApart) {
            // the block kernel adds to y, so it is priced as the pair (CSR part, blocks) less the CSR part: the
            // CSR part rewrites y before every launch of the blocks
            double pair = 0.0;
            rc = time_loop(plan, warm, iters, [&]() -> int {
                int r = launch_csr_part(plan, x_dev, y_dev, 0, s, nullptr, nullptr, wide);
                if (r) return r;
                MX_HIP(mx::launch_tiles(plan->dtype, plan->strips, x_dev, y_dev, 1, s));
                return MX_OK;
            }, &pair);
            if (rc) return rc;
            *ms_tile += std::max(0.0, pair - t);
        }
    }
    // leave y holding the product
    rc = spmv_on(plan, x_dev, y_dev, s);
    if (rc) return rc;
    MX_HIP(hipStreamSynchronize(s));
    return MX_OK;
}

extern "C" int mx_time_rotate(mx_plan *const *plans, const void *const *x_dev, void *const *y_dev, int n, int warm, int iters, double *ms)
{
    if (!plans || !x_dev || !y_dev || n < 1 || warm < 0 || iters <= 0 || !ms) {
        set_error("mx_time_rotate: bad argument");
        return MX_ERR_ARG;
    }
    for (int i = 0; i < n; ++i)
        if (!plans[i] || !x_dev[i] || !y_dev[i]) {
            set_error("mx_time_rotate: null plan or vector");
            return MX_ERR_ARG;
        }
    mx_plan *first = plans[0];
    hipStream_t s = first->stream;
    int turn = 0;
    return time_loop(first, warm, iters, [&]() -> int {
        const int i = turn;
        turn = (turn + 1) % n;
        return spmv_on(plans[i], x_dev[i], y_dev[i], s);
    }, ms);
}

// One record per kernel launch of a product, in launch order: its mean time alone (same protocol as
// mx_time) and its share of the algorithmic bytes -- entries at sizeof(valT) + 4 each go to the
// kernel that multiplies them, x to the first kernel that reads it, the row structure
// ((rows + 1) * 4) and y to the kernel that writes y -- so that the shares add up to
// mx_algorithmic_bytes of the whole matrix.
extern "C" int mx_time_kernels(mx_plan *plan, const void *x_dev, void *y_dev, int warm, int iters, mx_kernel_time *out,
                               int cap, int *n_kernels)
{
    if (!plan || !x_dev || !y_dev || warm < 0 || iters <= 0 || !out || cap < 1 || !n_kernels) {
        set_error("mx_time_kernels: bad argument");
        return MX_ERR_ARG;
    }
    hipStream_t s = plan->stream;
    const double es = mx::elem_size(plan->dtype);
    const char *vt = plan->dtype == MX_F64 ? "f64" : "f16";
    const double xBytes = (double)plan->cols * es, yBytes = ((double)plan->rows + 1) * 4 + (double)plan->rows * es;
    static const bool apart = std::getenv("MX_STRIPS_APART") && std::atoi(std::getenv("MX_STRIPS_APART"));
    const bool ride = plan->dtype == MX_F64 ? (plan->csr_variant == 1 && plan->strips.vidx != nullptr)
                                            : (!apart && plan->csr_variant == 1 && mx::strips_can_ride(plan->dtype, plan->strips, x_dev));
    void *wide = plan->tiles.nWaves > 0 ? plan->ywide : nullptr;
    int n = 0, rc = MX_OK;
    auto add = [&](const std::string &name, double bytes, int nnz, auto body) {
        if (rc || n >= cap) return;
        mx_kernel_time &K = out[n];
        std::memset(&K, 0, sizeof(K));
        std::snprintf(K.name, sizeof(K.name), "%s", name.c_str());
        K.algorithmic_bytes = bytes;
        K.nnz = nnz;
        rc = time_loop(plan, warm, iters, body, &K.ms);
        ++n;
    };
    if ((rc = check_x(plan, x_dev, "mx_time_kernels"))) return rc;
    bool xCounted = false;
    if (plan->csr_variant != 1 && plan->csr.nBlocks > 0) {
        const bool last = plan->csr_variant == 0;  // writes y for good
        add(std::string("csr_rows_kernel<") + vt + (plan->csr.useDict ? ",dict>" : ">"),
            (double)plan->csr.nnz * (es + 4) + xBytes + (last ? yBytes : 0.0), plan->csr.nnz, [&]() -> int {
                MX_HIP(mx::launch_csr(plan->dtype, plan->csr, x_dev, y_dev, 0, s, wide));
                return MX_OK;
            });
        xCounted = true;
    }
    if (plan->csr_variant == 1 && plan->fused && !ride) {
        // the one-launch form: one kernel multiplies, adds up and writes y
        add(std::string("csr_slice_kernel<") + vt + (plan->slices.useDict ? ",dict,fused>" : ",fused>"),
            (double)plan->slices.nnz * (es + 4) + xBytes + yBytes, plan->slices.nnz,
            [&]() -> int { return launch_csr_part(plan, x_dev, y_dev, 0, s, nullptr, nullptr, wide); });
    } else if (plan->csr_variant != 0) {
        add(std::string("csr_slice_kernel<") + vt + (plan->slices.useDict ? ",dict>" : ">"),
            (double)plan->slices.nnz * (es + 4) + (xCounted ? 0.0 : xBytes), plan->slices.nnz, [&]() -> int {
                MX_HIP(mx::launch_slices(plan->dtype, plan->slices, x_dev, y_dev, 0, s, 1));
                return MX_OK;
            });
        const int stripNnz = ride ? plan->strips.vals : 0;
        add(std::string("slice_combine_kernel<") + vt + (!ride ? ">" : plan->dtype == MX_F64 ? ",blocks>" : ",strips>"),
            (double)stripNnz * (es + 4) + yBytes, stripNnz,
            [&]() -> int {
                MX_HIP(mx::launch_slices(plan->dtype, plan->slices, x_dev, y_dev, 0, s, 2, ride ? &plan->strips : nullptr, wide));
                return MX_OK;
            });
    }
    if (plan->tiles.nWaves > 0)
        add(std::string("tile_kernel<") + vt + ">", (double)plan->tiles.vals * (es + 4), plan->tiles.vals, [&]() -> int {
            MX_HIP(mx::launch_tiles(plan->dtype, plan->tiles, x_dev, y_dev, 1, s, wide));
            return MX_OK;
        });
    if (!ride && plan->strips.nWaves > 0)
        add(plan->dtype == MX_F64 ? "tile_block_kernel<f64>" : "tile_dense_kernel<f16>", (double)plan->strips.vals * (es + 4),
            plan->strips.vals, [&]() -> int {
            MX_HIP(mx::launch_tiles(plan->dtype, plan->strips, x_dev, y_dev, 1, s));
            return MX_OK;
        });
    if (rc) return rc;
    *n_kernels = n;
    rc = spmv_on(plan, x_dev, y_dev, s);  // leave y holding the product
    if (rc) return rc;
    MX_HIP(hipStreamSynchronize(s));
    return MX_OK;
}

extern "C" int mx_tune_tau(const mx_csr *A, int levels, int flags, int warm, int iters, float *tau_c, float *tau_r,
                           mx_tau_point *table, int cap, int *n_points)
{
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
    const char *envNoStrips = std::getenv("MX_NO_STRIPS"), *envNoBlocks = std::getenv("MX_NO_BLOCKS");
    const bool wantStrips = A->dtype == MX_F16 && !(envNoStrips && std::atoi(envNoStrips));
    const bool wantBlocks = A->dtype == MX_F64 && !(envNoBlocks && std::atoi(envNoBlocks));
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
                                                  (double)cnt.stripEntries, (double)cnt.stripBlocks, &netNs);
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

// ---- reference surface: host pointers in, host pointers out ------------------------------

static int cdspmv_any(mx_dtype dtype, const void *csrVal, const int *csrRowPtr, const int *csrColInd, const void *x,
                      void *y, int rows, int cols, int nnz, int warm, int iters, double *cdTime, double *cdPre)
{
    if (!csrRowPtr || !x || !y || rows < 0 || cols < 0 || nnz < 0 || (nnz > 0 && (!csrVal || !csrColInd))) {
        set_error("cdspmv: bad argument");
        return MX_ERR_ARG;
    }
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
