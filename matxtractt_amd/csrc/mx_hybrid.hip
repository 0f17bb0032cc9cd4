// The host half of a hybrid plan (plan_host_parts in mx_plan.cpp) done on the device, for a
// matrix that lives in device memory: the extraction (mx_select_device, mx_split_device,
// mx_tiles_device), the fill gate of the fragments, the search for rows of dense binary16 strips
// and their grouping into chunks, the counts the plan's decision needs, the CSR part in the
// caller's numbering and the strips' step layout -- the same arrays, byte for byte, as the host
// route makes from the same matrix.  Only what is counted per strip chunk or per step crosses to
// the host (a few bytes each), never an entry of the matrix.  The reference does all of this on
// the host (test/test_autotc_spmv.cpp:1099-1421).
//
// The general tile form is laid out here as well (tile_chunks, tile_layout), and so is the binary64
// block form (block_chunks, block_layout): no form of the tile part sends a matrix to the host.
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

namespace mxh {

constexpr int kBlock = 256;
inline dim3 grid(long long n) { return dim3((unsigned)((std::max<long long>(n, 1) + kBlock - 1) / kBlock)); }

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

// sum over the grid of one count per lane (every lane of a wave must arrive here)
__device__ __forceinline__ void add_total(unsigned long long v, unsigned long long *dst)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    if ((threadIdx.x & 63) == 0 && v) atomicAdd(dst, v);
}

__global__ __launch_bounds__(kBlock) void mark_kernel(const int *__restrict__ list, int n, unsigned char *__restrict__ flag)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < n) flag[list[k]] = 1;
}
__global__ __launch_bounds__(kBlock) void unmarked_kernel(const unsigned char *__restrict__ flag, int n, int *__restrict__ out)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < n) out[k] = flag[k] ? 0 : 1;
}
// the caller's column of every column of the residual's numbering: the selected columns by rank,
// then the others in ascending order
__global__ __launch_bounds__(kBlock) void col_orig_kernel(const int *__restrict__ descColId, const unsigned char *__restrict__ flag,
                                                          const int *__restrict__ pos, int cols, int dCols, int *__restrict__ colOrig)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c >= cols) return;
    if (c < dCols) colOrig[c] = descColId[c];
    if (!flag[c]) colOrig[dCols + pos[c]] = c;
}
__global__ __launch_bounds__(kBlock) void dd_row_of_kernel(const int *__restrict__ rId, int dRows, int *__restrict__ ddRowOf)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < dRows) ddRowOf[rId[i]] = i;
}
__global__ __launch_bounds__(kBlock) void iota_kernel(int *__restrict__ v, int n)
{
    const int k = blockIdx.x * kBlock + threadIdx.x;
    if (k < n) v[k] = k;
}

// The blocks of eight consecutive columns (caller's numbering) that row i of A_dd touches: the first
// column of each, ascending.  The blocks start at multiples of eight, or, where that takes fewer
// blocks, at the row's own lowest column plus multiples of eight.  false when the row does not qualify
// as a row of a strip chunk: fewer than 4 or more than 64 entries, something in the residual, a column
// named twice, a block that would reach past the end of x, more than eight blocks, or blocks less than
// half full.
struct RowBlocks {
    int nb;
    int b[8];
};
// (0 = fine, 1 = too many blocks or one past the end of x, 2 = a column named twice)
__device__ int row_blocks_at(const int *__restrict__ ddCol, const int *__restrict__ descColId, int p0, int n, int cols, int shift,
                             RowBlocks &R)
{
    R.nb = 0;
    unsigned m[8];
    for (int k = 0; k < n; ++k) {
        const int c = descColId[ddCol[p0 + k]];
        const int first = ((c - shift) >> 3) * 8 + shift;
        const unsigned bit = 1u << (c - first);
        if (first + 8 > cols) return 1;
        int j = 0;
        while (j < R.nb && R.b[j] < first) ++j;
        if (j < R.nb && R.b[j] == first) {
            if (m[j] & bit) return 2;
            m[j] |= bit;
        } else {
            if (R.nb == 8) return 1;
            for (int t = R.nb; t > j; --t) {
                R.b[t] = R.b[t - 1];
                m[t] = m[t - 1];
            }
            R.b[j] = first;
            m[j] = bit;
            ++R.nb;
        }
    }
    return 0;
}
__device__ bool row_blocks(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol, const int *__restrict__ descColId,
                           const int *__restrict__ rId, const int *__restrict__ cdRowPtr, int i, int cols, RowBlocks &R)
{
    const int p0 = ddRowPtr[i], n = ddRowPtr[i + 1] - p0, r = rId[i];
    R.nb = 0;
    if (n < 4 || n > 64 || cdRowPtr[r + 1] != cdRowPtr[r]) return false;
    const int on = row_blocks_at(ddCol, descColId, p0, n, cols, 0, R);
    if (on == 2) return false;
    int lowest = descColId[ddCol[p0]];
    for (int k = 1; k < n; ++k) lowest = min(lowest, descColId[ddCol[p0 + k]]);
    const int shift = lowest & 7;
    bool ok = on == 0;
    if (shift) {
        RowBlocks own;
        if (row_blocks_at(ddCol, descColId, p0, n, cols, shift, own) == 0 && (!ok || own.nb < R.nb)) {
            R = own;
            ok = true;
        }
    }
    return ok && 2 * n >= R.nb * 8;
}

__global__ __launch_bounds__(kBlock) void strip_candidates_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                                  const int *__restrict__ descColId, const int *__restrict__ rId,
                                                                  const int *__restrict__ cdRowPtr, int dRows, int cols,
                                                                  int *__restrict__ isCand)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= dRows) return;
    RowBlocks R;
    isCand[i] = row_blocks(ddRowPtr, ddCol, descColId, rId, cdRowPtr, i, cols, R) ? 1 : 0;
}
// candidates in row order: their row of A_dd, the first columns of their blocks (-1 = none) and how many
__global__ __launch_bounds__(kBlock) void candidate_keys_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                                const int *__restrict__ descColId, const int *__restrict__ rId,
                                                                const int *__restrict__ cdRowPtr, const int *__restrict__ isCand,
                                                                const int *__restrict__ candPos, int dRows, int cols,
                                                                int *__restrict__ candRow, int *__restrict__ candKey,
                                                                int *__restrict__ candNb)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= dRows || !isCand[i]) return;
    RowBlocks R;
    (void)row_blocks(ddRowPtr, ddCol, descColId, rId, cdRowPtr, i, cols, R);
    const int j = candPos[i];
    candRow[j] = i;
    candNb[j] = R.nb;
    for (int k = 0; k < 8; ++k) candKey[(size_t)j * 8 + k] = k < R.nb ? R.b[k] : -1;
}
// the k-th block of every candidate in the current order, as an unsigned sort key (none = 0)
__global__ __launch_bounds__(kBlock) void pass_keys_kernel(const int *__restrict__ candKey, const int *__restrict__ perm, int n, int k,
                                                           unsigned *__restrict__ key)
{
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j < n) key[j] = (unsigned)(candKey[(size_t)perm[j] * 8 + k] + 1);
}
__global__ __launch_bounds__(kBlock) void run_heads_kernel(const int *__restrict__ candKey, const int *__restrict__ perm, int n,
                                                           int *__restrict__ head)
{
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j >= n) return;
    bool h = j == 0;
    if (!h) {
        const int *a = candKey + (size_t)perm[j] * 8, *b = candKey + (size_t)perm[j - 1] * 8;
        for (int k = 0; k < 8; ++k) h = h || a[k] != b[k];
    }
    head[j] = h ? 1 : 0;
}
__global__ __launch_bounds__(kBlock) void run_starts_kernel(const int *__restrict__ head, const int *__restrict__ runIdIncl, int n,
                                                            int *__restrict__ runStart)
{
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j >= n) return;
    if (head[j]) runStart[runIdIncl[j] - 1] = j;
    if (j == n - 1) runStart[runIdIncl[j]] = n;
}
// chunks of a run of candidates with the same blocks: eight rows each, a last one of at least four
__global__ __launch_bounds__(kBlock) void run_chunks_kernel(const int *__restrict__ runStart, int nRuns, int *__restrict__ runChunks)
{
    const int u = blockIdx.x * kBlock + threadIdx.x;
    if (u >= nRuns) return;
    const int len = runStart[u + 1] - runStart[u];
    runChunks[u] = len / 8 + ((len % 8) >= 4 ? 1 : 0);
}
__global__ __launch_bounds__(kBlock) void chunk_members_kernel(const int *__restrict__ perm, const int *__restrict__ candRow,
                                                               const int *__restrict__ candKey, const int *__restrict__ candNb,
                                                               const int *__restrict__ runIdIncl, const int *__restrict__ runStart,
                                                               const int *__restrict__ runChunks, const int *__restrict__ runChunk0,
                                                               const int *__restrict__ ddRowPtr, const int *__restrict__ rId, int n,
                                                               unsigned char *__restrict__ taken, int *__restrict__ memberChunk,
                                                               int *__restrict__ chunkRows, int *__restrict__ chunkKey,
                                                               int *__restrict__ chunkNb, int *__restrict__ chunkNnz)
{
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j >= n) return;
    const int u = runIdIncl[j] - 1, pos = j - runStart[u], q = pos >> 3;
    if (q >= runChunks[u]) {
        memberChunk[j] = -1;
        return;
    }
    const int chunk = runChunk0[u] + q, jj = pos & 7, cand = perm[j], i = candRow[cand];
    memberChunk[j] = chunk;
    taken[i] = 1;
    chunkRows[(size_t)chunk * 8 + jj] = rId[i];
    if (jj == 0) {
        chunkNb[chunk] = candNb[cand];
        for (int k = 0; k < 8; ++k) chunkKey[(size_t)chunk * 8 + k] = candKey[(size_t)cand * 8 + k];
        const int nr = min(runStart[u + 1] - j, 8);
        int e = 0;
        for (int t = 0; t < nr; ++t) {
            const int it = candRow[perm[j + t]];
            e += ddRowPtr[it + 1] - ddRowPtr[it];
        }
        chunkNnz[chunk] = e;
    }
}

// The fill gate on what the taken rows leave of every fragment (binary16: one thread per chunk of
// the reference's numbering): fragments and entries that pass, summed.
__global__ __launch_bounds__(kBlock) void gate_f16_kernel(const int *__restrict__ chunkPtr, const unsigned long long *__restrict__ fragBit,
                                                          const unsigned char *__restrict__ taken, int chunkNum, int dRows, int minVals,
                                                          unsigned long long *__restrict__ totals)
{
    const int w = blockIdx.x * kBlock + threadIdx.x;
    unsigned long long frags = 0, entries = 0;
    if (w < chunkNum) {
        unsigned long long rowsLeft = 0;
        for (int r = 0; r < 8; ++r) {
            const int i = w * 8 + r;
            if (i < dRows && !(taken && taken[i])) rowsLeft |= 0xffull << (r * 8);
        }
        for (int f = chunkPtr[w]; f < chunkPtr[w + 1]; ++f) {
            const int vals = __popcll(fragBit[f] & rowsLeft);
            if (vals > 0 && vals >= minVals) {
                ++frags;
                entries += (unsigned)vals;
            }
        }
    }
    add_total(frags, totals);
    add_total(entries, totals + 1);
}
__global__ __launch_bounds__(kBlock) void gate_counts_kernel(const int *__restrict__ fragPtr, int nFrags, int minVals,
                                                             unsigned long long *__restrict__ totals)
{
    const int f = blockIdx.x * kBlock + threadIdx.x;
    unsigned long long frags = 0, entries = 0;
    if (f < nFrags) {
        const int vals = fragPtr[f + 1] - fragPtr[f];
        if (vals > 0 && vals >= minVals) {
            frags = 1;
            entries = (unsigned)vals;
        }
    }
    add_total(frags, totals);
    add_total(entries, totals + 1);
}

// binary64: (block row, block column) of every entry of A_dd that is not followed by a twin
__global__ __launch_bounds__(kBlock) void block_keys_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                            const int *__restrict__ descColId, const int *__restrict__ rId, int dRows,
                                                            int nDD, unsigned long long *__restrict__ key)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= nDD) return;
    int lo = 0, hi = dRows - 1;
    while (lo < hi) {  // last i with ddRowPtr[i] <= p
        const int mid = (lo + hi + 1) >> 1;
        if (ddRowPtr[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    const bool twin = p + 1 < ddRowPtr[lo + 1] && ddCol[p + 1] == ddCol[p];
    key[p] = twin ? ~0ull : ((unsigned long long)(unsigned)(rId[lo] >> 3) << 32) | (unsigned)(descColId[ddCol[p]] >> 3);
}
// runs of one key at least `need` long whose block lies inside x: blocks and entries, summed
__global__ __launch_bounds__(kBlock) void block_runs_kernel(const unsigned long long *__restrict__ key, int n, int need, int cols,
                                                            unsigned long long *__restrict__ totals)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    unsigned long long blocks = 0, entries = 0;
    if (p < n && key[p] != ~0ull && (p == 0 || key[p - 1] != key[p])) {
        int e = p + 1;
        while (e < n && e - p < 64 && key[e] == key[p]) ++e;  // (a block holds at most 64 entries that are not twins)
        const int bc = (int)(unsigned)key[p];
        if (e - p >= need && bc + 1 <= cols / 8) {
            blocks = 1;
            entries = (unsigned)(e - p);
        }
    }
    add_total(blocks, totals);
    add_total(entries, totals + 1);
}

// ---- the CSR part: every row's residual entries, then the entries of A_dd that stay
__global__ __launch_bounds__(kBlock) void part_lengths_kernel(const int *__restrict__ cdRowPtr, const int *__restrict__ ddRowPtr,
                                                              const int *__restrict__ ddRowOf, const unsigned char *__restrict__ taken,
                                                              int rows, int *__restrict__ len, char *__restrict__ stripRows)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r > rows) return;
    if (r == rows) {
        len[r] = 0;
        return;
    }
    int n = cdRowPtr[r + 1] - cdRowPtr[r];
    const int i = ddRowOf[r];
    const bool gone = i >= 0 && taken && taken[i];
    if (i >= 0 && !gone) n += ddRowPtr[i + 1] - ddRowPtr[i];
    len[r] = n;
    if (stripRows) stripRows[r] = gone ? 1 : 0;
}
template <typename V>
__global__ __launch_bounds__(kBlock) void part_residual_kernel(const int *__restrict__ cdRowPtr, const int *__restrict__ cdCol,
                                                               const V *__restrict__ cdVal, const int *__restrict__ colOrig,
                                                               const int *__restrict__ outPtr, int rows, int nCD, int *__restrict__ col,
                                                               V *__restrict__ val)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= nCD) return;
    int lo = 0, hi = rows - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (cdRowPtr[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    const int q = outPtr[lo] + (p - cdRowPtr[lo]);
    col[q] = colOrig[cdCol[p]];
    val[q] = cdVal[p];
}
template <typename V>
__global__ __launch_bounds__(kBlock) void part_dense_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                            const V *__restrict__ ddVal, const int *__restrict__ descColId,
                                                            const int *__restrict__ rId, const unsigned char *__restrict__ taken,
                                                            const int *__restrict__ cdRowPtr, const int *__restrict__ outPtr, int dRows,
                                                            int nDD, int *__restrict__ col, V *__restrict__ val)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= nDD) return;
    int lo = 0, hi = dRows - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (ddRowPtr[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    if (taken && taken[lo]) return;
    const int r = rId[lo];
    const int q = outPtr[r] + (cdRowPtr[r + 1] - cdRowPtr[r]) + (p - ddRowPtr[lo]);
    col[q] = descColId[ddCol[p]];
    val[q] = ddVal[p];
}

// ---- the strips' steps.  stepDesc[s] = {chunk of half 0, chunk of half 1 (-1 none, -2 the same chunk
// goes on), flags, blocks in half 0, blocks in half 1, first value, first value and blocks in half 0
// of the step four further on}; one wave per step writes its header and column ids.
__global__ __launch_bounds__(64) void strip_steps_kernel(const int *__restrict__ stepDesc, const int *__restrict__ chunkRows,
                                                         const int *__restrict__ chunkKey, int steps, int *__restrict__ hdr,
                                                         int *__restrict__ atox)
{
    const int s = blockIdx.x, l = threadIdx.x;
    if (s >= steps) return;
    const int *d = stepDesc + (size_t)s * 8;
    const int A = d[0], B = d[1], n0 = d[3], n1 = d[4];
    auto first_col = [&](int slot) {  // first column of the block in a slot, -1 = none
        const int half = slot >> 2, i = slot & 3;
        if (half == 0) return i < n0 ? chunkKey[(size_t)A * 8 + i] : -1;
        if (i >= n1) return -1;
        return B >= 0 ? chunkKey[(size_t)B * 8 + i] : chunkKey[(size_t)A * 8 + 4 + i];
    };
    if (l < mx::kTileHdr) {
        int v = 0;
        if (l < 8) v = chunkRows[(size_t)A * 8 + l];
        else if (l < 16) v = B >= 0 ? chunkRows[(size_t)B * 8 + (l - 8)] : -1;
        else if (l == 16) v = d[2];
        else if (l == 17) v = n0;
        else if (l == 18) v = n1;
        else if (l == 19) v = d[6];
        else if (l == 20) v = d[7];
        else if (l < 29) v = first_col(l - 21);
        hdr[(size_t)s * mx::kTileHdr + l] = v;
    }
    const int c0 = first_col(l >> 3);
    atox[(size_t)s * 64 + l] = c0 >= 0 ? c0 + (l & 7) : -1;
}
// the values of every member row into its chunk's blocks (8 x 8, row-major, zeros elsewhere)
__global__ __launch_bounds__(kBlock) void strip_values_kernel(const int *__restrict__ perm, const int *__restrict__ candRow,
                                                              const int *__restrict__ memberChunk, const int *__restrict__ runIdIncl,
                                                              const int *__restrict__ runStart, const int *__restrict__ chunkKey,
                                                              const int *__restrict__ chunkNb, const int *__restrict__ chunkBlock0,
                                                              const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                              const unsigned short *__restrict__ ddVal, const int *__restrict__ descColId,
                                                              int n, unsigned short *__restrict__ tcVal)
{
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j >= n) return;
    const int chunk = memberChunk[j];
    if (chunk < 0) return;
    const int jj = (j - runStart[runIdIncl[j] - 1]) & 7, i = candRow[perm[j]], nb = chunkNb[chunk];
    const int *b = chunkKey + (size_t)chunk * 8;
    const size_t base = (size_t)chunkBlock0[chunk] * 64;
    for (int p = ddRowPtr[i]; p < ddRowPtr[i + 1]; ++p) {
        const int c = descColId[ddCol[p]];
        int k = 0;
        while (k < nb - 1 && b[k] + 8 <= c) ++k;
        tcVal[base + (size_t)k * 64 + jj * 8 + (c - b[k])] = ddVal[p];
    }
}


// ---- the general tile form: the reference's fragments that pass the gate, re-blocked.
// One thread per chunk of the reference's numbering: which of its fragments pass the gate on what the
// taken rows leave (selFrag), which of their column positions are still in use -- one sort key
// (chunk, caller's column) each, all ones for a position out of use -- how many there are, and how
// many of the chunk's column ids are real (the list is padded with zeros to whole fragments).
template <bool F64>
__global__ __launch_bounds__(kBlock) void chunk_refs_kernel(const int *__restrict__ chunkPtr, const void *__restrict__ fragBit,
                                                            const int *__restrict__ atox, const int *__restrict__ descColId,
                                                            const unsigned char *__restrict__ taken, int chunkNum, int dRows, int minVals,
                                                            unsigned char *__restrict__ selFrag, unsigned long long *__restrict__ refKey,
                                                            int *__restrict__ nrefs, int *__restrict__ usedCols)
{
    constexpr int K = F64 ? 4 : 8;
    const int w = blockIdx.x * kBlock + threadIdx.x;
    if (w >= chunkNum) return;
    unsigned long long rowsLeft = 0;
    for (int r = 0; r < 8; ++r) {
        const int i = w * 8 + r;
        if (i < dRows && !(taken && taken[i])) rowsLeft |= (F64 ? 0xfull : 0xffull) << (r * K);
    }
    const int f0 = chunkPtr[w], f1 = chunkPtr[w + 1];
    int n = 0;
    for (int f = f0; f < f1; ++f) {
        const unsigned long long bm = F64 ? (unsigned long long)((const unsigned *)fragBit)[f] : ((const unsigned long long *)fragBit)[f];
        const unsigned long long left = bm & rowsLeft;
        const int vals = __popcll(left);
        const bool pass = vals > 0 && vals >= minVals;
        selFrag[f] = pass ? 1 : 0;
        for (int c = 0; c < K; ++c) {
            const unsigned long long colBits = (F64 ? 0x11111111ull : 0x0101010101010101ull) << c;
            const bool used = pass && (left & colBits) != 0;
            refKey[(size_t)f * K + c] =
                used ? ((unsigned long long)(unsigned)w << 32) | (unsigned)descColId[atox[(size_t)f * K + c]] : ~0ull;
            n += used;
        }
    }
    nrefs[w] = n;
    int u = (f1 - f0) * K;
    const int *a = atox + (size_t)f0 * K;
    while (u > 1 && a[u - 1] == 0) --u;
    usedCols[w] = u;
}
// sorted position -> the column there and, for the (fragment, position) it came from, its place in the chunk
__global__ __launch_bounds__(kBlock) void ref_places_kernel(const unsigned long long *__restrict__ key, const int *__restrict__ pay,
                                                            const int *__restrict__ refStart, int n, int *__restrict__ sortedCol,
                                                            int *__restrict__ where)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const unsigned long long k = key[i];
    const int w = (int)(k >> 32);
    sortedCol[i] = (int)(unsigned)k;
    where[pay[i]] = i - refStart[w];
}
__global__ __launch_bounds__(kBlock) void chunk_blocks_kernel(const int *__restrict__ nrefs, int chunkNum, int K, int *__restrict__ isSel)
{
    const int w = blockIdx.x * kBlock + threadIdx.x;
    if (w <= chunkNum) isSel[w] = w < chunkNum && nrefs[w] > 0 ? 1 : 0;
}
__global__ __launch_bounds__(kBlock) void sel_chunks_kernel(const int *__restrict__ nrefs, const int *__restrict__ isSel,
                                                            const int *__restrict__ selPos, int chunkNum, int K, int *__restrict__ selW,
                                                            int *__restrict__ selNb)
{
    const int w = blockIdx.x * kBlock + threadIdx.x;
    if (w >= chunkNum || !isSel[w]) return;
    selW[selPos[w]] = w;
    selNb[selPos[w]] = (nrefs[w] + K - 1) / K;
}
// stepDesc[s] = {selected chunk of half 0, of half 1 (-1 none, -2 the first goes on), flags, blocks in
// half 0, blocks in half 1, first value, first value and blocks in half 0 of the step four further on,
// first block of half 0 inside its chunk}; one wave per step writes header and column ids.
template <bool F64>
__global__ __launch_bounds__(64) void tile_steps_kernel(const int *__restrict__ stepDesc, const int *__restrict__ selW,
                                                        const int *__restrict__ nrefs, const int *__restrict__ refStart,
                                                        const int *__restrict__ sortedCol, const unsigned char *__restrict__ taken,
                                                        const int *__restrict__ rId, int dRows, int steps, int *__restrict__ hdr,
                                                        int *__restrict__ atox)
{
    constexpr int K = F64 ? 4 : 8, SLOTS = F64 ? 16 : 8;
    const int s = blockIdx.x, l = threadIdx.x;
    if (s >= steps) return;
    const int *d = stepDesc + (size_t)s * 10;
    const int A = selW[d[0]], B = d[1] >= 0 ? selW[d[1]] : d[1], n0 = d[3], n1 = d[4], i0 = d[8];
    // column c of the block in a slot, -1 = none
    auto column = [&](int slot, int c) {
        const int half = F64 ? (slot & 1) : (slot >> 2), i = F64 ? (slot >> 1) : (slot & 3);
        int X, b;
        if (half == 0) {
            if (i >= n0) return -1;
            X = A;
            b = i0 + i;
        } else {
            if (i >= n1) return -1;
            X = B >= 0 ? B : A;
            b = B >= 0 ? i : i0 + n0 + i;
        }
        const int at = b * K + c;
        return at < nrefs[X] ? sortedCol[refStart[X] + at] : -1;
    };
    auto out_row = [&](int X, int i) {
        const int local = X * 8 + i;
        return local < dRows && !(taken && taken[local]) ? rId[local] : -1;
    };
    if (l < mx::kTileHdr) {
        int v = 0;
        if (l < 8) v = out_row(A, l);
        else if (l < 16) v = B >= 0 ? out_row(B, l - 8) : -1;
        else if (l == 16) v = d[2];
        else if (l == 17) v = n0;
        else if (l == 18) v = n1;
        else if (l == 19) v = d[6];
        else if (l == 20) v = d[7];
        else if (l < 29) v = SLOTS == 8 ? column(l - 21, 0) : -1;
        hdr[(size_t)s * mx::kTileHdr + l] = v;
    }
    atox[(size_t)s * 64 + l] = column(l / K, l % K);
}
// One thread per row of A_dd walks the row beside its chunk's column list (both ascending), which
// gives every entry its fragment and position.  COUNT: how many entries stay in the CSR part (the row's
// earlier twins and the entries of fragments that failed the gate; none of a taken row).  Otherwise:
// those entries written behind the row's residual entries, and the others into the tile values.
template <typename V, bool COUNT>
__global__ __launch_bounds__(kBlock) void dd_rows_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                         const V *__restrict__ ddVal, const int *__restrict__ descColId,
                                                         const int *__restrict__ rId, const unsigned char *__restrict__ taken,
                                                         const int *__restrict__ chunkPtr, const int *__restrict__ atox,
                                                         const int *__restrict__ usedCols, const unsigned char *__restrict__ selFrag,
                                                         int dRows, int K, int *__restrict__ kept,
                                                         // (not COUNT)
                                                         const int *__restrict__ cdRowPtr, const int *__restrict__ outPtr,
                                                         int *__restrict__ col, V *__restrict__ val, const int *__restrict__ where,
                                                         const int *__restrict__ selPos, const int *__restrict__ chunkBlock0,
                                                         V *__restrict__ tcVal)
{
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= dRows) return;
    const int p0 = ddRowPtr[i], p1 = ddRowPtr[i + 1];
    const bool rowTaken = taken && taken[i];
    if (rowTaken) {
        if (COUNT) kept[i] = 0;
        return;
    }
    const int w = i >> 3, r8 = i & 7, f0 = chunkPtr[w], na = usedCols[w];
    const int *a = atox + (size_t)f0 * K;
    int rank = 0, n = 0, q = 0;
    size_t base = 0;
    if (!COUNT) {
        const int r = rId[i];
        q = outPtr[r] + (cdRowPtr[r + 1] - cdRowPtr[r]);
        base = (size_t)chunkBlock0[selPos[w]] * 8 * K;  // (read only when the chunk has selected fragments)
    }
    for (int p = p0; p < p1; ++p) {
        const int c = ddCol[p];
        while (rank < na && a[rank] < c) ++rank;
        const bool earlierTwin = p + 1 < p1 && ddCol[p + 1] == c;
        const int f = f0 + rank / K;
        const bool keep = earlierTwin || !selFrag[f];
        if (COUNT) {
            n += keep;
        } else if (keep) {
            col[q] = descColId[c];
            val[q] = ddVal[p];
            ++q;
        } else {
            const int at = where[(size_t)f * K + rank % K];  // place of the column among the chunk's, ascending by caller's id
            tcVal[base + (size_t)(at / K) * 8 * K + r8 * K + at % K] = ddVal[p];
        }
    }
    if (COUNT) kept[i] = n;
}
__global__ __launch_bounds__(kBlock) void part_lengths_kept_kernel(const int *__restrict__ cdRowPtr, const int *__restrict__ kept,
                                                                   const int *__restrict__ ddRowOf, const unsigned char *__restrict__ taken,
                                                                   int rows, int *__restrict__ len, char *__restrict__ stripRows)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r > rows) return;
    if (r == rows) {
        len[r] = 0;
        return;
    }
    const int i = ddRowOf[r];
    len[r] = cdRowPtr[r + 1] - cdRowPtr[r] + (i >= 0 ? kept[i] : 0);
    if (stripRows) stripRows[r] = i >= 0 && taken && taken[i] ? 1 : 0;
}


// ---- the binary64 block form: the qualifying runs of the sorted (block row, block column) keys.
__global__ __launch_bounds__(kBlock) void block_heads_kernel(const unsigned long long *__restrict__ key, int n, int need, int cols,
                                                             int *__restrict__ selHead)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p > n) return;
    int h = 0;
    if (p < n && key[p] != ~0ull && (p == 0 || key[p - 1] != key[p])) {
        int e = p + 1;
        while (e < n && e - p < 64 && key[e] == key[p]) ++e;
        h = e - p >= need && (int)(unsigned)key[p] + 1 <= cols / 8 ? 1 : 0;
    }
    selHead[p] = h;
}
// per block (numbered in key order): its block row and column; per entry of A_dd: its block, -1 = none
__global__ __launch_bounds__(kBlock) void block_records_kernel(const unsigned long long *__restrict__ key, const int *__restrict__ pay,
                                                               const int *__restrict__ selHead, const int *__restrict__ blockId, int n,
                                                               int *__restrict__ blkBr, int *__restrict__ blkBc,
                                                               int *__restrict__ entryBlock)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= n || !selHead[p]) return;
    const int g = blockId[p];
    blkBr[g] = (int)(key[p] >> 32);
    blkBc[g] = (int)(unsigned)key[p];
    for (int e = p; e < n && e - p < 64 && key[e] == key[p]; ++e) entryBlock[pay[e]] = g;
}
__global__ __launch_bounds__(kBlock) void block_chunk_heads_kernel(const int *__restrict__ blkBr, int nBlocks, int *__restrict__ head)
{
    const int g = blockIdx.x * kBlock + threadIdx.x;
    if (g < nBlocks) head[g] = g == 0 || blkBr[g] != blkBr[g - 1] ? 1 : 0;
}
__global__ __launch_bounds__(kBlock) void block_chunk_starts_kernel(const int *__restrict__ head, const int *__restrict__ chunkIdIncl,
                                                                    const int *__restrict__ blkBr, int nBlocks,
                                                                    int *__restrict__ chunkStart, int *__restrict__ chunkBr)
{
    const int g = blockIdx.x * kBlock + threadIdx.x;
    if (g >= nBlocks) return;
    if (head[g]) {
        chunkStart[chunkIdIncl[g] - 1] = g;
        chunkBr[chunkIdIncl[g] - 1] = blkBr[g];
    }
    if (g == nBlocks - 1) chunkStart[chunkIdIncl[g]] = nBlocks;
}
__global__ __launch_bounds__(kBlock) void block_chunk_sizes_kernel(const int *__restrict__ chunkStart, int nChunks, int *__restrict__ nb)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c < nChunks) nb[c] = chunkStart[c + 1] - chunkStart[c];
}
// marks of the rows of block chunks (2: the block waves fetch the sums of these rows' virtual rows themselves)
__global__ __launch_bounds__(kBlock) void block_marks_kernel(const int *__restrict__ chunkBr, int nChunks, int rows, char *__restrict__ marks)
{
    const int c = blockIdx.x * kBlock + threadIdx.x;
    if (c >= nChunks) return;
    for (int j = 0; j < 8; ++j) {
        const int r = chunkBr[c] * 8 + j;
        if (r < rows) marks[r] = 2;
    }
}
// stepDesc as for the general form (10 ints per step, chunks numbered in block-row order)
__global__ __launch_bounds__(64) void block_steps_kernel(const int *__restrict__ stepDesc, const int *__restrict__ chunkStart,
                                                         const int *__restrict__ chunkBr, const int *__restrict__ blkBc, int rows,
                                                         int steps, int *__restrict__ hdr, int *__restrict__ atox)
{
    const int s = blockIdx.x, l = threadIdx.x;
    if (s >= steps) return;
    const int *d = stepDesc + (size_t)s * 10;
    const int A = d[0], B = d[1], n0 = d[3], n1 = d[4], i0 = d[8];
    auto first_col = [&](int slot) {
        const int half = slot >> 2, i = slot & 3;
        if (half == 0) return i < n0 ? blkBc[chunkStart[A] + i0 + i] * 8 : -1;
        if (i >= n1) return -1;
        return (B >= 0 ? blkBc[chunkStart[B] + i] : blkBc[chunkStart[A] + i0 + n0 + i]) * 8;
    };
    auto out_row = [&](int X, int j) {
        const int r = chunkBr[X] * 8 + j;
        return r < rows ? r : -1;
    };
    if (l < mx::kTileHdr) {
        int v = 0;
        if (l < 8) v = out_row(A, l);
        else if (l < 16) v = B >= 0 ? out_row(B, l - 8) : -1;
        else if (l == 16) v = d[2];
        else if (l == 17) v = n0;
        else if (l == 18) v = n1;
        else if (l == 19) v = d[6];
        else if (l == 20) v = d[7];
        else if (l < 29) v = first_col(l - 21);
        hdr[(size_t)s * mx::kTileHdr + l] = v;
    }
    const int c0 = first_col(l >> 3);
    atox[(size_t)s * 64 + l] = c0 >= 0 ? c0 + (l & 7) : -1;
}
__global__ __launch_bounds__(kBlock) void block_values_kernel(const int *__restrict__ entryBlock, const int *__restrict__ chunkIdIncl,
                                                              const int *__restrict__ chunkStart, const int *__restrict__ chunkBlock0,
                                                              const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                              const double *__restrict__ ddVal, const int *__restrict__ descColId,
                                                              const int *__restrict__ rId, int dRows, int nDD, double *__restrict__ tcVal)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= nDD) return;
    const int g = entryBlock[p];
    if (g < 0) return;
    int lo = 0, hi = dRows - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (ddRowPtr[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    const int chunk = chunkIdIncl[g] - 1, r = rId[lo], c = descColId[ddCol[p]];
    tcVal[((size_t)chunkBlock0[chunk] + (g - chunkStart[chunk])) * 64 + (r & 7) * 8 + (c & 7)] = ddVal[p];
}
// the CSR part beside blocks: an entry stays unless a block took it
__global__ __launch_bounds__(kBlock) void block_keep_kernel(const int *__restrict__ entryBlock, int nDD, int *__restrict__ keep)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p <= nDD) keep[p] = p < nDD && entryBlock[p] < 0 ? 1 : 0;
}
__global__ __launch_bounds__(kBlock) void part_lengths_scan_kernel(const int *__restrict__ cdRowPtr, const int *__restrict__ ddRowPtr,
                                                                   const int *__restrict__ ddRowOf, const int *__restrict__ keptBefore,
                                                                   int rows, int *__restrict__ len)
{
    const int r = blockIdx.x * kBlock + threadIdx.x;
    if (r > rows) return;
    if (r == rows) {
        len[r] = 0;
        return;
    }
    const int i = ddRowOf[r];
    len[r] = cdRowPtr[r + 1] - cdRowPtr[r] + (i >= 0 ? keptBefore[ddRowPtr[i + 1]] - keptBefore[ddRowPtr[i]] : 0);
}
template <typename V>
__global__ __launch_bounds__(kBlock) void part_dense_scan_kernel(const int *__restrict__ ddRowPtr, const int *__restrict__ ddCol,
                                                                 const V *__restrict__ ddVal, const int *__restrict__ descColId,
                                                                 const int *__restrict__ rId, const int *__restrict__ entryBlock,
                                                                 const int *__restrict__ keptBefore, const int *__restrict__ cdRowPtr,
                                                                 const int *__restrict__ outPtr, int dRows, int nDD, int *__restrict__ col,
                                                                 V *__restrict__ val)
{
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= nDD || entryBlock[p] >= 0) return;
    int lo = 0, hi = dRows - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (ddRowPtr[mid] <= p) lo = mid;
        else hi = mid - 1;
    }
    const int r = rId[lo];
    const int q = outPtr[r] + (cdRowPtr[r + 1] - cdRowPtr[r]) + (keptBefore[p] - keptBefore[ddRowPtr[lo]]);
    col[q] = descColId[ddCol[p]];
    val[q] = ddVal[p];
}

}  // namespace mxh

#define MXH_TRY(call)                                                                                 \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            mx::set_error(std::string("hybrid plan on the device: ") + #call + ": " + hipGetErrorString(e_)); \
            return e_ == hipErrorOutOfMemory ? MX_ERR_ALLOC : MX_ERR_DEVICE;                          \
        }                                                                                             \
    } while (0)

namespace mx {

using mxh::Buf;
using mxh::grid;
using mxh::kBlock;

struct HybridDevice::Impl {
    mx_dtype dtype = MX_F64;
    int rows = 0, cols = 0, nnz = 0, dRows = 0, dCols = 0, nDD = 0, nCD = 0;
    hipStream_t s = nullptr;
    // the extraction
    Buf order;  // descColId [cols], descRowId [rows]
    int *dc = nullptr, *dr = nullptr;
    Buf split;  // ddRowPtr, ddColInd, ddVal, cdRowPtr, cdColInd, cdVal
    int *ddp = nullptr, *ddc = nullptr, *cdp = nullptr, *cdc = nullptr;
    void *ddv = nullptr, *cdv = nullptr;
    mx_device_tiles T{};
    Buf colOrig, ddRowOf, taken;
    // strip chunks
    int nCand = 0, nChunks = 0;
    Buf perm, candRow, candKey, candNb, runIdIncl, runStart, memberChunk, chunkRows, chunkKey, chunkNb, chunkNnz;
    // the general tile form (tile_chunks)
    int minVals = 1, nSel = 0;
    Buf selFrag, usedCols, nrefs, refStart, sortedCol, where, selPos, selW, tileBlock0;
    // the binary64 block form (analyse keeps the sorted keys; block_chunks, block_layout)
    int nBlk = 0, nBlkChunks = 0;
    Buf blkKey, blkPay, blkBr, blkBc, entryBlock, blkChunkIdIncl, blkChunkStart, blkChunkBr;
    void *tileVal = nullptr;  // the values of the general tile layout (owned by the caller's DeviceTiles): csr_part fills them
    bool borrowed = false;    // the extraction's arrays belong to a partition's twin: not released here
    ~Impl()
    {
        if (borrowed) {
            (void)order.take();
            (void)split.take();
        } else {
            mx_tiles_device_free(&T);
        }
    }
};

static int analyse_tail(HybridDevice::Impl &I, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts);

HybridDevice::~HybridDevice() { delete impl; }

int HybridDevice::analyse(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev,
                          float tau_c, float tau_r, int minVals, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts,
                          hipStream_t s)
{
    using namespace mxh;
    delete impl;
    impl = new Impl();
    Impl &I = *impl;
    I.dtype = dtype;
    I.rows = rows;
    I.cols = cols;
    I.nnz = nnz;
    I.s = s;
    I.minVals = minVals;
    *counts = HybridCounts();
    const size_t es = (size_t)mx::elem_size(dtype);
    auto al = [](size_t b) { return (b + 255) & ~(size_t)255; };
    {
        const size_t dcB = al((size_t)cols * 4 + 4), drB = al((size_t)rows * 4 + 4);
        MXH_TRY(hipMalloc(&I.order.p, dcB + drB));
        I.dc = (int *)I.order.p;
        I.dr = (int *)((unsigned char *)I.order.p + dcB);
    }
    mx_selection sel{};
    int rc = mx_select_device(rows, cols, nnz, rowPtr_dev, col_dev, tau_c, tau_r, I.dc, I.dr, &sel, s);
    if (rc != MX_OK) return rc;
    I.dRows = sel.dRows;
    I.dCols = sel.dCols;
    I.nDD = sel.nnzRowD;
    I.nCD = nnz - sel.nnzRowD;
    {
        const size_t ddpB = al(((size_t)I.dRows + 1) * 4), ddcB = al((size_t)I.nDD * 4 + 4), ddvB = al((size_t)I.nDD * es + 8),
                     cdpB = al(((size_t)rows + 1) * 4), cdcB = al((size_t)I.nCD * 4 + 4), cdvB = al((size_t)I.nCD * es + 8);
        MXH_TRY(hipMalloc(&I.split.p, ddpB + ddcB + ddvB + cdpB + cdcB + cdvB));
        unsigned char *b = (unsigned char *)I.split.p;
        I.ddp = (int *)b;
        I.ddc = (int *)(b + ddpB);
        I.ddv = b + ddpB + ddcB;
        I.cdp = (int *)(b + ddpB + ddcB + ddvB);
        I.cdc = (int *)(b + ddpB + ddcB + ddvB + cdpB);
        I.cdv = b + ddpB + ddcB + ddvB + cdpB + cdcB;
    }
    rc = mx_split_device(dtype, rows, cols, nnz, rowPtr_dev, col_dev, val_dev, &sel, I.dc, I.dr, I.ddp, I.ddc, I.ddv, I.cdp, I.cdc, I.cdv, s);
    if (rc != MX_OK) return rc;
    rc = mx_tiles_device(dtype, I.dRows, I.dCols, I.nDD, I.ddp, I.ddc, I.ddv, &I.T, s);
    if (rc != MX_OK) return rc;
    return analyse_tail(I, wantGeneral, wantStrips, wantBlocks, counts);
}

int HybridDevice::adopt(const PartitionTwin &W, int minVals, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts,
                        hipStream_t s)
{
    delete impl;
    impl = new Impl();
    Impl &I = *impl;
    I.dtype = W.dtype;
    I.rows = W.rows;
    I.cols = W.cols;
    I.nnz = W.nnz;
    I.s = s;
    I.minVals = minVals;
    I.dRows = W.dRows;
    I.dCols = W.dCols;
    I.nDD = W.nDD;
    I.nCD = W.nCD;
    I.borrowed = true;
    I.order.p = W.order;
    I.dc = W.dc;
    I.dr = W.dr;
    I.split.p = W.split;
    I.ddp = W.ddp;
    I.ddc = W.ddc;
    I.ddv = W.ddv;
    I.cdp = W.cdp;
    I.cdc = W.cdc;
    I.cdv = W.cdv;
    I.T = W.T;
    *counts = HybridCounts();
    return analyse_tail(I, wantGeneral, wantStrips, wantBlocks, counts);
}

// What follows the extraction, whoever made it: the maps back to the caller's numbering, the strip rows, the
// blocks, the fill gate, and the counts the plan decides from.
static int analyse_tail(HybridDevice::Impl &I, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts)
{
    using namespace mxh;
    const mx_dtype dtype = I.dtype;
    const int rows = I.rows, cols = I.cols, minVals = I.minVals;
    hipStream_t s = I.s;
    // columns of the residual's numbering -> the caller's; the row of A_dd of every row
    {
        Buf flag, notSel, pos, tmp;
        size_t scanBytes = 0;
        MXH_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, (size_t)cols, rocprim::plus<int>(), s));
        MXH_TRY(hipMalloc(&flag.p, (size_t)cols + 4));
        MXH_TRY(hipMalloc(&notSel.p, (size_t)cols * 4 + 4));
        MXH_TRY(hipMalloc(&pos.p, (size_t)cols * 4 + 4));
        MXH_TRY(hipMalloc(&tmp.p, scanBytes + 256));
        MXH_TRY(hipMalloc(&I.colOrig.p, (size_t)cols * 4 + 4));
        MXH_TRY(hipMemsetAsync(flag.p, 0, (size_t)cols + 4, s));
        if (I.dCols > 0) {
            hipLaunchKernelGGL(mark_kernel, grid(I.dCols), dim3(kBlock), 0, s, (const int *)I.dc, I.dCols, flag.as<unsigned char>());
            MXH_TRY(hipGetLastError());
        }
        hipLaunchKernelGGL(unmarked_kernel, grid(cols), dim3(kBlock), 0, s, (const unsigned char *)flag.p, cols, notSel.as<int>());
        MXH_TRY(hipGetLastError());
        MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)notSel.p, pos.as<int>(), 0, (size_t)cols, rocprim::plus<int>(), s));
        hipLaunchKernelGGL(col_orig_kernel, grid(cols), dim3(kBlock), 0, s, (const int *)I.dc, (const unsigned char *)flag.p,
                           (const int *)pos.p, cols, I.dCols, I.colOrig.as<int>());
        MXH_TRY(hipGetLastError());
        MXH_TRY(hipMalloc(&I.ddRowOf.p, (size_t)rows * 4 + 4));
        MXH_TRY(hipMemsetAsync(I.ddRowOf.p, 0xff, (size_t)rows * 4 + 4, s));
        if (I.dRows > 0) {
            hipLaunchKernelGGL(dd_row_of_kernel, grid(I.dRows), dim3(kBlock), 0, s, (const int *)I.dr, I.dRows, I.ddRowOf.as<int>());
            MXH_TRY(hipGetLastError());
        }
        MXH_TRY(hipStreamSynchronize(s));
    }
    MXH_TRY(hipMalloc(&I.taken.p, (size_t)I.dRows + 4));
    MXH_TRY(hipMemsetAsync(I.taken.p, 0, (size_t)I.dRows + 4, s));
    Buf totals;
    MXH_TRY(hipMalloc(&totals.p, 8 * 8));
    MXH_TRY(hipMemsetAsync(totals.p, 0, 8 * 8, s));
    unsigned long long *tot = totals.as<unsigned long long>();

    // ---- binary16: rows of dense strips, grouped by their set of blocks
    if (wantStrips && dtype == MX_F16 && I.dRows > 0 && I.nDD > 0) {
        Buf isCand, candPos, tmp;
        size_t scanBytes = 0, b2 = 0;
        MXH_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, (size_t)I.dRows + 1, rocprim::plus<int>(), s));
        MXH_TRY(rocprim::inclusive_scan(nullptr, b2, (const int *)nullptr, (int *)nullptr, (size_t)I.dRows + 1, rocprim::plus<int>(), s));
        scanBytes = std::max(scanBytes, b2);
        MXH_TRY(hipMalloc(&isCand.p, ((size_t)I.dRows + 1) * 4));
        MXH_TRY(hipMalloc(&candPos.p, ((size_t)I.dRows + 1) * 4));
        MXH_TRY(hipMalloc(&tmp.p, scanBytes + 256));
        MXH_TRY(hipMemsetAsync(isCand.p, 0, ((size_t)I.dRows + 1) * 4, s));
        hipLaunchKernelGGL(strip_candidates_kernel, grid(I.dRows), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc, (const int *)I.dc,
                           (const int *)I.dr, (const int *)I.cdp, I.dRows, cols, isCand.as<int>());
        MXH_TRY(hipGetLastError());
        MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)isCand.p, candPos.as<int>(), 0, (size_t)I.dRows + 1, rocprim::plus<int>(), s));
        int nCand = 0;
        MXH_TRY(hipMemcpyAsync(&nCand, candPos.as<int>() + I.dRows, 4, hipMemcpyDeviceToHost, s));
        MXH_TRY(hipStreamSynchronize(s));
        I.nCand = nCand;
        if (nCand > 0) {
            const size_t nc = (size_t)nCand;
            MXH_TRY(hipMalloc(&I.candRow.p, nc * 4));
            MXH_TRY(hipMalloc(&I.candKey.p, nc * 8 * 4));
            MXH_TRY(hipMalloc(&I.candNb.p, nc * 4));
            hipLaunchKernelGGL(candidate_keys_kernel, grid(I.dRows), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc,
                               (const int *)I.dc, (const int *)I.dr, (const int *)I.cdp, (const int *)isCand.p, (const int *)candPos.p, I.dRows,
                               cols, I.candRow.as<int>(), I.candKey.as<int>(), I.candNb.as<int>());
            MXH_TRY(hipGetLastError());
            // by (block 0, .., block 7, row): eight stable passes, the last block first
            Buf permB, keyA, keyB, sortTmp;
            unsigned bits = 1;
            while (bits < 32 && (1ull << bits) < (unsigned long long)cols + 2ull) ++bits;  // (the keys are first columns + 1)
            size_t sortBytes = 0;
            MXH_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned *)nullptr, (unsigned *)nullptr, (const int *)nullptr,
                                              (int *)nullptr, nc, 0u, bits, s));
            MXH_TRY(hipMalloc(&I.perm.p, nc * 4));
            MXH_TRY(hipMalloc(&permB.p, nc * 4));
            MXH_TRY(hipMalloc(&keyA.p, nc * 4));
            MXH_TRY(hipMalloc(&keyB.p, nc * 4));
            MXH_TRY(hipMalloc(&sortTmp.p, sortBytes + 256));
            hipLaunchKernelGGL(iota_kernel, grid(nCand), dim3(kBlock), 0, s, I.perm.as<int>(), nCand);
            MXH_TRY(hipGetLastError());
            for (int k = 7; k >= 0; --k) {
                hipLaunchKernelGGL(pass_keys_kernel, grid(nCand), dim3(kBlock), 0, s, (const int *)I.candKey.p, (const int *)I.perm.p, nCand, k,
                                   keyA.as<unsigned>());
                MXH_TRY(hipGetLastError());
                MXH_TRY(rocprim::radix_sort_pairs(sortTmp.p, sortBytes, (const unsigned *)keyA.p, keyB.as<unsigned>(), (const int *)I.perm.p,
                                                  permB.as<int>(), nc, 0u, bits, s));
                std::swap(I.perm.p, permB.p);
            }
            // runs of equal block sets and their chunks
            Buf head, runChunks, runChunk0;
            MXH_TRY(hipMalloc(&head.p, (nc + 1) * 4));
            MXH_TRY(hipMalloc(&I.runIdIncl.p, (nc + 1) * 4));
            MXH_TRY(hipMalloc(&I.runStart.p, (nc + 2) * 4));
            hipLaunchKernelGGL(run_heads_kernel, grid(nCand), dim3(kBlock), 0, s, (const int *)I.candKey.p, (const int *)I.perm.p, nCand,
                               head.as<int>());
            MXH_TRY(hipGetLastError());
            MXH_TRY(rocprim::inclusive_scan(tmp.p, scanBytes, (const int *)head.p, I.runIdIncl.as<int>(), nc, rocprim::plus<int>(), s));
            int nRuns = 0;
            MXH_TRY(hipMemcpyAsync(&nRuns, I.runIdIncl.as<int>() + (nc - 1), 4, hipMemcpyDeviceToHost, s));
            MXH_TRY(hipStreamSynchronize(s));
            hipLaunchKernelGGL(run_starts_kernel, grid(nCand), dim3(kBlock), 0, s, (const int *)head.p, (const int *)I.runIdIncl.p, nCand,
                               I.runStart.as<int>());
            MXH_TRY(hipGetLastError());
            MXH_TRY(hipMalloc(&runChunks.p, ((size_t)nRuns + 1) * 4));
            MXH_TRY(hipMalloc(&runChunk0.p, ((size_t)nRuns + 1) * 4));
            MXH_TRY(hipMemsetAsync(runChunks.p, 0, ((size_t)nRuns + 1) * 4, s));
            hipLaunchKernelGGL(run_chunks_kernel, grid(nRuns), dim3(kBlock), 0, s, (const int *)I.runStart.p, nRuns, runChunks.as<int>());
            MXH_TRY(hipGetLastError());
            // (nRuns <= nCand <= dRows: the scan's temporary storage is large enough)
            MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)runChunks.p, runChunk0.as<int>(), 0, (size_t)nRuns + 1,
                                            rocprim::plus<int>(), s));
            int nChunks = 0;
            MXH_TRY(hipMemcpyAsync(&nChunks, runChunk0.as<int>() + nRuns, 4, hipMemcpyDeviceToHost, s));
            MXH_TRY(hipStreamSynchronize(s));
            I.nChunks = nChunks;
            if (nChunks > 0) {
                const size_t nk = (size_t)nChunks;
                MXH_TRY(hipMalloc(&I.memberChunk.p, nc * 4));
                MXH_TRY(hipMalloc(&I.chunkRows.p, nk * 8 * 4));
                MXH_TRY(hipMalloc(&I.chunkKey.p, nk * 8 * 4));
                MXH_TRY(hipMalloc(&I.chunkNb.p, nk * 4));
                MXH_TRY(hipMalloc(&I.chunkNnz.p, nk * 4));
                MXH_TRY(hipMemsetAsync(I.chunkRows.p, 0xff, nk * 8 * 4, s));
                hipLaunchKernelGGL(chunk_members_kernel, grid(nCand), dim3(kBlock), 0, s, (const int *)I.perm.p, (const int *)I.candRow.p,
                                   (const int *)I.candKey.p, (const int *)I.candNb.p, (const int *)I.runIdIncl.p, (const int *)I.runStart.p,
                                   (const int *)runChunks.p, (const int *)runChunk0.p, (const int *)I.ddp, (const int *)I.dr, nCand,
                                   I.taken.as<unsigned char>(), I.memberChunk.as<int>(), I.chunkRows.as<int>(), I.chunkKey.as<int>(),
                                   I.chunkNb.as<int>(), I.chunkNnz.as<int>());
                MXH_TRY(hipGetLastError());
                std::vector<int> nb(nk), ne(nk), key(nk * 8);
                MXH_TRY(hipMemcpyAsync(nb.data(), I.chunkNb.p, nk * 4, hipMemcpyDeviceToHost, s));
                MXH_TRY(hipMemcpyAsync(ne.data(), I.chunkNnz.p, nk * 4, hipMemcpyDeviceToHost, s));
                MXH_TRY(hipMemcpyAsync(key.data(), I.chunkKey.p, nk * 8 * 4, hipMemcpyDeviceToHost, s));
                MXH_TRY(hipStreamSynchronize(s));
                for (size_t k = 0; k < nk; ++k) {
                    counts->stripBlocks += nb[k];
                    counts->stripEntries += ne[k];
                    if (key[k * 8] & 7) counts->stripBlocksOff += nb[k];  // (a chunk's blocks share their offset from the grid)
                }
                counts->stripChunkBlocks.swap(nb);
                counts->stripChunkEntries.swap(ne);
            }
        }
    }
    // ---- binary64: aligned 8 x 8 blocks at least three quarters full (counted here; block_chunks lays them out)
    if (wantBlocks && dtype == MX_F64 && I.dRows > 0 && I.nDD > 0) {
        Buf keyIn, payIn, sortTmp;
        const size_t n = (size_t)I.nDD;
        size_t sortBytes = 0;
        MXH_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                          (const int *)nullptr, (int *)nullptr, n, 0u, 64u, s));
        MXH_TRY(hipMalloc(&keyIn.p, n * 8));
        MXH_TRY(hipMalloc(&payIn.p, n * 4));
        MXH_TRY(hipMalloc(&I.blkKey.p, n * 8));
        MXH_TRY(hipMalloc(&I.blkPay.p, n * 4));
        MXH_TRY(hipMalloc(&sortTmp.p, sortBytes + 256));
        hipLaunchKernelGGL(block_keys_kernel, grid(I.nDD), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc, (const int *)I.dc,
                           (const int *)I.dr, I.dRows, I.nDD, keyIn.as<unsigned long long>());
        MXH_TRY(hipGetLastError());
        hipLaunchKernelGGL(iota_kernel, grid(I.nDD), dim3(kBlock), 0, s, payIn.as<int>(), I.nDD);
        MXH_TRY(hipGetLastError());
        MXH_TRY(rocprim::radix_sort_pairs(sortTmp.p, sortBytes, (const unsigned long long *)keyIn.p, I.blkKey.as<unsigned long long>(),
                                          (const int *)payIn.p, I.blkPay.as<int>(), n, 0u, 64u, s));
        hipLaunchKernelGGL(block_runs_kernel, grid(I.nDD), dim3(kBlock), 0, s, (const unsigned long long *)I.blkKey.p, I.nDD, 48, cols, tot + 2);
        MXH_TRY(hipGetLastError());
    }
    // ---- the fill gate of the reference's fragments
    const int nFrags = I.T.totalTcFrags;
    if (wantGeneral && nFrags > 0) {
        if (dtype == MX_F16)
            hipLaunchKernelGGL(gate_f16_kernel, grid(I.T.chunkNum), dim3(kBlock), 0, s, (const int *)I.T.chunkPtr,
                               (const unsigned long long *)I.T.fragBit, I.nChunks > 0 ? (const unsigned char *)I.taken.p : nullptr, I.T.chunkNum,
                               I.dRows, minVals, tot);
        else
            hipLaunchKernelGGL(gate_counts_kernel, grid(nFrags), dim3(kBlock), 0, s, (const int *)I.T.fragPtr, nFrags, minVals, tot);
        MXH_TRY(hipGetLastError());
    }
    unsigned long long h[4] = {0, 0, 0, 0};
    MXH_TRY(hipMemcpyAsync(h, totals.p, sizeof(h), hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    counts->generalFrags = (long long)h[0];
    counts->generalEntries = (long long)h[1];
    if (h[2] > 0) {
        counts->blocks64 = true;
        counts->stripBlocks = (long long)h[2];
        counts->stripEntries = (long long)h[3];
    }
    counts->dRows = I.dRows;
    counts->dCols = I.dCols;
    counts->nnzRowD = I.nDD;
    counts->frags = I.T.totalTcFrags;
    return MX_OK;
}

template <typename V>
static int csr_part_t(HybridDevice::Impl &I, bool keepStrips, bool keepGeneral, bool keepBlocks, int **rowPtrOut, int **colOut, void **valOut,
                      int *nnzOut, char **stripRowsOut)
{
    using namespace mxh;
    hipStream_t s = I.s;
    const int rows = I.rows, K = mx::frag_k(I.dtype);
    const unsigned char *taken = keepStrips && I.nChunks > 0 ? (const unsigned char *)I.taken.p : nullptr;
    const bool general = keepGeneral && I.nSel > 0 && I.dRows > 0;
    if (general && !I.tileVal) {
        mx::set_error("hybrid plan on the device: the tile layout has to be made before the CSR part");
        return MX_ERR_ARG;
    }
    const bool blocks = keepBlocks && I.nBlkChunks > 0;
    if (blocks && (general || taken)) {
        mx::set_error("hybrid plan on the device: blocks do not go with strips or general tiles");
        return MX_ERR_ARG;
    }
    Buf len, ptr, tmp, col, val, marks, kept, keptBefore;
    size_t scanBytes = 0;
    MXH_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, (size_t)std::max(rows, blocks ? I.nDD : 0) + 1,
                                    rocprim::plus<int>(), s));
    MXH_TRY(hipMalloc(&len.p, ((size_t)rows + 1) * 4));
    MXH_TRY(hipMalloc(&ptr.p, ((size_t)rows + 1) * 4));
    MXH_TRY(hipMalloc(&tmp.p, scanBytes + 256));
    if (taken) MXH_TRY(hipMalloc(&marks.p, (size_t)rows + 4));
    if (blocks) {
        Buf keep;
        MXH_TRY(hipMalloc(&keep.p, ((size_t)I.nDD + 1) * 4));
        MXH_TRY(hipMalloc(&keptBefore.p, ((size_t)I.nDD + 1) * 4));
        MXH_TRY(hipMalloc(&marks.p, (size_t)rows + 4));
        MXH_TRY(hipMemsetAsync(marks.p, 0, (size_t)rows + 4, s));
        hipLaunchKernelGGL(block_keep_kernel, grid((long long)I.nDD + 1), dim3(kBlock), 0, s, (const int *)I.entryBlock.p, I.nDD, keep.as<int>());
        MXH_TRY(hipGetLastError());
        MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)keep.p, keptBefore.as<int>(), 0, (size_t)I.nDD + 1, rocprim::plus<int>(), s));
        hipLaunchKernelGGL(part_lengths_scan_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, (const int *)I.cdp, (const int *)I.ddp,
                           (const int *)I.ddRowOf.p, (const int *)keptBefore.p, rows, len.as<int>());
        MXH_TRY(hipGetLastError());
        hipLaunchKernelGGL(block_marks_kernel, grid(I.nBlkChunks), dim3(kBlock), 0, s, (const int *)I.blkChunkBr.p, I.nBlkChunks, rows,
                           marks.as<char>());
        MXH_TRY(hipStreamSynchronize(s));  // (`keep` leaves scope)
    } else if (general) {
        MXH_TRY(hipMalloc(&kept.p, (size_t)I.dRows * 4 + 4));
        hipLaunchKernelGGL((dd_rows_kernel<V, true>), grid(I.dRows), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc,
                           (const V *)I.ddv, (const int *)I.dc, (const int *)I.dr, taken, (const int *)I.T.chunkPtr,
                           (const int *)I.T.sparse_AToX_index, (const int *)I.usedCols.p, (const unsigned char *)I.selFrag.p, I.dRows, K,
                           kept.as<int>(), (const int *)nullptr, (const int *)nullptr, (int *)nullptr, (V *)nullptr, (const int *)nullptr,
                           (const int *)nullptr, (const int *)nullptr, (V *)nullptr);
        MXH_TRY(hipGetLastError());
        hipLaunchKernelGGL(part_lengths_kept_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, (const int *)I.cdp, (const int *)kept.p,
                           (const int *)I.ddRowOf.p, taken, rows, len.as<int>(), taken ? marks.as<char>() : nullptr);
    } else {
        hipLaunchKernelGGL(part_lengths_kernel, grid((long long)rows + 1), dim3(kBlock), 0, s, (const int *)I.cdp, (const int *)I.ddp,
                           (const int *)I.ddRowOf.p, taken, rows, len.as<int>(), taken ? marks.as<char>() : nullptr);
    }
    MXH_TRY(hipGetLastError());
    MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)len.p, ptr.as<int>(), 0, (size_t)rows + 1, rocprim::plus<int>(), s));
    int n = 0;
    MXH_TRY(hipMemcpyAsync(&n, ptr.as<int>() + rows, 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    MXH_TRY(hipMalloc(&col.p, (size_t)n * 4 + 4));
    MXH_TRY(hipMalloc(&val.p, (size_t)n * sizeof(V) + 8));
    if (I.nCD > 0) {
        hipLaunchKernelGGL(part_residual_kernel<V>, grid(I.nCD), dim3(kBlock), 0, s, (const int *)I.cdp, (const int *)I.cdc, (const V *)I.cdv,
                           (const int *)I.colOrig.p, (const int *)ptr.p, rows, I.nCD, col.as<int>(), val.as<V>());
        MXH_TRY(hipGetLastError());
    }
    if (blocks) {
        hipLaunchKernelGGL(part_dense_scan_kernel<V>, grid(I.nDD), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc, (const V *)I.ddv,
                           (const int *)I.dc, (const int *)I.dr, (const int *)I.entryBlock.p, (const int *)keptBefore.p, (const int *)I.cdp,
                           (const int *)ptr.p, I.dRows, I.nDD, col.as<int>(), val.as<V>());
        MXH_TRY(hipGetLastError());
    } else if (general) {
        hipLaunchKernelGGL((dd_rows_kernel<V, false>), grid(I.dRows), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc,
                           (const V *)I.ddv, (const int *)I.dc, (const int *)I.dr, taken, (const int *)I.T.chunkPtr,
                           (const int *)I.T.sparse_AToX_index, (const int *)I.usedCols.p, (const unsigned char *)I.selFrag.p, I.dRows, K,
                           (int *)nullptr, (const int *)I.cdp, (const int *)ptr.p, col.as<int>(), val.as<V>(), (const int *)I.where.p,
                           (const int *)I.selPos.p, (const int *)I.tileBlock0.p, (V *)I.tileVal);
        MXH_TRY(hipGetLastError());
    } else if (I.nDD > 0) {
        hipLaunchKernelGGL(part_dense_kernel<V>, grid(I.nDD), dim3(kBlock), 0, s, (const int *)I.ddp, (const int *)I.ddc, (const V *)I.ddv,
                           (const int *)I.dc, (const int *)I.dr, taken, (const int *)I.cdp, (const int *)ptr.p, I.dRows, I.nDD, col.as<int>(),
                           val.as<V>());
        MXH_TRY(hipGetLastError());
    }
    MXH_TRY(hipStreamSynchronize(s));
    *nnzOut = n;
    *rowPtrOut = (int *)ptr.take();
    *colOut = (int *)col.take();
    *valOut = val.take();
    *stripRowsOut = (char *)marks.take();
    return MX_OK;
}

int HybridDevice::csr_part(bool keepStrips, bool keepGeneral, bool keepBlocks, int **rowPtr_dev, int **col_dev, void **val_dev, int *nnz,
                           char **stripRows_dev)
{
    if (!impl) return MX_ERR_ARG;
    if (impl->dtype == MX_F64)
        return csr_part_t<double>(*impl, keepStrips, keepGeneral, keepBlocks, rowPtr_dev, col_dev, val_dev, nnz, stripRows_dev);
    return csr_part_t<unsigned short>(*impl, keepStrips, keepGeneral, keepBlocks, rowPtr_dev, col_dev, val_dev, nnz, stripRows_dev);
}

// The chunks of the binary64 block form: per block row with at least one block, in ascending order, how
// many blocks it has (`blocks`) and which block row it is (`blockRows`).
int HybridDevice::block_chunks(std::vector<int> &blocks, std::vector<int> &blockRows)
{
    using namespace mxh;
    blocks.clear();
    blockRows.clear();
    if (!impl || impl->dtype != MX_F64) return MX_ERR_ARG;
    Impl &I = *impl;
    hipStream_t s = I.s;
    I.nBlk = I.nBlkChunks = 0;
    if (!I.blkKey.p || I.nDD <= 0) return MX_OK;
    const size_t n = (size_t)I.nDD;
    Buf selHead, blockId, tmp, head, nb;
    size_t scanBytes = 0, b2 = 0;
    MXH_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, n + 1, rocprim::plus<int>(), s));
    MXH_TRY(rocprim::inclusive_scan(nullptr, b2, (const int *)nullptr, (int *)nullptr, n + 1, rocprim::plus<int>(), s));
    scanBytes = std::max(scanBytes, b2);
    MXH_TRY(hipMalloc(&selHead.p, (n + 1) * 4));
    MXH_TRY(hipMalloc(&blockId.p, (n + 1) * 4));
    MXH_TRY(hipMalloc(&tmp.p, scanBytes + 256));
    MXH_TRY(hipMalloc(&I.entryBlock.p, n * 4 + 4));
    MXH_TRY(hipMemsetAsync(I.entryBlock.p, 0xff, n * 4 + 4, s));
    hipLaunchKernelGGL(block_heads_kernel, grid((long long)n + 1), dim3(kBlock), 0, s, (const unsigned long long *)I.blkKey.p, I.nDD, 48, I.cols,
                       selHead.as<int>());
    MXH_TRY(hipGetLastError());
    MXH_TRY(rocprim::exclusive_scan(tmp.p, scanBytes, (const int *)selHead.p, blockId.as<int>(), 0, n + 1, rocprim::plus<int>(), s));
    int nBlk = 0;
    MXH_TRY(hipMemcpyAsync(&nBlk, blockId.as<int>() + n, 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    if (nBlk <= 0) return MX_OK;
    const size_t nbk = (size_t)nBlk;
    MXH_TRY(hipMalloc(&I.blkBr.p, nbk * 4 + 4));
    MXH_TRY(hipMalloc(&I.blkBc.p, nbk * 4 + 4));
    MXH_TRY(hipMalloc(&head.p, nbk * 4 + 4));
    MXH_TRY(hipMalloc(&I.blkChunkIdIncl.p, nbk * 4 + 4));
    hipLaunchKernelGGL(block_records_kernel, grid(I.nDD), dim3(kBlock), 0, s, (const unsigned long long *)I.blkKey.p, (const int *)I.blkPay.p,
                       (const int *)selHead.p, (const int *)blockId.p, I.nDD, I.blkBr.as<int>(), I.blkBc.as<int>(), I.entryBlock.as<int>());
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(block_chunk_heads_kernel, grid(nBlk), dim3(kBlock), 0, s, (const int *)I.blkBr.p, nBlk, head.as<int>());
    MXH_TRY(hipGetLastError());
    // (nBlk <= nDD: the scan's temporary storage is large enough)
    MXH_TRY(rocprim::inclusive_scan(tmp.p, scanBytes, (const int *)head.p, I.blkChunkIdIncl.as<int>(), nbk, rocprim::plus<int>(), s));
    int nChunks = 0;
    MXH_TRY(hipMemcpyAsync(&nChunks, I.blkChunkIdIncl.as<int>() + (nbk - 1), 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    MXH_TRY(hipMalloc(&I.blkChunkStart.p, ((size_t)nChunks + 1) * 4));
    MXH_TRY(hipMalloc(&I.blkChunkBr.p, ((size_t)nChunks + 1) * 4));
    MXH_TRY(hipMalloc(&nb.p, ((size_t)nChunks + 1) * 4));
    hipLaunchKernelGGL(block_chunk_starts_kernel, grid(nBlk), dim3(kBlock), 0, s, (const int *)head.p, (const int *)I.blkChunkIdIncl.p,
                       (const int *)I.blkBr.p, nBlk, I.blkChunkStart.as<int>(), I.blkChunkBr.as<int>());
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(block_chunk_sizes_kernel, grid(nChunks), dim3(kBlock), 0, s, (const int *)I.blkChunkStart.p, nChunks, nb.as<int>());
    MXH_TRY(hipGetLastError());
    blocks.assign((size_t)nChunks, 0);
    blockRows.assign((size_t)nChunks, 0);
    MXH_TRY(hipMemcpyAsync(blocks.data(), nb.p, (size_t)nChunks * 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipMemcpyAsync(blockRows.data(), I.blkChunkBr.p, (size_t)nChunks * 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    I.nBlk = nBlk;
    I.nBlkChunks = nChunks;
    return MX_OK;
}

int HybridDevice::block_layout(const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0, const std::vector<int> &waveDesc,
                               long long totalBlocks, DeviceTiles &T)
{
    using namespace mxh;
    if (!impl || impl->nBlkChunks <= 0 || (int)chunkBlock0.size() != impl->nBlkChunks) return MX_ERR_ARG;
    Impl &I = *impl;
    hipStream_t s = I.s;
    const int steps = (int)(stepDesc.size() / 10);
    Buf dDesc, dBlock0;
    MXH_TRY(hipMalloc(&dDesc.p, stepDesc.size() * 4 + 4));
    MXH_TRY(hipMalloc(&dBlock0.p, chunkBlock0.size() * 4 + 4));
    MXH_TRY(hipMemcpyAsync(dDesc.p, stepDesc.data(), stepDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMemcpyAsync(dBlock0.p, chunkBlock0.data(), chunkBlock0.size() * 4, hipMemcpyHostToDevice, s));
    const size_t nWave = waveDesc.size() + 64, nHdr = (size_t)steps * kTileHdr + 256, nAtox = (size_t)steps * 64 + 256,
                 valBytes = (size_t)totalBlocks * 64 * 8 + 8192;
    MXH_TRY(hipMalloc((void **)&T.waveDesc, nWave * 4));
    MXH_TRY(hipMemsetAsync(T.waveDesc, 0, nWave * 4, s));
    MXH_TRY(hipMemcpyAsync(T.waveDesc, waveDesc.data(), waveDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMalloc((void **)&T.hdr, nHdr * 4));
    MXH_TRY(hipMemsetAsync(T.hdr, 0, nHdr * 4, s));
    MXH_TRY(hipMalloc((void **)&T.atox, nAtox * 4));
    MXH_TRY(hipMemsetAsync(T.atox, 0, nAtox * 4, s));
    MXH_TRY(hipMalloc(&T.tcVal, valBytes));
    MXH_TRY(hipMemsetAsync(T.tcVal, 0, valBytes, s));
    hipLaunchKernelGGL(block_steps_kernel, dim3(steps), dim3(64), 0, s, (const int *)dDesc.p, (const int *)I.blkChunkStart.p,
                       (const int *)I.blkChunkBr.p, (const int *)I.blkBc.p, I.rows, steps, T.hdr, T.atox);
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(block_values_kernel, grid(I.nDD), dim3(kBlock), 0, s, (const int *)I.entryBlock.p, (const int *)I.blkChunkIdIncl.p,
                       (const int *)I.blkChunkStart.p, (const int *)dBlock0.p, (const int *)I.ddp, (const int *)I.ddc, (const double *)I.ddv,
                       (const int *)I.dc, (const int *)I.dr, I.dRows, I.nDD, (double *)T.tcVal);
    MXH_TRY(hipGetLastError());
    MXH_TRY(hipStreamSynchronize(s));
    return MX_OK;
}

// The chunks of the general tile form: the fragments that pass the gate on what the strips leave,
// their columns in use sorted by the caller's ids inside every chunk.  blocks: per chunk with at
// least one such column, in chunk order, the number of blocks of fragK columns it needs.
int HybridDevice::tile_chunks(bool keepStrips, std::vector<int> &blocks)
{
    using namespace mxh;
    blocks.clear();
    if (!impl) return MX_ERR_ARG;
    Impl &I = *impl;
    hipStream_t s = I.s;
    const int K = mx::frag_k(I.dtype), chunkNum = I.T.chunkNum, nFrags = I.T.totalTcFrags;
    I.nSel = 0;
    if (chunkNum <= 0 || nFrags <= 0) return MX_OK;
    const unsigned char *taken = keepStrips && I.nChunks > 0 ? (const unsigned char *)I.taken.p : nullptr;
    const size_t nKey = (size_t)nFrags * K;
    Buf keyIn, keyOut, payIn, payOut, sortTmp, isSel, scanTmp, selNb;
    size_t sortBytes = 0, scanBytes = 0;
    MXH_TRY(rocprim::radix_sort_pairs(nullptr, sortBytes, (const unsigned long long *)nullptr, (unsigned long long *)nullptr,
                                      (const int *)nullptr, (int *)nullptr, nKey, 0u, 64u, s));
    MXH_TRY(rocprim::exclusive_scan(nullptr, scanBytes, (const int *)nullptr, (int *)nullptr, 0, (size_t)chunkNum + 1, rocprim::plus<int>(), s));
    MXH_TRY(hipMalloc(&I.selFrag.p, (size_t)nFrags + 4));
    MXH_TRY(hipMalloc(&I.usedCols.p, (size_t)chunkNum * 4 + 4));
    MXH_TRY(hipMalloc(&I.nrefs.p, ((size_t)chunkNum + 1) * 4));
    MXH_TRY(hipMalloc(&I.refStart.p, ((size_t)chunkNum + 1) * 4));
    MXH_TRY(hipMalloc(&I.selPos.p, ((size_t)chunkNum + 1) * 4));
    MXH_TRY(hipMalloc(&I.where.p, nKey * 4 + 4));
    MXH_TRY(hipMalloc(&keyIn.p, nKey * 8));
    MXH_TRY(hipMalloc(&keyOut.p, nKey * 8));
    MXH_TRY(hipMalloc(&payIn.p, nKey * 4));
    MXH_TRY(hipMalloc(&payOut.p, nKey * 4));
    MXH_TRY(hipMalloc(&sortTmp.p, sortBytes + 256));
    MXH_TRY(hipMalloc(&scanTmp.p, scanBytes + 256));
    MXH_TRY(hipMalloc(&isSel.p, ((size_t)chunkNum + 1) * 4));
    MXH_TRY(hipMemsetAsync(I.nrefs.p, 0, ((size_t)chunkNum + 1) * 4, s));
    MXH_TRY(hipMemsetAsync(I.where.p, 0xff, nKey * 4 + 4, s));
    if (I.dtype == MX_F64)
        hipLaunchKernelGGL(chunk_refs_kernel<true>, grid(chunkNum), dim3(kBlock), 0, s, (const int *)I.T.chunkPtr, (const void *)I.T.fragBit,
                           (const int *)I.T.sparse_AToX_index, (const int *)I.dc, taken, chunkNum, I.dRows, I.minVals,
                           I.selFrag.as<unsigned char>(), keyIn.as<unsigned long long>(), I.nrefs.as<int>(), I.usedCols.as<int>());
    else
        hipLaunchKernelGGL(chunk_refs_kernel<false>, grid(chunkNum), dim3(kBlock), 0, s, (const int *)I.T.chunkPtr, (const void *)I.T.fragBit,
                           (const int *)I.T.sparse_AToX_index, (const int *)I.dc, taken, chunkNum, I.dRows, I.minVals,
                           I.selFrag.as<unsigned char>(), keyIn.as<unsigned long long>(), I.nrefs.as<int>(), I.usedCols.as<int>());
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(iota_kernel, grid((long long)nKey), dim3(kBlock), 0, s, payIn.as<int>(), (int)nKey);
    MXH_TRY(hipGetLastError());
    MXH_TRY(rocprim::radix_sort_pairs(sortTmp.p, sortBytes, (const unsigned long long *)keyIn.p, keyOut.as<unsigned long long>(),
                                      (const int *)payIn.p, payOut.as<int>(), nKey, 0u, 64u, s));
    MXH_TRY(rocprim::exclusive_scan(scanTmp.p, scanBytes, (const int *)I.nrefs.p, I.refStart.as<int>(), 0, (size_t)chunkNum + 1,
                                    rocprim::plus<int>(), s));
    hipLaunchKernelGGL(chunk_blocks_kernel, grid((long long)chunkNum + 1), dim3(kBlock), 0, s, (const int *)I.nrefs.p, chunkNum, K,
                       isSel.as<int>());
    MXH_TRY(hipGetLastError());
    MXH_TRY(rocprim::exclusive_scan(scanTmp.p, scanBytes, (const int *)isSel.p, I.selPos.as<int>(), 0, (size_t)chunkNum + 1,
                                    rocprim::plus<int>(), s));
    int nRefs = 0, nSel = 0;
    MXH_TRY(hipMemcpyAsync(&nRefs, I.refStart.as<int>() + chunkNum, 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipMemcpyAsync(&nSel, I.selPos.as<int>() + chunkNum, 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    if (nSel <= 0 || nRefs <= 0) return MX_OK;
    MXH_TRY(hipMalloc(&I.sortedCol.p, (size_t)nRefs * 4 + 4));
    MXH_TRY(hipMalloc(&I.selW.p, (size_t)nSel * 4 + 4));
    MXH_TRY(hipMalloc(&selNb.p, (size_t)nSel * 4 + 4));
    hipLaunchKernelGGL(ref_places_kernel, grid(nRefs), dim3(kBlock), 0, s, (const unsigned long long *)keyOut.p, (const int *)payOut.p,
                       (const int *)I.refStart.p, nRefs, I.sortedCol.as<int>(), I.where.as<int>());
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(sel_chunks_kernel, grid(chunkNum), dim3(kBlock), 0, s, (const int *)I.nrefs.p, (const int *)isSel.p,
                       (const int *)I.selPos.p, chunkNum, K, I.selW.as<int>(), selNb.as<int>());
    MXH_TRY(hipGetLastError());
    blocks.assign((size_t)nSel, 0);
    MXH_TRY(hipMemcpyAsync(blocks.data(), selNb.p, (size_t)nSel * 4, hipMemcpyDeviceToHost, s));
    MXH_TRY(hipStreamSynchronize(s));
    I.nSel = nSel;
    return MX_OK;
}

// The general tile layout: headers and column ids of every step, and the (zeroed) values, which
// csr_part fills as it walks the rows of A_dd -- so this comes first.
int HybridDevice::tile_layout(bool keepStrips, const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0,
                              const std::vector<int> &waveDesc, long long totalBlocks, DeviceTiles &T)
{
    using namespace mxh;
    if (!impl || impl->nSel <= 0 || (int)chunkBlock0.size() != impl->nSel) return MX_ERR_ARG;
    Impl &I = *impl;
    hipStream_t s = I.s;
    const int steps = (int)(stepDesc.size() / 10), K = mx::frag_k(I.dtype);
    const size_t es = (size_t)mx::elem_size(I.dtype);
    const unsigned char *taken = keepStrips && I.nChunks > 0 ? (const unsigned char *)I.taken.p : nullptr;
    Buf dDesc;
    MXH_TRY(hipMalloc(&dDesc.p, stepDesc.size() * 4 + 4));
    MXH_TRY(hipMemcpyAsync(dDesc.p, stepDesc.data(), stepDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMalloc(&I.tileBlock0.p, ((size_t)I.nSel + 1) * 4));
    MXH_TRY(hipMemsetAsync(I.tileBlock0.p, 0, ((size_t)I.nSel + 1) * 4, s));
    MXH_TRY(hipMemcpyAsync(I.tileBlock0.p, chunkBlock0.data(), chunkBlock0.size() * 4, hipMemcpyHostToDevice, s));
    const size_t nWave = waveDesc.size() + 64, nHdr = (size_t)steps * kTileHdr + 256, nAtox = (size_t)steps * 64 + 256,
                 valBytes = (size_t)totalBlocks * 8 * K * es + 8192;
    MXH_TRY(hipMalloc((void **)&T.waveDesc, nWave * 4));
    MXH_TRY(hipMemsetAsync(T.waveDesc, 0, nWave * 4, s));
    MXH_TRY(hipMemcpyAsync(T.waveDesc, waveDesc.data(), waveDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMalloc((void **)&T.hdr, nHdr * 4));
    MXH_TRY(hipMemsetAsync(T.hdr, 0, nHdr * 4, s));
    MXH_TRY(hipMalloc((void **)&T.atox, nAtox * 4));
    MXH_TRY(hipMemsetAsync(T.atox, 0, nAtox * 4, s));
    MXH_TRY(hipMalloc(&T.tcVal, valBytes));
    MXH_TRY(hipMemsetAsync(T.tcVal, 0, valBytes, s));
    if (I.dtype == MX_F64)
        hipLaunchKernelGGL(tile_steps_kernel<true>, dim3(steps), dim3(64), 0, s, (const int *)dDesc.p, (const int *)I.selW.p,
                           (const int *)I.nrefs.p, (const int *)I.refStart.p, (const int *)I.sortedCol.p, taken, (const int *)I.dr, I.dRows,
                           steps, T.hdr, T.atox);
    else
        hipLaunchKernelGGL(tile_steps_kernel<false>, dim3(steps), dim3(64), 0, s, (const int *)dDesc.p, (const int *)I.selW.p,
                           (const int *)I.nrefs.p, (const int *)I.refStart.p, (const int *)I.sortedCol.p, taken, (const int *)I.dr, I.dRows,
                           steps, T.hdr, T.atox);
    MXH_TRY(hipGetLastError());
    MXH_TRY(hipStreamSynchronize(s));
    I.tileVal = T.tcVal;
    return MX_OK;
}

int HybridDevice::strip_layout(const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0, const std::vector<int> &waveDesc,
                               long long totalBlocks, DeviceTiles &T)
{
    using namespace mxh;
    if (!impl || impl->dtype != MX_F16 || impl->nChunks <= 0 || (int)chunkBlock0.size() != impl->nChunks) return MX_ERR_ARG;
    Impl &I = *impl;
    hipStream_t s = I.s;
    const int steps = (int)(stepDesc.size() / 8);
    Buf dDesc, dBlock0;
    MXH_TRY(hipMalloc(&dDesc.p, stepDesc.size() * 4 + 4));
    MXH_TRY(hipMalloc(&dBlock0.p, chunkBlock0.size() * 4 + 4));
    MXH_TRY(hipMemcpyAsync(dDesc.p, stepDesc.data(), stepDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMemcpyAsync(dBlock0.p, chunkBlock0.data(), chunkBlock0.size() * 4, hipMemcpyHostToDevice, s));
    // (sizes and zero padding as the host route uploads them)
    const size_t nWave = waveDesc.size() + 64, nHdr = (size_t)steps * kTileHdr + 256, nAtox = (size_t)steps * 64 + 256,
                 valBytes = (size_t)totalBlocks * 64 * 2 + 8192;
    MXH_TRY(hipMalloc((void **)&T.waveDesc, nWave * 4));
    MXH_TRY(hipMemsetAsync(T.waveDesc, 0, nWave * 4, s));
    MXH_TRY(hipMemcpyAsync(T.waveDesc, waveDesc.data(), waveDesc.size() * 4, hipMemcpyHostToDevice, s));
    MXH_TRY(hipMalloc((void **)&T.hdr, nHdr * 4));
    MXH_TRY(hipMemsetAsync(T.hdr, 0, nHdr * 4, s));
    MXH_TRY(hipMalloc((void **)&T.atox, nAtox * 4));
    MXH_TRY(hipMemsetAsync(T.atox, 0, nAtox * 4, s));
    MXH_TRY(hipMalloc(&T.tcVal, valBytes));
    MXH_TRY(hipMemsetAsync(T.tcVal, 0, valBytes, s));
    hipLaunchKernelGGL(strip_steps_kernel, dim3(steps), dim3(64), 0, s, (const int *)dDesc.p, (const int *)I.chunkRows.p,
                       (const int *)I.chunkKey.p, steps, T.hdr, T.atox);
    MXH_TRY(hipGetLastError());
    hipLaunchKernelGGL(strip_values_kernel, grid(I.nCand), dim3(kBlock), 0, s, (const int *)I.perm.p, (const int *)I.candRow.p,
                       (const int *)I.memberChunk.p, (const int *)I.runIdIncl.p, (const int *)I.runStart.p, (const int *)I.chunkKey.p,
                       (const int *)I.chunkNb.p, (const int *)dBlock0.p, (const int *)I.ddp, (const int *)I.ddc,
                       (const unsigned short *)I.ddv, (const int *)I.dc, I.nCand, (unsigned short *)T.tcVal);
    MXH_TRY(hipGetLastError());
    MXH_TRY(hipStreamSynchronize(s));
    return MX_OK;
}

}  // namespace mx
