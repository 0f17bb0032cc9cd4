// gfx950 kernels of the hybrid SpMV and their launchers.
//
//   csr_rows_kernel    residual / plain CSR part, x gathered from memory (stands in for
//                      cdspmv_kernel, src/spmv_kernel/cdSpMV.cu:244-392).
//   csr_slice_kernel   the same part with a slice of x resident in LDS, for matrices with
//   slice_combine_kernel   scattered columns: rows are cut at the slice borders into "virtual
//                      rows", the first kernel sums those, the second adds up each row's.
//   tile_kernel<double>    8x4 tiles through v_mfma_f64_16x16x4_f64 (stands in for
//                      tcspmv_kernel_fp64, src/spmv_kernel/du_tcSpMV_fp64.cu:81-160).
//   tile_kernel<_Float16>  8x8 tiles through v_mfma_f32_16x16x32_f16, f32 accumulation
//                      (stands in for tcspmv_kernel_fp16_v2, du_tcSpMV_fp16_v2.cu:4-110).
//
// Row ownership: every output row is written by exactly one lane of one workgroup in each
// kernel, so there are no atomics anywhere; the tile kernel runs after the CSR kernel on the
// same stream and adds its rows on top with a plain read-modify-write.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <type_traits>
#include <vector>

#include "mx_device.h"

namespace mxk {

typedef double v4f64 __attribute__((ext_vector_type(4)));
typedef float v4f32 __attribute__((ext_vector_type(4)));
typedef _Float16 v8f16 __attribute__((ext_vector_type(8)));
typedef int v4i32 __attribute__((ext_vector_type(4)));
typedef double v2f64 __attribute__((ext_vector_type(2)));
typedef int v2i32 __attribute__((ext_vector_type(2)));
typedef v4i32 v4i32u __attribute__((aligned(2)));  // 16 bytes at the alignment of a binary16 element

constexpr int kBlock = 256;  // 4 wave64 per workgroup
using mx::kSliceBytes;
using mx::kSliceThreads;
using mx::kSliceWaves;

// Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its own L2.
// Re-map so that every XCD walks one contiguous range of logical blocks: neighbouring rows
// (and the x entries they share) then live in a single L2 instead of all eight.
__device__ __forceinline__ int xcd_contiguous_block(int bid, int nb)
{
    const int q = nb >> 3, rem = nb & 7;
    const int xcd = bid & 7, idx = bid >> 3;
    return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

// ---- cross-lane moves -------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp(double v)
{
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_update_dpp(0, (int)b, CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, (int)(b >> 32), CTRL, 0xf, 0xf, false);
    return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)(unsigned)lo);
}
__device__ __forceinline__ float swizzle_x16(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
}
__device__ __forceinline__ double swizzle_x16(double v)
{
    const long long b = __builtin_bit_cast(long long, v);
    const int lo = __builtin_amdgcn_ds_swizzle((int)b, 0x401F);
    const int hi = __builtin_amdgcn_ds_swizzle((int)(b >> 32), 0x401F);
    return __builtin_bit_cast(double, ((long long)hi << 32) | (long long)(unsigned)lo);
}

// Sum over aligned groups of W lanes (W a power of two <= 64); every lane of the group ends
// up with the total.  Steps 1,2 are quad permutes, 4 and 8 row mirrors (DPP), 16 a
// ds_swizzle lane-xor, 32 a bpermute.
template <int W, typename T>
__device__ __forceinline__ T group_sum(T v)
{
    if (W >= 2) v += dpp<0xB1>(v);   // quad_perm [1,0,3,2]
    if (W >= 4) v += dpp<0x4E>(v);   // quad_perm [2,3,0,1]
    if (W >= 8) v += dpp<0x141>(v);  // row_half_mirror
    if (W >= 16) v += dpp<0x140>(v); // row_mirror
    if (W >= 32) v += swizzle_x16(v);
    if (W >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// ---- CSR part ---------------------------------------------------------------------------
template <typename VT>
struct Acc;
template <>
struct Acc<double> {
    typedef double type;
};
template <>
struct Acc<_Float16> {
    typedef float type;
};

// One wave's share of a tile: 64*NPT consecutive entries starting at the 16-byte aligned
// position `pos` (wave-uniform).  wave_stream moves indices and values with 128-bit loads into
// the wave's own LDS region (in entry order); wave_gather reads them back transposed, so that
// in every x gather lane l holds entry 64j+l: neighbouring lanes then ask for neighbouring
// entries of a row, whose sorted columns share cache lines, and the address unit serves them
// together instead of one lane per cycle.  It returns the products
// p[j] = val[pos+64j+l] * x[col[pos+64j+l]].
//   cs, vs : this wave's LDS regions, 64*NPT ints / accumulators.
//   C16   : the column ids are stored as 16-bit offsets from x (the caller has moved x to the
//           workgroup's lowest column); lim = the largest offset that is still inside x
//   DICT  : the matrix has at most 256 distinct values; `val` then points at one byte per entry,
//           an index into `dict` (the distinct values as accumulators, in LDS)
template <typename VT, int NPT, bool C16, bool DICT = false>
__device__ __forceinline__ void wave_stream(const void *__restrict__ colv, const VT *__restrict__ val, int pos, int lane,
                                            int *cs, typename Acc<VT>::type *vs,
                                            const typename Acc<VT>::type *dict = nullptr)
{
    // every load instruction reads one contiguous stretch (lane l right after lane l-1): a
    // streamed line is then asked for once, not once per instruction that touches a piece of it
    if constexpr (C16) {
        const unsigned short *col = (const unsigned short *)colv;
        unsigned short *c16 = (unsigned short *)cs;
        if constexpr (NPT == 4) {
            *(v2i32 *)(c16 + 4 * lane) = __builtin_nontemporal_load((const v2i32 *)(col + pos + 4 * lane));
        } else {
#pragma unroll
            for (int q = 0; q < NPT / 8; ++q) {
                const int e = 512 * q + 8 * lane;
                *(v4i32 *)(c16 + e) = __builtin_nontemporal_load((const v4i32 *)(col + pos + e));
            }
        }
    } else {
        const int *col = (const int *)colv;
#pragma unroll
        for (int q = 0; q < NPT / 4; ++q) {
            const int e = 256 * q + 4 * lane;
            *(v4i32 *)(cs + e) = __builtin_nontemporal_load((const v4i32 *)(col + pos + e));
        }
    }
    if constexpr (DICT) {
        // lane l takes the NPT codes NPT*l .. NPT*l+NPT-1 of the wave's stretch: one load of NPT bytes
        static_assert(NPT == 4 || NPT == 8 || NPT == 16, "codes come in 4, 8 or 16 bytes per lane");
        const unsigned char *codes = (const unsigned char *)val + pos + NPT * lane;
        unsigned w[NPT / 4];
        if constexpr (NPT == 4) {
            w[0] = __builtin_nontemporal_load((const unsigned *)codes);
        } else if constexpr (NPT == 8) {
            const v2i32 t = __builtin_nontemporal_load((const v2i32 *)codes);
            w[0] = (unsigned)t.x, w[1] = (unsigned)t.y;
        } else {
            const v4i32 t = __builtin_nontemporal_load((const v4i32 *)codes);
            w[0] = (unsigned)t.x, w[1] = (unsigned)t.y, w[2] = (unsigned)t.z, w[3] = (unsigned)t.w;
        }
#pragma unroll
        for (int k = 0; k < NPT; ++k) vs[NPT * lane + k] = dict[(w[k / 4] >> (8 * (k % 4))) & 255u];
    } else if constexpr (sizeof(VT) == 8) {
#pragma unroll
        for (int q = 0; q < NPT / 2; ++q) {
            const int e = 128 * q + 2 * lane;
            *(v2f64 *)(vs + e) = __builtin_nontemporal_load((const v2f64 *)(val + pos + e));
        }
    } else {
#pragma unroll
        for (int q = 0; q < NPT / 8; ++q) {
            const int e = 512 * q + 8 * lane;
            const v8f16 hv = __builtin_nontemporal_load((const v8f16 *)(val + pos + e));
            v4f32 fa, fb;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                fa[j] = (float)hv[j];
                fb[j] = (float)hv[4 + j];
            }
            *(v4f32 *)(vs + e) = fa;
            *(v4f32 *)(vs + e + 4) = fb;
        }
    }
}

template <typename VT, int NPT, bool C16>
__device__ __forceinline__ void wave_gather(const VT *__restrict__ x, int lane, const int *cs,
                                            const typename Acc<VT>::type *vs, typename Acc<VT>::type (&p)[NPT], int lim)
{
    typedef typename Acc<VT>::type AT;
    __builtin_amdgcn_wave_barrier();
    AT xv[NPT];
    if constexpr (C16) {
        const unsigned short *c16 = (const unsigned short *)cs;
#pragma unroll
        // entries of the neighbouring workgroups share the wave's aligned loads; their offsets
        // belong to another base, so keep them inside x (their products are dropped later)
        for (int j = 0; j < NPT; ++j) xv[j] = (AT)x[min((int)c16[64 * j + lane], lim)];
    } else {
#pragma unroll
        for (int j = 0; j < NPT; ++j) xv[j] = (AT)x[cs[64 * j + lane]];
    }
#pragma unroll
    for (int j = 0; j < NPT; ++j) p[j] = vs[64 * j + lane] * xv[j];
}

// Sums the rows of one tile out of LDS: W lanes per row, `rowOff` holds the rows' start
// offsets inside the tile (nrows+1 entries).
template <typename VT, int W>
__device__ __forceinline__ void reduce_rows(const typename Acc<VT>::type *prod, const unsigned short *rowOff, int r0,
                                            int nrows, VT *__restrict__ y, int accumulate, int tid,
                                            typename Acc<VT>::type *__restrict__ ywide)
{
    typedef typename Acc<VT>::type AT;
    constexpr int rowsPerPass = kBlock / W;
    const int g = tid / W, l = tid % W;
    for (int rr = g; rr < nrows; rr += rowsPerPass) {
        const int a = rowOff[rr], b = rowOff[rr + 1];
        AT s = 0;
        for (int i = a + l; i < b; i += W) s += prod[i];
        s = group_sum<W>(s);
        if (l == 0) {
            if (accumulate) s += (AT)y[r0 + rr];
            y[r0 + rr] = (VT)s;
            if (ywide) ywide[r0 + rr] = s;
        }
    }
}

// The same sums for tiles whose rows differ a lot in length (a few long rows would keep their
// W lanes busy while all others wait).  Every lane owns NPT consecutive products and walks
// them once: `head` (LDS, one int per entry) holds row+1 where a row starts and 0 elsewhere.
// A row that starts and ends inside a lane's stretch is stored right away; what is left is,
// per lane, the sum before its first row start (it belongs to a row opened by an earlier lane)
// and the sum after its last one (a row that goes on in later lanes).  Those are stitched
// together by a segmented scan over the 256 lanes (shuffles inside a wave, one LDS exchange
// between the waves), and the lane in which a row starts closes the row that was open before.
struct ScanItem {
    int f;  // a row starts in this lane (or in one that the item has absorbed)
    int r;  // row open at the end
};
template <typename VT, int NPT>
__device__ __forceinline__ void reduce_scan(const typename Acc<VT>::type *prod, const int *head, const unsigned short *rowOff,
                                            int r0, int nrows, VT *__restrict__ y, int accumulate, int tid,
                                            typename Acc<VT>::type *carryV, int *carryF, int *carryR,
                                            typename Acc<VT>::type *__restrict__ ywide)
{
    typedef typename Acc<VT>::type AT;
    const int lane = tid & 63, wave = tid >> 6;
    auto store = [&](int row, AT v) {
        if (accumulate) v += (AT)y[r0 + row];
        y[r0 + row] = (VT)v;
        if (ywide) ywide[r0 + row] = v;
    };
    AT v[NPT];
    int h[NPT];
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        v[j] = prod[NPT * tid + j];
        h[j] = head[NPT * tid + j];
    }
    AT before = 0, run = 0;  // before: sum ahead of the first row start
    int cur = -1;            // row open right now, -1 = the one inherited from earlier lanes
    int f = 0;
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        if (h[j] != 0) {
            if (f) store(cur, run);
            else before = run;
            f = 1;
            cur = h[j] - 1;
            run = 0;
        }
        run += v[j];
    }
    if (!f) before = run;
    // inclusive segmented scan of (f, value, row): value = sum since the last row start
    AT sv = run;  // with no start in the lane, run == before == the lane's whole sum
    int sf = f, sr = cur;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const AT pv = __shfl_up(sv, d, 64);
        const int pf = __shfl_up(sf, d, 64), pr = __shfl_up(sr, d, 64);
        if (lane >= d) {
            if (!sf) {
                sv += pv;
                sr = pr;
            }
            sf |= pf;
        }
    }
    if (lane == 63) {
        carryV[wave] = sv;
        carryF[wave] = sf;
        carryR[wave] = sr;
    }
    // what the lane before this one ends with, inside the wave
    AT ev = __shfl_up(sv, 1, 64);
    int ef = __shfl_up(sf, 1, 64), er = __shfl_up(sr, 1, 64);
    if (lane == 0) {
        ev = 0;
        ef = 0;
        er = -1;
    }
    __syncthreads();
    // fold in the waves before this one
    AT cv = 0;
    int cf = 0, cr = -1;
    for (int w = 0; w < wave; ++w) {
        if (carryF[w]) {
            cv = carryV[w];
            cr = carryR[w];
            cf = 1;
        } else {
            cv += carryV[w];
        }
    }
    if (!ef) {
        ev += cv;
        er = cr;
    }
    (void)cf;
    // a lane in which a row starts closes the row that was open before it
    if (f && er >= 0) store(er, ev + before);
    // the last lane closes the row that is still open at the end of the tile
    if (tid == kBlock - 1) {
        AT tv = sv;
        int tr = sr;
        if (!sf) {
            tv += cv;
            tr = cr;
        }
        if (tr >= 0) store(tr, tv);
    }
    // rows without entries
    for (int rr = tid; rr < nrows; rr += kBlock)
        if (rowOff[rr] == rowOff[rr + 1]) store(rr, (AT)0);
}

// One workgroup owns the whole rows [r0, r1) named by its descriptor {r0, r1, p0, p1}
// (p = positions of the first and one-past-last entry).  The host packs rows so that their
// entries fit one tile of kBlock*NPT products and at most kBlock*NPT rows (a single longer
// row gets a workgroup of its own).  Phase 1 issues the loads of the rows' start offsets and
// lets each wave form the products of its quarter of the tile (wave_products), parked in
// LDS.  Phase 2 sums each row from LDS with W lanes per row, W picked from the mean row length
// of the tile; it touches global memory only to store y.  A row longer than a tile is swept
// tile by tile with the same loads, each lane keeping a running sum.  col/val are padded by
// the host so that aligned 128-bit loads may run past the end.  With C16 the column ids are
// 16-bit offsets from colBase[workgroup] (the host uses this form when the columns of every
// workgroup span fewer than 65536), which takes a third off the bytes of an FP16 entry and
// a sixth off an FP64 one.
// With SCAN the rows of a tile are summed by reduce_scan instead of reduce_rows (the host asks
// for it when row lengths vary a lot).
// With DICT the values are one byte per entry, indices into the matrix's at most 256 distinct
// values (`dictG`, copied to LDS first): a stencil or a graph matrix then streams 3 bytes per
// entry instead of 10.
// `ywide` (optional): the sums as accumulators, unrounded, for a kernel that adds to these rows
// afterwards (binary16 plans with tiles on shared rows: y is then rounded once, at the end).
template <typename VT, int NPT, bool XCD, bool C16, bool SCAN, bool DICT = false>
__global__ __launch_bounds__(kBlock) void csr_rows_kernel(const int *__restrict__ rowPtr, const void *__restrict__ col,
                                                          const VT *__restrict__ val, const VT *__restrict__ xfull,
                                                          VT *__restrict__ y, const int4 *__restrict__ blockDesc,
                                                          const int *__restrict__ colBase, int xcols, int accumulate,
                                                          const VT *__restrict__ dictG,
                                                          typename Acc<VT>::type *__restrict__ ywide)
{
    typedef typename Acc<VT>::type AT;
    __shared__ AT dictL[DICT ? 256 : 1];
    constexpr int TILE = kBlock * NPT;
    constexpr int WTILE = 64 * NPT;
    __shared__ __attribute__((aligned(16))) AT prod[TILE];
    __shared__ __attribute__((aligned(16))) int cols[TILE];
    __shared__ unsigned short rowOff[TILE + 2];  // offsets inside the tile fit 16 bits
    __shared__ AT wsum[kBlock / 64];
    __shared__ int wflag[kBlock / 64], wrow[kBlock / 64];

    const int b = XCD ? xcd_contiguous_block(blockIdx.x, gridDim.x) : (int)blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int4 d = blockDesc[b];
    const int r0 = d.x, r1 = d.y, p0 = d.z, p1 = d.w;
    const int nrows = r1 - r0;
    if (nrows <= 0) return;
    if constexpr (DICT) {
        dictL[tid] = (AT)dictG[tid];  // kBlock == 256 entries (the host pads the dictionary)
        __syncthreads();
    }
    const int cb = C16 ? colBase[b] : 0;
    const VT *x = xfull + cb;
    const int lim = xcols - 1 - cb;
    const int base = p0 & ~(NPT - 1);
    int *cs = cols + wave * WTILE;
    AT *vs = prod + wave * WTILE;
    if (p1 - base <= TILE) {
        // row offsets: lane t takes rows t, t+256, ... (at most NPT+1 of them)
        int ro[NPT + 1];
#pragma unroll
        for (int k = 0; k <= NPT; ++k) {
            const int rr = tid + k * kBlock;
            ro[k] = rr <= nrows ? rowPtr[r0 + rr] : 0;
        }
        const bool active = base + wave * WTILE < p1;
        if (active) wave_stream<VT, NPT, C16, DICT>(col, val, base + wave * WTILE, lane, cs, vs, dictL);
        if (active) {
            AT p[NPT];
            wave_gather<VT, NPT, C16>(x, lane, cs, vs, p, lim);
#pragma unroll
            for (int j = 0; j < NPT; ++j) {
                // reduce_scan walks the whole tile: what is not this workgroup's must be zero
                const int e = base + wave * WTILE + 64 * j + lane;
                vs[64 * j + lane] = (!SCAN || (e >= p0 && e < p1)) ? p[j] : (AT)0;
            }
        } else if (SCAN) {
#pragma unroll
            for (int j = 0; j < NPT; ++j) vs[64 * j + lane] = 0;
        }
        if constexpr (SCAN) {  // the wave's column ids are spent: its region becomes row-start marks
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int j = 0; j < NPT; ++j) cs[64 * j + lane] = 0;
        }
#pragma unroll
        for (int k = 0; k <= NPT; ++k) {
            const int rr = tid + k * kBlock;
            if (rr <= nrows) rowOff[rr] = (unsigned short)(ro[k] - base);
        }
        if constexpr (SCAN) {
            __syncthreads();
            // rows that start at the same entry are empty except the last of them: the highest wins
#pragma unroll
            for (int k = 0; k < NPT; ++k) {
                const int rr = tid + k * kBlock, pos = ro[k] - base;
                if (rr < nrows && pos < TILE) atomicMax(&cols[pos], rr + 1);
            }
        }
        __syncthreads();
        if constexpr (SCAN) {
            reduce_scan<VT, NPT>(prod, cols, rowOff, r0, nrows, y, accumulate, tid, wsum, wflag, wrow, ywide);
            return;
        }
        const int mean = (p1 - p0) / nrows;
        if (mean <= 2) reduce_rows<VT, 1>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else if (mean <= 4) reduce_rows<VT, 2>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else if (mean <= 8) reduce_rows<VT, 4>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else if (mean <= 16) reduce_rows<VT, 8>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else if (mean <= 32) reduce_rows<VT, 16>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else if (mean <= 64) reduce_rows<VT, 32>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
        else reduce_rows<VT, 64>(prod, rowOff, r0, nrows, y, accumulate, tid, ywide);
    } else {
        // a single row longer than one tile
        AT s = 0;
        for (int t0 = base + wave * WTILE; t0 < p1; t0 += TILE) {
            AT p[NPT];
            wave_stream<VT, NPT, C16, DICT>(col, val, t0, lane, cs, vs, dictL);
            wave_gather<VT, NPT, C16>(x, lane, cs, vs, p, lim);
#pragma unroll
            for (int j = 0; j < NPT; ++j) {
                const int e = t0 + 64 * j + lane;
                if (e >= p0 && e < p1) s += p[j];
            }
            __builtin_amdgcn_wave_barrier();
        }
        s = group_sum<64>(s);
        if (lane == 0) wsum[wave] = s;
        __syncthreads();
        if (tid == 0) {
            AT t = 0;
#pragma unroll
            for (int w = 0; w < kBlock / 64; ++w) t += wsum[w];
            if (accumulate) t += (AT)y[r0];
            y[r0] = (VT)t;
            if (ywide) ywide[r0] = t;
        }
    }
}

// ---- CSR part, x resident in LDS ----------------------------------------------------------
// For matrices whose x gathers are scattered, every gather from L2 moves a whole cache line
// for one value and a CU can take in only so many bytes per cycle: the kernel is bound by that
// instead of HBM.  Gathers from LDS cost next to nothing.  The columns are cut into S slices
// (a slice of x fits LDS); a workgroup -- one per CU -- copies one slice into LDS once and then
// streams entries whose columns fall into it.  Those are laid out as sliced ELL over "virtual
// rows" (see DeviceSlices): one virtual row per lane, one entry per lane per step, steps
// contiguous across the wave, so a lane sums its virtual row in a register with no cross-lane
// traffic at all, and at the end of a chunk of 64 virtual rows every lane stores one sum,
// the wave 64 consecutive ones.  A second kernel adds up the virtual rows of every matrix row.
// No atomics anywhere: every sum and every y has one owner.
// How the slice kernel reads its entries.  Streaming (non-temporal) loads leave the caches to x and the sums,
// and what they bring does not stay in the memory-side cache once other traffic asks for room there: right for a
// matrix that fits no cache, and for a product that finds the caches cold.  Plain loads let a matrix that fits
// the L2s or the memory-side cache live there from product to product.  The kind of load is a property of the
// instruction, so it is a kernel variant, chosen per plan (DeviceSlices::keep).
template <bool KEEP, typename T>
__device__ __forceinline__ T stream_load(const T *p)
{
    if constexpr (KEEP) return *p;
    else return __builtin_nontemporal_load(p);
}
template <typename VT>
struct SliceBatch;  // what one lane reads per batch: 8 column offsets, 8 values
template <>
struct SliceBatch<double> {
    v4i32 c;
    v2f64 v[4];
    template <bool KEEP>
    __device__ __forceinline__ void load(const unsigned short *ecol, const double *eval, size_t batch, int lane)
    {
        c = stream_load<KEEP>((const v4i32 *)(ecol + (batch * 64 + lane) * 8));
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = stream_load<KEEP>((const v2f64 *)(eval + batch * 512 + j * 128 + lane * 2));
    }
    // what entry k of the batch multiplies with: its x (a lane asks for all of a batch's before it uses
    // the first, so the LDS answers them in one go) ...
    __device__ __forceinline__ double gather(const double *xs, int k) const
    {
        const unsigned w = (unsigned)c[k >> 1];
        return (k & 1) ? xs[w >> 16] : xs[w & 0xffffu];
    }
    // ... and value * x
    __device__ __forceinline__ double term(int k, double xk) const { return ((k & 1) ? v[k >> 1].y : v[k >> 1].x) * xk; }
};
template <>
struct SliceBatch<_Float16> {
    v4i32 c, v;
    template <bool KEEP>
    __device__ __forceinline__ void load(const unsigned short *ecol, const _Float16 *eval, size_t batch, int lane)
    {
        c = stream_load<KEEP>((const v4i32 *)(ecol + (batch * 64 + lane) * 8));
        v = stream_load<KEEP>((const v4i32 *)(eval + (batch * 64 + lane) * 8));
    }
    __device__ __forceinline__ _Float16 gather(const _Float16 *xs, int k) const
    {
        const unsigned cw = (unsigned)c[k >> 1];
        return xs[(k & 1) ? cw >> 16 : cw & 0xffffu];
    }
    __device__ __forceinline__ float term(int k, _Float16 xk) const
    {
        const unsigned vw = (unsigned)v[k >> 1];
        const unsigned vi = (k & 1) ? vw >> 16 : vw & 0xffffu;
        return (float)__builtin_bit_cast(_Float16, (unsigned short)vi) * (float)xk;
    }
};
// The same with a value dictionary: a byte per entry that names one of at most 256 distinct
// values (kept as accumulators in LDS) in place of the value itself.
template <typename VT>
struct SliceBatchDict {
    typedef typename Acc<VT>::type AT;
    v4i32 c;
    v2i32 k;
    template <bool KEEP>
    __device__ __forceinline__ void load(const unsigned short *ecol, const unsigned char *ecode, size_t batch, int lane)
    {
        c = stream_load<KEEP>((const v4i32 *)(ecol + (batch * 64 + lane) * 8));
        k = stream_load<KEEP>((const v2i32 *)(ecode + (batch * 64 + lane) * 8));
    }
    __device__ __forceinline__ VT gather(const VT *xs, int j) const
    {
        const unsigned cw = (unsigned)c[j >> 1];
        return xs[(j & 1) ? cw >> 16 : cw & 0xffffu];
    }
    __device__ __forceinline__ AT value(const AT *dict, int j) const { return dict[((unsigned)k[j >> 2] >> (8 * (j & 3))) & 255u]; }
};
static_assert(mx::kSliceBatchEntries == 8, "SliceBatch holds 8 entries per lane");

// What a CU can take in from L2 or beyond is bounded in bytes (about 32 per cycle, whatever
// the width of the loads).  A lane keeps kSliceRing batches in flight: a stream no longer than
// the ring is loaded whole before anything else happens; a longer one runs a loop in which
// every consumed batch is reloaded with the batch one ring length ahead.
constexpr int kSliceRing = 6;

// What the one-launch form hands the kernel beyond the arguments of the slice kernel.
struct FusedArgs {
    void *y = nullptr;               // [rows] of the value type
    void *ywide = nullptr;           // optional accumulators, one per row
    const int *wgGroups = nullptr;   // [workgroups][2]
    const int *groupNeed = nullptr;  // [groups]
    int *groupCount = nullptr;       // [groups]
    const int *target = nullptr;     // [chunks * 64] where every virtual row puts its sum
    void *sums = nullptr;            // the sums, laid out for the one who adds
    unsigned *misplaced = nullptr;   // host memory: set when two workgroups of a launch took the same work
    unsigned *claim = nullptr;       // [workgroups] how often each logical workgroup's work has been taken
    unsigned seq = 0;                // launches of this layout before this one
    int rows = 0, placesPerRow = 4, accumulate = 0;
    int ldsCount = 0;                // where in LDS the workgroup counts the groups that fall to it (bytes)
};

// The XCD this wave runs on (XCC_ID, bits 3:0 of hardware register 20).
__device__ __forceinline__ int xcc_id() { return (int)(__builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15u); }

// The largest v of the wave's 64 lanes, in every lane (as a scalar).
__device__ __forceinline__ int wave_max(int v)
{
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x141, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x140, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_ds_swizzle(v, 0x401F));
    return max(__builtin_amdgcn_readlane(v, 0), __builtin_amdgcn_readlane(v, 32));
}

// A load that is served by the L2 and never by this CU's L1 (sc0): what another workgroup on the
// same XCD stored before it counted itself off is in that L2.
template <typename T>
__device__ __forceinline__ T load_from_l2(const T *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// The last step of the one-launch form: the rows of the `nl` groups in `list` added up by one workgroup.
// A lane takes R rows at a time, one from each of R groups (2 groups side by side in a workgroup of
// 512), and asks for everything it needs -- every place of every row, used or not: a place that no
// virtual row owns holds the zero it was made with -- before it uses any of it: one trip for the lot,
// and nothing is read that this launch did not write.  A row has fa.placesPerRow places, at most P
// (what is read per group is places x 2 KB or 1 KB, and reading is what the adding costs).  The 64 rows of a wave are consecutive, so every
// load is one contiguous stretch.  Sums in the order of the places, whoever adds: y does not depend on
// who came last.
template <typename VT, int P, int R>
__device__ __forceinline__ void fused_add(const FusedArgs &fa, const int *list, int nl, int tid)
{
    typedef typename Acc<VT>::type AT;
    constexpr int GR = mx::kFusedGroupRows, SIDE = kSliceThreads / GR;  // groups side by side
    static_assert(kSliceThreads % GR == 0 && GR == 256, "a lane keeps its place inside the group from slot to slot");
    const AT *sums = (const AT *)fa.sums;
    VT *y = (VT *)fa.y;
    AT *ywide = (AT *)fa.ywide;
    const int half = __builtin_amdgcn_readfirstlane(tid / GR), rl = tid % GR;
    const int places = fa.placesPerRow;
    for (int j0 = 0; j0 < nl; j0 += SIDE * R) {
        int row[R];
        AT v[R][P], old[R];
#pragma unroll
        for (int i = 0; i < R; ++i) {
            // (whether a slot holds a group is the same for all lanes of a wave: a branch, not a mask, so
            // that an empty slot costs no traffic; nothing is waited for between the slots)
            const int li = j0 + half + SIDE * i;
            row[i] = -1;
            old[i] = 0;
#pragma unroll
            for (int k = 0; k < P; ++k) v[i][k] = 0;
            if (li < nl) {
                const int g = list[li];
                if (g * GR + rl < fa.rows) row[i] = g * GR + rl;
                const AT *p = sums + (size_t)g * places * GR + rl;
#pragma unroll
                for (int k = 0; k < P; ++k)
                    if (k < places) v[i][k] = load_from_l2(p + (size_t)k * GR);
                if (fa.accumulate) old[i] = (AT)y[max(row[i], 0)];
            }
        }
#pragma unroll
        for (int i = 0; i < R; ++i) {
            AT sum = old[i];
#pragma unroll
            for (int k = 0; k < P; ++k) sum += v[i][k];
            if (row[i] >= 0) {
                y[row[i]] = (VT)sum;
                if (ywide) ywide[row[i]] = sum;
            }
        }
    }
}

// DICT: `eval` points at one byte per entry (same places as the column offsets) and `dictG` at the
// 256 values they name; a workgroup keeps those in LDS behind the chunk ends.
// FUSED: the one-launch form.  The layout gives every XCD the same number of logical workgroups
// and puts all of them that hold sums of a group of kFusedGroupRows rows on one XCD (DeviceSlices).
// A workgroup takes its work by where it runs: logical workgroup (XCC_ID, blockIdx / 8) -- the
// dispatcher deals consecutive workgroups round-robin to the XCDs, from a starting XCD that depends
// on what ran before, so the workgroups that land on one XCD have distinct blockIdx / 8 and every
// logical workgroup is taken once.  That one assumption is checked in every launch: each logical
// workgroup's `claim` is counted up by whoever takes it (together with the group counters, at the end),
// and a count that is not the launch's number means that two took the same; the launch's y cannot be
// trusted then and the host is told.
// The sums are stored where the one who adds finds them without an index list (DeviceSlices::fusedSums;
// a workgroup keeps the places of its own virtual rows in LDS).  After its stream a workgroup waits until its own
// stores have reached the L2 (s_waitcnt vmcnt(0): a store counts as done when the L2 has it),
// adds one to the counter of each of its groups with an atomic that executes in that L2, and for
// every group whose count it completes adds the sums of the group's rows up -- in the order of the
// row's places, whoever does it, so y does not depend on who came last -- and writes y.  It clears
// the counter for the next launch.  No workgroup ever waits for another.
template <typename VT, bool DICT = false, bool FUSED = false, bool KEEP = false>
__global__ __launch_bounds__(kSliceThreads) void csr_slice_kernel(const int4 *__restrict__ wgDesc,
                                                                  const int4 *__restrict__ waveDesc,
                                                                  const int *__restrict__ chunkEnd,
                                                                  const unsigned short *__restrict__ ecol,
                                                                  const VT *__restrict__ eval, const VT *__restrict__ x,
                                                                  typename Acc<VT>::type *__restrict__ partial, int cols,
                                                                  int sliceCols, const VT *__restrict__ dictG,
                                                                  int maxWgChunks, FusedArgs fa)
{
    typedef typename Acc<VT>::type AT;
    typedef typename std::conditional<DICT, SliceBatchDict<VT>, SliceBatch<VT>>::type Batch;
    typedef typename std::conditional<DICT, unsigned char, VT>::type StreamT;
    const StreamT *estream = (const StreamT *)eval;
    // (a step is one entry per lane; binary64 values as they are leave registers for a ring of five)
    constexpr int SPB = mx::kSliceBatchEntries, NB = (sizeof(VT) == 8 && !DICT) ? kSliceRing - 1 : kSliceRing;
    constexpr int EPV = 16 / (int)sizeof(VT);
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    VT *xs = (VT *)smem;                                           // [sliceCols]
    int *endsL = (int *)(smem + (size_t)sliceCols * sizeof(VT));   // [chunks of the workgroup]
    AT *dictL = (AT *)(endsL + ((maxWgChunks + 3) & ~3));            // [256] with DICT
    int *targetL = (int *)(dictL + (DICT ? 256 : 0));                // [chunks of the workgroup][64] with FUSED
    if constexpr (DICT) {
        if (threadIdx.x < 256) dictL[threadIdx.x] = (AT)dictG[threadIdx.x];  // visible after the barrier below
    }

    // the workgroups of a slice are numbered consecutively: with every XCD on one contiguous range
    // of them a slice of x is fetched into one L2, not into all eight
    const int tid = threadIdx.x, lane = tid & 63;
    const int b = FUSED ? min(xcc_id(), mx::kFusedXcds - 1) * ((int)gridDim.x / mx::kFusedXcds) + (int)blockIdx.x / mx::kFusedXcds
                        : xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int4 gd = wgDesc[b];
    const int4 d = waveDesc[b * kSliceWaves + wave];
    const int slice = gd.x, wgChunk0 = gd.y, wgChunks = gd.z;
    int group0 = 0, nGroupsMine = 0, need = 0;
    if constexpr (FUSED) {
        group0 = fa.wgGroups[2 * b];
        nGroupsMine = fa.wgGroups[2 * b + 1];
        // (asked for now, looked at when the stream is done; a workgroup has fewer groups than lanes)
        need = fa.groupNeed[group0 + min(tid, max(nGroupsMine - 1, 0))];
    }
    const int batch0 = __builtin_amdgcn_readfirstlane(d.x), nb = __builtin_amdgcn_readfirstlane(d.y);
    const int chunk0 = __builtin_amdgcn_readfirstlane(d.z), nChunks = __builtin_amdgcn_readfirstlane(d.w);
    // Every load below is unconditional -- indices are clamped instead, and what a clamped load
    // brings is masked or never used -- because the compiler can count the loads in flight, and so
    // wait for exactly the one it needs, only along paths on which the loads are certain.  After
    // a conditional load it waits for all of them at every use, and the pipeline is gone.
    //
    // chunk ends of the workgroup, and the slice (all of it at once, one 16-byte vector per
    // lane and round).  The last vector of x may be partial: it is read whole (an aligned 16-byte
    // read cannot leave the page its first byte is on) and the elements beyond x are zeroed.
    const int ce = chunkEnd[wgChunk0 + max(min(tid, wgChunks - 1), 0)];
    constexpr int CB = kSliceBytes / 16 / kSliceThreads;  // rounds of a full slice
    const int lastVec = (cols + EPV - 1) / EPV - 1;
    v4i32 xv[CB];
#pragma unroll
    for (int q = 0; q < CB; ++q) {
        const int gi = slice * (sliceCols / EPV) + tid + q * kSliceThreads;
        xv[q] = ((const v4i32 *)x)[min(gi, lastVec)];
    }
    // (one-launch form: where the sums of the workgroup's first chunks go -- asked for before the ring, so that
    // putting them into LDS waits for them and for x, and not for the ring behind them)
    constexpr int TR = FUSED ? 4 : 1;
    int tg[TR];
    if constexpr (FUSED) {
#pragma unroll
        for (int q = 0; q < TR; ++q)
            tg[q] = fa.target[(size_t)wgChunk0 * 64 + max(min(tid + q * kSliceThreads, wgChunks * 64 - 1), 0)];
    }
    // the ring: the first batches of the wave's stream (the last one again and again when the
    // stream is shorter than the ring)
    Batch buf[NB];
    const int lastBatch = batch0 + max(nb - 1, 0);
#pragma unroll
    for (int k = 0; k < NB; ++k) buf[k].template load<KEEP>(ecol, estream, (size_t)min(batch0 + k, lastBatch), lane);
    endsL[max(min(tid, wgChunks - 1), 0)] = ce;
    if constexpr (FUSED) {
        if (tid == 0) *(int *)(smem + fa.ldsCount) = 0;  // (read after the stream, behind two barriers)
#pragma unroll
        for (int q = 0; q < TR; ++q)
            if (tid + q * kSliceThreads < wgChunks * 64) targetL[tid + q * kSliceThreads] = tg[q];
    }
    if ((slice + 1) * sliceCols <= cols) {  // the whole slice lies inside x
#pragma unroll
        for (int q = 0; q < CB; ++q) *(v4i32 *)(xs + (tid + q * kSliceThreads) * EPV) = xv[q];
    } else {
#pragma unroll
        for (int q = 0; q < CB; ++q) {
            const int i = tid + q * kSliceThreads;
            const int have = cols - (slice * sliceCols + i * EPV);  // elements of this vector inside x
            v4i32 v = xv[q];
#pragma unroll
            for (int d = 0; d < 4; ++d) {  // dword d holds half an element, or two
                const int lo = sizeof(VT) == 8 ? d / 2 : 2 * d, hi = sizeof(VT) == 8 ? d / 2 : 2 * d + 1;
                v[d] &= (have > lo ? 0xffff : 0) | (have > hi ? 0xffff0000 : 0);
            }
            *(v4i32 *)(xs + i * EPV) = v;
        }
    }
    for (int i = kSliceThreads + tid; i < wgChunks; i += kSliceThreads) endsL[i] = chunkEnd[wgChunk0 + i];
    if constexpr (FUSED) {
        // (a workgroup with more than 32 chunks: the rest, behind the ring)
        for (int i = TR * kSliceThreads + tid; i < wgChunks * 64; i += kSliceThreads) targetL[i] = fa.target[(size_t)wgChunk0 * 64 + i];
    }
    __syncthreads();
    // (the chunk ends are the same for all lanes of the wave: kept in scalar registers)
    // and 64 at a time, lane i holding the end of the wave's chunk 64 * (ci / 64) + i, so that the next end is
    // there without a trip to the LDS when a chunk is done (chunks of a few entries end every few steps)
    auto ends64 = [&](int c0) { return endsL[chunk0 + min(c0 + lane, max(nChunks - 1, 0))]; };
    int endsV = ends64(0);
    int ci = 0, nextEnd = nChunks > 0 ? __builtin_amdgcn_readlane(endsV, 0) : -1;
    AT acc = 0;
    AT *out = partial + (size_t)(wgChunk0 + chunk0) * 64 + lane;
    auto flush = [&]() {
        if constexpr (FUSED) ((AT *)fa.sums)[targetL[(chunk0 + ci) * 64 + lane]] = acc;
        else out[(size_t)ci * 64] = acc;
        acc = 0;
        ++ci;
        if ((ci & 63) == 0) endsV = ends64(ci);
        nextEnd = ci < nChunks ? __builtin_amdgcn_readlane(endsV, ci & 63) : -1;
    };
    auto consume = [&](const Batch &B, int t) {  // t = number of the batch in the wave's stream
        // what the batch needs from LDS is asked for before the first product: with a request and its wait per
        // entry the wave would sit out one LDS round trip after the other
        VT xk[SPB];
        AT vk[DICT ? SPB : 1];
#pragma unroll
        for (int j = 0; j < SPB; ++j) xk[j] = B.gather(xs, j);
        if constexpr (DICT) {
#pragma unroll
            for (int j = 0; j < SPB; ++j) vk[j] = B.value(dictL, j);
        }
        auto add = [&](int j) {
            if constexpr (DICT) acc += vk[j] * (AT)xk[j];
            else acc += B.term(j, xk[j]);
        };
        if (nextEnd < 0 || nextEnd > (t + 1) * SPB) {  // no chunk ends inside the batch
#pragma unroll
            for (int j = 0; j < SPB; ++j) add(j);
        } else {
#pragma unroll
            for (int j = 0; j < SPB; ++j) {
                add(j);
                if (t * SPB + j + 1 == nextEnd) flush();
            }
        }
    };
    if (nb <= NB) {  // everything is in the ring already
#pragma unroll
        for (int k = 0; k < NB; ++k)
            if (k < nb) consume(buf[k], k);
    } else {
        int t = 0;
        // while a whole ring beyond the one in flight remains: consume and reload
        for (; t + 2 * NB <= nb; t += NB) {
#pragma unroll
            for (int k = 0; k < NB; ++k) {
                consume(buf[k], t + k);
                buf[k].template load<KEEP>(ecol, estream, (size_t)(batch0 + t + NB + k), lane);
            }
        }
        // one ring in flight and less than one more to come: consume and reload while batches
        // remain (the last one again after that), then those
#pragma unroll
        for (int k = 0; k < NB; ++k) {
            consume(buf[k], t + k);
            buf[k].template load<KEEP>(ecol, estream, (size_t)min(batch0 + t + NB + k, lastBatch), lane);
        }
#pragma unroll
        for (int k = 0; k < NB; ++k)
            if (t + NB + k < nb) consume(buf[k], t + NB + k);
    }
    if constexpr (FUSED) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's sums are in the L2
        __syncthreads();                                    // ... and so are the other waves'
        // (the chunk ends are done with: the groups that fall to this workgroup are listed in their place; how many,
        // in a word of its own that was cleared before the stream began)
        int *listL = endsL;
        int *countL = (int *)(smem + fa.ldsCount);
        // a lane per group, and one lane more for the workgroup's claim: one atomic each, all in one trip
        if (tid <= nGroupsMine) {
            const bool forClaim = tid == nGroupsMine;
            const int g = group0 + tid;
            unsigned *counter = forClaim ? fa.claim + b : (unsigned *)fa.groupCount + g;
            const unsigned old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (forClaim) {
                if (old != fa.seq || xcc_id() >= mx::kFusedXcds)
                    __hip_atomic_store(fa.misplaced, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            } else if ((int)old + 1 == need) {
                __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                listL[atomicAdd(countL, 1)] = g;
            }
        }
        __syncthreads();
        const int nl = *countL;
        if (nl == 0) return;
        if (fa.placesPerRow > 4) fused_add<VT, 8, 4>(fa, listL, nl, tid);
        else fused_add<VT, 4, 8>(fa, listL, nl, tid);
    }
}

// ---- tile part --------------------------------------------------------------------------
// The selected fragments arrive expanded to full blocks and regrouped into steps (see
// DeviceTiles): what one wave hands to the matrix core at a time.  A wave owns a run of steps
// made of whole chunks and walks it with everything prefetched: while step s is multiplied, the
// header, column ids and values of steps s+1 .. s+4 and the x values and old y of steps s+1 and
// s+2 are already on their way, so the dependent accesses of a step (column ids -> x, header ->
// rows -> y) never stall the wave.  Every lane loads the values it feeds to the matrix core
// itself, straight from the block, so only the gathered x goes through LDS.
//
// v_mfma_f64_16x16x4_f64 (wave64): lane L holds A[L%16][L/16] and B[L/16][L%16]; accumulator
// register g of lane L holds D[4*g + L/16][L%16].  One MFMA feeds two 8x4 blocks: A rows 0..7 =
// block j of half 0, rows 8..15 = block j of half 1; B column 0 = the 4 gathered x of the
// former, column 1 = those of the latter, other columns 0.  D[0..7][0] collects half 0 and
// D[8..15][1] half 1 over the 8 MFMAs of a step and all steps of a chunk, inside the matrix core.
//
// v_mfma_f32_16x16x32_f16 (wave64): lane L holds A[L%16][8*(L/16) .. +7], B[8*(L/16) .. +7][L%16];
// accumulator register g of lane L holds D[4*(L/16)+g][L%16].  One MFMA is a whole step: A rows
// 0..7 = the 4 blocks of half 0 side by side along K, rows 8..15 = those of half 1; B column 0 =
// the 32 gathered x of half 0, column 1 = those of half 1.  A lane's eight A elements are one
// row of one 8x8 block: 16 contiguous bytes.
using mx::kTileHdr;

// The MFMA calls of tile_kernel sit in code shared by both precisions; overloads pick the
// instruction.
__device__ __forceinline__ v4f64 tile_mma(double a, double b, v4f64 c)
{
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ v4f32 tile_mma(v8f16 a, v8f16 b, v4f32 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

template <typename VT>
struct TileStep {  // one step's loads, as one lane holds them
    int hdr;       // header dword lane%32: lanes 0..15 hold the output rows
    int ax;        // column id
    typename std::conditional<sizeof(VT) == 8, double[8], v4i32>::type v;  // A operands
    VT xr;         // gathered x, as loaded (looked at only when the step is multiplied)
    typename Acc<VT>::type yr;  // old y
};

// All loads of a step are unconditional: the count of loads in flight is then known at compile
// time and the wave can wait for one step while the next ones are still on their way.  A lane
// whose block is absent reads what follows the step's values (the host leaves slack at the end)
// and ignores it.  vo = first value of the step, na = blocks in its half 0.
template <typename VT>
__device__ __forceinline__ void tile_issue(TileStep<VT> &R, const int *__restrict__ hdr, const int *__restrict__ atox,
                                           const VT *__restrict__ tcVal, int step, int vo, int na, int lane)
{
    R.ax = atox[(size_t)step * 64 + lane];
    R.hdr = hdr[(size_t)step * kTileHdr + (lane & 31)];
    const int m = lane & 15, g = lane >> 4, h = m >> 3;
    if constexpr (sizeof(VT) == 8) {
        const VT *p = tcVal + vo + (h ? na : 0) * 32 + (m & 7) * 4 + g;
#pragma unroll
        for (int j = 0; j < 8; ++j) R.v[j] = __builtin_nontemporal_load(p + j * 32);
    } else {
        R.v = __builtin_nontemporal_load((const v4i32 *)(tcVal + vo + ((h ? na : 0) + g) * 64 + (m & 7) * 8));
    }
}

template <typename VT>
__global__ __launch_bounds__(kBlock) void tile_kernel(const int4 *__restrict__ waveDesc, const int *__restrict__ hdr,
                                                     const int *__restrict__ atox, const VT *__restrict__ tcVal,
                                                     const VT *__restrict__ x, VT *__restrict__ y, int nWaves,
                                                     int accumulate, const typename Acc<VT>::type *__restrict__ ywide)
{
    typedef typename Acc<VT>::type AT;
    constexpr bool F64 = sizeof(VT) == 8;
    struct Park {
        VT xv[64];
        AT out[16];
    };
    __shared__ __attribute__((aligned(16))) Park park[kBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // waves follow the chunks in order, and neighbouring chunks share columns of x and lines of
    // y: every XCD takes one contiguous range of them
    const int gw = xcd_contiguous_block(blockIdx.x, gridDim.x) * (kBlock / 64) + wave;
    if (gw >= nWaves) return;
    Park &P = park[wave];
    const int4 d0 = waveDesc[2 * gw], d1 = waveDesc[2 * gw + 1];
    const int s0 = __builtin_amdgcn_readfirstlane(d0.x), s1 = __builtin_amdgcn_readfirstlane(d0.y);
    if (s0 >= s1) return;
    const int last = s1 - 1;
    const int m = lane & 15, g = lane >> 4, h = m >> 3;

    // Five register sets take turns: the step being multiplied, the two after it (their gathers
    // are in flight or about to be issued) and two more whose header, column ids and values are
    // on their way.  Everything a step waits for was asked for two steps earlier.  The loop
    // below is unrolled five times so that no set is ever copied into another (a copy would have
    // to wait for the loads that fill it).
    typedef TileStep<VT> Regs;
    Regs R0, R1, R2, R3, R4;
    // x and old y of a step, once its column ids and header are there (lanes without a column
    // or a row read element 0 and ignore it)
    auto gather = [&](Regs &R) {
        R.xr = x[max(R.ax, 0)];
        // (old y: as the kernel before this one left it, unrounded where that kernel kept it so)
        const int yi = lane < 16 ? max(R.hdr, 0) : 0;
        R.yr = ywide ? ywide[yi] : (AT)y[yi];
    };
    typedef typename std::conditional<F64, v4f64, v4f32>::type AccV;
    AccV acc;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = 0;
    // one step: Ra is multiplied, Rg (two steps on) gets its gathers, Ri (four steps on) is issued
    auto step = [&](int s, Regs &Ra, Regs &Rg, Regs &Ri) {
        // where the values of step s+4 start is written in the header of step s
        tile_issue<VT>(Ri, hdr, atox, tcVal, min(s + 4, last), __builtin_amdgcn_readlane(Ra.hdr, 19),
                       __builtin_amdgcn_readlane(Ra.hdr, 20), lane);
        gather(Rg);
        P.xv[lane] = Ra.ax >= 0 ? Ra.xr : (VT)0;
        __builtin_amdgcn_wave_barrier();
        const int flags = __builtin_amdgcn_readlane(Ra.hdr, 16);
        const int nblk = h ? __builtin_amdgcn_readlane(Ra.hdr, 18) : __builtin_amdgcn_readlane(Ra.hdr, 17);
        if constexpr (F64) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const double a = j < nblk ? Ra.v[j] : 0.0;
                const double bv = m < 2 ? P.xv[(2 * j + m) * 4 + g] : 0.0;
                acc = tile_mma(a, bv, acc);
            }
        } else {
            const v4i32 z = {0, 0, 0, 0};
            const v8f16 a = __builtin_bit_cast(v8f16, g < nblk ? Ra.v : z);
            v8f16 bv = {0, 0, 0, 0, 0, 0, 0, 0};
            if (m < 2) bv = *(const v8f16 *)(P.xv + (4 * m + g) * 8);
            acc = tile_mma(a, bv, acc);
        }
        if (flags & 1) {
            // half 0 = D[0..7][0], half 1 = D[8..15][1]; hand them to lanes 0..15 through LDS
            if constexpr (F64) {
                // D[q][0] = reg 0 and D[q+4][0] = reg 1 of lane 16q; D[8+q][1] = reg 2, D[12+q][1] = reg 3 of lane 16q+1
                if (m == 0) {
                    P.out[g] = acc[0];
                    P.out[g + 4] = acc[1];
                }
                if (m == 1) {
                    P.out[8 + g] = acc[2];
                    P.out[12 + g] = acc[3];
                }
            } else {
                // D[0..3][0] in lane 0, D[4..7][0] in lane 16, D[8..11][1] in lane 33, D[12..15][1] in lane 49
                if (lane == 0 || lane == 16 || lane == 33 || lane == 49) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) P.out[4 * g + i] = acc[i];
                }
            }
            __builtin_amdgcn_wave_barrier();
            if (lane < 16 && Ra.hdr >= 0) {
                AT o = P.out[lane];
                if (!(flags & 2)) o += P.out[lane + 8];  // one chunk in both halves (only lanes 0..7 have rows)
                y[Ra.hdr] = (VT)((accumulate ? Ra.yr : (AT)0) + o);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = 0;
        }
        __builtin_amdgcn_wave_barrier();
    };
    const int na = __builtin_amdgcn_readfirstlane(d1.z);
    tile_issue<VT>(R0, hdr, atox, tcVal, s0, __builtin_amdgcn_readfirstlane(d0.z), na & 255, lane);
    tile_issue<VT>(R1, hdr, atox, tcVal, min(s0 + 1, last), __builtin_amdgcn_readfirstlane(d0.w), (na >> 8) & 255, lane);
    tile_issue<VT>(R2, hdr, atox, tcVal, min(s0 + 2, last), __builtin_amdgcn_readfirstlane(d1.x), (na >> 16) & 255, lane);
    tile_issue<VT>(R3, hdr, atox, tcVal, min(s0 + 3, last), __builtin_amdgcn_readfirstlane(d1.y), (na >> 24) & 255, lane);
    gather(R0);
    gather(R1);
    for (int s = s0; s < s1; s += 5) {
        step(s, R0, R2, R4);
        if (s + 1 < s1) step(s + 1, R1, R3, R0);
        if (s + 2 < s1) step(s + 2, R2, R4, R1);
        if (s + 3 < s1) step(s + 3, R3, R0, R2);
        if (s + 4 < s1) step(s + 4, R4, R1, R3);
    }
}

// The binary16 tile kernel for blocks whose eight columns are consecutive (dense strips), for
// chunks of at most one step whose rows receive nothing from the CSR part.  A lane's B operand --
// the eight x of one block -- is then one 16-byte read of x (at a multiple of 16 bytes when the
// block starts at a multiple of eight columns; a strip that starts elsewhere has blocks that start
// there, and the read is an unaligned one, which global memory serves), so the column ids, the
// gather, the trip through LDS and the old y all fall away: per step a header, the blocks and 16
// bytes of x per block.  The results
// leave from the four lanes that hold them.  Same step stream, headers and wave ranges as
// tile_kernel; the header carries the first column of every block slot in dwords 21..28.
struct DenseStep {
    int hdr;      // header dword lane%32
    v4i32 v, b;   // A operand (one block row), B operand (the eight x of the lane's block)
};
// One wave's range of steps (wave `gw` of the layout).  KEEP: the values are read with plain loads (a plan whose
// product fits the memory-side cache keeps them there, as it keeps the entries of its slices), streamed otherwise.
template <bool KEEP = false>
__device__ __forceinline__ void tile_dense_wave(const int4 *__restrict__ waveDesc, const int *__restrict__ hdr,
                                                const _Float16 *__restrict__ tcVal, const _Float16 *__restrict__ x,
                                                _Float16 *__restrict__ y, int gw, int lane)
{
    const int4 d0 = waveDesc[2 * gw], d1 = waveDesc[2 * gw + 1];
    const int s0 = __builtin_amdgcn_readfirstlane(d0.x), s1 = __builtin_amdgcn_readfirstlane(d0.y);
    if (s0 >= s1) return;
    const int last = s1 - 1;
    const int m = lane & 15, g = lane >> 4, h = m >> 3;
    auto issue = [&](DenseStep &R, int step, int vo, int na) {
        R.hdr = hdr[(size_t)step * kTileHdr + (lane & 31)];
        R.v = stream_load<KEEP>((const v4i32 *)(tcVal + vo + ((h ? na : 0) + g) * 64 + (m & 7) * 8));
    };
    // the x of the lane's block, once the header is there: B column m (0 = half 0, 1 = half 1),
    // rows 8g..8g+7 = slot 4m+g; the other lanes read what lane m&1 of their group reads
    auto fetch = [&](DenseStep &R) {
        const int base = __shfl(R.hdr, 21 + 4 * (m & 1) + g);
        R.b = *(const v4i32u *)(x + max(base, 0));
    };
    auto step = [&](int s, DenseStep &Ra, DenseStep &Rg, DenseStep &Ri) {
        issue(Ri, min(s + 4, last), __builtin_amdgcn_readlane(Ra.hdr, 19), __builtin_amdgcn_readlane(Ra.hdr, 20));
        fetch(Rg);
        const int n0 = __builtin_amdgcn_readlane(Ra.hdr, 17), n1 = __builtin_amdgcn_readlane(Ra.hdr, 18);
        const v4i32 z = {0, 0, 0, 0};
        const v8f16 a = __builtin_bit_cast(v8f16, g < (h ? n1 : n0) ? Ra.v : z);
        const v8f16 bv = __builtin_bit_cast(v8f16, (m < 2 && g < (m ? n1 : n0)) ? Ra.b : z);
        const v4f32 zero = {0.f, 0.f, 0.f, 0.f};
        v4f32 acc = tile_mma(a, bv, zero);
        // D[0..3][0] in lane 0, D[4..7][0] in lane 16, D[8..11][1] in lane 33, D[12..15][1] in lane 49:
        // register i of those lanes is output row 4g+i of the step.  A chunk that fills both
        // halves has its rows in the first two only: they add what the other two hold.
        if (!(__builtin_amdgcn_readlane(Ra.hdr, 16) & 2)) {
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] += __shfl(acc[i], (lane + 33) & 63);
        }
        int row[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) row[i] = __shfl(Ra.hdr, 4 * g + i);
        if (lane == 0 || lane == 16 || lane == 33 || lane == 49) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (row[i] >= 0) y[row[i]] = (_Float16)acc[i];
        }
    };
    DenseStep R0, R1, R2, R3, R4;
    const int na = __builtin_amdgcn_readfirstlane(d1.z);
    issue(R0, s0, __builtin_amdgcn_readfirstlane(d0.z), na & 255);
    issue(R1, min(s0 + 1, last), __builtin_amdgcn_readfirstlane(d0.w), (na >> 8) & 255);
    issue(R2, min(s0 + 2, last), __builtin_amdgcn_readfirstlane(d1.x), (na >> 16) & 255);
    issue(R3, min(s0 + 3, last), __builtin_amdgcn_readfirstlane(d1.y), (na >> 24) & 255);
    fetch(R0);
    fetch(R1);
    for (int s = s0; s < s1; s += 5) {
        step(s, R0, R2, R4);
        if (s + 1 < s1) step(s + 1, R1, R3, R0);
        if (s + 2 < s1) step(s + 2, R2, R4, R1);
        if (s + 3 < s1) step(s + 3, R3, R0, R2);
        if (s + 4 < s1) step(s + 4, R4, R1, R3);
    }
}

__global__ __launch_bounds__(kBlock) void tile_dense_kernel(const int4 *__restrict__ waveDesc, const int *__restrict__ hdr,
                                                           const _Float16 *__restrict__ tcVal,
                                                           const _Float16 *__restrict__ x, _Float16 *__restrict__ y,
                                                           int nWaves)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gw = xcd_contiguous_block(blockIdx.x, gridDim.x) * (kBlock / 64) + wave;
    if (gw < nWaves) tile_dense_wave(waveDesc, hdr, tcVal, x, y, gw, lane);
}

// The binary64 counterpart: aligned blocks of 8 x 8 (eight consecutive columns from a multiple of
// eight, on eight consecutive rows) that the plan finds in the extracted block -- the dense
// blocks of a block-structured matrix -- on rows that also have other entries.  Same step stream
// as the strips (two halves of up to four blocks, headers with the first column of every block
// slot, blocks stored whole and row-major, waves over whole chunks, four steps prefetched), with
// eight v_mfma_f64_16x16x4_f64 per step: MFMA 2p and 2p+1 take block p of both halves, the first
// the even columns of the block (k-th A column = block column 2k), the second the odd ones, so that
// a lane's two A values (row m%8, columns 2k and 2k+1) and its two B values (x[first + 2k],
// x[first + 2k + 1]) are each one aligned 16-byte load.  No column ids, nothing through LDS.
// The rows get the rest of their sum from the CSR part.  RIDE: the wave runs inside the combine
// kernel's launch and fetches the sums of the rows' virtual rows itself (vidx: per step and half,
// eight places per row, -1 = none), so that y is written once, here, and the combine kernel's own
// kinds leave these rows alone.  Otherwise y holds the CSR part's sum already and is added to.
// Waves are many and short -- the host gives each one step, more only to a chunk of more than
// eight blocks -- and keep nothing in flight beyond the step at hand: a step is two dependent
// rounds of loads (header, values and places; then x and the sums the places name), and what
// hides them is the number of waves a CU holds, so the wave is written for few registers.
template <bool RIDE>
__device__ __forceinline__ void tile_block_wave(const int4 *__restrict__ waveDesc, const int *__restrict__ hdr,
                                                const int *__restrict__ vidx, const double *__restrict__ tcVal,
                                                const double *__restrict__ x, const double *__restrict__ partial,
                                                double *__restrict__ y, int gw, int lane)
{
    const int4 d0 = waveDesc[2 * gw], d1 = waveDesc[2 * gw + 1];
    const int s0 = __builtin_amdgcn_readfirstlane(d0.x), s1 = __builtin_amdgcn_readfirstlane(d0.y);
    if (s0 >= s1) return;
    const int m = lane & 15, k = lane >> 4, h = m >> 3;
    // where the values of the next four steps start and how many blocks their first halves hold:
    // from the wave's descriptor at first, then from the header of the step four back
    int vo0 = __builtin_amdgcn_readfirstlane(d0.z), vo1 = __builtin_amdgcn_readfirstlane(d0.w);
    int vo2 = __builtin_amdgcn_readfirstlane(d1.x), vo3 = __builtin_amdgcn_readfirstlane(d1.y);
    const int na4 = __builtin_amdgcn_readfirstlane(d1.z);
    int na0 = na4 & 255, na1 = (na4 >> 8) & 255, na2 = (na4 >> 16) & 255, na3 = (na4 >> 24) & 255;
    v4f64 acc = {0.0, 0.0, 0.0, 0.0};
    for (int s = s0; s < s1; ++s) {
        // round one: header, the lane's A operands (block q of its half, row m%8, columns 2k and 2k+1:
        // a lane whose block is absent reads what follows the step's values and ignores it) and places
        const int hd = hdr[(size_t)s * kTileHdr + (lane & 31)];
        const double *p = tcVal + vo0 + (size_t)(h ? na0 : 0) * 64 + (m & 7) * 8 + 2 * k;
        v2f64 v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = __builtin_nontemporal_load((const v2f64 *)(p + q * 64));
        int vi0 = -1, vi1 = -1;
        if constexpr (RIDE) {
            vi0 = vidx[(size_t)s * 128 + lane];
            vi1 = vidx[(size_t)s * 128 + 64 + lane];
        }
        // round two: the B operands (lanes 0 and 1 of each 16: the x of block q of half 0 / half 1, one
        // aligned 16-byte read) and the other part of the rows' sums
        v2f64 bx[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int base = __shfl(hd, 21 + 4 * (m & 1) + q);
            bx[q] = *(const v2f64 *)(x + max(base, 0) + 2 * k);
        }
        double ps0, ps1;
        if constexpr (RIDE) {
            const double a = partial[max(vi0, 0)], b = partial[max(vi1, 0)];
            ps0 = vi0 >= 0 ? a : 0.0;
            ps1 = vi1 >= 0 ? b : 0.0;
        } else {
            const int r0 = __shfl(hd, lane >> 3), r1 = __shfl(hd, 8 + (lane >> 3));
            const double a = y[max(r0, 0)], b = y[max(r1, 0)];
            ps0 = ((lane & 7) == 0 && r0 >= 0) ? a : 0.0;
            ps1 = ((lane & 7) == 0 && r1 >= 0) ? b : 0.0;
        }
        const int n0 = __builtin_amdgcn_readlane(hd, 17), n1 = __builtin_amdgcn_readlane(hd, 18);
        const int na = h ? n1 : n0, nb = m ? n1 : n0;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const double a0 = q < na ? v[q].x : 0.0, a1 = q < na ? v[q].y : 0.0;
            const double b0 = (m < 2 && q < nb) ? bx[q].x : 0.0, b1 = (m < 2 && q < nb) ? bx[q].y : 0.0;
            acc = tile_mma(a0, b0, acc);
            acc = tile_mma(a1, b1, acc);
        }
        const int flags = __builtin_amdgcn_readlane(hd, 16);
        if (flags & 1) {
            // the other part of every row's sum: eight places per row, summed inside groups of 8 lanes
            const double c0 = group_sum<8>(ps0), c1 = group_sum<8>(ps1);
            // D[j][0] and D[4+j][0] are registers 0 and 1 of lane 16j; D[8+j][1] and D[12+j][1] are
            // registers 2 and 3 of lane 16j+1.  A chunk that fills both halves has its rows in the
            // first only: lane 16j adds what lane 16j+1 holds.
            const double u2 = __shfl(acc[2], (lane + 1) & 63), u3 = __shfl(acc[3], (lane + 1) & 63);
            // row j's other part sits in lanes 8j..8j+7, row 4+j's in lanes 32+8j..: lanes 16j and 16j+1 both want lane>>1
            const double t0 = __shfl(c0, lane >> 1), t1 = __shfl(c0, (lane >> 1) + 32);
            const double w0 = __shfl(c1, lane >> 1), w1 = __shfl(c1, (lane >> 1) + 32);
            const int ra = __shfl(hd, k), rb = __shfl(hd, 4 + k), rc = __shfl(hd, 8 + k), rd = __shfl(hd, 12 + k);
            if (m == 0) {
                const double e0 = (flags & 2) ? 0.0 : u2, e1 = (flags & 2) ? 0.0 : u3;
                if (ra >= 0) y[ra] = acc[0] + e0 + t0;
                if (rb >= 0) y[rb] = acc[1] + e1 + t1;
            }
            if (m == 1 && (flags & 2)) {
                if (rc >= 0) y[rc] = acc[2] + w0;
                if (rd >= 0) y[rd] = acc[3] + w1;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[i] = 0.0;
        }
        // the ring moves on: step s leaves, step s+4 comes in from the header of step s
        vo0 = vo1, vo1 = vo2, vo2 = vo3, na0 = na1, na1 = na2, na2 = na3;
        vo3 = __builtin_amdgcn_readlane(hd, 19);
        na3 = __builtin_amdgcn_readlane(hd, 20);
    }
}

// The blocks in a launch of their own, after the CSR part: y is added to.
__global__ __launch_bounds__(kBlock) void tile_block_kernel(const int4 *__restrict__ waveDesc, const int *__restrict__ hdr,
                                                           const double *__restrict__ tcVal, const double *__restrict__ x,
                                                           double *__restrict__ y, int nWaves)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int gw = xcd_contiguous_block(blockIdx.x, gridDim.x) * (kBlock / 64) + wave;
    if (gw < nWaves) tile_block_wave<false>(waveDesc, hdr, nullptr, tcVal, x, nullptr, y, gw, lane);
}

// The sums of the virtual rows become y in one launch of three kinds of workgroups:
//  * the first `nRowWG` walk the matrix rows, kCombineRows per lane: rowInfo[r] >= 0 names the one virtual
//    row of row r, whose sum is the row's result; -1 is a row without entries (zero, or left
//    alone when `skipEmpty`); anything else a row that the lists below cover;
//  * the next `nLightWG` take the rows with 2..kSliceLightSegs virtual rows, one lane each: the
//    row and its kSliceLightSegs indices into `partial` (-1 = none) lie at the lane's own place in
//    two arrays, so nothing the lane loads depends on another load but the sums themselves;
//  * the rest take the rows with more, sixteen lanes each.
constexpr int kCombineRows = 16;  // rows a lane of the first kind takes
template <typename VT, bool STRIPS, bool KEEP = false>  // STRIPS: an instance of its own, so that the plain one keeps its few registers
__global__ __launch_bounds__(kBlock) void slice_combine_kernel(const typename Acc<VT>::type *__restrict__ partial,
                                                              const int *__restrict__ rowInfo, int rows, int nRowWG,
                                                              const int *__restrict__ lightRow,
                                                              const int4 *__restrict__ lightIdx, int nLight, int nLightWG,
                                                              const int4 *__restrict__ heavyInfo, int nHeavy,
                                                              const int *__restrict__ segIdx, VT *__restrict__ y,
                                                              int accumulate, int skipEmpty,
                                                              typename Acc<VT>::type *__restrict__ ywide,
                                                              const int4 *__restrict__ stripWaveDesc,
                                                              const int *__restrict__ stripHdr,
                                                              const VT *__restrict__ stripVal, const VT *__restrict__ x,
                                                              int nStripWaves, int nStripWG, int nHeavyWG, int lightQuads,
                                                              const int *__restrict__ stripVidx)
{
    typedef typename Acc<VT>::type AT;
    const int tid = threadIdx.x;
    // A fourth kind of workgroup, first in the grid: the strips of a binary16 plan (the work of
    // tile_dense_kernel), which need nothing from the sums and write rows that the other kinds
    // leave alone (rowInfo -2).  In one launch they cost no dependent launch of their own.  (Spread
    // evenly among the other kinds instead of ahead of them they cost more than a launch: 80 us
    // against 73 us on the mixed workload.)
    if (STRIPS && (int)blockIdx.x < nStripWG) {
        if constexpr (STRIPS && sizeof(VT) == 2) {
            const int gw = xcd_contiguous_block(blockIdx.x, nStripWG) * (kBlock / 64) + (tid >> 6);
            if (gw < nStripWaves) tile_dense_wave<KEEP>(stripWaveDesc, stripHdr, stripVal, x, y, gw, tid & 63);
        }
        // binary64: the 8 x 8 blocks, whose waves also fetch the sums of their rows' virtual rows
        // (those rows are marked -2 in rowInfo and appear in none of the lists below)
        if constexpr (STRIPS && sizeof(VT) == 8) {
            const int gw = xcd_contiguous_block(blockIdx.x, nStripWG) * (kBlock / 64) + (tid >> 6);
            if (gw < nStripWaves)
                tile_block_wave<true>(stripWaveDesc, stripHdr, stripVidx, (const double *)stripVal, (const double *)x,
                                      (const double *)partial, (double *)y, gw, tid & 63);
        }
        return;
    }
    // Every kind of workgroup walks its rows in ascending order, and the sums of neighbouring rows
    // lie close together wherever their virtual rows fall into the same slice and length class:
    // one XCD per contiguous range of rows keeps those sectors in a single L2.
    int b = (int)blockIdx.x - nStripWG;
    if (b < nRowWG) b = xcd_contiguous_block(b, nRowWG);
    else if (b < nRowWG + nLightWG) b = nRowWG + xcd_contiguous_block(b - nRowWG, nLightWG);
    else b = nRowWG + nLightWG + xcd_contiguous_block(b - nRowWG - nLightWG, nHeavyWG);
    if (b < nRowWG) {
        // kCombineRows rows per lane, as quads a wave apart so that its loads and stores stay contiguous
        int dd[kCombineRows];
#pragma unroll
        for (int q = 0; q < kCombineRows / 4; ++q) {
            const int r0 = 4 * ((b * (kCombineRows / 4) + q) * kBlock + tid);
            const int4 d = r0 < rows ? ((const int4 *)rowInfo)[r0 >> 2] : int4{-2, -2, -2, -2};  // padded with -2
            dd[4 * q] = d.x, dd[4 * q + 1] = d.y, dd[4 * q + 2] = d.z, dd[4 * q + 3] = d.w;
        }
        // (asked for whether the row has a sum or not: see the light rows below)
        AT sum[kCombineRows];
#pragma unroll
        for (int j = 0; j < kCombineRows; ++j) sum[j] = partial[max(dd[j], 0)];
#pragma unroll
        for (int j = 0; j < kCombineRows; ++j) sum[j] = dd[j] >= 0 ? sum[j] : (AT)0;
#pragma unroll
        for (int j = 0; j < kCombineRows; ++j) {
            const int r = 4 * ((b * (kCombineRows / 4) + j / 4) * kBlock + tid) + j % 4;
            const bool mine = dd[j] >= 0 || (dd[j] == -1 && !skipEmpty);
            if (mine && accumulate) sum[j] += (AT)y[r];
            if (mine) y[r] = (VT)sum[j];
            if (mine && ywide) ywide[r] = sum[j];
        }
        return;
    }
    b -= nRowWG;
    if (b < nLightWG) {
        const int i = b * kBlock + tid;
        if (i >= nLight) return;
        static_assert(mx::kSliceLightSegs == 8, "two int4 of indices per light row");
        const int r = lightRow[i];
        // (a layout whose light rows all have at most four virtual rows keeps four places per row)
        const int4 none = {-1, -1, -1, -1};
        const int4 i0 = lightQuads == 1 ? lightIdx[i] : lightIdx[2 * i], i1 = lightQuads == 1 ? none : lightIdx[2 * i + 1];
        const int id[8] = {i0.x, i0.y, i0.z, i0.w, i1.x, i1.y, i1.z, i1.w};
        // (every sum is asked for whether the place is used or not -- an unused one names sum 0 and is not
        // added: behind a conditional load the compiler waits before it issues the next, and a row's sums
        // would arrive one trip after the other)
        AT v[8];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = partial[max(id[k], 0)];
        if (lightQuads != 1) {
#pragma unroll
            for (int k = 4; k < 8; ++k) v[k] = partial[max(id[k], 0)];
        } else {
#pragma unroll
            for (int k = 4; k < 8; ++k) v[k] = 0;
        }
        AT sum = accumulate ? (AT)y[r] : (AT)0;
#pragma unroll
        for (int k = 0; k < 8; ++k) sum += id[k] >= 0 ? v[k] : (AT)0;
        y[r] = (VT)sum;
        if (ywide) ywide[r] = sum;
        return;
    }
    b -= nLightWG;
    const int g = b * (kBlock / 16) + (tid >> 4), sub = tid & 15;
    const bool live = g < nHeavy;
    const int4 h = live ? heavyInfo[g] : int4{0, 0, 0, 0};
    AT sum = 0;
    for (int k = sub; k < h.z; k += 64) {
        // (four places of the row's list per lane and round, the row's last place again beyond its end, all
        // of them asked for before the first is used)
        int id[4];
        AT v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) id[j] = segIdx[h.y + min(k + 16 * j, h.z - 1)];
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = partial[id[j]];
#pragma unroll
        for (int j = 0; j < 4; ++j) sum += k + 16 * j < h.z ? v[j] : (AT)0;
    }
    sum = group_sum<16>(sum);
    if (live && sub == 0) {
        sum += accumulate ? (AT)y[h.x] : (AT)0;
        y[h.x] = (VT)sum;
        if (ywide) ywide[h.x] = sum;
    }
}

// Which logical workgroup each workgroup of a launch shaped like the one-launch form's would take
// (XCC_ID, blockIdx / 8): every one of them exactly once when the dispatcher deals the workgroups
// round-robin to eight XCDs.
__global__ __launch_bounds__(kSliceThreads) void xcc_probe_kernel(unsigned *taken, int rep)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    if (threadIdx.x == 0) {
        smem[0] = (unsigned char)rep;  // (the LDS is asked for so that one workgroup fills a CU, as in the real launch)
        const int xcc = xcc_id();
        if (xcc < mx::kFusedXcds) atomicAdd(taken + xcc * ((int)gridDim.x / mx::kFusedXcds) + (int)blockIdx.x / mx::kFusedXcds, 1u);
    }
}

// MFMA probes: one wave, operands and accumulators exchanged lane by lane (raw register
// contents), so a host test can check the operand layout the tile kernels rely on.
__global__ void probe_mfma_f64_kernel(const double *A /*[64]*/, const double *B /*[64]*/, double *D /*[64][4]*/)
{
    const int lane = threadIdx.x & 63;
    v4f64 acc = {0.0, 0.0, 0.0, 0.0};
    acc = __builtin_amdgcn_mfma_f64_16x16x4f64(A[lane], B[lane], acc, 0, 0, 0);
    for (int i = 0; i < 4; ++i) D[lane * 4 + i] = acc[i];
}
__global__ void probe_mfma_f16_kernel(const _Float16 *A /*[64][8]*/, const _Float16 *B /*[64][8]*/, float *D /*[64][4]*/)
{
    const int lane = threadIdx.x & 63;
    v8f16 a, b;
    for (int j = 0; j < 8; ++j) {
        a[j] = A[lane * 8 + j];
        b[j] = B[lane * 8 + j];
    }
    v4f32 acc = {0.f, 0.f, 0.f, 0.f};
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
    for (int i = 0; i < 4; ++i) D[lane * 4 + i] = acc[i];
}

}  // namespace mxk

// ---- launchers (called from mx_run.cpp and the plan files; plain functions so that those need no HIP syntax)
namespace mx {

constexpr int kMaxDevices = 64;

// Device memory that exists without any allocation call: one array per GPU, part of the
// library's code object, held from the moment the library is loaded on that GPU until the
// process ends.  Host code must not use the array's name as an address (it is a host-side
// stand-in): the device address is asked for once per device and kept.
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

hipError_t static_scratch(void **ptr)
{
    static std::mutex lock;
    static void *addr[kMaxDevices] = {};
    *ptr = nullptr;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> hold(lock);
    if (!addr[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        addr[dev] = p;
    }
    *ptr = addr[dev];
    return hipSuccess;
}

template <typename VT, int NPT>
static void launch_csr_t(const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s, void *ywide)
{
    typedef typename mxk::Acc<VT>::type AT;
#define MX_LAUNCH_ROWS(C16, SCAN, COLS, BASE)                                                                       \
    hipLaunchKernelGGL((mxk::csr_rows_kernel<VT, NPT, true, C16, SCAN>), dim3(A.nBlocks), dim3(mxk::kBlock), 0, s,      \
                       A.rowPtr, (const void *)(COLS), (const VT *)A.val, (const VT *)x, (VT *)y,                      \
                       (const int4 *)A.blockDesc, (const int *)(BASE), A.cols, accumulate, (const VT *)nullptr, (AT *)ywide)
#define MX_LAUNCH_ROWS_DICT(SCAN)                                                                                    \
    hipLaunchKernelGGL((mxk::csr_rows_kernel<VT, NPT, true, true, SCAN, true>), dim3(A.nBlocks), dim3(mxk::kBlock), 0, \
                       s, A.rowPtr, (const void *)A.col16, (const VT *)A.codes, (const VT *)x, (VT *)y,                  \
                       (const int4 *)A.blockDesc, (const int *)A.colBase, A.cols, accumulate, (const VT *)A.dict, (AT *)ywide)
    static_assert(mxk::kBlock == 256, "a workgroup copies the 256 dictionary entries, one per lane");
    if (A.useDict && A.col16 && A.codes && A.dict) {
        if (A.scan) MX_LAUNCH_ROWS_DICT(true);
        else MX_LAUNCH_ROWS_DICT(false);
    } else if (A.col16 && A.scan) MX_LAUNCH_ROWS(true, true, A.col16, A.colBase);
    else if (A.col16) MX_LAUNCH_ROWS(true, false, A.col16, A.colBase);
    else if (A.scan) MX_LAUNCH_ROWS(false, true, A.col, nullptr);
    else MX_LAUNCH_ROWS(false, false, A.col, nullptr);
#undef MX_LAUNCH_ROWS
#undef MX_LAUNCH_ROWS_DICT
}

hipError_t launch_csr(mx_dtype dtype, const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s, void *ywide)
{
    if (A.nBlocks <= 0) return hipSuccess;
    if (dtype == MX_F64) {
        if (A.npt == 8) launch_csr_t<double, 8>(A, x, y, accumulate, s, ywide);
        else if (A.npt == 4) launch_csr_t<double, 4>(A, x, y, accumulate, s, ywide);
        else return hipErrorInvalidValue;
    } else {
        if (A.npt == 16) launch_csr_t<_Float16, 16>(A, x, y, accumulate, s, ywide);
        else if (A.npt == 8) launch_csr_t<_Float16, 8>(A, x, y, accumulate, s, ywide);
        else return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// The slice kernels take more dynamic LDS than the default limit.  The limit is a function attribute and
// belongs to the device that is current when it is set: whoever makes a slice layout (a plan, on its device)
// calls this once it exists; the launchers take no lock and ask nothing about the device.
template <typename VT>
static hipError_t slice_kernel_attributes()
{
    const void *fn[8] = {(const void *)mxk::csr_slice_kernel<VT, false, false>,       (const void *)mxk::csr_slice_kernel<VT, true, false>,
                         (const void *)mxk::csr_slice_kernel<VT, false, true>,        (const void *)mxk::csr_slice_kernel<VT, true, true>,
                         (const void *)mxk::csr_slice_kernel<VT, false, false, true>, (const void *)mxk::csr_slice_kernel<VT, true, false, true>,
                         (const void *)mxk::csr_slice_kernel<VT, false, true, true>,  (const void *)mxk::csr_slice_kernel<VT, true, true, true>};
    for (const void *f : fn) {
        const hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, mx::kSliceLdsMax);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}
hipError_t prepare_slice_kernels(mx_dtype dtype)
{
    static std::mutex attrLock;
    static bool attrSet[kMaxDevices][2] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    const int t = dtype == MX_F64 ? 0 : 1;
    std::lock_guard<std::mutex> hold(attrLock);
    if (attrSet[dev][t]) return hipSuccess;
    e = dtype == MX_F64 ? slice_kernel_attributes<double>() : slice_kernel_attributes<_Float16>();
    if (e == hipSuccess) attrSet[dev][t] = true;
    return e;
}

template <typename VT>
static hipError_t launch_slices_t(const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s, int what,
                                  const DeviceTiles *strips, void *ywide)
{
    typedef typename mxk::Acc<VT>::type AT;
    const bool dict = P.useDict && P.ecode && P.dict;
    const size_t lds = (size_t)P.sliceCols * sizeof(VT) + (size_t)((P.maxWgChunks + 3) & ~3) * 4 + 64 + (dict ? 256 * sizeof(AT) : 0);
    if (lds > (size_t)mx::kSliceLdsMax || P.sliceCols != mx::slice_cols(sizeof(VT) == 8 ? MX_F64 : MX_F16))
        return hipErrorInvalidValue;
    if (what != 2 && P.nWG > 0) {
#define MX_LAUNCH_SLICES(DICT, KEEP, VALUES, TABLE)                                                                                  \
    hipLaunchKernelGGL((mxk::csr_slice_kernel<VT, DICT, false, KEEP>), dim3(P.nWG), dim3(kSliceThreads), lds, s, (const int4 *)P.wgDesc, \
                       (const int4 *)P.waveDesc, P.chunkEnd, P.ecol, (const VT *)(VALUES), (const VT *)x, (AT *)P.partial, P.cols,        \
                       P.sliceCols, (const VT *)(TABLE), P.maxWgChunks, mxk::FusedArgs())
        if (dict && P.keep) MX_LAUNCH_SLICES(true, true, P.ecode, P.dict);
        else if (dict) MX_LAUNCH_SLICES(true, false, P.ecode, P.dict);
        else if (P.keep) MX_LAUNCH_SLICES(false, true, P.eval, nullptr);
        else MX_LAUNCH_SLICES(false, false, P.eval, nullptr);
#undef MX_LAUNCH_SLICES
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || what == 1) return e;
    const int nRowWG = (P.rows + mxk::kCombineRows * mxk::kBlock - 1) / (mxk::kCombineRows * mxk::kBlock);
    const int nLightWG = (P.nLight + mxk::kBlock - 1) / mxk::kBlock;
    const int nHeavyWG = (P.nHeavy + mxk::kBlock / 16 - 1) / (mxk::kBlock / 16);
    // strips that ride along (binary16 only; the caller has checked that they may: dense form,
    // rows of their own, x aligned)
    const bool ride = strips && strips->nWaves > 0 && (sizeof(VT) == 2 || strips->vidx);
    const int nStripWG = ride ? (strips->nWaves + 3) / 4 : 0;
    if (nStripWG + nRowWG + nLightWG + nHeavyWG == 0) return hipSuccess;
#define MX_LAUNCH_COMBINE(STRIPS, KEEP)                                                                                    \
    hipLaunchKernelGGL((mxk::slice_combine_kernel<VT, STRIPS, KEEP>), dim3(nStripWG + nRowWG + nLightWG + nHeavyWG),           \
                       dim3(mxk::kBlock), 0, s, (const AT *)P.partial, P.rowInfo, P.rows, nRowWG, P.lightRow,                    \
                       (const int4 *)P.lightIdx, P.nLight, nLightWG, (const int4 *)P.heavyInfo, P.nHeavy, P.segIdx, (VT *)y,    \
                       (accumulate || P.subset) ? 1 : 0, P.subset ? 1 : 0, (AT *)ywide, ride ? (const int4 *)strips->waveDesc : nullptr,   \
                       ride ? strips->hdr : nullptr, ride ? (const VT *)strips->tcVal : nullptr, (const VT *)x,              \
                       ride ? strips->nWaves : 0, nStripWG, nHeavyWG, P.lightQuads, ride ? strips->vidx : nullptr)
    if (ride && P.keep && sizeof(VT) == 2) MX_LAUNCH_COMBINE(true, true);  // (the strips' values stay where the slices' entries stay)
    else if (ride) MX_LAUNCH_COMBINE(true, false);
    else MX_LAUNCH_COMBINE(false, false);
#undef MX_LAUNCH_COMBINE
    return hipGetLastError();
}
hipError_t launch_slices(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s,
                         int what, const DeviceTiles *strips, void *ywide)
{
    if (P.rows <= 0) return hipSuccess;
    if (dtype == MX_F64) return launch_slices_t<double>(P, x, y, accumulate, s, what, strips, ywide);
    return launch_slices_t<_Float16>(P, x, y, accumulate, s, what, strips, ywide);
}
bool strips_can_ride(mx_dtype dtype, const DeviceTiles &T, const void *x)
{
    return dtype == MX_F16 && T.nWaves > 0 && T.dense && T.ownedRows && !((uintptr_t)x & 15);
}

template <typename VT>
static hipError_t launch_fused_t(const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s, void *ywide,
                                 unsigned *misplaced, unsigned seq)
{
    typedef typename mxk::Acc<VT>::type AT;
    const bool dict = P.useDict && P.ecode && P.dict;
    // (the list of the groups that fall to a workgroup takes the place of its chunk ends; behind them the places of
    // the sums of the workgroup's chunks)
    const int ldsInts = std::max(P.maxWgChunks, P.maxWgGroups + 1);
    const size_t lds = (size_t)P.sliceCols * sizeof(VT) + (size_t)((ldsInts + 3) & ~3) * 4 + 64 + (dict ? 256 * sizeof(AT) : 0) +
                       (size_t)P.maxWgChunks * 256;
    if (lds > (size_t)mx::kSliceLdsMax || P.sliceCols != mx::slice_cols(sizeof(VT) == 8 ? MX_F64 : MX_F16) || !P.fused || !P.wgGroups ||
        !P.groupNeed || !P.groupCount || !P.fusedTarget || !P.fusedSums || !P.claim || !misplaced || P.placesPerRow < 1 || P.placesPerRow > mx::kSliceLightSegs ||
        P.nWG <= 0 || P.nWG % mx::kFusedXcds)
        return hipErrorInvalidValue;
    mxk::FusedArgs fa;
    fa.y = y;
    fa.ywide = ywide;
    fa.wgGroups = P.wgGroups;
    fa.groupNeed = P.groupNeed;
    fa.groupCount = P.groupCount;
    fa.target = P.fusedTarget;
    fa.sums = P.fusedSums;
    fa.misplaced = misplaced;
    fa.claim = P.claim;
    fa.seq = seq;
    fa.rows = P.rows;
    fa.placesPerRow = P.placesPerRow;
    fa.accumulate = accumulate;
    fa.ldsCount = (int)lds - 16;  // (in the 64 spare bytes at the end)
#define MX_LAUNCH_FUSED(DICT, KEEP, VALUES, TABLE)                                                                                  \
    hipLaunchKernelGGL((mxk::csr_slice_kernel<VT, DICT, true, KEEP>), dim3(P.nWG), dim3(kSliceThreads), lds, s, (const int4 *)P.wgDesc, \
                       (const int4 *)P.waveDesc, P.chunkEnd, P.ecol, (const VT *)(VALUES), (const VT *)x, (AT *)P.partial, P.cols,       \
                       P.sliceCols, (const VT *)(TABLE), ldsInts, fa)
    if (dict && P.keep) MX_LAUNCH_FUSED(true, true, P.ecode, P.dict);
    else if (dict) MX_LAUNCH_FUSED(true, false, P.ecode, P.dict);
    else if (P.keep) MX_LAUNCH_FUSED(false, true, P.eval, nullptr);
    else MX_LAUNCH_FUSED(false, false, P.eval, nullptr);
#undef MX_LAUNCH_FUSED
    return hipGetLastError();
}
hipError_t launch_fused(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s, void *ywide,
                        unsigned *misplaced, unsigned seq)
{
    if (P.rows <= 0) return hipSuccess;
    if (dtype == MX_F64) return launch_fused_t<double>(P, x, y, accumulate, s, ywide, misplaced, seq);
    return launch_fused_t<_Float16>(P, x, y, accumulate, s, ywide, misplaced, seq);
}

hipError_t fused_placement_ok(int nWG, int *ok)
{
    static std::mutex lock;
    static int known[kMaxDevices] = {}, knownGrid[kMaxDevices] = {};  // 1 = holds, 2 = does not
    *ok = 0;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices || nWG < 8) return hipSuccess;
    std::lock_guard<std::mutex> hold(lock);
    if (known[dev] && knownGrid[dev] == nWG) {
        *ok = known[dev] == 1;
        return hipSuccess;
    }
    e = hipFuncSetAttribute((const void *)mxk::xcc_probe_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, mx::kSliceLdsMax);
    if (e != hipSuccess) return e;
    unsigned *taken = nullptr;
    e = hipMalloc((void **)&taken, (size_t)nWG * 4);
    if (e != hipSuccess) return e;
    std::vector<unsigned> h((size_t)nWG);
    bool holds = nWG % mx::kFusedXcds == 0;
    e = hipMemset(taken, 0, (size_t)nWG * 4);
    // (a few launches in a row, the way products follow each other)
    const int reps = 4;
    for (int rep = 0; rep < reps && e == hipSuccess && holds; ++rep) {
        hipLaunchKernelGGL(mxk::xcc_probe_kernel, dim3(nWG), dim3(kSliceThreads), mx::kSliceBytes + 2048, nullptr, taken, rep);
        e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpy(h.data(), taken, (size_t)nWG * 4, hipMemcpyDeviceToHost);
    (void)hipFree(taken);
    if (e != hipSuccess) return e;
    for (int b = 0; b < nWG; ++b) holds = holds && h[b] == (unsigned)reps;
    known[dev] = holds ? 1 : 2;
    knownGrid[dev] = nWG;
    *ok = holds;
    return hipSuccess;
}

hipError_t launch_tiles(mx_dtype dtype, const DeviceTiles &T, const void *x, void *y, int accumulate, hipStream_t s,
                        const void *ywide)
{
    if (T.nWaves <= 0) return hipSuccess;
    const int grid = (T.nWaves + 3) / 4;
    // the strip form overwrites its rows: it runs when the caller overwrites, or adds to rows that
    // the plan knows hold zero at that point; and it reads x in aligned 16-byte pieces
    if (dtype == MX_F16 && T.dense && (!accumulate || T.ownedRows) && !((uintptr_t)x & 15)) {
        hipLaunchKernelGGL(mxk::tile_dense_kernel, dim3(grid), dim3(mxk::kBlock), 0, s, (const int4 *)T.waveDesc, T.hdr,
                           (const _Float16 *)T.tcVal, (const _Float16 *)x, (_Float16 *)y, T.nWaves);
        return hipGetLastError();
    }
    if (dtype == MX_F64 && T.dense) {
        // the 8 x 8 blocks in a launch of their own: they add to the y the CSR part has written
        if (!accumulate || ((uintptr_t)x & 15)) return hipErrorInvalidValue;
        hipLaunchKernelGGL(mxk::tile_block_kernel, dim3(grid), dim3(mxk::kBlock), 0, s, (const int4 *)T.waveDesc, T.hdr,
                           (const double *)T.tcVal, (const double *)x, (double *)y, T.nWaves);
        return hipGetLastError();
    }
    if (dtype == MX_F64)
        hipLaunchKernelGGL((mxk::tile_kernel<double>), dim3(grid), dim3(mxk::kBlock), 0, s, (const int4 *)T.waveDesc, T.hdr,
                           T.atox, (const double *)T.tcVal, (const double *)x, (double *)y, T.nWaves, accumulate, (const double *)ywide);
    else
        hipLaunchKernelGGL((mxk::tile_kernel<_Float16>), dim3(grid), dim3(mxk::kBlock), 0, s, (const int4 *)T.waveDesc, T.hdr,
                           T.atox, (const _Float16 *)T.tcVal, (const _Float16 *)x, (_Float16 *)y, T.nWaves, accumulate, (const float *)ywide);
    return hipGetLastError();
}

hipError_t launch_probe_f64(const double *A, const double *B, double *D, hipStream_t s)
{
    hipLaunchKernelGGL(mxk::probe_mfma_f64_kernel, dim3(1), dim3(64), 0, s, A, B, D);
    return hipGetLastError();
}
hipError_t launch_probe_f16(const void *A, const void *B, float *D, hipStream_t s)
{
    hipLaunchKernelGGL(mxk::probe_mfma_f16_kernel, dim3(1), dim3(64), 0, s, (const _Float16 *)A, (const _Float16 *)B, D);
    return hipGetLastError();
}

}  // namespace mx
