// Device-side views shared by the plan code and the kernel launchers.
#pragma once
#include <hip/hip_runtime_api.h>

#include "matxtract_hip.h"

namespace mx {

// CSR matrix resident on the device, plus the row ranges of the CSR kernel's workgroups.
// col/val carry kCsrPad extra zero entries so that a wave's aligned 128-bit loads may overrun.
struct DeviceCsr {
    int rows = 0, cols = 0, nnz = 0;
    int *rowPtr = nullptr;    // [rows+1]
    int *col = nullptr;       // [nnz + kCsrPad], or nullptr when the 16-bit form below is used
    unsigned short *col16 = nullptr;  // [nnz + kCsrPad] column ids as offsets from colBase[workgroup]
    int *colBase = nullptr;           // [nBlocks] lowest column of each workgroup's entries
    void *val = nullptr;      // [nnz + kCsrPad]
    int *blockDesc = nullptr; // [nBlocks][4] {first row, end row, first entry, end entry} per workgroup
    int nBlocks = 0;
    int npt = 0;              // entries per lane per tile the rows were packed for
};
constexpr int kCsrPad = 1088;  // a wave may read one whole wave tile (64*16 entries) past the end

// Entries per lane per tile of the CSR kernel (a tile is 256 lanes wide).
int csr_entries_per_lane(mx_dtype dtype);

// Bitmap tiles resident on the device (the reference's chunkPtr / fragPtr / fragBit / tcVal /
// sparse_AToX_index, restricted to the chunks the tile kernel executes).
struct DeviceTiles {
    int chunkNum = 0;  // executed chunks
    int dRows = 0;     // 8*chunkNum, or fewer when the last chunk is ragged
    int frags = 0, vals = 0;
    int *chunkPtr = nullptr;  // [chunkNum+1]
    int *fragPtr = nullptr;   // [frags+1]
    void *fragBit = nullptr;  // [frags] u32 | u64
    void *tcVal = nullptr;    // [vals]
    int *atox = nullptr;      // [frags*fragK] indices into the x handed to the kernel
    int *rowIdx = nullptr;    // [dRows] output row of each tile row; nullptr = identity
};

// The CSR part re-laid for x resident in LDS: columns cut into S slices of kSliceBytes of x,
// rows into groups; workgroup (group, slice) handles its rows in sub-blocks whose accumulators
// fit LDS.  Entries carry 16-bit row offsets inside their sub-block and column offsets inside
// their slice; the entries of each (workgroup, sub-block) are contiguous, row-major, padded
// with zero entries to a multiple of 8.
struct DeviceSlices {
    int nWG = 0, S = 0, rows = 0, cols = 0, maxSubRows = 0;
    long long entries = 0;
    int *wgSubPtr = nullptr;         // [nWG+1] range of each workgroup's sub-blocks in `subs`
    int *subs = nullptr;             // [subBlocks][4] {first row, rows, first entry, end entry}
    unsigned short *erow = nullptr;  // [entries] row - sub-block's first row
    unsigned short *ecol = nullptr;  // [entries] col - slice * slice_cols
    void *eval = nullptr;            // [entries]
    void *partial = nullptr;         // [S][rows] accumulators (only when S > 1)
};
constexpr int kSliceBytes = 131072;   // the slice of x a workgroup keeps in LDS
constexpr int kSliceThreads = 1024;   // one workgroup per CU
constexpr int kSliceAccBytes = 24576; // LDS left for the row accumulators of a sub-block
inline int slice_cols(mx_dtype d) { return kSliceBytes / (d == MX_F64 ? 8 : 2); }
inline int slice_sub_rows(mx_dtype d) { return kSliceAccBytes / (d == MX_F64 ? 8 : 4); }

// `what`: 0 = slice kernel then combine kernel, 1 = slice kernel only, 2 = combine kernel only
hipError_t launch_slices(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s,
                         int what = 0);
hipError_t launch_csr(mx_dtype dtype, const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_tiles(mx_dtype dtype, const DeviceTiles &T, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_probe_f64(const double *A, const double *B, double *D, hipStream_t s);
hipError_t launch_probe_f16(const void *A, const void *B, float *D, hipStream_t s);

}  // namespace mx
