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
    bool scan = false;        // sum the rows of a tile by a segmented scan (row lengths vary a lot)
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

// The CSR part re-laid for x resident in LDS.  The columns are cut into S slices of sliceCols
// columns (a slice of x fits LDS); every slice cuts the rows into groups of about equal entries of
// that slice, and a workgroup owns the entries of one group of one slice.  Inside a workgroup the group's rows are
// sorted by their number of entries in the slice and cut into chunks of 64 rows, one row per
// lane (a sliced-ELL layout: every row of a chunk is padded to the chunk's longest row, and the
// sort keeps that padding small).  A lane walks its row E entries -- one "step" -- at a time
// (E = 2 binary64, 4 binary16); chunks end on step boundaries.  The chunks of a workgroup are
// dealt to its waves so that the waves' step counts are about equal, a wave's chunks follow
// each other in the wave's stream, and the stream is stored in batches of kSliceBatchEntries
// entries per lane (zero-padded to a whole batch at the end): per batch the lanes' column
// offsets (lanes contiguous), then their values -- binary16: lanes contiguous; binary64: one
// sub-block of 16 bytes per lane for every step -- so that every load of a wave is one
// contiguous stretch.
struct DeviceSlices {
    int nWG = 0, S = 0, rows = 0, cols = 0, sliceCols = 0;
    int maxGroupRows = 0;             // rows of the largest group (their sums are parked in LDS)
    long long steps = 0;              // total steps stored (64 lanes * E entries each)
    int *wgDesc = nullptr;            // [nWG][4] {first row, rows, slice, first chunk}
    int *waveDesc = nullptr;          // [nWG*kSliceWaves][4] {first batch, batches, first chunk inside the workgroup, chunks}
    int *chunkEnd = nullptr;          // [chunks] step, counted from the wave's first, at which the chunk ends
    unsigned short *chunkRows = nullptr;  // [chunks][64] row - first row of the group; 0xffff = no row.
                                          // A group's chunks are padded to whole multiples of 64 rows.
    unsigned short *ecol = nullptr;   // [batches][64][kSliceBatchEntries] col - slice * sliceCols
    void *eval = nullptr;             // [batches] values, laid out as described above
    void *partial = nullptr;          // [S][rows] accumulators (only when S > 1)
};
constexpr int kSliceBytes = 131072;   // the slice of x a workgroup keeps in LDS
constexpr int kSliceLdsMax = 163840;  // LDS of a CU
constexpr int kSliceGroupRows = 3072; // most rows a group may have: their sums and row ids share the rest of LDS
constexpr int kSliceWaves = 8;        // waves per workgroup; one workgroup per CU
constexpr int kSliceThreads = 64 * kSliceWaves;
inline int slice_cols(mx_dtype d) { return kSliceBytes / (d == MX_F64 ? 8 : 2); }
constexpr int kSliceBatchEntries = 8;  // entries a lane loads at a time
inline int slice_step_entries(mx_dtype d) { return d == MX_F64 ? 2 : 4; }  // kSliceE

// `what`: 0 = slice kernel then combine kernel, 1 = slice kernel only, 2 = combine kernel only
hipError_t launch_slices(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s,
                         int what = 0);
hipError_t launch_csr(mx_dtype dtype, const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_tiles(mx_dtype dtype, const DeviceTiles &T, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_probe_f64(const double *A, const double *B, double *D, hipStream_t s);
hipError_t launch_probe_f16(const void *A, const void *B, float *D, hipStream_t s);

}  // namespace mx
