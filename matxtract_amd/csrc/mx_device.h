// Device-side views shared by the plan code and the kernel launchers.
#pragma once
#include <hip/hip_runtime_api.h>

#include "matxtract_hip.h"

namespace mx {

// CSR matrix resident on the device, plus the row ranges of the CSR kernel's workgroups.
// col/val carry kCsrPad extra zero entries so that a wave's aligned 128-bit loads may overrun.
struct DeviceCsr {
    int rows = 0, nnz = 0;
    int *rowPtr = nullptr;    // [rows+1]
    int *col = nullptr;       // [nnz + kCsrPad]
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

// The CSR part re-laid for LDS-staged x: rows cut into blocks (one workgroup each), columns
// into panels of kPanelBytes of x; the entries of every (block, panel) group are contiguous and
// carry 16-bit row and column offsets inside their block / panel.
struct DevicePanels {
    int nBlocks = 0, nPanels = 0, panelCols = 0, maxBlockRows = 0;
    long long entries = 0;             // stored entries including the zero padding of groups
    int *blockRow = nullptr;           // [nBlocks+1]
    int *listPtr = nullptr;            // [nBlocks+1] range of each block's groups in `list`
    int *list = nullptr;               // [groups][4] {panel, first entry, end entry, 0}; entry offsets are multiples of 8
    unsigned short *erow = nullptr;    // [entries] row - blockRow[b]
    unsigned short *ecol = nullptr;    // [entries] col - panel*panelCols
    void *eval = nullptr;              // [entries]
};
constexpr int kPanelBytes = 65536;     // one panel of x held in LDS
constexpr int kPanelThreads = 1024;    // one workgroup per CU
constexpr int kPanelListMax = 512;     // most panels one matrix may have for the panel kernel
constexpr int kPanelListPad = 6;       // a block's group list is padded to a multiple of this (the entry ring depth)
// The panel kernel copies x in 16-byte vectors: the column count must be a whole number of them.
inline bool panels_possible(mx_dtype d, int cols)
{
    const int epv = d == MX_F64 ? 2 : 8, pw = kPanelBytes / (d == MX_F64 ? 8 : 2);
    return cols >= epv && cols % epv == 0 && (cols + pw - 1) / pw <= kPanelListMax;
}
inline int panel_cols(mx_dtype d) { return kPanelBytes / (d == MX_F64 ? 8 : 2); }
inline int panel_max_block_rows(mx_dtype d) { return d == MX_F64 ? 4096 : 16384; }  // LDS accumulators

hipError_t launch_panels(mx_dtype dtype, const DevicePanels &P, const void *x, void *y, int cols, int accumulate,
                         hipStream_t s);
hipError_t launch_csr(mx_dtype dtype, const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_tiles(mx_dtype dtype, const DeviceTiles &T, const void *x, void *y, int accumulate, hipStream_t s);
hipError_t launch_probe_f64(const double *A, const double *B, double *D, hipStream_t s);
hipError_t launch_probe_f16(const void *A, const void *B, float *D, hipStream_t s);

}  // namespace mx
