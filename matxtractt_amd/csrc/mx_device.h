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
    // a matrix with at most 256 distinct values (a stencil, a graph): one byte per entry that
    // names the value, and the values themselves (padded to 256); used with col16 only
    unsigned char *codes = nullptr;  // [nnz + kCsrPad]
    void *dict = nullptr;            // [256]
    int nDict = 0;
    bool useDict = false;            // the plan found this form the faster one
};
constexpr int kCsrPad = 1088;  // a wave may read one whole wave tile (64*16 entries) past the end

// Entries per lane per tile of the CSR kernel (a tile is 256 lanes wide).
int csr_entries_per_lane(mx_dtype dtype);

// Tiles resident on the device, re-packed for the tile kernels.  The fragments the plan
// selects are expanded from the reference's encoding (bitmap + packed values) into full
// fragM x fragK blocks, zeros included (row-major inside a block), so that a lane can load
// exactly what the matrix core wants from it with no decoding; the plan only selects fragments
// that are mostly full.  The columns of a chunk's selected fragments are first put in ascending
// order of the caller's column ids and cut into blocks anew (the reference orders them by their
// rank among the dense columns, which scatters neighbours): gathers touch fewer lines, and dense
// strips become blocks of consecutive columns.  (Rows of binary16 strips do not come from the
// reference's chunks at all: the plan groups them into chunks of its own, see `dense`.)  The
// blocks are grouped into "steps" -- what one wave feeds to the matrix core at a time: two
// halves of up to tile_slots(dtype)/2 blocks.  A chunk with more
// selected fragments than half a step takes whole steps of its own (filling half 0 first; its
// two halves are added at the end); smaller chunks share a step, one per half.  Per step:
//   hdr    kTileHdr dwords: [0,16) output row of each of the 8 rows of half 0 and half 1
//          (-1 = none); [16] flags (1 = store the sums after this step, 2 = the halves are
//          different chunks); [17],[18] blocks in half 0 and half 1; [19],[20] first value
//          and blocks in half 0 of the step four further on (a wave learns where to prefetch
//          from there; its own last step when it has no such step); [21,29) first column of
//          the block in each slot (-1 = none), used by the strip form of the binary16 kernel.
//   atox   64 column ids (slot-major), -1 for unused ones
//   values the blocks of half 0, then those of half 1; nothing for absent blocks.
// Waves take whole chunks: waveDesc = {first step, end step, first value of the wave's first
// four steps, blocks in half 0 of each of them (one byte each), 0}.
struct DeviceTiles {
    int chunkNum = 0;  // chunks with at least one selected fragment
    int frags = 0, vals = 0;   // selected fragments, entries they hold
    long long stored = 0;      // values stored (zeros included)
    int steps = 0, nWaves = 0;
    bool dense = false;        // binary16 chunks the plan formed from rows of dense strips: every block's eight
                               // columns are consecutive and every chunk fits one step
                               // (two share a step when both fit a half): tile_dense_kernel can run it
    bool ownedRows = false;    // set by the plan: no row of these tiles gets anything from the CSR part
    // binary64 `dense` layouts (blocks of 8 x 8 on rows that the CSR part shares) when they ride in the
    // combine kernel's launch: per step 128 indices into the slice layout's sums -- half h, row i,
    // place j at [64h + 8i + j], -1 = none -- set on the step after which the half's sums are stored
    int *vidx = nullptr;
    int *waveDesc = nullptr;   // [nWaves][8]
    int *hdr = nullptr;        // [steps][kTileHdr]
    int *atox = nullptr;       // [steps][64]
    void *tcVal = nullptr;     // blocks
};
constexpr int kTileHdr = 32;
inline int tile_slots(mx_dtype d) { return d == MX_F64 ? 16 : 8; }  // fragment slots per step
// slot of block i of half h: binary64 MFMA j takes slots 2j and 2j+1, binary16 slots 0..3 and 4..7
inline int tile_slot(mx_dtype d, int half, int i) { return d == MX_F64 ? 2 * i + half : 4 * half + i; }

// The CSR part (or the rows of it that the plan selects) re-laid for x resident in LDS.  The
// columns are cut into S slices of sliceCols columns (a slice of x fits LDS).  The entries of
// a row that fall into one slice form a "virtual row"; one longer than the plan's cap is cut
// into several, so a matrix row owns one or more virtual rows and its result is the sum of
// theirs.  Per slice the virtual rows are sorted by length (among equals by the kind of their
// row -- sole virtual row, a few, many -- then by row) and cut into chunks of 64, one
// virtual row per lane (a sliced-ELL layout: every row of a chunk is padded to the chunk's
// longest, and the sort keeps that padding small).  A slice gets workgroups in proportion to
// its entries, its chunks are dealt to them longest first, and inside a workgroup to its waves
// the same way.  A lane walks its virtual row one entry -- one "step" -- at a time; a wave's
// chunks follow each other in the wave's stream, which is stored in batches of
// kSliceBatchEntries entries per lane
// (zero-padded to a whole batch at the end): per batch the lanes' column offsets (lanes
// contiguous), then their values -- binary16: lanes contiguous; binary64: one sub-block of 16
// bytes (two values) per lane -- so that every load of a wave is one contiguous stretch.
// Chunks are numbered workgroup by workgroup, wave by wave; virtual row v = 64 * chunk + lane
// puts its sum into partial[v], and a second kernel turns those into y: rowInfo[r] is the
// virtual row of a matrix row that owns exactly one, -1 for a row that owns none, -2 for a row
// that owns several.  Of those, the rows with up to kSliceLightSegs virtual rows are lightRow[i]
// with their virtual rows in lightIdx[i][kSliceLightSegs] (-1 = none); the rows with more are
// heavyInfo[i] = {row, first index into segIdx, count, 0} with their virtual rows listed in
// segIdx.
struct DeviceSlices {
    int nWG = 0, S = 0, rows = 0, cols = 0, sliceCols = 0;
    int maxWgChunks = 0;              // chunks of the largest workgroup (their ends are kept in LDS)
    long long steps = 0;              // total steps stored (64 lanes, one entry each)
    long long chunks = 0;             // total chunks
    int nnz = 0;                      // entries held
    int vrows = 0;                    // virtual rows
    bool subset = false;              // only some rows are held: their sums are added to y, the others left alone
    int *wgDesc = nullptr;            // [nWG][4] {slice, first chunk, chunks, 0}
    int *waveDesc = nullptr;          // [nWG*kSliceWaves][4] {first batch, batches, first chunk inside the workgroup, chunks}
    int *chunkEnd = nullptr;          // [chunks] step, counted from the wave's first, at which the chunk ends
    unsigned short *ecol = nullptr;   // [batches][64][kSliceBatchEntries] col - slice * sliceCols
    void *eval = nullptr;             // [batches] values, laid out as described above
    // a matrix with at most 256 distinct values: a byte per entry (at the place of its column
    // offset) that names the value, and the values (padded to 256)
    unsigned char *ecode = nullptr;   // [batches][64][kSliceBatchEntries]
    void *dict = nullptr;             // [256]
    int nDict = 0;
    bool useDict = false;             // the plan found this form the faster one
    void *partial = nullptr;          // [chunks*64] accumulators
    int *rowInfo = nullptr;           // [rows, padded to a multiple of 4 with -2]
    int *segIdx = nullptr;            // [vrows] virtual rows listed matrix row by matrix row
    int *lightRow = nullptr;          // [nLight]
    int *lightIdx = nullptr;          // [nLight][4 * lightQuads]
    int lightQuads = 2;               // 1 when no light row has more than four virtual rows
    int *heavyInfo = nullptr;         // [nHeavy][4]
    int nLight = 0, nHeavy = 0;
    int mostVrows = 0;                // most virtual rows of any row
    bool keep = false;                // the entries are read with plain loads (they may stay in the caches), not streamed
    // The one-launch form (csr_slice_kernel<.., FUSED>), when the layout was made for it: the rows are cut
    // into groups of kFusedGroupRows, the groups into one contiguous range per XCD, and the virtual rows
    // of a slice are ordered by group before length, so that a workgroup's chunks cover a contiguous run
    // of groups.  Logical workgroups [k * nWG / 8, (k + 1) * nWG / 8) belong to XCD k, and a workgroup of
    // the launch that runs on XCD k takes one of those (which one: blockIdx / 8), so all workgroups that
    // hold sums of a group share an L2: they store their sums with plain stores, which meet there,
    // count themselves off on the group's counter with an atomic that executes there, and the one that
    // completes the count adds the sums of the group's rows up and writes y.  Nobody waits.  The sums do
    // not go to `partial` in this form but to fusedSums, laid out for the one who adds: the k-th
    // virtual row of row r at [((r / G) * placesPerRow + k) * G + r % G], G = kFusedGroupRows, so that a
    // wave that adds 64 consecutive rows reads 64 consecutive sums per place and needs no index list;
    // fusedTarget names that place for every virtual row (a workgroup keeps its chunks' part of it in
    // LDS, which bounds the chunks a workgroup may have).  A place that no virtual row owns keeps the zero
    // it was allocated with, so the one who adds takes all placesPerRow places of a row without asking how
    // many count.  The arrays above stay valid for the two-launch form, which a plan falls back to.
    bool fused = false;
    int nGroups = 0, maxWgGroups = 0;
    int placesPerRow = 0;             // most virtual rows of a row (1 .. 8)
    int *wgGroups = nullptr;          // [nWG][2] {first group, groups} whose counters the workgroup bumps
    int *groupNeed = nullptr;         // [nGroups] workgroups that bump the group's counter
    int *groupCount = nullptr;        // [nGroups] the counters; zero between launches (the last arriver clears its own)
    int *fusedTarget = nullptr;       // [chunks * 64] where virtual row 64 * chunk + lane puts its sum (a spare place for padding lanes)
    void *fusedSums = nullptr;        // [nGroups * placesPerRow * G + 64] accumulators; zero where no virtual row writes
    unsigned *claim = nullptr;        // [nWG] launches in which each logical workgroup's work was taken (once each)
};
constexpr int kFusedGroupRows = 256;  // rows whose sums one arriver adds up at a time
constexpr int kFusedXcds = 8;         // L2 domains of the device the one-launch form is laid out for
constexpr int kFusedWgChunks = 96;    // most chunks of a workgroup in that form (their targets, 256 bytes each, share the LDS with x)
constexpr int kFusedWgGroups = 255;  // most groups a workgroup may hold sums of
constexpr int kFusedAddBytes = 100 * 1024;  // most bytes of sums under one workgroup (groups x places x a group's rows) for which
                                            // the form is taken unasked: the slowest workgroup of a launch reads that much after its last
                                            // chunk (about 70 ns per 2 KB), and beyond this a second launch is the faster way
constexpr int kFusedSlicesMost = 8;          // ... and most slices: every XCD copies every slice of x in this form (a slice's workgroups are
                                            // spread over all eight), 64 ns a slice more than when one XCD has a slice to itself
constexpr long long kKeepL2Bytes = 24LL << 20;      // entries of a slice layout up to this size fit the eight L2s beside x and the sums
constexpr long long kKeepCacheBytes = 192LL << 20;  // ... and up to this size the memory-side cache beside everything else a product touches
constexpr long long kKeepHandoffBytes = 10LL << 20;  // what the second launch must move per product (sums, row tables, y) to push streamed
                                                    // entries out of the memory-side cache fast enough for plain loads to pay
constexpr int kSliceBytes = 131072;   // the slice of x a workgroup keeps in LDS
constexpr int kSliceLdsMax = 163840;  // LDS of a CU
constexpr int kSliceWgChunks = 4096;  // most chunks a workgroup may have
constexpr int kSliceWaves = 8;        // waves per workgroup; one workgroup per CU
constexpr int kSliceThreads = 64 * kSliceWaves;
inline int slice_cols(mx_dtype d) { return kSliceBytes / (d == MX_F64 ? 8 : 2); }
constexpr int kSliceBatchEntries = 8;  // entries a lane loads at a time
constexpr int kSliceChunkCost = 2;     // what ending a chunk costs a wave, in steps of its stream (for dealing chunks out evenly)
inline int slice_step_entries(mx_dtype) { return 1; }  // entries a lane takes per step; chunks end between steps
constexpr int kSliceLightSegs = 8;     // rows with at most this many virtual rows are summed by one lane

// The sums of the virtual rows (DeviceSlices::partial) of mx_spmv_static live in a fixed array
// in device memory instead of the plan's own buffer: static_scratch gives the address of the
// current device's copy (looked up once per device, no allocation).
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;  // the largest benchmark workload needs 27 MB
hipError_t static_scratch(void **ptr);

}  // namespace mx
#include <vector>
namespace mx {
// One chunk of a slice on its way into the layout: `first` = index of its first virtual row in
// the sorted order of virtual rows, n = how many it has (64 but for the last of a slice), steps
// = the length of its longest (first) member.
struct SliceChunk {
    int first, n, steps;
};
// What plan_slice_chunks decides: the descriptors the kernels read (DeviceSlices) and, for every
// chunk in its final numbering (workgroup by workgroup, wave by wave), where it comes from and at
// which step of the streams it starts.
struct SlicePlan {
    int nWG = 0, maxWgChunks = 0;
    long long totalSteps = 0, totalChunks = 0;
    std::vector<int> wgDesc, waveDesc, chunkEnd;
    std::vector<int> chunkSlice, chunkFirst, chunkN, chunkSteps;
    std::vector<long long> chunkStep0;
    // one-launch form only
    int nGroups = 0, maxWgGroups = 0;
    std::vector<int> wgGroups, groupNeed;
};
int plan_slice_chunks(mx_dtype dtype, int budget, int S, const std::vector<std::vector<SliceChunk>> &sliceChunks, SlicePlan &P);
// The plan of the one-launch form from the records of the virtual rows (in the order of the rows, ascending
// columns inside a row: the numbering both layout routes use): `sorted` receives the order in which the
// virtual rows are laid out and P the workgroups, waves, chunks and groups.  `mode` 1: wherever the matrix
// suits the form; 2: only while the busiest workgroup has at most kFusedAddBytes of sums under it.  Returns 1
// when the form is taken (*places = places per row), 0 when it is not (nothing filled), a negative error code
// when the plan cannot be made (the error is set).
int plan_fused_records(mx_dtype dtype, int budget, int S, int rows, int cap, const int *rowPtr, const int *segPtr, const int *vSlice,
                       const int *vLen, int nV, int mode, std::vector<int> &sorted, SlicePlan &P, int *places);
// Where the virtual rows of the one-launch form put their sums (DeviceSlices::fusedTarget), from the places the
// layout gave them.
void fused_targets(int rows, int nGroups, int places, long long totalChunks, const int *segPtr, const int *segIdx, std::vector<int> &target);
constexpr int kSlicePadSteps = 16;  // spare zero steps after the last of the streams
// The slice layout built on the device from a CSR matrix in device memory (mx_layout.hip): the
// arrays of `D` equal those of the host route byte for byte.  `elsewhere_dev`: optional marks per
// row (device memory) as in the host route.  segPtrOut / segIdxOut (optional): host copies of the
// virtual rows of every row.  `fused` (1 or 2, as in plan_fused_records): the one-launch form where the matrix
// suits it (D.fused says whether it did) -- the records of the virtual rows come down, the plan goes up, the
// entries never leave the device.
int build_slices_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev,
                        int nCU, int S, const char *elsewhere_dev, DeviceSlices &D, hipStream_t s, std::vector<int> *segPtrOut = nullptr,
                        std::vector<int> *segIdxOut = nullptr, int fused = 0);

// For plans made from a matrix that lives in device memory: the caller's arrays looked at before
// they are used as addresses; the mean number of distinct lines of x per wave-wide gather (sampled
// as on the host); the row-tile form from device arrays (`desc` = pack_rows of the row pointers).
int check_csr_device(int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, hipStream_t s, const char *who);
int lines_per_gather_device(mx_dtype dtype, int nnz, const int *col_dev, hipStream_t s, double *out);
int upload_csr_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev,
                      const std::vector<int> &desc, bool scan, DeviceCsr &A, hipStream_t s);

// The host half of a hybrid plan done on the device (mx_hybrid.hip), for a matrix that lives in
// device memory.  analyse() runs the extraction and counts what the plan's decision needs;
// csr_part() assembles the CSR part (residual rows, then the entries of A_dd that stay) in the
// caller's numbering, in new device arrays that pass to the caller; strip_layout() lays the
// binary16 strip chunks out as steps (the caller plans the steps from the chunks' block counts,
// as the host route does).  All arrays equal the host route's byte for byte.
// The device arrays of a partition that was made on the device (mx_partition::twin): the two orders, A_dd and
// the residual, the tile encoding.  HybridDevice::adopt plans from them without any copy.
struct PartitionTwin {
    mx_dtype dtype = MX_F64;
    int rows = 0, cols = 0, nnz = 0, dRows = 0, dCols = 0, nDD = 0, nCD = 0;
    void *order = nullptr;  // descColId [cols], descRowId [rows] (its first dRows are rId)
    int *dc = nullptr, *dr = nullptr;
    void *split = nullptr;  // ddRowPtr, ddColInd, ddVal, cdRowPtr, cdColInd, cdVal
    int *ddp = nullptr, *ddc = nullptr, *cdp = nullptr, *cdc = nullptr;
    void *ddv = nullptr, *cdv = nullptr;
    mx_device_tiles T{};
};

struct HybridCounts {
    long long generalFrags = 0, generalEntries = 0;  // fragments that pass the fill gate (after the strips took their rows)
    long long stripEntries = 0, stripBlocks = 0;     // binary16 strip chunks, or binary64 8 x 8 blocks (blocks64)
    long long stripBlocksOff = 0;                    // of stripBlocks: blocks of chunks that start off the grid of eight columns
    bool blocks64 = false;
    int dRows = 0, dCols = 0, nnzRowD = 0, frags = 0;  // what the extraction selected; fragments of the tile encoding
    std::vector<int> stripChunkBlocks, stripChunkEntries;  // per strip chunk, in layout order
};
struct HybridDevice {
    struct Impl;
    Impl *impl = nullptr;
    HybridDevice() = default;
    HybridDevice(const HybridDevice &) = delete;
    HybridDevice &operator=(const HybridDevice &) = delete;
    ~HybridDevice();
    // minVals: entries a fragment needs to pass the gate; want*: which forms the flags allow
    int analyse(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *col_dev, const void *val_dev, float tau_c,
                float tau_r, int minVals, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts, hipStream_t s);
    // the same counts for an extraction that is there already: the arrays of `twin` are used where they are and
    // stay the twin's
    int adopt(const PartitionTwin &twin, int minVals, bool wantGeneral, bool wantStrips, bool wantBlocks, HybridCounts *counts, hipStream_t s);
    // stripRows_dev: marks of the rows the strips write (null when keepStrips is false or there are none).
    // keepGeneral: the fragments that pass the gate go to the general tile form -- tile_chunks and tile_layout
    // come first then, and the values of that layout are filled here.
    // keepBlocks (binary64, alone): the entries of the 8 x 8 blocks leave the CSR part and the rows of block chunks are
    // marked 2 -- block_chunks comes first then.
    int csr_part(bool keepStrips, bool keepGeneral, bool keepBlocks, int **rowPtr_dev, int **col_dev, void **val_dev, int *nnz,
                 char **stripRows_dev);
    // the binary64 block form: blocks per block row that has any and those block rows (ascending); then the layout
    // from the caller's steps (10 ints per step as for tile_layout)
    int block_chunks(std::vector<int> &blocks, std::vector<int> &blockRows);
    int block_layout(const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0, const std::vector<int> &waveDesc,
                     long long totalBlocks, DeviceTiles &T);
    // the general tile form: blocks per chunk that has any (chunk order); then the layout from the caller's steps --
    // stepDesc has 10 ints per step: the 8 of strip_layout with chunks numbered as in `blocks`, then the first block
    // of half 0 inside its chunk (a chunk of more blocks than a step holds takes several), then 0
    int tile_chunks(bool keepStrips, std::vector<int> &blocks);
    int tile_layout(bool keepStrips, const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0, const std::vector<int> &waveDesc,
                    long long totalBlocks, DeviceTiles &T);
    // stepDesc: 8 ints per step {chunk of half 0, chunk of half 1 (-1 none, -2 the first goes on), flags, blocks in half 0,
    // blocks in half 1, first value, first value and blocks in half 0 of the step four further on}; chunkBlock0: first block
    // of every chunk; T receives waveDesc, hdr, atox and tcVal
    int strip_layout(const std::vector<int> &stepDesc, const std::vector<int> &chunkBlock0, const std::vector<int> &waveDesc,
                     long long totalBlocks, DeviceTiles &T);
};

// `what`: 0 = slice kernel then combine kernel, 1 = slice kernel only, 2 = combine kernel only
// `strips` (optional): a tile layout in the dense binary16 form whose steps workgroups of the
// combine kernel's launch run as well (strips_can_ride says whether a layout may); the rows of
// those strips must be marked in the slice layout (rowInfo -2) so that the combine kernel leaves
// them alone.
// `ywide` (optional, all three launchers): an array of accumulators (binary32 for binary16
// plans), one per row.  The CSR launchers also store every sum they write to y there,
// unrounded; the tile launcher reads the old y of its rows from there instead of y, so that a
// row which gets sums from both parts is rounded to the value type once.
hipError_t launch_slices(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s,
                         int what = 0, const DeviceTiles *strips = nullptr, void *ywide = nullptr);
// Raises the dynamic-LDS limit of the slice kernels on the current device (idempotent).  Every route that makes
// a DeviceSlices calls it before handing the layout out; launch_slices and launch_fused rely on that.
hipError_t prepare_slice_kernels(mx_dtype dtype);
// The one-launch form of the same product (P.fused).  `misplaced`: a word in host memory that the
// device can write (one per process); a workgroup that finds itself on another XCD than the layout
// assumes sets it, and the product of that launch cannot be trusted.
// `seq`: how many one-launch products of this layout were queued before this one (the kernel holds
// the claims of its logical workgroups against it).
hipError_t launch_fused(mx_dtype dtype, const DeviceSlices &P, const void *x, void *y, int accumulate, hipStream_t s,
                        void *ywide, unsigned *misplaced, unsigned seq);
// Whether the workgroups of a launch of `nWG` workgroups shaped like the one-launch form's take every
// logical workgroup (XCC_ID, blockIdx / 8) exactly once on the current device (asked once per device
// and grid size, by launching a probe that reads the XCC_ID register); *ok = 0 when not -- a device
// without eight XCDs, or a dispatcher that does not deal workgroups round-robin.
hipError_t fused_placement_ok(int nWG, int *ok);
bool strips_can_ride(mx_dtype dtype, const DeviceTiles &T, const void *x);
hipError_t launch_csr(mx_dtype dtype, const DeviceCsr &A, const void *x, void *y, int accumulate, hipStream_t s,
                      void *ywide = nullptr);
hipError_t launch_tiles(mx_dtype dtype, const DeviceTiles &T, const void *x, void *y, int accumulate, hipStream_t s,
                        const void *ywide = nullptr);
hipError_t launch_probe_f64(const double *A, const double *B, double *D, hipStream_t s);
hipError_t launch_probe_f16(const void *A, const void *B, float *D, hipStream_t s);

}  // namespace mx
