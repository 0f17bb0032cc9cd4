// What the translation units behind the plans share: the host-side layouts (mx_host_layout.cpp), the plan and
// its making (mx_plan.cpp from host arrays, mx_plan_device.cpp from device arrays, mx_plan_view.cpp for
// looking into one), the products and their timing (mx_run.cpp), the search for the extraction fractions
// (mx_tune.cpp) and the reference's one-shot calls (mx_oneshot.cpp).
#pragma once
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "mx_device.h"
#include "mx_internal.h"

#define MX_HIP(call)                                                                                  \
    do {                                                                                              \
        hipError_t e_ = (call);                                                                       \
        if (e_ != hipSuccess) {                                                                       \
            mx::set_error(std::string(#call) + ": " + hipGetErrorString(e_));                         \
            return MX_ERR_DEVICE;                                                                     \
        }                                                                                             \
    } while (0)

namespace mxp {

using mx::set_error;

// ---- mx_host_layout.cpp --------------------------------------------------------------------------------
// MX_ERR_DEVICE (with the error text set) when the process sees no HIP device.
int need_device();
// hipMalloc + copy of n elements, `pad` zeroed elements behind them (at least one element is allocated).
template <typename T>
inline int upload(T **dst, const T *src, size_t n, size_t pad = 0)
{
    *dst = nullptr;
    const size_t total = std::max<size_t>(n + pad, 1);
    MX_HIP(hipMalloc((void **)dst, total * sizeof(T)));
    if (pad || n == 0) MX_HIP(hipMemset(*dst, 0, total * sizeof(T)));
    if (n) MX_HIP(hipMemcpy(*dst, src, n * sizeof(T), hipMemcpyHostToDevice));
    return MX_OK;
}
int upload_bytes(void **dst, const void *src, size_t n, size_t pad = 0);
void pack_rows(const int *rowPtr, int rows, int npt, std::vector<int> &desc);
void free_csr(mx::DeviceCsr &A);
void free_tiles(mx::DeviceTiles &T);
void free_slices(mx::DeviceSlices &P);
// Column slices of x a matrix of this shape gets on a machine with nCU compute units (0: the slice form does not fit).
int slice_count(mx_dtype dtype, int rows, int cols, int nnz, int nCU);
bool make_value_dict(int es, const void *val, int nnz, std::vector<unsigned char> &codes, std::vector<unsigned char> &dict,
                     int *nDict, int most = 256);

// The layout csr_slice_kernel runs on (see DeviceSlices), in host memory.
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
// Re-lays the rows `sel` marks (all rows when null) of a CSR matrix for csr_slice_kernel; `elsewhere` marks
// rows that the tile forms write (1: alone, 2: together with the CSR part); `fused`: the one-launch form is
// wanted -- 1: wherever the matrix suits it, 2: only where no workgroup has more than kFusedAddBytes of
// sums under it (D.fused says whether the matrix got it).  upload_slices does the same and puts the layout on the
// device -- built there when nothing asks for the host (a whole matrix, not fused, MX_LAYOUT unset).
int build_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                 const char *sel, HostSlices &D, const char *elsewhere = nullptr, int fused = 0);
int upload_slices(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int nCU, int S,
                  const char *sel, mx::DeviceSlices &D, const char *elsewhere = nullptr,
                  std::pair<std::vector<int>, std::vector<int>> *segOut = nullptr, int fused = 0);

// One block of the tile kernels: fragM x fragK values, row-major, zeros included, and the column
// of each of its fragK positions (-1 = unused).
struct TileBlock {
    std::vector<unsigned char> vals;
    int cols[8];
};
// A chunk the plan forms itself (binary16 strips, binary64 8 x 8 blocks): up to fragM rows (caller's
// numbering, -1 = none) with one and the same set of blocks of eight consecutive columns, and those blocks.
struct StripChunk {
    int rows[8];
    std::vector<TileBlock> blocks;
    int nnz;
};

// The layout the tile kernels run on (see DeviceTiles), in host memory.
struct HostTiles {
    int chunkNum = 0, frags = 0, vals = 0, steps = 0, nWaves = 0;
    long long stored = 0;
    bool dense = false;
    std::vector<int> waveDesc, hdr, atox, valOffset;  // valOffset: first value of every step (the kernels get it from the headers)
    std::vector<unsigned char> val;
};
// The fragments named by `selFrag` (all when null), expanded to full blocks and grouped into steps.  Column ids
// go through `colMap` and output rows through `rowMap` when given.  `rowTaken` (optional, per row of A_dd) marks
// rows whose entries the plan has put into chunks of its own: they are left out of the fragments here.  With
// `stripChunks` the canonical chunks are not used at all: the given chunks are laid out.  `nCU` only sizes the
// waves.  upload_tiles does the same and puts the layout on the device.
int build_tiles(mx_dtype dtype, int chunkNum, const char *selFrag, int dRows, const int *chunkPtr, const int *fragPtr,
                const void *fragBit, const void *tcVal, const int *atox, const int *colMap, const int *rowMap, int nCU,
                HostTiles &T, const char *rowTaken = nullptr, const std::vector<StripChunk> *stripChunks = nullptr);
int upload_tiles(mx_dtype dtype, int chunkNum, const char *selFrag, int dRows, const int *chunkPtr, const int *fragPtr,
                 const void *fragBit, const void *tcVal, const int *atox, const int *colMap, const int *rowMap,
                 mx::DeviceTiles &T, int *tile_nnz, const char *rowTaken = nullptr,
                 const std::vector<StripChunk> *stripChunks = nullptr, std::vector<int> *hdrOut = nullptr);
int upload_csr(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr, const int *col, const void *val,
               mx::DeviceCsr &A, double *pack_ms);
void tile_waves(int steps, int nCU, int perMin, const std::vector<int> &stepVo, const std::vector<int> &stepA,
                const std::vector<int> &stepChunkEnd, std::vector<int> &waveDesc, std::vector<int> &ahead);

// The MX_OPT_* bits of the environment as it was last read (mx::refresh_options).
inline int plan_opt_flags()
{
    const mx::Options &o = mx::opt();
    return (o.no_strips ? MX_OPT_NO_STRIPS : 0) | (o.no_blocks ? MX_OPT_NO_BLOCKS : 0) | (o.csr_dict == 0 ? MX_OPT_NO_DICT : 0) |
           (o.strips_apart ? MX_OPT_STRIPS_APART : 0) | (o.csr_kernel ? MX_OPT_CSR_KERNEL : 0) | (o.csr_fused >= 0 ? MX_OPT_CSR_FUSED : 0) | (o.csr_keep >= 0 ? MX_OPT_CSR_KEEP : 0) |
           (o.autotune ? MX_OPT_AUTOTUNE : 0) | (o.layout_host ? MX_OPT_LAYOUT_HOST : 0) |
           (o.slice_cap || o.split_len || o.csr_npt || o.tile_per || o.csr_reduce || !o.csr_col16 ? MX_OPT_TUNING : 0);
}

}  // namespace mxp

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
    // the switches of the environment that shaped the plan, as they read when it was made (MX_OPT_* bits and
    // the fill a fragment needed); the product looks at these, never at the environment
    int opt_flags = mxp::plan_opt_flags();
    double opt_tile_gate = mx::opt().tile_gate >= 0.0 ? mx::opt().tile_gate : 0.5;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
};

namespace mxp {

// Mean milliseconds per iteration of `body` over `iters` back-to-back runs after `warm`
// untimed ones, by events on the stream the kernels run on.
template <typename F>
int time_loop(mx_plan *plan, int warm, int iters, F body, double *ms)
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

// ---- mx_plan.cpp: what a plan is decided from -----------------------------------------------------------
// What the choice between the forms of the CSR part looks at: all of it is counted from the
// matrix, none of it is timed, so the same matrix gets the same plan on every run.
struct CsrStats {
    double linesPerGather = 0;  // mean number of distinct 64-byte lines of x that 64 consecutive entries name
    double vrows = 0;           // virtual rows the slice layout would have (distinct slices per row, long ones cut)
    bool fewValues = false;     // at most 255 distinct values: the one-byte-per-value forms exist
    int mostVrows = 0;          // most virtual rows of any row
};
// Which forms of the CSR part a plan may take (want[0] row tiles, [1] slices, [2] split) after the
// caller's flags, MX_CSR_KERNEL and -- when both of the first two are still open and nothing is to be
// timed -- the estimates.  S = slice_count() of the matrix.
struct CsrChoice {
    bool want[3] = {true, true, false};
    double usRows = 0, usSlices = 0;  // the estimates, when they decided
    bool fewValues = false;
    int mostVrows = -1;  // most virtual rows of a row (-1: not counted)
};
// MX_PLAN_LOG=1: the phases of mx_plan_create with their host time, on stderr
struct PhaseLog {
    bool on = mx::opt().plan_log;
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

// What the one-launch form saves of the slice form's estimate where it is taken (microseconds, measured): the
// second launch and its wait, less the adding at the end of the first.
constexpr double kFusedSavesUs = 1.8;
// Bytes of the sums of a plan's virtual rows (what upload_slices allocates for them).
size_t partial_bytes(const mx_plan *plan);
bool plan_autotune();
double tile_gate(mx_dtype dtype);
void csr_estimates(mx_dtype dtype, int cols, int nnz, const CsrStats &st, double *usRows, double *usSlices);
// 0: not wanted; 1: asked for (flag or environment); 2: by the default rule (the `fused` of build_slices)
int fused_wanted(int flags, mx_dtype dtype, int rows, int S, int mostVrows, int nCU);
// Sets plan->slices.keep for a plan whose CSR part is in slice form: how the slice kernel reads its entries.
void decide_keep(mx_plan *plan, int flags);
double touched_bytes(const mx_plan *plan);
CsrChoice choose_csr_form(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int flags, int nCU,
                          int S, bool mayFuse = false);
int setup_csr_part(mx_plan *plan, const int *rowPtr, const int *col, const void *val, int flags, const char *stripRows = nullptr,
                   std::pair<std::vector<int>, std::vector<int>> *segOut = nullptr);
int tiles_worth(mx_dtype dtype, int fragM, int fragK, bool blocks64, double generalEntries, double generalFrags, double stripEntries,
                double stripBlocks, double stripBlocksOff, double allEntries, double *netNs = nullptr);
int plan_host_parts(const mx_partition *P, int flags, HostPlanParts &H, PhaseLog &phase, bool noBlocks = false);

// ---- mx_plan_device.cpp -------------------------------------------------------------------------------
// `noBlocks`: a binary64 plan without the 8 x 8 block form.  `twin`: the extraction is there already, in the
// device arrays of a partition that was made on the device (the matrix arguments are not looked at then).
int create_plan_device(mx_dtype dtype, int rows, int cols, int nnz, const int *rowPtr_dev, const int *colInd_dev, const void *val_dev,
                       float tau_c, float tau_r, int flags, mx_plan **out, bool noBlocks, const mx::PartitionTwin *twin = nullptr);

// ---- mx_run.cpp ---------------------------------------------------------------------------------------
// Set once a one-launch product has reported a misplaced workgroup: no plan takes the form from then on.
extern std::atomic<bool> g_fused_off;
// The CSR part of one product on stream `s`.  `strips`: tiles that ride in the combine kernel's launch;
// `partial`: where the slice kernel puts the sums of the virtual rows, in place of the plan's own buffer.
int launch_csr_part(mx_plan *plan, const void *x, void *y, int accumulate, hipStream_t s, const mx::DeviceTiles *strips = nullptr,
                    void *partial = nullptr, void *ywide = nullptr);

}  // namespace mxp
