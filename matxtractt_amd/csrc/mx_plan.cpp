// A plan from a partition in host memory: what the tile kernels keep, which form the CSR part takes
// (counted from the matrix, never timed unless asked), and the upload of both.
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

// Bytes of the sums of a plan's virtual rows (what upload_slices allocates for them).
size_t mxp::partial_bytes(const mx_plan *plan)
{
    if (plan->csr_variant == 0) return 0;
    return ((size_t)plan->slices.chunks * 64 + 64) * (plan->dtype == MX_F64 ? 8 : 4);
}

// Row length from which a row of a split plan goes to the slice kernel (MX_SPLIT_LEN overrides).
static int split_length()
{
    const int v = mx::opt().split_len;
    return v > 0 ? v : 32;
}


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
    if (nnz >= 65536 && mx::opt().csr_dict != 0) {
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
void mxp::csr_estimates(mx_dtype dtype, int cols, int nnz, const CsrStats &st, double *usRows, double *usSlices)
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

bool mxp::plan_autotune()
{
    return mx::opt().autotune;
}
// Whether a plan asks for the one-launch form of the slices.  Never with MX_PLAN_NO_FUSE or
// MX_CSR_FUSED=0, after a misplaced workgroup was reported, or for a matrix with a row of more than
// eight virtual rows (mostVrows < 0: not counted, the layout will see).  MX_PLAN_FUSE (or
// MX_CSR_FUSED=1) takes it wherever the matrix suits it (return value 1).  Otherwise where it pays
// (return value 2): the workgroup that comes last to a group of rows adds that group up alone --
// a round of atomics, then one of loads, 2 KB (1 KB in binary16) per place of the group's rows at
// about 30 bytes a cycle, about 70 ns with the additions and the stores -- and the slowest
// workgroup comes last to all of its groups.  Against that stands the second launch with its wait,
// about 5 us.  Measured, one launch against two (us): block-clustered workload, 45 places under the
// busiest workgroup, 12.5 / 13.1 (7.8 / 9.3 at half size); 400 000 rows of 8 entries in two
// slices, 30 places, 13.9 / 15.6; 200 000 rows of 16 in four slices, 72 places, 15.7 / 14.6;
// 130 000 rows of 32 in eight slices, 144 places, 20.9 / 17.3.  So the form is taken while the
// busiest workgroup has at most kFusedAddBytes of sums under it, which only the layout knows
// (build_slices); here the average stands in for it, so that no layout is made in vain for a
// matrix that is far off.  And while the slices are few: the workgroups of a slice are spread over
// all XCDs in this form, so each XCD fetches every slice of x (16 384 rows in 32 slices, 32 places:
// 10.6 / 8.1).
int mxp::fused_wanted(int flags, mx_dtype dtype, int rows, int S, int mostVrows, int nCU)
{
    const int env = mx::opt().csr_fused;
    if ((flags & MX_PLAN_NO_FUSE) || env == 0 || g_fused_off.load()) return 0;
    if (mostVrows > mx::kSliceLightSegs || nCU % mx::kFusedXcds) return 0;
    if ((flags & MX_PLAN_FUSE) || env == 1) return 1;
    const double average = (double)rows * std::max(S, 1) * std::max(mostVrows, 1) * (dtype == MX_F64 ? 8 : 4) / std::max(nCU, 1);
    return average <= (double)mx::kFusedAddBytes && S <= mx::kFusedSlicesMost ? 2 : 0;
}

// Bytes of the entries of a plan's slice layout as they are stored (column offsets and values or value codes, with
// the padding), and what its second launch moves per product: the sums it is handed, the row tables, y.
static long long slice_entry_bytes(const mx_plan *plan)
{
    const mx::DeviceSlices &L = plan->slices;
    const long long es = mx::elem_size(plan->dtype), E = mx::slice_step_entries(plan->dtype);
    return (L.steps + mx::kSlicePadSteps) * 64 * E * (2 + (L.useDict ? 1 : es));
}
static long long slice_handoff_bytes(const mx_plan *plan)
{
    const mx::DeviceSlices &L = plan->slices;
    const long long es = mx::elem_size(plan->dtype);
    return (long long)mxp::partial_bytes(plan) + (long long)plan->rows * (4 + es) + (long long)L.nLight * (4 + 16 * L.lightQuads) + (long long)L.vrows * 4;
}
// What one product touches in device memory, as the plan stores it (mx_plan_info.touched_bytes): the CSR part in
// its form, the tile part, x and y.  (The algorithmic bytes of the matrix, which the roofline is priced on, count a
// value and a 4-byte column per entry whatever the plan stores.)
double mxp::touched_bytes(const mx_plan *plan)
{
    const double es = mx::elem_size(plan->dtype);
    double b = (double)plan->cols * es + (double)plan->rows * es;
    if (plan->csr_variant != 1) b += (double)plan->csr.nnz * ((plan->csr.useDict ? 1.0 : es) + 4.0) + ((double)plan->rows + 1) * 4;
    if (plan->csr_variant != 0) b += (double)slice_entry_bytes(plan) + (double)slice_handoff_bytes(plan) - (double)plan->rows * es;
    if (plan->tiles.steps)
        b += (double)plan->tiles.steps * (mx::kTileHdr * 4.0 + 64 * 4.0) + (double)plan->tiles.stored * es;
    if (plan->strips.steps) b += (double)plan->strips.steps * (mx::kTileHdr * 4.0) + (double)plan->strips.stored * es;
    return b;
}

// How the slice kernel of a plan reads its entries (DeviceSlices::keep).  Streaming loads are the faster way to
// read a matrix once: they leave the caches to x and the sums, and what they bring is the first to leave the
// memory-side cache when other traffic asks for room.  That is also their price: the second launch of a product
// asks for room every time (the sums it is handed, its row tables, y), so a streamed matrix that would fit the
// cache comes from HBM again in every product -- workload 4, 76 MB: 20.2 us streamed, the same in a rotation of
// copies as back to back, 18.2 us with plain loads (and 0.42 instead of 0.47 of the roofline in the rotation,
// 0.28 instead of 0.35 on cold caches: what plain loads cost when nothing can stay).  Plain loads where staying
// pays: the entries fit the L2s (workload 2 at half size, 22 MB: 7.2 against 8.6 us), or they fit the memory-side
// cache and the second launch moves enough to push them out (workload 3: 28.6 against 31.5 us; workload 2 at
// full size in two launches, 44 MB of entries and 7 MB for the second launch, is the case it does not pay: 14.4 against 13.2 -- workload 4 hands 21 MB over).
// The one-launch form has no second launch: only the first rule applies to it.
void mxp::decide_keep(mx_plan *plan, int flags)
{
    mx::DeviceSlices &L = plan->slices;
    L.keep = false;
    if (plan->csr_variant == 0) return;
    const int env = mx::opt().csr_keep;
    if ((flags & MX_PLAN_STREAM) || env == 0) return;
    if ((flags & MX_PLAN_KEEP) || env == 1) {
        L.keep = true;
        return;
    }
    const long long entryBytes = slice_entry_bytes(plan), handoff = slice_handoff_bytes(plan);
    // (everything a product touches has to fit beside the entries: the tile part rides in the second launch)
    const long long product = (long long)touched_bytes(plan);
    if (entryBytes <= mx::kKeepL2Bytes) L.keep = true;
    else if (!plan->fused && product <= mx::kKeepCacheBytes && handoff >= mx::kKeepHandoffBytes) L.keep = true;
}

CsrChoice mxp::choose_csr_form(mx_dtype dtype, int rows, int cols, const int *rowPtr, const int *col, const void *val, int flags,
                                int nCU, int S, bool mayFuse)
{
    CsrChoice c;
    const int env = mx::opt().csr_kernel;
    if (flags & MX_PLAN_CSR_ROWS) c.want[1] = c.want[2] = false;
    if (flags & MX_PLAN_CSR_SLICES) c.want[0] = c.want[2] = false;
    if (env == 1) c.want[0] = true, c.want[1] = c.want[2] = false;
    if (env == 2) c.want[1] = true, c.want[0] = c.want[2] = false;
    if (env == 3) c.want[2] = true, c.want[0] = c.want[1] = false;
    if (S == 0) c.want[1] = c.want[2] = false;
    if (c.want[0] && c.want[1] && !plan_autotune()) {
        const CsrStats st = csr_stats(dtype, rows, rowPtr, col, val, nCU);
        csr_estimates(dtype, cols, rowPtr[rows], st, &c.usRows, &c.usSlices);
        c.fewValues = st.fewValues;
        c.mostVrows = st.mostVrows;
        // (the one-launch form of the slices, where the plan would take it: the device's placement is looked at
        // later, and a plan whose strips ride in the second launch keeps both launches)
        if (mayFuse && fused_wanted(flags, dtype, rows, S, st.mostVrows, nCU)) c.usSlices -= kFusedSavesUs;
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
int mxp::setup_csr_part(mx_plan *plan, const int *rowPtr, const int *col, const void *val, int flags, const char *stripRows,
                        std::pair<std::vector<int>, std::vector<int>> *segOut)
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
    int wantFused = want[1] && !stripRows ? fused_wanted(flags, plan->dtype, rows, S, pick.mostVrows, nCU) : 0;
    if (wantFused) {
        int ok = 0;
        MX_HIP(mx::fused_placement_ok(nCU, &ok));
        if (!ok) wantFused = 0;
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
                if (!rc && (msDict < ms || mx::opt().csr_dict == 2)) ms = msDict;
                else plan->slices.useDict = false;
            }
            if (!rc && v == 0 && plan->csr.codes) {  // the same rows with one byte per value (MX_CSR_DICT=2: whatever the timing)
                double msDict = 0.0;
                plan->csr.useDict = true;
                rc = time_loop(plan, 3, 10, [&]() { return launch_csr_part(plan, tx, ty, 0, plan->stream); }, &msDict);
                if (!rc && (msDict < ms || mx::opt().csr_dict == 2)) ms = msDict;
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
    if (!rc) decide_keep(plan, flags);
    return rc;
}

// Minimum fill of a fragment for the MFMA tile kernel to take it (default plans;
// MX_TILE_GATE=<fraction> overrides).  A fragment costs its bitmap, its value offset and fragK
// column ids whatever it holds, and the decode work of a whole tile; below about half full the
// same entries are cheaper in the CSR part.
double mxp::tile_gate(mx_dtype)
{
    if (mx::opt().tile_gate >= 0.0) return mx::opt().tile_gate;
    return 0.5;
}

// Do the tiles pay for their launch?  (The reference gates its tile kernel on the size of the
// matrix and its fill, test/test_autotc_spmv.cpp:1507,1518.)  What they take off the CSR part
// saves es + 2 bytes per entry of its stream; what they cost is one more dependent launch and
// their own stream.  Rates as measured on MI355X: the CSR part and the binary16 strips move about
// 5000 bytes per ns (5 TB/s), the general tile kernel, bound by instruction issue, about 2200; a
// further launch in the sequence costs about 5 us with its ramp and tail.  The strips ride in the
// launch of the combine kernel and are charged 3 us for it: over the family of the mixed workload
// (5 to 40 % of the rows in strips, a quarter of the size and the full size, on and off the grid of
// eight columns) that is where they stop paying -- 3.3 and 6.5 M entries at a quarter of the size lose
// 0.3 to 1.3 us, 13 M there and everything from 7 M at full size wins.  At a quarter of the size the
// matrix stays in the memory-side cache and everything streams at 7 instead of 5 bytes per ns, which is
// what decides the 13 M entries off the grid there together with the price of their alignment (a block that
// starts off the grid of eight columns is charged a quarter more: they win by 0.5 us on the grid and lose
// about 1 us off it).  The binary64 8 x 8 blocks
// ride the same way but stream at the general kernel's rate: with 10, 25, 40 and 70 % of the
// block-clustered workload's entries in blocks they never came out ahead of the CSR part (a tie at
// 40 %, 17.6 against 12.7 us at 70 %), which is what this price says.
// general*: the reference's fragments that pass the fill gate; strip*: the chunks of the plan's
// own (binary16 strips, or binary64 8 x 8 blocks with `blocks64`).
// 0 = nothing pays, 1 = only the plan's own chunks do, 2 = keep both.
// `netNs` (optional): what the forms that are kept save per product by this estimate, in ns.
int mxp::tiles_worth(mx_dtype dtype, int fragM, int fragK, bool blocks64, double generalEntries, double generalFrags,
                     double stripEntries, double stripBlocks, double stripBlocksOff, double allEntries, double *netNs)
{
    const int es = mx::elem_size(dtype);
    const double blockBytes = (double)fragM * (blocks64 ? 8 : fragK) * es, slots = mx::tile_slots(dtype);
    const double generalBytes = generalFrags * blockBytes + generalFrags / slots * (mx::kTileHdr * 4.0 + 256.0);
    // (a block that starts off the grid of eight columns reads x across 16-byte boundaries: measured, a quarter more)
    const double stripBytes = (stripBlocks + 0.25 * stripBlocksOff) * blockBytes + stripBlocks / slots * (mx::kTileHdr * 4.0);
    // (a matrix whose entries stay in the memory-side cache between products streams faster, tiles or not:
    // what the strips take off the CSR part is then worth less time, and so is what they stream themselves)
    const bool resident = allEntries * (es + 2) <= 128e6;
    const double launchNs = 5000.0, stripLaunchNs = 3000.0, fastRate = resident ? 7000.0 : 5000.0, generalRate = 2200.0;  // bytes per ns
    const double savedNs = (generalEntries + stripEntries) * (es + 2) / fastRate;
    const double generalCost = generalFrags > 0 ? launchNs + generalBytes / generalRate : 0.0;
    const double stripCost = stripBlocks > 0 ? stripLaunchNs + stripBytes / (blocks64 ? generalRate : fastRate) : 0.0;
    if (netNs) *netNs = 0.0;
    if (savedNs <= generalCost + stripCost) return 0;
    if (generalFrags > 0 && generalEntries * (es + 2) / fastRate <= generalCost) {
        if (netNs) *netNs = stripEntries * (es + 2) / fastRate - stripCost;
        return 1;
    }
    if (netNs) *netNs = savedNs - generalCost - stripCost;
    return 2;
}



int mxp::plan_host_parts(const mx_partition *P, int flags, HostPlanParts &H, PhaseLog &phase, bool noBlocks)
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
        !mx::opt().no_strips) {
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
    if (P->dtype == MX_F64 && !noBlocks && !(flags & (MX_PLAN_NO_TILES | MX_PLAN_ALL_TILES)) && !mx::opt().no_blocks && P->dRows > 0) {
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
        double generalEntries = 0, generalFrags = 0, stripEntries = 0, stripBlocks = 0, stripBlocksOff = 0;
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
            if (!C.blocks.empty() && (C.blocks[0].cols[0] & 7)) stripBlocksOff += (double)C.blocks.size();
        }
        const int worth = tiles_worth(P->dtype, fragM, fragK, !inBlock.empty(), generalEntries, generalFrags, stripEntries, stripBlocks,
                                      stripBlocksOff, (double)P->nnz);
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
extern "C" int mx_plan_create(const mx_partition *P, int flags, mx_plan **out)
{
    mx::refresh_options();
    // A partition that was made on the device still has its arrays there: the plan is made from them where they
    // are -- the same plan, array for array, as from the host arrays (MX_LAYOUT=host, MX_CSR_KERNEL=split and
    // MX_PLAN_AUTOTUNE=1 keep the host route, which brings the arrays down first).
    if (P && out && P->twin && P->extracted) {
        if (!mx::opt().layout_host && mx::opt().csr_kernel != 3 && !plan_autotune())
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
    decide_keep(plan, flags);  // (again, now that the tile part is known: it counts towards what a product touches)
    *out = plan;
    return MX_OK;
}

