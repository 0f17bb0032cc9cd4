// The product of a plan (the launch sequence of one y = A x) and its timing.
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

// The word in host memory that the one-launch kernels write when a workgroup is misplaced: one per
// process, pinned and mapped, allocated at the first use (null when that fails).
std::atomic<bool> mxp::g_fused_off{false};
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
int mxp::launch_csr_part(mx_plan *plan, const void *x, void *y, int accumulate, hipStream_t s, const mx::DeviceTiles *strips, void *partial,
                         void *ywide)
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
    const bool apart = (plan->opt_flags & MX_OPT_STRIPS_APART) != 0;
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
    const bool apart = (plan->opt_flags & MX_OPT_STRIPS_APART) != 0;
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
    const bool apart = (plan->opt_flags & MX_OPT_STRIPS_APART) != 0;
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
        add(std::string("csr_slice_kernel<") + vt + (plan->slices.useDict ? ",dict" : "") + ",fused" + (plan->slices.keep ? ",keep>" : ">"),
            (double)plan->slices.nnz * (es + 4) + xBytes + yBytes, plan->slices.nnz,
            [&]() -> int { return launch_csr_part(plan, x_dev, y_dev, 0, s, nullptr, nullptr, wide); });
    } else if (plan->csr_variant != 0) {
        add(std::string("csr_slice_kernel<") + vt + (plan->slices.useDict ? ",dict" : "") + (plan->slices.keep ? ",keep>" : ">"),
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

