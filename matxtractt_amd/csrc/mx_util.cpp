// Error text and binary16 conversions shared by the host code.
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "mx_internal.h"

namespace mx {

static thread_local std::string g_error;

void set_error(const std::string &msg) { g_error = msg; }

// One set for the process (the planners read it from OpenMP workers too).  It is rewritten only when the
// environment reads differently from the last time, so threads that make plans side by side under one
// environment never write it.
static Options g_options;
static std::mutex g_options_mu;
const Options &opt() { return g_options; }
static bool same(const Options &a, const Options &b)
{
    return a.tile_gate == b.tile_gate && a.csr_dict == b.csr_dict && a.no_strips == b.no_strips && a.no_blocks == b.no_blocks &&
           a.strips_apart == b.strips_apart && a.csr_kernel == b.csr_kernel && a.csr_fused == b.csr_fused && a.csr_keep == b.csr_keep && a.autotune == b.autotune &&
           a.layout_host == b.layout_host && a.slice_cap == b.slice_cap && a.split_len == b.split_len && a.csr_npt == b.csr_npt &&
           a.tile_per == b.tile_per && a.csr_reduce == b.csr_reduce && a.csr_col16 == b.csr_col16 && a.plan_log == b.plan_log;
}
void refresh_options()
{
    Options o;
    auto text = [](const char *name) { return std::getenv(name); };
    auto number = [&](const char *name, int unset) {
        const char *e = text(name);
        return e ? std::atoi(e) : unset;
    };
    if (const char *e = text("MX_TILE_GATE")) {
        const double v = std::atof(e);
        if (v >= 0.0 && v <= 1.0) o.tile_gate = v;
    }
    o.csr_dict = number("MX_CSR_DICT", 1);
    o.no_strips = number("MX_NO_STRIPS", 0) != 0;
    o.no_blocks = number("MX_NO_BLOCKS", 0) != 0;
    o.strips_apart = number("MX_STRIPS_APART", 0) != 0;
    if (const char *e = text("MX_CSR_KERNEL")) o.csr_kernel = !std::strcmp(e, "rows") ? 1 : !std::strcmp(e, "slices") ? 2 : !std::strcmp(e, "split") ? 3 : 0;
    if (const char *e = text("MX_CSR_FUSED")) o.csr_fused = std::atoi(e) ? 1 : 0;
    if (const char *e = text("MX_CSR_KEEP")) o.csr_keep = std::atoi(e) ? 1 : 0;
    o.autotune = number("MX_PLAN_AUTOTUNE", 0) != 0;
    if (const char *e = text("MX_LAYOUT")) o.layout_host = !std::strcmp(e, "host");
    o.slice_cap = number("MX_SLICE_CAP", 0);
    o.split_len = number("MX_SPLIT_LEN", 0);
    o.csr_npt = number("MX_CSR_NPT", 0);
    o.tile_per = number("MX_TILE_PER", 0);
    if (const char *e = text("MX_CSR_REDUCE")) o.csr_reduce = !std::strcmp(e, "rows") ? 1 : !std::strcmp(e, "scan") ? 2 : 0;
    o.csr_col16 = number("MX_CSR_COL16", 1) != 0;
    o.plan_log = number("MX_PLAN_LOG", 0) != 0;
    std::lock_guard<std::mutex> lock(g_options_mu);
    if (!same(g_options, o)) g_options = o;
}

uint16_t f64_to_f16_bits(double v)
{
    uint64_t b;
    std::memcpy(&b, &v, 8);
    const uint16_t sign = (uint16_t)((b >> 48) & 0x8000u);
    const uint64_t ab = b & 0x7fffffffffffffffull;
    if (ab >= 0x7ff0000000000000ull) return (uint16_t)(sign | (ab == 0x7ff0000000000000ull ? 0x7c00u : 0x7e00u));
    const int e = (int)(ab >> 52) - 1023;
    uint64_t m = ab & 0xfffffffffffffull;
    if (e > 15) return (uint16_t)(sign | 0x7c00u);
    if (e >= -14) {
        uint32_t h = ((uint32_t)(e + 15) << 10) | (uint32_t)(m >> 42);
        const uint64_t rem = m & ((1ull << 42) - 1), half = 1ull << 41;
        if (rem > half || (rem == half && (h & 1u))) ++h;  // a carry into the exponent is the right answer
        return (uint16_t)(sign | h);
    }
    if (e < -25) return sign;
    m |= 1ull << 52;
    const int shift = 42 + (-14 - e);  // 43..53
    uint32_t hm = (uint32_t)(m >> shift);
    const uint64_t rem = m & ((1ull << shift) - 1), half = 1ull << (shift - 1);
    if (rem > half || (rem == half && (hm & 1u))) ++hm;
    return (uint16_t)(sign | hm);
}

float f16_bits_to_f32(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t ex = (h >> 10) & 0x1fu;
    const uint32_t man = h & 0x3ffu;
    float out;
    if (ex == 0) {
        // subnormal or zero: man * 2^-24, exact in binary32
        out = (float)man * (1.0f / 16777216.0f);
        uint32_t bits;
        std::memcpy(&bits, &out, 4);
        bits |= sign;
        std::memcpy(&out, &bits, 4);
        return out;
    }
    uint32_t bits = ex == 31 ? (sign | 0x7f800000u | (man << 13)) : (sign | ((ex + 112u) << 23) | (man << 13));
    std::memcpy(&out, &bits, 4);
    return out;
}

}  // namespace mx

extern "C" const char *mx_last_error(void) { return mx::g_error.c_str(); }

extern "C" uint16_t mx_f32_to_f16(float f) { return mx::f64_to_f16_bits((double)f); }
extern "C" float mx_f16_to_f32(uint16_t h) { return mx::f16_bits_to_f32(h); }
