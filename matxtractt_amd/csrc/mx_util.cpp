// Error text and binary16 conversions shared by the host code.
#include <cstring>

#include "mx_internal.h"

namespace mx {

static thread_local std::string g_error;

void set_error(const std::string &msg) { g_error = msg; }

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
