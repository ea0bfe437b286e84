// TEST INFRASTRUCTURE ONLY -- part of the CPU oracle; never linked into the product library.
//
// Software IEEE-754 binary16 <-> binary32 conversions (round-to-nearest-even, subnormals kept).
// g++ 11 has no _Float16 on x86, so the oracle carries its own bit-exact conversions; they are
// pinned against numpy's float16 in tests/test_oracle_fp16.py (all 65536 half patterns, and
// float->half on ties, subnormals, overflow and random bit patterns).
#ifndef PPLHIP_ORACLE_FP16_SOFT_H_
#define PPLHIP_ORACLE_FP16_SOFT_H_

#include <stdint.h>
#include <string.h>

namespace oracle {

static inline float bits_to_float(uint32_t u) {
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint32_t float_to_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

// binary16 bits -> binary32 value (exact).
static inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    if (exp == 0) {
        if (man == 0) return bits_to_float(sign);
        // subnormal: value = man * 2^-24; normalise
        int e = -1;
        do {
            ++e;
            man <<= 1;
        } while ((man & 0x400u) == 0);
        man &= 0x3ffu;
        return bits_to_float(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
    }
    if (exp == 31) return bits_to_float(sign | 0x7f800000u | (man << 13));
    return bits_to_float(sign | ((exp + 112u) << 23) | (man << 13));
}

// binary32 value -> binary16 bits, round-to-nearest-even; overflow -> inf; NaN -> quiet NaN.
static inline uint16_t float_to_half(float f) {
    const uint32_t x = float_to_bits(f);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) { // inf / nan
        if (absx == 0x7f800000u) return sign | 0x7c00u;
        return sign | 0x7e00u | (uint16_t)((absx >> 13) & 0x3ffu);
    }
    if (absx >= 0x477ff000u) { // >= 65520 rounds to inf
        return sign | 0x7c00u;
    }
    if (absx < 0x38800000u) { // < 2^-14: subnormal or zero in half
        if (absx < 0x33000000u) { // < 2^-25: rounds to zero (2^-25 itself ties to even = 0)
            return sign;
        }
        const int e = (int)(absx >> 23); // biased fp32 exponent, 102..112
        const uint32_t man = (absx & 0x7fffffu) | 0x800000u; // 24-bit significand
        const int shift = 126 - e; // result = man >> shift, in units of 2^-24; shift in 14..24
        const uint32_t q = man >> shift;
        const uint32_t rem = man & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1);
        uint32_t r = q;
        if (rem > halfway || (rem == halfway && (q & 1u))) ++r;
        return sign | (uint16_t)r; // may carry into the smallest normal, which is the right bit pattern
    }
    // normal range
    uint32_t r = absx - 0x38000000u; // rebias exponent (127 -> 15)
    const uint32_t rem = r & 0x1fffu;
    r >>= 13;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) ++r; // carry may bump the exponent; still correct
    return sign | (uint16_t)r;
}

} // namespace oracle

#endif
