// hip/hip_fp16.h of the tests' SIMT simulator: IEEE binary16 storage with round-to-nearest-even conversions.
#pragma once

#include <cstdint>
#include <cstring>

struct __half {
    uint16_t bits;
};
struct __half2 {
    __half x, y;
};

inline float __half2float(__half h) {
    const uint32_t sign = (uint32_t)(h.bits & 0x8000u) << 16;
    uint32_t exponent = (h.bits >> 10) & 0x1Fu, mantissa = h.bits & 0x3FFu, out;
    if (exponent == 0) {
        if (mantissa == 0) {
            out = sign;
        } else {   // subnormal: normalise
            int shift = 0;
            while (!(mantissa & 0x400u)) {
                mantissa <<= 1;
                ++shift;
            }
            out = sign | ((uint32_t)(113 - shift) << 23) | ((mantissa & 0x3FFu) << 13);
        }
    } else if (exponent == 31) {
        out = sign | 0x7F800000u | (mantissa << 13);
    } else {
        out = sign | ((exponent + 112) << 23) | (mantissa << 13);
    }
    float f;
    std::memcpy(&f, &out, 4);
    return f;
}

inline __half __float2half_rn(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    const uint32_t magnitude = x & 0x7FFFFFFFu;
    __half h;
    if (magnitude >= 0x7F800000u) {   // infinity or NaN
        h.bits = (uint16_t)(sign | 0x7C00u | (magnitude > 0x7F800000u ? 0x200u | ((magnitude >> 13) & 0x3FFu) : 0u));
        return h;
    }
    if (magnitude >= 0x477FF000u) {   // rounds to infinity
        h.bits = (uint16_t)(sign | 0x7C00u);
        return h;
    }
    if (magnitude < 0x33000001u) {    // rounds to zero
        h.bits = sign;
        return h;
    }
    const int exponent = (int)(magnitude >> 23) - 127;
    uint32_t mantissa = (magnitude & 0x7FFFFFu) | 0x800000u;
    int shift;
    uint32_t base;
    if (exponent < -14) {   // subnormal result
        shift = 13 + (-14 - exponent);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(exponent + 15) << 10;
        mantissa &= 0x7FFFFFu;
    }
    uint32_t kept = mantissa >> shift;
    const uint32_t rest = mantissa & ((1u << shift) - 1u), half = 1u << (shift - 1);
    if (rest > half || (rest == half && (kept & 1u))) ++kept;
    h.bits = (uint16_t)(sign | (base + kept));   // a carry out of the mantissa moves into the exponent, as it should
    return h;
}

inline __half2 __halves2half2(__half a, __half b) { return __half2{a, b}; }
inline float __low2float(__half2 h) { return __half2float(h.x); }
inline float __high2float(__half2 h) { return __half2float(h.y); }
