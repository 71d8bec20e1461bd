// IEEE binary16 host type of the veneer (mirrors gpgpu/include/gblas_half.h:24-46: a 2-byte
// struct with the bits in `x`, built from and converted to float).  Conversions are computed
// arithmetically with round-to-nearest-even, the rounding the device applies when it narrows a
// float result to half.
#ifndef DLFX_VENEER_GBLAS_HALF_H_
#define DLFX_VENEER_GBLAS_HALF_H_

#include <cstdint>
#include <cstring>
#include <ostream>

namespace gpgpu { namespace blas {

struct alignas(2) half {
    unsigned short x;

    half() : x(0) {}
    half(const float f) : x(from_float(f)) {}
    half& operator=(const float f) { x = from_float(f); return *this; }
    operator float() const { return to_float(x); }

    static unsigned short from_float(float value) {
        uint32_t u;
        std::memcpy(&u, &value, 4);
        const uint32_t sign = (u >> 16) & 0x8000u;
        const uint32_t mag = u & 0x7fffffffu;
        if (mag >= 0x7f800000u)                                  // infinity, NaN (kept quiet, payload dropped)
            return static_cast<unsigned short>(sign | 0x7c00u | (mag > 0x7f800000u ? 0x200u : 0u));
        if (mag >= 0x477ff000u) return static_cast<unsigned short>(sign | 0x7c00u);   // rounds past 65504
        if (mag < 0x33000001u) return static_cast<unsigned short>(sign);              // at most half the smallest subnormal
        const int exp = static_cast<int>(mag >> 23) - 127;
        uint32_t frac = (mag & 0x7fffffu) | 0x800000u;           // 24-bit significand
        int shift = 13;                                          // normal halves keep 11 of the 24 bits
        uint32_t biased = static_cast<uint32_t>(exp + 15);
        if (exp < -14) {                                         // subnormal half
            shift = 13 + (-14 - exp);
            biased = 0;
        }
        const uint32_t kept = frac >> shift;
        const uint32_t rest = frac & ((1u << shift) - 1u);
        const uint32_t halfway = 1u << (shift - 1);
        uint32_t out = (biased ? ((biased - 1) << 10) : 0u) + kept;      // the hidden bit carries into the exponent
        if (rest > halfway || (rest == halfway && (kept & 1u))) ++out;
        return static_cast<unsigned short>(sign | out);
    }

    static float to_float(unsigned short bits) {
        const uint32_t sign = static_cast<uint32_t>(bits & 0x8000u) << 16;
        const uint32_t exp = (bits >> 10) & 0x1fu;
        uint32_t frac = bits & 0x3ffu;
        uint32_t u;
        if (exp == 0x1fu) {
            u = sign | 0x7f800000u | (frac << 13);
        } else if (exp != 0) {
            u = sign | ((exp + 112u) << 23) | (frac << 13);
        } else if (frac == 0) {
            u = sign;
        } else {
            int e = -1;
            do {
                ++e;
                frac <<= 1;
            } while (!(frac & 0x400u));
            u = sign | (static_cast<uint32_t>(112 - e) << 23) | ((frac & 0x3ffu) << 13);
        }
        float f;
        std::memcpy(&f, &u, 4);
        return f;
    }
};

inline std::ostream& operator<<(std::ostream& os, const half& v) { return os << static_cast<float>(v); }

}}  // namespace gpgpu::blas

#endif
