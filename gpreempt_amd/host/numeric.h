// Host-side numeric helpers: seeded random numbers and 16-bit float conversion (the host
// compiler has no native half type).
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

namespace foo {
namespace numeric {

// splitmix64 -> uniform / Box-Muller normal; fixed across platforms so that random-init
// weights are reproducible.
class Rng {
public:
    explicit Rng(uint64_t seed) : s_(seed) {}
    uint64_t next() {
        uint64_t z = (s_ += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform01() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    float uniform(float lo, float hi) { return (float)(lo + (hi - lo) * uniform01()); }
    float normal() {
        if (has_spare_) { has_spare_ = false; return spare_; }
        double u1 = uniform01(), u2 = uniform01();
        if (u1 < 1e-300) u1 = 1e-300;
        double r = std::sqrt(-2.0 * std::log(u1)), a = 6.283185307179586 * u2;
        spare_ = (float)(r * std::sin(a));
        has_spare_ = true;
        return (float)(r * std::cos(a));
    }

private:
    uint64_t s_;
    bool has_spare_ = false;
    float spare_ = 0.f;
};

inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);  // quiet NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// IEEE binary32 -> binary16, round to nearest even, with subnormals, infinities and NaN.
inline uint16_t f32_to_f16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0));
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // rounds to >= 65520 -> inf
    if (ax < 0x38800000u) {                                     // subnormal half or zero
        if (ax < 0x33000000u) return (uint16_t)sign;            // < 2^-25 -> 0
        uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
        int shift = 126 - (int)(ax >> 23);                      // 14..24
        uint32_t half = mant >> shift;
        uint32_t rem = mant & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) ++half;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((ax - 0x38000000u) >> 13);
    uint32_t rem = ax & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) ++half;
    return (uint16_t)(sign | half);
}
inline float f16_to_f32(uint16_t h) {
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16, exp = (h >> 10) & 0x1f, mant = h & 0x3ffu, u;
    if (exp == 0) {
        if (mant == 0) u = sign;
        else {
            int e = -1;
            do { mant <<= 1; ++e; } while (!(mant & 0x400u));
            u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((mant & 0x3ffu) << 13);
        }
    } else if (exp == 31) u = sign | 0x7f800000u | (mant << 13);
    else u = sign | ((exp + 112) << 23) | (mant << 13);
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

}  // namespace numeric
}  // namespace foo
