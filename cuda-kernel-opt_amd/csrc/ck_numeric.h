// Host-side numeric helpers: 16-bit float conversions by bit manipulation (no compiler _Float16
// support needed) and the counter-based SplitMix64 generator.
#ifndef CK_NUMERIC_H
#define CK_NUMERIC_H

#include <stdint.h>
#include <string.h>

namespace ck {

inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

// IEEE binary32 -> binary16, round to nearest even, overflow to infinity, subnormals kept.
inline uint16_t float_to_half_bits(float f) {
    const uint32_t x = f32_bits(f);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x0200u | ((ax >> 13) & 0x3ffu) : 0));
    if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);  // >= 65520 rounds to infinity
    if (ax >= 0x38800000u) {                                   // normal half
        const uint32_t m = ax - 0x38000000u;                    // rebias exponent 127 -> 15
        const uint32_t r = m + 0x00000fffu + ((m >> 13) & 1u);  // round to nearest even at bit 13
        return (uint16_t)(sign | (r >> 13));
    }
    if (ax < 0x33000000u) return (uint16_t)sign;  // < 2^-25 rounds to zero
    // subnormal half: value = mant * 2^(e-150), target unit 2^-24
    const int e = (int)(ax >> 23);
    const uint32_t mant = (ax & 0x7fffffu) | 0x800000u;
    const int shift = 126 - e;  // in [14, 24]
    const uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
    const uint32_t r = q + ((rem > half || (rem == half && (q & 1u))) ? 1u : 0u);
    return (uint16_t)(sign | r);
}

inline float half_bits_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1f) return bits_f32(sign | 0x7f800000u | (m << 13));
    if (e) return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    if (!m) return bits_f32(sign);
    // subnormal: m * 2^-24
    const float v = (float)m * (1.0f / 16777216.0f);
    return bits_f32(f32_bits(v) | sign);
}

// IEEE binary32 -> bfloat16, round to nearest even; NaNs stay NaNs.
inline uint16_t float_to_bf16_bits(float f) {
    const uint32_t x = f32_bits(f);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u);
    return (uint16_t)((x + 0x7fffu + ((x >> 16) & 1u)) >> 16);
}
inline float bf16_bits_to_float(uint16_t h) { return bits_f32((uint32_t)h << 16); }

// Output number `index` (0-based) of Vigna's SplitMix64 started from state `base`:
// the state advances by the golden-ratio increment before every output.
inline uint64_t splitmix64_at(uint64_t base, uint64_t index) {
    uint64_t z = base + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

}  // namespace ck
#endif  // CK_NUMERIC_H
