// binary16 on the host side of the engine: `half` is the compiler's _Float16
// (hipcc / clang), the type the reference API spells `half`.
#pragma once
#include <cstdint>
#include <cstring>

using half = _Float16;

namespace et {
inline half half_from_bits(uint16_t bits) {
    half h;
    std::memcpy(&h, &bits, sizeof h);
    return h;
}
inline uint16_t half_bits(half h) {
    uint16_t bits;
    std::memcpy(&bits, &h, sizeof bits);
    return bits;
}
}  // namespace et

// The constants the reference defines in lib/utils.h:36-39.
static const half half_one = et::half_from_bits(0x3c00);
static const half half_zero = et::half_from_bits(0x0000);
static const half half_inf = et::half_from_bits(0x7c00);
static const half half_ninf = et::half_from_bits(0xfc00);

inline half __float2half_rn(float f) { return static_cast<half>(f); }  // round-to-nearest-even
inline half __float2half(float f) { return static_cast<half>(f); }
inline float __half2float(half h) { return static_cast<float>(h); }
