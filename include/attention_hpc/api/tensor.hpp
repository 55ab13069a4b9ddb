// 16-bit storage types of the public API.  The reference declares half and bfloat16 with
// float conversions but never defines them (src/api/tensor.hpp:39-66); here they are defined:
// round-to-nearest-even, NaN preserved, overflow to infinity - the same rule the device kernels
// use, so host-converted and device-converted tensors agree bit for bit.  The reference's
// Tensor<T> container and MemoryManager are not part of the attention path and are not provided.
#pragma once

#include <cstdint>
#include <cstring>

#include "attention_interface.hpp"

namespace attention_hpc {

namespace detail {
inline uint32_t f32_bits(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float bits_f32(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

inline uint16_t f32_to_bf16_bits(float x) {
    uint32_t u = f32_bits(x);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return static_cast<uint16_t>(u >> 16);
}

inline uint16_t f32_to_f16_bits(float x) {
    const uint32_t u = f32_bits(x);
    const uint16_t sign = static_cast<uint16_t>((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return static_cast<uint16_t>(sign | 0x7E00u | ((a >> 13) & 0x1FFu));
    if (a >= 0x47800000u) return static_cast<uint16_t>(sign | 0x7C00u);
    if (a >= 0x38800000u) {
        const uint32_t m = a - 0x38000000u;
        return static_cast<uint16_t>(sign | ((m + 0x0FFFu + ((m >> 13) & 1u)) >> 13));
    }
    if (a < 0x33000000u) return sign;
    const int shift = 126 - static_cast<int>(a >> 23);
    const uint32_t m = (a & 0x7FFFFFu) | 0x800000u;
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    return static_cast<uint16_t>(sign | q);
}

inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0x1Fu) return bits_f32(sign | 0x7F800000u | (m << 13));
    if (e != 0) return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
    const float f = static_cast<float>(m) * (1.0f / 16777216.0f);
    return sign ? -f : f;
}
}  // namespace detail

struct half {
    uint16_t data = 0;
    half() = default;
    half(float f) : data(detail::f32_to_f16_bits(f)) {}
    operator float() const { return detail::f16_bits_to_f32(data); }
};

struct bfloat16 {
    uint16_t data = 0;
    bfloat16() = default;
    bfloat16(float f) : data(detail::f32_to_bf16_bits(f)) {}
    operator float() const { return detail::bits_f32(static_cast<uint32_t>(data) << 16); }
};

template <typename T> struct DataTypeOf;
template <> struct DataTypeOf<float> { static constexpr DataType value = DataType::FLOAT32; };
template <> struct DataTypeOf<half> { static constexpr DataType value = DataType::FLOAT16; };
template <> struct DataTypeOf<bfloat16> { static constexpr DataType value = DataType::BFLOAT16; };

}  // namespace attention_hpc
