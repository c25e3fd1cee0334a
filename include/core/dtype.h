// Storage and compute type tags of the operator interface.
// Mirrors the caller-visible part of the reference's include/core/dtype.h:10-59, 145-150.
#pragma once

#include <cstddef>
#include <cstdint>
#include <stdexcept>

#include "cgptx.h"

enum class Dtype : std::uint8_t { F16, BF16, F32, I32 };

constexpr std::size_t dtype_size(const Dtype dtype) {
    switch (dtype) {
        case Dtype::F16:
        case Dtype::BF16: return 2;
        case Dtype::F32:
        case Dtype::I32: return 4;
    }
    throw std::invalid_argument("Dtype not supported");
}

[[nodiscard]] constexpr bool is_floating_point(const Dtype dtype) noexcept {
    return dtype == Dtype::F16 || dtype == Dtype::BF16 || dtype == Dtype::F32;
}

// Accepted for source compatibility; every contraction here accumulates in fp32 on the matrix cores.
enum class ComputeType { F32, TF32 };

namespace cgptx_detail {
// Dtype -> C-ABI dtype code; I32 is not a floating storage type of any operator.
inline int dtype_code(const Dtype dtype) {
    switch (dtype) {
        case Dtype::F16: return CGPTX_F16;
        case Dtype::BF16: return CGPTX_BF16;
        case Dtype::F32: return CGPTX_F32;
        default: throw std::invalid_argument("operator tensors must be F16, BF16 or F32");
    }
}

// IEEE binary16 bits -> float (exact), without relying on a compiler half type.
inline float half_bits_to_float(const std::uint16_t bits) {
    const std::uint32_t sign = static_cast<std::uint32_t>(bits & 0x8000u) << 16;
    std::uint32_t exponent = (bits >> 10) & 0x1Fu;
    std::uint32_t mantissa = bits & 0x3FFu;
    std::uint32_t word;
    if (exponent == 0x1Fu) {
        word = sign | 0x7F800000u | (mantissa << 13);
    } else if (exponent != 0) {
        word = sign | ((exponent + 112u) << 23) | (mantissa << 13);
    } else if (mantissa == 0) {
        word = sign;
    } else {  // subnormal: renormalise
        exponent = 113u;
        while ((mantissa & 0x400u) == 0) {
            mantissa <<= 1;
            --exponent;
        }
        word = sign | (exponent << 23) | ((mantissa & 0x3FFu) << 13);
    }
    float value;
    static_assert(sizeof(value) == sizeof(word));
    __builtin_memcpy(&value, &word, sizeof(value));
    return value;
}

// float -> IEEE binary16 bits, round to nearest even (what static_cast<__half>(float) does on the host).
inline std::uint16_t float_to_half_bits(const float value) {
    std::uint32_t word;
    __builtin_memcpy(&word, &value, sizeof(word));
    const std::uint16_t sign = static_cast<std::uint16_t>((word >> 16) & 0x8000u);
    const std::uint32_t magnitude = word & 0x7FFFFFFFu;
    if (magnitude >= 0x7F800000u)  // infinity or NaN (quiet, payload's top bits kept)
        return static_cast<std::uint16_t>(sign | 0x7C00u | (magnitude > 0x7F800000u ? 0x200u | ((magnitude >> 13) & 0x3FFu) : 0u));
    if (magnitude >= 0x477FF000u) return static_cast<std::uint16_t>(sign | 0x7C00u);  // rounds to 65536 or more
    if (magnitude < 0x33000001u) return sign;                                          // at most half the smallest subnormal
    std::uint32_t mantissa, shift;
    std::int32_t exponent = static_cast<std::int32_t>(magnitude >> 23) - 127 + 15;
    if (exponent <= 0) {  // subnormal half: shift the 24-bit significand into place
        mantissa = (magnitude & 0x7FFFFFu) | 0x800000u;
        shift = static_cast<std::uint32_t>(14 - exponent);
        exponent = 0;
    } else {
        mantissa = magnitude & 0x7FFFFFu;
        shift = 13;
    }
    std::uint32_t result = (static_cast<std::uint32_t>(exponent) << 10) + (mantissa >> shift);
    const std::uint32_t remainder = mantissa & ((1u << shift) - 1u), halfway = 1u << (shift - 1u);
    if (remainder > halfway || (remainder == halfway && (result & 1u))) ++result;  // a carry moves into the exponent
    return static_cast<std::uint16_t>(sign | result);
}

// float -> bfloat16 bits, round to nearest even; NaN stays NaN.
inline std::uint16_t float_to_bf16_bits(const float value) {
    std::uint32_t word;
    __builtin_memcpy(&word, &value, sizeof(word));
    if ((word & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<std::uint16_t>((word >> 16) | 0x40u);
    return static_cast<std::uint16_t>((word + 0x7FFFu + ((word >> 16) & 1u)) >> 16);
}

inline float bf16_bits_to_float(const std::uint16_t bits) {
    const std::uint32_t word = static_cast<std::uint32_t>(bits) << 16;
    float value;
    __builtin_memcpy(&value, &word, sizeof(value));
    return value;
}
}  // namespace cgptx_detail
