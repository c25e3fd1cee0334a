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
}  // namespace cgptx_detail
