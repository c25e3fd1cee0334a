// rmsnorm_forward — same signature as the reference's include/ops/rmsnorm.h:20-26 with a HIP stream.
#pragma once

#include "core/status.h"
#include "core/tensor.h"

inline void rmsnorm_forward(Tensor& output, const Tensor& input, const Tensor& weight, float epsilon,
                            hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "rmsnorm_forward";
    require_device(op, {&output, &input, &weight});
    require_same_dtype(op, input, {&output, &weight});
    if (input.dim() == 0 || weight.dim() != 1 || weight.size(0) != input.shape().back() || output.shape() != input.shape())
        throw std::invalid_argument("rmsnorm_forward: incompatible shapes");
    const std::size_t hidden = input.shape().back();
    check(cgptx_rmsnorm_forward(output.raw_data(), input.raw_data(), weight.raw_data(), input.numel() / hidden, hidden,
                                epsilon, dtype_code(input.dtype()), stream));
}

// Allocating overload (reference: include/ops/rmsnorm.h:37-42).
inline Tensor rmsnorm_forward(const Tensor& input, const Tensor& weight, float epsilon, hipStream_t stream = nullptr) {
    Tensor output(input.shape(), DeviceType::GPU, input.dtype());
    rmsnorm_forward(output, input, weight, epsilon, stream);
    return output;
}
