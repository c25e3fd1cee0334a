// rmsnorm_backward — reference: include/ops/backward/rmsnorm_backward.h:21-29.
#pragma once

#include "core/status.h"
#include "core/tensor.h"

inline void rmsnorm_backward(Tensor& grad_input, Tensor& grad_weight, const Tensor& grad_output, const Tensor& input,
                             const Tensor& weight, float epsilon, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "rmsnorm_backward";
    require_device(op, {&grad_input, &grad_weight, &grad_output, &input, &weight});
    require_same_dtype(op, input, {&grad_input, &grad_weight, &grad_output, &weight});
    if (input.dim() == 0 || weight.dim() != 1 || weight.size(0) != input.shape().back() ||
        grad_weight.shape() != weight.shape())
        throw std::invalid_argument("rmsnorm_backward: incompatible shapes");
    require_same_shape(op, input, {&grad_input, &grad_output});
    const std::size_t hidden = input.shape().back();
    check(cgptx_rmsnorm_backward(grad_input.raw_data(), grad_weight.raw_data(), grad_output.raw_data(), input.raw_data(),
                                 weight.raw_data(), input.numel() / hidden, hidden, epsilon, dtype_code(input.dtype()),
                                 stream));
}
