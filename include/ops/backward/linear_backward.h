// linear_backward — reference: include/ops/backward/linear_backward.h:10-46.
// dX = dY·W, dW = dYᵀ·X, db = column sums of dY; each accumulate flag adds into the output.
#pragma once

#include "core/gemm_context.h"
#include "core/status.h"
#include "core/tensor.h"

struct LinearBackwardOptions {
    ComputeType compute_type = ComputeType::F32;
    std::size_t workspace_bytes = 32ULL * 1024ULL * 1024ULL;
    bool accumulate_input = false;
    bool accumulate_weight = false;
    bool accumulate_bias = false;
};

inline void linear_backward(Tensor& grad_input, Tensor& grad_weight, Tensor& grad_bias, const Tensor& grad_output,
                            const Tensor& input, const Tensor& weight, const GemmContext&, hipStream_t stream = nullptr,
                            const LinearBackwardOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "linear_backward";
    require_device(op, {&grad_input, &grad_weight, &grad_bias, &grad_output, &input, &weight});
    require_same_dtype(op, input, {&grad_input, &grad_weight, &grad_bias, &grad_output, &weight});
    if (weight.dim() != 2 || input.dim() == 0 || input.shape().back() != weight.size(1) ||
        grad_output.shape().back() != weight.size(0) || grad_weight.shape() != weight.shape() ||
        grad_bias.numel() != weight.size(0) || grad_output.numel() / weight.size(0) != input.numel() / weight.size(1))
        throw std::invalid_argument("linear_backward: incompatible tensors");
    require_same_shape(op, input, {&grad_input});
    check(cgptx_linear_backward(grad_input.raw_data(), grad_weight.raw_data(), grad_bias.raw_data(), grad_output.raw_data(),
                                input.raw_data(), weight.raw_data(), input.numel() / weight.size(1), weight.size(1),
                                weight.size(0), options.accumulate_input, options.accumulate_weight,
                                options.accumulate_bias, dtype_code(input.dtype()), stream));
}
