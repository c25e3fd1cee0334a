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

// The weight gradients of several layers of one shape in one launch: grad_output [count, rows, out], input
// [count, rows, in], grad_weight [count, out, in], all contiguous — `count` calls of linear_backward that ask for the
// weight gradient only, as the reference's block backward makes them for every block of a model
// (src/core/transformer_block.cu:660-745). No single reference function corresponds.
inline void linear_backward_weights_stacked(Tensor& grad_weight, const Tensor& grad_output, const Tensor& input,
                                            const GemmContext&, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "linear_backward_weights_stacked";
    require_device(op, {&grad_weight, &grad_output, &input});
    require_same_dtype(op, input, {&grad_weight, &grad_output});
    if (grad_weight.dim() != 3 || grad_output.dim() != 3 || input.dim() != 3 || grad_output.size(0) != grad_weight.size(0) ||
        input.size(0) != grad_weight.size(0) || grad_output.size(1) != input.size(1) ||
        grad_output.size(2) != grad_weight.size(1) || input.size(2) != grad_weight.size(2))
        throw std::invalid_argument("linear_backward_weights_stacked: incompatible tensors");
    check(cgptx_linear_backward_weights_stacked(grad_weight.raw_data(), grad_output.raw_data(), input.raw_data(), input.size(1),
                                                input.size(2), grad_output.size(2), grad_weight.size(0),
                                                grad_output.size(1) * grad_output.size(2), input.size(1) * input.size(2),
                                                dtype_code(input.dtype()), stream));
}
