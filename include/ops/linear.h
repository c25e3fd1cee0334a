// linear_forward — reference: include/ops/linear.h:10-45. Y[.., out] = X[.., in]·W[out, in]ᵀ (+ bias).
#pragma once

#include "core/gemm_context.h"
#include "core/status.h"
#include "core/tensor.h"

struct LinearOptions {
    ComputeType compute_type = ComputeType::TF32;         // accepted, not used: accumulation is fp32
    std::size_t workspace_bytes = 32U * 1024U * 1024U;    // accepted, not used: scratch is the library's own
};

namespace cgptx_detail {
inline void linear_forward_impl(Tensor& output, const Tensor& input, const Tensor& weight, const Tensor* bias,
                                hipStream_t stream) {
    const char* op = "linear_forward";
    require_device(op, {&output, &input, &weight});
    require_same_dtype(op, input, {&output, &weight});
    if (weight.dim() != 2 || input.dim() == 0 || output.dim() != input.dim() || input.shape().back() != weight.size(1) ||
        output.shape().back() != weight.size(0) || output.numel() / weight.size(0) != input.numel() / weight.size(1))
        throw std::invalid_argument("linear_forward: incompatible tensors");
    if (bias != nullptr) {
        require_device(op, {bias});
        require_same_dtype(op, input, {bias});
        if (bias->numel() != weight.size(0)) throw std::invalid_argument("linear_forward: bias must have out_features elements");
    }
    check(cgptx_linear_forward(output.raw_data(), input.raw_data(), weight.raw_data(), bias ? bias->raw_data() : nullptr,
                               input.numel() / weight.size(1), weight.size(1), weight.size(0), dtype_code(input.dtype()),
                               stream));
}
}  // namespace cgptx_detail

inline void linear_forward(Tensor& output, const Tensor& input, const Tensor& weight, const GemmContext&,
                           hipStream_t stream = nullptr, const LinearOptions& = {}) {
    cgptx_detail::linear_forward_impl(output, input, weight, nullptr, stream);
}

inline void linear_forward(Tensor& output, const Tensor& input, const Tensor& weight, const Tensor& bias,
                           const GemmContext&, hipStream_t stream = nullptr, const LinearOptions& = {}) {
    cgptx_detail::linear_forward_impl(output, input, weight, &bias, stream);
}

// The feed-forward's gate and up projections and its SwiGLU as one call: the sequence
// linear_forward(gate), linear_forward(up), swiglu_forward(activated, gate, up) of the reference's
// src/core/transformer_block.cu:586-590 over the concatenated layouts of include/ops/swiglu.h:33-37
// (weight = [gate_proj; up_proj], gate_up = [gate | up]); no single reference function corresponds.
inline void linear_swiglu_forward(Tensor& gate_up, Tensor& activated, const Tensor& input, const Tensor& weight,
                                  const GemmContext&, hipStream_t stream = nullptr) {
    const char* op = "linear_swiglu_forward";
    cgptx_detail::require_device(op, {&gate_up, &activated, &input, &weight});
    cgptx_detail::require_same_dtype(op, input, {&gate_up, &activated, &weight});
    if (weight.dim() != 2 || weight.size(0) % 2 != 0 || input.numel() == 0 || input.dim() == 0 || input.shape().back() != weight.size(1) ||
        gate_up.numel() != input.numel() / weight.size(1) * weight.size(0) || activated.numel() * 2 != gate_up.numel())
        throw std::invalid_argument("linear_swiglu_forward: incompatible tensors");
    cgptx_detail::check(cgptx_linear_swiglu_forward(gate_up.raw_data(), activated.raw_data(), input.raw_data(), weight.raw_data(),
                                                    input.numel() / weight.size(1), weight.size(1), weight.size(0) / 2,
                                                    cgptx_detail::dtype_code(input.dtype()), stream));
}

// The input gradient of the down projection and the SwiGLU gradient as one call: the sequence
// linear_backward(down) (input gradient), swiglu_backward of the reference's
// src/core/transformer_block.cu:663-666 over the concatenated layouts of
// src/ops/backward/swiglu_backward.cu:830-883 (gate_up = the forward's [gate | up], grad_gate_up =
// [dgate | dup]); grad_activated is working memory. No single reference function corresponds.
inline void linear_swiglu_backward(Tensor& grad_gate_up, Tensor& grad_activated, const Tensor& grad_output, const Tensor& weight,
                                   const Tensor& gate_up, const GemmContext&, hipStream_t stream = nullptr) {
    const char* op = "linear_swiglu_backward";
    cgptx_detail::require_device(op, {&grad_gate_up, &grad_activated, &grad_output, &weight, &gate_up});
    cgptx_detail::require_same_dtype(op, grad_output, {&grad_gate_up, &grad_activated, &weight, &gate_up});
    if (weight.dim() != 2 || grad_output.numel() == 0 || grad_output.dim() == 0 || grad_output.shape().back() != weight.size(0) ||
        grad_activated.numel() != grad_output.numel() / weight.size(0) * weight.size(1) ||
        gate_up.numel() != 2 * grad_activated.numel() || grad_gate_up.numel() != gate_up.numel())
        throw std::invalid_argument("linear_swiglu_backward: incompatible tensors");
    cgptx_detail::check(cgptx_linear_swiglu_backward(grad_gate_up.raw_data(), grad_activated.raw_data(), grad_output.raw_data(),
                                                     weight.raw_data(), gate_up.raw_data(), grad_output.numel() / weight.size(0),
                                                     weight.size(1), weight.size(0), cgptx_detail::dtype_code(grad_output.dtype()),
                                                     stream));
}
