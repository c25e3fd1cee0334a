// swiglu_forward, separate and concatenated inputs — reference: include/ops/swiglu.h:16-37.
#pragma once

#include "core/status.h"
#include "core/tensor.h"

inline void swiglu_forward(Tensor& output, const Tensor& gate, const Tensor& up, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "swiglu_forward";
    require_device(op, {&output, &gate, &up});
    require_same_dtype(op, gate, {&output, &up});
    require_same_shape(op, gate, {&output, &up});
    check(cgptx_swiglu_forward(output.raw_data(), gate.raw_data(), up.raw_data(), gate.numel(), dtype_code(gate.dtype()),
                               stream));
}

// gate_up holds [gate | up] along its last dimension.
inline void swiglu_forward(Tensor& output, const Tensor& gate_up, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "swiglu_forward";
    require_device(op, {&output, &gate_up});
    require_same_dtype(op, gate_up, {&output});
    if (gate_up.dim() == 0 || gate_up.shape().back() % 2 != 0)
        throw std::invalid_argument("swiglu_forward: the last gate_up dimension must be even");
    const std::size_t hidden = gate_up.shape().back() / 2;
    if (output.dim() != gate_up.dim() || output.shape().back() != hidden || output.numel() * 2 != gate_up.numel())
        throw std::invalid_argument("swiglu_forward: output shape must match gate_up except for its last dimension");
    if (output.numel() == 0) return;  // nothing to do (src/ops/swiglu.cu:581-583)
    check(cgptx_swiglu_forward_packed(output.raw_data(), gate_up.raw_data(), output.numel() / hidden, hidden,
                                      dtype_code(gate_up.dtype()), stream));
}
