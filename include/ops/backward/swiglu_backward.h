// swiglu_backward — reference: include/ops/backward/swiglu_backward.h:9-38; the concatenated
// overload is defined in src/ops/backward/swiglu_backward.cu:830-883.
#pragma once

#include "core/status.h"
#include "core/tensor.h"

struct SwiGLUBackwardOptions {
    bool accumulate_gate = false;
    bool accumulate_up = false;
    bool accumulate_gate_up = false;
};

inline void swiglu_backward(Tensor& grad_gate, Tensor& grad_up, const Tensor& grad_output, const Tensor& gate,
                            const Tensor& up, hipStream_t stream = nullptr, const SwiGLUBackwardOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "swiglu_backward";
    require_device(op, {&grad_gate, &grad_up, &grad_output, &gate, &up});
    require_same_dtype(op, gate, {&grad_gate, &grad_up, &grad_output, &up});
    require_same_shape(op, gate, {&grad_gate, &grad_up, &grad_output, &up});
    check(cgptx_swiglu_backward(grad_gate.raw_data(), grad_up.raw_data(), grad_output.raw_data(), gate.raw_data(),
                                up.raw_data(), gate.numel(), options.accumulate_gate, options.accumulate_up,
                                dtype_code(gate.dtype()), stream));
}

inline void swiglu_backward(Tensor& grad_gate_up, const Tensor& grad_output, const Tensor& gate_up,
                            hipStream_t stream = nullptr, const SwiGLUBackwardOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "swiglu_backward";
    require_device(op, {&grad_gate_up, &grad_output, &gate_up});
    require_same_dtype(op, gate_up, {&grad_gate_up, &grad_output});
    require_same_shape(op, gate_up, {&grad_gate_up});
    if (gate_up.dim() == 0 || gate_up.shape().back() % 2 != 0 || grad_output.numel() * 2 != gate_up.numel())
        throw std::invalid_argument("swiglu_backward: gate_up must hold [gate | up] for every grad_output row");
    if (grad_output.numel() == 0) return;  // nothing to do (src/ops/backward/swiglu_backward.cu:839-841)
    const std::size_t hidden = gate_up.shape().back() / 2;
    check(cgptx_swiglu_backward_packed(grad_gate_up.raw_data(), grad_output.raw_data(), gate_up.raw_data(),
                                       grad_output.numel() / hidden, hidden, options.accumulate_gate_up,
                                       dtype_code(gate_up.dtype()), stream));
}
