// cut_cross_entropy_forward_backward — reference: include/ops/cut_cross_entropy.h:25-33.
// Loss and both gradients of the classifier product without ever holding all logits. Beyond the
// reference (F32 only): 16-bit storage with fp32 accumulation.
#pragma once

#include "core/status.h"
#include "core/tensor.h"
#include "core/token_id.h"

inline void cut_cross_entropy_forward_backward(Tensor& loss, Tensor& input_gradient, Tensor& classifier_gradient,
                                               const Tensor& input, const Tensor& classifier,
                                               const bpe::TokenId* device_targets, std::size_t target_count,
                                               hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "cut_cross_entropy_forward_backward";
    require_device(op, {&loss, &input_gradient, &classifier_gradient, &input, &classifier});
    require_same_dtype(op, input, {&input_gradient, &classifier_gradient, &classifier});
    require_same_shape(op, input, {&input_gradient});
    require_same_shape(op, classifier, {&classifier_gradient});
    if (loss.dtype() != Dtype::F32 || loss.numel() != 1 || classifier.dim() != 2 || input.dim() == 0 ||
        input.shape().back() != classifier.size(1) || target_count == 0 ||
        input.numel() != target_count * classifier.size(1) || device_targets == nullptr)
        throw std::invalid_argument("cut_cross_entropy_forward_backward: incompatible tensors or target count");
    check(cgptx_cut_cross_entropy_forward_backward(static_cast<float*>(loss.raw_data()), input_gradient.raw_data(),
                                                   classifier_gradient.raw_data(), input.raw_data(), classifier.raw_data(),
                                                   device_targets, target_count, classifier.size(1), classifier.size(0),
                                                   1.0F, 0, dtype_code(input.dtype()), stream));
}
