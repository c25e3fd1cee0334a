// cross_entropy_forward[_backward] — reference: include/ops/cross_entropy.h:25-45. loss is one F32
// value (mean over rows); gradient = (softmax − onehot)·gradient_scale / rows in the logits dtype.
#pragma once

#include "core/status.h"
#include "core/tensor.h"
#include "core/token_id.h"

inline void cross_entropy_forward_backward(Tensor& loss, Tensor& gradient, const Tensor& logits,
                                           const bpe::TokenId* device_targets, std::size_t target_count,
                                           hipStream_t stream = nullptr, float gradient_scale = 1.0F) {
    using namespace cgptx_detail;
    const char* op = "cross_entropy_forward_backward";
    require_device(op, {&loss, &gradient, &logits});
    require_same_dtype(op, logits, {&gradient});
    require_same_shape(op, logits, {&gradient});
    if (loss.dtype() != Dtype::F32 || loss.numel() != 1 || logits.dim() == 0 || target_count == 0 ||
        logits.numel() != target_count * logits.shape().back() || device_targets == nullptr)
        throw std::invalid_argument("cross_entropy_forward_backward: incompatible tensors or target count");
    check(cgptx_cross_entropy_forward_backward(static_cast<float*>(loss.raw_data()), gradient.raw_data(), logits.raw_data(),
                                               device_targets, target_count, logits.shape().back(), gradient_scale,
                                               dtype_code(logits.dtype()), stream));
}

inline void cross_entropy_forward(Tensor& loss, const Tensor& logits, const bpe::TokenId* device_targets,
                                  std::size_t target_count, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    const char* op = "cross_entropy_forward";
    require_device(op, {&loss, &logits});
    if (loss.dtype() != Dtype::F32 || loss.numel() != 1 || logits.dim() == 0 || target_count == 0 ||
        logits.numel() != target_count * logits.shape().back() || device_targets == nullptr)
        throw std::invalid_argument("cross_entropy_forward: incompatible tensors or target count");
    check(cgptx_cross_entropy_forward(static_cast<float*>(loss.raw_data()), logits.raw_data(), device_targets, target_count,
                                      logits.shape().back(), dtype_code(logits.dtype()), stream));
}
