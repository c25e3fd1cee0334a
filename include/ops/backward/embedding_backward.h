// embedding_backward — reference: include/ops/backward/embedding_backward.h:10-42.
// dW[id_t, :] += dY[t, :]; dW is cleared first unless accumulate_weight. Rows are summed in token
// order, so the result does not depend on scheduling.
#pragma once

#include "core/status.h"
#include "core/tensor.h"
#include "core/token_id.h"

struct EmbeddingBackwardOptions {
    int block_size = 0;  // accepted, not used
    bool bounds_check = true;
    bool accumulate_weight = false;
};

inline void embedding_backward(Tensor& grad_weight, const Tensor& grad_output, const bpe::TokenId* device_token_ids,
                               std::size_t token_count, hipStream_t stream = nullptr,
                               const EmbeddingBackwardOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "embedding_backward";
    require_device(op, {&grad_weight, &grad_output});
    require_same_dtype(op, grad_weight, {&grad_output});
    if (grad_weight.dim() != 2 || grad_output.numel() != token_count * grad_weight.size(1) || device_token_ids == nullptr)
        throw std::invalid_argument("embedding_backward: incompatible tensors or token count");
    check(cgptx_embedding_backward(grad_weight.raw_data(), grad_output.raw_data(), device_token_ids, token_count,
                                   grad_weight.size(0), grad_weight.size(1), options.bounds_check,
                                   options.accumulate_weight, dtype_code(grad_weight.dtype()), stream));
}
