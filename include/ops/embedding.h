// embedding_forward — reference: include/ops/embedding.h:10-50. out[t, :] = weight[id_t, :].
#pragma once

#include <span>

#include "core/status.h"
#include "core/tensor.h"
#include "core/token_id.h"

struct EmbeddingOptions {
    int block_size = 0;         // accepted, not used
    bool bounds_check = true;   // ids >= vocabulary give a zero row
};

// Copies token ids to device memory on the stream (reference: embedding_upload_token_ids).
inline void embedding_upload_token_ids(bpe::TokenId* device_destination, std::span<const bpe::TokenId> token_ids,
                                       hipStream_t stream = nullptr) {
    if (token_ids.empty()) return;
    if (device_destination == nullptr) throw std::invalid_argument("embedding_upload_token_ids: null destination");
    if (hipMemcpyAsync(device_destination, token_ids.data(), token_ids.size_bytes(), hipMemcpyHostToDevice, stream) != hipSuccess)
        throw std::runtime_error("embedding_upload_token_ids: copy failed");
}

inline void embedding_forward(Tensor& output, const bpe::TokenId* device_token_ids, std::size_t token_count,
                              const Tensor& weight, hipStream_t stream = nullptr, const EmbeddingOptions& = {}) {
    using namespace cgptx_detail;
    const char* op = "embedding_forward";
    require_device(op, {&output, &weight});
    require_same_dtype(op, weight, {&output});
    if (weight.dim() != 2 || output.numel() != token_count * weight.size(1) || device_token_ids == nullptr)
        throw std::invalid_argument("embedding_forward: incompatible tensors or token count");
    check(cgptx_embedding_forward(output.raw_data(), device_token_ids, token_count, weight.raw_data(), weight.size(0),
                                  weight.size(1), dtype_code(weight.dtype()), stream));
}
