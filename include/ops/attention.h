// flash_gqa_attention_forward[_with_lse] and FlashAttentionOptions — reference: include/ops/attention.h:8-78.
// query/output [batch, q_seq, q_heads, head_dim]; key/value [batch, kv_seq, kv_heads, head_dim];
// logsumexp F32 [batch, q_seq, q_heads] (natural log of the sum of exp of the scaled scores).
#pragma once

#include "core/status.h"
#include "core/tensor.h"

struct FlashAttentionOptions {
    std::size_t num_query_heads = 0;
    std::size_t num_kv_heads = 0;
    std::size_t head_dim = 0;
    float attention_scale = 0.0F;  // <= 0: 1 / sqrt(head_dim)
    bool causal = true;
    std::size_t query_position_offset = 0;
    int key_tile_size = 16;        // the three tuning fields are accepted and not used
    int block_size = 128;
    bool use_tensor_cores = true;
};

namespace cgptx_detail {
struct AttentionShape {
    std::size_t batch, query_sequence, kv_sequence;
};
inline AttentionShape attention_shape(const char* op, const Tensor& query, const Tensor& key, const Tensor& value,
                                      const FlashAttentionOptions& o) {
    if (query.dim() != 4 || key.dim() != 4 || key.shape() != value.shape() || query.size(0) != key.size(0) ||
        query.size(2) != o.num_query_heads || key.size(2) != o.num_kv_heads || query.size(3) != o.head_dim ||
        key.size(3) != o.head_dim)
        throw std::invalid_argument(std::string(op) + ": tensors do not match the attention options");
    return {query.size(0), query.size(1), key.size(1)};
}
}  // namespace cgptx_detail

inline void flash_gqa_attention_forward_with_lse(Tensor& output, Tensor& logsumexp, const Tensor& query, const Tensor& key,
                                                 const Tensor& value, hipStream_t stream = nullptr,
                                                 const FlashAttentionOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "flash_gqa_attention_forward_with_lse";
    require_device(op, {&output, &logsumexp, &query, &key, &value});
    require_same_dtype(op, query, {&output, &key, &value});
    require_same_shape(op, query, {&output});
    const AttentionShape s = attention_shape(op, query, key, value, options);
    if (logsumexp.dtype() != Dtype::F32 || logsumexp.numel() != s.batch * s.query_sequence * options.num_query_heads)
        throw std::invalid_argument("flash_gqa_attention_forward_with_lse: logsumexp must be F32 [batch, sequence, heads]");
    check(cgptx_flash_gqa_attention_forward(output.raw_data(), static_cast<float*>(logsumexp.raw_data()), query.raw_data(),
                                            key.raw_data(), value.raw_data(), s.batch, s.query_sequence, s.kv_sequence,
                                            options.num_query_heads, options.num_kv_heads, options.head_dim,
                                            options.attention_scale, options.causal, options.query_position_offset,
                                            dtype_code(query.dtype()), stream));
}

inline void flash_gqa_attention_forward(Tensor& output, const Tensor& query, const Tensor& key, const Tensor& value,
                                        hipStream_t stream = nullptr, const FlashAttentionOptions& options = {}) {
    using namespace cgptx_detail;
    const char* op = "flash_gqa_attention_forward";
    require_device(op, {&output, &query, &key, &value});
    require_same_dtype(op, query, {&output, &key, &value});
    require_same_shape(op, query, {&output});
    const AttentionShape s = attention_shape(op, query, key, value, options);
    check(cgptx_flash_gqa_attention_forward(output.raw_data(), nullptr, query.raw_data(), key.raw_data(), value.raw_data(),
                                            s.batch, s.query_sequence, s.kv_sequence, options.num_query_heads,
                                            options.num_kv_heads, options.head_dim, options.attention_scale, options.causal,
                                            options.query_position_offset, dtype_code(query.dtype()), stream));
}
