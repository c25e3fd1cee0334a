// flash_gqa_attention_backward[_with_lse] — reference: include/ops/backward/attention_backward.h:24-70.
#pragma once

#include "ops/attention.h"

inline void flash_gqa_attention_backward_with_lse(Tensor& grad_query, Tensor& grad_key, Tensor& grad_value,
                                                  const Tensor& grad_output, const Tensor& output, const Tensor& logsumexp,
                                                  const Tensor& query, const Tensor& key, const Tensor& value,
                                                  hipStream_t stream = nullptr, const FlashAttentionOptions& options = {},
                                                  bool accumulate_grads = false) {
    using namespace cgptx_detail;
    const char* op = "flash_gqa_attention_backward_with_lse";
    require_device(op, {&grad_query, &grad_key, &grad_value, &grad_output, &output, &logsumexp, &query, &key, &value});
    require_same_dtype(op, query, {&grad_query, &grad_key, &grad_value, &grad_output, &output, &key, &value});
    require_same_shape(op, query, {&grad_query, &grad_output, &output});
    require_same_shape(op, key, {&grad_key, &grad_value});
    const AttentionShape s = attention_shape(op, query, key, value, options);
    if (logsumexp.dtype() != Dtype::F32 || logsumexp.numel() != s.batch * s.query_sequence * options.num_query_heads)
        throw std::invalid_argument("flash_gqa_attention_backward_with_lse: logsumexp must be F32 [batch, sequence, heads]");
    check(cgptx_flash_gqa_attention_backward_with_lse(
        grad_query.raw_data(), grad_key.raw_data(), grad_value.raw_data(), grad_output.raw_data(), output.raw_data(),
        static_cast<const float*>(logsumexp.raw_data()), query.raw_data(), key.raw_data(), value.raw_data(), s.batch,
        s.query_sequence, s.kv_sequence, options.num_query_heads, options.num_kv_heads, options.head_dim,
        options.attention_scale, options.causal, options.query_position_offset, accumulate_grads,
        dtype_code(query.dtype()), stream));
}

// Recomputes the output and the log-sum-exp first.
inline void flash_gqa_attention_backward(Tensor& grad_query, Tensor& grad_key, Tensor& grad_value, const Tensor& grad_output,
                                         const Tensor& query, const Tensor& key, const Tensor& value,
                                         hipStream_t stream = nullptr, const FlashAttentionOptions& options = {},
                                         bool accumulate_grads = false) {
    using namespace cgptx_detail;
    const char* op = "flash_gqa_attention_backward";
    require_device(op, {&grad_query, &grad_key, &grad_value, &grad_output, &query, &key, &value});
    require_same_dtype(op, query, {&grad_query, &grad_key, &grad_value, &grad_output, &key, &value});
    require_same_shape(op, query, {&grad_query, &grad_output});
    require_same_shape(op, key, {&grad_key, &grad_value});
    const AttentionShape s = attention_shape(op, query, key, value, options);
    check(cgptx_flash_gqa_attention_backward(grad_query.raw_data(), grad_key.raw_data(), grad_value.raw_data(),
                                             grad_output.raw_data(), query.raw_data(), key.raw_data(), value.raw_data(),
                                             s.batch, s.query_sequence, s.kv_sequence, options.num_query_heads,
                                             options.num_kv_heads, options.head_dim, options.attention_scale,
                                             options.causal, options.query_position_offset, accumulate_grads,
                                             dtype_code(query.dtype()), stream));
}
