// rope_backward — reference: include/ops/backward/rope_backward.h:22-31.
#pragma once

#include "ops/rope.h"

inline void rope_backward(Tensor& grad_query, Tensor& grad_key, const Tensor& grad_rotated_query,
                          const Tensor& grad_rotated_key, const Tensor& cos_cache, const Tensor& sin_cache,
                          hipStream_t stream = nullptr, const RopeOptions& rope_options = {}) {
    using namespace cgptx_detail;
    const char* op = "rope_backward";
    require_device(op, {&grad_query, &grad_key, &grad_rotated_query, &grad_rotated_key, &cos_cache, &sin_cache});
    require_same_dtype(op, grad_rotated_query, {&grad_query, &grad_key, &grad_rotated_key, &cos_cache, &sin_cache});
    require_same_shape(op, grad_rotated_query, {&grad_query});
    require_same_shape(op, grad_rotated_key, {&grad_key});
    const RopeShape s = rope_shape(op, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache, rope_options);
    check(cgptx_rope_backward(grad_query.raw_data(), grad_key.raw_data(), grad_rotated_query.raw_data(),
                              grad_rotated_key.raw_data(), cos_cache.raw_data(), sin_cache.raw_data(), s.batch, s.sequence,
                              s.query_heads, s.kv_heads, s.head_dim, s.rotary_dim, rope_options.position_offset,
                              s.positions, dtype_code(grad_rotated_query.dtype()), stream));
}
