// rope_forward and RopeOptions — reference: include/ops/rope.h:6-31. query/key are
// [batch, sequence, heads, head_dim]; cos/sin caches are [positions, rotary_dim / 2].
#pragma once

#include "core/status.h"
#include "core/tensor.h"

struct RopeOptions {
    std::size_t rotary_dim = 0;  // 0: the whole head dimension
    std::size_t position_offset = 0;
};

namespace cgptx_detail {
struct RopeShape {
    std::size_t batch, sequence, query_heads, kv_heads, head_dim, rotary_dim, positions;
};
inline RopeShape rope_shape(const char* op, const Tensor& query, const Tensor& key, const Tensor& cos_cache,
                            const Tensor& sin_cache, const RopeOptions& options) {
    if (query.dim() != 4 || key.dim() != 4 || query.size(0) != key.size(0) || query.size(1) != key.size(1) ||
        query.size(3) != key.size(3))
        throw std::invalid_argument(std::string(op) + ": query and key must be [batch, sequence, heads, head_dim]");
    const std::size_t rotary = options.rotary_dim == 0 ? query.size(3) : options.rotary_dim;
    if (cos_cache.dim() != 2 || cos_cache.shape() != sin_cache.shape() || cos_cache.size(1) * 2 != rotary)
        throw std::invalid_argument(std::string(op) + ": caches must be [positions, rotary_dim / 2]");
    return {query.size(0), query.size(1), query.size(2), key.size(2), query.size(3), rotary, cos_cache.size(0)};
}
}  // namespace cgptx_detail

// In place on query and key.
inline void rope_forward(Tensor& query, Tensor& key, const Tensor& cos_cache, const Tensor& sin_cache, hipStream_t stream,
                         const RopeOptions& rope_options = {}) {
    using namespace cgptx_detail;
    const char* op = "rope_forward";
    require_device(op, {&query, &key, &cos_cache, &sin_cache});
    require_same_dtype(op, query, {&key, &cos_cache, &sin_cache});
    const RopeShape s = rope_shape(op, query, key, cos_cache, sin_cache, rope_options);
    check(cgptx_rope_forward(query.raw_data(), key.raw_data(), cos_cache.raw_data(), sin_cache.raw_data(), s.batch,
                             s.sequence, s.query_heads, s.kv_heads, s.head_dim, s.rotary_dim, rope_options.position_offset,
                             s.positions, dtype_code(query.dtype()), stream));
}
