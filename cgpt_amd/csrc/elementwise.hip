// Bandwidth-bound elementwise kernels for gfx950: RoPE forward/backward,
// SwiGLU forward/backward (separate and packed layouts), residual add.
//
// Each thread moves 128 bits per access in a grid-stride loop; adjacent lanes
// touch adjacent 16-byte words, so a wavefront reads/writes 1 KiB contiguous
// per instruction. All arithmetic is fp32 and results are rounded once to the
// storage dtype. Shapes or pointers that do not allow 128-bit access fall back
// to an element-wise kernel with the same arithmetic.
//
// Reference arithmetic: src/ops/cpu/backward/rope_backward_cpu.cpp:110-141,
// src/ops/cpu/rope_cpu.cpp:110-120, src/ops/cpu/backward/swiglu_backward_cpu.cpp:92-182,
// src/ops/cpu/swiglu_cpu.cpp:150-165, src/core/transformer_block.cu:134-144.
#include "common.hpp"

#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;

int grid_for(std::size_t work_items) {
    const std::size_t wanted = (work_items + kThreads - 1) / kThreads;
    const std::size_t cap = static_cast<std::size_t>(compute_units()) * 16;
    const std::size_t blocks = wanted < cap ? wanted : cap;
    return static_cast<int>(blocks == 0 ? 1 : blocks);
}

// ----------------------------------------------------------------------- RoPE
// Rotation of the pair (x, y) by +angle (forward) or -angle (backward).
template <bool Inverse>
__device__ __forceinline__ void rotate(float x, float y, float c, float s, float& ox, float& oy) {
    if constexpr (Inverse) {
        ox = fmaf(y, s, x * c);
        oy = fmaf(-x, s, y * c);
    } else {
        ox = fmaf(-y, s, x * c);
        oy = fmaf(x, s, y * c);
    }
}

struct RopeDims {
    std::uint32_t sequence, query_heads, kv_heads, head_dim, rotary_dim, position_offset;
    std::size_t query_vectors;  // work items belonging to q (vectors or elements)
    std::size_t total_vectors;
};

template <typename T, bool Inverse>
__global__ __launch_bounds__(kThreads) void rope_vec_kernel(T* __restrict__ out_q, T* __restrict__ out_k,
                                                            const T* in_q, const T* in_k,
                                                            const T* __restrict__ cos_cache,
                                                            const T* __restrict__ sin_cache, RopeDims d) {
    constexpr int VEC = kVec128<T>;
    constexpr int HALF = VEC / 2;
    const std::uint32_t pairs = d.rotary_dim / 2;
    for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < d.total_vectors;
         v += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const bool is_q = v < d.query_vectors;
        const std::size_t local = is_q ? v : v - d.query_vectors;
        const std::uint32_t heads = is_q ? d.query_heads : d.kv_heads;
        const T* in = is_q ? in_q : in_k;
        T* out = is_q ? out_q : out_k;
        const std::size_t elem = local * VEC;
        const std::uint32_t per_token = heads * d.head_dim;
        const std::size_t token = elem / per_token;
        const std::uint32_t dim = static_cast<std::uint32_t>(elem % per_token) % d.head_dim;
        const vec_t<T, VEC> raw = load_vec<T, VEC>(in + elem);
        if (dim < d.rotary_dim) {
            const std::uint32_t pos = d.position_offset + static_cast<std::uint32_t>(token % d.sequence);
            const std::size_t cache_index = static_cast<std::size_t>(pos) * pairs + dim / 2;
            const vec_t<float, HALF> c = vec_to_f32<T, HALF>(load_vec<T, HALF>(cos_cache + cache_index));
            const vec_t<float, HALF> s = vec_to_f32<T, HALF>(load_vec<T, HALF>(sin_cache + cache_index));
            const vec_t<float, VEC> x = vec_to_f32<T, VEC>(raw);
            vec_t<float, VEC> r;
#pragma unroll
            for (int p = 0; p < HALF; ++p) {
                float a, b;
                rotate<Inverse>(x[2 * p], x[2 * p + 1], c[p], s[p], a, b);
                r[2 * p] = a;
                r[2 * p + 1] = b;
            }
            store_vec<T, VEC>(out + elem, vec_from_f32<T, VEC>(r));
        } else if (out != in) {
            store_vec<T, VEC>(out + elem, raw);
        }
    }
}

// One work item per pair (inside rotary_dim) or per pair of tail elements.
template <typename T, bool Inverse>
__global__ __launch_bounds__(kThreads) void rope_pair_kernel(T* __restrict__ out_q, T* __restrict__ out_k,
                                                             const T* in_q, const T* in_k,
                                                             const T* __restrict__ cos_cache,
                                                             const T* __restrict__ sin_cache, RopeDims d) {
    const std::uint32_t pairs = d.rotary_dim / 2;
    for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < d.total_vectors;
         v += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const bool is_q = v < d.query_vectors;
        const std::size_t local = is_q ? v : v - d.query_vectors;
        const std::uint32_t heads = is_q ? d.query_heads : d.kv_heads;
        const T* in = is_q ? in_q : in_k;
        T* out = is_q ? out_q : out_k;
        const std::size_t elem = local * 2;
        const std::uint32_t per_token = heads * d.head_dim;
        const std::size_t token = elem / per_token;
        const std::uint32_t dim = static_cast<std::uint32_t>(elem % per_token) % d.head_dim;
        const float x = to_f32(in[elem]), y = to_f32(in[elem + 1]);
        if (dim < d.rotary_dim) {
            const std::uint32_t pos = d.position_offset + static_cast<std::uint32_t>(token % d.sequence);
            const std::size_t cache_index = static_cast<std::size_t>(pos) * pairs + dim / 2;
            float a, b;
            rotate<Inverse>(x, y, to_f32(cos_cache[cache_index]), to_f32(sin_cache[cache_index]), a, b);
            out[elem] = from_f32<T>(a);
            out[elem + 1] = from_f32<T>(b);
        } else if (out != in) {
            out[elem] = in[elem];
            out[elem + 1] = in[elem + 1];
        }
    }
}

bool rope_is_empty(std::size_t batch, std::size_t sequence, std::size_t query_heads, std::size_t kv_heads,
                   std::size_t head_dim) {
    return batch == 0 || sequence == 0 || query_heads == 0 || kv_heads == 0 || head_dim == 0;
}

int validate_rope(const char* name, const void* q, const void* k, const void* c, const void* s, std::size_t batch,
                  std::size_t sequence, std::size_t query_heads, std::size_t kv_heads, std::size_t head_dim,
                  std::size_t& rotary_dim, std::size_t position_offset, std::size_t cache_positions, int dtype) {
    const std::string n(name);
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, n + ": unsupported dtype");
    if (q == nullptr || k == nullptr || c == nullptr || s == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, n + ": null tensor");
    if (rotary_dim == 0) rotary_dim = head_dim;
    if (batch == 0 || sequence == 0 || query_heads == 0 || kv_heads == 0 || head_dim == 0)
        return fail(CGPTX_INVALID_ARGUMENT, n + ": empty shape");
    if ((head_dim & 1u) != 0 || rotary_dim > head_dim || (rotary_dim & 1u) != 0)
        return fail(CGPTX_INVALID_ARGUMENT,
                    n + ": head_dim and rotary_dim must be even, with rotary_dim in [2, head_dim]");
    if (position_offset > std::numeric_limits<std::size_t>::max() - sequence ||
        cache_positions < position_offset + sequence)
        return fail(CGPTX_INVALID_ARGUMENT, n + ": cache does not cover the requested rotary positions");
    constexpr std::size_t u32max = std::numeric_limits<std::uint32_t>::max();
    if (sequence > u32max || query_heads > u32max || kv_heads > u32max || head_dim > u32max ||
        position_offset + sequence > u32max || query_heads * head_dim > u32max || kv_heads * head_dim > u32max)
        return fail(CGPTX_OVERFLOW, n + ": dimension exceeds uint32_t range");
    return CGPTX_OK;
}

template <bool Inverse>
int launch_rope(void* out_q, void* out_k, const void* in_q, const void* in_k, const void* cos_cache,
                const void* sin_cache, std::size_t batch, std::size_t sequence, std::size_t query_heads,
                std::size_t kv_heads, std::size_t head_dim, std::size_t rotary_dim, std::size_t position_offset,
                int dtype, hipStream_t stream) {
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        constexpr std::size_t VEC = kVec128<T>;
        const std::size_t q_elems = batch * sequence * query_heads * head_dim;
        const std::size_t k_elems = batch * sequence * kv_heads * head_dim;
        RopeDims d{static_cast<std::uint32_t>(sequence),   static_cast<std::uint32_t>(query_heads),
                   static_cast<std::uint32_t>(kv_heads),   static_cast<std::uint32_t>(head_dim),
                   static_cast<std::uint32_t>(rotary_dim), static_cast<std::uint32_t>(position_offset),
                   0,                                      0};
        const bool vector_ok = head_dim % VEC == 0 && rotary_dim % VEC == 0 && is_aligned16(out_q) &&
                               is_aligned16(out_k) && is_aligned16(in_q) && is_aligned16(in_k) &&
                               (reinterpret_cast<std::uintptr_t>(cos_cache) % (VEC / 2 * sizeof(T))) == 0 &&
                               (reinterpret_cast<std::uintptr_t>(sin_cache) % (VEC / 2 * sizeof(T))) == 0;
        if (vector_ok) {
            d.query_vectors = q_elems / VEC;
            d.total_vectors = d.query_vectors + k_elems / VEC;
            hipLaunchKernelGGL((rope_vec_kernel<T, Inverse>), dim3(grid_for(d.total_vectors)), dim3(kThreads), 0,
                               stream, static_cast<T*>(out_q), static_cast<T*>(out_k), static_cast<const T*>(in_q),
                               static_cast<const T*>(in_k), static_cast<const T*>(cos_cache),
                               static_cast<const T*>(sin_cache), d);
        } else {
            d.query_vectors = q_elems / 2;
            d.total_vectors = d.query_vectors + k_elems / 2;
            hipLaunchKernelGGL((rope_pair_kernel<T, Inverse>), dim3(grid_for(d.total_vectors)), dim3(kThreads), 0,
                               stream, static_cast<T*>(out_q), static_cast<T*>(out_k), static_cast<const T*>(in_q),
                               static_cast<const T*>(in_k), static_cast<const T*>(cos_cache),
                               static_cast<const T*>(sin_cache), d);
        }
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

// --------------------------------------------------------------------- SwiGLU
__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

// Packed: row-major [rows, 2*hidden] with gate in the first half of each row.
// Separate layout is the special case handled by passing distinct pointers.
// A workgroup takes tiles of kSwigluUnroll x 256 consecutive vectors: a thread requests its kSwigluUnroll
// vectors of all three inputs (and of the old gradients when accumulating) before it computes anything, so that
// twelve 128-bit loads per lane are in flight, and the position inside a packed row comes from 32-bit
// arithmetic (a shift when a row holds a power-of-two number of vectors).
constexpr int kSwigluUnroll = 4;
template <typename T, bool AccGate, bool AccUp>
__global__ __launch_bounds__(kThreads) void swiglu_backward_vec_kernel(
    T* grad_gate, T* grad_up, const T* __restrict__ grad_output, const T* __restrict__ gate,
    const T* __restrict__ up, std::size_t vectors, unsigned int row_vectors, int row_shift,
    std::size_t packed_row_stride) {
    // packed_row_stride == 0: flat separate tensors. Otherwise gate/up/grad_* are
    // views into [rows, 2*hidden] and index = row * stride + col. row_shift >= 0: row_vectors == 1 << row_shift.
    constexpr int VEC = kVec128<T>;
    constexpr std::size_t kTile = static_cast<std::size_t>(kThreads) * kSwigluUnroll;
    for (std::size_t base = static_cast<std::size_t>(blockIdx.x) * kTile; base < vectors;
         base += static_cast<std::size_t>(gridDim.x) * kTile) {
        vec_t<T, VEC> dy_raw[kSwigluUnroll], g_raw[kSwigluUnroll], u_raw[kSwigluUnroll], og_raw[kSwigluUnroll],
            ou_raw[kSwigluUnroll];
        std::size_t index[kSwigluUnroll];
        bool live[kSwigluUnroll];
#pragma unroll
        for (int k = 0; k < kSwigluUnroll; ++k) {
            const std::size_t v = base + static_cast<std::size_t>(k) * kThreads + threadIdx.x;
            live[k] = v < vectors;
            index[k] = v * VEC;
            if (packed_row_stride != 0) {
                std::size_t row;
                if (row_shift >= 0) row = v >> row_shift;
                else if (vectors <= 0xFFFFFFFFull) row = static_cast<unsigned int>(v) / row_vectors;
                else row = v / row_vectors;
                index[k] = row * packed_row_stride + (v - row * row_vectors) * VEC;
            }
            if (live[k]) {
                dy_raw[k] = load_vec<T, VEC>(grad_output + v * VEC);
                g_raw[k] = load_vec<T, VEC>(gate + index[k]);
                u_raw[k] = load_vec<T, VEC>(up + index[k]);
                if constexpr (AccGate) og_raw[k] = load_vec<T, VEC>(grad_gate + index[k]);
                if constexpr (AccUp) ou_raw[k] = load_vec<T, VEC>(grad_up + index[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < kSwigluUnroll; ++k) {
            if (!live[k]) continue;
            const vec_t<float, VEC> dy = vec_to_f32<T, VEC>(dy_raw[k]);
            const vec_t<float, VEC> g = vec_to_f32<T, VEC>(g_raw[k]);
            const vec_t<float, VEC> u = vec_to_f32<T, VEC>(u_raw[k]);
            vec_t<float, VEC> dg, du;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float s = sigmoid_f32(g[e]);
                dg[e] = dy[e] * u[e] * (s * (1.0f + g[e] * (1.0f - s)));
                du[e] = dy[e] * (g[e] * s);
            }
            if constexpr (AccGate) dg += vec_to_f32<T, VEC>(og_raw[k]);
            if constexpr (AccUp) du += vec_to_f32<T, VEC>(ou_raw[k]);
            store_vec<T, VEC>(grad_gate + index[k], vec_from_f32<T, VEC>(dg));
            store_vec<T, VEC>(grad_up + index[k], vec_from_f32<T, VEC>(du));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_backward_scalar_kernel(
    T* grad_gate, T* grad_up, const T* __restrict__ grad_output, const T* __restrict__ gate,
    const T* __restrict__ up, std::size_t count, std::size_t row_elems, std::size_t packed_row_stride, bool acc_gate,
    bool acc_up) {
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads) {
        std::size_t index = i;
        if (packed_row_stride != 0) {
            const std::size_t row = i / row_elems;
            index = row * packed_row_stride + (i - row * row_elems);
        }
        const float dy = to_f32(grad_output[i]), g = to_f32(gate[index]), u = to_f32(up[index]);
        const float s = sigmoid_f32(g);
        float dg = dy * u * (s * (1.0f + g * (1.0f - s)));
        float du = dy * (g * s);
        if (acc_gate) dg += to_f32(grad_gate[index]);
        if (acc_up) du += to_f32(grad_up[index]);
        grad_gate[index] = from_f32<T>(dg);
        grad_up[index] = from_f32<T>(du);
    }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_forward_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                                                 const T* __restrict__ up, std::size_t count,
                                                                 bool vector_ok) {
    constexpr int VEC = kVec128<T>;
    const std::size_t vectors = vector_ok ? count / VEC : 0;
    for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < vectors;
         v += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const vec_t<float, VEC> g = vec_to_f32<T, VEC>(load_vec<T, VEC>(gate + v * VEC));
        const vec_t<float, VEC> u = vec_to_f32<T, VEC>(load_vec<T, VEC>(up + v * VEC));
        vec_t<float, VEC> r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) r[e] = g[e] * sigmoid_f32(g[e]) * u[e];
        store_vec<T, VEC>(out + v * VEC, vec_from_f32<T, VEC>(r));
    }
    for (std::size_t i = vectors * VEC + static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const float g = to_f32(gate[i]);
        out[i] = from_f32<T>(g * sigmoid_f32(g) * to_f32(up[i]));
    }
}

// Packed input [rows, 2*hidden] = [gate | up] (src/ops/swiglu.cu:152-170): out[r, c] =
// silu(gate_up[r, c]) * gate_up[r, hidden + c].
template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_forward_packed_kernel(T* __restrict__ out,
                                                                        const T* __restrict__ gate_up,
                                                                        std::size_t rows, std::size_t hidden,
                                                                        bool vector_ok) {
    constexpr int VEC = kVec128<T>;
    const std::size_t count = rows * hidden;
    if (vector_ok) {
        const std::size_t row_vectors = hidden / VEC;
        const std::size_t vectors = rows * row_vectors;
        for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < vectors;
             v += static_cast<std::size_t>(gridDim.x) * kThreads) {
            const std::size_t row = v / row_vectors, col = (v - row * row_vectors) * VEC;
            const T* in = gate_up + row * 2 * hidden + col;
            const vec_t<float, VEC> g = vec_to_f32<T, VEC>(load_vec<T, VEC>(in));
            const vec_t<float, VEC> u = vec_to_f32<T, VEC>(load_vec<T, VEC>(in + hidden));
            vec_t<float, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r[e] = g[e] * sigmoid_f32(g[e]) * u[e];
            store_vec<T, VEC>(out + row * hidden + col, vec_from_f32<T, VEC>(r));
        }
        return;
    }
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const std::size_t row = i / hidden, col = i - row * hidden;
        const float g = to_f32(gate_up[row * 2 * hidden + col]);
        out[i] = from_f32<T>(g * sigmoid_f32(g) * to_f32(gate_up[row * 2 * hidden + hidden + col]));
    }
}

template <typename T>
int launch_swiglu_backward(T* grad_gate, T* grad_up, const T* grad_output, const T* gate, const T* up,
                           std::size_t count, std::size_t row_elems, std::size_t packed_row_stride, bool acc_gate,
                           bool acc_up, hipStream_t stream) {
    constexpr std::size_t VEC = kVec128<T>;
    const bool vector_ok = count % VEC == 0 && row_elems % VEC == 0 && packed_row_stride % VEC == 0 &&
                           is_aligned16(grad_gate) && is_aligned16(grad_up) && is_aligned16(grad_output) &&
                           is_aligned16(gate) && is_aligned16(up);
    if (!vector_ok) {
        hipLaunchKernelGGL((swiglu_backward_scalar_kernel<T>), dim3(grid_for(count)), dim3(kThreads), 0, stream,
                           grad_gate, grad_up, grad_output, gate, up, count, row_elems, packed_row_stride, acc_gate,
                           acc_up);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    }
    const std::size_t vectors = count / VEC;
    if (packed_row_stride != 0 && row_elems / VEC > 0xFFFFFFFFull)
        return fail(CGPTX_OVERFLOW, "swiglu_backward: row length exceeds uint32_t range");
    const auto row_vectors = packed_row_stride != 0 ? static_cast<unsigned int>(row_elems / VEC) : 0u;
    int row_shift = -1;
    if (row_vectors != 0 && (row_vectors & (row_vectors - 1)) == 0) row_shift = __builtin_ctz(row_vectors);
    // One tile per workgroup and pass; the grid is capped like the other streaming kernels'.
    const dim3 grid(grid_for((vectors + kSwigluUnroll - 1) / kSwigluUnroll)), block(kThreads);
#define CGPTX_SWIGLU_CASE(G, U)                                                                               \
    if (acc_gate == G && acc_up == U)                                                                         \
        hipLaunchKernelGGL((swiglu_backward_vec_kernel<T, G, U>), grid, block, 0, stream, grad_gate, grad_up, \
                           grad_output, gate, up, vectors, row_vectors, row_shift, packed_row_stride);
    CGPTX_SWIGLU_CASE(false, false)
    CGPTX_SWIGLU_CASE(true, false)
    CGPTX_SWIGLU_CASE(false, true)
    CGPTX_SWIGLU_CASE(true, true)
#undef CGPTX_SWIGLU_CASE
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

// ------------------------------------------------------------------------ add
template <typename T>
__global__ __launch_bounds__(kThreads) void add_kernel(T* out, const T* a, const T* b, std::size_t count,
                                                      bool vector_ok) {
    constexpr int VEC = kVec128<T>;
    const std::size_t vectors = vector_ok ? count / VEC : 0;
    for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < vectors;
         v += static_cast<std::size_t>(gridDim.x) * kThreads) {
        const vec_t<float, VEC> x = vec_to_f32<T, VEC>(load_vec<T, VEC>(a + v * VEC));
        const vec_t<float, VEC> y = vec_to_f32<T, VEC>(load_vec<T, VEC>(b + v * VEC));
        store_vec<T, VEC>(out + v * VEC, vec_from_f32<T, VEC>(x + y));
    }
    for (std::size_t i = vectors * VEC + static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads) {
        out[i] = from_f32<T>(to_f32(a[i]) + to_f32(b[i]));
    }
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_rope_backward(void* grad_query, void* grad_key, const void* grad_rotated_query,
                                   const void* grad_rotated_key, const void* cos_cache, const void* sin_cache,
                                   size_t batch, size_t sequence, size_t query_heads, size_t kv_heads,
                                   size_t head_dim, size_t rotary_dim, size_t position_offset, size_t cache_positions,
                                   int dtype, cgptx_stream stream) {
    using namespace cgptx;
    // Tensors without elements: nothing to do, as in the reference (src/ops/backward/rope_backward.cu:243-245, 326-328).
    if (valid_dtype(dtype) && rope_is_empty(batch, sequence, query_heads, kv_heads, head_dim)) return CGPTX_OK;
    if (grad_rotated_query == nullptr || grad_rotated_key == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "rope_backward: null tensor");
    if (int s = validate_rope("rope_backward", grad_query, grad_key, cos_cache, sin_cache, batch, sequence,
                              query_heads, kv_heads, head_dim, rotary_dim, position_offset, cache_positions, dtype))
        return s;
    return launch_rope<true>(grad_query, grad_key, grad_rotated_query, grad_rotated_key, cos_cache, sin_cache, batch,
                             sequence, query_heads, kv_heads, head_dim, rotary_dim, position_offset, dtype,
                             static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_rope_forward(void* query, void* key, const void* cos_cache, const void* sin_cache, size_t batch,
                                  size_t sequence, size_t query_heads, size_t kv_heads, size_t head_dim,
                                  size_t rotary_dim, size_t position_offset, size_t cache_positions, int dtype,
                                  cgptx_stream stream) {
    using namespace cgptx;
    // Tensors without elements: nothing to do, as in the reference (src/ops/rope.cu:606-608).
    if (valid_dtype(dtype) && rope_is_empty(batch, sequence, query_heads, kv_heads, head_dim)) return CGPTX_OK;
    if (int s = validate_rope("rope_forward", query, key, cos_cache, sin_cache, batch, sequence, query_heads,
                              kv_heads, head_dim, rotary_dim, position_offset, cache_positions, dtype))
        return s;
    return launch_rope<false>(query, key, query, key, cos_cache, sin_cache, batch, sequence, query_heads, kv_heads,
                              head_dim, rotary_dim, position_offset, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_swiglu_backward(void* grad_gate, void* grad_up, const void* grad_output, const void* gate,
                                     const void* up, size_t count, int accumulate_gate, int accumulate_up, int dtype,
                                     cgptx_stream stream) {
    using namespace cgptx;
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, "swiglu_backward: unsupported dtype");
    if (count == 0) return CGPTX_OK;  // nothing to do, as in the reference (src/ops/backward/swiglu_backward.cu:772-774)
    if (grad_gate == nullptr || grad_up == nullptr || grad_output == nullptr || gate == nullptr || up == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "swiglu_backward: null tensor");
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        return launch_swiglu_backward<T>(static_cast<T*>(grad_gate), static_cast<T*>(grad_up),
                                         static_cast<const T*>(grad_output), static_cast<const T*>(gate),
                                         static_cast<const T*>(up), count, count, 0, accumulate_gate != 0,
                                         accumulate_up != 0, static_cast<hipStream_t>(stream));
    });
}

extern "C" int cgptx_swiglu_backward_packed(void* grad_gate_up, const void* grad_output, const void* gate_up,
                                            size_t rows, size_t hidden, int accumulate_gate_up, int dtype,
                                            cgptx_stream stream) {
    using namespace cgptx;
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, "swiglu_backward: unsupported dtype");
    if (rows == 0 || hidden == 0) return CGPTX_OK;  // nothing to do (src/ops/backward/swiglu_backward.cu:839-841)
    if (grad_gate_up == nullptr || grad_output == nullptr || gate_up == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "swiglu_backward: null tensor");
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* out = static_cast<T*>(grad_gate_up);
        auto* in = static_cast<const T*>(gate_up);
        const bool acc = accumulate_gate_up != 0;
        return launch_swiglu_backward<T>(out, out + hidden, static_cast<const T*>(grad_output), in, in + hidden,
                                         rows * hidden, hidden, 2 * hidden, acc, acc,
                                         static_cast<hipStream_t>(stream));
    });
}

extern "C" int cgptx_swiglu_forward(void* output, const void* gate, const void* up, size_t count, int dtype,
                                    cgptx_stream stream) {
    using namespace cgptx;
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, "swiglu_forward: unsupported dtype");
    if (count == 0) return CGPTX_OK;  // nothing to do, as in the reference (src/ops/swiglu.cu:530-532)
    if (output == nullptr || gate == nullptr || up == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "swiglu_forward: null tensor");
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const bool vector_ok = is_aligned16(output) && is_aligned16(gate) && is_aligned16(up);
        hipLaunchKernelGGL((swiglu_forward_kernel<T>), dim3(grid_for(count / kVec128<T> + 1)), dim3(kThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T*>(output), static_cast<const T*>(gate),
                           static_cast<const T*>(up), count, vector_ok);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

extern "C" int cgptx_swiglu_forward_packed(void* output, const void* gate_up, size_t rows, size_t hidden, int dtype,
                                           cgptx_stream stream) {
    using namespace cgptx;
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, "swiglu_forward: unsupported dtype");
    if (rows == 0 || hidden == 0) return CGPTX_OK;  // nothing to do (src/ops/swiglu.cu:581-583)
    if (output == nullptr || gate_up == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "swiglu_forward: null tensor");
    if (rows > std::numeric_limits<std::size_t>::max() / (2 * hidden))
        return fail(CGPTX_OVERFLOW, "swiglu_forward: element count overflows");
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const bool vector_ok = is_aligned16(output) && is_aligned16(gate_up) && hidden % kVec128<T> == 0;
        hipLaunchKernelGGL((swiglu_forward_packed_kernel<T>), dim3(grid_for(rows * hidden / kVec128<T> + 1)),
                           dim3(kThreads), 0, static_cast<hipStream_t>(stream), static_cast<T*>(output),
                           static_cast<const T*>(gate_up), rows, hidden, vector_ok);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

extern "C" int cgptx_add(void* output, const void* a, const void* b, size_t count, int dtype, cgptx_stream stream) {
    using namespace cgptx;
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, "add: unsupported dtype");
    if (output == nullptr || a == nullptr || b == nullptr || count == 0)
        return fail(CGPTX_INVALID_ARGUMENT, "add: null or empty tensor");
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const bool vector_ok = is_aligned16(output) && is_aligned16(a) && is_aligned16(b);
        hipLaunchKernelGGL((add_kernel<T>), dim3(grid_for(count / kVec128<T> + 1)), dim3(kThreads), 0,
                           static_cast<hipStream_t>(stream), static_cast<T*>(output), static_cast<const T*>(a),
                           static_cast<const T*>(b), count, vector_ok);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}
