// Embedding gather (forward) and embedding-gradient scatter (backward) for gfx950.
//
// Backward semantics: include/ops/backward/embedding_backward.h:35-42. The
// reference scatters with storage-dtype atomics (src/ops/backward/embedding_backward.cu:68-92),
// so its rounding depends on arrival order. Here the token list is stably sorted
// by id (integer work, order-independent), then one wavefront per distinct id
// walks that id's tokens in ascending token order and adds their rows with one
// rounding to the storage dtype per add — the arithmetic of the reference's CPU
// operator (src/ops/cpu/backward/embedding_backward_cpu.cpp:99-112). The result is
// deterministic and no float atomics are used. Lanes cover the hidden dimension
// with 128-bit accesses, so each token row is read once, fully coalesced.
#include "common.hpp"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWave;

__global__ __launch_bounds__(kThreads) void embedding_keys_kernel(unsigned int* __restrict__ keys,
                                                                 unsigned int* __restrict__ values,
                                                                 const std::uint32_t* __restrict__ ids,
                                                                 unsigned int count, unsigned int vocab) {
    const unsigned int t = blockIdx.x * kThreads + threadIdx.x;
    if (t >= count) return;
    const std::uint32_t id = ids[t];
    keys[t] = id < vocab ? id : vocab;  // out-of-range ids sort to the end and are skipped
    values[t] = t;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void fill_zero_kernel(T* __restrict__ out, std::size_t count, bool aligned) {
    constexpr int VEC = kVec128<T>;
    const std::size_t vectors = aligned ? count / VEC : 0;
    for (std::size_t v = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; v < vectors;
         v += static_cast<std::size_t>(gridDim.x) * kThreads)
        store_vec<T, VEC>(out + v * VEC, vec_t<T, VEC>(0));
    for (std::size_t i = vectors * VEC + static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads)
        out[i] = from_f32<T>(0.0f);
}

// One wavefront per sorted position; only segment heads do work.
template <typename T, bool Vector>
__global__ __launch_bounds__(kThreads) void embedding_segment_kernel(T* __restrict__ grad_weight,
                                                                    const T* __restrict__ grad_output,
                                                                    const unsigned int* __restrict__ keys,
                                                                    const unsigned int* __restrict__ tokens,
                                                                    unsigned int count, unsigned int vocab,
                                                                    unsigned int hidden, bool accumulate) {
    constexpr int VEC = Vector ? kVec128<T> : 1;
    const unsigned int lane = threadIdx.x & (kWave - 1);
    const unsigned int position = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (position >= count) return;
    const unsigned int key = keys[position];
    if (key >= vocab) return;
    if (position > 0 && keys[position - 1] == key) return;
    unsigned int end = position + 1;
    while (end < count && keys[end] == key) ++end;
    T* row = grad_weight + static_cast<std::size_t>(key) * hidden;
    for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC) {
        vec_t<float, VEC> acc;
        if (accumulate) {
            acc = vec_to_f32<T, VEC>(load_vec<T, VEC>(row + col));
        } else {
            acc = vec_t<float, VEC>(0.0f);
        }
        for (unsigned int j = position; j < end; ++j) {
            const T* src = grad_output + static_cast<std::size_t>(tokens[j]) * hidden + col;
            const vec_t<float, VEC> dy = vec_to_f32<T, VEC>(load_vec<T, VEC>(src));
            // one rounding to the storage dtype per add
            acc = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(acc + dy));
        }
        store_vec<T, VEC>(row + col, vec_from_f32<T, VEC>(acc));
    }
}

// Short token lists (up to kDirectTokens) skip the sort: one wavefront per token compares its id with all the
// others. The first occurrence of an id owns the row and adds the later occurrences in ascending token order —
// the segment kernel's arithmetic, in one launch instead of six. Lane c keeps the 64-bit match mask of tokens
// 64 c .. 64 c + 63.
constexpr unsigned int kDirectTokens = 4096;
template <typename T, bool Vector>
__global__ __launch_bounds__(kThreads) void embedding_direct_kernel(T* __restrict__ grad_weight,
                                                                   const T* __restrict__ grad_output,
                                                                   const std::uint32_t* __restrict__ ids,
                                                                   unsigned int count, unsigned int vocab,
                                                                   unsigned int hidden, bool accumulate) {
    constexpr int VEC = Vector ? kVec128<T> : 1;
    const unsigned int lane = threadIdx.x & (kWave - 1);
    const unsigned int token = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (token >= count) return;
    const std::uint32_t id = ids[token];
    if (id >= vocab) return;
    for (unsigned int first = 0; first < token; first += kWave) {
        const unsigned int j = first + lane;
        if (__ballot(j < token && ids[j] == id) != 0) return;  // an earlier token owns this row
    }
    const unsigned int chunks = (count + kWave - 1) / kWave, own_chunk = token / kWave;
    unsigned long long later = 0;
    for (unsigned int c = own_chunk; c < chunks; ++c) {
        const unsigned int j = c * kWave + lane;
        const unsigned long long mask = __ballot(j > token && j < count && ids[j] == id);
        if (lane == c) later = mask;
    }
    T* row = grad_weight + static_cast<std::size_t>(id) * hidden;
    for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC) {
        vec_t<float, VEC> acc;
        if (accumulate) {
            acc = vec_to_f32<T, VEC>(load_vec<T, VEC>(row + col));
        } else {
            acc = vec_t<float, VEC>(0.0f);
        }
        const vec_t<float, VEC> own = vec_to_f32<T, VEC>(load_vec<T, VEC>(grad_output + static_cast<std::size_t>(token) * hidden + col));
        acc = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(acc + own));  // one rounding to the storage dtype per add
        for (unsigned int c = own_chunk; c < chunks; ++c) {
            // v_readlane reads any lane, active or not (the lanes past the row's width are inactive here).
            const int holder = __builtin_amdgcn_readfirstlane(static_cast<int>(c));
            unsigned long long mask =
                static_cast<unsigned long long>(static_cast<unsigned int>(__builtin_amdgcn_readlane(static_cast<int>(later), holder))) |
                (static_cast<unsigned long long>(static_cast<unsigned int>(__builtin_amdgcn_readlane(static_cast<int>(later >> 32), holder))) << 32);
            while (mask != 0) {
                const unsigned int j = c * kWave + static_cast<unsigned int>(__builtin_ctzll(mask));
                mask &= mask - 1;
                const vec_t<float, VEC> dy = vec_to_f32<T, VEC>(load_vec<T, VEC>(grad_output + static_cast<std::size_t>(j) * hidden + col));
                acc = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(acc + dy));
            }
        }
        store_vec<T, VEC>(row + col, vec_from_f32<T, VEC>(acc));
    }
}

template <typename T, bool Vector>
__global__ __launch_bounds__(kThreads) void embedding_gather_kernel(T* __restrict__ out,
                                                                   const std::uint32_t* __restrict__ ids,
                                                                   const T* __restrict__ weight, unsigned int count,
                                                                   unsigned int vocab, unsigned int hidden) {
    constexpr int VEC = Vector ? kVec128<T> : 1;
    const unsigned int lane = threadIdx.x & (kWave - 1);
    const unsigned int token = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (token >= count) return;
    const std::uint32_t id = ids[token];
    T* dst = out + static_cast<std::size_t>(token) * hidden;
    if (id < vocab) {
        const T* src = weight + static_cast<std::size_t>(id) * hidden;
        for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC)
            store_vec<T, VEC>(dst + col, load_vec<T, VEC>(src + col));
    } else {
        for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC)
            store_vec<T, VEC>(dst + col, vec_t<T, VEC>(0));
    }
}

int bits_for(unsigned int max_value) {
    int bits = 1;
    while (bits < 32 && (max_value >> bits) != 0) ++bits;
    return bits;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_embedding_backward(void* grad_weight, const void* grad_output, const uint32_t* token_ids,
                                        size_t token_count, size_t vocab, size_t hidden, int bounds_check,
                                        int accumulate_weight, int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    (void)bounds_check;  // out-of-range ids are skipped either way
    const char* name = "embedding_backward";
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (grad_weight == nullptr || grad_output == nullptr || token_ids == nullptr || token_count == 0 || vocab == 0 ||
        hidden == 0)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": incompatible tensors or token count");
    constexpr std::size_t u32max = std::numeric_limits<std::uint32_t>::max();
    if (token_count >= u32max / 2 || vocab >= u32max || hidden > u32max)
        return fail(CGPTX_OVERFLOW, std::string(name) + ": dimension exceeds uint32_t range");
    auto stream = static_cast<hipStream_t>(stream_);
    const auto count = static_cast<unsigned int>(token_count);
    const auto v = static_cast<unsigned int>(vocab);
    const int end_bit = bits_for(v);

    const bool direct = token_count <= kDirectTokens;
    unsigned int* keys_out = nullptr;
    unsigned int* values_out = nullptr;
    if (!direct) {
        // Scratch: keys_in | keys_out | values_in | values_out | rocPRIM temporary storage.
        const std::size_t array_bytes = (token_count * sizeof(unsigned int) + 255) & ~std::size_t{255};
        std::size_t temp_bytes = 0;
        CGPTX_HIP(rocprim::radix_sort_pairs(nullptr, temp_bytes, static_cast<unsigned int*>(nullptr),
                                            static_cast<unsigned int*>(nullptr), static_cast<unsigned int*>(nullptr),
                                            static_cast<unsigned int*>(nullptr), token_count, 0, end_bit, stream));
        void* mem = nullptr;
        if (int s = scratch(stream, 4 * array_bytes + temp_bytes + 256, &mem)) return s;
        auto* base = static_cast<char*>(mem);
        auto* keys_in = reinterpret_cast<unsigned int*>(base);
        keys_out = reinterpret_cast<unsigned int*>(base + array_bytes);
        auto* values_in = reinterpret_cast<unsigned int*>(base + 2 * array_bytes);
        values_out = reinterpret_cast<unsigned int*>(base + 3 * array_bytes);
        void* temp = base + 4 * array_bytes;

        hipLaunchKernelGGL(embedding_keys_kernel, dim3((count + kThreads - 1) / kThreads), dim3(kThreads), 0, stream,
                           keys_in, values_in, token_ids, count, v);
        CGPTX_LAUNCH_CHECK();
        CGPTX_HIP(rocprim::radix_sort_pairs(temp, temp_bytes, keys_in, keys_out, values_in, values_out, token_count, 0,
                                            end_bit, stream));
    }
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* dw = static_cast<T*>(grad_weight);
        auto* dy = static_cast<const T*>(grad_output);
        const bool vector_ok = hidden % kVec128<T> == 0 && is_aligned16(dw) && is_aligned16(dy);
        if (!accumulate_weight) {
            const std::size_t total = vocab * hidden;
            const std::size_t blocks = (total / kVec128<T> + kThreads) / kThreads;
            const std::size_t cap = static_cast<std::size_t>(compute_units()) * 16;
            hipLaunchKernelGGL((fill_zero_kernel<T>), dim3(static_cast<unsigned int>(blocks < cap ? blocks : cap)),
                               dim3(kThreads), 0, stream, dw, total, is_aligned16(dw));
            CGPTX_LAUNCH_CHECK();
        }
        const dim3 grid((count + kWavesPerBlock - 1) / kWavesPerBlock);
        const auto h = static_cast<unsigned int>(hidden);
        if (direct) {
            if (vector_ok) {
                hipLaunchKernelGGL((embedding_direct_kernel<T, true>), grid, dim3(kThreads), 0, stream, dw, dy, token_ids,
                                   count, v, h, accumulate_weight != 0);
            } else {
                hipLaunchKernelGGL((embedding_direct_kernel<T, false>), grid, dim3(kThreads), 0, stream, dw, dy, token_ids,
                                   count, v, h, accumulate_weight != 0);
            }
        } else if (vector_ok) {
            hipLaunchKernelGGL((embedding_segment_kernel<T, true>), grid, dim3(kThreads), 0, stream, dw, dy, keys_out,
                               values_out, count, v, h, accumulate_weight != 0);
        } else {
            hipLaunchKernelGGL((embedding_segment_kernel<T, false>), grid, dim3(kThreads), 0, stream, dw, dy,
                               keys_out, values_out, count, v, h, accumulate_weight != 0);
        }
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

extern "C" int cgptx_embedding_forward(void* output, const uint32_t* token_ids, size_t token_count,
                                       const void* weight, size_t vocab, size_t hidden, int dtype,
                                       cgptx_stream stream_) {
    using namespace cgptx;
    const char* name = "embedding_forward";
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (output == nullptr || weight == nullptr || token_ids == nullptr || token_count == 0 || vocab == 0 || hidden == 0)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": incompatible tensors or token count");
    constexpr std::size_t u32max = std::numeric_limits<std::uint32_t>::max();
    if (token_count >= u32max || vocab >= u32max || hidden > u32max)
        return fail(CGPTX_OVERFLOW, std::string(name) + ": dimension exceeds uint32_t range");
    auto stream = static_cast<hipStream_t>(stream_);
    const auto count = static_cast<unsigned int>(token_count);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* out = static_cast<T*>(output);
        auto* w = static_cast<const T*>(weight);
        const bool vector_ok = hidden % kVec128<T> == 0 && is_aligned16(out) && is_aligned16(w);
        const dim3 grid((count + kWavesPerBlock - 1) / kWavesPerBlock);
        if (vector_ok) {
            hipLaunchKernelGGL((embedding_gather_kernel<T, true>), grid, dim3(kThreads), 0, stream, out, token_ids, w,
                               count, static_cast<unsigned int>(vocab), static_cast<unsigned int>(hidden));
        } else {
            hipLaunchKernelGGL((embedding_gather_kernel<T, false>), grid, dim3(kThreads), 0, stream, out, token_ids,
                               w, count, static_cast<unsigned int>(vocab), static_cast<unsigned int>(hidden));
        }
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}
