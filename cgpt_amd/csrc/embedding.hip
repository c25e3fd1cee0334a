// Embedding gather (forward) and embedding-gradient scatter (backward) for gfx950.
//
// Backward semantics: include/ops/backward/embedding_backward.h:35-42. The
// reference scatters with storage-dtype atomics (src/ops/backward/embedding_backward.cu:68-92),
// so its rounding depends on arrival order. Here the tokens are grouped by id with a counting
// sort over the vocabulary (integer work: histogram, scan, fill — one launch), then one wavefront
// per vocabulary row adds that row's tokens in ascending token order with one rounding to the
// storage dtype per add — the arithmetic of the reference's CPU operator
// (src/ops/cpu/backward/embedding_backward_cpu.cpp:99-112). The result is deterministic and no
// float atomics are used. Lanes cover the hidden dimension with 128-bit accesses, so each token
// row is read once, fully coalesced; rows that no token names are zero-filled by the same launch
// when the gradient is not accumulated.
#include "common.hpp"

#include <cstring>
#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWave;

// ---- grouping: counting sort of the token positions by id -------------------------------------------
// Workgroup b owns the ids [b R, (b+1) R) and reads the whole id list twice: first it counts its ids in an
// LDS histogram and, on the side, the tokens with smaller ids (which is where its part of the output begins:
// no workgroup waits for another); after an exclusive scan of the histogram it hands every token of its range
// the next free slot of its id's segment. Slots are handed out with LDS integer atomics, so the order inside a
// segment is whatever order the lanes arrived in: the row kernel puts each segment into ascending order itself.
// offsets[id] .. offsets[id + 1] is id's segment of `order`; ids >= vocab belong to nobody and are skipped.
constexpr int kGroupThreads = 1024;
constexpr unsigned int kGroupMaxIds = 32768;  // LDS histogram entries of one workgroup (128 KiB)
constexpr int kGroupBatch = 8;                // 128-bit id loads a thread keeps in flight

// The id list is walked in batches of kGroupBatch x 4 ids per thread, all of a batch's loads requested before the
// first id is looked at (one dependent load per id would cost a memory round trip each). visit(id, t) sees every
// token once; the order within a workgroup does not matter to any caller.
template <typename Visit>
__device__ __forceinline__ void for_each_id(const std::uint32_t* __restrict__ ids, unsigned int count, bool aligned, Visit&& visit) {
    using u32x4 = vec_t<unsigned int, 4>;
    const unsigned int quads = aligned ? count / 4 : 0;
    const auto* wide = reinterpret_cast<const u32x4*>(ids);
    for (unsigned int base = 0; base < quads; base += kGroupBatch * kGroupThreads) {
        u32x4 held[kGroupBatch];
#pragma unroll
        for (int k = 0; k < kGroupBatch; ++k) {
            const unsigned int q = base + k * kGroupThreads + threadIdx.x;
            if (q < quads) held[k] = wide[q];
        }
#pragma unroll
        for (int k = 0; k < kGroupBatch; ++k) {
            const unsigned int q = base + k * kGroupThreads + threadIdx.x;
            if (q < quads) {
#pragma unroll
                for (int e = 0; e < 4; ++e) visit(held[k][e], 4 * q + e);
            }
        }
    }
    for (unsigned int t = 4 * quads + threadIdx.x; t < count; t += kGroupThreads) visit(ids[t], t);
}

__global__ __launch_bounds__(kGroupThreads) void embedding_group_kernel(unsigned int* __restrict__ offsets,
                                                                       unsigned int* __restrict__ order,
                                                                       const std::uint32_t* __restrict__ ids,
                                                                       unsigned int count, unsigned int vocab,
                                                                       unsigned int ids_per_group, bool aligned) {
    extern __shared__ unsigned int bins[];  // [ids_per_group]
    __shared__ unsigned int wave_totals[kGroupThreads / kWave];
    __shared__ unsigned int smaller_total;
    const unsigned int lo = blockIdx.x * ids_per_group;
    const unsigned int width = min(ids_per_group, vocab - lo);
    const unsigned int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
    for (unsigned int i = tid; i < width; i += kGroupThreads) bins[i] = 0;
    if (tid == 0) smaller_total = 0;
    __syncthreads();
    unsigned int smaller = 0;
    for_each_id(ids, count, aligned, [&](unsigned int id, unsigned int) {
        if (id < lo) ++smaller;
        else if (id - lo < width) atomicAdd(&bins[id - lo], 1u);
    });
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) smaller += __shfl_xor(smaller, offset, kWave);
    if (lane == 0 && smaller != 0) atomicAdd(&smaller_total, smaller);
    __syncthreads();
    // Exclusive scan of bins[0, width) in place, starting at the number of tokens with smaller ids: thread i
    // owns the contiguous piece [i per, (i + 1) per).
    const unsigned int per = (width + kGroupThreads - 1) / kGroupThreads;
    const unsigned int first = min(tid * per, width), last = min(first + per, width);
    unsigned int mine = 0;
    for (unsigned int i = first; i < last; ++i) mine += bins[i];
    unsigned int inclusive = mine;
#pragma unroll
    for (int offset = 1; offset < kWave; offset <<= 1) {
        const unsigned int other = __shfl_up(inclusive, offset, kWave);
        if (lane >= static_cast<unsigned int>(offset)) inclusive += other;
    }
    if (lane == kWave - 1) wave_totals[wave] = inclusive;
    __syncthreads();
    unsigned int before = smaller_total;
    for (unsigned int w = 0; w < wave; ++w) before += wave_totals[w];
    unsigned int running = before + inclusive - mine;
    for (unsigned int i = first; i < last; ++i) {
        const unsigned int n = bins[i];
        bins[i] = running;
        offsets[lo + i] = running;
        running += n;
    }
    if (lo + width == vocab && tid == kGroupThreads - 1) offsets[vocab] = running;  // the piece that ends the last range
    __syncthreads();
    for_each_id(ids, count, aligned, [&](unsigned int id, unsigned int t) {
        if (id >= lo && id - lo < width) order[atomicAdd(&bins[id - lo], 1u)] = t;
    });
}

// ---- rows: one wavefront per vocabulary row -------------------------------------------------------
// Adds, into row `id` of the table, the rows of grad_output of the tokens with that id, in ascending token
// order with one rounding to the storage dtype per add. Segments of up to 64 tokens are ordered in registers
// (lane i holds the token of rank i); longer ones are walked by scanning the id list itself, 64 tokens per
// step, which yields them in ascending order by construction. Rows without tokens are zero-filled unless the
// gradient is accumulated.
template <typename T, bool Vector>
__global__ __launch_bounds__(kThreads) void embedding_rows_kernel(T* __restrict__ grad_weight,
                                                                 const T* __restrict__ grad_output,
                                                                 const std::uint32_t* __restrict__ ids,
                                                                 const unsigned int* __restrict__ offsets,
                                                                 const unsigned int* __restrict__ order,
                                                                 unsigned int count, unsigned int vocab,
                                                                 unsigned int hidden, bool accumulate) {
    constexpr int VEC = Vector ? kVec128<T> : 1;
    using vec_f = vec_t<float, VEC>;
    const unsigned int lane = threadIdx.x & (kWave - 1);
    const unsigned int id = blockIdx.x * kWavesPerBlock + threadIdx.x / kWave;
    if (id >= vocab) return;
    const unsigned int begin = offsets[id], tokens = offsets[id + 1] - begin;
    T* row = grad_weight + static_cast<std::size_t>(id) * hidden;
    if (tokens == 0) {
        if (!accumulate)
            for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC) store_vec<T, VEC>(row + col, vec_t<T, VEC>(0));
        return;
    }
    auto add_row = [&](vec_f acc, unsigned int token, unsigned int col) {
        const vec_f dy = vec_to_f32<T, VEC>(load_vec<T, VEC>(grad_output + static_cast<std::size_t>(token) * hidden + col));
        return vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(acc + dy));  // one rounding to the storage dtype per add
    };
    if (tokens <= kWave) {
        const unsigned int mine = lane < tokens ? order[begin + lane] : 0xFFFFFFFFu;
        // rank = number of tokens of the segment below mine; sorted = the token of rank `lane`.
        unsigned int rank = 0;
        for (unsigned int j = 0; j < tokens; ++j)
            rank += static_cast<unsigned int>(__builtin_amdgcn_readlane(static_cast<int>(mine), static_cast<int>(j))) < mine ? 1u : 0u;
        const unsigned int sorted = static_cast<unsigned int>(
            __builtin_amdgcn_ds_permute(static_cast<int>(rank << 2), static_cast<int>(mine)));  // lane `rank` receives mine
        for (unsigned int col = lane * VEC; col < hidden; col += kWave * VEC) {
            vec_f acc = accumulate ? vec_to_f32<T, VEC>(load_vec<T, VEC>(row + col)) : vec_f(0.0f);
            // Four token rows are requested at a time; the additions keep their order.
            for (unsigned int j0 = 0; j0 < tokens; j0 += 4) {
                vec_t<T, VEC> dy[4];
#pragma unroll
                for (unsigned int u = 0; u < 4; ++u)
                    if (j0 + u < tokens) {
                        const auto token = static_cast<unsigned int>(
                            __builtin_amdgcn_readlane(static_cast<int>(sorted), static_cast<int>(j0 + u)));
                        dy[u] = load_vec<T, VEC>(grad_output + static_cast<std::size_t>(token) * hidden + col);
                    }
#pragma unroll
                for (unsigned int u = 0; u < 4; ++u)
                    if (j0 + u < tokens)  // one rounding to the storage dtype per add
                        acc = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(acc + vec_to_f32<T, VEC>(dy[u])));
            }
            store_vec<T, VEC>(row + col, vec_from_f32<T, VEC>(acc));
        }
        return;
    }
    for (unsigned int col0 = 0; col0 < hidden; col0 += kWave * VEC) {
        const unsigned int col = col0 + lane * VEC;
        const bool live = col < hidden;
        vec_f acc = (accumulate && live) ? vec_to_f32<T, VEC>(load_vec<T, VEC>(row + col)) : vec_f(0.0f);
        for (unsigned int first = 0; first < count; first += kWave) {
            const unsigned int t = first + lane;
            unsigned long long matches = __ballot(t < count && ids[t] == id);  // every lane takes part
            while (matches != 0) {
                const unsigned int token = first + static_cast<unsigned int>(__builtin_ctzll(matches));
                matches &= matches - 1;
                if (live) acc = add_row(acc, token, col);
            }
        }
        if (live) store_vec<T, VEC>(row + col, vec_from_f32<T, VEC>(acc));
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

    // Scratch: offsets[vocab + 1] | order[token_count].
    const std::size_t offsets_bytes = ((vocab + 1) * sizeof(unsigned int) + 255) & ~std::size_t{255};
    void* mem = nullptr;
    if (int s = scratch(stream, offsets_bytes + token_count * sizeof(unsigned int), &mem)) return s;
    auto* offsets = static_cast<unsigned int*>(mem);
    auto* order = reinterpret_cast<unsigned int*>(static_cast<char*>(mem) + offsets_bytes);
    // Ranges of at least 1024 ids, at most one workgroup per compute unit, each histogram within the LDS.
    unsigned int ids_per_group = 1024;
    const unsigned int units = static_cast<unsigned int>(compute_units());
    while (ids_per_group < kGroupMaxIds && (v + ids_per_group - 1) / ids_per_group > units) ids_per_group *= 2;
    const unsigned int groups = (v + ids_per_group - 1) / ids_per_group;
    const std::size_t group_lds = ids_per_group * sizeof(unsigned int);
    {
        static bool configured = false;
        if (!configured) {
            CGPTX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(embedding_group_kernel),
                                          hipFuncAttributeMaxDynamicSharedMemorySize,
                                          static_cast<int>(kGroupMaxIds * sizeof(unsigned int))));
            configured = true;
        }
    }
    hipLaunchKernelGGL(embedding_group_kernel, dim3(groups), dim3(kGroupThreads), group_lds, stream, offsets, order, token_ids,
                       count, v, ids_per_group, is_aligned16(token_ids));
    CGPTX_LAUNCH_CHECK();
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* dw = static_cast<T*>(grad_weight);
        auto* dy = static_cast<const T*>(grad_output);
        const bool vector_ok = hidden % kVec128<T> == 0 && is_aligned16(dw) && is_aligned16(dy);
        const dim3 grid((v + kWavesPerBlock - 1) / kWavesPerBlock);
        const auto h = static_cast<unsigned int>(hidden);
        if (vector_ok) {
            hipLaunchKernelGGL((embedding_rows_kernel<T, true>), grid, dim3(kThreads), 0, stream, dw, dy, token_ids, offsets,
                               order, count, v, h, accumulate_weight != 0);
        } else {
            hipLaunchKernelGGL((embedding_rows_kernel<T, false>), grid, dim3(kThreads), 0, stream, dw, dy, token_ids, offsets,
                               order, count, v, h, accumulate_weight != 0);
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
