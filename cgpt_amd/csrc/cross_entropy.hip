// Dense softmax cross-entropy (loss + logits gradient) for gfx950.
//
// Semantics: include/ops/cross_entropy.h:25-42; arithmetic of
// src/ops/cpu/backward/cross_entropy_backward_cpu.cpp:122-148:
//   loss = mean_r [ y_r < V ] (log Σ_j e^{z_rj} − z_{r,y_r}),
//   grad_rj = (softmax(z_r)_j − [j = y_r]) · scale / rows   (stored in the logits dtype).
//
// One block per row. Rows of up to 8192 128-bit vectors (65536 16-bit logits) are loaded once
// into registers, reduced to (max, Σexp) and turned into the gradient from the registers: one
// read and one write of the logits. Longer or unaligned rows stream: pass 1 keeps an online
// (max, Σexp) pair per thread, pass 2 re-reads the row through the caches. Per-row losses go to
// scratch and one block adds them in a fixed order, where the reference uses a float atomicAdd
// (src/ops/cross_entropy.cu:134-245).
#include "cross_entropy.hpp"

#include <cmath>
#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;

struct MaxSum {
    float m, s;
};

__device__ __forceinline__ MaxSum combine(MaxSum a, MaxSum b) {
    const float m = fmaxf(a.m, b.m);
    if (m == -INFINITY) return {m, 0.0f};
    return {m, a.s * __expf(a.m - m) + b.s * __expf(b.m - m)};
}

template <int WAVES = kWaves>
__device__ __forceinline__ MaxSum block_combine(MaxSum v, MaxSum* stage) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        MaxSum other{__shfl_xor(v.m, offset, kWave), __shfl_xor(v.s, offset, kWave)};
        v = combine(v, other);
    }
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) stage[wave] = v;
    __syncthreads();
    MaxSum total = stage[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) total = combine(total, stage[w]);
    return total;
}

// Streaming kernel for rows that are too long to hold or not 16-byte aligned (a vocabulary that is not a
// multiple of the vector width moves every row's start): each row is split into the elements before its first
// 16-byte boundary, whole 128-bit vectors, and the rest. vector_ok: logits and gradient rows have the same
// alignment phase (or there is no gradient).
template <typename T, bool WithGradient>
__global__ __launch_bounds__(kThreads) void cross_entropy_row_kernel(float* __restrict__ row_loss,
                                                                    T* gradient,  // may alias logits (in place)
                                                                    const T* logits,
                                                                    const std::uint32_t* __restrict__ targets,
                                                                    unsigned int vocab, float factor,
                                                                    bool vector_ok) {
    constexpr int VEC = kVec128<T>;
    __shared__ MaxSum stage[kWaves];
    const std::size_t base = static_cast<std::size_t>(blockIdx.x) * vocab;
    const T* row = logits + base;
    const unsigned int to_boundary =
        static_cast<unsigned int>(((16u - (reinterpret_cast<std::uintptr_t>(row) & 15u)) & 15u) / sizeof(T));
    const unsigned int head = vector_ok ? (to_boundary < vocab ? to_boundary : vocab) : vocab;
    const unsigned int vectors = (vocab - head) / VEC;
    const unsigned int body_end = head + vectors * VEC;
    const unsigned int edge = head + (vocab - body_end);  // elements handled one by one
    const T* body = row + head;
    const std::uint32_t target = targets[blockIdx.x];
    // Read before the barrier below: in-place use overwrites the row in pass 2.
    const float target_logit = (threadIdx.x == 0 && target < vocab) ? to_f32(row[target]) : 0.0f;

    MaxSum acc{-INFINITY, 0.0f};
    for (unsigned int v = threadIdx.x; v < vectors; v += kThreads) {
        const vec_t<float, VEC> x = vec_to_f32<T, VEC>(load_vec<T, VEC>(body + v * VEC));
        float vmax = x[0];
#pragma unroll
        for (int e = 1; e < VEC; ++e) vmax = fmaxf(vmax, x[e]);
        if (vmax > acc.m) {
            acc.s *= __expf(acc.m - vmax);
            acc.m = vmax;
        }
        if (acc.m != -INFINITY) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc.s += __expf(x[e] - acc.m);
        }
    }
    for (unsigned int k = threadIdx.x; k < edge; k += kThreads) {
        const unsigned int i = k < head ? k : body_end + (k - head);
        const float x = to_f32(row[i]);
        if (x > acc.m) {
            acc.s *= __expf(acc.m - x);
            acc.m = x;
        }
        if (acc.m != -INFINITY) acc.s += __expf(x - acc.m);
    }
    const MaxSum total = block_combine(acc, stage);
    if (threadIdx.x == 0) {
        float loss = 0.0f;
        if (target < vocab) loss = __logf(total.s) + total.m - target_logit;
        row_loss[blockIdx.x] = loss;
    }
    if constexpr (WithGradient) {
        const float inv = 1.0f / total.s;
        T* out = gradient + base;
        for (unsigned int v = threadIdx.x; v < vectors; v += kThreads) {
            const vec_t<float, VEC> x = vec_to_f32<T, VEC>(load_vec<T, VEC>(body + v * VEC));
            vec_t<float, VEC> g;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float value = __expf(x[e] - total.m) * inv;
                if (head + v * VEC + e == target) value -= 1.0f;
                g[e] = value * factor;
            }
            store_vec<T, VEC>(out + head + v * VEC, vec_from_f32<T, VEC>(g));
        }
        for (unsigned int k = threadIdx.x; k < edge; k += kThreads) {
            const unsigned int i = k < head ? k : body_end + (k - head);
            float value = __expf(to_f32(row[i]) - total.m) * inv;
            if (i == target) value -= 1.0f;
            out[i] = from_f32<T>(value * factor);
        }
    }
}

// Rows of up to kResidentThreads * SLOTS 128-bit vectors stay in registers between the two passes:
// every load of the row is in flight at once, and the memory system sees exactly one read and one
// write of the row (the streaming kernel's second pass finds the row in L2 only while the rows in
// flight on an XCD fit there, which 8 rows of 64 KB per CU do not).
constexpr int kResidentThreads = 512;
template <typename T, int SLOTS, bool WithGradient>
__global__ __launch_bounds__(kResidentThreads) void cross_entropy_row_resident_kernel(
    float* __restrict__ row_loss, T* gradient /* may alias logits */, const T* logits,
    const std::uint32_t* __restrict__ targets, unsigned int vocab, float factor) {
    constexpr int VEC = kVec128<T>;
    constexpr int WAVES = kResidentThreads / kWave;
    __shared__ MaxSum stage[WAVES];
    const std::size_t base = static_cast<std::size_t>(blockIdx.x) * vocab;
    const T* row = logits + base;
    const unsigned int vectors = vocab / VEC;
    const std::uint32_t target = targets[blockIdx.x];
    // Read before the barrier in block_combine: in-place use overwrites the row after it.
    const float target_logit = (threadIdx.x == 0 && target < vocab) ? to_f32(row[target]) : 0.0f;

    vec_t<T, VEC> held[SLOTS];
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        const unsigned int v = s * kResidentThreads + threadIdx.x;
        if (v < vectors) held[s] = load_vec<T, VEC>(row + v * VEC);
    }
    MaxSum acc{-INFINITY, 0.0f};
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
        if (s * kResidentThreads + threadIdx.x < vectors) {
            const vec_t<float, VEC> x = vec_to_f32<T, VEC>(held[s]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc.m = fmaxf(acc.m, x[e]);
        }
    }
    if (acc.m != -INFINITY) {
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            if (s * kResidentThreads + threadIdx.x < vectors) {
                const vec_t<float, VEC> x = vec_to_f32<T, VEC>(held[s]);
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc.s += __expf(x[e] - acc.m);
            }
        }
    }
    const MaxSum total = block_combine<WAVES>(acc, stage);
    if (threadIdx.x == 0) {
        float loss = 0.0f;
        if (target < vocab) loss = __logf(total.s) + total.m - target_logit;
        row_loss[blockIdx.x] = loss;
    }
    if constexpr (WithGradient) {
        const float inv = 1.0f / total.s;
        T* out = gradient + base;
#pragma unroll
        for (int s = 0; s < SLOTS; ++s) {
            const unsigned int v = s * kResidentThreads + threadIdx.x;
            if (v < vectors) {
                const vec_t<float, VEC> x = vec_to_f32<T, VEC>(held[s]);
                vec_t<float, VEC> g;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float value = __expf(x[e] - total.m) * inv;
                    if (v * VEC + e == target) value -= 1.0f;
                    g[e] = value * factor;
                }
                store_vec<T, VEC>(out + v * VEC, vec_from_f32<T, VEC>(g));
            }
        }
    }
}

template <typename T, int SLOTS>
void launch_resident(float* row_loss, T* gradient, const T* logits, const std::uint32_t* targets, unsigned int rows,
                     unsigned int vocab, float factor, hipStream_t stream) {
    if (gradient != nullptr)
        hipLaunchKernelGGL((cross_entropy_row_resident_kernel<T, SLOTS, true>), dim3(rows), dim3(kResidentThreads), 0,
                           stream, row_loss, gradient, logits, targets, vocab, factor);
    else
        hipLaunchKernelGGL((cross_entropy_row_resident_kernel<T, SLOTS, false>), dim3(rows), dim3(kResidentThreads), 0,
                           stream, row_loss, gradient, logits, targets, vocab, factor);
}

}  // namespace

// Shared with the cut-cross-entropy path: loss[0] = (Σ row_loss) / rows, fixed order.
__global__ __launch_bounds__(1024) void mean_reduce_kernel(float* __restrict__ loss,
                                                          const float* __restrict__ row_loss, unsigned int rows,
                                                          float inv_rows) {
    __shared__ double stage[1024];
    // Four independent partial sums per thread keep four loads in flight; the order of additions is
    // fixed by (rows, thread count), so the result is reproducible.
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    unsigned int i = threadIdx.x;
    for (; i + 3 * 1024 < rows; i += 4 * 1024) {
        s0 += static_cast<double>(row_loss[i]);
        s1 += static_cast<double>(row_loss[i + 1024]);
        s2 += static_cast<double>(row_loss[i + 2 * 1024]);
        s3 += static_cast<double>(row_loss[i + 3 * 1024]);
    }
    for (; i < rows; i += 1024) s0 += static_cast<double>(row_loss[i]);
    stage[threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int stride = 512; stride > 0; stride >>= 1) {
        if (threadIdx.x < static_cast<unsigned int>(stride)) stage[threadIdx.x] += stage[threadIdx.x + stride];
        __syncthreads();
    }
    if (threadIdx.x == 0) loss[0] = static_cast<float>(stage[0]) * inv_rows;
}

// Per-row pass: row_loss[r] and (optionally) the gradient, factor = gradient_scale / total_rows.
int cross_entropy_rows(float* row_loss, void* gradient, const void* logits, const std::uint32_t* targets,
                       std::size_t rows, std::size_t vocab, float factor, int dtype, hipStream_t stream) {
    const auto r = static_cast<unsigned int>(rows), v = static_cast<unsigned int>(vocab);
    const bool with_gradient = gradient != nullptr;
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const bool vector_ok = vocab % kVec128<T> == 0 && is_aligned16(logits) &&
                               (!with_gradient || is_aligned16(gradient));
        // The streaming kernel finds each row's own 16-byte boundary; logits and gradient rows must share it.
        const bool same_phase = !with_gradient || ((reinterpret_cast<std::uintptr_t>(logits) ^
                                                    reinterpret_cast<std::uintptr_t>(gradient)) & 15u) == 0;
        const unsigned int vectors = v / kVec128<T>;
        if (vector_ok && vectors <= 16u * kResidentThreads) {
            auto* g = static_cast<T*>(gradient);
            auto* z = static_cast<const T*>(logits);
            if (vectors <= 2u * kResidentThreads) launch_resident<T, 2>(row_loss, g, z, targets, r, v, factor, stream);
            else if (vectors <= 8u * kResidentThreads) launch_resident<T, 8>(row_loss, g, z, targets, r, v, factor, stream);
            else launch_resident<T, 16>(row_loss, g, z, targets, r, v, factor, stream);
        } else if (with_gradient) {
            hipLaunchKernelGGL((cross_entropy_row_kernel<T, true>), dim3(r), dim3(kThreads), 0, stream, row_loss,
                               static_cast<T*>(gradient), static_cast<const T*>(logits), targets, v, factor, same_phase);
        } else {
            hipLaunchKernelGGL((cross_entropy_row_kernel<T, false>), dim3(r), dim3(kThreads), 0, stream, row_loss,
                               static_cast<T*>(nullptr), static_cast<const T*>(logits), targets, v, factor, same_phase);
        }
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

int mean_reduce(float* loss, const float* row_loss, std::size_t rows, hipStream_t stream) {
    hipLaunchKernelGGL(mean_reduce_kernel, dim3(1), dim3(1024), 0, stream, loss, row_loss,
                       static_cast<unsigned int>(rows), 1.0f / static_cast<float>(rows));
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

namespace {

int run(float* loss, void* gradient, const void* logits, const std::uint32_t* targets, std::size_t rows,
        std::size_t vocab, float gradient_scale, int dtype, hipStream_t stream, bool with_gradient,
        const char* name) {
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (loss == nullptr || logits == nullptr || targets == nullptr || rows == 0 || vocab == 0 ||
        (with_gradient && gradient == nullptr))
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": invalid tensors or targets");
    if (with_gradient && (!std::isfinite(gradient_scale) || gradient_scale <= 0.0f))
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": gradient scale must be finite and positive");
    constexpr std::size_t i32max = std::numeric_limits<int>::max();
    if (rows > i32max || vocab > i32max) return fail(CGPTX_OVERFLOW, std::string(name) + ": dimension exceeds int range");
    void* mem = nullptr;
    if (int s = scratch(stream, rows * sizeof(float), &mem)) return s;
    auto* row_loss = static_cast<float*>(mem);
    const float factor = gradient_scale / static_cast<float>(rows);
    if (int s = cross_entropy_rows(row_loss, with_gradient ? gradient : nullptr, logits, targets, rows, vocab, factor,
                                   dtype, stream))
        return s;
    return mean_reduce(loss, row_loss, rows, stream);
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_cross_entropy_forward_backward(float* loss, void* gradient, const void* logits,
                                                    const uint32_t* targets, size_t rows, size_t vocab,
                                                    float gradient_scale, int dtype, cgptx_stream stream) {
    return cgptx::run(loss, gradient, logits, targets, rows, vocab, gradient_scale, dtype,
                      static_cast<hipStream_t>(stream), true, "cross_entropy_forward_backward");
}

extern "C" int cgptx_cross_entropy_forward(float* loss, const void* logits, const uint32_t* targets, size_t rows,
                                           size_t vocab, int dtype, cgptx_stream stream) {
    return cgptx::run(loss, nullptr, logits, targets, rows, vocab, 1.0f, dtype, static_cast<hipStream_t>(stream),
                      false, "cross_entropy_forward");
}
