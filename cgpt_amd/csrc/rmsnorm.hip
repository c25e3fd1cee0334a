// RMSNorm forward and backward for gfx950.
//
// Backward (reference semantics: src/ops/cpu/backward/rmsnorm_backward_cpu.cpp:86-133,
// CUDA dispatch src/ops/backward/rmsnorm_backward.cu:445-547):
//   r = 1/sqrt(mean(x^2)+eps);  c = (sum_j dy_j w_j x_j) r^3 / H
//   dx = dy w r - x c;          dgamma_j = sum_rows dy x r
//
// Fast path: one pass over x and dy. A wavefront owns 64/LPR rows at a time
// (LPR lanes per row, 128-bit accesses), keeps the row in registers between the
// reduction and the dx store, and accumulates its dgamma columns in registers.
// Per-block dgamma partials go to scratch and a second small kernel sums them in
// a fixed order, so the result does not depend on scheduling. HBM traffic is
// read x + read dy + write dx (+ partials, ~2% at 32768x1024).
//
// Generic path (any H, any alignment): row kernel with a second, cache-served
// read, then a column kernel over saved 1/rms.
#include "common.hpp"
#include "reduce.hpp"

#include <cmath>
#include <limits>
#include <mutex>
#include <unordered_map>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kWavesPerBlock = kThreads / kWave;
// Groups of four rows a wavefront of the dense norm + rotary kernel requests at a time: the backward pass holds three
// times the registers per group, and more of them in flight cost it more in resident wavefronts than they bring.
template <bool Backward>
constexpr int kRopeDenseUnroll = Backward ? 2 : 4;

// Rotary embedding applied to the rows on the way (rows are heads of head_dim = hidden elements):
// forward  y = rope(round(rmsnorm(x)));  backward  the incoming gradient is rotated back (and
// rounded) first. The roundings are those of the separate operators' stores, so the fused pass gives
// bit for bit what rmsnorm and rope give one after the other.
struct RopeArgs {
    const void* cos_cache;  // [positions, rotary_dim/2], element type of the rows
    const void* sin_cache;
    int heads;      // rows per token
    int sequence;   // tokens per sequence: position = offset + token % sequence
    int rotary_dim;
    int position_offset;
};

// Rotation of the pair (x, y) by +angle (forward) or -angle (backward); the arithmetic of the
// separate rotary kernels.
template <bool Inverse>
__device__ __forceinline__ void rotate_pair(float x, float y, float c, float s, float& ox, float& oy) {
    if constexpr (Inverse) {
        ox = fmaf(y, s, x * c);
        oy = fmaf(-x, s, y * c);
    } else {
        ox = fmaf(-y, s, x * c);
        oy = fmaf(x, s, y * c);
    }
}

template <typename T, bool Inverse>
__device__ __forceinline__ vec_t<float, kVec128<T>> rope_vector(vec_t<float, kVec128<T>> v, const RopeArgs& rope, int row,
                                                                int col) {
    constexpr int VEC = kVec128<T>;
    constexpr int HALF = VEC / 2;
    // What the separate operator would have read back from memory.
    v = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(v));
    if (col >= rope.rotary_dim) return v;
    const int token = row / rope.heads;
    const int pos = rope.position_offset + token % rope.sequence;
    const std::size_t index = static_cast<std::size_t>(pos) * (rope.rotary_dim / 2) + col / 2;
    const vec_t<float, HALF> c = vec_to_f32<T, HALF>(load_vec<T, HALF>(static_cast<const T*>(rope.cos_cache) + index));
    const vec_t<float, HALF> s = vec_to_f32<T, HALF>(load_vec<T, HALF>(static_cast<const T*>(rope.sin_cache) + index));
    vec_t<float, VEC> r;
#pragma unroll
    for (int p = 0; p < HALF; ++p) {
        float a, b;
        rotate_pair<Inverse>(v[2 * p], v[2 * p + 1], c[p], s[p], a, b);
        r[2 * p] = a;
        r[2 * p + 1] = b;
    }
    return r;
}

// ------------------------------------------------------------------ fast path
template <typename T, int LPR, int K, bool Backward, bool Rope = false>
__global__ __launch_bounds__(kThreads) void rmsnorm_rows_kernel(
    T* out,                         // dx (backward) or y (forward)
    float* __restrict__ partial,    // [gridDim.x, H] dgamma partials (backward)
    const T* dy,                    // backward only; may be out itself
    const T* residual,              // backward only, optional: added to dx (may be out itself)
    const T* __restrict__ x, const T* __restrict__ w, int rows, int hidden, float inv_hidden, float eps,
    RopeArgs rope = RopeArgs{}) {
    constexpr int VEC = kVec128<T>;
    constexpr int RPW = kWave / LPR;  // rows per wavefront iteration
    using F = vec_t<float, VEC>;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int sub = lane % LPR;   // lane within the row
    const int rsel = lane / LPR;  // which of the RPW rows

    F wv[K];
    F acc[K];
    bool live[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
        const int col = (c * LPR + sub) * VEC;
        live[c] = col < hidden;
        wv[c] = live[c] ? vec_to_f32<T, VEC>(load_vec<T, VEC>(w + col)) : F(0.0f);
        acc[c] = F(0.0f);
    }

    const int groups = (rows + RPW - 1) / RPW;
    const int wave_global = blockIdx.x * kWavesPerBlock + wave;
    const int wave_count = gridDim.x * kWavesPerBlock;
    for (int g = wave_global; g < groups; g += wave_count) {
        const int row = g * RPW + rsel;
        const bool row_live = row < rows;
        const std::size_t base = static_cast<std::size_t>(row) * hidden;
        F xv[K], gv[K];
        vec_t<T, VEC> rv[K];  // residual, requested with the other operands: one memory round trip per row
#pragma unroll
        for (int c = 0; c < K; ++c) {
            const int col = (c * LPR + sub) * VEC;
            if (row_live && live[c]) {
                xv[c] = vec_to_f32<T, VEC>(load_vec<T, VEC>(x + base + col));
                if constexpr (Backward) {
                    if (residual != nullptr) rv[c] = load_vec<T, VEC>(residual + base + col);
                    gv[c] = vec_to_f32<T, VEC>(load_vec<T, VEC>(dy + base + col));
                    if constexpr (Rope) gv[c] = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(rope_vector<T, true>(gv[c], rope, row, col)));
                }
            } else {
                xv[c] = F(0.0f);
                if constexpr (Backward) gv[c] = F(0.0f);
            }
        }
        float ss = 0.0f, dd = 0.0f;
#pragma unroll
        for (int c = 0; c < K; ++c) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                ss = fmaf(xv[c][e], xv[c][e], ss);
                if constexpr (Backward) dd = fmaf(gv[c][e] * wv[c][e], xv[c][e], dd);
            }
        }
        ss = wave_sum<LPR>(ss);
        const float inv = 1.0f / sqrtf(ss * inv_hidden + eps);
        if constexpr (Backward) {
            dd = wave_sum<LPR>(dd);
            const float corr = dd * inv * inv * inv * inv_hidden;
#pragma unroll
            for (int c = 0; c < K; ++c) {
                F r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    r[e] = gv[c][e] * wv[c][e] * inv - xv[c][e] * corr;
                    acc[c][e] = fmaf(gv[c][e], xv[c][e] * inv, acc[c][e]);
                }
                const int col = (c * LPR + sub) * VEC;
                if (row_live && live[c]) {
                    if (residual != nullptr) r += vec_to_f32<T, VEC>(rv[c]);
                    store_vec<T, VEC>(out + base + col, vec_from_f32<T, VEC>(r));
                }
            }
        } else {
#pragma unroll
            for (int c = 0; c < K; ++c) {
                F r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) r[e] = xv[c][e] * inv * wv[c][e];
                const int col = (c * LPR + sub) * VEC;
                if (row_live && live[c]) {
                    if constexpr (Rope) r = rope_vector<T, false>(r, rope, row, col);
                    store_vec<T, VEC>(out + base + col, vec_from_f32<T, VEC>(r));
                }
            }
        }
    }

    if constexpr (Backward) {
        // Fold the RPW row slots of the wavefront, then the block's wavefronts.
        __shared__ float stage[kWavesPerBlock][LPR * K * VEC];
#pragma unroll
        for (int c = 0; c < K; ++c) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                float v = acc[c][e];
#pragma unroll
                for (int offset = LPR; offset < kWave; offset <<= 1) v += __shfl_xor(v, offset, kWave);
                if (rsel == 0) stage[wave][(c * LPR + sub) * VEC + e] = v;
            }
        }
        __syncthreads();
        for (int col = threadIdx.x; col < hidden; col += kThreads) {
            float v = 0.0f;
#pragma unroll
            for (int s = 0; s < kWavesPerBlock; ++s) v += stage[s][col];
            partial[static_cast<std::size_t>(blockIdx.x) * hidden + col] = v;
        }
    }
}

// The fused per-head norm + rotary pass at the shape a training step gives it: rows of exactly 16 vectors (head_dim 128
// in 16-bit storage), all of them rotated, a multiple of four rows, tensors and tables below 4 GiB. Same arithmetic,
// in the same order, as rmsnorm_rows_kernel<T, 16, 1, Backward, true>; what differs is the bookkeeping, which at 2 KiB
// of rows per wavefront and trip is what that kernel spends most of its instructions on: no per-lane predicates, 32-bit
// byte offsets that advance by a constant, and the token position carried from trip to trip (head index and position
// advance by constants with one carry each) instead of two integer divisions per trip. A trip requests U groups of
// four rows before it uses the first, so that a wavefront has U times the bytes in flight.
template <typename T, bool Backward, int U>
__global__ __launch_bounds__(kThreads) void rmsnorm_rope_dense_kernel(
    T* out, float* __restrict__ partial, const T* dy /* may be out itself */, const T* __restrict__ x,
    const T* __restrict__ w, int rows, float inv_hidden, float eps, RopeArgs rope) {
    constexpr int VEC = kVec128<T>;
    constexpr int HALF = VEC / 2;
    constexpr int LPR = 16;
    constexpr int RPW = kWave / LPR;
    constexpr int HIDDEN = LPR * VEC;
    using F = vec_t<float, VEC>;
    using H = vec_t<float, HALF>;

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int sub = lane % LPR;
    const int rsel = lane / LPR;
    const F wv = vec_to_f32<T, VEC>(load_vec<T, VEC>(w + sub * VEC));
    F acc(0.0f);

    const int groups = rows / RPW;
    const int wave_global = blockIdx.x * kWavesPerBlock + wave;
    const int wave_count = gridDim.x * kWavesPerBlock;
    const int first_row = wave_global * RPW + rsel;
    const int stride_rows = wave_count * RPW;
    int head = first_row % rope.heads;
    int pos = (first_row / rope.heads) % rope.sequence;
    const int head_step = stride_rows % rope.heads;
    const int pos_step = (stride_rows / rope.heads) % rope.sequence;
    unsigned offset = (static_cast<unsigned>(first_row) * HIDDEN + sub * VEC) * static_cast<unsigned>(sizeof(T));
    const unsigned offset_step = static_cast<unsigned>(stride_rows) * HIDDEN * static_cast<unsigned>(sizeof(T));
    const unsigned table_lane = sub * HALF * static_cast<unsigned>(sizeof(T));
    constexpr unsigned kTableRow = (HIDDEN / 2) * sizeof(T);
    const auto at = [](const void* base, unsigned bytes) {
        return reinterpret_cast<const T*>(static_cast<const char*>(base) + bytes);
    };

    struct Fetched {
        vec_t<T, VEC> x, g;
        vec_t<T, HALF> c, s;
        unsigned offset;
    };
    // Requests the operands of the group at `offset` / `pos` and moves both on to the wavefront's next group.
    const auto fetch = [&]() {
        Fetched f;
        const unsigned table = static_cast<unsigned>(rope.position_offset + pos) * kTableRow + table_lane;
        f.c = load_vec<T, HALF>(at(rope.cos_cache, table));
        f.s = load_vec<T, HALF>(at(rope.sin_cache, table));
        f.x = load_vec<T, VEC>(at(x, offset));
        if constexpr (Backward) f.g = load_vec<T, VEC>(at(dy, offset));
        f.offset = offset;
        offset += offset_step;
        head += head_step;
        const int carry = head >= rope.heads ? 1 : 0;
        head -= carry ? rope.heads : 0;
        pos += pos_step + carry;
        pos -= pos >= rope.sequence ? rope.sequence : 0;
        return f;
    };
    const auto finish = [&](const Fetched& f) {
        const H c = vec_to_f32<T, HALF>(f.c);
        const H s = vec_to_f32<T, HALF>(f.s);
        const F xv = vec_to_f32<T, VEC>(f.x);
        F gv;
        if constexpr (Backward) {
            // The incoming gradient rotated back and rounded: what the separate rotary operator would have stored.
            const F raw = vec_to_f32<T, VEC>(f.g);
            F turned;
#pragma unroll
            for (int p = 0; p < HALF; ++p) {
                float a, b;
                rotate_pair<true>(raw[2 * p], raw[2 * p + 1], c[p], s[p], a, b);
                turned[2 * p] = a;
                turned[2 * p + 1] = b;
            }
            gv = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(turned));
        }
        float ss = 0.0f, dd = 0.0f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            ss = fmaf(xv[e], xv[e], ss);
            if constexpr (Backward) dd = fmaf(gv[e] * wv[e], xv[e], dd);
        }
        ss = wave_sum<LPR>(ss);
        const float inv = 1.0f / sqrtf(ss * inv_hidden + eps);
        F r;
        if constexpr (Backward) {
            dd = wave_sum<LPR>(dd);
            const float corr = dd * inv * inv * inv * inv_hidden;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                r[e] = gv[e] * wv[e] * inv - xv[e] * corr;
                acc[e] = fmaf(gv[e], xv[e] * inv, acc[e]);
            }
        } else {
            F y;
#pragma unroll
            for (int e = 0; e < VEC; ++e) y[e] = xv[e] * inv * wv[e];
            y = vec_to_f32<T, VEC>(vec_from_f32<T, VEC>(y));  // the norm's own store, before the rotation
#pragma unroll
            for (int p = 0; p < HALF; ++p) {
                float a, b;
                rotate_pair<false>(y[2 * p], y[2 * p + 1], c[p], s[p], a, b);
                r[2 * p] = a;
                r[2 * p + 1] = b;
            }
        }
        store_vec<T, VEC>(const_cast<T*>(at(out, f.offset)), vec_from_f32<T, VEC>(r));
    };

    int g = wave_global;
    for (; g + (U - 1) * wave_count < groups; g += U * wave_count) {
        Fetched f[U];
#pragma unroll
        for (int u = 0; u < U; ++u) f[u] = fetch();
        __builtin_amdgcn_sched_barrier(0);  // every request of the trip goes out before the first use
#pragma unroll
        for (int u = 0; u < U; ++u) finish(f[u]);
    }
    for (; g < groups; g += wave_count) finish(fetch());

    if constexpr (Backward) {
        // Fold the four row slots of the wavefront, then the block's wavefronts.
        __shared__ float stage[kWavesPerBlock][HIDDEN];
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float v = acc[e];
#pragma unroll
            for (int across = LPR; across < kWave; across <<= 1) v += __shfl_xor(v, across, kWave);
            if (rsel == 0) stage[wave][sub * VEC + e] = v;
        }
        __syncthreads();
        for (int col = threadIdx.x; col < HIDDEN; col += kThreads) {
            float v = 0.0f;
#pragma unroll
            for (int s = 0; s < kWavesPerBlock; ++s) v += stage[s][col];
            partial[static_cast<std::size_t>(blockIdx.x) * HIDDEN + col] = v;
        }
    }
}

// Two RMSNorms of the same rows with different weights (the block's attention and feed-forward norms
// both read the block input): one pass reads x once.
//   forward   y_a = x r w_a,  y_f = x r w_f
//   backward  dx = g r - x (sum_j g_j x_j) r^3 / H + residual  with g = dy_a w_a + dy_f w_f  (the two
//             gradients add up before the row reduction: the norm is the same for both),
//             dgamma_a = sum_rows dy_a x r,  dgamma_f = sum_rows dy_f x r
template <typename T, int LPR, int K, bool Backward>
__global__ __launch_bounds__(kThreads) void rmsnorm_dual_rows_kernel(
    T* out_a,                       // y_a (forward) or dx (backward)
    T* out_f,                       // y_f (forward)
    float* __restrict__ partial_a,  // [gridDim.x, H] dgamma partials (backward)
    float* __restrict__ partial_f,
    const T* __restrict__ dy_a, const T* __restrict__ dy_f,  // backward only
    const T* residual,              // backward only, optional: added to dx (may be out_a itself)
    const T* __restrict__ x, const T* __restrict__ w_a, const T* __restrict__ w_f, int rows, int hidden,
    float inv_hidden, float eps) {
    constexpr int VEC = kVec128<T>;
    constexpr int RPW = kWave / LPR;
    using F = vec_t<float, VEC>;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int sub = lane % LPR;
    const int rsel = lane / LPR;

    F wa[K], wf[K], acc_a[K], acc_f[K];
    bool live[K];
#pragma unroll
    for (int c = 0; c < K; ++c) {
        const int col = (c * LPR + sub) * VEC;
        live[c] = col < hidden;
        wa[c] = live[c] ? vec_to_f32<T, VEC>(load_vec<T, VEC>(w_a + col)) : F(0.0f);
        wf[c] = live[c] ? vec_to_f32<T, VEC>(load_vec<T, VEC>(w_f + col)) : F(0.0f);
        acc_a[c] = F(0.0f);
        acc_f[c] = F(0.0f);
    }
    const int groups = (rows + RPW - 1) / RPW;
    const int wave_global = blockIdx.x * kWavesPerBlock + wave;
    const int wave_count = gridDim.x * kWavesPerBlock;
    for (int g = wave_global; g < groups; g += wave_count) {
        const int row = g * RPW + rsel;
        const bool row_live = row < rows;
        const std::size_t base = static_cast<std::size_t>(row) * hidden;
        F xv[K], ga[K], gf[K];
        vec_t<T, VEC> rv[K];  // residual, requested with the other operands: one memory round trip per row
#pragma unroll
        for (int c = 0; c < K; ++c) {
            const int col = (c * LPR + sub) * VEC;
            const bool on = row_live && live[c];
            xv[c] = on ? vec_to_f32<T, VEC>(load_vec<T, VEC>(x + base + col)) : F(0.0f);
            if constexpr (Backward) {
                ga[c] = on ? vec_to_f32<T, VEC>(load_vec<T, VEC>(dy_a + base + col)) : F(0.0f);
                gf[c] = on ? vec_to_f32<T, VEC>(load_vec<T, VEC>(dy_f + base + col)) : F(0.0f);
                if (on && residual != nullptr) rv[c] = load_vec<T, VEC>(residual + base + col);
            }
        }
        float ss = 0.0f, dd = 0.0f;
#pragma unroll
        for (int c = 0; c < K; ++c) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                ss = fmaf(xv[c][e], xv[c][e], ss);
                if constexpr (Backward) dd = fmaf(fmaf(ga[c][e], wa[c][e], gf[c][e] * wf[c][e]), xv[c][e], dd);
            }
        }
        ss = wave_sum<LPR>(ss);
        const float inv = 1.0f / sqrtf(ss * inv_hidden + eps);
        if constexpr (Backward) {
            dd = wave_sum<LPR>(dd);
            const float corr = dd * inv * inv * inv * inv_hidden;
#pragma unroll
            for (int c = 0; c < K; ++c) {
                F r;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float scaled = xv[c][e] * inv;
                    r[e] = fmaf(ga[c][e], wa[c][e], gf[c][e] * wf[c][e]) * inv - xv[c][e] * corr;
                    acc_a[c][e] = fmaf(ga[c][e], scaled, acc_a[c][e]);
                    acc_f[c][e] = fmaf(gf[c][e], scaled, acc_f[c][e]);
                }
                const int col = (c * LPR + sub) * VEC;
                if (row_live && live[c]) {
                    if (residual != nullptr) r += vec_to_f32<T, VEC>(rv[c]);
                    store_vec<T, VEC>(out_a + base + col, vec_from_f32<T, VEC>(r));
                }
            }
        } else {
#pragma unroll
            for (int c = 0; c < K; ++c) {
                F ra, rf;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    ra[e] = xv[c][e] * inv * wa[c][e];
                    rf[e] = xv[c][e] * inv * wf[c][e];
                }
                const int col = (c * LPR + sub) * VEC;
                if (row_live && live[c]) {
                    store_vec<T, VEC>(out_a + base + col, vec_from_f32<T, VEC>(ra));
                    store_vec<T, VEC>(out_f + base + col, vec_from_f32<T, VEC>(rf));
                }
            }
        }
    }
    if constexpr (Backward) {
        // Fold the RPW row slots of the wavefront, then the block's wavefronts; first one weight, then the other.
        __shared__ float stage[kWavesPerBlock][LPR * K * VEC];
#pragma unroll
        for (int which = 0; which < 2; ++which) {
#pragma unroll
            for (int c = 0; c < K; ++c) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    float v = which == 0 ? acc_a[c][e] : acc_f[c][e];
#pragma unroll
                    for (int offset = LPR; offset < kWave; offset <<= 1) v += __shfl_xor(v, offset, kWave);
                    if (rsel == 0) stage[wave][(c * LPR + sub) * VEC + e] = v;
                }
            }
            __syncthreads();
            float* partial = which == 0 ? partial_a : partial_f;
            for (int col = threadIdx.x; col < hidden; col += kThreads) {
                float v = 0.0f;
#pragma unroll
                for (int s = 0; s < kWavesPerBlock; ++s) v += stage[s][col];
                partial[static_cast<std::size_t>(blockIdx.x) * hidden + col] = v;
            }
            __syncthreads();
        }
    }
}

// --------------------------------------------------------------- generic path
template <typename T, bool Backward>
__global__ __launch_bounds__(kThreads) void rmsnorm_row_generic_kernel(
    T* __restrict__ out, float* __restrict__ inv_rms, const T* __restrict__ dy, const T* __restrict__ x,
    const T* __restrict__ w, int rows, int hidden, float inv_hidden, float eps) {
    __shared__ float red[2][kWavesPerBlock];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    for (int row = blockIdx.x; row < rows; row += gridDim.x) {
        const std::size_t base = static_cast<std::size_t>(row) * hidden;
        float ss = 0.0f, dd = 0.0f;
        for (int col = threadIdx.x; col < hidden; col += kThreads) {
            const float xv = to_f32(x[base + col]);
            ss = fmaf(xv, xv, ss);
            if constexpr (Backward) dd = fmaf(to_f32(dy[base + col]) * to_f32(w[col]), xv, dd);
        }
        ss = wave_sum(ss);
        dd = wave_sum(dd);
        __syncthreads();  // protects red[] against the previous iteration's readers
        if (lane == 0) {
            red[0][wave] = ss;
            red[1][wave] = dd;
        }
        __syncthreads();
        ss = 0.0f;
        dd = 0.0f;
#pragma unroll
        for (int s = 0; s < kWavesPerBlock; ++s) {
            ss += red[0][s];
            dd += red[1][s];
        }
        const float inv = 1.0f / sqrtf(ss * inv_hidden + eps);
        if constexpr (Backward) {
            const float corr = dd * inv * inv * inv * inv_hidden;
            if (threadIdx.x == 0) inv_rms[row] = inv;
            for (int col = threadIdx.x; col < hidden; col += kThreads) {
                out[base + col] = from_f32<T>(to_f32(dy[base + col]) * to_f32(w[col]) * inv -
                                              to_f32(x[base + col]) * corr);
            }
        } else {
            for (int col = threadIdx.x; col < hidden; col += kThreads) {
                out[base + col] = from_f32<T>(to_f32(x[base + col]) * inv * to_f32(w[col]));
            }
        }
    }
}

// partial[blockIdx.y, col] = sum over this block's row slice of dy*x*inv_rms.
template <typename T>
__global__ __launch_bounds__(kThreads) void rmsnorm_dgamma_generic_kernel(
    float* __restrict__ partial, const T* __restrict__ dy, const T* __restrict__ x,
    const float* __restrict__ inv_rms, int rows, int hidden, int rows_per_slice) {
    __shared__ float stage[kWavesPerBlock][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = blockIdx.x * kWave + lane;
    const int row_begin = blockIdx.y * rows_per_slice;
    const int row_end = min(rows, row_begin + rows_per_slice);
    float v = 0.0f;
    if (col < hidden) {
        for (int row = row_begin + slice; row < row_end; row += kWavesPerBlock) {
            const std::size_t index = static_cast<std::size_t>(row) * hidden + col;
            v = fmaf(to_f32(dy[index]), to_f32(x[index]) * inv_rms[row], v);
        }
    }
    stage[slice][lane] = v;
    __syncthreads();
    if (slice == 0 && col < hidden) {
        float total = 0.0f;
#pragma unroll
        for (int s = 0; s < kWavesPerBlock; ++s) total += stage[s][lane];
        partial[static_cast<std::size_t>(blockIdx.y) * hidden + col] = total;
    }
}

// ------------------------------------------------------------------- dispatch
struct FastShape {
    int lpr = 0;
    int k = 0;
};

template <typename T>
FastShape pick_fast_shape(int hidden) {
    constexpr int VEC = kVec128<T>;
    if (hidden % VEC != 0) return {};
    const int vecs = hidden / VEC;
    if (vecs <= 16) return {16, 1};
    if (vecs <= 32) return {32, 1};
    if (vecs <= 64) return {64, 1};
    if (vecs <= 128) return {64, 2};
    if (vecs <= 256) return {64, 4};
    return {};
}

// Whether rmsnorm_rope_dense_kernel serves the pass: rows of exactly 16 vectors, all of them rotated, whole groups of
// four rows, and every byte offset it forms (tensor and table) below 2^32.
template <typename T>
bool rope_dense(int rows, int hidden, const RopeArgs& rope) {
    constexpr int VEC = kVec128<T>;
    const unsigned long long tensor_bytes = static_cast<unsigned long long>(rows) * hidden * sizeof(T);
    const unsigned long long table_bytes =
        (static_cast<unsigned long long>(rope.position_offset) + rope.sequence) * (hidden / 2) * sizeof(T);
    return hidden == 16 * VEC && rope.rotary_dim == hidden && rows % 4 == 0 && tensor_bytes < (1ull << 32) &&
           table_bytes < (1ull << 32);
}

template <typename T, bool Backward>
int launch_fast(const FastShape shape, T* out, float* partial, const T* dy, const T* residual, const T* x, const T* w,
                int rows, int hidden, float eps, int blocks, hipStream_t stream, const RopeArgs* rope = nullptr) {
    const float inv_hidden = 1.0f / static_cast<float>(hidden);
    if (rope != nullptr) {
        if (shape.lpr != 16 || shape.k != 1) return fail(CGPTX_RUNTIME, "rmsnorm: no rotary kernel for shape");
        if (rope_dense<T>(rows, hidden, *rope)) {
            hipLaunchKernelGGL((rmsnorm_rope_dense_kernel<T, Backward, kRopeDenseUnroll<Backward>>), dim3(blocks), dim3(kThreads), 0, stream, out,
                               partial, dy, x, w, rows, inv_hidden, eps, *rope);
            return CGPTX_OK;
        }
        hipLaunchKernelGGL((rmsnorm_rows_kernel<T, 16, 1, Backward, true>), dim3(blocks), dim3(kThreads), 0, stream, out,
                           partial, dy, residual, x, w, rows, hidden, inv_hidden, eps, *rope);
        return CGPTX_OK;
    }
#define CGPTX_RMS_CASE(L, KK)                                                                             \
    if (shape.lpr == L && shape.k == KK) {                                                                \
        hipLaunchKernelGGL((rmsnorm_rows_kernel<T, L, KK, Backward>), dim3(blocks), dim3(kThreads), 0,   \
                           stream, out, partial, dy, residual, x, w, rows, hidden, inv_hidden, eps);                \
        return CGPTX_OK;                                                                                  \
    }
    CGPTX_RMS_CASE(16, 1)
    CGPTX_RMS_CASE(32, 1)
    CGPTX_RMS_CASE(64, 1)
    CGPTX_RMS_CASE(64, 2)
    CGPTX_RMS_CASE(64, 4)
#undef CGPTX_RMS_CASE
    return fail(CGPTX_RUNTIME, "rmsnorm: no kernel for shape");
}

// The kernel launch_fast would launch (null when there is none).
template <typename T, bool Backward>
const void* fast_kernel(const FastShape shape, bool rope, bool dense = false) {
    if (rope) {
        if (shape.lpr != 16 || shape.k != 1) return nullptr;
        return dense ? reinterpret_cast<const void*>(&rmsnorm_rope_dense_kernel<T, Backward, kRopeDenseUnroll<Backward>>)
                     : reinterpret_cast<const void*>(&rmsnorm_rows_kernel<T, 16, 1, Backward, true>);
    }
#define CGPTX_RMS_CASE(L, KK) \
    if (shape.lpr == L && shape.k == KK) return reinterpret_cast<const void*>(&rmsnorm_rows_kernel<T, L, KK, Backward>);
    CGPTX_RMS_CASE(16, 1)
    CGPTX_RMS_CASE(32, 1)
    CGPTX_RMS_CASE(64, 1)
    CGPTX_RMS_CASE(64, 2)
    CGPTX_RMS_CASE(64, 4)
#undef CGPTX_RMS_CASE
    return nullptr;
}

// Blocks of `kernel` the device holds at once. The row kernels are grid-stride loops with equal
// shares: launched with more blocks than fit, the surplus would run as a second, mostly idle round.
int resident_blocks(const void* kernel) {
    static std::mutex guard;
    static std::unordered_map<const void*, int> known;
    std::lock_guard<std::mutex> lock(guard);
    auto found = known.find(kernel);
    if (found == known.end()) {
        int per_cu = 0;
        if (kernel == nullptr || hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, kThreads, 0) != hipSuccess ||
            per_cu < 1) {
            (void)hipGetLastError();
            per_cu = 1;
        }
        found = known.emplace(kernel, per_cu).first;
    }
    return found->second * compute_units();
}

int fast_blocks(const FastShape shape, int rows, const void* kernel) {
    const int rpw = kWave / shape.lpr;
    const long groups = (static_cast<long>(rows) + rpw - 1) / rpw;
    const long wanted = (groups + kWavesPerBlock - 1) / kWavesPerBlock;
    const long cap = resident_blocks(kernel);
    return static_cast<int>(wanted < cap ? wanted : cap);
}

int validate(const void* a, const void* b, const void* c, std::size_t rows, std::size_t hidden, float eps, int dtype,
             const char* name) {
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (!std::isfinite(eps) || eps <= 0.0f)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": epsilon must be finite and positive");
    if (a == nullptr || b == nullptr || c == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null tensor");
    if (rows == 0 || hidden == 0) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": empty shape");
    if (rows > static_cast<std::size_t>(std::numeric_limits<int>::max()) ||
        hidden > static_cast<std::size_t>(std::numeric_limits<int>::max()))
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": dimensions exceed supported range");
    return CGPTX_OK;
}

}  // namespace

bool rmsnorm_rope_fusable(const void* a, const void* b, const void* c, const void* weight, const void* cos_cache,
                          const void* sin_cache, std::size_t head_dim, std::size_t rotary_dim, int dtype) {
    if (!valid_dtype(dtype) || head_dim == 0 || head_dim > 4096) return false;
    const std::size_t elem = dtype_size(dtype), vec = 16 / elem;
    bool shape_ok = false;
    dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(static_cast<int>(head_dim));
        shape_ok = shape.lpr == 16 && shape.k == 1;
        return CGPTX_OK;
    });
    const auto half_aligned = [&](const void* p) { return (reinterpret_cast<std::uintptr_t>(p) % (vec / 2 * elem)) == 0; };
    return shape_ok && rotary_dim % vec == 0 && rotary_dim <= head_dim && is_aligned16(a) && is_aligned16(b) &&
           (c == nullptr || is_aligned16(c)) && is_aligned16(weight) && half_aligned(cos_cache) && half_aligned(sin_cache);
}

namespace {
RopeArgs make_rope(const void* cos_cache, const void* sin_cache, std::size_t heads, std::size_t sequence,
                   std::size_t rotary_dim, std::size_t position_offset) {
    return RopeArgs{cos_cache, sin_cache, static_cast<int>(heads), static_cast<int>(sequence), static_cast<int>(rotary_dim),
                    static_cast<int>(position_offset)};
}
}  // namespace

// Memory for a pass's partial sums: from the sink when one is given and has room (the reductions are then recorded
// and run later by the caller), else from the per-stream arena (the reductions then run at once).
int partial_memory(ColumnReduceSink* sink, hipStream_t stream, std::size_t bytes, void** out, bool* deferred) {
    *out = sink != nullptr ? sink->take(bytes) : nullptr;
    *deferred = *out != nullptr;
    return *deferred ? CGPTX_OK : scratch(stream, bytes, out);
}

// dw[h] = column sums of partial[blocks, h]: two small launches now, or an entry in the sink.
template <typename T>
int reduce_columns(ColumnReduceSink* sink, bool deferred, T* dw, float* partial, float* second, int blocks, int h,
                   int slices, int dtype, hipStream_t stream) {
    if (deferred) {
        sink->entries.push_back(ColumnReduceEntry{partial, second, dw, blocks, h, slices, dtype});
        return CGPTX_OK;
    }
    const int reduce_blocks = (h + kWave - 1) / kWave;
    if (slices > 1) {
        hipLaunchKernelGGL(column_partial_fold_kernel, dim3(reduce_blocks, slices), dim3(kThreads), 0, stream, second,
                           partial, blocks, h);
        CGPTX_LAUNCH_CHECK();
        hipLaunchKernelGGL((column_partial_reduce_kernel<T>), dim3(reduce_blocks), dim3(kThreads), 0, stream, dw, second,
                           slices, h, 0);
    } else {
        hipLaunchKernelGGL((column_partial_reduce_kernel<T>), dim3(reduce_blocks), dim3(kThreads), 0, stream, dw, partial,
                           blocks, h, 0);
    }
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

int run_column_reductions(const ColumnReduceEntry* table, int count, int max_hidden, int max_slices, hipStream_t stream) {
    if (count <= 0) return CGPTX_OK;
    const int groups = (max_hidden + kWave - 1) / kWave;
    if (max_slices > 1) {
        hipLaunchKernelGGL(column_partial_fold_table_kernel, dim3(groups, max_slices, count), dim3(kThreads), 0, stream, table);
        CGPTX_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(column_partial_reduce_table_kernel, dim3(groups, count), dim3(kThreads), 0, stream, table);
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

int rmsnorm_rope_forward(void* output, const void* input, const void* weight, const void* cos_cache, const void* sin_cache,
                         std::size_t rows, std::size_t head_dim, std::size_t heads, std::size_t sequence,
                         std::size_t rotary_dim, std::size_t position_offset, float epsilon, int dtype, hipStream_t stream) {
    if (int s = validate(output, input, weight, rows, head_dim, epsilon, dtype, "rmsnorm_rope_forward")) return s;
    if (cos_cache == nullptr || sin_cache == nullptr || heads == 0 || sequence == 0 ||
        !rmsnorm_rope_fusable(output, input, nullptr, weight, cos_cache, sin_cache, head_dim, rotary_dim, dtype))
        return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_rope_forward: shape or alignment not served by the fused pass");
    const int r = static_cast<int>(rows), h = static_cast<int>(head_dim);
    const RopeArgs rope = make_rope(cos_cache, sin_cache, heads, sequence, rotary_dim, position_offset);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(h);
        if (int s = launch_fast<T, false>(shape, static_cast<T*>(output), nullptr, nullptr, nullptr,
                                          static_cast<const T*>(input), static_cast<const T*>(weight), r, h, epsilon,
                                          fast_blocks(shape, r, fast_kernel<T, false>(shape, true, rope_dense<T>(r, h, rope))), stream, &rope))
            return s;
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

int rmsnorm_rope_backward(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                          const void* weight, const void* cos_cache, const void* sin_cache, std::size_t rows,
                          std::size_t head_dim, std::size_t heads, std::size_t sequence, std::size_t rotary_dim,
                          std::size_t position_offset, float epsilon, int dtype, hipStream_t stream, ColumnReduceSink* sink) {
    if (int s = validate(grad_input, grad_output, input, rows, head_dim, epsilon, dtype, "rmsnorm_rope_backward")) return s;
    if (grad_weight == nullptr || weight == nullptr || cos_cache == nullptr || sin_cache == nullptr || heads == 0 ||
        sequence == 0 ||
        !rmsnorm_rope_fusable(grad_input, grad_output, input, weight, cos_cache, sin_cache, head_dim, rotary_dim, dtype))
        return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_rope_backward: shape or alignment not served by the fused pass");
    const int r = static_cast<int>(rows), h = static_cast<int>(head_dim);
    const RopeArgs rope = make_rope(cos_cache, sin_cache, heads, sequence, rotary_dim, position_offset);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(h);
        const int blocks = fast_blocks(shape, r, fast_kernel<T, true>(shape, true, rope_dense<T>(r, h, rope)));
        const int slices = wide_reduce_slices(blocks, h, compute_units());
        void* mem = nullptr;
        bool deferred = false;
        const std::size_t partial_bytes = static_cast<std::size_t>(blocks) * head_dim * sizeof(float);
        if (int s = partial_memory(sink, stream, partial_bytes + static_cast<std::size_t>(slices) * head_dim * sizeof(float), &mem,
                                   &deferred))
            return s;
        auto* partial = static_cast<float*>(mem);
        if (int s = launch_fast<T, true>(shape, static_cast<T*>(grad_input), partial, static_cast<const T*>(grad_output),
                                         nullptr, static_cast<const T*>(input), static_cast<const T*>(weight), r, h, epsilon,
                                         blocks, stream, &rope))
            return s;
        CGPTX_LAUNCH_CHECK();
        auto* second = reinterpret_cast<float*>(static_cast<char*>(mem) + partial_bytes);
        if (int s = reduce_columns<T>(sink, deferred, static_cast<T*>(grad_weight), partial, second, blocks, h, slices, dtype,
                                      stream))
            return s;
        return CGPTX_OK;
    });
}

bool rmsnorm_dual_fusable(const void* a, const void* b, const void* c, const void* d, const void* e, std::size_t hidden,
                          int dtype) {
    if (!valid_dtype(dtype) || hidden == 0 || hidden > (1u << 20)) return false;
    bool shape_ok = false;
    dispatch_dtype(dtype, [&]<typename T>() -> int {
        shape_ok = pick_fast_shape<T>(static_cast<int>(hidden)).lpr != 0;
        return CGPTX_OK;
    });
    return shape_ok && is_aligned16(a) && is_aligned16(b) && is_aligned16(c) && is_aligned16(d) && is_aligned16(e);
}

namespace {
template <typename T, bool Backward>
int launch_dual(const FastShape shape, T* out_a, T* out_f, float* partial_a, float* partial_f, const T* dy_a, const T* dy_f,
                const T* residual, const T* x, const T* w_a, const T* w_f, int rows, int hidden, float eps, int blocks,
                hipStream_t stream) {
    const float inv_hidden = 1.0f / static_cast<float>(hidden);
#define CGPTX_RMS_CASE(L, KK)                                                                                         \
    if (shape.lpr == L && shape.k == KK) {                                                                            \
        hipLaunchKernelGGL((rmsnorm_dual_rows_kernel<T, L, KK, Backward>), dim3(blocks), dim3(kThreads), 0, stream,   \
                           out_a, out_f, partial_a, partial_f, dy_a, dy_f, residual, x, w_a, w_f, rows, hidden,      \
                           inv_hidden, eps);                                                                          \
        return CGPTX_OK;                                                                                              \
    }
    CGPTX_RMS_CASE(16, 1)
    CGPTX_RMS_CASE(32, 1)
    CGPTX_RMS_CASE(64, 1)
    CGPTX_RMS_CASE(64, 2)
    CGPTX_RMS_CASE(64, 4)
#undef CGPTX_RMS_CASE
    return fail(CGPTX_RUNTIME, "rmsnorm: no kernel for shape");
}
}  // namespace

namespace {
template <typename T, bool Backward>
const void* dual_kernel(const FastShape shape) {
#define CGPTX_RMS_CASE(L, KK) \
    if (shape.lpr == L && shape.k == KK) return reinterpret_cast<const void*>(&rmsnorm_dual_rows_kernel<T, L, KK, Backward>);
    CGPTX_RMS_CASE(16, 1)
    CGPTX_RMS_CASE(32, 1)
    CGPTX_RMS_CASE(64, 1)
    CGPTX_RMS_CASE(64, 2)
    CGPTX_RMS_CASE(64, 4)
#undef CGPTX_RMS_CASE
    return nullptr;
}
}  // namespace

int rmsnorm_forward_dual(void* output_a, void* output_f, const void* input, const void* weight_a, const void* weight_f,
                         std::size_t rows, std::size_t hidden, float epsilon, int dtype, hipStream_t stream) {
    if (int s = validate(output_a, output_f, input, rows, hidden, epsilon, dtype, "rmsnorm_forward_dual")) return s;
    if (weight_a == nullptr || weight_f == nullptr ||
        !rmsnorm_dual_fusable(output_a, output_f, input, weight_a, weight_f, hidden, dtype))
        return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_forward_dual: shape or alignment not served by the fused pass");
    const int r = static_cast<int>(rows), h = static_cast<int>(hidden);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(h);
        if (int s = launch_dual<T, false>(shape, static_cast<T*>(output_a), static_cast<T*>(output_f), nullptr, nullptr, nullptr,
                                          nullptr, nullptr, static_cast<const T*>(input), static_cast<const T*>(weight_a),
                                          static_cast<const T*>(weight_f), r, h, epsilon,
                                          fast_blocks(shape, r, dual_kernel<T, false>(shape)), stream))
            return s;
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}

int rmsnorm_backward_dual(void* grad_input, void* grad_weight_a, void* grad_weight_f, const void* grad_output_a,
                          const void* grad_output_f, const void* input, const void* weight_a, const void* weight_f,
                          const void* residual, std::size_t rows, std::size_t hidden, float epsilon, int dtype,
                          hipStream_t stream, ColumnReduceSink* sink) {
    if (int s = validate(grad_input, grad_output_a, input, rows, hidden, epsilon, dtype, "rmsnorm_backward_dual")) return s;
    if (grad_weight_a == nullptr || grad_weight_f == nullptr || weight_a == nullptr || weight_f == nullptr ||
        grad_output_f == nullptr ||
        !rmsnorm_dual_fusable(grad_input, grad_output_a, grad_output_f, input, residual, hidden, dtype) ||
        !is_aligned16(weight_a) || !is_aligned16(weight_f))
        return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_backward_dual: shape or alignment not served by the fused pass");
    const int r = static_cast<int>(rows), h = static_cast<int>(hidden);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(h);
        const int blocks = fast_blocks(shape, r, dual_kernel<T, true>(shape));
        const int slices = wide_reduce_slices(blocks, h, compute_units());
        void* mem = nullptr;
        bool deferred = false;
        const std::size_t partial_bytes = static_cast<std::size_t>(blocks) * hidden * sizeof(float);
        const std::size_t second_bytes = (static_cast<std::size_t>(slices) * hidden * sizeof(float) + 255) & ~std::size_t{255};
        if (int s = partial_memory(sink, stream, 2 * partial_bytes + 2 * second_bytes, &mem, &deferred)) return s;
        auto* partial_a = static_cast<float*>(mem);
        auto* partial_f = reinterpret_cast<float*>(static_cast<char*>(mem) + partial_bytes);
        auto* second_a = reinterpret_cast<float*>(static_cast<char*>(mem) + 2 * partial_bytes);
        auto* second_f = reinterpret_cast<float*>(static_cast<char*>(mem) + 2 * partial_bytes + second_bytes);
        if (int s = launch_dual<T, true>(shape, static_cast<T*>(grad_input), nullptr, partial_a, partial_f,
                                         static_cast<const T*>(grad_output_a), static_cast<const T*>(grad_output_f),
                                         static_cast<const T*>(residual), static_cast<const T*>(input),
                                         static_cast<const T*>(weight_a), static_cast<const T*>(weight_f), r, h, epsilon, blocks,
                                         stream))
            return s;
        CGPTX_LAUNCH_CHECK();
        if (int s = reduce_columns<T>(sink, deferred, static_cast<T*>(grad_weight_a), partial_a, second_a, blocks, h, slices,
                                      dtype, stream))
            return s;
        if (int s = reduce_columns<T>(sink, deferred, static_cast<T*>(grad_weight_f), partial_f, second_f, blocks, h, slices,
                                      dtype, stream))
            return s;
        return CGPTX_OK;
    });
}

namespace {
// Where rmsnorm_backward's partial sums go: the per-stream arena (fixed == nullptr), or a caller-provided block
// of `fixed_bytes` that is never exceeded (a larger need is an error, nothing is allocated).
struct Workspace {
    hipStream_t stream;
    void* fixed;
    std::size_t fixed_bytes;
    ColumnReduceSink* sink = nullptr;  // when given and roomy enough, the weight-gradient reduction is recorded there
    int get(std::size_t bytes, void** out) const {
        if (fixed == nullptr) return scratch(stream, bytes, out);
        if (bytes > fixed_bytes)
            return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_backward_static: the shape needs " + std::to_string(bytes) +
                                                    " bytes of working memory, the built-in block holds " +
                                                    std::to_string(fixed_bytes));
        *out = fixed;
        return CGPTX_OK;
    }
};

int rmsnorm_backward_impl(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                          const void* weight, const void* residual, std::size_t rows, std::size_t hidden,
                          float epsilon, int dtype, hipStream_t stream, const Workspace& workspace) {
    if (int s = validate(grad_input, grad_output, input, rows, hidden, epsilon, dtype, "rmsnorm_backward")) return s;
    if (grad_weight == nullptr || weight == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "rmsnorm_backward: null weight tensor");
    const int r = static_cast<int>(rows), h = static_cast<int>(hidden);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* dx = static_cast<T*>(grad_input);
        auto* res = static_cast<const T*>(residual);
        auto* dw = static_cast<T*>(grad_weight);
        auto* dy = static_cast<const T*>(grad_output);
        auto* x = static_cast<const T*>(input);
        auto* w = static_cast<const T*>(weight);
        const FastShape shape = pick_fast_shape<T>(h);
        const bool aligned = is_aligned16(dx) && is_aligned16(dy) && is_aligned16(x) && is_aligned16(w) && is_aligned16(res);
        const int reduce_blocks = (h + kWave - 1) / kWave;
        if (shape.lpr != 0 && aligned) {
            const int blocks = fast_blocks(shape, r, fast_kernel<T, true>(shape, false));
            const int slices = wide_reduce_slices(blocks, h, compute_units());
            void* mem = nullptr;
            const std::size_t partial_bytes = static_cast<std::size_t>(blocks) * hidden * sizeof(float);
            const std::size_t bytes = partial_bytes + static_cast<std::size_t>(slices) * hidden * sizeof(float);
            if (workspace.sink != nullptr) mem = workspace.sink->take(bytes);
            const bool deferred = mem != nullptr;
            if (!deferred) {
                if (int s = workspace.get(bytes, &mem)) return s;
            }
            auto* partial = static_cast<float*>(mem);
            if (int s = launch_fast<T, true>(shape, dx, partial, dy, res, x, w, r, h, epsilon, blocks, stream)) return s;
            CGPTX_LAUNCH_CHECK();
            auto* second = reinterpret_cast<float*>(static_cast<char*>(mem) + partial_bytes);
            return reduce_columns<T>(workspace.sink, deferred, dw, partial, second, blocks, h, slices, dtype, stream);
        }
        const int slices = r < 256 ? 1 : (r < 65536 ? 64 : 256);
        const int rows_per_slice = (r + slices - 1) / slices;
        void* mem = nullptr;
        const std::size_t inv_bytes = (rows * sizeof(float) + 255) & ~std::size_t{255};
        if (int s = workspace.get(inv_bytes + static_cast<std::size_t>(slices) * hidden * sizeof(float), &mem))
            return s;
        auto* inv_rms = static_cast<float*>(mem);
        auto* partial = reinterpret_cast<float*>(static_cast<char*>(mem) + inv_bytes);
        const int row_blocks = r < compute_units() * 8 ? r : compute_units() * 8;
        hipLaunchKernelGGL((rmsnorm_row_generic_kernel<T, true>), dim3(row_blocks), dim3(kThreads), 0, stream, dx,
                           inv_rms, dy, x, w, r, h, 1.0f / static_cast<float>(h), epsilon);
        CGPTX_LAUNCH_CHECK();
        hipLaunchKernelGGL((rmsnorm_dgamma_generic_kernel<T>), dim3(reduce_blocks, slices), dim3(kThreads), 0, stream,
                           partial, dy, x, inv_rms, r, h, rows_per_slice);
        CGPTX_LAUNCH_CHECK();
        hipLaunchKernelGGL((column_partial_reduce_kernel<T>), dim3(reduce_blocks), dim3(kThreads), 0, stream, dw,
                           partial, slices, h, 0);
        CGPTX_LAUNCH_CHECK();
        if (res != nullptr) return cgptx_add(dx, dx, res, rows * hidden, dtype, stream);
        return CGPTX_OK;
    });
}
}  // namespace

// What one backward pass takes from a ColumnReduceSink (0 when the shape runs on kernels that do not defer their
// reduction). The same arithmetic as in the passes below; a caller sizes its sink with it before the first pass.
std::size_t rmsnorm_backward_sink_bytes(NormPass pass, std::size_t rows, std::size_t hidden, int dtype) {
    if (!valid_dtype(dtype) || rows == 0 || hidden == 0 || rows > (1u << 30) || hidden > (1u << 20)) return 0;
    const int r = static_cast<int>(rows), h = static_cast<int>(hidden);
    std::size_t bytes = 0;
    dispatch_dtype(dtype, [&]<typename T>() -> int {
        const FastShape shape = pick_fast_shape<T>(h);
        if (shape.lpr == 0) return CGPTX_OK;
        const void* kernel = pass == NormPass::dual ? dual_kernel<T, true>(shape) : fast_kernel<T, true>(shape, pass == NormPass::with_rope);
        if (kernel == nullptr) return CGPTX_OK;
        int blocks = fast_blocks(shape, r, kernel);
        int slices = wide_reduce_slices(blocks, h, compute_units());
        if (pass == NormPass::with_rope) {
            // The pass picks between two kernels by properties of its rotary tables that are not known here: room
            // for whichever of them takes more.
            const int other = fast_blocks(shape, r, fast_kernel<T, true>(shape, true, true));
            const int other_slices = wide_reduce_slices(other, h, compute_units());
            blocks = other > blocks ? other : blocks;
            slices = other_slices > slices ? other_slices : slices;
        }
        const std::size_t partial_bytes = static_cast<std::size_t>(blocks) * hidden * sizeof(float);
        const std::size_t second_bytes = static_cast<std::size_t>(slices) * hidden * sizeof(float);
        bytes = pass == NormPass::dual ? 2 * partial_bytes + 2 * ((second_bytes + 255) & ~std::size_t{255}) : partial_bytes + second_bytes;
        bytes = (bytes + 255) & ~std::size_t{255};  // ColumnReduceSink::take hands out multiples of 256
        return CGPTX_OK;
    });
    return bytes;
}

int rmsnorm_backward_residual(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                              const void* weight, const void* residual, std::size_t rows, std::size_t hidden,
                              float epsilon, int dtype, hipStream_t stream, ColumnReduceSink* sink) {
    return rmsnorm_backward_impl(grad_input, grad_weight, grad_output, input, weight, residual, rows, hidden, epsilon, dtype,
                                 stream, Workspace{stream, nullptr, 0, sink});
}

}  // namespace cgptx

// ---- rmsnorm_backward without any allocation ------------------------------------------------------------------
// The partial sums of the weight gradient live in a block that is part of the library's device image: every
// GPU the library runs on holds its own copy, at its own address, until the process ends. Host code reaches it
// only through the address hipGetSymbolAddress returns for the current device (the array's name is a host-side
// stand-in, not a device address), looked up once per device and kept.
namespace {
constexpr std::size_t kStaticScratchBytes = std::size_t{16} << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_static_scratch_mutex;
void* g_static_scratch_address[kMaxDevices] = {};  // per device; null until first use on that device

int static_scratch_address(void** out) {
    int device = 0;
    CGPTX_HIP(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return cgptx::fail(CGPTX_RUNTIME, "rmsnorm_backward_static: device index out of range");
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_address[device] == nullptr) {
        void* address = nullptr;
        CGPTX_HIP(hipGetSymbolAddress(&address, HIP_SYMBOL(g_static_scratch)));
        if (address == nullptr) return cgptx::fail(CGPTX_RUNTIME, "rmsnorm_backward_static: no device address for the working block");
        g_static_scratch_address[device] = address;
    }
    *out = g_static_scratch_address[device];
    return CGPTX_OK;
}
}  // namespace

extern "C" int cgptx_rmsnorm_backward_static(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                                             const void* weight, size_t rows, size_t hidden, float epsilon, int dtype,
                                             cgptx_stream stream_) {
    void* block = nullptr;
    if (int s = static_scratch_address(&block)) return s;
    auto stream = static_cast<hipStream_t>(stream_);
    // Nothing in the block has to start at zero: the row kernel writes every partial-sum row it is launched
    // with before the reduction kernels, later on the same stream, read them.
    return cgptx::rmsnorm_backward_impl(grad_input, grad_weight, grad_output, input, weight, nullptr, rows, hidden, epsilon,
                                        dtype, stream, cgptx::Workspace{stream, block, kStaticScratchBytes});
}

extern "C" int cgptx_rmsnorm_backward(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                                      const void* weight, size_t rows, size_t hidden, float epsilon, int dtype,
                                      cgptx_stream stream) {
    return cgptx::rmsnorm_backward_residual(grad_input, grad_weight, grad_output, input, weight, nullptr, rows, hidden,
                                            epsilon, dtype, static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_rmsnorm_forward(void* output, const void* input, const void* weight, size_t rows, size_t hidden,
                                     float epsilon, int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    if (int s = validate(output, input, weight, rows, hidden, epsilon, dtype, "rmsnorm_forward")) return s;
    auto stream = static_cast<hipStream_t>(stream_);
    const int r = static_cast<int>(rows), h = static_cast<int>(hidden);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        auto* y = static_cast<T*>(output);
        auto* x = static_cast<const T*>(input);
        auto* w = static_cast<const T*>(weight);
        const FastShape shape = pick_fast_shape<T>(h);
        if (shape.lpr != 0 && is_aligned16(y) && is_aligned16(x) && is_aligned16(w)) {
            const int blocks = fast_blocks(shape, r, fast_kernel<T, false>(shape, false));
            if (int s = launch_fast<T, false>(shape, y, nullptr, nullptr, nullptr, x, w, r, h, epsilon, blocks, stream)) return s;
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        }
        const int row_blocks = r < compute_units() * 8 ? r : compute_units() * 8;
        hipLaunchKernelGGL((rmsnorm_row_generic_kernel<T, false>), dim3(row_blocks), dim3(kThreads), 0, stream, y,
                           nullptr, nullptr, x, w, r, h, 1.0f / static_cast<float>(h), epsilon);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}
