// Causal grouped-query flash attention for gfx950: forward with log-sum-exp,
// and the backward (delta, dQ, dK/dV) on the matrix cores.
//
// Reference semantics: include/ops/attention.h:47-78, include/ops/backward/attention_backward.h:24-70,
// formulas of src/ops/cpu/backward/attention_backward_cpu.cpp:206-280:
//   P = exp(scale·QKᵀ − LSE) (key j visible to query i iff j <= offset + i when causal),
//   delta = rowsum(dO∘O), dS = P∘(dO·Vᵀ − delta), dQ = scale·dS·K,
//   dK = scale·Σ_{h in group} dSᵀ·Q, dV = Σ_{h in group} Pᵀ·dO.
//
// Layout idea shared by the three MFMA kernels (v_mfma_f32_32x32x16, 64 lanes):
// the score tile is always produced so that the *stationary* index of the kernel
// is the lane and the *streamed* index lives in the lane's 16 accumulator
// registers. Row statistics (max, sum, LSE, delta) of the stationary index are then
// lane-private scalars, and the converted accumulator registers are, as they are,
// the k-operand of the second product (P·V, dS·K, Pᵀ·dO, dSᵀ·Q) — nothing is
// written back to LDS between the two products. The other operand of the second
// product needs the streamed index as its contraction index while the tile sits in
// LDS with the head dimension contiguous; ds_read_b64_tr_b16 delivers exactly that
// fragment (4 streamed rows x 16 head-dim columns per 16 lanes) in the same
// {0-3, 8-11 | 4-7, 12-15} row order the accumulator registers have.
//
//   forward : block = 128 queries of one (batch, q-head), wave = 32 queries;
//             streams 64-key K/V tiles through LDS; Sᵀ = K·Qᵀ, Oᵀ += Vᵀ·Pᵀ.
//   dQ      : same shape; Sᵀ = K·Qᵀ, dPᵀ = V·dOᵀ, dQᵀ += Kᵀ·dSᵀ.
//   dK/dV   : block = 128 keys of one (batch, kv-head), wave = 32 keys, K/V
//             fragments live in registers; streams 64-query Q/dO tiles of every
//             q-head of the group through LDS, so the group sum happens in the
//             accumulators: no atomics, results independent of scheduling.
//             S = Q·Kᵀ, dP = dO·Vᵀ, dVᵀ += dOᵀ·P, dKᵀ += Qᵀ·dS.
// Causal tiles above the diagonal are skipped; ragged sequence ends are masked.
// Two families implement this scheme: the register-staged kernels (templated on the padded head
// dimension 32 / 64 / 128) and, further down, the LDS-direct kernels (padded width 128), which
// serve every call whose operands fit 32-bit offsets.
#include "common.hpp"

#include <cmath>
#include <cstdlib>
#include <limits>
#include <utility>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kBlockRows = 128;  // stationary rows per block (32 per wave)
constexpr int kStream = 64;      // streamed rows per LDS tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

using acc_t = vec_t<float, 16>;
using s16x4 = vec_t<short, 4>;

template <typename T>
struct Mma;
// The compiler places result and addend (this file is built with MFMA results in vector registers, where the
// softmax arithmetic reads them without a copy).
template <>
struct Mma<bf16_t> {
    using frag = vec_t<bf16_t, 8>;
    __device__ static __forceinline__ acc_t run(frag a, frag b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mma<f16_t> {
    using frag = vec_t<f16_t, 8>;
    __device__ static __forceinline__ acc_t run(frag a, frag b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

struct Params {
    void* out0;  // forward: O      | dq: dQ | dkv: dK
    void* out1;  // forward: unused |        | dkv: dV
    float* lse_out;
    const void* q;
    const void* k;
    const void* v;
    const void* dout;
    const float* lse;
    const float* delta;
    int batch, qs, ks, hq, hkv, d;
    float scale;
    int causal, offset, accumulate;
    int paired;  // dK/dV, LDS-direct family: a workgroup takes key blocks (i, last - i) instead of one
};

template <int DP>
constexpr int lds_stride() { return DP + 8; }

// Register-staged copy of a [ROWS x DP] tile of a [.., seq, heads, d] tensor into LDS (row-major,
// stride DP+8): element (r, c) comes from base[(row0 + r) * row_stride + c]. load() only issues
// the 128-bit global loads (rows past the end are clamped to a valid address and zeroed by a
// select, so there is no branch and the loads stay in flight); store() writes them to LDS later,
// after the MFMAs of the previous tile.
template <typename T, int ROWS, int DP>
struct TileRegs {
    static constexpr int kChunksPerRow = DP / 8;
    static constexpr int kPerThread = ROWS * kChunksPerRow / kThreads;
    using chunk_t = vec_t<unsigned int, 4>;
    chunk_t regs[kPerThread];
    int row0_ = 0, row_limit_ = 0, d_ = 0;

    __device__ __forceinline__ void load(const T* base, long row_stride, int row0, int row_limit, int d) {
        row0_ = row0;
        row_limit_ = row_limit;
        d_ = d;
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int c = threadIdx.x + i * kThreads;
            const int r = c / kChunksPerRow, col = (c % kChunksPerRow) * 8;
            const int safe_row = min(row0 + r, row_limit - 1);
            const int safe_col = min(col, d - 8);
            regs[i] = *reinterpret_cast<const chunk_t*>(base + static_cast<long>(safe_row) * row_stride + safe_col);
        }
    }
    // The zeroing of out-of-range chunks happens here, not in load(), so that nothing waits for
    // the loaded data before the tile is actually needed.
    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int c = threadIdx.x + i * kThreads;
            const int r = c / kChunksPerRow, col = (c % kChunksPerRow) * 8;
            const bool live = row0_ + r < row_limit_ && col < d_;
            chunk_t value;
#pragma unroll
            for (int e = 0; e < 4; ++e) value[e] = live ? regs[i][e] : 0u;
            *reinterpret_cast<chunk_t*>(lds + r * lds_stride<DP>() + col) = value;
        }
    }
};

// Fragment with the head dimension as contraction index, read straight from LDS:
// lane -> tile row (row0 + lane%32), elements d = 16*step + 8*(lane/32) .. +7.
template <typename T, int DP>
__device__ __forceinline__ typename Mma<T>::frag direct_frag(const T* lds, int row0, int step) {
    const int lane = threadIdx.x & 63;
    return *reinterpret_cast<const typename Mma<T>::frag*>(lds + (row0 + (lane & 31)) * lds_stride<DP>() + step * 16 +
                                                            (lane >> 5) * 8);
}

// Same fragment taken from global memory (for the operand that stays in registers).
template <typename T>
__device__ __forceinline__ typename Mma<T>::frag global_frag(const T* row_ptr, bool live, int step, int d) {
    const int lane = threadIdx.x & 63;
    const int col = step * 16 + (lane >> 5) * 8;
    using frag = typename Mma<T>::frag;
    if (live && col < d) return *reinterpret_cast<const frag*>(row_ptr + col);
    return frag(static_cast<T>(0.0f));
}

// Fragment with tile rows as contraction index (transposing LDS read): lane -> column
// d0 + lane%32; elements = rows kbase + {0-3, 8-11} (lanes 0-31) or {4-7, 12-15} (lanes 32-63).
template <typename T, int DP>
__device__ __forceinline__ typename Mma<T>::frag transposed_frag(const T* lds, int kbase, int d0) {
    const int lane = threadIdx.x & 63;
    const int row = kbase + (lane >> 5) * 4 + ((lane & 15) >> 2);
    const int col = d0 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
    const T* p = lds + row * lds_stride<DP>() + col;
    using lds_ptr = __attribute__((address_space(3))) s16x4*;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(p + 8 * lds_stride<DP>()));
    vec_t<short, 8> both;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        both[e] = lo[e];
        both[4 + e] = hi[e];
    }
    return __builtin_bit_cast(typename Mma<T>::frag, both);
}

// Accumulator registers 8*step .. 8*step+7 as a 16-bit k-operand.
template <typename T>
__device__ __forceinline__ typename Mma<T>::frag acc_frag(const acc_t& acc, int step) {
    vec_t<float, 8> f;
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = acc[8 * step + e];
    return vec_from_f32<T, 8>(f);
}

// Streamed index of accumulator register i: 8*(i/4) + 4*(lane/32) + i%4.
__device__ __forceinline__ int acc_row(int i) { return 8 * (i >> 2) + 4 * ((threadIdx.x & 63) >> 5) + (i & 3); }

// Query block, head and batch entry of a workgroup of the forward and dQ kernels (grid: query blocks
// x heads x batch). Workgroups start in the order of their linear id, as slots become free, and go
// to the 8 XCDs round-robin. Under a causal mask a query block's work grows with its position, so
// the linear id is read position-major with the last (longest) query blocks first: the work that
// is handed out last is the shortest, which keeps the tail of the launch short, and every XCD
// receives the same mix of lengths.
// Each XCD has its own L2, and the workgroups that stream the same K and V are the heads of one GQA group
// at every query position: when the (batch, kv-head) pairs divide evenly over the 8 XCDs, XCD x (linear id
// mod 8) takes pairs x, x + 8, ... and walks positions (longest first) x its pairs x the heads of the group,
// so that the workgroups resident on an XCD at any time share a few K/V streams instead of each bringing
// its own from memory.
struct BlockCoordinates {
    int q_block;  // first query row
    int h, b;
};
__device__ __forceinline__ BlockCoordinates block_coordinates(int hkv) {
    constexpr unsigned int kXcds = 8;
    const unsigned int linear = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    const unsigned int heads = gridDim.y, batch = gridDim.z, positions = gridDim.x;
    const unsigned int pairs = batch * static_cast<unsigned int>(hkv), group = heads / static_cast<unsigned int>(hkv);
    BlockCoordinates c;
    if (pairs % kXcds == 0) {
        const unsigned int xcd = linear % kXcds, local = linear / kXcds;
        const unsigned int per_position = (pairs / kXcds) * group;
        const unsigned int position = local / per_position, rest = local - position * per_position;
        const unsigned int pair = xcd + kXcds * (rest / group), head_in_group = rest % group;
        c.q_block = static_cast<int>(positions - 1 - position) * kBlockRows;
        c.b = static_cast<int>(pair / static_cast<unsigned int>(hkv));
        c.h = static_cast<int>((pair % static_cast<unsigned int>(hkv)) * group + head_in_group);
        return c;
    }
    const unsigned int per_position = heads * batch;
    const unsigned int position = linear / per_position, rest = linear - position * per_position;
    c.q_block = static_cast<int>(positions - 1 - position) * kBlockRows;
    c.h = static_cast<int>(rest % heads);
    c.b = static_cast<int>(rest / heads);
    return c;
}

// ------------------------------------------------------------------- forward
template <typename T, int DP>
__global__ __launch_bounds__(kThreads) void attention_forward_kernel(Params p) {
    constexpr int STEPS = DP / 16, DT = DP / 32;
    __shared__ __align__(16) T k_lds[kStream * lds_stride<DP>()];
    __shared__ __align__(16) T v_lds[kStream * lds_stride<DP>()];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const BlockCoordinates where = block_coordinates(p.hkv);
    const int b = where.b, h = where.h, kvh = h / (p.hq / p.hkv);
    const int q_block = where.q_block;
    const int q_row = q_block + wave * 32 + (lane & 31);
    const bool q_live = q_row < p.qs;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const T* q_ptr = static_cast<const T*>(p.q) + (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
    const T* k_base = static_cast<const T*>(p.k) + static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;
    const T* v_base = static_cast<const T*>(p.v) + static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;

    typename Mma<T>::frag qf[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) qf[s] = global_frag<T>(q_ptr, q_live, s, p.d);

    acc_t o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) o[t] = acc_t(0.0f);
    float m = -INFINITY, l = 0.0f;
    const float scale2 = p.scale * kLog2e;
    const int last_q_block = min(q_block + kBlockRows, p.qs) - 1;
    const int k_end = p.causal ? min(p.ks, p.offset + last_q_block + 1) : p.ks;
    const int wave_last_q = min(q_block + wave * 32 + 31, p.qs - 1);
    const int q_limit = p.causal ? p.offset + q_row : p.ks;  // largest visible key of this lane's query

    TileRegs<T, kStream, DP> k_regs, v_regs;
    if (k_end > 0) {
        k_regs.load(k_base, kv_stride, 0, p.ks, p.d);
        v_regs.load(v_base, kv_stride, 0, p.ks, p.d);
    }
    for (int k0 = 0; k0 < k_end; k0 += kStream) {
        __syncthreads();  // every wavefront is done reading the previous tile
        k_regs.store(k_lds);
        v_regs.store(v_lds);
        __syncthreads();
        if (k0 + kStream < k_end) {  // next tile's loads fly during this tile's MFMAs
            k_regs.load(k_base, kv_stride, k0 + kStream, p.ks, p.d);
            v_regs.load(v_base, kv_stride, k0 + kStream, p.ks, p.d);
        }
        if (q_block + wave * 32 >= p.qs) continue;
        if (p.causal && k0 > p.offset + wave_last_q) continue;
        acc_t st[2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            st[sub] = acc_t(0.0f);
            typename Mma<T>::frag ka[STEPS];  // all LDS reads first, then the MFMA chain
#pragma unroll
            for (int s = 0; s < STEPS; ++s) ka[s] = direct_frag<T, DP>(k_lds, sub * 32, s);
            __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of the MFMA chain
#pragma unroll
            for (int s = 0; s < STEPS; ++s) st[sub] = Mma<T>::run(ka[s], qf[s], st[sub]);
        }
        float tile_max = -INFINITY;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = k0 + sub * 32 + acc_row(i);
                const bool visible = key < p.ks && key <= q_limit;
                const float s = visible ? st[sub][i] * scale2 : -INFINITY;
                st[sub][i] = s;
                tile_max = fmaxf(tile_max, s);
            }
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, kWave));
        const float m_new = fmaxf(m, tile_max);
        const float alpha = m_new == -INFINITY ? 1.0f : exp2f(m - m_new);
        float tile_sum = 0.0f;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = m_new == -INFINITY ? 0.0f : exp2f(st[sub][i] - m_new);
                st[sub][i] = e;
                tile_sum += e;
            }
        }
        l = l * alpha + tile_sum;
        m = m_new;
#pragma unroll
        for (int t = 0; t < DT; ++t) o[t] *= alpha;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const typename Mma<T>::frag pf = acc_frag<T>(st[sub], s);
                typename Mma<T>::frag vt[DT];
#pragma unroll
                for (int t = 0; t < DT; ++t) vt[t] = transposed_frag<T, DP>(v_lds, sub * 32 + s * 16, t * 32);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < DT; ++t) o[t] = Mma<T>::run(vt[t], pf, o[t]);
            }
        }
    }
    l += __shfl_xor(l, 32, kWave);
    if (!q_live) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    T* o_ptr = static_cast<T*>(p.out0) + (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
            if (d0 >= p.d) continue;
            vec_t<float, 4> v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = o[t][4 * g + e] * inv;
            store_vec<T, 4>(o_ptr + d0, vec_from_f32<T, 4>(v));
        }
    }
    if (p.lse_out != nullptr && lane < 32)
        p.lse_out[(static_cast<long>(b) * p.qs + q_row) * p.hq + h] = (m + log2f(l)) * kLn2;
}

// --------------------------------------------------------------------- delta
// delta[b, t, h] = Σ_d dO·O (and LSE·log2 e next to it), one group of LPR lanes per row, 128-bit loads.
template <typename T, int LPR>
__global__ __launch_bounds__(kThreads) void attention_delta_kernel(float* __restrict__ delta,
                                                                  float* __restrict__ lse2,
                                                                  const float* __restrict__ lse,
                                                                  const T* __restrict__ dout,
                                                                  const T* __restrict__ out, long rows, int d) {
    const long row = (static_cast<long>(blockIdx.x) * kThreads + threadIdx.x) / LPR;
    const int sub = threadIdx.x % LPR;
    float sum = 0.0f;
    if (row < rows && sub * 8 < d) {
        const vec_t<float, 8> a = vec_to_f32<T, 8>(load_vec<T, 8>(dout + row * d + sub * 8));
        const vec_t<float, 8> b = vec_to_f32<T, 8>(load_vec<T, 8>(out + row * d + sub * 8));
#pragma unroll
        for (int e = 0; e < 8; ++e) sum = fmaf(a[e], b[e], sum);
    }
    sum = wave_sum<LPR>(sum);
    if (row < rows && sub == 0) {
        delta[row] = sum;
        lse2[row] = lse[row] * kLog2e;  // the exponent the wide backward kernels subtract, in base 2
    }
}

// ------------------------------------------------------------------------ dQ
template <typename T, int DP>
__global__ __launch_bounds__(kThreads) void attention_dq_kernel(Params p) {
    constexpr int STEPS = DP / 16, DT = DP / 32;
    __shared__ __align__(16) T k_lds[kStream * lds_stride<DP>()];
    __shared__ __align__(16) T v_lds[kStream * lds_stride<DP>()];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const BlockCoordinates where = block_coordinates(p.hkv);
    const int b = where.b, h = where.h, kvh = h / (p.hq / p.hkv);
    const int q_block = where.q_block;
    const int q_row = q_block + wave * 32 + (lane & 31);
    const bool q_live = q_row < p.qs;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const long q_offset = (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
    const T* k_base = static_cast<const T*>(p.k) + static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;
    const T* v_base = static_cast<const T*>(p.v) + static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;

    typename Mma<T>::frag qf[STEPS], dof[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        qf[s] = global_frag<T>(static_cast<const T*>(p.q) + q_offset, q_live, s, p.d);
        dof[s] = global_frag<T>(static_cast<const T*>(p.dout) + q_offset, q_live, s, p.d);
    }
    const long stat_index = (static_cast<long>(b) * p.qs + q_row) * p.hq + h;
    const float lse2 = q_live ? p.lse[stat_index] * kLog2e : 0.0f;
    const float delta = q_live ? p.delta[stat_index] : 0.0f;

    acc_t dq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) dq[t] = acc_t(0.0f);
    const float scale2 = p.scale * kLog2e;
    const int last_q_block = min(q_block + kBlockRows, p.qs) - 1;
    const int k_end = p.causal ? min(p.ks, p.offset + last_q_block + 1) : p.ks;
    const int wave_last_q = min(q_block + wave * 32 + 31, p.qs - 1);
    const int q_limit = p.causal ? p.offset + q_row : p.ks;

    TileRegs<T, kStream, DP> k_regs, v_regs;
    if (k_end > 0) {
        k_regs.load(k_base, kv_stride, 0, p.ks, p.d);
        v_regs.load(v_base, kv_stride, 0, p.ks, p.d);
    }
    for (int k0 = 0; k0 < k_end; k0 += kStream) {
        __syncthreads();  // every wavefront is done reading the previous tile
        k_regs.store(k_lds);
        v_regs.store(v_lds);
        __syncthreads();
        if (k0 + kStream < k_end) {  // next tile's loads fly during this tile's MFMAs
            k_regs.load(k_base, kv_stride, k0 + kStream, p.ks, p.d);
            v_regs.load(v_base, kv_stride, k0 + kStream, p.ks, p.d);
        }
        if (q_block + wave * 32 >= p.qs) continue;
        if (p.causal && k0 > p.offset + wave_last_q) continue;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            acc_t st(0.0f), dpt(0.0f);
            typename Mma<T>::frag ka[STEPS], va[STEPS];  // all LDS reads first, then two independent MFMA chains
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                ka[s] = direct_frag<T, DP>(k_lds, sub * 32, s);
                va[s] = direct_frag<T, DP>(v_lds, sub * 32, s);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of the MFMA chains
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                st = Mma<T>::run(ka[s], qf[s], st);
                dpt = Mma<T>::run(va[s], dof[s], dpt);
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = k0 + sub * 32 + acc_row(i);
                const bool visible = q_live && key < p.ks && key <= q_limit;
                const float prob = visible ? exp2f(st[i] * scale2 - lse2) : 0.0f;
                st[i] = prob * (dpt[i] - delta);
            }
#pragma unroll
            for (int s = 0; s < 2; ++s) {
                const typename Mma<T>::frag dsf = acc_frag<T>(st, s);
                typename Mma<T>::frag kt[DT];
#pragma unroll
                for (int t = 0; t < DT; ++t) kt[t] = transposed_frag<T, DP>(k_lds, sub * 32 + s * 16, t * 32);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int t = 0; t < DT; ++t) dq[t] = Mma<T>::run(kt[t], dsf, dq[t]);
            }
        }
    }
    if (!q_live) return;
    T* out = static_cast<T*>(p.out0) + q_offset;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
            if (d0 >= p.d) continue;
            vec_t<float, 4> v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = dq[t][4 * g + e] * p.scale;
            if (p.accumulate) v += vec_to_f32<T, 4>(load_vec<T, 4>(out + d0));
            store_vec<T, 4>(out + d0, vec_from_f32<T, 4>(v));
        }
    }
}

// --------------------------------------------------------------------- dK/dV
template <typename T, int DP>
__global__ __launch_bounds__(kThreads) void attention_dkv_kernel(Params p) {
    constexpr int STEPS = DP / 16, DT = DP / 32;
    __shared__ __align__(16) T q_lds[kStream * lds_stride<DP>()];
    __shared__ __align__(16) T do_lds[kStream * lds_stride<DP>()];
    __shared__ float lse_lds[kStream];
    __shared__ float delta_lds[kStream];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int b = blockIdx.z, kvh = blockIdx.y, group = p.hq / p.hkv;
    const int k_block = blockIdx.x * kBlockRows;
    const int k_row = k_block + wave * 32 + (lane & 31);
    const bool k_live = k_row < p.ks;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const long k_offset = (static_cast<long>(b) * p.ks + k_row) * kv_stride + kvh * p.d;

    typename Mma<T>::frag kf[STEPS], vf[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        kf[s] = global_frag<T>(static_cast<const T*>(p.k) + k_offset, k_live, s, p.d);
        vf[s] = global_frag<T>(static_cast<const T*>(p.v) + k_offset, k_live, s, p.d);
    }
    acc_t dk[DT], dv[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        dk[t] = acc_t(0.0f);
        dv[t] = acc_t(0.0f);
    }
    const float scale2 = p.scale * kLog2e;
    // First query that can see any key of this block / of this wave.
    const int q_begin = p.causal ? max(0, k_block - p.offset) / kStream * kStream : 0;
    const int wave_first_key = k_block + wave * 32;

    // The (head of the group, query tile) pairs form one flat sequence so that the next tile can be
    // prefetched across the head boundary.
    const int tiles_per_head = q_begin < p.qs ? (p.qs - q_begin + kStream - 1) / kStream : 0;
    const int total_tiles = tiles_per_head * group;
    const T* q_batch = static_cast<const T*>(p.q) + static_cast<long>(b) * p.qs * q_stride;
    const T* do_batch = static_cast<const T*>(p.dout) + static_cast<long>(b) * p.qs * q_stride;
    TileRegs<T, kStream, DP> q_regs, do_regs;
    float lse_reg = 0.0f, delta_reg = 0.0f;
    auto prefetch = [&](int tile) {
        const int h = kvh * group + tile / tiles_per_head;
        const int q0 = q_begin + (tile % tiles_per_head) * kStream;
        q_regs.load(q_batch + h * p.d, q_stride, q0, p.qs, p.d);
        do_regs.load(do_batch + h * p.d, q_stride, q0, p.qs, p.d);
        if (threadIdx.x < kStream) {
            const int q = min(q0 + static_cast<int>(threadIdx.x), p.qs - 1);
            const long index = (static_cast<long>(b) * p.qs + q) * p.hq + h;
            lse_reg = p.lse[index] * kLog2e;
            delta_reg = p.delta[index];
        }
    };
    if (total_tiles > 0) prefetch(0);
    for (int tile = 0; tile < total_tiles; ++tile) {
        {
            const int q0 = q_begin + (tile % tiles_per_head) * kStream;
            __syncthreads();  // every wavefront is done reading the previous tile
            q_regs.store(q_lds);
            do_regs.store(do_lds);
            if (threadIdx.x < kStream) {
                lse_lds[threadIdx.x] = lse_reg;
                delta_lds[threadIdx.x] = delta_reg;
            }
            __syncthreads();
            if (tile + 1 < total_tiles) prefetch(tile + 1);
            if (wave_first_key >= p.ks) continue;
            // every query of the tile sees at most keys <= offset + q0 + 63
            if (p.causal && wave_first_key > p.offset + q0 + kStream - 1) continue;
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                acc_t s_acc(0.0f), dp_acc(0.0f);
                typename Mma<T>::frag qa[STEPS], da[STEPS];  // all LDS reads first, then two MFMA chains
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    qa[s] = direct_frag<T, DP>(q_lds, sub * 32, s);
                    da[s] = direct_frag<T, DP>(do_lds, sub * 32, s);
                }
                __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of the MFMA chains
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    s_acc = Mma<T>::run(qa[s], kf[s], s_acc);
                    dp_acc = Mma<T>::run(da[s], vf[s], dp_acc);
                }
#pragma unroll
                for (int i = 0; i < 16; ++i) {
                    const int local = sub * 32 + acc_row(i);
                    const int q = q0 + local;
                    const bool visible = k_live && q < p.qs && (!p.causal || k_row <= p.offset + q);
                    const float lse_q = lse_lds[local], delta_q = delta_lds[local];  // unconditional reads
                    const float e = exp2f(s_acc[i] * scale2 - lse_q);
                    const float prob = visible ? e : 0.0f;
                    s_acc[i] = prob;
                    dp_acc[i] = prob * (dp_acc[i] - delta_q);
                }
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const typename Mma<T>::frag pf = acc_frag<T>(s_acc, s);
                    const typename Mma<T>::frag dsf = acc_frag<T>(dp_acc, s);
                    typename Mma<T>::frag dot[DT], qt[DT];
#pragma unroll
                    for (int t = 0; t < DT; ++t) {
                        dot[t] = transposed_frag<T, DP>(do_lds, sub * 32 + s * 16, t * 32);
                        qt[t] = transposed_frag<T, DP>(q_lds, sub * 32 + s * 16, t * 32);
                    }
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int t = 0; t < DT; ++t) {
                        dv[t] = Mma<T>::run(dot[t], pf, dv[t]);
                        dk[t] = Mma<T>::run(qt[t], dsf, dk[t]);
                    }
                }
            }
        }
    }
    if (!k_live) return;
    T* dk_out = static_cast<T*>(p.out0) + k_offset;
    T* dv_out = static_cast<T*>(p.out1) + k_offset;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
            if (d0 >= p.d) continue;
            vec_t<float, 4> a, c;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a[e] = dk[t][4 * g + e] * p.scale;
                c[e] = dv[t][4 * g + e];
            }
            if (p.accumulate) {
                a += vec_to_f32<T, 4>(load_vec<T, 4>(dk_out + d0));
                c += vec_to_f32<T, 4>(load_vec<T, 4>(dv_out + d0));
            }
            store_vec<T, 4>(dk_out + d0, vec_from_f32<T, 4>(a));
            store_vec<T, 4>(dv_out + d0, vec_from_f32<T, 4>(c));
        }
    }
}

// ============================================================================================
// LDS-direct family (padded width W = 128, or 64 for head dimensions up to 64): the streamed tiles
// go from global memory straight into LDS with buffer_load ... lds — no staging registers, no LDS
// stores, no address arithmetic in the loop (one loop-invariant per-lane offset, the tile position
// is a scalar offset), rows past the end of the sequence and columns past head_dim zero-filled by
// the buffer's range check. Two LDS stages, one barrier per tile, at least two blocks per CU so
// that one block's softmax runs under the other's MFMAs.
//
// A wavefront-wide LDS-direct load writes 64 x 16 B contiguously, so LDS rows are exactly 2 W bytes
// and cannot be padded. Instead the 16-byte chunk c of tile row r is kept at chunk position
// c ^ swizzle(r). W = 128 (256-byte rows, 16 chunks): swizzle(r) = (r%4)*4 + (r/4)%4 — the 16 rows a
// ds_read_b128 fragment read touches hit 16 different chunk positions, and the 4 rows x 64 B a
// ds_read_b64_tr_b16 touches hit four different 64-byte windows. W = 64 (128-byte rows, 8 chunks,
// two rows per 256-byte bank period): swizzle(r) = ((r/2)%2)*4 + (r/4)%4 — rows of equal parity among
// 16 consecutive ones get 8 different chunk positions, and of the 4 rows of a transposed read the
// two of equal parity get different 64-byte halves. Both conflict-free. The lane that owns LDS slot
// (r, c') simply fetches global chunk c' ^ swizzle(r).
template <int W>
constexpr int kWideTile = kStream * W;  // elements of one 64 x W tile

constexpr int kSchedMfma = 0x008, kSchedDsRead = 0x100;
template <int CLASS, int COUNT>
__device__ __forceinline__ void sched_group() {
    if constexpr (COUNT > 0) __builtin_amdgcn_sched_group_barrier(CLASS, COUNT, 0);
}
// LEAD LDS reads up front, then MFMAS matrix instructions with the remaining READS - LEAD reads
// spread between the first ones of them.
template <int MFMAS, int READS, int LEAD, int I = 0>
__device__ __forceinline__ void sched_reads_under_mfmas() {
    if constexpr (I == 0) sched_group<kSchedDsRead, LEAD>();
    if constexpr (I < MFMAS) {
        constexpr int kRest = READS - LEAD;
        constexpr int kSpan = MFMAS - 2;  // the last two MFMAs need no further reads
        constexpr int kDone = I < kSpan ? (I * kRest) / kSpan : kRest;
        constexpr int kNext = I + 1 < kSpan ? ((I + 1) * kRest) / kSpan : kRest;
        sched_group<kSchedMfma, 1>();
        sched_group<kSchedDsRead, kNext - kDone>();
        sched_reads_under_mfmas<MFMAS, READS, LEAD, I + 1>();
    }
}

// MFMAS matrix instructions with READS LDS reads, VALU vector and TRANS transcendental instructions of
// independent work dealt out evenly between them (reads lead by a few so that operands arrive in time).
constexpr int kSchedValu = 0x002, kSchedTrans = 0x400;
template <int MFMAS, int READS, int VALU, int TRANS, int I = 0>
__device__ __forceinline__ void sched_pipeline() {
    if constexpr (I == 0) sched_group<kSchedDsRead, (READS < 6 ? READS : 6)>();
    if constexpr (I < MFMAS) {
        constexpr int kLead = READS < 6 ? READS : 6;
        constexpr int kRest = READS - kLead;
        sched_group<kSchedMfma, 1>();
        sched_group<kSchedDsRead, ((I + 1) * kRest) / MFMAS - (I * kRest) / MFMAS>();
        sched_group<kSchedValu, ((I + 1) * VALU) / MFMAS - (I * VALU) / MFMAS>();
        sched_group<kSchedTrans, ((I + 1) * TRANS) / MFMAS - (I * TRANS) / MFMAS>();
        sched_pipeline<MFMAS, READS, VALU, TRANS, I + 1>();
    }
}

template <int W>
__device__ __forceinline__ int swizzle(int row) {
    static_assert(W == 64 || W == 128, "padded widths of the LDS-direct kernels");
    if constexpr (W == 128) return ((row & 3) << 2) | ((row >> 2) & 3);
    else return (((row >> 1) & 1) << 2) | ((row >> 2) & 3);
}

using lds_void_ptr = __attribute__((address_space(3))) void*;

// Where a lane's 16 bytes of a streamed tile come from. One load instruction fills 1 KiB = R rows
// (R = 4 for W = 128, 8 for W = 64); load i of wavefront w covers tile rows 4 R i + R w .. + R - 1,
// lane l owning LDS slot (row R w + l / chunks per row, chunk l % chunks per row).
struct TileSource {
    __amdgpu_buffer_rsrc_t rsrc;
    int voffset;    // bytes, loop-invariant
    int row_bytes;  // bytes between consecutive sequence positions
};

// last_row: elements of the last row that belong to the buffer (head_dim when base points at one
// head, the whole row when the head is chosen by the scalar offset of each load).
template <typename T, int W>
__device__ __forceinline__ TileSource make_source(const T* base, long row_stride, int rows, int d, int wave,
                                                  long last_row) {
    constexpr int kChunks = W / 8, kRowsPerLoad = 64 / kChunks;
    const int lane = threadIdx.x & 63;
    TileSource s;
    s.row_bytes = static_cast<int>(row_stride * sizeof(T));
    const int bytes = static_cast<int>(((rows - 1) * row_stride + last_row) * sizeof(T));
    s.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(base), 0, bytes, 0x00020000);
    const int r = wave * kRowsPerLoad + lane / kChunks;
    const int chunk = (lane % kChunks) ^ swizzle<W>(r);
    // Chunks beyond head_dim get an offset past every valid byte: the load then returns zeros.
    s.voffset = chunk * 8 < d ? r * s.row_bytes + chunk * 16 : (1 << 30);
    return s;
}

template <typename T, int W>
__device__ __forceinline__ void stream_tile(const TileSource& s, int row0, T* tile, int wave) {
    constexpr int kRowsPerLoad = 64 / (W / 8), kLoads = kStream / (4 * kRowsPerLoad);
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(s.rsrc, (lds_void_ptr)(tile + (i * 4 + wave) * kRowsPerLoad * W), 16,
                                                 s.voffset, (row0 + i * 4 * kRowsPerLoad) * s.row_bytes, 0, 0);
}

// Element offset (within a 32-row block of a swizzled tile) of the lane's ds_read_b128 fragment:
// row lane%32, head-dim elements 16*step + 8*(lane/32) .. +7.
template <int W>
__device__ __forceinline__ int wide_direct_offset(int lane, int step) {
    const int row = lane & 31;
    return row * W + (((2 * step + (lane >> 5)) ^ swizzle<W>(row)) * 8);
}
// Element offset (within a 16-row block) of the lane's ds_read_b64_tr_b16 address for head-dim
// columns 32t .. 32t+31: rows {0-3 | 4-7} (+8 for the second read), see transposed_frag.
template <int W>
__device__ __forceinline__ int wide_transposed_offset(int lane, int t, int second) {
    const int row = (lane >> 5) * 4 + ((lane & 15) >> 2) + second * 8;
    const int chunk = t * 4 + ((lane >> 4) & 1) * 2 + ((lane & 3) >> 1);
    return row * W + ((chunk ^ swizzle<W>(row)) * 8) + (lane & 1) * 4;
}
template <typename T>
__device__ __forceinline__ typename Mma<T>::frag wide_transposed_frag(const T* block, int first, int second) {
    using lds_ptr = __attribute__((address_space(3))) s16x4*;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(block + first));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(block + second));
    vec_t<short, 8> both;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        both[e] = lo[e];
        both[4 + e] = hi[e];
    }
    return __builtin_bit_cast(typename Mma<T>::frag, both);
}

// max(a, b, c) in one instruction; the operands are never NaN here.
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

constexpr float kRescaleThreshold = 8.0f;  // log2 of the factor by which probabilities may exceed 1

// Exchange between lane l and lane l^32.
__device__ __forceinline__ float other_half(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}

template <typename T, int W>
__global__ __launch_bounds__(kThreads, 2) void attention_forward_wide_kernel(Params p) {
    using frag = typename Mma<T>::frag;
    constexpr int STEPS = W / 16, DT = W / 32;
    __shared__ __align__(1024) T lds[4 * kWideTile<W>];  // [stage][K | V]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const BlockCoordinates where = block_coordinates(p.hkv);
    const int b = where.b, h = where.h, kvh = h / (p.hq / p.hkv);
    const int q_block = where.q_block;
    const int q_row = q_block + wave * 32 + (lane & 31);
    const bool q_live = q_row < p.qs;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const T* q_ptr = static_cast<const T*>(p.q) + (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
    const long kv_offset = static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;
    const TileSource k_src = make_source<T, W>(static_cast<const T*>(p.k) + kv_offset, kv_stride, p.ks, p.d, wave, p.d);
    const TileSource v_src = make_source<T, W>(static_cast<const T*>(p.v) + kv_offset, kv_stride, p.ks, p.d, wave, p.d);

    const int last_q_block = min(q_block + kBlockRows, p.qs) - 1;
    const int k_end = p.causal ? min(p.ks, p.offset + last_q_block + 1) : p.ks;
    const int tiles = (k_end + kStream - 1) / kStream;
    if (tiles > 0) {
        stream_tile<T, W>(k_src, 0, lds, wave);
        stream_tile<T, W>(v_src, 0, lds + kWideTile<W>, wave);
    }

    frag qf[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) qf[s] = global_frag<T>(q_ptr, q_live, s, p.d);
    int k_off[STEPS], v_off[DT][2];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) k_off[s] = wide_direct_offset<W>(lane, s);
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        v_off[t][0] = wide_transposed_offset<W>(lane, t, 0);
        v_off[t][1] = wide_transposed_offset<W>(lane, t, 1);
    }

    acc_t o[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) o[t] = acc_t(0.0f);
    // The running maximum m is kept on the raw scores (the scale is positive, so it commutes with
    // max); probabilities are exp2(s*scale2 - m*scale2), one FMA and one v_exp_f32 per score.
    float m = -INFINITY, mb = 0.0f, l = 0.0f;  // mb = m * scale2 (0 while m is -inf)
    const float scale2 = p.scale * kLog2e;
    const int wave_first_q = q_block + wave * 32;
    const int wave_last_q = min(wave_first_q + 31, p.qs - 1);
    const bool wave_live = wave_first_q < p.qs;
    const int q_limit = p.causal ? p.offset + q_row : p.ks;  // largest visible key of this lane's query
    // Tiles whose last key is visible to the wave's first query need no masking at all.
    const int clear_limit = p.causal ? min(p.ks - 1, p.offset + wave_first_q) : p.ks - 1;

    for (int j = 0; j < tiles; ++j) {
        const int k0 = j * kStream;
        const T* k_tile = lds + (j & 1) * 2 * kWideTile<W>;
        const T* v_tile = k_tile + kWideTile<W>;
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's part of tile j is in LDS
        __syncthreads();                     // ... and everybody else's; stage (j+1)%2 is free
        if (j + 1 < tiles) {
            T* next = lds + ((j + 1) & 1) * 2 * kWideTile<W>;
            stream_tile<T, W>(k_src, k0 + kStream, next, wave);
            stream_tile<T, W>(v_src, k0 + kStream, next + kWideTile<W>, wave);
        }
        if (!wave_live || (p.causal && k0 > p.offset + wave_last_q)) continue;

        acc_t st[2] = {acc_t(0.0f), acc_t(0.0f)};
        {
            frag ka[2][STEPS];
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                ka[0][s] = *reinterpret_cast<const frag*>(k_tile + k_off[s]);
                ka[1][s] = *reinterpret_cast<const frag*>(k_tile + 32 * W + k_off[s]);
            }
#pragma unroll
            for (int s = 0; s < STEPS; ++s) {
                st[0] = Mma<T>::run(ka[0][s], qf[s], st[0]);
                st[1] = Mma<T>::run(ka[1][s], qf[s], st[1]);
            }
            sched_reads_under_mfmas<2 * STEPS, 2 * STEPS, 4>();
        }
        __builtin_amdgcn_sched_barrier(0);

        if (k0 + kStream - 1 > clear_limit) {
            // key = k0 + 32 sub + 8 (i/4) + 4 (lane/32) + i%4 is visible iff key <= min(q_limit, ks-1):
            // one comparison of a per-lane bound with a literal per score.
            const int bound = min(q_limit, p.ks - 1) - k0 - 4 * (lane >> 5);
            asm volatile("" ::: "memory");  // keeps the masking out of the common path (no if-conversion)
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    st[sub][i] = (sub * 32 + 8 * (i >> 2) + (i & 3) <= bound) ? st[sub][i] : -INFINITY;
        }
        float tile_max = max3(st[0][0], st[1][0], st[0][1]);
        tile_max = max3(tile_max, st[1][1], st[0][2]);
#pragma unroll
        for (int i = 2; i < 16; ++i) tile_max = max3(tile_max, st[1][i], i + 1 < 16 ? st[0][i + 1] : st[1][i]);
        tile_max = fmaxf(tile_max, other_half(tile_max));
        // The reference point m of the exponentials only follows the running maximum when it has
        // moved by more than 2^8 in probability terms for some query of the wavefront: until then
        // probabilities are merely scaled by up to 2^8 (harmless in fp32 sums and bf16/f16 factors,
        // and cancelled by the final division), and the accumulator rescaling is skipped.
        if (__any(tile_max > m && (tile_max - m) * scale2 > kRescaleThreshold)) {
            const float m_new = fmaxf(m, tile_max);
            const float mb_new = m_new == -INFINITY ? 0.0f : m_new * scale2;
            const float alpha = __builtin_amdgcn_exp2f(m == -INFINITY ? -INFINITY : m * scale2 - mb_new);
            l *= alpha;
#pragma unroll
            for (int t = 0; t < DT; ++t) o[t] *= alpha;
            m = m_new;
            mb = mb_new;
        }
        float tile_sum = 0.0f;
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float e = __builtin_amdgcn_exp2f(fmaf(st[sub][i], scale2, -mb));
                st[sub][i] = e;
                tile_sum += e;
            }
        l += tile_sum;
        __builtin_amdgcn_sched_barrier(0);

        {
            frag pf[2][2], vt[2][2][DT];
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    pf[sub][s] = acc_frag<T>(st[sub], s);
                    const T* block = v_tile + (sub * 32 + s * 16) * W;
#pragma unroll
                    for (int t = 0; t < DT; ++t) vt[sub][s][t] = wide_transposed_frag<T>(block, v_off[t][0], v_off[t][1]);
                }
#pragma unroll
            for (int sub = 0; sub < 2; ++sub)
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int t = 0; t < DT; ++t) o[t] = Mma<T>::run(vt[sub][s][t], pf[sub][s], o[t]);
            sched_reads_under_mfmas<4 * DT, 8 * DT, 8>();
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    l += other_half(l);
    if (!q_live) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    T* o_ptr = static_cast<T*>(p.out0) + (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
            if (d0 >= p.d) continue;
            vec_t<float, 4> v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = o[t][4 * g + e] * inv;
            store_vec<T, 4>(o_ptr + d0, vec_from_f32<T, 4>(v));
        }
    }
    if (p.lse_out != nullptr && lane < 32)
        p.lse_out[(static_cast<long>(b) * p.qs + q_row) * p.hq + h] = (mb + log2f(l)) * kLn2;
}

// dQ, LDS-direct family: the forward kernel's streaming scheme; per 32-key half tile
// Sᵀ = K·Qᵀ and dPᵀ = V·dOᵀ (two independent MFMA chains), dS = P∘(dP − delta) in registers,
// dQᵀ += Kᵀ·dSᵀ with K read back transposed. lse2 holds LSE·log2(e).
template <typename T, int W>
__global__ __launch_bounds__(kThreads, 2) void attention_dq_wide_kernel(Params p) {
    using frag = typename Mma<T>::frag;
    constexpr int STEPS = W / 16, DT = W / 32;
    __shared__ __align__(1024) T lds[4 * kWideTile<W>];  // [stage][K | V]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const BlockCoordinates where = block_coordinates(p.hkv);
    const int b = where.b, h = where.h, kvh = h / (p.hq / p.hkv);
    const int q_block = where.q_block;
    const int q_row = q_block + wave * 32 + (lane & 31);
    const bool q_live = q_row < p.qs;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const long q_offset = (static_cast<long>(b) * p.qs + q_row) * q_stride + h * p.d;
    const long kv_offset = static_cast<long>(b) * p.ks * kv_stride + kvh * p.d;
    const TileSource k_src = make_source<T, W>(static_cast<const T*>(p.k) + kv_offset, kv_stride, p.ks, p.d, wave, p.d);
    const TileSource v_src = make_source<T, W>(static_cast<const T*>(p.v) + kv_offset, kv_stride, p.ks, p.d, wave, p.d);

    const int last_q_block = min(q_block + kBlockRows, p.qs) - 1;
    const int k_end = p.causal ? min(p.ks, p.offset + last_q_block + 1) : p.ks;
    const int tiles = (k_end + kStream - 1) / kStream;
    if (tiles > 0) {
        stream_tile<T, W>(k_src, 0, lds, wave);
        stream_tile<T, W>(v_src, 0, lds + kWideTile<W>, wave);
    }

    frag qf[STEPS], dof[STEPS];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        qf[s] = global_frag<T>(static_cast<const T*>(p.q) + q_offset, q_live, s, p.d);
        dof[s] = global_frag<T>(static_cast<const T*>(p.dout) + q_offset, q_live, s, p.d);
    }
    const long stat_index = (static_cast<long>(b) * p.qs + q_row) * p.hq + h;
    const float lse2 = q_live ? p.lse[stat_index] : 0.0f;
    const float delta = q_live ? p.delta[stat_index] : 0.0f;
    int k_off[STEPS], kt_off[DT][2];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) k_off[s] = wide_direct_offset<W>(lane, s);
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        kt_off[t][0] = wide_transposed_offset<W>(lane, t, 0);
        kt_off[t][1] = wide_transposed_offset<W>(lane, t, 1);
    }

    acc_t dq[DT];
#pragma unroll
    for (int t = 0; t < DT; ++t) dq[t] = acc_t(0.0f);
    const float scale2 = p.scale * kLog2e;
    const int wave_first_q = q_block + wave * 32;
    const int wave_last_q = min(wave_first_q + 31, p.qs - 1);
    const bool wave_live = wave_first_q < p.qs;
    const int q_limit = p.causal ? p.offset + q_row : p.ks;
    const int clear_limit = p.causal ? min(p.ks - 1, p.offset + wave_first_q) : p.ks - 1;

    for (int j = 0; j < tiles; ++j) {
        const int k0 = j * kStream;
        const T* k_tile = lds + (j & 1) * 2 * kWideTile<W>;
        const T* v_tile = k_tile + kWideTile<W>;
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        if (j + 1 < tiles) {
            T* next = lds + ((j + 1) & 1) * 2 * kWideTile<W>;
            stream_tile<T, W>(k_src, k0 + kStream, next, wave);
            stream_tile<T, W>(v_src, k0 + kStream, next + kWideTile<W>, wave);
        }
        if (!wave_live || (p.causal && k0 > p.offset + wave_last_q)) continue;
        const bool masked = k0 + kStream - 1 > clear_limit;
        const int bound = min(q_limit, p.ks - 1) - k0 - 4 * (lane >> 5);
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            acc_t st(0.0f), dpt(0.0f);
            {
                frag ka[STEPS], va[STEPS];
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    ka[s] = *reinterpret_cast<const frag*>(k_tile + sub * 32 * W + k_off[s]);
                    va[s] = *reinterpret_cast<const frag*>(v_tile + sub * 32 * W + k_off[s]);
                }
#pragma unroll
                for (int s = 0; s < STEPS; ++s) {
                    st = Mma<T>::run(ka[s], qf[s], st);
                    dpt = Mma<T>::run(va[s], dof[s], dpt);
                }
                sched_reads_under_mfmas<2 * STEPS, 2 * STEPS, 4>();
            }
            __builtin_amdgcn_sched_barrier(0);
            if (masked) {
                asm volatile("" ::: "memory");  // keeps the masking out of the common path (no if-conversion)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    st[i] = (sub * 32 + 8 * (i >> 2) + (i & 3) <= bound) ? st[i] : -INFINITY;
            }
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const float prob = __builtin_amdgcn_exp2f(fmaf(st[i], scale2, -lse2));
                st[i] = prob * (dpt[i] - delta);
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                frag dsf[2], kt[2][DT];
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    dsf[s] = acc_frag<T>(st, s);
                    const T* block = k_tile + (sub * 32 + s * 16) * W;
#pragma unroll
                    for (int t = 0; t < DT; ++t) kt[s][t] = wide_transposed_frag<T>(block, kt_off[t][0], kt_off[t][1]);
                }
#pragma unroll
                for (int s = 0; s < 2; ++s)
#pragma unroll
                    for (int t = 0; t < DT; ++t) dq[t] = Mma<T>::run(kt[s][t], dsf[s], dq[t]);
                sched_reads_under_mfmas<2 * DT, 4 * DT, 6>();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (!q_live) return;
    T* out = static_cast<T*>(p.out0) + q_offset;
#pragma unroll
    for (int t = 0; t < DT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
            if (d0 >= p.d) continue;
            vec_t<float, 4> v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = dq[t][4 * g + e] * p.scale;
            if (p.accumulate) v += vec_to_f32<T, 4>(load_vec<T, 4>(out + d0));
            store_vec<T, 4>(out + d0, vec_from_f32<T, 4>(v));
        }
    }
}

// dK/dV, LDS-direct family. A block owns 128 keys of one (batch, kv-head) — 32 per
// wavefront, K and V fragments and the two accumulator tiles in registers — and streams the 64-query
// Q/dO tiles (plus their LSE·log2 e and delta values) of every q-head of the group through two LDS
// stages with LDS-direct loads. Registers allow one wavefront per SIMD here; the tile is handled
// as two 32-query halves, each as Sᵀ,dPᵀ (MFMAs with the fragment reads placed between them by
// sched_group_barrier) | P, dS (VALU) | dV, dK (MFMAs over transposed fragment reads). Issuing one
// half's P, dS arithmetic between the other half's MFMAs (a software pipeline over the halves, the
// mask applied as selects) was measured 3 % slower than this plain order.
// Key blocks are handled in pairs (i, last-i) by one block: under a causal mask block i sees
// (last-i+1)/(last+1) of the queries, so every pair carries the same work and 256 equal blocks fill
// 256 CUs exactly at the training shape.
// Queries past the end of the sequence need no masking: their dO rows and delta arrive as zeros
// (buffer range check), so P·dO and P∘(dP−delta) vanish whatever P is.
template <int W>
constexpr int kWideDkvSmem = 4 * kWideTile<W> * 2 + 4 * kStream * static_cast<int>(sizeof(float));

template <typename T, int W>
__global__ __launch_bounds__(kThreads, 1) void attention_dkv_wide_kernel(Params p) {
    using frag = typename Mma<T>::frag;
    constexpr int STEPS = W / 16, DT = W / 32;
    extern __shared__ __align__(1024) unsigned char wide_smem[];
    T* lds = reinterpret_cast<T*>(wide_smem);                             // [stage][Q | dO]
    float* stats = reinterpret_cast<float*>(wide_smem + 4 * kWideTile<W> * sizeof(T));  // [stage][lse2 | delta][64]
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Workgroup -> (key-block pair, kv head, batch entry). The pairs of one (batch, kv-head) stream the same Q and
    // dO rows: when the (batch, kv-head) pairs divide evenly over the 8 XCDs (workgroups go to them round-robin by
    // linear id), XCD x takes pairs x, x + 8, ... with all key-block pairs of each next to each other, so that they
    // run at the same time behind the same L2.
    int pair_x = static_cast<int>(blockIdx.x), b = static_cast<int>(blockIdx.z), kvh = static_cast<int>(blockIdx.y);
    {
        constexpr unsigned int kXcds = 8;
        const unsigned int linear = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned int owners = gridDim.y * gridDim.z;
        if (owners % kXcds == 0) {
            const unsigned int xcd = linear % kXcds, local = linear / kXcds;
            const unsigned int owner = xcd + kXcds * (local / gridDim.x);
            pair_x = static_cast<int>(local % gridDim.x);
            kvh = static_cast<int>(owner % gridDim.y);
            b = static_cast<int>(owner / gridDim.y);
        }
    }
    const int group = p.hq / p.hkv;
    const long q_stride = static_cast<long>(p.hq) * p.d, kv_stride = static_cast<long>(p.hkv) * p.d;
    const float scale2 = p.scale * kLog2e;

    // Sources: Q and dO of this batch element (the head is part of the scalar offset), and the two
    // per-(query, head) statistics, one float per lane.
    const long q_batch = static_cast<long>(b) * p.qs * q_stride;
    const TileSource q_src = make_source<T, W>(static_cast<const T*>(p.q) + q_batch, q_stride, p.qs, p.d, wave, q_stride);
    const TileSource do_src = make_source<T, W>(static_cast<const T*>(p.dout) + q_batch, q_stride, p.qs, p.d, wave, q_stride);
    const int stat_bytes = p.qs * p.hq * static_cast<int>(sizeof(float));
    const float* stat_base = (wave == 0 ? p.lse : p.delta) + static_cast<long>(b) * p.qs * p.hq;
    const __amdgpu_buffer_rsrc_t stat_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(stat_base), 0, stat_bytes, 0x00020000);
    const int stat_voffset = lane * p.hq * static_cast<int>(sizeof(float));

    int q_off[STEPS], t_off[DT][2];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) q_off[s] = wide_direct_offset<W>(lane, s);
#pragma unroll
    for (int t = 0; t < DT; ++t) {
        t_off[t][0] = wide_transposed_offset<W>(lane, t, 0);
        t_off[t][1] = wide_transposed_offset<W>(lane, t, 1);
    }

    const int key_blocks = (p.ks + kBlockRows - 1) / kBlockRows;
    for (int half = 0; half < (p.paired ? 2 : 1); ++half) {
        const int block_index = half == 0 ? pair_x : key_blocks - 1 - pair_x;
        if (half == 1 && block_index <= pair_x) break;
        const int k_block = block_index * kBlockRows;
        const int k_row = k_block + wave * 32 + (lane & 31);
        const bool k_live = k_row < p.ks;
        const long k_offset = (static_cast<long>(b) * p.ks + k_row) * kv_stride + kvh * p.d;
        frag kf[STEPS], vf[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            kf[s] = global_frag<T>(static_cast<const T*>(p.k) + k_offset, k_live, s, p.d);
            vf[s] = global_frag<T>(static_cast<const T*>(p.v) + k_offset, k_live, s, p.d);
        }
        acc_t dk[DT], dv[DT];
#pragma unroll
        for (int t = 0; t < DT; ++t) {
            dk[t] = acc_t(0.0f);
            dv[t] = acc_t(0.0f);
        }
        // First query tile that can see any key of this block; the (head of the group, query tile)
        // pairs form one flat sequence so that the next tile is prefetched across head boundaries.
        const int q_begin = p.causal ? max(0, k_block - p.offset) / kStream * kStream : 0;
        const int tiles_per_head = q_begin < p.qs ? (p.qs - q_begin + kStream - 1) / kStream : 0;
        const int total_tiles = tiles_per_head * group;
        const int wave_first_key = k_block + wave * 32;
        const int wave_last_key = wave_first_key + 31;

        // Where the next tile comes from (requested during the current tile's first MFMAs).
        struct NextTile {
            bool live;
            int soffset;  // bytes: first row of the tile + head
            T* stage;
            int stat_soffset;
            float* stat_stage;
        };
        auto next_tile = [&](int tile) {
            NextTile n;
            n.live = tile < total_tiles;
            const int h = kvh * group + tile / max(tiles_per_head, 1);
            const int q0 = q_begin + (tile % max(tiles_per_head, 1)) * kStream;
            n.soffset = q0 * q_src.row_bytes + h * p.d * static_cast<int>(sizeof(T));
            n.stage = lds + (tile & 1) * 2 * kWideTile<W>;
            n.stat_soffset = (q0 * p.hq + h) * static_cast<int>(sizeof(float));
            n.stat_stage = stats + (tile & 1) * 2 * kStream + wave * kStream;
            return n;
        };
        constexpr int kRowsPerLoad = 64 / (W / 8), kLoads = kStream / (4 * kRowsPerLoad);
        // Part `i` of a tile request: rows 4 R i + R w .. of Q and dO (i < kLoads), then the statistics.
        auto request_part = [&](const NextTile& n, int i) {
            if (!n.live) return;
            if (i < kLoads) {
                const int soffset = n.soffset + i * 4 * kRowsPerLoad * q_src.row_bytes;
                T* rows = n.stage + (i * 4 + wave) * kRowsPerLoad * W;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(q_src.rsrc, (lds_void_ptr)(rows), 16, q_src.voffset, soffset, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(do_src.rsrc, (lds_void_ptr)(rows + kWideTile<W>), 16, do_src.voffset,
                                                         soffset, 0, 0);
            } else if (i == kLoads && wave < 2) {
                __builtin_amdgcn_raw_ptr_buffer_load_lds(stat_rsrc, (lds_void_ptr)(n.stat_stage), 4, stat_voffset, n.stat_soffset, 0,
                                                         0);
            }
        };

        // One 64-query tile = 4 N MFMAs (N = W / 8) in four phases over its two 32-query halves:
        //   Sᵀ,dPᵀ(0) | Sᵀ,dPᵀ(1) + P,dS(0) | dV,dK(0) + P,dS(1) | dV,dK(1)
        // A wavefront's VALU instructions run in the shadow of its own MFMAs when they do not depend on them,
        // but only if they stand between them in program order (an MFMA waits at issue for the previous one,
        // and everything behind it waits too). So the tile is written as 4 N slots of one MFMA each, with a
        // scheduling fence after every slot; a slot also carries the LDS reads of the operand needed kLookAhead
        // slots later, and its share of what else the tile has to do: the requests for the next tile and the
        // reads of LSE·log2 e and delta in phase 0, the exponentials and products of half 0 in phase 1, of half 1
        // in phase 2 (two scores per slot pair: fma, exp | subtract, multiply, packed converts).
        // MASKED: some (query, key) pairs of this wavefront are hidden (causal mask, keys past the end);
        // first = first visible register coordinate for this lane's key. Two separate straight-line bodies.
        auto tile_body = [&]<bool MASKED>(const T* q_tile, const T* do_tile, const float* stat, int first, const NextTile& next) {
            constexpr int N = W / 8, kLookAhead = 4;
            acc_t s_acc[2], dp_acc[2];
            vec_t<unsigned int, 4> p_words[2][2], ds_words[2][2];  // [half][16-query step]: the k-operands of dV, dK
            vec_t<float, 4> lse_q[2][4], delta_q[2][4];
            float prob_pair[2][16];
            frag operand[4 * N];
            auto read_operand = [&]<int K>() {
                constexpr int phase = K / N, j = K % N;
                if constexpr (phase < 2) {
                    const T* tile = (j & 1) ? do_tile : q_tile;
                    operand[K] = *reinterpret_cast<const frag*>(tile + phase * 32 * W + q_off[j >> 1]);
                } else {
                    constexpr int s = j / (2 * DT), t = (j / 2) % DT;
                    const T* tile = (j & 1) ? q_tile : do_tile;
                    operand[K] = wide_transposed_frag<T>(tile + ((phase - 2) * 32 + s * 16) * W, t_off[t][0], t_off[t][1]);
                }
            };
            auto multiply = [&]<int K>() {
                constexpr int phase = K / N, j = K % N;
                if constexpr (phase < 2) {
                    constexpr int s = j >> 1;
                    if constexpr (j & 1) dp_acc[phase] = Mma<T>::run(operand[K], vf[s], s == 0 ? acc_t(0.0f) : dp_acc[phase]);
                    else s_acc[phase] = Mma<T>::run(operand[K], kf[s], s == 0 ? acc_t(0.0f) : s_acc[phase]);
                } else {
                    constexpr int s = j / (2 * DT), t = (j / 2) % DT;
                    if constexpr (j & 1) dk[t] = Mma<T>::run(operand[K], __builtin_bit_cast(frag, ds_words[phase - 2][s]), dk[t]);
                    else dv[t] = Mma<T>::run(operand[K], __builtin_bit_cast(frag, p_words[phase - 2][s]), dv[t]);
                }
            };
            auto statistics = [&]<int SUB, int I>() {  // read I of 8
                constexpr int g = I >> 1;
                const int local = SUB * 32 + 8 * g + 4 * (lane >> 5);
                if constexpr (I & 1) delta_q[SUB][g] = *reinterpret_cast<const vec_t<float, 4>*>(stat + kStream + local);
                else lse_q[SUB][g] = *reinterpret_cast<const vec_t<float, 4>*>(stat + local);
            };
            // Half-slice H of 16 for half SUB: scores 2 (H/2), 2 (H/2) + 1. Even H: P; odd H: dS and both packs.
            auto softmax_part = [&]<int SUB, int H>() {
                constexpr int i0 = 2 * (H / 2), i1 = i0 + 1;
                if constexpr ((H & 1) == 0) {
                    float a = __builtin_amdgcn_exp2f(fmaf(s_acc[SUB][i0], scale2, -lse_q[SUB][i0 >> 2][i0 & 3]));
                    float c = __builtin_amdgcn_exp2f(fmaf(s_acc[SUB][i1], scale2, -lse_q[SUB][i1 >> 2][i1 & 3]));
                    if constexpr (MASKED) {
                        a = (SUB * 32 + 8 * (i0 >> 2) + (i0 & 3) >= first) ? a : 0.0f;
                        c = (SUB * 32 + 8 * (i1 >> 2) + (i1 & 3) >= first) ? c : 0.0f;
                    }
                    prob_pair[SUB][i0] = a;
                    prob_pair[SUB][i1] = c;
                } else {
                    const float a = prob_pair[SUB][i0], c = prob_pair[SUB][i1];
                    vec_t<float, 2> pv, dsv;
                    pv[0] = a;
                    pv[1] = c;
                    dsv[0] = a * (dp_acc[SUB][i0] - delta_q[SUB][i0 >> 2][i0 & 3]);
                    dsv[1] = c * (dp_acc[SUB][i1] - delta_q[SUB][i1 >> 2][i1 & 3]);
                    constexpr int word = i0 / 2;  // 8 words per half: 4 per 16-query step
                    p_words[SUB][word / 4][word % 4] = __builtin_bit_cast(unsigned int, vec_from_f32<T, 2>(pv));
                    ds_words[SUB][word / 4][word % 4] = __builtin_bit_cast(unsigned int, vec_from_f32<T, 2>(dsv));
                }
            };
            auto slot = [&]<int K>() {
                constexpr int phase = K / N, j = K % N;
                if constexpr (K + kLookAhead < 4 * N) read_operand.template operator()<K + kLookAhead>();
                multiply.template operator()<K>();
                if constexpr (phase == 0) {
                    if constexpr (j <= kLoads) request_part(next, j);
                }
                if constexpr (phase < 2) {  // statistics of half `phase`, read while its scores are multiplied
                    constexpr int per_slot = 8 / N > 0 ? 8 / N : 1;
                    if constexpr (j * per_slot < 8) {
                        statistics.template operator()<phase, j * per_slot>();
                        if constexpr (per_slot == 2) statistics.template operator()<phase, j * per_slot + 1>();
                    }
                }
                if constexpr (phase == 1 || phase == 2) {  // P, dS of half phase - 1
                    constexpr int per_slot = 16 / N;
#pragma unroll
                    for (int unused = 0; unused < 1; ++unused) {
                        softmax_part.template operator()<phase - 1, j * per_slot>();
                        if constexpr (per_slot == 2) softmax_part.template operator()<phase - 1, j * per_slot + 1>();
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            };
            [&]<int... K>(std::integer_sequence<int, K...>) {
                (read_operand.template operator()<K>(), ...);
            }(std::make_integer_sequence<int, kLookAhead>{});
            __builtin_amdgcn_sched_barrier(0);
            [&]<int... K>(std::integer_sequence<int, K...>) { (slot.template operator()<K>(), ...); }(
                std::make_integer_sequence<int, 4 * N>{});
        };

        // Every wavefront runs every tile (no divergent paths around the accumulators): pairs the causal mask
        // hides, and keys past the end of the sequence, get P = 0. Register i of half `sub` holds query
        // q0 + 32 sub + 8 (i/4) + 4 (lane/32) + i%4; this lane's key sees it iff that query is >= key - offset.
        // Per head the tiles that need the mask come first (the ones on the diagonal; all of them for a
        // wavefront with keys past the end): two loops with one straight-line body each, so that the
        // accumulators stay where they are from tile to tile.
        int masked_per_head = 0;
        if (wave_last_key >= p.ks) masked_per_head = tiles_per_head;
        else if (p.causal) masked_per_head = min(tiles_per_head, max(0, (wave_last_key - p.offset - q_begin + kStream - 1) / kStream));
        auto arrive = [&]() {
            __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wavefront's part of the tile is in LDS
            __syncthreads();                     // ... and everybody else's; the other stage is free
        };
        {
            const NextTile first_tile = next_tile(0);
#pragma unroll
            for (int i = 0; i <= kLoads; ++i) request_part(first_tile, i);
        }
        for (int head = 0; head < group; ++head) {
            const int tile0 = head * tiles_per_head;
            for (int t = 0; t < masked_per_head; ++t) {
                const int tile = tile0 + t, q0 = q_begin + t * kStream;
                const T* q_tile = lds + (tile & 1) * 2 * kWideTile<W>;
                arrive();
                const int causal_first = p.causal ? k_row - p.offset - q0 - 4 * (lane >> 5) : -(1 << 30);
                tile_body.template operator()<true>(q_tile, q_tile + kWideTile<W>, stats + (tile & 1) * 2 * kStream,
                                                    k_live ? causal_first : (1 << 30), next_tile(tile + 1));
            }
            for (int t = masked_per_head; t < tiles_per_head; ++t) {
                const int tile = tile0 + t;
                const T* q_tile = lds + (tile & 1) * 2 * kWideTile<W>;
                arrive();
                tile_body.template operator()<false>(q_tile, q_tile + kWideTile<W>, stats + (tile & 1) * 2 * kStream, 0,
                                                     next_tile(tile + 1));
            }
        }
        __syncthreads();  // the next key block's first loads overwrite stage 0
        if (k_live) {
            T* dk_out = static_cast<T*>(p.out0) + k_offset;
            T* dv_out = static_cast<T*>(p.out1) + k_offset;
#pragma unroll
            for (int t = 0; t < DT; ++t) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int d0 = t * 32 + g * 8 + (lane >> 5) * 4;
                    if (d0 >= p.d) continue;
                    vec_t<float, 4> a, c;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        a[e] = dk[t][4 * g + e] * p.scale;
                        c[e] = dv[t][4 * g + e];
                    }
                    if (p.accumulate) {
                        a += vec_to_f32<T, 4>(load_vec<T, 4>(dk_out + d0));
                        c += vec_to_f32<T, 4>(load_vec<T, 4>(dv_out + d0));
                    }
                    store_vec<T, 4>(dk_out + d0, vec_from_f32<T, 4>(a));
                    store_vec<T, 4>(dv_out + d0, vec_from_f32<T, 4>(c));
                }
            }
        }
    }
}


// ============================================================================================
// Scalar family: fp32 storage, head dimensions that are not multiples of 8, and tensors that are not
// 16-byte aligned — what the reference serves with its warp-per-row kernels
// (src/ops/backward/attention_backward.cu:352-504, dispatch 2044-2068). Correct, not fast: one
// wavefront per output row, fp32 arithmetic throughout, lane l holding head-dim elements l and l + 64.
// No atomics: dQ rows and (key, kv-head) rows each have one owner that adds its terms in a fixed order
// (heads of the group ascending, queries ascending), so results do not depend on scheduling.
template <typename T>
struct RowPair {
    float a, b;  // elements lane and lane + 64 of a head_dim-long row (0 past the end)
    __device__ __forceinline__ static RowPair load(const T* row, int d) {
        const int lane = threadIdx.x & 63;
        RowPair r;
        r.a = lane < d ? to_f32(row[lane]) : 0.0f;
        r.b = lane + 64 < d ? to_f32(row[lane + 64]) : 0.0f;
        return r;
    }
    __device__ __forceinline__ void store(T* row, int d, bool accumulate) const {
        const int lane = threadIdx.x & 63;
        if (lane < d) row[lane] = from_f32<T>(accumulate ? a + to_f32(row[lane]) : a);
        if (lane + 64 < d) row[lane + 64] = from_f32<T>(accumulate ? b + to_f32(row[lane + 64]) : b);
    }
};
template <typename T>
__device__ __forceinline__ float row_dot(const RowPair<T>& x, const RowPair<T>& y) {
    return wave_sum(fmaf(x.a, y.a, x.b * y.b));
}

constexpr int kScalarWaves = 4;  // rows per 256-thread block

// O and LSE of one (batch, query, head) row per wavefront; lse_out and delta-style outputs are fp32.
template <typename T>
__global__ __launch_bounds__(kThreads) void attention_forward_scalar_kernel(Params p) {
    const long row = static_cast<long>(blockIdx.x) * kScalarWaves + (threadIdx.x >> 6);
    const long rows = static_cast<long>(p.batch) * p.qs * p.hq;
    if (row >= rows) return;
    const int h = static_cast<int>(row % p.hq);
    const int q = static_cast<int>((row / p.hq) % p.qs);
    const int b = static_cast<int>(row / (static_cast<long>(p.hq) * p.qs));
    const int kvh = h / (p.hq / p.hkv);
    const RowPair<T> qr = RowPair<T>::load(static_cast<const T*>(p.q) + row * p.d, p.d);
    const T* k_base = static_cast<const T*>(p.k) + (static_cast<long>(b) * p.ks * p.hkv + kvh) * p.d;
    const T* v_base = static_cast<const T*>(p.v) + (static_cast<long>(b) * p.ks * p.hkv + kvh) * p.d;
    const long kv_stride = static_cast<long>(p.hkv) * p.d;
    const int k_end = p.causal ? min(p.ks, p.offset + q + 1) : p.ks;
    float m = -INFINITY, l = 0.0f;
    RowPair<T> o{0.0f, 0.0f};
    for (int j = 0; j < k_end; ++j) {
        const float s = row_dot(qr, RowPair<T>::load(k_base + j * kv_stride, p.d)) * p.scale;
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new), e = expf(s - m_new);  // exp(-inf) = 0 on the first key
        const RowPair<T> vr = RowPair<T>::load(v_base + j * kv_stride, p.d);
        l = l * alpha + e;
        o.a = fmaf(e, vr.a, o.a * alpha);
        o.b = fmaf(e, vr.b, o.b * alpha);
        m = m_new;
    }
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    o.a *= inv;
    o.b *= inv;
    o.store(static_cast<T*>(p.out0) + row * p.d, p.d, false);
    if (p.lse_out != nullptr && (threadIdx.x & 63) == 0) p.lse_out[row] = m + logf(l);
}

// dQ of one (batch, query, head) row per wavefront; also leaves delta = rowsum(dO∘O) for the dK/dV pass.
template <typename T>
__global__ __launch_bounds__(kThreads) void attention_dq_scalar_kernel(Params p, const void* out, float* delta_out) {
    const long row = static_cast<long>(blockIdx.x) * kScalarWaves + (threadIdx.x >> 6);
    const long rows = static_cast<long>(p.batch) * p.qs * p.hq;
    if (row >= rows) return;
    const int h = static_cast<int>(row % p.hq);
    const int q = static_cast<int>((row / p.hq) % p.qs);
    const int b = static_cast<int>(row / (static_cast<long>(p.hq) * p.qs));
    const int kvh = h / (p.hq / p.hkv);
    const RowPair<T> qr = RowPair<T>::load(static_cast<const T*>(p.q) + row * p.d, p.d);
    const RowPair<T> dor = RowPair<T>::load(static_cast<const T*>(p.dout) + row * p.d, p.d);
    const float delta = row_dot(dor, RowPair<T>::load(static_cast<const T*>(out) + row * p.d, p.d));
    if ((threadIdx.x & 63) == 0) delta_out[row] = delta;
    const float lse = p.lse[row];
    const T* k_base = static_cast<const T*>(p.k) + (static_cast<long>(b) * p.ks * p.hkv + kvh) * p.d;
    const T* v_base = static_cast<const T*>(p.v) + (static_cast<long>(b) * p.ks * p.hkv + kvh) * p.d;
    const long kv_stride = static_cast<long>(p.hkv) * p.d;
    const int k_end = p.causal ? min(p.ks, p.offset + q + 1) : p.ks;
    RowPair<T> dq{0.0f, 0.0f};
    for (int j = 0; j < k_end; ++j) {
        const RowPair<T> kr = RowPair<T>::load(k_base + j * kv_stride, p.d);
        const float prob = expf(row_dot(qr, kr) * p.scale - lse);
        const float ds = prob * (row_dot(dor, RowPair<T>::load(v_base + j * kv_stride, p.d)) - delta);
        dq.a = fmaf(ds, kr.a, dq.a);
        dq.b = fmaf(ds, kr.b, dq.b);
    }
    dq.a *= p.scale;
    dq.b *= p.scale;
    dq.store(static_cast<T*>(p.out0) + row * p.d, p.d, p.accumulate != 0);
}

// dK and dV of one (batch, key, kv-head) row per wavefront: the heads of the group in ascending order,
// each over the queries that see the key in ascending order.
template <typename T>
__global__ __launch_bounds__(kThreads) void attention_dkv_scalar_kernel(Params p) {
    const long row = static_cast<long>(blockIdx.x) * kScalarWaves + (threadIdx.x >> 6);
    const long rows = static_cast<long>(p.batch) * p.ks * p.hkv;
    if (row >= rows) return;
    const int kvh = static_cast<int>(row % p.hkv);
    const int j = static_cast<int>((row / p.hkv) % p.ks);
    const int b = static_cast<int>(row / (static_cast<long>(p.hkv) * p.ks));
    const int group = p.hq / p.hkv;
    const RowPair<T> kr = RowPair<T>::load(static_cast<const T*>(p.k) + row * p.d, p.d);
    const RowPair<T> vr = RowPair<T>::load(static_cast<const T*>(p.v) + row * p.d, p.d);
    const int q_begin = p.causal ? max(0, j - p.offset) : 0;
    RowPair<T> dk{0.0f, 0.0f}, dv{0.0f, 0.0f};
    for (int g = 0; g < group; ++g) {
        const int h = kvh * group + g;
        for (int q = q_begin; q < p.qs; ++q) {
            const long q_row = (static_cast<long>(b) * p.qs + q) * p.hq + h;
            const RowPair<T> qr = RowPair<T>::load(static_cast<const T*>(p.q) + q_row * p.d, p.d);
            const RowPair<T> dor = RowPair<T>::load(static_cast<const T*>(p.dout) + q_row * p.d, p.d);
            const float prob = expf(row_dot(qr, kr) * p.scale - p.lse[q_row]);
            const float ds = prob * (row_dot(dor, vr) - p.delta[q_row]);
            dv.a = fmaf(prob, dor.a, dv.a);
            dv.b = fmaf(prob, dor.b, dv.b);
            dk.a = fmaf(ds, qr.a, dk.a);
            dk.b = fmaf(ds, qr.b, dk.b);
        }
    }
    dk.a *= p.scale;
    dk.b *= p.scale;
    dk.store(static_cast<T*>(p.out0) + row * p.d, p.d, p.accumulate != 0);
    dv.store(static_cast<T*>(p.out1) + row * p.d, p.d, p.accumulate != 0);
}

// ---------------------------------------------------------------------- host
struct Shape {
    std::size_t batch, qs, ks, hq, hkv, d;
    float scale;
    int causal;
    std::size_t offset;
    int dtype;
};

int validate(const char* name, const Shape& s) {
    const std::string n(name);
    if (!valid_dtype(s.dtype)) return fail(CGPTX_INVALID_ARGUMENT, n + ": unsupported dtype");
    if (s.batch == 0 || s.qs == 0 || s.ks == 0 || s.hq == 0 || s.hkv == 0 || s.d == 0 || s.hq % s.hkv != 0)
        return fail(CGPTX_INVALID_ARGUMENT, n + ": invalid tensors or options");
    if (!std::isfinite(s.scale)) return fail(CGPTX_INVALID_ARGUMENT, n + ": attention scale must be finite");
    if (s.causal && (s.offset > s.ks || s.qs > s.ks - s.offset))
        return fail(CGPTX_INVALID_ARGUMENT, n + ": causal range exceeds the key sequence");
    if (s.d > 128)  // as src/ops/backward/attention_backward.cu:1886-1887
        return fail(CGPTX_INVALID_ARGUMENT, n + ": head_dim must not exceed 128");
    constexpr std::size_t limit = 1u << 30;
    if (s.batch > 65535 || s.qs > limit || s.ks > limit || s.hq > 65535 || s.offset > limit ||
        s.hq * s.d > limit)
        return fail(CGPTX_OVERFLOW, n + ": dimension exceeds the supported range");
    return CGPTX_OK;
}

Params make_params(const Shape& s) {
    Params p{};
    p.batch = static_cast<int>(s.batch);
    p.qs = static_cast<int>(s.qs);
    p.ks = static_cast<int>(s.ks);
    p.hq = static_cast<int>(s.hq);
    p.hkv = static_cast<int>(s.hkv);
    p.d = static_cast<int>(s.d);
    p.scale = s.scale > 0.0f ? s.scale : 1.0f / std::sqrt(static_cast<float>(s.d));
    p.causal = s.causal ? 1 : 0;
    p.offset = static_cast<int>(s.offset);
    return p;
}

// The LDS-direct kernels take every supported head dimension (padded to 64 or 128 with zeros in LDS
// and registers; at B=32, T=1024: head_dim 64, 12:4 heads, forward 86 vs 162 us and backward 279 vs
// 878 us against the register-staged kernels; head_dim 32, 16:4 heads, 103 vs 163 and 325 vs 665 us).
// They address K/V (and Q/dO) of one batch element with 32-bit byte offsets; what exceeds that, and
// CGPTX_ATTENTION_WIDE=0 (for comparisons and tests), runs on the register-staged kernels.
// Bytes reserved for one float per (batch, query, head), rounded so that blocks stay 256-byte aligned.
std::size_t stat_block_bytes(std::size_t rows) { return (rows * sizeof(float) + 255) & ~std::size_t{255}; }

bool wide_path(const Shape& s) {
    constexpr std::size_t limit = std::size_t{1} << 30;
    const char* text = std::getenv("CGPTX_ATTENTION_WIDE");  // read per call
    const bool enabled = text == nullptr || text[0] != '0';
    return enabled && s.ks * s.hkv * s.d * 2 < limit && s.qs * s.hq * s.d * 2 < limit;
}

template <typename Fn>
int dispatch_head_dim(std::size_t d, Fn&& fn) {
    if (d <= 32) return fn.template operator()<32>();
    if (d <= 64) return fn.template operator()<64>();
    return fn.template operator()<128>();
}

template <typename Fn>
int dispatch_16bit(int dtype, Fn&& fn) {
    return dtype == CGPTX_F16 ? fn.template operator()<f16_t>() : fn.template operator()<bf16_t>();
}

bool aligned16_all(std::initializer_list<const void*> pointers) {
    for (const void* ptr : pointers)
        if (ptr != nullptr && !is_aligned16(ptr)) return false;
    return true;
}

// The matrix-core kernels take 16-bit storage, head dimensions in multiples of 8 (128-bit row chunks) and
// 16-byte aligned tensors; everything else the interface accepts runs on the scalar family.
bool scalar_path(const Shape& s, std::initializer_list<const void*> pointers) {
    return s.dtype == CGPTX_F32 || s.d % 8 != 0 || !aligned16_all(pointers);
}

unsigned int scalar_blocks(std::size_t rows) { return static_cast<unsigned int>((rows + kScalarWaves - 1) / kScalarWaves); }

int launch_forward(const Shape& s, Params p, bool scalar, hipStream_t stream) {
    if (scalar) {
        const std::size_t rows = s.batch * s.qs * s.hq;
        if (rows / kScalarWaves >= (std::size_t{1} << 31)) return fail(CGPTX_OVERFLOW, "attention: grid too large");
        return dispatch_dtype(s.dtype, [&]<typename T>() -> int {
            hipLaunchKernelGGL((attention_forward_scalar_kernel<T>), dim3(scalar_blocks(rows)), dim3(kThreads), 0, stream, p);
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        });
    }
    const dim3 grid(static_cast<unsigned int>((s.qs + kBlockRows - 1) / kBlockRows), static_cast<unsigned int>(s.hq),
                    static_cast<unsigned int>(s.batch));
    return dispatch_16bit(s.dtype, [&]<typename T>() -> int {
        if (wide_path(s)) {
            if (s.d <= 64) hipLaunchKernelGGL((attention_forward_wide_kernel<T, 64>), grid, dim3(kThreads), 0, stream, p);
            else hipLaunchKernelGGL((attention_forward_wide_kernel<T, 128>), grid, dim3(kThreads), 0, stream, p);
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        }
        return dispatch_head_dim(s.d, [&]<int DP>() -> int {
            hipLaunchKernelGGL((attention_forward_kernel<T, DP>), grid, dim3(kThreads), 0, stream, p);
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        });
    });
}

int launch_backward(const Shape& s, Params p, void* dq, void* dk, void* dv, const void* dout, const void* out,
                    const float* lse, int accumulate, bool scalar, hipStream_t stream) {
    const std::size_t rows = s.batch * s.qs * s.hq;
    const std::size_t stat_bytes = stat_block_bytes(rows);
    void* mem = nullptr;
    if (int st = scratch(stream, 2 * stat_bytes, &mem)) return st;  // [delta | LSE·log2 e]
    auto* delta = static_cast<float*>(mem);
    auto* lse2 = reinterpret_cast<float*>(static_cast<char*>(mem) + stat_bytes);
    p.dout = dout;
    p.lse = lse;
    p.delta = delta;
    p.accumulate = accumulate;
    if (scalar) {
        const std::size_t key_rows = s.batch * s.ks * s.hkv;
        if (rows / kScalarWaves >= (std::size_t{1} << 31) || key_rows / kScalarWaves >= (std::size_t{1} << 31))
            return fail(CGPTX_OVERFLOW, "attention: grid too large");
        return dispatch_dtype(s.dtype, [&]<typename T>() -> int {
            Params pq = p;
            pq.out0 = dq;
            hipLaunchKernelGGL((attention_dq_scalar_kernel<T>), dim3(scalar_blocks(rows)), dim3(kThreads), 0, stream, pq,
                               out, delta);
            CGPTX_LAUNCH_CHECK();
            Params pk = p;
            pk.out0 = dk;
            pk.out1 = dv;
            hipLaunchKernelGGL((attention_dkv_scalar_kernel<T>), dim3(scalar_blocks(key_rows)), dim3(kThreads), 0, stream, pk);
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        });
    }
    return dispatch_16bit(s.dtype, [&]<typename T>() -> int {
        const int lpr = s.d <= 32 ? 4 : (s.d <= 64 ? 8 : 16);
        const unsigned int delta_blocks = static_cast<unsigned int>((rows * lpr + kThreads - 1) / kThreads);
        auto* dout_t = static_cast<const T*>(dout);
        auto* out_t = static_cast<const T*>(out);
        const long r = static_cast<long>(rows);
        const int d = static_cast<int>(s.d);
        if (lpr == 4)
            hipLaunchKernelGGL((attention_delta_kernel<T, 4>), dim3(delta_blocks), dim3(kThreads), 0, stream, delta,
                               lse2, lse, dout_t, out_t, r, d);
        else if (lpr == 8)
            hipLaunchKernelGGL((attention_delta_kernel<T, 8>), dim3(delta_blocks), dim3(kThreads), 0, stream, delta,
                               lse2, lse, dout_t, out_t, r, d);
        else
            hipLaunchKernelGGL((attention_delta_kernel<T, 16>), dim3(delta_blocks), dim3(kThreads), 0, stream, delta,
                               lse2, lse, dout_t, out_t, r, d);
        CGPTX_LAUNCH_CHECK();
        return dispatch_head_dim(s.d, [&]<int DP>() -> int {
            Params pq = p;
            pq.out0 = dq;
            const dim3 q_grid(static_cast<unsigned int>((s.qs + kBlockRows - 1) / kBlockRows),
                              static_cast<unsigned int>(s.hq), static_cast<unsigned int>(s.batch));
            if (wide_path(s)) {
                pq.lse = lse2;
                if (s.d <= 64) hipLaunchKernelGGL((attention_dq_wide_kernel<T, 64>), q_grid, dim3(kThreads), 0, stream, pq);
                else hipLaunchKernelGGL((attention_dq_wide_kernel<T, 128>), q_grid, dim3(kThreads), 0, stream, pq);
            } else {
                hipLaunchKernelGGL((attention_dq_kernel<T, DP>), q_grid, dim3(kThreads), 0, stream, pq);
            }
            CGPTX_LAUNCH_CHECK();
            Params pk = p;
            pk.out0 = dk;
            pk.out1 = dv;
            const unsigned int key_blocks = static_cast<unsigned int>((s.ks + kBlockRows - 1) / kBlockRows);
            if (wide_path(s)) {
                pk.lse = lse2;
                // Pairs equalise the work under a causal mask; without one every block carries the same work, and a
                // grid that leaves compute units idle is better off with twice the workgroups (the longest single
                // block is shorter than the pair that contains it).
                const std::size_t single_blocks = static_cast<std::size_t>(key_blocks) * s.hkv * s.batch;
                pk.paired = s.causal && single_blocks > static_cast<std::size_t>(compute_units());
                const dim3 pair_grid(pk.paired ? (key_blocks + 1) / 2 : key_blocks, static_cast<unsigned int>(s.hkv),
                                     static_cast<unsigned int>(s.batch));
                auto launch = [&]<int W>() -> int {
                    auto kernel = attention_dkv_wide_kernel<T, W>;
                    static bool configured = false;
                    if (!configured) {
                        CGPTX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                                      hipFuncAttributeMaxDynamicSharedMemorySize, kWideDkvSmem<W>));
                        configured = true;
                    }
                    hipLaunchKernelGGL(kernel, pair_grid, dim3(kThreads), kWideDkvSmem<W>, stream, pk);
                    return CGPTX_OK;
                };
                if (int st = s.d <= 64 ? launch.template operator()<64>() : launch.template operator()<128>()) return st;
            } else {
                const dim3 k_grid(key_blocks, static_cast<unsigned int>(s.hkv), static_cast<unsigned int>(s.batch));
                hipLaunchKernelGGL((attention_dkv_kernel<T, DP>), k_grid, dim3(kThreads), 0, stream, pk);
            }
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        });
    });
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_flash_gqa_attention_forward(void* output, float* logsumexp, const void* query, const void* key,
                                                 const void* value, size_t batch, size_t query_sequence,
                                                 size_t kv_sequence, size_t query_heads, size_t kv_heads,
                                                 size_t head_dim, float attention_scale, int causal,
                                                 size_t query_position_offset, int dtype, cgptx_stream stream) {
    using namespace cgptx;
    const char* name = "flash_gqa_attention_forward";
    const Shape s{batch, query_sequence, kv_sequence, query_heads, kv_heads, head_dim, attention_scale, causal,
                  query_position_offset, dtype};
    if (int st = validate(name, s)) return st;
    if (output == nullptr || query == nullptr || key == nullptr || value == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null tensor");
    Params p = make_params(s);
    p.out0 = output;
    p.lse_out = logsumexp;
    p.q = query;
    p.k = key;
    p.v = value;
    return launch_forward(s, p, scalar_path(s, {output, query, key, value}), static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_flash_gqa_attention_backward_with_lse(
    void* grad_query, void* grad_key, void* grad_value, const void* grad_output, const void* output,
    const float* logsumexp, const void* query, const void* key, const void* value, size_t batch,
    size_t query_sequence, size_t kv_sequence, size_t query_heads, size_t kv_heads, size_t head_dim,
    float attention_scale, int causal, size_t query_position_offset, int accumulate_grads, int dtype,
    cgptx_stream stream) {
    using namespace cgptx;
    const char* name = "flash_gqa_attention_backward_with_lse";
    const Shape s{batch, query_sequence, kv_sequence, query_heads, kv_heads, head_dim, attention_scale, causal,
                  query_position_offset, dtype};
    if (int st = validate(name, s)) return st;
    if (grad_query == nullptr || grad_key == nullptr || grad_value == nullptr || grad_output == nullptr ||
        output == nullptr || logsumexp == nullptr || query == nullptr || key == nullptr || value == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null tensor");
    Params p = make_params(s);
    p.q = query;
    p.k = key;
    p.v = value;
    const bool scalar = scalar_path(s, {grad_query, grad_key, grad_value, grad_output, output, query, key, value});
    return launch_backward(s, p, grad_query, grad_key, grad_value, grad_output, output, logsumexp,
                           accumulate_grads != 0, scalar, static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_flash_gqa_attention_backward(void* grad_query, void* grad_key, void* grad_value,
                                                  const void* grad_output, const void* query, const void* key,
                                                  const void* value, size_t batch, size_t query_sequence,
                                                  size_t kv_sequence, size_t query_heads, size_t kv_heads,
                                                  size_t head_dim, float attention_scale, int causal,
                                                  size_t query_position_offset, int accumulate_grads, int dtype,
                                                  cgptx_stream stream_) {
    using namespace cgptx;
    const char* name = "flash_gqa_attention_backward";
    const Shape s{batch, query_sequence, kv_sequence, query_heads, kv_heads, head_dim, attention_scale, causal,
                  query_position_offset, dtype};
    if (int st = validate(name, s)) return st;
    if (grad_query == nullptr || grad_key == nullptr || grad_value == nullptr || grad_output == nullptr ||
        query == nullptr || key == nullptr || value == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null tensor");
    const bool scalar = scalar_path(s, {grad_query, grad_key, grad_value, grad_output, query, key, value});
    auto stream = static_cast<hipStream_t>(stream_);
    // Recompute the output and the log-sum-exp into scratch, then run the LSE path. The scratch
    // block is laid out [delta | LSE·log2 e | lse | output] so that launch_backward's request for
    // the two-block prefix returns the same base pointer.
    const std::size_t rows = batch * query_sequence * query_heads;
    const std::size_t stat_bytes = stat_block_bytes(rows);
    const std::size_t out_bytes = rows * head_dim * dtype_size(dtype);
    void* mem = nullptr;
    if (int st = scratch(stream, 3 * stat_bytes + out_bytes, &mem)) return st;
    auto* lse = reinterpret_cast<float*>(static_cast<char*>(mem) + 2 * stat_bytes);
    void* out = static_cast<char*>(mem) + 3 * stat_bytes;
    Params p = make_params(s);
    p.q = query;
    p.k = key;
    p.v = value;
    Params fwd = p;
    fwd.out0 = out;
    fwd.lse_out = lse;
    if (int st = launch_forward(s, fwd, scalar, stream)) return st;
    return launch_backward(s, p, grad_query, grad_key, grad_value, grad_output, out, lse, accumulate_grads != 0,
                           scalar, stream);
}
