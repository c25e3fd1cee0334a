// Dense contraction kernels for gfx950 (CDNA4): C[M,N] (+)= op(A)·op(B), 16-bit
// inputs, fp32 accumulation on the matrix cores.
//
// One kernel family serves the three contractions of a linear layer
// (reference: src/ops/linear.cu:634-667, src/ops/backward/linear_backward.cu:268-285,
// where cuBLASLt does this work):
//   forward  Y  = X·Wᵀ      A[M,K] k-contiguous, B[N,K] k-contiguous
//   dX       dX = dY·W      A[M,K] k-contiguous, B[K,N] n-contiguous
//   dW       dW = dYᵀ·X     A[K,M] m-contiguous, B[K,N] n-contiguous
//
// Design
//   * 256 threads = 4 wavefronts in a 2x2 grid; a block owns a BM x BN tile of C
//     and walks K in steps of 64. Each wavefront owns (BM/2) x (BN/2) and issues
//     v_mfma_f32_32x32x16 (bf16 or f16), so every LDS fragment read feeds
//     (BM/64)·(BN/64) MFMAs.
//   * Both operands are staged in LDS k-contiguous with a row stride of 72
//     elements (144 B): the 16 rows a quarter-wavefront reads with one
//     ds_read_b128 then fall in 16 distinct bank groups.
//   * Operands that are not k-contiguous in memory (dX's weight, both dW
//     operands) are transposed in registers on their way to LDS: a thread loads
//     an 8(k) x 8(n) block with eight coalesced 128-bit loads, regroups it with
//     v_perm_b32 into eight k-contiguous 128-bit rows and stores those. No
//     separate transpose pass over HBM and no 16-bit LDS accesses.
//   * Global loads of tile t+1 are issued before the MFMAs of tile t and land in
//     the other LDS buffer afterwards: one barrier per K step.
//   * MFMA is issued as (B-fragment, A-fragment), so a lane ends up holding four
//     consecutive n for one m per accumulator group; the finished tile is staged in
//     LDS as fp32 and written out row by row (512 contiguous bytes per wavefront
//     store), with bias / accumulate added in fp32 and one rounding to the dtype.
//   * Block ids are remapped so that the 8 XCDs (blocks are dealt round-robin to
//     them) each walk a contiguous range of tiles, and tiles are ordered in groups
//     of 8 tile-rows so that the tiles resident on one XCD share A and B panels in
//     that XCD's L2.
//   * dW has few output tiles and K = rows (32768): K is split across blockIdx.y,
//     fp32 partial tiles go to scratch and a second kernel adds them in slice order
//     (deterministic), applying accumulate and the dtype conversion.
//
// Shapes the MFMA path does not cover (K not a multiple of 64, leading dimensions
// or pointers not 16-byte aligned, fp32 storage) run on a plain LDS-tiled fp32
// kernel with the same semantics.
#include "gemm.hpp"

#include <algorithm>
#include <cstdlib>
#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kBK = 64;          // K step per LDS tile
constexpr int kLdsStride = 72;   // elements per LDS row (64 + 8 padding)
constexpr int kXcds = 8;
constexpr int kGroupRows = 8;    // tile-rows per L2 locality group

using acc_t = vec_t<float, 16>;

template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
    using frag = vec_t<bf16_t, 8>;
    __device__ static __forceinline__ acc_t run(frag a, frag b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <>
struct Mfma<f16_t> {
    using frag = vec_t<f16_t, 8>;
    __device__ static __forceinline__ acc_t run(frag a, frag b, acc_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

using u32x4 = vec_t<unsigned int, 4>;

struct KernelArgs {
    const void* a;
    const void* b;
    void* c;            // T* (or float* when c_f32), or float partials when split
    const void* bias;
    int m, n, k;
    long lda, ldb, ldc;
    int tiles_m, tiles_n;
    int k_tiles_per_slice;  // K tiles (of 64) handled by one blockIdx.y
    int accumulate;
    int c_f32;
};

// ---- k-contiguous operand: rows x 64 tile, 128-bit chunks ---------------------
template <int ROWS>
struct DirectTile {
    static constexpr int kChunks = ROWS * (kBK / 8) / kThreads;  // per thread
    u32x4 regs[kChunks];

    template <typename T>
    __device__ __forceinline__ void load(const T* base, long ld, int row0, int row_limit, int k0) {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int chunk = threadIdx.x + i * kThreads;
            const int row = chunk >> 3, kc = chunk & 7;
            // Rows past the edge are clamped to the last valid row instead of being predicated: they
            // only feed C rows/columns that are never stored, and a branch-free loop lets the loads
            // stay in flight across the MFMAs of the current tile.
            const int safe = min(row0 + row, row_limit - 1);
            regs[i] = *reinterpret_cast<const u32x4*>(base + static_cast<long>(safe) * ld + k0 + kc * 8);
        }
    }
    template <typename T>
    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < kChunks; ++i) {
            const int chunk = threadIdx.x + i * kThreads;
            const int row = chunk >> 3, kc = chunk & 7;
            *reinterpret_cast<u32x4*>(lds + row * kLdsStride + kc * 8) = regs[i];
        }
    }
};

// ---- n-contiguous operand: 64(k) x COLS tile, transposed in registers ---------
template <int COLS, int THREAD_SHIFT>
struct TransposedTile {
    static constexpr int kTasks = (kBK / 8) * (COLS / 8);
    static constexpr int kPerThread = (kTasks + kThreads - 1) / kThreads;
    u32x4 regs[kPerThread][8];

    __device__ __forceinline__ static int task_of(int i) {
        return ((threadIdx.x + THREAD_SHIFT) & (kThreads - 1)) + i * kThreads;
    }
    template <typename T>
    __device__ __forceinline__ void load(const T* base, long ld, int col0, int col_limit, int k0) {
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int task = task_of(i);
            const int safe_task = min(task, kTasks - 1);
            // Eight adjacent lanes take the eight k-groups of one column block: their 16-byte loads
            // fill one 128-byte line per k row, and their LDS stores below fall in one contiguous
            // 128-byte row segment (no bank conflicts).
            const int kg = safe_task % (kBK / 8), nc = safe_task / (kBK / 8);
            // Column blocks past the edge are clamped (see DirectTile::load); col_limit is a multiple of 8.
            const int safe_col = min(col0 + nc * 8, col_limit - 8);
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                regs[i][r] = *reinterpret_cast<const u32x4*>(base + static_cast<long>(k0 + kg * 8 + r) * ld +
                                                             safe_col);
            }
        }
    }
    template <typename T>
    __device__ __forceinline__ void store(T* lds) const {
#pragma unroll
        for (int i = 0; i < kPerThread; ++i) {
            const int task = task_of(i);
            if (task >= kTasks) continue;
            const int kg = task % (kBK / 8), nc = task / (kBK / 8);
#pragma unroll
            for (int j = 0; j < 8; ++j) {  // output row: column nc*8 + j, k = kg*8 .. kg*8+7
                u32x4 out;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const unsigned int lo = regs[i][2 * q][j >> 1];
                    const unsigned int hi = regs[i][2 * q + 1][j >> 1];
                    out[q] = (j & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u)
                                     : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
                }
                *reinterpret_cast<u32x4*>(lds + (nc * 8 + j) * kLdsStride + kg * 8) = out;
            }
        }
    }
};

template <typename T, int BM, int BN, bool A_K, bool B_K, bool SPLIT>
__global__ __launch_bounds__(kThreads) void gemm_mfma_kernel(KernelArgs p) {
    using frag_t = typename Mfma<T>::frag;
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / 32, TN = WN / 32;
    extern __shared__ __align__(16) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    constexpr int kATile = BM * kLdsStride, kBTile = BN * kLdsStride;
    // Stage s holds [A tile | B tile] at smem + s * kStage. Offsets are added to the one shared base
    // so that every access is provably an LDS access (ds_read/ds_write, counted by lgkmcnt only).
    constexpr int kStage = kATile + kBTile;

    // XCD-contiguous, grouped tile order.
    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    const int logical = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (logical >= total) return;
    const int group_size = kGroupRows * p.tiles_n;
    const int group = logical / group_size;
    const int first_m = group * kGroupRows;
    const int rows_in_group = min(p.tiles_m - first_m, kGroupRows);
    const int in_group = logical - group * group_size;
    const int tile_m = first_m + in_group % rows_in_group;
    const int tile_n = in_group / rows_in_group;
    const int m0 = tile_m * BM, n0 = tile_n * BN;

    const int k_tiles_total = p.k / kBK;
    const int kt_begin = blockIdx.y * p.k_tiles_per_slice;
    const int kt_end = min(k_tiles_total, kt_begin + p.k_tiles_per_slice);

    const T* A = static_cast<const T*>(p.a);
    const T* B = static_cast<const T*>(p.b);

    DirectTile<BM> a_direct;
    DirectTile<BN> b_direct;
    TransposedTile<BM, 0> a_trans;
    TransposedTile<BN, (A_K ? 0 : kThreads / 2)> b_trans;

    auto load_tiles = [&](int kt) {
        const int k0 = kt * kBK;
        if constexpr (A_K) a_direct.load(A, p.lda, m0, p.m, k0); else a_trans.load(A, p.lda, m0, p.m, k0);
        if constexpr (B_K) b_direct.load(B, p.ldb, n0, p.n, k0); else b_trans.load(B, p.ldb, n0, p.n, k0);
    };
    auto store_tiles = [&](int buf) {
        if constexpr (A_K) a_direct.store(smem + buf * kStage); else a_trans.store(smem + buf * kStage);
        if constexpr (B_K) b_direct.store(smem + buf * kStage + kATile); else b_trans.store(smem + buf * kStage + kATile);
    };

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;
    const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;

    acc_t acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = acc_t(0.0f);

    if (kt_begin < kt_end) {
        load_tiles(kt_begin);
        store_tiles(0);
    }
    __syncthreads();
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        const int buf = (kt - kt_begin) & 1;
        const bool more = kt + 1 < kt_end;
        if (more) load_tiles(kt + 1);
        const T* as = smem + buf * kStage + (wm * WM + frag_row) * kLdsStride + frag_k;
        const T* bs = smem + buf * kStage + kATile + (wn * WN + frag_row) * kLdsStride + frag_k;
        // Fragments of K sub-step kk+1 are requested before the MFMAs of sub-step kk are issued.
        frag_t af[2][TM], bf[2][TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[0][i] = *reinterpret_cast<const frag_t*>(as + i * 32 * kLdsStride);
#pragma unroll
        for (int j = 0; j < TN; ++j) bf[0][j] = *reinterpret_cast<const frag_t*>(bs + j * 32 * kLdsStride);
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk + 1 < kBK / 16) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    af[nxt][i] = *reinterpret_cast<const frag_t*>(as + i * 32 * kLdsStride + (kk + 1) * 16);
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    bf[nxt][j] = *reinterpret_cast<const frag_t*>(bs + j * 32 * kLdsStride + (kk + 1) * 16);
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = Mfma<T>::run(bf[cur][j], af[cur][i], acc[i][j]);
        }
        if (more) store_tiles(buf ^ 1);
        __syncthreads();
    }

    // Epilogue. acc[i][j][4g+e] holds C[m, n] with m = lane%32, n = 8g + 4*(lane/32) + e. The tile
    // goes through LDS (fp32, row stride BN+4 so that the 16 lanes of a ds_write_b128 pass hit 16
    // different bank groups) and leaves it row by row, so that a wavefront stores 512 contiguous
    // bytes of C per instruction instead of 32 separate 16-byte pieces. Rounding to the storage
    // dtype still happens once, after bias and accumulate were added in fp32.
    constexpr int kStageStride = BN + 4;
    constexpr int kSmemBytes = 2 * (BM + BN) * kLdsStride * static_cast<int>(sizeof(T));
    constexpr int kPassRows = (BM * kStageStride * 4 <= kSmemBytes) ? BM : BM / 2;
    constexpr int kPasses = BM / kPassRows;
    static_assert(kPassRows * kStageStride * 4 <= kSmemBytes, "epilogue staging does not fit in LDS");
    static_assert(kPasses == 1 || kPassRows == WM, "a pass must be one row of wavefronts");
    float* stage = reinterpret_cast<float*>(smem_raw);
    const int m_lane = lane & 31, n_lane = (lane >> 5) * 4;
#pragma unroll
    for (int pass = 0; pass < kPasses; ++pass) {
        if (kPasses == 1 || wm == pass) {
            const int row_base = kPasses == 1 ? wm * WM : 0;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        vec_t<float, 4> v;
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * g + e];
                        const int row = row_base + i * 32 + m_lane;
                        const int col = wn * WN + j * 32 + g * 8 + n_lane;
                        *reinterpret_cast<vec_t<float, 4>*>(stage + row * kStageStride + col) = v;
                    }
                }
            }
        }
        __syncthreads();
        constexpr int kChunksPerRow = BN / 4;
        constexpr int kChunks = kPassRows * kChunksPerRow;
        for (int c = threadIdx.x; c < kChunks; c += kThreads) {
            const int r = c / kChunksPerRow, col = (c % kChunksPerRow) * 4;
            const int m = m0 + pass * kPassRows + r, n = n0 + col;
            if (m >= p.m || n >= p.n) continue;
            vec_t<float, 4> v = *reinterpret_cast<const vec_t<float, 4>*>(stage + r * kStageStride + col);
            if constexpr (SPLIT) {
                float* out = static_cast<float*>(p.c) +
                             (static_cast<long>(blockIdx.y) * p.m + m) * static_cast<long>(p.n) + n;
                *reinterpret_cast<vec_t<float, 4>*>(out) = v;
            } else {
                if (p.bias != nullptr) v += vec_to_f32<T, 4>(load_vec<T, 4>(static_cast<const T*>(p.bias) + n));
                if (p.c_f32) {
                    float* out = static_cast<float*>(p.c) + static_cast<long>(m) * p.ldc + n;
                    if (p.accumulate) v += *reinterpret_cast<const vec_t<float, 4>*>(out);
                    *reinterpret_cast<vec_t<float, 4>*>(out) = v;
                } else {
                    T* out = static_cast<T*>(p.c) + static_cast<long>(m) * p.ldc + n;
                    if (p.accumulate) v += vec_to_f32<T, 4>(load_vec<T, 4>(out));
                    store_vec<T, 4>(out, vec_from_f32<T, 4>(v));
                }
            }
        }
        if (pass + 1 < kPasses) __syncthreads();
    }
}

// C = Σ_slices partial (+ C) (+ bias), four columns per thread, slices in order.
template <typename T>
__global__ __launch_bounds__(kThreads) void splitk_reduce_kernel(void* __restrict__ c,
                                                                const float* __restrict__ partial,
                                                                const T* __restrict__ bias, int m, int n, long ldc,
                                                                int slices, int accumulate, int c_f32) {
    const long quads = static_cast<long>(m) * (n / 4);
    const long stride = static_cast<long>(m) * n;
    for (long q = static_cast<long>(blockIdx.x) * kThreads + threadIdx.x; q < quads;
         q += static_cast<long>(gridDim.x) * kThreads) {
        const long row = q / (n / 4);
        const int col = static_cast<int>(q - row * (n / 4)) * 4;
        vec_t<float, 4> v = *reinterpret_cast<const vec_t<float, 4>*>(partial + row * n + col);
        for (int s = 1; s < slices; ++s)
            v += *reinterpret_cast<const vec_t<float, 4>*>(partial + s * stride + row * n + col);
        if (bias != nullptr) v += vec_to_f32<T, 4>(load_vec<T, 4>(bias + col));
        if (c_f32) {
            float* out = static_cast<float*>(c) + row * ldc + col;
            if (accumulate) v += *reinterpret_cast<const vec_t<float, 4>*>(out);
            *reinterpret_cast<vec_t<float, 4>*>(out) = v;
        } else {
            T* out = static_cast<T*>(c) + row * ldc + col;
            if (accumulate) v += vec_to_f32<T, 4>(load_vec<T, 4>(out));
            store_vec<T, 4>(out, vec_from_f32<T, 4>(v));
        }
    }
}

// ---- plain fp32 kernel for everything the MFMA path does not take -------------
constexpr int kGenericTile = 32;

template <typename T>
__global__ __launch_bounds__(kGenericTile* kGenericTile / 4) void gemm_generic_kernel(KernelArgs p, int a_k, int b_k) {
    // 32x32 tile of C per block of 16x16 threads, 2x2 outputs per thread, K step 32.
    __shared__ float as[kGenericTile][kGenericTile + 1];
    __shared__ float bs[kGenericTile][kGenericTile + 1];
    const T* A = static_cast<const T*>(p.a);
    const T* B = static_cast<const T*>(p.b);
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const long m0 = static_cast<long>(blockIdx.y) * kGenericTile, n0 = static_cast<long>(blockIdx.x) * kGenericTile;
    float acc[2][2] = {{0.0f, 0.0f}, {0.0f, 0.0f}};
    for (long k0 = 0; k0 < p.k; k0 += kGenericTile) {
        for (int e = threadIdx.x; e < kGenericTile * kGenericTile; e += kGenericTile * kGenericTile / 4) {
            const int r = e / kGenericTile, c = e % kGenericTile;  // r: m (or n), c: k
            const long m = m0 + r, n = n0 + r, k = k0 + c;
            float av = 0.0f, bv = 0.0f;
            if (k < p.k) {
                if (m < p.m) av = to_f32(a_k ? A[m * p.lda + k] : A[k * p.lda + m]);
                if (n < p.n) bv = to_f32(b_k ? B[n * p.ldb + k] : B[k * p.ldb + n]);
            }
            as[r][c] = av;
            bs[r][c] = bv;
        }
        __syncthreads();
#pragma unroll 8
        for (int k = 0; k < kGenericTile; ++k) {
            const float a0 = as[ty][k], a1 = as[ty + 16][k];
            const float b0 = bs[tx][k], b1 = bs[tx + 16][k];
            acc[0][0] = fmaf(a0, b0, acc[0][0]);
            acc[0][1] = fmaf(a0, b1, acc[0][1]);
            acc[1][0] = fmaf(a1, b0, acc[1][0]);
            acc[1][1] = fmaf(a1, b1, acc[1][1]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const long m = m0 + ty + 16 * i, n = n0 + tx + 16 * j;
            if (m >= p.m || n >= p.n) continue;
            float v = acc[i][j];
            if (p.bias != nullptr) v += to_f32(static_cast<const T*>(p.bias)[n]);
            if (p.c_f32) {
                float* out = static_cast<float*>(p.c) + m * p.ldc + n;
                *out = p.accumulate ? v + *out : v;
            } else {
                T* out = static_cast<T*>(p.c) + m * p.ldc + n;
                *out = from_f32<T>(p.accumulate ? v + to_f32(*out) : v);
            }
        }
    }
}

// ------------------------------------------------------------------- host side
template <typename T, int BM, int BN, bool A_K, bool B_K, bool SPLIT>
int launch_mfma(const KernelArgs& p, int slices, hipStream_t stream) {
    constexpr std::size_t smem = 2 * static_cast<std::size_t>(BM + BN) * kLdsStride * sizeof(T);
    auto kernel = gemm_mfma_kernel<T, BM, BN, A_K, B_K, SPLIT>;
    static bool configured = false;
    if (!configured) {
        CGPTX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)));
        configured = true;
    }
    const int total = p.tiles_m * p.tiles_n;
    const int per_xcd = (total + kXcds - 1) / kXcds;
    hipLaunchKernelGGL(kernel, dim3(per_xcd * kXcds, slices), dim3(kThreads), smem, stream, p);
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

template <typename T, int BM, int BN, bool SPLIT>
int launch_layout(const KernelArgs& p, bool a_k, bool b_k, int slices, hipStream_t stream) {
    if (a_k && b_k) return launch_mfma<T, BM, BN, true, true, SPLIT>(p, slices, stream);
    if (a_k && !b_k) return launch_mfma<T, BM, BN, true, false, SPLIT>(p, slices, stream);
    if (!a_k && !b_k) return launch_mfma<T, BM, BN, false, false, SPLIT>(p, slices, stream);
    return fail(CGPTX_RUNTIME, "gemm: unsupported operand layout");
}

// CGPTX_GEMM_TILE=128|256 pins the tile size (for experiments); anything else = automatic.
int forced_tile() {
    static const int value = [] {
        const char* text = std::getenv("CGPTX_GEMM_TILE");
        if (text == nullptr) return 0;
        const int v = std::atoi(text);
        return (v == 128 || v == 256) ? v : 0;
    }();
    return value;
}

template <typename T, int BM, int BN>
int run_config(const GemmArgs& g, KernelArgs p, hipStream_t stream) {
    p.tiles_m = (p.m + BM - 1) / BM;
    p.tiles_n = (p.n + BN - 1) / BN;
    const int k_tiles = p.k / kBK;
    const long tiles = static_cast<long>(p.tiles_m) * p.tiles_n;
    const long want_blocks = static_cast<long>(compute_units()) * (BM == 256 ? 1 : 2);
    int slices = 1;
    if (!g.no_split && tiles < want_blocks && k_tiles >= 16) {
        slices = static_cast<int>(std::min<long>((want_blocks + tiles - 1) / tiles, k_tiles / 8));
        if (slices < 1) slices = 1;
    }
    p.k_tiles_per_slice = (k_tiles + slices - 1) / slices;
    slices = (k_tiles + p.k_tiles_per_slice - 1) / p.k_tiles_per_slice;
    if (slices == 1) return launch_layout<T, BM, BN, false>(p, g.a_k_contiguous, g.b_k_contiguous, 1, stream);
    void* mem = nullptr;
    if (int s = scratch(stream, static_cast<std::size_t>(slices) * g.m * g.n * sizeof(float), &mem)) return s;
    KernelArgs split = p;
    split.c = mem;
    if (int s = launch_layout<T, BM, BN, true>(split, g.a_k_contiguous, g.b_k_contiguous, slices, stream)) return s;
    const long quads = static_cast<long>(p.m) * (p.n / 4);
    const long blocks = std::min<long>((quads + kThreads - 1) / kThreads, static_cast<long>(compute_units()) * 8);
    hipLaunchKernelGGL((splitk_reduce_kernel<T>), dim3(static_cast<unsigned int>(blocks)), dim3(kThreads), 0, stream,
                       g.c, static_cast<const float*>(mem), static_cast<const T*>(g.bias), p.m, p.n, p.ldc, slices,
                       p.accumulate, p.c_f32);
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

template <typename T>
int run_typed(const GemmArgs& g, hipStream_t stream) {
    KernelArgs p{};
    p.a = g.a;
    p.b = g.b;
    p.c = g.c;
    p.bias = g.bias;
    p.m = static_cast<int>(g.m);
    p.n = static_cast<int>(g.n);
    p.k = static_cast<int>(g.k);
    p.lda = static_cast<long>(g.lda);
    p.ldb = static_cast<long>(g.ldb);
    p.ldc = static_cast<long>(g.ldc);
    p.accumulate = g.accumulate ? 1 : 0;
    p.c_f32 = g.c_is_f32 ? 1 : 0;

    bool fast = false;
    if constexpr (!std::is_same_v<T, float>) {
        const std::size_t c_elem = g.c_is_f32 ? 4 : sizeof(T);
        fast = g.k % kBK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.n % 8 == 0 && g.m % 8 == 0 &&
               is_aligned16(g.a) && is_aligned16(g.b) && (g.ldc * c_elem) % 16 == 0 && is_aligned16(g.c) &&
               (g.bias == nullptr || (reinterpret_cast<std::uintptr_t>(g.bias) & 7u) == 0) &&
               !(!g.a_k_contiguous && g.b_k_contiguous);
    }
    if (!fast) {
        const dim3 grid(static_cast<unsigned int>((g.n + kGenericTile - 1) / kGenericTile),
                        static_cast<unsigned int>((g.m + kGenericTile - 1) / kGenericTile));
        hipLaunchKernelGGL((gemm_generic_kernel<T>), grid, dim3(kGenericTile * kGenericTile / 4), 0, stream, p,
                           g.a_k_contiguous ? 1 : 0, g.b_k_contiguous ? 1 : 0);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    }
    if constexpr (!std::is_same_v<T, float>) {
        // 256x256 tiles (one block per CU, 64 MFMAs per wavefront and K step) when they still give
        // every CU a tile; otherwise 128x128 tiles, with K split when even those are too few.
        const long big_tiles = static_cast<long>((g.m + 255) / 256) * static_cast<long>((g.n + 255) / 256);
        const int forced = forced_tile();
        const bool big = forced == 256 || (forced == 0 && big_tiles * 5 >= static_cast<long>(compute_units()) * 4);
        if (big) return run_config<T, 256, 256>(g, p, stream);
        return run_config<T, 128, 128>(g, p, stream);
    }
    return CGPTX_OK;
}

}  // namespace

int gemm(const GemmArgs& g, hipStream_t stream) {
    if (g.a == nullptr || g.b == nullptr || g.c == nullptr || g.m == 0 || g.n == 0 || g.k == 0)
        return fail(CGPTX_INVALID_ARGUMENT, "gemm: null or empty operand");
    constexpr std::size_t i32max = std::numeric_limits<int>::max();
    if (g.m > i32max || g.n > i32max || g.k > i32max)
        return fail(CGPTX_OVERFLOW, "gemm: dimension exceeds int range");
    return dispatch_dtype(g.dtype, [&]<typename T>() -> int { return run_typed<T>(g, stream); });
}

}  // namespace cgptx
