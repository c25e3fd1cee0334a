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
//     and walks K in steps of 32. Each wavefront owns (BM/2) x (BN/2) and issues
//     v_mfma_f32_16x16x32 (bf16 or f16): per flop that form moves half the accumulator
//     data of the 32x32x16 one, which counts on a chip whose clock is power-limited.
//   * The kernel is persistent: one block per CU slot walks its share of the work items
//     (output tile x K slice). The 8 XCDs (blocks are dealt round-robin to them) each take
//     a contiguous eighth of the items, ordered in groups of 8 tile-rows, so that the
//     tiles in flight on one XCD share A and B panels in that XCD's L2 (2 tile-rows for
//     the kernel whose epilogue reads and writes whole rows of a wider matrix).
//   * Operand tiles go global -> LDS with buffer_load ... lds (no staging registers, no
//     LDS stores, one loop-invariant per-lane offset) into a ring of five LDS stages:
//     one being multiplied, up to three K tiles in flight, one being refilled. LDS rows
//     cannot be padded that way; a chunk swizzle keeps the fragment reads conflict-free.
//   * Operands that are not k-contiguous in memory (dX's weight, both dW operands) sit
//     in LDS as they are in memory and are transposed by the LDS read itself
//     (ds_read_b64_tr_b16): no transpose pass over HBM, no VALU shuffles.
//   * The K loop is a software pipeline with one barrier per K tile whose issue order is
//     pinned in the source: every MFMA is followed by its share of the fragment reads and
//     of the loads, the wait for the next K tile sits in the middle of the tile, and the
//     loop has no data-dependent branch (edges are clamped or zero-filled by the buffer
//     range check, never predicated).
//   * MFMA is issued as (B-fragment, A-fragment), so a lane ends up holding four
//     consecutive n for one m per accumulator; each wavefront stages its part of the
//     finished tile in a private piece of LDS and writes it out row by row (256
//     contiguous bytes per row), with bias / residual / old C added in fp32 and one
//     rounding to the dtype. The next item's first K tiles are requested meanwhile.
//   * dW has few output tiles and K = rows (32768): K is split into slices (work items),
//     fp32 partial tiles go to scratch and a second kernel adds them in slice order
//     (deterministic), applying accumulate and the dtype conversion.
//
// Shapes the streamed path does not cover (K not a multiple of 32, leading dimensions
// or pointers not 16-byte aligned, fp32 storage) run on an fp32 matrix-core kernel
// (v_mfma_f32_32x32x2_f32, register-staged operand tiles) with the same semantics.
#include "gemm.hpp"

#include <algorithm>
#include <type_traits>
#include <utility>
#include <cstdlib>
#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kBK = 32;          // K step per LDS stage
// LDS stages of a block: one being multiplied, one being refilled, the rest in flight. 256x256
// blocks own a CU (5 x 32 KiB), 128x128 blocks run two per CU (5 x 16 KiB each).
constexpr int stages_for(int /*bm*/, int /*bn*/) { return 5; }
constexpr int kXcds = 8;


using acc_t = vec_t<float, 4>;

// c += a x b with v_mfma_f32_16x16x32 (a: 16 rows x 32 k, b: 32 k x 16 columns; lane l holds row or
// column l%16, k = 8*(l/16) .. +7; c: lane l holds rows 4*(l/16) .. +3 of column l%16). Written as
// assembly so that the accumulator is updated in place: the four-register form of the instruction
// does not tie its result to its addend, and with all 256 accumulator registers in use the register
// allocator would otherwise shuffle accumulators around every MFMA. The kernel keeps the distances
// the hardware asks for by construction: an accumulator is touched once per K tile (64 or 16 MFMAs
// apart), zeroed long before its first MFMA and read by the epilogue only after a barrier.
template <typename T>
struct Mfma;
template <>
struct Mfma<bf16_t> {
    using frag = vec_t<bf16_t, 8>;
    __device__ static __forceinline__ void run(acc_t& c, const frag& a, const frag& b) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    // c = a x b: the first K tile of an item starts the sums, so the accumulators are never cleared.
    __device__ static __forceinline__ void start(acc_t& c, const frag& a, const frag& b) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }
};
template <>
struct Mfma<f16_t> {
    using frag = vec_t<f16_t, 8>;
    __device__ static __forceinline__ void run(acc_t& c, const frag& a, const frag& b) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    }
    __device__ static __forceinline__ void start(acc_t& c, const frag& a, const frag& b) {
        asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
    }
};

using u32x4 = vec_t<unsigned int, 4>;

struct KernelSegments {
    const void* ptr[3];
    long ld[3];
    int cols[3];
    int count;
};

struct KernelArgs {
    const void* a;
    const void* b;
    void* c;            // T* (or float* when c_f32), or float partials when split
    const void* bias;
    const void* residual;  // T*, row stride ldr, or null
    const float* addend;   // fp32 [M, N], row stride ld_addend, added before anything else, or null
    long ld_addend;
    int m, n, k;
    long lda, ldb, ldc, ldr;
    int tiles_m, tiles_n;
    int k_tiles_per_slice;  // K tiles handled by one work item
    int slices;             // K slices per output tile
    int accumulate;
    int c_f32;
    KernelSegments a_seg, c_seg;  // column segments of A (as stored) and of C; count 0 = one buffer
    // ceil(2^32 / (group rows * tiles_n)) when multiplying by it divides every item index of the
    // launch exactly, else 0 (the kernel then divides).
    unsigned int group_reciprocal;
    int group_rows_log2;  // tile-rows per L2 locality group: 1 << group_rows_log2
    void* act;      // SWIGLU kernels: [M, inter] = silu(gate) * up, T*
    long ld_act;
    const void* saved;  // GRAD kernels: the forward's [M, 2 * inter] = [gate | up], T*
    long ld_saved;
    int inter;      // SWIGLU kernels: columns of gate (= of up); n = 2 * inter
    // Stacked products (weight-gradient layout only): rows of C per product (0 = one product) and what a and b (or
    // A's segments) move by from one product to the next, in elements.
    int batch_rows;
    long a_batch_stride, b_batch_stride;
    long a_seg_batch_stride[3];
};

// The column segment (of up to three) that holds column `col`, picked with selects: indexing the
// kernel-argument arrays by a run-time value would move them to private memory.
struct SegmentPick {
    const void* ptr;
    long ld;
    int first;  // first column of the segment
    int cols;
    int index;  // which segment
};
__device__ __forceinline__ SegmentPick pick_segment(const KernelSegments& seg, int col) {
    const int end0 = seg.cols[0], end1 = end0 + seg.cols[1];
    const bool in1 = seg.count > 1 && col >= end0;
    const bool in2 = seg.count > 2 && col >= end1;
    SegmentPick pick;
    pick.ptr = in2 ? seg.ptr[2] : in1 ? seg.ptr[1] : seg.ptr[0];
    pick.ld = in2 ? seg.ld[2] : in1 ? seg.ld[1] : seg.ld[0];
    pick.first = in2 ? end1 : in1 ? end0 : 0;
    pick.cols = in2 ? seg.cols[2] : in1 ? seg.cols[1] : seg.cols[0];
    pick.index = in2 ? 2 : in1 ? 1 : 0;
    return pick;
}

// s_waitcnt immediate that waits until at most `count` vector-memory operations are outstanding
// (and for nothing else).
constexpr int vmcnt_immediate(int count) { return (count & 15) | ((count >> 4) << 14) | 0x0F70; }

// Buffer descriptor (raw buffer, range-checked) over `bytes` bytes starting at base (both the same
// for all lanes). The words are pinned to scalar registers: 64-bit comparisons have no scalar form,
// and one of them on the way would drag the descriptor, and every address derived with it, into
// vector registers.
__device__ __forceinline__ u32x4 make_rsrc(const void* base, long bytes) {
    const unsigned long address = reinterpret_cast<unsigned long>(base);
    const unsigned int size_low = static_cast<unsigned int>(bytes);
    const unsigned int size_high = static_cast<unsigned int>(static_cast<unsigned long>(bytes) >> 32);
    u32x4 words;
    words[0] = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(address));
    words[1] = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(address >> 32) & 0xFFFFu);  // stride 0
    words[2] = __builtin_amdgcn_readfirstlane(size_high != 0 ? 0xFFFFFFFFu : size_low);
    words[3] = 0x00020000u;
    return words;
}

// One wavefront-wide 16-byte-per-lane load from a buffer straight into LDS: lane l's bytes land at
// lds_base + LDS_OFFSET + 16 l. Returns soffset + step, the scalar offset of the operand's next load
// (that addition sits between the write of M0 and the load, which need one instruction between them
// anyway). Written as assembly on purpose: the compiler would order every later LDS read after *all*
// outstanding loads of this kind (vmcnt(0)), which defeats keeping several K tiles in flight; the
// kernel counts its loads itself (vmcnt_immediate). M0 is used by nothing else here.
template <int LDS_OFFSET>
__device__ __forceinline__ unsigned int load_to_lds(const u32x4& rsrc, unsigned int lds_base, int voffset,
                                                    unsigned int soffset, unsigned int step) {
    unsigned int next;
    asm volatile("s_add_u32 m0, %1, %2\n\ts_add_u32 %0, %3, %4\n\tbuffer_load_dwordx4 %5, %6, %3 offen lds"
                 : "=&s"(next)
                 : "s"(lds_base), "n"(LDS_OFFSET), "s"(soffset), "s"(step), "v"(voffset), "s"(rsrc)
                 : "scc");
    return next;
}

// Workgroup barrier without the fence __syncthreads() carries: LDS reads still in flight may
// cross it (their registers are waited for where they are used).
__device__ __forceinline__ void barrier_only() { asm volatile("s_barrier" ::: "memory"); }

// Where a wavefront's loads of one operand's K tile come from: load i reads at scalar offset
// soffset + i * step.
struct TileCursor {
    u32x4 rsrc;
    int voffset;
    unsigned int soffset;
    unsigned int step;
    unsigned int step2;  // advance after the operand's odd-numbered loads (differs from step only for SWIGLU's B)
};

template <int BEGIN, int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
    (f(std::integral_constant<int, BEGIN + I>{}), ...);
}
// f(integral_constant<int, i>) for i = BEGIN .. END-1, unrolled at compile time.
template <int BEGIN, int END, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    static_for_impl<BEGIN>(std::make_integer_sequence<int, (END > BEGIN ? END - BEGIN : 0)>{}, f);
}

template <typename T>
__device__ __forceinline__ unsigned int lds_address_of(const T* p) {
    return static_cast<unsigned int>(reinterpret_cast<unsigned long>((__attribute__((address_space(3))) const T*)(p)));
}

// Operand tiles travel global -> LDS with buffer_load ... lds: a wavefront-wide load drops
// 64 x 16 B contiguously into LDS, no staging registers and no LDS stores, and the only per-lane
// address is a loop-invariant byte offset (the K position is a scalar offset). LDS rows therefore
// cannot be padded; bank conflicts are avoided by storing 16-byte chunk c of a row at chunk
// position c ^ swizzle(row) — the lane that owns an LDS slot fetches the matching global chunk.

// ---- operand stored [ROWS, K] (k-contiguous): ROWS x kBK slab, unpadded LDS rows ---------------
// One load instruction covers 1024 B = kRowsPerLoad rows; wavefront w issues the loads of row
// groups w, w+4, ... The chunk swizzle is (row / rows per 256 B) mod chunks per row: the 16 rows a
// quarter-wavefront reads with ds_read_b128 then hit the 16 different 16-byte positions of a
// 256-byte bank period.
template <typename T, int ROWS>
struct KTile {
    using frag_t = typename Mfma<T>::frag;
    static constexpr int kChunksPerRow = kBK / 8;
    static constexpr int kRowsPerLoad = 64 / kChunksPerRow;
    static constexpr int kElems = ROWS * kBK;
    static constexpr int kLoads = ROWS / kRowsPerLoad / kWaves;  // load instructions per wavefront and tile

    u32x4 rsrc = {0u, 0u, 0u, 0u};
    int voffset = 0;
    unsigned int group_bytes = 0;  // kRowsPerLoad rows further in global memory

    __device__ __forceinline__ static int swizzle(int row) { return (row / (128 / kBK)) % kChunksPerRow; }

    // base: element (row0, 0) of the operand; rows past rows_left only feed C rows that are never
    // stored (they read zeros or whatever follows, never out of the allocation's last row).
    __device__ __forceinline__ void init(const T* base, long ld, int rows_left, int k_total, int wave) {
        const int lane = threadIdx.x & (kWave - 1);
        rsrc = make_rsrc(base, (static_cast<long>(rows_left - 1) * ld + k_total) * static_cast<long>(sizeof(T)));
        const int row = lane / kChunksPerRow;
        // The tile row of this lane's slot is (i*4 + wave) * kRowsPerLoad + row; its swizzle does not depend on i.
        voffset = static_cast<int>(row * ld * sizeof(T)) +
                  (((lane % kChunksPerRow) ^ swizzle(wave * kRowsPerLoad + row)) * 16);
        group_bytes = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(kRowsPerLoad * ld * sizeof(T)));
    }
    // Scalar offset of wavefront `wave`'s first load of the tile that starts at column k0.
    __device__ __forceinline__ unsigned int first_offset(int k0, int wave) const {
        return wave * group_bytes + k0 * static_cast<unsigned int>(sizeof(T));
    }
    // Element offset of the lane's fragment within a 16-row block (the whole K tile is one MFMA
    // step): row lane%16, k = 8 (lane/16) .. +7. The swizzle of a row does not depend on the block.
    __device__ __forceinline__ static int lane_offset(int lane) {
        return (lane & 15) * kBK + (((lane >> 4) ^ swizzle(lane & 15)) * 8);
    }
    __device__ __forceinline__ static frag_t frag(const T* tile, int block0, int offset) {
        return *reinterpret_cast<const frag_t*>(tile + block0 * kBK + offset);
    }
};

// ---- operand stored [K, COLS] (n-contiguous): 32 x COLS slab kept in that order in LDS ---------
// The transpose happens on the way out of LDS: ds_read_b64_tr_b16 hands lane n of a 16-lane group
// the four k-values of column n from a 4(k) x 16(n) block, so two of them build the 8-k fragment of
// one column. swizzle(k row) = 4*(row%4) on the chunk index: the four k rows that 32 lanes read sit
// in four different 64-byte windows of the 256-byte bank period.
template <typename T, int COLS>
struct NTile {
    using frag_t = typename Mfma<T>::frag;
    static constexpr int kChunksPerRow = COLS / 8;
    static constexpr int kRowsPerLoad = 64 / kChunksPerRow;  // k rows one load instruction covers (2 or 4)
    static constexpr int kElems = kBK * COLS;
    static constexpr int kLoads = kBK / kRowsPerLoad / kWaves;

    u32x4 rsrc = {0u, 0u, 0u, 0u};
    int voffset = 0;
    unsigned int group_bytes = 0;  // kRowsPerLoad k rows further in global memory

    // base: element (0, col0) of the operand. Column chunks past cols_left are clamped to the last
    // valid chunk: they only feed C columns that are never stored.
    __device__ __forceinline__ void init(const T* base, long ld, int cols_left, int k_total, int wave) {
        const int lane = threadIdx.x & (kWave - 1);
        rsrc = make_rsrc(base, (static_cast<long>(k_total - 1) * ld + cols_left) * static_cast<long>(sizeof(T)));
        const int row = lane / kChunksPerRow;                  // within the instruction's rows
        const int k_row = (wave * kRowsPerLoad + row) & 3;     // low bits of the tile row (groups step by 4*kRowsPerLoad)
        const int chunk = min((lane % kChunksPerRow) ^ (k_row << 2), cols_left / 8 - 1);
        voffset = static_cast<int>(row * ld * sizeof(T)) + chunk * 16;
        group_bytes = __builtin_amdgcn_readfirstlane(static_cast<unsigned int>(kRowsPerLoad * ld * sizeof(T)));
    }
    // Scalar offset of wavefront `wave`'s first load of the tile that starts at row k0.
    __device__ __forceinline__ unsigned int first_offset(int k0, int wave) const {
        return (wave + k0 / kRowsPerLoad) * group_bytes;
    }
    // Lane i of a 16-lane group addresses k row i/4, columns 4*(i%4) .. +3 of the group's 4 x 16
    // block; group g (lanes 16g .. 16g+15) takes the k values 8g .. 8g+7 of the fragment's 16
    // columns in two reads (k rows +0..3, +4..7). The offset is for the first read; block0 is a
    // multiple of 16.
    __device__ __forceinline__ static int lane_offset(int lane, int block0) {
        const int k_row = (lane >> 4) * 8 + ((lane & 15) >> 2);
        const int chunk = ((block0 / 8) ^ ((k_row & 3) << 2)) + ((lane & 3) >> 1);
        return k_row * COLS + chunk * 8 + (lane & 1) * 4;
    }
    __device__ __forceinline__ static frag_t frag(const T* tile, int offset) {
        using s16x4 = vec_t<short, 4>;
        using lds_ptr = __attribute__((address_space(3))) s16x4*;
        const T* q = tile + offset;
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(q + 4 * COLS));
        vec_t<short, 8> both;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            both[e] = lo[e];
            both[4 + e] = hi[e];
        }
        return __builtin_bit_cast(frag_t, both);
    }
};

template <typename T, int BM, int BN, bool A_K, bool B_K>
struct TileLayout {
    using ATile = std::conditional_t<A_K, KTile<T, BM>, NTile<T, BM>>;
    using BTile = std::conditional_t<B_K, KTile<T, BN>, NTile<T, BN>>;
    static constexpr int kStage = ATile::kElems + BTile::kElems;  // elements per LDS stage: [A | B]
    static constexpr int kStages = stages_for(BM, BN);
    static constexpr int kSmemBytes = kStages * kStage * static_cast<int>(sizeof(T));
};

// One workgroup per CU slot walks its share of the work items (output tile x K slice) one after
// the other: the first K tiles of the next item are requested before the epilogue of the current
// one, whose stores then drain under the next item's MFMAs.
// SEGMENTED: A is stored [M, K] in up to three column segments (separate buffers along K).
// RESIDUAL: the epilogue adds a residual to a 16-bit result and nothing else (the output
// projections of a transformer block); a kernel of its own, so that each kernel carries one
// straight-line epilogue besides the general one.
// SWIGLU: B is the concatenated [gate; up] weight ([2·inter, K]) and C the concatenated [gate | up]
// activation; the kernel also writes silu(gate)·up. A tile's 256 columns are 128 gate columns and
// the 128 up columns of the same indices, interleaved in units of 64 so that each wavefront holds
// gate and up of its 64 indices in the same lanes: the B rows of an LDS tile are
// [gate 0-63 | up 0-63 | gate 64-127 | up 64-127] (one unit per load instruction of a wavefront,
// so only the scalar offsets of the loads change), and the epilogue computes the product from the
// rounded gate and up values, as the separate operator would from memory.
template <typename T, int BM, int BN, bool A_K, bool B_K, bool SPLIT, bool SEGMENTED, bool RESIDUAL = false,
          bool SWIGLU = false, bool GRAD = false>
__global__ __launch_bounds__(kThreads) void gemm_mfma_kernel(KernelArgs p) {
    static_assert(!GRAD || (A_K && !B_K && !SPLIT && !SEGMENTED && !RESIDUAL && !SWIGLU && BN == 256),
                  "the SwiGLU gradient epilogue belongs to the plain input-gradient kernel with 256-wide tiles");
    static_assert(!SEGMENTED || (A_K && !SPLIT), "segments along K are read by the unsplit kernels only");
    static_assert(!RESIDUAL || (!SPLIT && !SEGMENTED), "the residual epilogue belongs to plain unsplit kernels");
    static_assert(!SWIGLU || (A_K && B_K && !SPLIT && !SEGMENTED && !RESIDUAL && BN == 256),
                  "the SwiGLU epilogue belongs to the plain forward kernel with 256-wide tiles");
    using frag_t = typename Mfma<T>::frag;
    using Layout = TileLayout<T, BM, BN, A_K, B_K>;
    using ATile = typename Layout::ATile;
    using BTile = typename Layout::BTile;
    static_assert(BM == BN, "the epilogue staging assumes square tiles");
    constexpr int WM = BM / 2, WN = BN / 2;
    constexpr int TM = WM / 16, TN = WN / 16;  // 16 x 16 MFMA blocks of a wavefront's part
    extern __shared__ __align__(1024) unsigned char smem_raw[];
    T* smem = reinterpret_cast<T*>(smem_raw);
    // Stage s holds [A tile | B tile] at smem + s * kStage.
    constexpr int kStage = Layout::kStage;
    constexpr int kStages = Layout::kStages;
    constexpr int kATile = ATile::kElems;
    constexpr unsigned int kStageBytes = kStage * sizeof(T);

    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int wm = wave >> 1, wn = wave & 1;

    // Work items are numbered slice-major (all tiles of K slice 0, then of slice 1, ...), tiles in
    // groups of 1 << group_rows_log2 tile-rows, down the rows first. Blocks are dealt round-robin to the 8
    // XCDs, so XCD x takes the x-th eighth of the items and its blocks walk it side by side: the
    // items in flight on one XCD are neighbours and share A and B panels in that XCD's L2.
    const int tiles = p.tiles_m * p.tiles_n;
    const int items = tiles * p.slices;
    const int per_xcd = (items + kXcds - 1) / kXcds;
    const int item_stride = gridDim.x / kXcds;
    const int item_end = min(items, static_cast<int>(blockIdx.x % kXcds + 1) * per_xcd);
    int item = static_cast<int>(blockIdx.x % kXcds) * per_xcd + static_cast<int>(blockIdx.x / kXcds);
    if (item >= item_end) return;

    struct Item {
        int m0, n0, slice, kt_begin, kt_end;
    };
    auto locate = [&](int index) __attribute__((always_inline)) {
        // Integer divisions by run-time values cost some thirty scalar instructions each, with
        // nothing to hide them between two items: unsplit launches skip the first, the second is a
        // multiplication by a reciprocal the host prepared, the third a shift in all but the last,
        // ragged group of tile rows.
        Item w;
        w.slice = p.slices == 1 ? 0 : index / tiles;
        const int logical = index - w.slice * tiles;
        const int group_rows = 1 << p.group_rows_log2;
        const int group_size = p.tiles_n << p.group_rows_log2;
        const int group = p.group_reciprocal != 0u
                              ? static_cast<int>(__umulhi(static_cast<unsigned int>(logical), p.group_reciprocal))
                              : logical / group_size;
        const int first_m = group << p.group_rows_log2;
        const int rows_in_group = min(p.tiles_m - first_m, group_rows);
        const int in_group = logical - group * group_size;
        const int column = rows_in_group == group_rows ? in_group >> p.group_rows_log2 : in_group / rows_in_group;
        w.m0 = (first_m + in_group - column * rows_in_group) * BM;
        w.n0 = column * BN;
        w.kt_begin = w.slice * p.k_tiles_per_slice;
        w.kt_end = min(p.k / kBK, w.kt_begin + p.k_tiles_per_slice);
        return w;
    };

    // The operand sources of the item whose K tiles are being requested. A may be given as up to
    // three column segments in separate buffers. Stored [M, K]: the K range is segmented and the
    // source changes along the K loop (boundaries a_end0 / a_end1). Stored [K, M]: the M range is
    // segmented and the item's rows pick their buffer once.
    ATile a_src, a_src1, a_src2;
    BTile b_src;
    int a_end0 = std::numeric_limits<int>::max(), a_end1 = std::numeric_limits<int>::max();
    int src_begin = 0, src_end = 0;  // K tiles of that item
    auto open = [&](const Item& w) __attribute__((always_inline)) {
        const int m0 = w.m0, n0 = w.n0;
        src_begin = w.kt_begin;
        src_end = w.kt_end;
        long b_shift = 0;
        if constexpr (A_K && !SEGMENTED) {
            a_src.init(static_cast<const T*>(p.a) + static_cast<long>(m0) * p.lda, p.lda, p.m - m0, p.k, wave);
        } else if constexpr (A_K) {
            // All three sources are set up unconditionally (absent segments repeat the first and
            // are never selected): conditional set-up would be merged into one piece of code that
            // writes through a pointer, which keeps the sources in memory.
            const int segments = p.a_seg.count;
            const void* ptr0 = segments == 0 ? p.a : p.a_seg.ptr[0];
            const long ld0 = segments == 0 ? p.lda : p.a_seg.ld[0];
            const int cols0 = segments == 0 ? p.k : p.a_seg.cols[0];
            const void* ptr1 = segments > 1 ? p.a_seg.ptr[1] : ptr0;
            const long ld1 = segments > 1 ? p.a_seg.ld[1] : ld0;
            const int cols1 = segments > 1 ? p.a_seg.cols[1] : cols0;
            const void* ptr2 = segments > 2 ? p.a_seg.ptr[2] : ptr0;
            const long ld2 = segments > 2 ? p.a_seg.ld[2] : ld0;
            const int cols2 = segments > 2 ? p.a_seg.cols[2] : cols0;
            a_src.init(static_cast<const T*>(ptr0) + static_cast<long>(m0) * ld0, ld0, p.m - m0, cols0, wave);
            a_src1.init(static_cast<const T*>(ptr1) + static_cast<long>(m0) * ld1, ld1, p.m - m0, cols1, wave);
            a_src2.init(static_cast<const T*>(ptr2) + static_cast<long>(m0) * ld2, ld2, p.m - m0, cols2, wave);
            a_end0 = segments > 1 ? cols0 : std::numeric_limits<int>::max();
            a_end1 = segments > 2 ? cols0 + cols1 : std::numeric_limits<int>::max();
        } else {
            // Stacked products: the tile's rows of C name the product, and the operands move with it.
            long product = 0;
            int local_m0 = m0, rows = p.m;
            if constexpr (!B_K) {
                if (p.batch_rows > 0) {
                    product = m0 / p.batch_rows;
                    local_m0 = m0 - static_cast<int>(product) * p.batch_rows;
                    rows = p.batch_rows;
                    b_shift = product * p.b_batch_stride;
                }
            }
            const T* base = static_cast<const T*>(p.a) + product * p.a_batch_stride;
            long ld = p.lda;
            int first = 0, width = rows;
            if (p.a_seg.count > 0) {
                const SegmentPick pick = pick_segment(p.a_seg, local_m0);
                const long stride = pick.index == 2 ? p.a_seg_batch_stride[2]
                                    : pick.index == 1 ? p.a_seg_batch_stride[1] : p.a_seg_batch_stride[0];
                base = static_cast<const T*>(pick.ptr) + product * stride;
                ld = pick.ld;
                first = pick.first;
                width = pick.cols;
            }
            a_src.init(base + (local_m0 - first), ld, width - (local_m0 - first), p.k, wave);
        }
        if constexpr (SWIGLU) b_src.init(static_cast<const T*>(p.b) + static_cast<long>(n0 / 2) * p.ldb, p.ldb, p.n - n0 / 2, p.k, wave);
        else if constexpr (B_K) b_src.init(static_cast<const T*>(p.b) + static_cast<long>(n0) * p.ldb, p.ldb, p.n - n0, p.k, wave);
        else b_src.init(static_cast<const T*>(p.b) + b_shift + n0, p.ldb, p.n - n0, p.k, wave);
    };
    // K tiles past the end of the slice are still "loaded" (the loop stays free of data-dependent
    // branches and every wavefront always has the same number of loads in flight), but from an
    // offset beyond the buffer: the range check answers those at once with zeros, no memory traffic.
    // The source of a tile is picked with scalar selects, not branches, so that the loads can be
    // issued one by one between MFMAs.
    auto cursors = [&](int t, TileCursor& ca, TileCursor& cb) __attribute__((always_inline)) {
        const unsigned int past_end = src_begin + t >= src_end ? 0x80000000u : 0u;
        const int k0 = min(src_begin + t, src_end - 1) * kBK;
        if constexpr (SEGMENTED) {
            // Values first, then selects: a conditional between the objects' members would select
            // an address and keep all three sources in memory.
            const bool in1 = k0 >= a_end0, in2 = k0 >= a_end1;
            const u32x4 rsrc0 = a_src.rsrc, rsrc1 = a_src1.rsrc, rsrc2 = a_src2.rsrc;
            const int voffset0 = a_src.voffset, voffset1 = a_src1.voffset, voffset2 = a_src2.voffset;
            const unsigned int bytes0 = a_src.group_bytes, bytes1 = a_src1.group_bytes, bytes2 = a_src2.group_bytes;
            const int end0 = a_end0, end1 = a_end1;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const unsigned int w0 = rsrc0[e], w1 = rsrc1[e], w2 = rsrc2[e];
                ca.rsrc[e] = in2 ? w2 : in1 ? w1 : w0;
            }
            ca.voffset = in2 ? voffset2 : in1 ? voffset1 : voffset0;
            const unsigned int group_bytes = in2 ? bytes2 : in1 ? bytes1 : bytes0;
            const int start = in2 ? end1 : in1 ? end0 : 0;
            ca.soffset = (wave * group_bytes + (k0 - start) * static_cast<unsigned int>(sizeof(T))) | past_end;
            ca.step = kWaves * group_bytes;
            ca.step2 = ca.step;
        } else {
            ca.rsrc = a_src.rsrc;
            ca.voffset = a_src.voffset;
            ca.soffset = a_src.first_offset(k0, wave) | past_end;
            ca.step = kWaves * a_src.group_bytes;
            ca.step2 = ca.step;
        }
        cb.rsrc = b_src.rsrc;
        cb.voffset = b_src.voffset;
        cb.soffset = b_src.first_offset(k0, wave) | past_end;
        cb.step = kWaves * b_src.group_bytes;
        cb.step2 = cb.step;
        if constexpr (SWIGLU) {
            // gate unit -> up unit of the same rows (inter rows further), then back and 64 rows on.
            const unsigned int up = __builtin_amdgcn_readfirstlane(
                static_cast<unsigned int>(static_cast<long>(p.inter) * p.ldb * static_cast<long>(sizeof(T))));
            cb.step2 = cb.step - up;
            cb.step = up;
        }
    };
    // Load l of a K tile (A's loads first, then B's) into the stage whose LDS address, advanced to
    // this wavefront's first 1 KiB slot, is stage_lds. One load fills 1 KiB; the wavefronts' slots
    // interleave, so a wavefront's consecutive loads are kWaves KiB apart.
    constexpr int kLoadBytes = 64 * 16;
    constexpr int kATileBytes = kATile * static_cast<int>(sizeof(T));
    auto issue_one = [&](auto index, unsigned int stage_lds, TileCursor& ca, TileCursor& cb) __attribute__((always_inline)) {
        constexpr int l = decltype(index)::value;
        if constexpr (l < ATile::kLoads) {
            ca.soffset = load_to_lds<l * kWaves * kLoadBytes>(ca.rsrc, stage_lds, ca.voffset, ca.soffset, ca.step);
        } else {
            constexpr int lb = l - ATile::kLoads;
            cb.soffset = load_to_lds<kATileBytes + lb * kWaves * kLoadBytes>(cb.rsrc, stage_lds, cb.voffset, cb.soffset,
                                                                            (lb & 1) ? cb.step2 : cb.step);
        }
    };
    constexpr int kTileLoads = ATile::kLoads + BTile::kLoads;  // per wavefront and K tile
    static_assert(kTileLoads % 2 == 0, "a K tile's loads are dealt out in two equal halves, and the vmcnt waits count both");
    const unsigned int lds_wave = lds_address_of(smem) + wave * kLoadBytes;
    TileCursor ca, cb;
    // Requests K tiles FIRST .. LAST-1 of the opened item into the stages of the same numbers.
    auto request_tiles = [&]<int FIRST, int LAST>() __attribute__((always_inline)) {
        static_for<FIRST, LAST>([&](auto index) {
            constexpr int t = decltype(index)::value;
            cursors(t, ca, cb);
            static_for<0, kTileLoads>([&](auto l) { issue_one(l, lds_wave + t * kStageBytes, ca, cb); });
        });
    };

    // Per-lane LDS offsets of the fragments: one for a k-contiguous operand (the block is a
    // scalar offset), one per 16-column block for an n-contiguous one (the swizzle depends on it).
    constexpr int kAOffsets = A_K ? 1 : TM, kBOffsets = B_K ? 1 : TN;
    int a_off[kAOffsets], b_off[kBOffsets];
    if constexpr (A_K) {
        a_off[0] = ATile::lane_offset(lane);
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) a_off[i] = ATile::lane_offset(lane, wm * WM + i * 16);
    }
    if constexpr (B_K) {
        b_off[0] = BTile::lane_offset(lane);
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j) b_off[j] = BTile::lane_offset(lane, wn * WN + j * 16);
    }

    acc_t acc[TM][TN];
    frag_t af[TM], bf[TN];
    // Fragment F (A's TM blocks first, then B's TN) of the K tile in `stage_tile`.
    auto read_frag = [&]<int F>(const T* stage_tile) __attribute__((always_inline)) {
        if constexpr (F < TM) {
            if constexpr (A_K) af[F] = ATile::frag(stage_tile, wm * WM + F * 16, a_off[0]);
            else af[F] = ATile::frag(stage_tile, a_off[F]);
        } else {
            constexpr int j = F - TM;
            if constexpr (B_K) bf[j] = BTile::frag(stage_tile + kATile, wn * WN + j * 16, b_off[0]);
            else bf[j] = BTile::frag(stage_tile + kATile, b_off[j]);
        }
    };

    // Epilogue staging. acc[i][j][e] holds C[m, n] with m = lane%16, n = 4*(lane/16) + e, relative
    // to the 16 x 16 block (i, j) of the wavefront's WM x WN part of the tile. Each wavefront passes
    // its part through a private quarter of the last LDS stage (the only one the first K tiles of
    // the next item do not fill), 32 rows at a time, and stores it row by row: whole contiguous
    // row segments of C per instruction instead of 32 separate 8-byte pieces, and no workgroup
    // barrier. When bias, residual or the old C are added (or the output is fp32 / a split-K
    // partial) the staging is fp32, half the columns per pass, and rounding to the storage dtype
    // still happens once, after the additions; otherwise the values are rounded in registers and
    // staged in the storage dtype. A staged row is kRowBytes long; its 16-byte chunk c sits at
    // chunk position c ^ sw(row), which spreads both the column-wise writes and the row-wise reads
    // over all banks.
    constexpr int kRowBytes = WN * static_cast<int>(sizeof(T));
    constexpr int kRowChunks = kRowBytes / 16;
    static_assert(32 * kRowBytes * kWaves == static_cast<int>(kStageBytes), "staging is a quarter stage per wavefront");
    unsigned char* region = smem_raw + (kStages - 1) * kStageBytes + wave * (kStageBytes / kWaves);
    auto sw = [](int row) { return (row / (256 / kRowBytes)) % kRowChunks; };
    const int m_lane = lane & 15, q_lane = lane >> 4;
    // Writes blocks (2r, j0 .. j0+JP-1) and (2r+1, ...) into the wavefront's staging region as element type S.
    auto stage = [&]<typename S, int JP>(int r, int j0) __attribute__((always_inline)) {
        static_assert(JP * 16 * sizeof(S) == kRowBytes, "a pass fills whole staged rows");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int ii = 0; ii < 2; ++ii) {
            const int row = ii * 16 + m_lane;
            unsigned char* write_row = region + row * kRowBytes;
#pragma unroll
            for (int jj = 0; jj < JP; ++jj) {
                // Read out of the accumulator registers here and now: left to the register allocator,
                // some kernels copy all 256 accumulators to vector registers right after the K loop
                // and spill what does not fit.
                acc_t v;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x;
                    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(x) : "a"(acc[2 * r + ii][j0 + jj][e]));
                    v[e] = x;
                }
                const int byte = (jj * 16 + q_lane * 4) * static_cast<int>(sizeof(S));
                unsigned char* slot = write_row + (((byte / 16) ^ sw(row)) * 16) + byte % 16;
                if constexpr (std::is_same_v<S, float>) *reinterpret_cast<vec_t<float, 4>*>(slot) = v;
                else store_vec<T, 4>(reinterpret_cast<T*>(slot), vec_from_f32<T, 4>(v));
            }
        }
        __builtin_amdgcn_wave_barrier();
    };
    // Stages those blocks, 32 rows, and hands each lane 8 consecutive staged elements at a time:
    // consume(round, row, col, pointer to the 8 elements' first chunk, to the second chunk when S is
    // float), row/col relative to the wavefront's part; in round u the lane gets element
    // q = 64 u + lane of the 32 x (8-element groups per row) grid, row-major.
    auto pass = [&]<typename S, int JP>(int r, int j0, auto&& consume) __attribute__((always_inline)) {
        stage.template operator()<S, JP>(r, j0);
        constexpr int kLanesPerRow = kRowBytes / (8 * static_cast<int>(sizeof(S)));
        constexpr int kChunksPerLane = 8 * static_cast<int>(sizeof(S)) / 16;
        constexpr int kRounds = 32 * kLanesPerRow / kWave;
#pragma unroll
        for (int u = 0; u < kRounds; ++u) {
            const int q = u * kWave + lane;
            const int row = q / kLanesPerRow, part = q % kLanesPerRow;
            const unsigned char* base = region + row * kRowBytes;
            const int first = part * kChunksPerLane;
            consume(u, r * 32 + row, j0 * 16 + part * 8, base + ((first ^ sw(row)) * 16),
                    base + (((first + kChunksPerLane - 1) ^ sw(row)) * 16));
        }
    };
    constexpr int kRowBlocks = WM / 32;  // 32-row blocks of a wavefront's part
    auto request_share = [&](int r) __attribute__((always_inline)) {
        static_for<0, kRowBlocks>([&](auto index) {
            constexpr int block = decltype(index)::value;
            if (r == block)
                request_tiles.template operator()<block * (kStages - 1) / kRowBlocks, (block + 1) * (kStages - 1) / kRowBlocks>();
        });
    };
    // Before 32-row block r of the tile is staged and stored, its share of the first K tiles of the next item
    // are requested (if there is one): a burst of requests would hold the wavefront up for as long as
    // the memory system takes to accept them, between the stores it costs nothing.
    auto store_tile = [&](const Item& w, bool request) __attribute__((always_inline)) {
        // C may be given as column segments too: this tile's columns then belong to one of them.
        void* c_base = p.c;
        long c_ld = p.ldc;
        int c_col0 = w.n0, c_cols = p.n;
        if (p.c_seg.count > 0) {
            const SegmentPick pick = pick_segment(p.c_seg, w.n0);
            c_base = const_cast<void*>(pick.ptr);
            c_ld = pick.ld;
            c_col0 = w.n0 - pick.first;
            c_cols = pick.cols;
        }
        const int row0 = w.m0 + wm * WM, col0 = wn * WN;  // of the wavefront's part; columns relative to n0
        // The two fp32-staged cases of the training step get straight-line code as well: split-K
        // partial tiles (nothing added, fp32 out) and a residual added to a 16-bit result. Half the
        // columns are staged per pass; lane l of round u holds 8 consecutive columns (group l%8) of
        // row 8u + l/8.
        constexpr int kGroups = WN / 2 / 8, kRowsF = kWave / kGroups, kRoundsF = 32 / kRowsF;
        const int f_row = lane / kGroups, f_col = (lane % kGroups) * 8;  // f_col within the staged half
        auto read_staged = [&](int u, vec_t<float, 4>& v0, vec_t<float, 4>& v1) __attribute__((always_inline)) {
            const int row = u * kRowsF + f_row;
            const unsigned char* base = region + row * kRowBytes;
            v0 = *reinterpret_cast<const vec_t<float, 4>*>(base + (((f_col / 4) ^ sw(row)) * 16));
            v1 = *reinterpret_cast<const vec_t<float, 4>*>(base + (((f_col / 4 + 1) ^ sw(row)) * 16));
        };
        // The same staged half, dealt out so that every store instruction of fp32 values covers whole cache lines: lane l
        // of round u takes columns 4 (l % 8) .. + 3 and, for its second store, the four columns 32 further on, of row
        // 8u + l/8 (with eight consecutive fp32 columns per lane, each store instruction would write every other 16 bytes
        // of a line, and lines reach memory in parts).
        const int l_col = (lane % kGroups) * 4;  // first column of the lane's first quad within the staged half
        auto read_staged_lines = [&](int u, vec_t<float, 4>& v0, vec_t<float, 4>& v1) __attribute__((always_inline)) {
            const int row = u * kRowsF + f_row;
            const unsigned char* base = region + row * kRowBytes;
            v0 = *reinterpret_cast<const vec_t<float, 4>*>(base + (((l_col / 4) ^ sw(row)) * 16));
            v1 = *reinterpret_cast<const vec_t<float, 4>*>(base + (((l_col / 4 + kGroups) ^ sw(row)) * 16));
        };
        // Descriptor over a wavefront's part of a row-major matrix (see the 16-bit case above).
        auto part_rsrc = [&](const void* origin, long ld, int elem, int rows_left, int cols_left) __attribute__((always_inline)) {
            const long extent = rows_left > 0 && cols_left > 0 ? (static_cast<long>(rows_left - 1) * ld + cols_left) * elem : 0;
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(origin), 0, static_cast<int>(extent), 0x00020000);
        };
        const int rows_left = min(WM, p.m - row0);
        if constexpr (SWIGLU) {
            // The wavefront's 128 staged columns are gate g0 .. g0+63 and up g0 .. g0+63. Lane l of
            // round u takes 8 gate and the 8 matching up values of row 8u + l/8 from the staging
            // region, stores both where the concatenated layout wants them, and the product beside.
            const int g0 = w.n0 / 2 + wn * (WN / 2);
            const int cols_left = min(WN / 2, p.inter - g0);
            const T* c_origin = static_cast<const T*>(p.c) + static_cast<long>(row0) * p.ldc + g0;
            const __amdgpu_buffer_rsrc_t gate_rsrc = part_rsrc(c_origin, p.ldc, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t up_rsrc = part_rsrc(c_origin + p.inter, p.ldc, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t act_rsrc = part_rsrc(static_cast<const T*>(p.act) + static_cast<long>(row0) * p.ld_act + g0,
                                                              p.ld_act, sizeof(T), rows_left, cols_left);
            const int c_row_bytes = static_cast<int>(p.ldc * static_cast<long>(sizeof(T)));
            const int act_row_bytes = static_cast<int>(p.ld_act * static_cast<long>(sizeof(T)));
            const bool live = f_col < cols_left;
            const int c_voffset = live ? f_row * c_row_bytes + f_col * static_cast<int>(sizeof(T)) : std::numeric_limits<int>::min();
            const int act_voffset = live ? f_row * act_row_bytes + f_col * static_cast<int>(sizeof(T)) : std::numeric_limits<int>::min();
#pragma unroll
            for (int r = 0; r < kRowBlocks; ++r) {
                __builtin_amdgcn_sched_barrier(0);
                if (request) request_share(r);
                stage.template operator()<T, TN>(r, 0);
                u32x4 gate[kRoundsF], up[kRoundsF];
#pragma unroll
                for (int u = 0; u < kRoundsF; ++u) {
                    const int row = u * kRowsF + f_row;
                    const unsigned char* base = region + row * kRowBytes;
                    gate[u] = *reinterpret_cast<const u32x4*>(base + (((f_col / 8) ^ sw(row)) * 16));
                    up[u] = *reinterpret_cast<const u32x4*>(base + (((kGroups + f_col / 8) ^ sw(row)) * 16));
                }
#pragma unroll
                for (int u = 0; u < kRoundsF; ++u) {
                    const int row = r * 32 + u * kRowsF;
                    __builtin_amdgcn_raw_buffer_store_b128(gate[u], gate_rsrc, c_voffset, row * c_row_bytes, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(up[u], up_rsrc, c_voffset, row * c_row_bytes, 0);
                    const vec_t<float, 8> g = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, gate[u]));
                    const vec_t<float, 8> v = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, up[u]));
                    vec_t<float, 8> product;
#pragma unroll
                    for (int e = 0; e < 8; ++e) product[e] = g[e] * (1.0f / (1.0f + __expf(-g[e]))) * v[e];
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, vec_from_f32<T, 8>(product)), act_rsrc,
                                                           act_voffset, row * act_row_bytes, 0);
                }
            }
            return;
        }
        if constexpr (GRAD) {
            // The contraction is the gradient of silu(gate)·up; what is written is the gradient of
            // [gate | up]: dgate = d·up·s·(1 + gate·(1 - s)), dup = d·gate·s with s = sigmoid(gate),
            // from d rounded to the storage dtype (the bits the separate operator reads) and the
            // forward's saved gate and up. The tile is staged in the storage dtype; lane l of round u
            // holds 8 consecutive columns (chunk l%16) of row 4u + l/16, loads the matching gate and up
            // values one 32-row block ahead and stores both gradients.
            const int g0 = w.n0 + col0;  // first gate column of the wavefront's part
            const int cols_left = min(WN, p.inter - g0);
            const T* out_origin = static_cast<const T*>(p.c) + static_cast<long>(row0) * p.ldc + g0;
            const T* in_origin = static_cast<const T*>(p.saved) + static_cast<long>(row0) * p.ld_saved + g0;
            const __amdgpu_buffer_rsrc_t dgate_rsrc = part_rsrc(out_origin, p.ldc, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t dup_rsrc = part_rsrc(out_origin + p.inter, p.ldc, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t gate_rsrc = part_rsrc(in_origin, p.ld_saved, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t up_rsrc = part_rsrc(in_origin + p.inter, p.ld_saved, sizeof(T), rows_left, cols_left);
            constexpr int kLanesPerRow = kRowBytes / 16, kRowsPerRound = kWave / kLanesPerRow, kRounds = 32 / kRowsPerRound;
            const int lane_row = lane / kLanesPerRow, lane_chunk = lane % kLanesPerRow;
            const int out_row_bytes = static_cast<int>(p.ldc * static_cast<long>(sizeof(T)));
            const int in_row_bytes = static_cast<int>(p.ld_saved * static_cast<long>(sizeof(T)));
            const bool live = lane_chunk * 8 < cols_left;
            const int out_voffset = live ? lane_row * out_row_bytes + lane_chunk * 16 : std::numeric_limits<int>::min();
            const int in_voffset = live ? lane_row * in_row_bytes + lane_chunk * 16 : std::numeric_limits<int>::min();
            u32x4 ahead[2][2][kRounds];
            auto request_saved = [&](int r, u32x4 (&into)[2][kRounds]) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int soffset = (r * 32 + u * kRowsPerRound) * in_row_bytes;
                    into[0][u] = __builtin_amdgcn_raw_buffer_load_b128(gate_rsrc, in_voffset, soffset, 0);
                    into[1][u] = __builtin_amdgcn_raw_buffer_load_b128(up_rsrc, in_voffset, soffset, 0);
                }
            };
            request_saved(0, ahead[0]);
#pragma unroll
            for (int r = 0; r < kRowBlocks; ++r) {
                __builtin_amdgcn_sched_barrier(0);
                if (request) request_share(r);
                if (r + 1 < kRowBlocks) request_saved(r + 1, ahead[(r + 1) & 1]);
                stage.template operator()<T, TN>(r, 0);
                u32x4 data[kRounds];
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int row = u * kRowsPerRound + lane_row;
                    data[u] = *reinterpret_cast<const u32x4*>(region + row * kRowBytes + ((lane_chunk ^ sw(row)) * 16));
                }
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const vec_t<float, 8> d = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, data[u]));
                    const vec_t<float, 8> g = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, ahead[r & 1][0][u]));
                    const vec_t<float, 8> v = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, ahead[r & 1][1][u]));
                    vec_t<float, 8> dg, du;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float sg = 1.0f / (1.0f + __expf(-g[e]));
                        dg[e] = d[e] * v[e] * (sg * (1.0f + g[e] * (1.0f - sg)));
                        du[e] = d[e] * (g[e] * sg);
                    }
                    const int soffset = (r * 32 + u * kRowsPerRound) * out_row_bytes;
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, vec_from_f32<T, 8>(dg)), dgate_rsrc, out_voffset, soffset, 0);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, vec_from_f32<T, 8>(du)), dup_rsrc, out_voffset, soffset, 0);
                }
            }
            return;
        }
        if constexpr (RESIDUAL) {
            const int cols_left = min(WN, c_cols - (c_col0 + col0));
            const T* out_origin = static_cast<const T*>(c_base) + static_cast<long>(row0) * c_ld + (c_col0 + col0);
            const T* res_origin = static_cast<const T*>(p.residual) + static_cast<long>(row0) * p.ldr + (w.n0 + col0);
            const __amdgpu_buffer_rsrc_t out_rsrc = part_rsrc(out_origin, c_ld, sizeof(T), rows_left, cols_left);
            const __amdgpu_buffer_rsrc_t res_rsrc = part_rsrc(res_origin, p.ldr, sizeof(T), rows_left, cols_left);
            const int out_row_bytes = static_cast<int>(c_ld * static_cast<long>(sizeof(T)));
            const int res_row_bytes = static_cast<int>(p.ldr * static_cast<long>(sizeof(T)));
            // The residual of a 32-row block is requested one block ahead (the first one before
            // anything is staged): its memory round trip passes under the previous block's work.
            u32x4 ahead[2][2][kRoundsF];
            auto request_residual = [&](int r, u32x4 (&into)[2][kRoundsF]) __attribute__((always_inline)) {
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int col = half * (WN / 2) + f_col;
                    const int voffset = col < cols_left ? f_row * res_row_bytes + col * static_cast<int>(sizeof(T))
                                                        : std::numeric_limits<int>::min();
#pragma unroll
                    for (int u = 0; u < kRoundsF; ++u)
                        into[half][u] = __builtin_amdgcn_raw_buffer_load_b128(res_rsrc, voffset, (r * 32 + u * kRowsF) * res_row_bytes, 0);
                }
            };
            request_residual(0, ahead[0]);
#pragma unroll
            for (int r = 0; r < kRowBlocks; ++r) {
                __builtin_amdgcn_sched_barrier(0);
                if (request) request_share(r);
                if (r + 1 < kRowBlocks) request_residual(r + 1, ahead[(r + 1) & 1]);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    stage.template operator()<float, TN / 2>(r, half * (TN / 2));
                    const int col = half * (WN / 2) + f_col;
                    const int voffset = col < cols_left ? f_row * out_row_bytes + col * static_cast<int>(sizeof(T))
                                                        : std::numeric_limits<int>::min();
                    vec_t<float, 4> v0[kRoundsF], v1[kRoundsF];
#pragma unroll
                    for (int u = 0; u < kRoundsF; ++u) read_staged(u, v0[u], v1[u]);
#pragma unroll
                    for (int u = 0; u < kRoundsF; ++u) {
                        const vec_t<float, 8> add = vec_to_f32<T, 8>(__builtin_bit_cast(vec_t<T, 8>, ahead[r & 1][half][u]));
                        vec_t<float, 8> sum;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            sum[e] = v0[u][e] + add[e];
                            sum[4 + e] = v1[u][e] + add[4 + e];
                        }
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, vec_from_f32<T, 8>(sum)), out_rsrc, voffset,
                                                               (r * 32 + u * kRowsF) * out_row_bytes, 0);
                    }
                }
            }
            return;
        }
        bool plain = false;
        if constexpr (!SPLIT) plain = p.bias == nullptr && p.residual == nullptr && p.addend == nullptr && !p.accumulate && !p.c_f32;
        if (plain) {
            // Straight-line code, no per-lane predicates or address arithmetic (with one wavefront per
            // SIMD every branch and every dependent wait is exposed): the stores go through a buffer
            // descriptor over the wavefront's part of C, whose range ends with the last valid row, so
            // rows past the matrix are dropped by the range check; a lane whose columns lie past the
            // matrix gets an offset beyond every range. Lane l of round u holds 16 bytes of row
            // 4u + l/16 (256-byte rows): the row advance is a scalar offset.
            T* part = static_cast<T*>(c_base) + static_cast<long>(row0) * c_ld + (c_col0 + col0);
            const int rows_left = min(WM, p.m - row0), cols_left = min(WN, c_cols - (c_col0 + col0));
            const long extent = rows_left > 0 && cols_left > 0
                                    ? (static_cast<long>(rows_left - 1) * c_ld + cols_left) * static_cast<long>(sizeof(T))
                                    : 0;
            const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(part, 0, static_cast<int>(extent), 0x00020000);
            constexpr int kLanesPerRow = kRowBytes / 16, kRowsPerRound = kWave / kLanesPerRow, kRounds = 32 / kRowsPerRound;
            const int lane_row = lane / kLanesPerRow, lane_chunk = lane % kLanesPerRow;
            const int row_bytes = static_cast<int>(c_ld * static_cast<long>(sizeof(T)));
            const int voffset = lane_chunk * 8 < cols_left ? lane_row * row_bytes + lane_chunk * 16 : std::numeric_limits<int>::min();
#pragma unroll
            for (int r = 0; r < kRowBlocks; ++r) {
                // Accumulators leave their registers block by block: read ahead of their block they
                // would not fit the vector registers.
                __builtin_amdgcn_sched_barrier(0);
                if (request) request_share(r);
                stage.template operator()<T, TN>(r, 0);
                u32x4 data[kRounds];
#pragma unroll
                for (int u = 0; u < kRounds; ++u) {
                    const int row = u * kRowsPerRound + lane_row;
                    data[u] = *reinterpret_cast<const u32x4*>(region + row * kRowBytes + ((lane_chunk ^ sw(row)) * 16));
                }
#pragma unroll
                for (int u = 0; u < kRounds; ++u)
                    __builtin_amdgcn_raw_buffer_store_b128(data[u], rsrc, voffset, (r * 32 + u * kRowsPerRound) * row_bytes, 0);
            }
            return;
        }
        if constexpr (SPLIT) {
            const float* origin = static_cast<const float*>(p.c) +
                                  (static_cast<long>(w.slice) * p.m + row0) * static_cast<long>(p.n) + (w.n0 + col0);
            const int cols_left = min(WN, p.n - (w.n0 + col0));
            const __amdgpu_buffer_rsrc_t rsrc = part_rsrc(origin, p.n, 4, rows_left, cols_left);
            const int row_bytes = p.n * 4;
#pragma unroll
            for (int r = 0; r < kRowBlocks; ++r) {
                __builtin_amdgcn_sched_barrier(0);
                if (request) request_share(r);
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    stage.template operator()<float, TN / 2>(r, half * (TN / 2));
                    const int col = half * (WN / 2) + l_col;
                    constexpr int kSecond = kGroups * 4;  // columns between a lane's two quads
                    const int voffset0 = col < cols_left ? f_row * row_bytes + col * 4 : std::numeric_limits<int>::min();
                    const int voffset1 = col + kSecond < cols_left ? f_row * row_bytes + (col + kSecond) * 4 : std::numeric_limits<int>::min();
                    vec_t<float, 4> v0[kRoundsF], v1[kRoundsF];
#pragma unroll
                    for (int u = 0; u < kRoundsF; ++u) read_staged_lines(u, v0[u], v1[u]);
#pragma unroll
                    for (int u = 0; u < kRoundsF; ++u) {
                        const int soffset = (r * 32 + u * kRowsF) * row_bytes;
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v0[u]), rsrc, voffset0, soffset, 0);
                        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v1[u]), rsrc, voffset1, soffset, 0);
                    }
                }
            }
            return;
        }
#pragma unroll
        for (int r = 0; r < kRowBlocks; ++r) {
            __builtin_amdgcn_sched_barrier(0);
            if (request) request_share(r);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                pass.template operator()<float, TN / 2>(r, half * (TN / 2), [&](int, int row, int col, const unsigned char* lo,
                                                                              const unsigned char* hi) {
                    const int m = row0 + row, n = w.n0 + col0 + col, c_col = c_col0 + col0 + col;
                    vec_t<float, 4> v0 = *reinterpret_cast<const vec_t<float, 4>*>(lo);
                    vec_t<float, 4> v1 = *reinterpret_cast<const vec_t<float, 4>*>(hi);
                    if (m >= p.m || c_col >= c_cols) return;
                    {
                        if (p.addend != nullptr) {
                            const float* addend = p.addend + static_cast<long>(m) * p.ld_addend + n;
                            v0 += *reinterpret_cast<const vec_t<float, 4>*>(addend);
                            v1 += *reinterpret_cast<const vec_t<float, 4>*>(addend + 4);
                        }
                        if (p.bias != nullptr) {
                            const T* bias = static_cast<const T*>(p.bias) + n;
                            v0 += vec_to_f32<T, 4>(load_vec<T, 4>(bias));
                            v1 += vec_to_f32<T, 4>(load_vec<T, 4>(bias + 4));
                        }
                        if (p.residual != nullptr) {
                            const T* residual = static_cast<const T*>(p.residual) + static_cast<long>(m) * p.ldr + n;
                            v0 += vec_to_f32<T, 4>(load_vec<T, 4>(residual));
                            v1 += vec_to_f32<T, 4>(load_vec<T, 4>(residual + 4));
                        }
                        if (p.c_f32) {
                            float* out = static_cast<float*>(c_base) + static_cast<long>(m) * c_ld + c_col;
                            if (p.accumulate) {
                                v0 += *reinterpret_cast<const vec_t<float, 4>*>(out);
                                v1 += *reinterpret_cast<const vec_t<float, 4>*>(out + 4);
                            }
                            *reinterpret_cast<vec_t<float, 4>*>(out) = v0;
                            *reinterpret_cast<vec_t<float, 4>*>(out + 4) = v1;
                        } else {
                            T* out = static_cast<T*>(c_base) + static_cast<long>(m) * c_ld + c_col;
                            if (p.accumulate) {
                                const vec_t<T, 8> old = load_vec<T, 8>(out);
#pragma unroll
                                for (int e = 0; e < 4; ++e) {
                                    v0[e] += to_f32(old[e]);
                                    v1[e] += to_f32(old[4 + e]);
                                }
                            }
                            vec_t<T, 8> packed;
                            const vec_t<T, 4> r0 = vec_from_f32<T, 4>(v0), r1 = vec_from_f32<T, 4>(v1);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                packed[e] = r0[e];
                                packed[4 + e] = r1[e];
                            }
                            store_vec<T, 8>(out, packed);
                        }
                    }
                });
            }
        }
    };

    // Software pipeline over the K tiles t = 0 .. count-1 of an item (tile t lives in LDS stage
    // t % kStages; tiles t+1 .. t+kStages-2 are in flight or landed). A K tile is one MFMA step
    // (k = 32) of TM x TN MFMAs, taken as two column halves (all rows x the left TN/2 blocks, then
    // all rows x the right ones) so that one set of fragment registers suffices: a fragment is read
    // for the next tile as soon as its last MFMA of this tile has been issued.
    //   left half    MFMAs ‖ LDS reads of this tile's right-half B fragments ‖ the second half of the loads of
    //                tile t+kStages-2 (into the stage freed one tile ago)
    //   wait         this wavefront's loads of tile t+1 have landed; barrier: everybody's have, and
    //                nobody reads stage (t-1) % kStages any more
    //   right half   MFMAs ‖ the first half of the loads of tile t+kStages-1 into that stage ‖ tile t+1's
    //                left-half B fragments (first thing) and its A fragment i after row i
    // so LDS latency and kStages-2 K tiles of global latency sit in the shadow of MFMAs. With one
    // wavefront per SIMD nothing else hides an instruction that is not next to an MFMA, so every
    // MFMA is followed by its share of the loads and fragment reads and a scheduling fence keeps
    // them there.
    constexpr int kMfmas = TM * TN;
    constexpr int kHalf = TN / 2;
    static_assert(TN % 2 == 0 && kHalf <= TM, "the left-half B fragments are read one per row");
    // HALF 0: this_tile = tile t (its right-half B fragments are read); HALF 1: next_tile = tile t+1.
    auto multiply_half = [&]<int HALF, bool FIRST>(const T* tile, unsigned int free_lds) __attribute__((always_inline)) {
        static_for<0, kMfmas / 2>([&](auto index) {
            constexpr int m = decltype(index)::value;
            // Rows one after the other, their columns left to right and right to left alternately:
            // consecutive MFMAs always share an operand (measurably less power on a power-limited chip).
            constexpr int i = m / kHalf, jj = m % kHalf, j = HALF * kHalf + ((i & 1) ? kHalf - 1 - jj : jj);
            if constexpr (FIRST) Mfma<T>::start(acc[i][j], bf[j], af[i]);
            else Mfma<T>::run(acc[i][j], bf[j], af[i]);
            if constexpr (HALF == 0) {
                // Right-half B fragment i of this tile after the first MFMA of row i (rows 0 .. kHalf-1).
                if constexpr (jj == 0 && i < kHalf) read_frag.template operator()<TM + kHalf + i>(tile);
            } else {
                // Left-half B fragment i of the next tile after the first MFMA of row i (its last use
                // was in the left half), A fragment i after the last MFMA of row i.
                if constexpr (jj == 0 && i < kHalf) read_frag.template operator()<TM + i>(tile);
                if constexpr (jj == kHalf - 1) read_frag.template operator()<i>(tile);
                // The first half of the loads of tile t+kStages-1 (one load per kMfmas / kTileLoads MFMAs).
                static_for<(m * (kTileLoads / 2)) / (kMfmas / 2), ((m + 1) * (kTileLoads / 2)) / (kMfmas / 2)>(
                    [&](auto l) { issue_one(l, free_lds, ca, cb); });
            }
            if constexpr (HALF == 0 && !FIRST) {
                // The second half of the loads that the previous tile's right half began: a wavefront's load
                // instruction keeps it from issuing for about as long as an MFMA runs, so the loads are dealt out
                // evenly over the whole tile instead of twice as densely over one half.
                static_for<kTileLoads / 2 + (m * (kTileLoads / 2)) / (kMfmas / 2),
                           kTileLoads / 2 + ((m + 1) * (kTileLoads / 2)) / (kMfmas / 2)>(
                    [&](auto l) { issue_one(l, free_lds, ca, cb); });
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // Per round: multiply an item, request the first K tiles of the next one, store the finished
    // tile (its stores drain under the MFMAs that follow). The sources are opened every round, also
    // when no item is left (then for the last one again, unused): values that are set on every path
    // stay in scalar registers.
    Item current = locate(item);
    open(current);
    request_tiles.template operator()<0, kStages - 1>();
    while (true) {
        const int count = current.kt_end - current.kt_begin;
        // Loads and stores retire in the order they were issued: at most the loads of K tiles
        // 1 .. kStages-2 (and no older store of the previous epilogue) may still be outstanding.
        __builtin_amdgcn_s_waitcnt(vmcnt_immediate((kStages - 2) * kTileLoads));
        barrier_only();
        static_for<0, TM + kHalf>([&](auto f) { read_frag.template operator()<decltype(f)::value>(smem); });
        int stage = 0;                 // of tile t
        int free_stage = kStages - 1;  // of tile t-1, refilled with tile t+kStages-1
        auto multiply_tile = [&]<bool FIRST>(int t) __attribute__((always_inline)) {
            const int next_stage = stage + 1 == kStages ? 0 : stage + 1;
            // The left half finishes the requests of tile t+kStages-2 (cursors and stage of the previous tile: the
            // stage before free_stage), then the cursors move on to tile t+kStages-1.
            const int previous_free = free_stage == 0 ? kStages - 1 : free_stage - 1;
            multiply_half.template operator()<0, FIRST>(smem + stage * kStage, lds_wave + previous_free * kStageBytes);
            cursors(t + kStages - 1, ca, cb);
            __builtin_amdgcn_s_waitcnt(vmcnt_immediate((kStages - 3) * kTileLoads));
            barrier_only();
            multiply_half.template operator()<1, FIRST>(smem + next_stage * kStage, lds_wave + free_stage * kStageBytes);
            free_stage = stage;
            stage = next_stage;
        };
        // The first K tile starts the sums (MFMA with a zero addend): no pass over the 256
        // accumulator registers to clear them. Every item has at least one K tile (the host makes
        // K slices non-empty).
        multiply_tile.template operator()<true>(0);
        for (int t = 1; t < count; ++t) multiply_tile.template operator()<false>(t);
        // The loads still outstanding are of K tiles past the end (zeros, but they do write LDS):
        // once they have landed and every wavefront has read its last fragments, all stages are free.
        __builtin_amdgcn_s_waitcnt(vmcnt_immediate(0));
        barrier_only();
        item += item_stride;
        const bool more = item < item_end;
        const Item next = locate(more ? item : item_end - 1);
        open(next);
        store_tile(current, more);
        if (!more) break;
        current = next;
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

// ---- fp32 matrix-core kernel for everything the streamed 16-bit path does not take ---------------
// fp32 storage (the reference serves it through its tensor-core library too: src/ops/linear.cu:634-667,
// src/ops/backward/linear_backward.cu:79-82), and 16-bit storage whose K is not a multiple of 32 or whose rows are
// not 16-byte aligned. Any shape, any alignment, all three operand layouts: a 128 x 128 tile of C per block, K in
// steps of 16; the four wavefronts own 64 x 64 each and multiply with v_mfma_f32_32x32x2_f32 on fp32 operands
// (16-bit storage is widened on the way into LDS, so the products are exact and the sums fp32, as in the streamed
// kernels). Operand tiles go through registers into a K-major LDS layout ([k][m], [k][n]) — the fragment of an
// MFMA step is then 32 consecutive floats per half-wavefront — with the next tile's loads in flight during the
// multiplication; rows, columns and K positions past the matrices read as zeros.
constexpr int kF32Tile = 128;  // rows and columns of C per block
constexpr int kF32K = 16;      // K per LDS stage
constexpr int kF32Pad = 4;
using acc16_t = vec_t<float, 16>;

template <typename T>
__global__ __launch_bounds__(kThreads) void gemm_f32_mfma_kernel(KernelArgs p, int a_k, int b_k) {
    __shared__ float as[2][kF32K][kF32Tile + kF32Pad];
    __shared__ float bs[2][kF32K][kF32Tile + kF32Pad];
    const T* A = static_cast<const T*>(p.a);
    const T* B = static_cast<const T*>(p.b);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int wm = wave >> 1, wn = wave & 1;
    const long m0 = static_cast<long>(blockIdx.y) * kF32Tile, n0 = static_cast<long>(blockIdx.x) * kF32Tile;
    constexpr int kPerThread = kF32Tile * kF32K / kThreads;  // elements of each operand tile a thread moves
    float a_regs[kPerThread], b_regs[kPerThread];
    // Element e of a thread's share: consecutive threads walk the operand's contiguous index.
    auto coordinates = [&](int e, bool k_contiguous, int& row, int& k) {
        const int index = threadIdx.x + e * kThreads;
        if (k_contiguous) {
            row = index / kF32K;
            k = index % kF32K;
        } else {
            k = index / kF32Tile;
            row = index % kF32Tile;
        }
    };
    auto fetch = [&](long k0) {
#pragma unroll
        for (int e = 0; e < kPerThread; ++e) {
            int row, k;
            coordinates(e, a_k != 0, row, k);
            const long m = m0 + row, ka = k0 + k;
            a_regs[e] = (m < p.m && ka < p.k) ? to_f32(a_k ? A[m * p.lda + ka] : A[ka * p.lda + m]) : 0.0f;
            coordinates(e, b_k != 0, row, k);
            const long n = n0 + row, kb = k0 + k;
            b_regs[e] = (n < p.n && kb < p.k) ? to_f32(b_k ? B[n * p.ldb + kb] : B[kb * p.ldb + n]) : 0.0f;
        }
    };
    auto deposit = [&](int stage) {
#pragma unroll
        for (int e = 0; e < kPerThread; ++e) {
            int row, k;
            coordinates(e, a_k != 0, row, k);
            as[stage][k][row] = a_regs[e];
            coordinates(e, b_k != 0, row, k);
            bs[stage][k][row] = b_regs[e];
        }
    };
    acc16_t acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = acc16_t(0.0f);
    fetch(0);
    deposit(0);
    __syncthreads();
    int stage = 0;
    for (long k0 = 0; k0 < p.k; k0 += kF32K) {
        const bool more = k0 + kF32K < p.k;
        if (more) fetch(k0 + kF32K);  // in flight during the multiplication below
#pragma unroll
        for (int kk = 0; kk < kF32K; kk += 2) {
            // MFMA step of k = 2: lane l holds row (column) l % 32 at k = l / 32.
            float a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) a[i] = as[stage][kk + (lane >> 5)][wm * 64 + i * 32 + (lane & 31)];
#pragma unroll
            for (int j = 0; j < 2; ++j) b[j] = bs[stage][kk + (lane >> 5)][wn * 64 + j * 32 + (lane & 31)];
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }
        if (more) {
            deposit(stage ^ 1);  // nobody reads that stage: the barrier below closed its last use
            __syncthreads();
            stage ^= 1;
        }
    }
    // Register r of a block holds row 8 (r / 4) + 4 (lane / 32) + r % 4 of column lane % 32.
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const long n = n0 + wn * 64 + j * 32 + (lane & 31);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const long m = m0 + wm * 64 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
                if (m >= p.m || n >= p.n) continue;
                float v = acc[i][j][r];
                if (p.addend != nullptr) v += p.addend[m * p.ld_addend + n];
                if (p.bias != nullptr) v += to_f32(static_cast<const T*>(p.bias)[n]);
                if (p.residual != nullptr) v += to_f32(static_cast<const T*>(p.residual)[m * p.ldr + n]);
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
}

// ------------------------------------------------------------------- host side
template <typename T, int BM, int BN, bool A_K, bool B_K, bool SPLIT, bool SEGMENTED, bool RESIDUAL = false,
          bool SWIGLU = false, bool GRAD = false>
int launch_mfma(const KernelArgs& p, int slices, hipStream_t stream) {
    constexpr std::size_t smem = TileLayout<T, BM, BN, A_K, B_K>::kSmemBytes;
    auto kernel = gemm_mfma_kernel<T, BM, BN, A_K, B_K, SPLIT, SEGMENTED, RESIDUAL, SWIGLU, GRAD>;
    static bool configured = false;
    if (!configured) {
        CGPTX_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(smem)));
        configured = true;
    }
    // One block per CU slot (256x256 tiles: one per CU; 128x128: two), a multiple of the XCD count
    // so that every XCD gets the same number of blocks; fewer when there are fewer work items.
    KernelArgs args = p;
    args.slices = slices;
    const long items = static_cast<long>(p.tiles_m) * p.tiles_n * slices;
    {
        // x * ceil(2^32 / d) >> 32 == x / d for every x with x * d < 2^32.
        // Tile-rows per L2 locality group. 8 (x 4 tile-columns = the 32 tiles in flight on an XCD) shares operand
        // panels best. The SwiGLU-gradient epilogue moves four times the bytes of a plain one, two loads and two
        // stores of whole [gate | up] rows: there the tiles in flight on an XCD are better spread along the rows
        // (2 tile-rows x all 8 tile-columns of the training shape: 250 -> 212 us per launch; 1, 2 and 4 tile-rows
        // measure the same, every other kernel is at its best with 8).
        args.group_rows_log2 = GRAD ? 1 : 3;
        const unsigned long divisor = (1ul << args.group_rows_log2) * static_cast<unsigned long>(p.tiles_n);
        const unsigned long tiles = static_cast<unsigned long>(p.tiles_m) * static_cast<unsigned long>(p.tiles_n);
        const bool exact = divisor > 1 && tiles * divisor < (1ul << 32);
        args.group_reciprocal = exact ? static_cast<unsigned int>(((1ul << 32) + divisor - 1) / divisor) : 0u;
    }
    const long slots = static_cast<long>(compute_units()) * (BM == 256 ? 1 : 2) / kXcds * kXcds;
    const long blocks = std::min<long>((items + kXcds - 1) / kXcds * kXcds, std::max<long>(slots, kXcds));
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned int>(blocks)), dim3(kThreads), smem, stream, args);
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

template <typename T, int BM, int BN, bool SPLIT>
int launch_layout(const KernelArgs& p, bool a_k, bool b_k, int slices, hipStream_t stream) {
    // A given in segments along K has kernels of its own (the source of a K tile is then picked
    // per tile), and only unsplit ones.
    const bool segmented = a_k && p.a_seg.count > 0;
    if constexpr (!SPLIT) {
        if (segmented && b_k) return launch_mfma<T, BM, BN, true, true, false, true>(p, slices, stream);
        if (segmented && !b_k) return launch_mfma<T, BM, BN, true, false, false, true>(p, slices, stream);
    }
    if (segmented) return fail(CGPTX_RUNTIME, "gemm: a segmented operand cannot be split along K");
    if constexpr (!SPLIT && BN == 256) {
        if (p.act != nullptr) return launch_mfma<T, BM, BN, true, true, false, false, false, true>(p, slices, stream);
    }
    if (p.act != nullptr) return fail(CGPTX_RUNTIME, "gemm: the SwiGLU epilogue needs 256-wide unsplit tiles");
    if constexpr (!SPLIT && BN == 256) {
        if (p.saved != nullptr) return launch_mfma<T, BM, BN, true, false, false, false, false, false, true>(p, slices, stream);
    }
    if (p.saved != nullptr) return fail(CGPTX_RUNTIME, "gemm: the SwiGLU gradient epilogue needs 256-wide unsplit tiles");
    if constexpr (!SPLIT) {
        if (a_k && b_k && p.bias == nullptr && p.addend == nullptr && !p.c_f32) {
            if (p.residual != nullptr && !p.accumulate) return launch_mfma<T, BM, BN, true, true, false, false, true>(p, slices, stream);
            if (p.residual == nullptr && p.accumulate && p.c_seg.count == 0) {
                // C += A·B in the storage dtype is the same epilogue with C as its own residual
                // (every lane reads the elements it later writes, and reads them first).
                KernelArgs self = p;
                self.residual = p.c;
                self.ldr = p.ldc;
                self.accumulate = 0;
                return launch_mfma<T, BM, BN, true, true, false, false, true>(self, slices, stream);
            }
        }
    }
    if (a_k && b_k) return launch_mfma<T, BM, BN, true, true, SPLIT, false>(p, slices, stream);
    if (a_k && !b_k) return launch_mfma<T, BM, BN, true, false, SPLIT, false>(p, slices, stream);
    if (!a_k && !b_k) return launch_mfma<T, BM, BN, false, false, SPLIT, false>(p, slices, stream);
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
    const bool k_segments = g.a_k_contiguous && g.a_segments.count > 0;
    const bool may_split = !g.no_split || g.split_workspace != nullptr;
    if (may_split && g.residual == nullptr && g.addend_f32 == nullptr && g.swiglu_out == nullptr && g.swiglu_saved == nullptr &&
        g.c_segments.count == 0 && !k_segments &&
        tiles < want_blocks && k_tiles >= 32) {
        // As many slices as fit the CU slots in one go: one item more than that would cost a
        // second round of the persistent blocks.
        slices = static_cast<int>(std::min<long>(want_blocks / tiles, k_tiles / 16));
        if (slices < 1) slices = 1;
    }
    if (g.batch_rows != 0 && may_split && k_tiles >= 32) {
        // A stack of products brings any number of tiles: the slice count that needs the least time, counted in
        // rounds of the persistent blocks times the length of a slice (fewer slices on a tie: fewer partial tiles).
        double best = 0.0;
        for (int s = 1; s <= 8 && k_tiles / s >= 16; ++s) {
            const long rounds = (tiles * s + want_blocks - 1) / want_blocks;
            const double time = static_cast<double>(rounds) / s * (s > 1 ? 1.02 : 1.0);
            if (s == 1 || time < best * 0.999) {
                best = time;
                slices = s;
            }
        }
    }
    if (g.no_split && static_cast<std::size_t>(slices) * g.m * g.n * sizeof(float) > g.split_workspace_bytes) slices = 1;
    p.k_tiles_per_slice = (k_tiles + slices - 1) / slices;
    slices = (k_tiles + p.k_tiles_per_slice - 1) / p.k_tiles_per_slice;
    if (slices == 1) return launch_layout<T, BM, BN, false>(p, g.a_k_contiguous, g.b_k_contiguous, 1, stream);
    void* mem = g.no_split ? g.split_workspace : nullptr;
    if (mem == nullptr) {
        if (int s = scratch(stream, static_cast<std::size_t>(slices) * g.m * g.n * sizeof(float), &mem)) return s;
    }
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

// Validates column segments (widths multiples of `granule` except the last, summing to `total`,
// 16-byte aligned rows) and copies them into the kernel arguments.
int copy_segments(const GemmSegments& in, std::size_t total, std::size_t granule, KernelSegments& out) {
    out = KernelSegments{};
    if (in.count == 0) return CGPTX_OK;
    if (in.count < 0 || in.count > 3) return fail(CGPTX_INVALID_ARGUMENT, "gemm: one to three segments");
    std::size_t sum = 0;
    for (int s = 0; s < in.count; ++s) {
        const bool last = s + 1 == in.count;
        if (in.ptr[s] == nullptr || in.cols[s] == 0 || in.ld[s] < in.cols[s] || in.ld[s] % 8 != 0 || in.cols[s] % 8 != 0 ||
            !is_aligned16(in.ptr[s]) || (!last && in.cols[s] % granule != 0) ||
            in.cols[s] > static_cast<std::size_t>(std::numeric_limits<int>::max()))
            return fail(CGPTX_INVALID_ARGUMENT, "gemm: malformed operand segment");
        out.ptr[s] = in.ptr[s];
        out.ld[s] = static_cast<long>(in.ld[s]);
        out.cols[s] = static_cast<int>(in.cols[s]);
        sum += in.cols[s];
    }
    if (sum != total) return fail(CGPTX_INVALID_ARGUMENT, "gemm: segments do not cover the operand");
    out.count = in.count;
    return CGPTX_OK;
}

// The streamed loads address an operand relative to the block's tile origin with 32-bit byte
// offsets: a tile's rows (k-contiguous operand) or the whole K extent (n-contiguous operand).
bool offsets_fit_32bit(const GemmArgs& g, std::size_t elem) {
    // Below 2 GiB: bit 31 of a scalar offset is what pushes the loads of K tiles past the end out of range.
    constexpr std::size_t limit = (std::size_t{1} << 31) - (std::size_t{1} << 20);
    const std::size_t a_span = g.a_k_contiguous ? (256 * g.lda + g.k) * elem : (g.k * g.lda + 256) * elem;
    const std::size_t b_span = g.b_k_contiguous ? (256 * g.ldb + g.k) * elem : (g.k * g.ldb + 256) * elem;
    // The epilogues address a wavefront's part of C (of the residual, of a split-K partial tile)
    // through a range-checked descriptor with 32-bit offsets as well: up to 256 rows.
    std::size_t c_ld = std::max(g.ldc, g.n);
    for (int s = 0; s < g.c_segments.count; ++s) c_ld = std::max(c_ld, g.c_segments.ld[s]);
    const std::size_t c_span = 256 * c_ld * 4;
    const std::size_t r_span = g.residual != nullptr ? 256 * g.ldr * elem : 0;
    return a_span < limit && b_span < limit && c_span < limit && r_span < limit;
}

template <typename T>
int run_typed(const GemmArgs& g, hipStream_t stream) {
    KernelArgs p{};
    p.a = g.a;
    p.b = g.b;
    p.c = g.c;
    p.bias = g.bias;
    p.residual = g.residual;
    p.ldr = static_cast<long>(g.ldr);
    p.addend = g.addend_f32;
    p.ld_addend = static_cast<long>(g.ld_addend);
    p.m = static_cast<int>(g.m);
    p.n = static_cast<int>(g.n);
    p.k = static_cast<int>(g.k);
    p.lda = static_cast<long>(g.lda);
    p.ldb = static_cast<long>(g.ldb);
    p.ldc = static_cast<long>(g.ldc);
    p.accumulate = g.accumulate ? 1 : 0;
    p.c_f32 = g.c_is_f32 ? 1 : 0;
    if (g.swiglu_out != nullptr) {
        if (!gemm_fuses_swiglu(g)) return fail(CGPTX_INVALID_ARGUMENT, "gemm: this call cannot carry the SwiGLU epilogue");
        p.act = g.swiglu_out;
        p.ld_act = static_cast<long>(g.ld_swiglu);
        p.inter = static_cast<int>(g.n / 2);
    }
    if (g.swiglu_saved != nullptr) {
        if (!gemm_fuses_swiglu_gradient(g)) return fail(CGPTX_INVALID_ARGUMENT, "gemm: this call cannot carry the SwiGLU gradient epilogue");
        p.saved = g.swiglu_saved;
        p.ld_saved = static_cast<long>(g.ld_swiglu);
        p.inter = static_cast<int>(g.n);
    }
    if (g.batch_rows != 0) {
        if (!gemm_takes_batch(g)) return fail(CGPTX_INVALID_ARGUMENT, "gemm: this call cannot be a stack of products");
        p.batch_rows = static_cast<int>(g.batch_rows);
        p.a_batch_stride = static_cast<long>(g.a_batch_stride);
        p.b_batch_stride = static_cast<long>(g.b_batch_stride);
        for (int s = 0; s < 3; ++s) p.a_seg_batch_stride[s] = static_cast<long>(g.a_segment_batch_stride[s]);
    }
    const bool segmented = g.a_segments.count > 0 || g.c_segments.count > 0;
    if (segmented) {
        if (int s = copy_segments(g.a_segments, g.a_k_contiguous ? g.k : (g.batch_rows != 0 ? g.batch_rows : g.m),
                                  g.a_k_contiguous ? kBK : 256, p.a_seg))
            return s;
        if (int s = copy_segments(g.c_segments, g.n, 256, p.c_seg)) return s;
        if (g.c_segments.count > 0 && (g.c_is_f32 || g.residual != nullptr))
            return fail(CGPTX_INVALID_ARGUMENT, "gemm: a segmented output takes neither fp32 storage nor a residual");
        if (std::is_same_v<T, float>) return fail(CGPTX_INVALID_ARGUMENT, "gemm: segmented operands need 16-bit storage");
    }

    bool fast = false;
    if constexpr (!std::is_same_v<T, float>) {
        const std::size_t c_elem = g.c_is_f32 ? 4 : sizeof(T);
        GemmArgs whole = g;  // alignment of segmented operands was checked per segment
        if (g.a_segments.count > 0) {
            whole.a = g.a_segments.ptr[0];
            whole.lda = g.a_segments.ld[0];
        }
        if (g.c_segments.count > 0) {
            whole.c = const_cast<void*>(g.c_segments.ptr[0]);
            whole.ldc = g.c_segments.ld[0];
        }
        const GemmArgs& g = whole;
        fast = g.k % kBK == 0 && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.n % 8 == 0 && g.m % 8 == 0 &&
               is_aligned16(g.a) && is_aligned16(g.b) && (g.ldc * c_elem) % 16 == 0 && is_aligned16(g.c) &&
               (g.bias == nullptr || (reinterpret_cast<std::uintptr_t>(g.bias) & 7u) == 0) &&
               (g.residual == nullptr || ((reinterpret_cast<std::uintptr_t>(g.residual) & 7u) == 0 && g.ldr % 4 == 0)) &&
               (g.addend_f32 == nullptr || (is_aligned16(g.addend_f32) && g.ld_addend % 4 == 0)) &&
               !(!g.a_k_contiguous && g.b_k_contiguous) && offsets_fit_32bit(g, sizeof(T));
    }
    if (!fast && segmented) return fail(CGPTX_INVALID_ARGUMENT, "gemm: segmented operands need the aligned MFMA path");
    if (!fast && g.batch_rows != 0) return fail(CGPTX_INVALID_ARGUMENT, "gemm: a stack of products needs the aligned MFMA path");
    if (!fast) {
        const dim3 grid(static_cast<unsigned int>((g.n + kF32Tile - 1) / kF32Tile),
                        static_cast<unsigned int>((g.m + kF32Tile - 1) / kF32Tile));
        if (grid.y > 65535u) return fail(CGPTX_OVERFLOW, "gemm: too many rows for the fp32 kernel's grid");
        hipLaunchKernelGGL((gemm_f32_mfma_kernel<T>), grid, dim3(kThreads), 0, stream, p, g.a_k_contiguous ? 1 : 0,
                           g.b_k_contiguous ? 1 : 0);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    }
    if constexpr (!std::is_same_v<T, float>) {
        // 256x256 tiles (one block per CU, 64 MFMAs per wavefront and K step) when they still give
        // every CU a tile, or when K is long enough to be split across the idle CUs without the
        // fp32 partial tiles outweighing the contraction (at least 8 tiles, so at most 32 slices);
        // otherwise 128x128 tiles, with K split when even those are too few.
        const long big_tiles = static_cast<long>((g.m + 255) / 256) * static_cast<long>((g.n + 255) / 256);
        const int forced = forced_tile();
        const long units = compute_units();
        const bool fills = big_tiles * 5 >= units * 4;
        const bool splits = (!g.no_split || g.split_workspace != nullptr) && g.residual == nullptr && g.addend_f32 == nullptr &&
                            g.c_segments.count == 0 && big_tiles >= 8 &&
                            g.k / kBK >= static_cast<std::size_t>(32 * ((units + big_tiles - 1) / big_tiles));
        const bool big = g.swiglu_out != nullptr || g.swiglu_saved != nullptr || g.batch_rows != 0 || forced == 256 ||
                         (forced == 0 && (fills || splits));
        if (big) return run_config<T, 256, 256>(g, p, stream);
        return run_config<T, 128, 128>(g, p, stream);
    }
    return CGPTX_OK;
}

}  // namespace

bool gemm_fuses_swiglu(const GemmArgs& g) {
    if (g.swiglu_out == nullptr || g.dtype == CGPTX_F32 || !g.a_k_contiguous || !g.b_k_contiguous || g.bias != nullptr ||
        g.residual != nullptr || g.accumulate || g.c_is_f32 || g.a_segments.count > 0 || g.c_segments.count > 0 ||
        g.a == nullptr || g.b == nullptr || g.c == nullptr)
        return false;
    const std::size_t elem = 2, inter = g.n / 2;
    // Whole 128-column units of gate and of up per tile, tiles that fill the chip (the 256x256
    // configuration), 16-byte aligned rows everywhere, and the whole weight within 32-bit offsets.
    if (g.n % 256 != 0 || g.m % 8 != 0 || g.k % kBK != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0 || g.ldc % 8 != 0 ||
        g.ld_swiglu % 8 != 0 || g.ld_swiglu < inter || !is_aligned16(g.a) || !is_aligned16(g.b) || !is_aligned16(g.c) ||
        !is_aligned16(g.swiglu_out))
        return false;
    const long tiles = static_cast<long>((g.m + 255) / 256) * static_cast<long>(g.n / 256);
    if (forced_tile() == 128 || tiles * 5 < static_cast<long>(compute_units()) * 4) return false;
    constexpr std::size_t limit = (std::size_t{1} << 31) - (std::size_t{1} << 20);
    return offsets_fit_32bit(g, elem) && (g.n * g.ldb + g.k) * elem < limit && 256 * g.ld_swiglu * elem < limit;
}

bool gemm_fuses_swiglu_gradient(const GemmArgs& g) {
    if (g.swiglu_saved == nullptr || g.swiglu_out != nullptr || g.dtype == CGPTX_F32 || !g.a_k_contiguous || g.b_k_contiguous ||
        g.bias != nullptr || g.residual != nullptr || g.accumulate || g.c_is_f32 || g.a_segments.count > 0 ||
        g.c_segments.count > 0 || g.a == nullptr || g.b == nullptr || g.c == nullptr)
        return false;
    const std::size_t elem = 2;
    // 16-byte chunks of whole rows everywhere, tiles that fill the chip (the 256x256 configuration),
    // and a wavefront's 128 rows of the saved and of the written [gate | up] within 32-bit offsets.
    if (g.n % 8 != 0 || g.m % 8 != 0 || g.k % kBK != 0 || g.lda % 8 != 0 || g.ldb % 8 != 0 || g.ldc % 8 != 0 ||
        g.ld_swiglu % 8 != 0 || g.ldc < 2 * g.n || g.ld_swiglu < 2 * g.n || !is_aligned16(g.a) || !is_aligned16(g.b) ||
        !is_aligned16(g.c) || !is_aligned16(g.swiglu_saved))
        return false;
    const long tiles = static_cast<long>((g.m + 255) / 256) * static_cast<long>((g.n + 255) / 256);
    if (forced_tile() == 128 || tiles * 5 < static_cast<long>(compute_units()) * 4) return false;
    constexpr std::size_t limit = (std::size_t{1} << 31) - (std::size_t{1} << 20);
    return offsets_fit_32bit(g, elem) && 256 * g.ld_swiglu * elem < limit;
}

bool gemm_takes_batch(const GemmArgs& g) {
    if (g.batch_rows == 0) return true;
    if (g.dtype == CGPTX_F32 || g.a_k_contiguous || g.b_k_contiguous || g.bias != nullptr || g.residual != nullptr ||
        g.addend_f32 != nullptr || g.accumulate || g.c_is_f32 || g.c_segments.count > 0 || g.swiglu_out != nullptr ||
        g.swiglu_saved != nullptr || g.no_split || g.c == nullptr || g.b == nullptr)
        return false;
    if (g.batch_rows % 256 != 0 || g.m % g.batch_rows != 0 || g.n % 8 != 0 || g.k % kBK != 0 || g.ldb % 8 != 0 ||
        g.ldc % 8 != 0 || g.b_batch_stride % 8 != 0)
        return false;
    if (g.a_segments.count == 0) return g.a != nullptr && g.lda % 8 == 0 && g.a_batch_stride % 8 == 0;
    for (int s = 0; s < g.a_segments.count && s < 3; ++s)
        if (g.a_segment_batch_stride[s] % 8 != 0) return false;
    return true;
}

int gemm(const GemmArgs& g, hipStream_t stream) {
    if ((g.a == nullptr && g.a_segments.count == 0) || g.b == nullptr || (g.c == nullptr && g.c_segments.count == 0) ||
        g.m == 0 || g.n == 0 || g.k == 0)
        return fail(CGPTX_INVALID_ARGUMENT, "gemm: null or empty operand");
    constexpr std::size_t i32max = std::numeric_limits<int>::max();
    if (g.m > i32max || g.n > i32max || g.k > i32max)
        return fail(CGPTX_OVERFLOW, "gemm: dimension exceeds int range");
    return dispatch_dtype(g.dtype, [&]<typename T>() -> int { return run_typed<T>(g, stream); });
}

}  // namespace cgptx
