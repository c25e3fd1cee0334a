// Shared device/host helpers for the gfx950 kernels: storage types, 128-bit
// vector access, wavefront (64-lane) reductions, status plumbing and the
// per-stream scratch arena.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

#include "cgptx.h"

namespace cgptx {

using bf16_t = __bf16;
using f16_t = _Float16;

constexpr int kWave = 64;

template <typename T, int N>
struct VecOf {
    typedef T type __attribute__((ext_vector_type(N)));
};
template <typename T, int N>
using vec_t = typename VecOf<T, N>::type;

// Elements of T in one 128-bit access.
template <typename T>
constexpr int kVec128 = 16 / sizeof(T);

template <typename T>
__device__ __forceinline__ float to_f32(T v) { return static_cast<float>(v); }
template <typename T>
__device__ __forceinline__ T from_f32(float v) { return static_cast<T>(v); }

// Round a float through storage type T (what a store followed by a load does).
template <typename T>
__device__ __forceinline__ float round_to(float v) { return static_cast<float>(static_cast<T>(v)); }

template <typename T, int N>
__device__ __forceinline__ vec_t<float, N> vec_to_f32(vec_t<T, N> v) {
    return __builtin_convertvector(v, vec_t<float, N>);
}
template <typename T, int N>
__device__ __forceinline__ vec_t<T, N> vec_from_f32(vec_t<float, N> v) {
    return __builtin_convertvector(v, vec_t<T, N>);
}

template <typename T, int N>
__device__ __forceinline__ vec_t<T, N> load_vec(const T* p) {
    return *reinterpret_cast<const vec_t<T, N>*>(p);
}
template <typename T, int N>
__device__ __forceinline__ void store_vec(T* p, vec_t<T, N> v) {
    *reinterpret_cast<vec_t<T, N>*>(p) = v;
}

// The value of lane (lane ^ offset) for offset 8, 4, 2 or 1 inside a row of 16 lanes, taken through the data-parallel
// operand path of the vector unit instead of the LDS crossbar. Offsets 8, 2 and 1 are exact lane exchanges (a row
// rotation by 8, two quad permutations). Offset 4 is a row rotation by 4, which hands lane i the value of lane
// (i ^ 4) or (i ^ 4 ^ 8): the same bits whenever lanes i and i ^ 8 hold equal values, which is the case right after
// the offset-8 step of a butterfly that runs from large offsets to small ones.
template <int offset>
__device__ __forceinline__ float row_exchange(float v) {
    static_assert(offset == 8 || offset == 4 || offset == 2 || offset == 1);
    constexpr int control = offset == 8 ? 0x128 : offset == 4 ? 0x124 : offset == 2 ? 0x4E : 0xB1;
    const int bits = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(bits, control, 0xF, 0xF, true));
}

// Butterfly reductions across `width` adjacent lanes (width a power of two <= 64), from the largest offset down.
// Steps across rows of 16 lanes go through the LDS crossbar, the last four stay in the vector unit; the result has
// the bits of the plain butterfly (a + b and max(a, b) do not depend on which of the two equal partners is read).
template <int width = kWave>
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int offset = width / 2; offset > 8; offset >>= 1) v += __shfl_xor(v, offset, kWave);
    if constexpr (width >= 16) v += row_exchange<8>(v);
    if constexpr (width >= 16) v += row_exchange<4>(v);
    else if constexpr (width >= 8) v += __shfl_xor(v, 4, kWave);
    if constexpr (width >= 4) v += row_exchange<2>(v);
    if constexpr (width >= 2) v += row_exchange<1>(v);
    return v;
}
template <int width = kWave>
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int offset = width / 2; offset > 8; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
    if constexpr (width >= 16) v = fmaxf(v, row_exchange<8>(v));
    if constexpr (width >= 16) v = fmaxf(v, row_exchange<4>(v));
    else if constexpr (width >= 8) v = fmaxf(v, __shfl_xor(v, 4, kWave));
    if constexpr (width >= 4) v = fmaxf(v, row_exchange<2>(v));
    if constexpr (width >= 2) v = fmaxf(v, row_exchange<1>(v));
    return v;
}

inline bool is_aligned16(const void* p) { return (reinterpret_cast<std::uintptr_t>(p) & 15u) == 0; }

// ---- status ---------------------------------------------------------------
int fail(int code, const std::string& message);   // records the message, returns code
int check_hip(hipError_t error, const char* what); // CGPTX_OK or CGPTX_RUNTIME
void clear_error();

#define CGPTX_HIP(expr)                                              \
    do {                                                             \
        if (int status_ = ::cgptx::check_hip((expr), #expr)) return status_; \
    } while (0)

#define CGPTX_LAUNCH_CHECK() CGPTX_HIP(hipGetLastError())

inline bool valid_dtype(int dtype) { return dtype == CGPTX_F16 || dtype == CGPTX_BF16 || dtype == CGPTX_F32; }
inline std::size_t dtype_size(int dtype) { return dtype == CGPTX_F32 ? 4 : 2; }

// Calls fn.template operator()<T>() with T chosen from a dtype code.
template <typename Fn>
int dispatch_dtype(int dtype, Fn&& fn) {
    switch (dtype) {
        case CGPTX_F16: return fn.template operator()<f16_t>();
        case CGPTX_BF16: return fn.template operator()<bf16_t>();
        case CGPTX_F32: return fn.template operator()<float>();
        default: return fail(CGPTX_INVALID_ARGUMENT, "unsupported dtype");
    }
}

// ---- weight-gradient reductions of several norm-backward passes as one pair of launches ----------
// A norm-backward pass leaves per-workgroup partial sums of the weight gradient [parts, hidden] and reduces them
// over the parts in two small launches. A caller that runs many such passes (the train step: four per block) may
// hand them a sink instead: the pass then takes its partial-sum memory from the sink (which must outlive the pass,
// unlike the per-stream arena that the next operator reuses), records what is to be reduced, and the caller runs
// all recorded reductions with run_column_reductions — the same arithmetic in the same order, two launches in all.
struct ColumnReduceEntry {
    const float* partial;  // [parts, hidden]
    float* second;         // [slices, hidden] (used when slices > 1)
    void* out;             // T[hidden]
    int parts, hidden, slices, dtype;
    bool operator==(const ColumnReduceEntry& o) const {
        return partial == o.partial && second == o.second && out == o.out && parts == o.parts && hidden == o.hidden &&
               slices == o.slices && dtype == o.dtype;
    }
};
struct ColumnReduceSink {
    char* memory = nullptr;      // device memory owned by the caller
    std::size_t capacity = 0;    // bytes behind `memory`
    std::size_t used = 0;        // bytes handed out since begin()
    std::size_t wanted = 0;      // bytes asked for since begin(), served or not
    std::vector<ColumnReduceEntry> entries;
    void begin() {
        used = 0;
        wanted = 0;
        entries.clear();
    }
    // 256-byte aligned block, or nullptr when it does not fit (the pass then reduces at once, from the arena).
    void* take(std::size_t bytes) {
        bytes = (bytes + 255) & ~std::size_t{255};
        wanted += bytes;
        if (memory == nullptr || used + bytes > capacity) return nullptr;
        void* block = memory + used;
        used += bytes;
        return block;
    }
};
// Bytes one norm-backward pass of the given kind takes from a sink (0: that shape reduces at once, from the arena).
enum class NormPass { plain, with_rope, dual };
std::size_t rmsnorm_backward_sink_bytes(NormPass pass, std::size_t rows, std::size_t hidden, int dtype);
// Runs the reductions recorded in `table` (device copy of `count` entries). max_hidden / max_slices: the largest
// values among the entries (they size the grid).
int run_column_reductions(const ColumnReduceEntry* table, int count, int max_hidden, int max_slices, hipStream_t stream);

// ---- fused variants used by the composed train step --------------------------
// rmsnorm backward with grad_input = (norm gradient) + residual; residual may be null or alias
// grad_input. Same validation and results as cgptx_rmsnorm_backward otherwise.
int rmsnorm_backward_residual(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                              const void* weight, const void* residual, std::size_t rows, std::size_t hidden,
                              float epsilon, int dtype, hipStream_t stream, ColumnReduceSink* sink = nullptr);

// Per-head RMSNorm and rotary embedding in one pass over [rows = tokens x heads, head_dim]:
//   forward   output = rope(rmsnorm(input));   backward   the gradient of that, with the weight gradient.
// Bit for bit what the separate operators give (their intermediate roundings are kept). Positions are
// position_offset + token % sequence, token = row / heads. `rmsnorm_rope_fusable` says whether the shape,
// dtype and alignment are served; callers run the separate operators otherwise.
bool rmsnorm_rope_fusable(const void* a, const void* b, const void* c, const void* weight, const void* cos_cache,
                          const void* sin_cache, std::size_t head_dim, std::size_t rotary_dim, int dtype);
int rmsnorm_rope_forward(void* output, const void* input, const void* weight, const void* cos_cache, const void* sin_cache,
                         std::size_t rows, std::size_t head_dim, std::size_t heads, std::size_t sequence,
                         std::size_t rotary_dim, std::size_t position_offset, float epsilon, int dtype, hipStream_t stream);
int rmsnorm_rope_backward(void* grad_input, void* grad_weight, const void* grad_output, const void* input,
                          const void* weight, const void* cos_cache, const void* sin_cache, std::size_t rows,
                          std::size_t head_dim, std::size_t heads, std::size_t sequence, std::size_t rotary_dim,
                          std::size_t position_offset, float epsilon, int dtype, hipStream_t stream,
                          ColumnReduceSink* sink = nullptr);

// Two RMSNorms of the same rows with different weights in one pass (x is read once):
//   forward   output_a = rmsnorm(input; weight_a), output_f = rmsnorm(input; weight_f)
//   backward  grad_input = d(norm_a) + d(norm_f) + residual (residual may be null or alias grad_input),
//             and both weight gradients. `rmsnorm_dual_fusable` says whether shape, dtype and the
//             alignment of the five tensors are served.
bool rmsnorm_dual_fusable(const void* a, const void* b, const void* c, const void* d, const void* e, std::size_t hidden,
                          int dtype);
int rmsnorm_forward_dual(void* output_a, void* output_f, const void* input, const void* weight_a, const void* weight_f,
                         std::size_t rows, std::size_t hidden, float epsilon, int dtype, hipStream_t stream);
int rmsnorm_backward_dual(void* grad_input, void* grad_weight_a, void* grad_weight_f, const void* grad_output_a,
                          const void* grad_output_f, const void* input, const void* weight_a, const void* weight_f,
                          const void* residual, std::size_t rows, std::size_t hidden, float epsilon, int dtype,
                          hipStream_t stream, ColumnReduceSink* sink = nullptr);

// ---- the batched AdamW update in parts, for a caller that records it into a graph ----------------------------
// adamw_bind: first use of a workspace (device copies of the entry list; allocates and synchronises). adamw_set_options:
// one small launch that writes the options where the update's kernels read them; it stays outside a recording, since
// the learning rate changes from step to step. adamw_enqueue: the three launches of the update, recordable.
// cgptx_adamw_step_many_async is the three of them in a row.
int adamw_bind(cgptx_adamw_workspace* workspace, const cgptx_adamw_entry* entries, std::size_t entry_count,
               std::uint64_t initial_step, hipStream_t stream);
int adamw_set_options(cgptx_adamw_workspace* workspace, const cgptx_adamw_options* options, hipStream_t stream);
int adamw_enqueue(cgptx_adamw_workspace* workspace, const cgptx_adamw_entry* entries, std::size_t entry_count,
                  std::uint64_t initial_step, hipStream_t stream);

// ---- scratch arena ----------------------------------------------------------
// Returns `bytes` of device scratch bound to (current device, stream), 256-byte
// aligned. Grows by reallocation on eager calls; refuses to grow during capture.
int scratch(hipStream_t stream, std::size_t bytes, void** out);

// Identifies the block currently behind the (current device, stream) arena: it changes whenever that
// arena is reallocated (a larger request) and reads 0 after cgptx_release_scratch. A captured graph
// holds the block's address, so whoever replays one compares this value with the one at capture time
// and captures again when they differ.
std::uint64_t scratch_generation(hipStream_t stream);

// Number of compute units of the current device (cached).
int compute_units();

}  // namespace cgptx
