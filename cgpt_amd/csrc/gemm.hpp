// Internal GEMM interface shared by the linear ops and cut-cross-entropy.
#pragma once

#include "common.hpp"

namespace cgptx {

// C[M,N] (+)= op(A)·op(B) with fp32 accumulation.
//   a_k_contiguous: A is stored [M, K] (row stride lda) — otherwise [K, M].
//   b_k_contiguous: B is stored [N, K] (row stride ldb) — otherwise [K, N].
// C is row-major [M, N] with row stride ldc, in the storage dtype of A and B
// (or fp32 when c_is_f32). accumulate adds into C. residual (optional, [M, N], storage dtype, row
// stride ldr, may be C itself) is added elementwise. bias (optional, [N], storage
// dtype) is added to every row after the product.
// Up to three column ranges of one logical matrix that live in separate row-major buffers
// (e.g. the query, key and value activations next to each other). count == 0: not used.
struct GemmSegments {
    const void* ptr[3] = {nullptr, nullptr, nullptr};
    std::size_t ld[3] = {0, 0, 0};
    std::size_t cols[3] = {0, 0, 0};
    int count = 0;
};

struct GemmArgs {
    const void* a = nullptr;
    const void* b = nullptr;
    void* c = nullptr;
    const void* bias = nullptr;
    const void* residual = nullptr;
    const float* addend_f32 = nullptr;  // optional fp32 [M, N] (row stride ld_addend) added to the product first
    std::size_t ld_addend = 0;
    std::size_t m = 0, n = 0, k = 0;
    std::size_t lda = 0, ldb = 0, ldc = 0, ldr = 0;
    bool a_k_contiguous = true;
    bool b_k_contiguous = true;
    bool accumulate = false;
    bool c_is_f32 = false;
    bool no_split = false;  // never use split-K scratch (the caller owns the arena)
    // Memory for split-K partial tiles from a caller that owns the arena (used instead of the arena when the
    // launch is split along K; a launch whose partials would not fit runs unsplit).
    void* split_workspace = nullptr;
    std::size_t split_workspace_bytes = 0;
    int dtype = CGPTX_BF16;
    // Column segments of A as stored (its K range when k-contiguous, its M range otherwise) and of
    // C (written through; not combined with split-K, residual or fp32 output). Segment widths are
    // multiples of 256 (of 32 for a k-contiguous A) except the last; a and lda / c and ldc are
    // ignored for a segmented operand.
    GemmSegments a_segments, c_segments;
    // Forward projection into the concatenated [gate | up] layout (n = 2·inter, b = [gate; up]
    // weights) that also writes swiglu_out[m, inter] = silu(gate)·up, computed from the rounded
    // gate and up values (the bits the separate operator would produce). Only for calls that
    // gemm_fuses_swiglu() accepts.
    void* swiglu_out = nullptr;
    std::size_t ld_swiglu = 0;
    // Input gradient of the down projection (c = dY·W with n = inter) that writes the gradient of
    // the forward's [gate | up] instead of the gradient of silu(gate)·up: c is [m, 2·inter] = [dgate |
    // dup] (ldc >= 2·inter), swiglu_saved the forward's [m, 2·inter] = [gate | up] with row stride
    // ld_swiglu. The contraction is rounded to the storage dtype before the SwiGLU gradient is
    // applied (the bits of the two separate operators). Only for calls that
    // gemm_fuses_swiglu_gradient() accepts.
    const void* swiglu_saved = nullptr;
    // Several products of one shape in one launch (weight gradients of equal layers): C is the stack of their results,
    // [m, n] with m = batch x batch_rows, and the rows batch_rows j .. batch_rows (j + 1) - 1 of it are
    // A_j^T B_j with A_j = a + j a_batch_stride and B_j = b + j b_batch_stride (elements; for a segmented A every
    // segment moves by its own stride). Only for the layout of a weight gradient (neither operand k-contiguous),
    // 16-bit storage and batch_rows a multiple of 256; batch_rows = 0: one product. Only for calls that
    // gemm_takes_batch() accepts.
    std::size_t batch_rows = 0;
    std::size_t a_batch_stride = 0, b_batch_stride = 0;
    std::size_t a_segment_batch_stride[3] = {0, 0, 0};
};

int gemm(const GemmArgs& args, hipStream_t stream);
// Whether gemm() serves args.swiglu_out for this call (shape, layout and alignment of the fused kernel).
bool gemm_fuses_swiglu(const GemmArgs& args);
bool gemm_fuses_swiglu_gradient(const GemmArgs& args);
// Whether gemm() serves args.batch_rows for this call.
bool gemm_takes_batch(const GemmArgs& args);

}  // namespace cgptx
