// linear_forward / linear_backward on top of the MFMA contraction kernels.
//
// Reference interfaces: include/ops/linear.h (Y = X·Wᵀ + b) and
// include/ops/backward/linear_backward.h:36-46 (dX = dY·W, dW = dYᵀ·X,
// db = Σ_rows dY), CPU arithmetic src/ops/cpu/backward/linear_backward_cpu.cpp:131-165.
#include "gemm.hpp"
#include "reduce.hpp"

#include <limits>

namespace cgptx {
namespace {

int validate(const char* name, std::size_t rows, std::size_t in_features, std::size_t out_features, int dtype) {
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (rows == 0 || in_features == 0 || out_features == 0)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": empty shape");
    constexpr std::size_t i32max = std::numeric_limits<int>::max();
    if (rows > i32max || in_features > i32max || out_features > i32max)
        return fail(CGPTX_OVERFLOW, std::string(name) + ": dimension exceeds int range");
    return CGPTX_OK;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_linear_forward(void* output, const void* input, const void* weight, const void* bias,
                                    size_t rows, size_t in_features, size_t out_features, int dtype,
                                    cgptx_stream stream) {
    using namespace cgptx;
    if (int s = validate("linear_forward", rows, in_features, out_features, dtype)) return s;
    if (output == nullptr || input == nullptr || weight == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "linear_forward: null tensor");
    GemmArgs g;
    g.a = input;
    g.b = weight;
    g.c = output;
    g.bias = bias;
    g.m = rows;
    g.n = out_features;
    g.k = in_features;
    g.lda = in_features;
    g.ldb = in_features;
    g.ldc = out_features;
    g.dtype = dtype;
    return gemm(g, static_cast<hipStream_t>(stream));
}

extern "C" int cgptx_linear_swiglu_forward(void* gate_up, void* activated, const void* input, const void* weight,
                                           size_t rows, size_t in_features, size_t hidden, int dtype,
                                           cgptx_stream stream_) {
    using namespace cgptx;
    if (hidden > std::numeric_limits<std::size_t>::max() / 2)
        return fail(CGPTX_OVERFLOW, "linear_swiglu_forward: dimension exceeds int range");
    if (int s = validate("linear_swiglu_forward", rows, in_features, 2 * hidden, dtype)) return s;
    if (gate_up == nullptr || activated == nullptr || input == nullptr || weight == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "linear_swiglu_forward: null tensor");
    auto stream = static_cast<hipStream_t>(stream_);
    GemmArgs g;
    g.a = input;
    g.b = weight;
    g.c = gate_up;
    g.m = rows;
    g.n = 2 * hidden;
    g.k = in_features;
    g.lda = in_features;
    g.ldb = in_features;
    g.ldc = 2 * hidden;
    g.dtype = dtype;
    g.swiglu_out = activated;
    g.ld_swiglu = hidden;
    if (gemm_fuses_swiglu(g)) return gemm(g, stream);
    // Shapes the fused kernel does not take: the two operators one after the other (same bits).
    g.swiglu_out = nullptr;
    if (int s = gemm(g, stream)) return s;
    return cgptx_swiglu_forward_packed(activated, gate_up, rows, hidden, dtype, stream_);
}

extern "C" int cgptx_linear_swiglu_backward(void* grad_gate_up, void* grad_activated, const void* grad_output,
                                            const void* weight, const void* gate_up, size_t rows, size_t hidden,
                                            size_t out_features, int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    if (hidden > std::numeric_limits<std::size_t>::max() / 2)
        return fail(CGPTX_OVERFLOW, "linear_swiglu_backward: dimension exceeds int range");
    if (int s = validate("linear_swiglu_backward", rows, 2 * hidden, out_features, dtype)) return s;
    if (grad_gate_up == nullptr || grad_activated == nullptr || grad_output == nullptr || weight == nullptr || gate_up == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "linear_swiglu_backward: null tensor");
    auto stream = static_cast<hipStream_t>(stream_);
    GemmArgs g;  // d(activated)[rows, hidden] = dY[rows, out] · W[out, hidden]
    g.a = grad_output;
    g.b = weight;
    g.c = grad_gate_up;
    g.m = rows;
    g.n = hidden;
    g.k = out_features;
    g.lda = out_features;
    g.ldb = hidden;
    g.ldc = 2 * hidden;
    g.b_k_contiguous = false;
    g.dtype = dtype;
    g.swiglu_saved = gate_up;
    g.ld_swiglu = 2 * hidden;
    if (gemm_fuses_swiglu_gradient(g)) return gemm(g, stream);
    // Shapes the fused kernel does not take: the two operators one after the other (same bits).
    g.swiglu_saved = nullptr;
    g.c = grad_activated;
    g.ldc = hidden;
    if (int s = gemm(g, stream)) return s;
    return cgptx_swiglu_backward_packed(grad_gate_up, grad_activated, gate_up, rows, hidden, 0, dtype, stream_);
}

extern "C" int cgptx_linear_backward_weights_stacked(void* grad_weight, const void* grad_output, const void* input,
                                                     size_t rows, size_t in_features, size_t out_features,
                                                     size_t count, size_t grad_output_stride, size_t input_stride,
                                                     int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    if (int s = validate("linear_backward_weights_stacked", rows, in_features, out_features, dtype)) return s;
    if (grad_weight == nullptr || grad_output == nullptr || input == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "linear_backward_weights_stacked: null tensor");
    if (count == 0) return fail(CGPTX_INVALID_ARGUMENT, "linear_backward_weights_stacked: empty stack");
    if (count > static_cast<std::size_t>(std::numeric_limits<int>::max()) / out_features)
        return fail(CGPTX_OVERFLOW, "linear_backward_weights_stacked: dimension exceeds int range");
    auto stream = static_cast<hipStream_t>(stream_);
    GemmArgs g;  // rows j out .. (j + 1) out - 1 of dW = dY_jᵀ[out, rows] · X_j[rows, in]
    g.a = grad_output;
    g.b = input;
    g.c = grad_weight;
    g.m = count * out_features;
    g.n = in_features;
    g.k = rows;
    g.lda = out_features;
    g.ldb = in_features;
    g.ldc = in_features;
    g.a_k_contiguous = false;
    g.b_k_contiguous = false;
    g.dtype = dtype;
    g.batch_rows = out_features;
    g.a_batch_stride = grad_output_stride;
    g.b_batch_stride = input_stride;
    if (count > 1 && gemm_takes_batch(g) && is_aligned16(grad_output) && is_aligned16(input) && is_aligned16(grad_weight) &&
        rows % 32 == 0)
        return gemm(g, stream);
    // Shapes the stacked launch does not take: one weight gradient after the other.
    const std::size_t elem = dtype_size(dtype);
    for (std::size_t j = 0; j < count; ++j) {
        if (int s = cgptx_linear_backward(nullptr, static_cast<char*>(grad_weight) + j * out_features * in_features * elem,
                                          nullptr, static_cast<const char*>(grad_output) + j * grad_output_stride * elem,
                                          static_cast<const char*>(input) + j * input_stride * elem, nullptr, rows,
                                          in_features, out_features, 0, 0, 0, dtype, stream_))
            return s;
    }
    return CGPTX_OK;
}

extern "C" int cgptx_linear_backward(void* grad_input, void* grad_weight, void* grad_bias, const void* grad_output,
                                     const void* input, const void* weight, size_t rows, size_t in_features,
                                     size_t out_features, int accumulate_input, int accumulate_weight,
                                     int accumulate_bias, int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    if (int s = validate("linear_backward", rows, in_features, out_features, dtype)) return s;
    if (grad_output == nullptr || (grad_input != nullptr && weight == nullptr) ||
        (grad_weight != nullptr && input == nullptr))
        return fail(CGPTX_INVALID_ARGUMENT, "linear_backward: null tensor");
    auto stream = static_cast<hipStream_t>(stream_);
    if (grad_input != nullptr) {  // dX[rows, in] = dY[rows, out] · W[out, in]
        GemmArgs g;
        g.a = grad_output;
        g.b = weight;
        g.c = grad_input;
        g.m = rows;
        g.n = in_features;
        g.k = out_features;
        g.lda = out_features;
        g.ldb = in_features;
        g.ldc = in_features;
        g.b_k_contiguous = false;
        g.accumulate = accumulate_input != 0;
        g.dtype = dtype;
        if (int s = gemm(g, stream)) return s;
    }
    if (grad_weight != nullptr) {  // dW[out, in] = dYᵀ[out, rows] · X[rows, in]
        GemmArgs g;
        g.a = grad_output;
        g.b = input;
        g.c = grad_weight;
        g.m = out_features;
        g.n = in_features;
        g.k = rows;
        g.lda = out_features;
        g.ldb = in_features;
        g.ldc = in_features;
        g.a_k_contiguous = false;
        g.b_k_contiguous = false;
        g.accumulate = accumulate_weight != 0;
        g.dtype = dtype;
        if (int s = gemm(g, stream)) return s;
    }
    if (grad_bias != nullptr) {  // db[out] = Σ_rows dY
        const int cols = static_cast<int>(out_features);
        const int slices = rows < 256 ? 1 : (rows < 65536 ? 64 : 256);
        const long rows_per_slice = (static_cast<long>(rows) + slices - 1) / slices;
        void* mem = nullptr;
        if (int s = scratch(stream, static_cast<std::size_t>(slices) * out_features * sizeof(float), &mem)) return s;
        auto* partial = static_cast<float*>(mem);
        const int col_blocks = (cols + kWave - 1) / kWave;
        return dispatch_dtype(dtype, [&]<typename T>() -> int {
            hipLaunchKernelGGL((column_sum_partial_kernel<T>), dim3(col_blocks, slices), dim3(kReduceThreads), 0,
                               stream, partial, static_cast<const T*>(grad_output), static_cast<long>(rows), cols,
                               rows_per_slice);
            CGPTX_LAUNCH_CHECK();
            hipLaunchKernelGGL((column_partial_reduce_kernel<T>), dim3(col_blocks), dim3(kReduceThreads), 0, stream,
                               static_cast<T*>(grad_bias), partial, slices, cols, accumulate_bias != 0 ? 1 : 0);
            CGPTX_LAUNCH_CHECK();
            return CGPTX_OK;
        });
    }
    return CGPTX_OK;
}
