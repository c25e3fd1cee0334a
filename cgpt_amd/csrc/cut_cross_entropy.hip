// Cut cross-entropy: loss and both gradients of a linear classifier without ever
// holding the [rows, vocabulary] logits.
//
// Semantics: include/ops/cut_cross_entropy.h:25-33 (src/ops/cut_cross_entropy.cu:97-221):
//   z = X·Cᵀ, loss = mean_r(logsumexp z_r − z_{r,y_r}),
//   dX = (softmax(z) − onehot)·C / rows, dC = (softmax(z) − onehot)ᵀ·X / rows.
// The reference recomputes full dot products per thread (O(rows·hidden²·vocab)), which
// cannot run at training size. Here rows are processed in chunks: one MFMA contraction
// produces the chunk's logits into scratch, the softmax kernel turns them into the
// scaled logit gradient in place, and two more contractions consume that gradient
// (dX for the chunk's rows; dC accumulated in fp32 across chunks, so the classifier
// gradient is rounded once). Scratch is chunk·vocab logits + vocab·hidden fp32,
// independent of the number of rows, and three vocabulary-sized contractions are done
// instead of four because the chunk's logits stay resident between loss and gradient.
//
// Extensions over the reference: any storage dtype, a gradient scale (loss scaling),
// and accumulate_classifier for tied embeddings.
#include "cross_entropy.hpp"
#include "gemm.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <limits>

namespace cgptx {
namespace {

constexpr int kThreads = 256;

// out = (accumulate ? out : 0) + acc, element-wise, acc in fp32.
template <typename T>
__global__ __launch_bounds__(kThreads) void finish_classifier_kernel(T* __restrict__ out,
                                                                    const float* __restrict__ acc,
                                                                    std::size_t count, int accumulate) {
    for (std::size_t i = static_cast<std::size_t>(blockIdx.x) * kThreads + threadIdx.x; i < count;
         i += static_cast<std::size_t>(gridDim.x) * kThreads) {
        float v = acc[i];
        if (accumulate) v += to_f32(out[i]);
        out[i] = from_f32<T>(v);
    }
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_cut_cross_entropy_forward_backward(float* loss, void* input_gradient, void* classifier_gradient,
                                                        const void* input, const void* classifier,
                                                        const uint32_t* targets, size_t rows, size_t hidden,
                                                        size_t vocab, float gradient_scale,
                                                        int accumulate_classifier, int dtype, cgptx_stream stream_) {
    using namespace cgptx;
    const char* name = "cut_cross_entropy";
    if (!valid_dtype(dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (loss == nullptr || input_gradient == nullptr || classifier_gradient == nullptr || input == nullptr ||
        classifier == nullptr || targets == nullptr || rows == 0 || hidden == 0 || vocab == 0)
        return fail(CGPTX_INVALID_ARGUMENT,
                    std::string(name) + ": input and classifier must be non-empty matrices with gradients and targets");
    if (!std::isfinite(gradient_scale) || gradient_scale <= 0.0f)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": gradient scale must be finite and positive");
    constexpr std::size_t i32max = std::numeric_limits<int>::max();
    if (rows > i32max || hidden > i32max || vocab > i32max)
        return fail(CGPTX_OVERFLOW, std::string(name) + ": dimension exceeds int range");
    auto stream = static_cast<hipStream_t>(stream_);
    const std::size_t elem = dtype_size(dtype);
    // Chunk so that the logits scratch stays within 2 GiB whatever the number of rows (a small fraction of this
    // GPU's memory; CGPTX_CUT_CE_LOGITS_BYTES, read per call, sets another bound), while each chunk still gives
    // the three contractions enough 256x256 tiles to fill the chip. The rows are split evenly over the chunks.
    // 32768 rows at V=32000 are one chunk: the classifier gradient then comes straight out of its contraction,
    // rounded once, without the fp32 accumulator and the pass that folds it into the gradient.
    // The bound itself stays 1 MiB under 2^31: the streamed contraction kernels address an operand with 32-bit
    // byte offsets below that, and a chunk beyond it would fall back to the plain kernels.
    constexpr std::size_t kMaxLogitsBytes = (std::size_t{1} << 31) - (std::size_t{1} << 20);
    std::size_t logits_bytes = kMaxLogitsBytes;
    if (const char* text = std::getenv("CGPTX_CUT_CE_LOGITS_BYTES")) {
        const unsigned long long asked = std::strtoull(text, nullptr, 0);
        if (asked > 0) logits_bytes = std::min<std::size_t>(static_cast<std::size_t>(asked), kMaxLogitsBytes);
    }
    std::size_t limit = logits_bytes / (vocab * elem);
    limit = std::max<std::size_t>(256, limit / 256 * 256);
    const std::size_t pieces = (rows + limit - 1) / limit;
    std::size_t chunk = ((rows + pieces - 1) / pieces + 255) / 256 * 256;
    chunk = std::min(chunk, rows);
    const bool single = chunk >= rows;
    const std::size_t loss_bytes = (rows * sizeof(float) + 255) & ~std::size_t{255};
    const std::size_t acc_bytes = single ? 0 : (vocab * hidden * sizeof(float) + 255) & ~std::size_t{255};
    const std::size_t logit_bytes = (chunk * vocab * elem + 255) & ~std::size_t{255};
    void* mem = nullptr;
    // Arena layout: [row_loss | acc | logits]. The contractions below run with no_split, so they
    // never ask the arena for split-K scratch of their own.
    if (int s = scratch(stream, loss_bytes + acc_bytes + logit_bytes, &mem)) return s;
    auto* base = static_cast<char*>(mem);
    auto* row_loss = reinterpret_cast<float*>(base);
    auto* acc = reinterpret_cast<float*>(base + loss_bytes);
    void* logits = base + loss_bytes + acc_bytes;
    const float factor = gradient_scale / static_cast<float>(rows);
    for (std::size_t r0 = 0; r0 < rows; r0 += chunk) {
        const std::size_t r = std::min(chunk, rows - r0);
        const void* x = static_cast<const char*>(input) + r0 * hidden * elem;
        GemmArgs z;  // logits[r, V] = X[r, H]·C[V, H]ᵀ
        z.a = x;
        z.b = classifier;
        z.c = logits;
        z.m = r;
        z.n = vocab;
        z.k = hidden;
        z.lda = hidden;
        z.ldb = hidden;
        z.ldc = vocab;
        z.dtype = dtype;
        z.no_split = true;
        if (int s = gemm(z, stream)) return s;
        if (int s = cross_entropy_rows(row_loss + r0, logits, logits, targets + r0, r, vocab, factor, dtype, stream))
            return s;
        GemmArgs dx;  // dX[r, H] = dZ[r, V]·C[V, H]
        dx.a = logits;
        dx.b = classifier;
        dx.c = static_cast<char*>(input_gradient) + r0 * hidden * elem;
        dx.m = r;
        dx.n = hidden;
        dx.k = vocab;
        dx.lda = vocab;
        dx.ldb = hidden;
        dx.ldc = hidden;
        dx.b_k_contiguous = false;
        dx.dtype = dtype;
        dx.no_split = true;
        if (int s = gemm(dx, stream)) return s;
        GemmArgs dc;  // acc[V, H] (+)= dZᵀ[V, r]·X[r, H], fp32; a single chunk writes the gradient itself
        dc.a = logits;
        dc.b = x;
        dc.c = single ? classifier_gradient : static_cast<void*>(acc);
        dc.m = vocab;
        dc.n = hidden;
        dc.k = r;
        dc.lda = vocab;
        dc.ldb = hidden;
        dc.ldc = hidden;
        dc.a_k_contiguous = false;
        dc.b_k_contiguous = false;
        dc.accumulate = single ? accumulate_classifier != 0 : r0 != 0;
        dc.c_is_f32 = !single;
        dc.dtype = dtype;
        dc.no_split = true;
        if (int s = gemm(dc, stream)) return s;
    }
    if (int s = mean_reduce(loss, row_loss, rows, stream)) return s;
    if (single) return CGPTX_OK;
    const std::size_t count = vocab * hidden;
    const std::size_t blocks = std::min<std::size_t>((count + kThreads - 1) / kThreads,
                                                     static_cast<std::size_t>(compute_units()) * 16);
    return dispatch_dtype(dtype, [&]<typename T>() -> int {
        hipLaunchKernelGGL((finish_classifier_kernel<T>), dim3(static_cast<unsigned int>(blocks)), dim3(kThreads), 0,
                           stream, static_cast<T*>(classifier_gradient), acc, count, accumulate_classifier);
        CGPTX_LAUNCH_CHECK();
        return CGPTX_OK;
    });
}
