// Cut cross-entropy: loss and both gradients of a linear classifier without ever
// holding the [rows, vocabulary] logits.
//
// Semantics: include/ops/cut_cross_entropy.h:25-33 (src/ops/cut_cross_entropy.cu:97-221):
//   z = X·Cᵀ, loss = mean_r(logsumexp z_r − z_{r,y_r}),
//   dX = (softmax(z) − onehot)·C / rows, dC = (softmax(z) − onehot)ᵀ·X / rows.
// The reference recomputes full dot products per thread (O(rows·hidden²·vocab)), which
// cannot run at training size. Here rows are processed in chunks of at most 1 GiB of logits: one
// MFMA contraction produces the chunk's logits into scratch, the softmax kernel turns them into
// the scaled logit gradient in place, and two more contractions consume that gradient (dX for the
// chunk's rows; dC accumulated in fp32 across chunks — the last chunk's contraction adds the
// accumulator in its epilogue — so the classifier gradient is rounded once; a single chunk writes
// it straight out of its contraction, which rounds the same sum in another order of additions).
// Scratch is chunk·vocab logits + vocab·hidden fp32, independent of the number of rows, and three
// vocabulary-sized contractions are done instead of four because the chunk's logits stay resident
// between loss and gradient.
//
// Extensions over the reference: any storage dtype, a gradient scale (loss scaling),
// and accumulate_classifier for tied embeddings.
#include "cross_entropy.hpp"
#include "gemm.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <limits>

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
    // Rows are processed in chunks so that the logits scratch stays within 1 GiB whatever the number of rows
    // (CGPTX_CUT_CE_LOGITS_BYTES, read per call, sets another bound, up to 2 GiB - 1 MiB: the streamed contraction
    // kernels address an operand with 32-bit byte offsets below that). The rows are split evenly over the chunks.
    // At V = 32000 in 16-bit storage the bound gives chunks of 16384 rows, which still fill the chip: 64 x 4 tiles
    // of a chunk's input gradient, one per compute unit. Measured at [32768, 1024] x [32000, 1024]: 1 GiB costs
    // nothing against one 2 GiB chunk (6.04 - 6.12 against 6.03 - 6.05 ms), 512 MiB 3.5 % (the input gradient of an
    // 8192-row chunk has to be split along K), 256 MiB 8 %.
    constexpr std::size_t kMaxLogitsBytes = (std::size_t{1} << 31) - (std::size_t{1} << 20);
    std::size_t logits_bytes = std::size_t{1} << 30;
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
    // A chunk's input gradient has few output tiles ([chunk, hidden]) and a long K (the vocabulary): with several
    // chunks it is split along K into up to `units / tiles` slices, whose fp32 partial tiles need room of their own.
    const std::size_t dx_tiles = ((chunk + 255) / 256) * ((hidden + 255) / 256);
    const std::size_t dx_slices = single ? 1 : std::max<std::size_t>(1, static_cast<std::size_t>(compute_units()) / std::max<std::size_t>(dx_tiles, 1));
    const std::size_t split_bytes = dx_slices > 1 ? (dx_slices * chunk * hidden * sizeof(float) + 255) & ~std::size_t{255} : 0;
    void* mem = nullptr;
    // Arena layout: [row_loss | acc | split-K partials | logits]. The contractions below run with no_split: they
    // never ask the arena for scratch of their own, and split only into the room given to them here.
    if (int s = scratch(stream, loss_bytes + acc_bytes + split_bytes + logit_bytes, &mem)) return s;
    auto* base = static_cast<char*>(mem);
    auto* row_loss = reinterpret_cast<float*>(base);
    auto* acc = reinterpret_cast<float*>(base + loss_bytes);
    void* split_room = split_bytes != 0 ? base + loss_bytes + acc_bytes : nullptr;
    void* logits = base + loss_bytes + acc_bytes + split_bytes;
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
        dx.split_workspace = split_room;
        dx.split_workspace_bytes = split_bytes;
        if (int s = gemm(dx, stream)) return s;
        // dC = Σ_chunks dZᵀ[V, r]·X[r, H]: all chunks but the last add their product to acc (fp32; the first one
        // starts it), the last one adds acc to its own and writes the gradient, rounded once. A single chunk
        // writes the gradient itself.
        const bool last = r0 + chunk >= rows;
        GemmArgs dc;
        dc.a = logits;
        dc.b = x;
        dc.c = last ? classifier_gradient : static_cast<void*>(acc);
        dc.m = vocab;
        dc.n = hidden;
        dc.k = r;
        dc.lda = vocab;
        dc.ldb = hidden;
        dc.ldc = hidden;
        dc.a_k_contiguous = false;
        dc.b_k_contiguous = false;
        dc.accumulate = last ? accumulate_classifier != 0 : r0 != 0;
        dc.c_is_f32 = !last;
        if (last && !single) {
            dc.addend_f32 = acc;
            dc.ld_addend = hidden;
        }
        dc.dtype = dtype;
        dc.no_split = true;
        if (int s = gemm(dc, stream)) return s;
    }
    return mean_reduce(loss, row_loss, rows, stream);
}
