// Internal interface of the softmax cross-entropy row kernels (used by the dense and the cut path).
#pragma once

#include "common.hpp"

namespace cgptx {

// row_loss[r] = [y_r < V](logsumexp z_r − z_{r,y_r}); gradient (may be null) = (softmax − onehot)·factor.
int cross_entropy_rows(float* row_loss, void* gradient, const void* logits, const std::uint32_t* targets,
                       std::size_t rows, std::size_t vocab, float factor, int dtype, hipStream_t stream);

// loss[0] = (Σ row_loss) / rows, summed in a fixed order.
int mean_reduce(float* loss, const float* row_loss, std::size_t rows, hipStream_t stream);

}  // namespace cgptx
