// Column reductions shared by the norm and linear kernels.
#pragma once

#include "common.hpp"

namespace cgptx {

constexpr int kReduceThreads = 256;
constexpr int kReduceWaves = kReduceThreads / kWave;

// Sums partial[P, H] over P in a fixed order and stores (or adds) in T.
template <typename T>
__global__ __launch_bounds__(kReduceThreads) void column_partial_reduce_kernel(
    T* __restrict__ out, const float* __restrict__ partial, int parts, int hidden, int accumulate) {
    __shared__ float stage[kReduceWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = blockIdx.x * kWave + lane;
    float v0 = 0.0f, v1 = 0.0f, v2 = 0.0f, v3 = 0.0f;
    if (col < hidden) {
        int p = slice;
        for (; p + 3 * kReduceWaves < parts; p += 4 * kReduceWaves) {
            v0 += partial[static_cast<std::size_t>(p) * hidden + col];
            v1 += partial[static_cast<std::size_t>(p + kReduceWaves) * hidden + col];
            v2 += partial[static_cast<std::size_t>(p + 2 * kReduceWaves) * hidden + col];
            v3 += partial[static_cast<std::size_t>(p + 3 * kReduceWaves) * hidden + col];
        }
        for (; p < parts; p += kReduceWaves) v0 += partial[static_cast<std::size_t>(p) * hidden + col];
    }
    stage[slice][lane] = (v0 + v1) + (v2 + v3);
    __syncthreads();
    if (slice == 0 && col < hidden) {
        float v = 0.0f;
#pragma unroll
        for (int s = 0; s < kReduceWaves; ++s) v += stage[s][lane];
        if (accumulate) v += to_f32(out[col]);
        out[col] = from_f32<T>(v);
    }
}


// First level for many parts: block (x, y) of a (column groups, slices) grid folds the parts of
// slice y for its 64 columns into second[y, col]; column_partial_reduce_kernel over the `slices`
// rows of `second` finishes. (A single launch whose last block finishes would need device-scope
// fences, which cost more here than the second launch.)
static __global__ __launch_bounds__(kReduceThreads) void column_partial_fold_kernel(float* __restrict__ second,
                                                                            const float* __restrict__ partial,
                                                                            int parts, int hidden) {
    __shared__ float stage[kReduceWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = blockIdx.x * kWave + lane;
    const int slices = gridDim.y;
    const int chunk = (parts + slices - 1) / slices;
    const int begin = blockIdx.y * chunk;
    const int end = begin + chunk < parts ? begin + chunk : parts;
    float v0 = 0.0f, v1 = 0.0f;
    if (col < hidden) {
        int p = begin + slice;
        for (; p + kReduceWaves < end; p += 2 * kReduceWaves) {
            v0 += partial[static_cast<std::size_t>(p) * hidden + col];
            v1 += partial[static_cast<std::size_t>(p + kReduceWaves) * hidden + col];
        }
        if (p < end) v0 += partial[static_cast<std::size_t>(p) * hidden + col];
    }
    stage[slice][lane] = v0 + v1;
    __syncthreads();
    if (slice == 0 && col < hidden) {
        float v = 0.0f;
#pragma unroll
        for (int s = 0; s < kReduceWaves; ++s) v += stage[s][lane];
        second[static_cast<std::size_t>(blockIdx.y) * hidden + col] = v;
    }
}

// Slices for the kernel above: enough blocks to fill the chip, at least sixteen parts each.
inline int wide_reduce_slices(int parts, int hidden, int units) {
    const int groups = (hidden + kWave - 1) / kWave;
    int slices = 2 * units / groups;
    if (slices > parts / 16) slices = parts / 16;
    return slices < 1 ? 1 : slices;
}

// partial[blockIdx.y, col] = Σ over this block's row slice of in[row, col] (fp32).
template <typename T>
__global__ __launch_bounds__(kReduceThreads) void column_sum_partial_kernel(float* __restrict__ partial,
                                                                           const T* __restrict__ in, long rows,
                                                                           int cols, long rows_per_slice) {
    __shared__ float stage[kReduceWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = blockIdx.x * kWave + lane;
    const long row_begin = blockIdx.y * rows_per_slice;
    const long row_end = row_begin + rows_per_slice < rows ? row_begin + rows_per_slice : rows;
    float v = 0.0f;
    if (col < cols) {
        for (long row = row_begin + slice; row < row_end; row += kReduceWaves) v += to_f32(in[row * cols + col]);
    }
    stage[slice][lane] = v;
    __syncthreads();
    if (slice == 0 && col < cols) {
        float total = 0.0f;
#pragma unroll
        for (int s = 0; s < kReduceWaves; ++s) total += stage[s][lane];
        partial[static_cast<long>(blockIdx.y) * cols + col] = total;
    }
}

}  // namespace cgptx
