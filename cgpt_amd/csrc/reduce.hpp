// Column reductions shared by the norm and linear kernels.
#pragma once

#include "common.hpp"

namespace cgptx {

constexpr int kReduceThreads = 256;
constexpr int kReduceWaves = kReduceThreads / kWave;

// Sums partial[P, H] over P in a fixed order and stores (or adds) in T; `group` = which 64 columns.
template <typename T>
__device__ __forceinline__ void column_partial_reduce_body(T* __restrict__ out, const float* __restrict__ partial,
                                                           int parts, int hidden, int accumulate, int group) {
    __shared__ float stage[kReduceWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = group * kWave + lane;
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
template <typename T>
__global__ __launch_bounds__(kReduceThreads) void column_partial_reduce_kernel(
    T* __restrict__ out, const float* __restrict__ partial, int parts, int hidden, int accumulate) {
    column_partial_reduce_body<T>(out, partial, parts, hidden, accumulate, static_cast<int>(blockIdx.x));
}

// First level for many parts: block (group, index) of a (column groups, slices) grid folds the parts of
// slice `index` for its 64 columns into second[index, col]; column_partial_reduce_kernel over the `slices`
// rows of `second` finishes. (A single launch whose last block finishes would need device-scope
// fences, which cost more here than the second launch.)
__device__ __forceinline__ void column_partial_fold_body(float* __restrict__ second, const float* __restrict__ partial,
                                                         int parts, int hidden, int slices, int index, int group) {
    __shared__ float stage[kReduceWaves][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int slice = threadIdx.x / kWave;
    const int col = group * kWave + lane;
    const int chunk = (parts + slices - 1) / slices;
    const int begin = index * chunk;
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
        second[static_cast<std::size_t>(index) * hidden + col] = v;
    }
}
static __global__ __launch_bounds__(kReduceThreads) void column_partial_fold_kernel(float* __restrict__ second,
                                                                            const float* __restrict__ partial,
                                                                            int parts, int hidden) {
    column_partial_fold_body(second, partial, parts, hidden, static_cast<int>(gridDim.y), static_cast<int>(blockIdx.y),
                             static_cast<int>(blockIdx.x));
}

// The two kernels above over a table of reductions (blockIdx.z, or blockIdx.y of the second, picks the entry):
// the same additions in the same order for every entry, whatever else is in the table.
static __global__ __launch_bounds__(kReduceThreads) void column_partial_fold_table_kernel(
    const ColumnReduceEntry* __restrict__ table) {
    const ColumnReduceEntry e = table[blockIdx.z];
    if (e.slices <= 1 || static_cast<int>(blockIdx.y) >= e.slices || static_cast<int>(blockIdx.x) * kWave >= e.hidden) return;
    column_partial_fold_body(e.second, e.partial, e.parts, e.hidden, e.slices, static_cast<int>(blockIdx.y),
                             static_cast<int>(blockIdx.x));
}
static __global__ __launch_bounds__(kReduceThreads) void column_partial_reduce_table_kernel(
    const ColumnReduceEntry* __restrict__ table) {
    const ColumnReduceEntry e = table[blockIdx.y];
    if (static_cast<int>(blockIdx.x) * kWave >= e.hidden) return;
    const float* source = e.slices > 1 ? e.second : e.partial;
    const int parts = e.slices > 1 ? e.slices : e.parts;
    const int group = static_cast<int>(blockIdx.x);
    switch (e.dtype) {
        case CGPTX_F16: column_partial_reduce_body<f16_t>(static_cast<f16_t*>(e.out), source, parts, e.hidden, 0, group); break;
        case CGPTX_BF16: column_partial_reduce_body<bf16_t>(static_cast<bf16_t*>(e.out), source, parts, e.hidden, 0, group); break;
        default: column_partial_reduce_body<float>(static_cast<float*>(e.out), source, parts, e.hidden, 0, group); break;
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
