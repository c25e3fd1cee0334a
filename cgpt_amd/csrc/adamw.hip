// Fused multi-tensor AdamW for gfx950.
//
// Semantics: src/optim/adamw.cu:74-187 (gradient statistics, device-side step
// preparation, batched update) and 269-435 (host entry points). The reference
// launches two kernels per tensor (181 launches for the 104m model); here the
// whole parameter list is covered by three launches:
//   1. stats:   the tensors are cut into 4096-element chunks; a block takes eight
//               consecutive chunks, requests all their 128-bit gradient loads
//               before it adds anything and writes one partial Σ(g/scale)² per
//               chunk; a non-finite value sets an integer flag.
//   2. prepare: one block sums the partials in a fixed order (in double), decides
//               skip / step++ / bias corrections / clip factor on the device.
//   3. update:  one chunk per block; reads g, m, v, master, writes m, v, master, param.
// The non-finite flag exists twice and the calls alternate between the two (the
// call counter lives on the device, so a captured sequence alternates as well):
// prepare clears the one the next call will use, which saves a launch that only
// cleared a flag.
// The block → (tensor, offset) map is a binary search in a small prefix table
// that lives in the workspace. HBM traffic per parameter: g twice, m/v/master
// read+write, param write = 30 B with 16-bit params.
//
// The squared norm is order-independent here (fixed partial order), where the
// reference adds block sums with float atomics.
#include "common.hpp"

#include <cmath>
#include <limits>
#include <vector>

namespace cgptx {
namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 4096;  // elements per block

struct DeviceEntry {
    void* parameter;
    const void* gradient;
    float* master;
    float* first;
    float* second;
    unsigned long long count;
    int dtype;
    int pad;
};

struct Hyper {
    float learning_rate, beta1, beta2, epsilon, weight_decay, loss_scale, max_grad_norm;
};

// Device-side scalars of one workspace.
struct DeviceState {
    unsigned int non_finite;           // this call skips its update (set by prepare, read by update and the host)
    unsigned int observed_non_finite;
    unsigned long long step;
    float scalars[4];  // bias_correction1, bias_correction2, clip, unused
    float squared_norm;
    unsigned int calls;                // completed prepare passes; its parity picks the flag a call uses
    unsigned int found_non_finite[2];  // set by the statistics pass of a call, cleared by the previous call's prepare
    // The options of the call in progress. The three kernels read them from here, not from their arguments, so
    // that a captured sequence of them follows a learning rate that changes from step to step: the caller
    // writes the options (adamw_set_hyper_kernel, outside the capture) before every launch of the graph.
    Hyper hyper;
    unsigned int pad;
};

__device__ __forceinline__ int find_entry(const unsigned int* __restrict__ chunk_begin, int entries,
                                          unsigned int chunk) {
    int lo = 0, hi = entries;  // chunk_begin[lo] <= chunk < chunk_begin[hi]
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (chunk_begin[mid] <= chunk) lo = mid; else hi = mid;
    }
    return lo;
}

__device__ __forceinline__ float block_sum(float v, float* stage) {
    v = wave_sum(v);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    if (lane == 0) stage[wave] = v;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < kThreads / kWave; ++w) total += stage[w];
    return total;
}

constexpr int kStatsChunks = 4;  // consecutive chunks per block of the statistics pass

// g / loss_scale. A power-of-two scale (the usual choice) divides exactly by multiplying with its reciprocal,
// which takes one instruction instead of a dozen; any other scale is divided by, so that the value is the one
// the update uses.
struct Unscale {
    float scale, reciprocal;
    bool exact;  // reciprocal is a power of two
};
__device__ __forceinline__ float unscale(float g, const Unscale& s) { return s.exact ? g * s.reciprocal : g / s.scale; }

// A non-finite gradient makes its sum non-finite (and so does an overflowing sum): the sums are checked, not
// every element; the squared norm of a pass that found one is not used.
// Σ (g / loss_scale)² over the calling thread's elements of one chunk (vector v = thread, thread + 256, ... of the
// chunk, then the elements past the last whole vector), in that order; `bad` is set by a non-finite value.
// Vector loads are requested together, before any arithmetic.
template <typename T>
__device__ __forceinline__ float stats_chunk(const T* __restrict__ g, unsigned long long begin, unsigned long long end,
                                             const Unscale& scale, bool& bad) {
    constexpr int VEC = kVec128<T>;
    constexpr int kPasses = kChunk / (kThreads * VEC) > 0 ? kChunk / (kThreads * VEC) : 1;
    const bool aligned = (reinterpret_cast<std::uintptr_t>(g + begin) & 15u) == 0;
    const unsigned long long count = end - begin;
    const unsigned long long vectors = aligned ? count / VEC : 0;
    float sum = 0.0f;
    vec_t<T, VEC> held[kPasses];
#pragma unroll
    for (int k = 0; k < kPasses; ++k) {
        const unsigned long long v = static_cast<unsigned long long>(k) * kThreads + threadIdx.x;
        if (v < vectors) held[k] = load_vec<T, VEC>(g + begin + v * VEC);
    }
#pragma unroll
    for (int k = 0; k < kPasses; ++k) {
        const unsigned long long v = static_cast<unsigned long long>(k) * kThreads + threadIdx.x;
        if (v >= vectors) continue;
        const vec_t<float, VEC> x = vec_to_f32<T, VEC>(held[k]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float grad = unscale(x[e], scale);
            sum = fmaf(grad, grad, sum);
        }
    }
    for (unsigned long long i = begin + vectors * VEC + threadIdx.x; i < end; i += kThreads) {
        const float grad = unscale(to_f32(g[i]), scale);
        sum = fmaf(grad, grad, sum);
    }
    if (!isfinite(sum)) bad = true;
    return sum;
}

// kStatsChunks whole chunks of one tensor, 16-byte aligned: every load of the block is requested before the first
// addition. The additions per chunk are those of stats_chunk, in its order.
template <typename T>
__device__ __forceinline__ void stats_run(const T* __restrict__ g, const Unscale& scale, float (&sums)[kStatsChunks], bool& bad) {
    constexpr int VEC = kVec128<T>;
    constexpr int kPasses = kChunk / (kThreads * VEC);
    static_assert(kPasses >= 1 && kPasses * kThreads * VEC == kChunk, "a chunk is a whole number of block-wide vector passes");
    vec_t<T, VEC> held[kStatsChunks][kPasses];
#pragma unroll
    for (int c = 0; c < kStatsChunks; ++c)
#pragma unroll
        for (int k = 0; k < kPasses; ++k) held[c][k] = load_vec<T, VEC>(g + c * kChunk + (k * kThreads + threadIdx.x) * VEC);
#pragma unroll
    for (int c = 0; c < kStatsChunks; ++c) {
        float sum = 0.0f;
#pragma unroll
        for (int k = 0; k < kPasses; ++k) {
            const vec_t<float, VEC> x = vec_to_f32<T, VEC>(held[c][k]);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const float grad = unscale(x[e], scale);
                sum = fmaf(grad, grad, sum);
            }
        }
        if (!isfinite(sum)) bad = true;
        sums[c] = sum;
    }
}

__global__ void adamw_set_hyper_kernel(DeviceState* state, Hyper hyper) { state->hyper = hyper; }

__global__ __launch_bounds__(kThreads) void adamw_stats_kernel(const DeviceEntry* __restrict__ entries,
                                                              const unsigned int* __restrict__ chunk_begin,
                                                              int entry_count, unsigned int total_chunks,
                                                              float* __restrict__ partial, DeviceState* state) {
    const float loss_scale = state->hyper.loss_scale;
    __shared__ float stage[kStatsChunks][kThreads / kWave];
    __shared__ int any_bad;
    if (threadIdx.x == 0) any_bad = 0;
    __syncthreads();
    const unsigned int first_chunk = blockIdx.x * kStatsChunks;
    // The tensor of the block's first chunk is found by bisection, those of the following chunks by stepping on.
    int e = find_entry(chunk_begin, entry_count, first_chunk);
    float sums[kStatsChunks];
    bool bad = false;
    int exponent = 0;
    const Unscale scale{loss_scale, 1.0f / loss_scale, frexpf(loss_scale, &exponent) == 0.5f};
    const DeviceEntry head = entries[e];
    const unsigned long long head_begin = static_cast<unsigned long long>(first_chunk - chunk_begin[e]) * kChunk;
    const std::size_t elem = head.dtype == CGPTX_F32 ? 4 : 2;
    const bool whole_run = head_begin + static_cast<unsigned long long>(kStatsChunks) * kChunk <= head.count &&
                           ((reinterpret_cast<std::uintptr_t>(head.gradient) + head_begin * elem) & 15u) == 0;
    if (whole_run) {
        switch (head.dtype) {
            case CGPTX_F16: stats_run(static_cast<const f16_t*>(head.gradient) + head_begin, scale, sums, bad); break;
            case CGPTX_BF16: stats_run(static_cast<const bf16_t*>(head.gradient) + head_begin, scale, sums, bad); break;
            default: stats_run(static_cast<const float*>(head.gradient) + head_begin, scale, sums, bad); break;
        }
    } else {
#pragma unroll
        for (int c = 0; c < kStatsChunks; ++c) {
            const unsigned int chunk = first_chunk + c;
            sums[c] = 0.0f;
            if (chunk >= total_chunks) continue;
            while (chunk >= chunk_begin[e + 1]) ++e;
            const DeviceEntry entry = entries[e];
            const unsigned long long begin = static_cast<unsigned long long>(chunk - chunk_begin[e]) * kChunk;
            const unsigned long long end = begin + kChunk < entry.count ? begin + kChunk : entry.count;
            switch (entry.dtype) {
                case CGPTX_F16: sums[c] = stats_chunk(static_cast<const f16_t*>(entry.gradient), begin, end, scale, bad); break;
                case CGPTX_BF16: sums[c] = stats_chunk(static_cast<const bf16_t*>(entry.gradient), begin, end, scale, bad); break;
                default: sums[c] = stats_chunk(static_cast<const float*>(entry.gradient), begin, end, scale, bad); break;
            }
        }
    }
    if (bad) any_bad = 1;  // benign race: every writer stores 1
    // One partial per chunk: lanes of a wavefront by butterfly, then the wavefronts in order.
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int c = 0; c < kStatsChunks; ++c) {
        const float v = wave_sum(sums[c]);
        if (lane == 0) stage[c][wave] = v;
    }
    __syncthreads();
    if (threadIdx.x < kStatsChunks && first_chunk + threadIdx.x < total_chunks) {
        float total = 0.0f;
#pragma unroll
        for (int w = 0; w < kThreads / kWave; ++w) total += stage[threadIdx.x][w];
        partial[first_chunk + threadIdx.x] = total;
    }
    if (threadIdx.x == 0 && any_bad) atomicExch(&state->found_non_finite[state->calls & 1u], 1u);
}

// One block. Fixed-order sum of the partials, then the decision logic of
// adamw_prepare_step_kernel (src/optim/adamw.cu:166-187).
constexpr int kPrepareThreads = 1024;
__global__ __launch_bounds__(kPrepareThreads) void adamw_prepare_kernel(const float* __restrict__ partial,
                                                                       unsigned int partial_count, DeviceState* state,
                                                                       int advance_step) {
    __shared__ double stage[kPrepareThreads];
    // Four independent sums per thread keep four loads in flight (one block adds some 25,000 partials for the 104m
    // model); the order of the additions is fixed by the partial count alone.
    double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
    unsigned int i = threadIdx.x;
    for (; i + 3 * kPrepareThreads < partial_count; i += 4 * kPrepareThreads) {
        s0 += static_cast<double>(partial[i]);
        s1 += static_cast<double>(partial[i + kPrepareThreads]);
        s2 += static_cast<double>(partial[i + 2 * kPrepareThreads]);
        s3 += static_cast<double>(partial[i + 3 * kPrepareThreads]);
    }
    for (; i < partial_count; i += kPrepareThreads) s0 += static_cast<double>(partial[i]);
    stage[threadIdx.x] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    for (int stride = kPrepareThreads / 2; stride > 0; stride >>= 1) {
        if (threadIdx.x < stride) stage[threadIdx.x] += stage[threadIdx.x + stride];
        __syncthreads();
    }
    if (threadIdx.x != 0) return;
    const float squared = static_cast<float>(stage[0]);
    state->squared_norm = squared;
    const unsigned int parity = state->calls & 1u;
    const bool found = state->found_non_finite[parity] != 0u;
    state->found_non_finite[parity ^ 1u] = 0u;  // the flag of the next call
    state->calls += 1u;
    if (found || !isfinite(squared)) {
        state->non_finite = 1u;
        state->observed_non_finite = 1u;
        return;
    }
    state->non_finite = 0u;
    const float beta1 = state->hyper.beta1, beta2 = state->hyper.beta2, max_grad_norm = state->hyper.max_grad_norm;
    if (advance_step) {
        const unsigned long long next_step = state->step + 1ull;
        state->step = next_step;
        state->scalars[0] = 1.0f - powf(beta1, static_cast<float>(next_step));
        state->scalars[1] = 1.0f - powf(beta2, static_cast<float>(next_step));
    }
    if (isinf(max_grad_norm)) {
        state->scalars[2] = 1.0f;
    } else {
        const float norm = sqrtf(squared);
        state->scalars[2] = norm > max_grad_norm ? max_grad_norm / norm : 1.0f;
    }
}

__device__ __forceinline__ void adamw_element(float grad_raw, float& m, float& v, float& master, const Hyper& h,
                                              float bc1, float bc2, float clip) {
    const float grad = grad_raw / h.loss_scale * clip;
    m = h.beta1 * m + (1.0f - h.beta1) * grad;
    v = h.beta2 * v + (1.0f - h.beta2) * grad * grad;
    const float normalized = m / bc1 / (sqrtf(v / bc2) + h.epsilon);
    master = master * (1.0f - h.learning_rate * h.weight_decay) - h.learning_rate * normalized;
}

template <typename T>
__device__ __forceinline__ void update_chunk(const DeviceEntry& entry, unsigned long long begin,
                                             unsigned long long end, const Hyper& h, float bc1, float bc2,
                                             float clip) {
    constexpr int VEC = 4;  // elements per lane and access: 128 bits of each fp32 state tensor
    T* p = static_cast<T*>(entry.parameter);
    const T* g = static_cast<const T*>(entry.gradient);
    const bool aligned = ((reinterpret_cast<std::uintptr_t>(p + begin) | reinterpret_cast<std::uintptr_t>(g + begin)) &
                          (VEC * sizeof(T) - 1)) == 0 &&
                         ((reinterpret_cast<std::uintptr_t>(entry.master + begin) |
                           reinterpret_cast<std::uintptr_t>(entry.first + begin) |
                           reinterpret_cast<std::uintptr_t>(entry.second + begin)) & 15u) == 0;
    const unsigned long long count = end - begin;
    const unsigned long long vectors = aligned ? count / VEC : 0;
    // A thread requests everything it will touch in the chunk before it computes anything: kPasses groups of four
    // elements, each group's position in the chunk chosen so that every access instruction of a wavefront covers one
    // contiguous kilobyte of an fp32 state tensor (512 B of 16-bit gradients or parameters) - whole cache lines per
    // instruction for the loads and, which matters more, for the stores.
    constexpr int kPasses = kChunk / (kThreads * VEC) > 0 ? kChunk / (kThreads * VEC) : 1;
    for (unsigned long long v0 = 0; v0 < vectors; v0 += static_cast<unsigned long long>(kPasses) * kThreads) {
        vec_t<T, VEC> gr[kPasses];
        vec_t<float, 4> mm[kPasses], vv[kPasses], ww[kPasses];
        bool live[kPasses];
#pragma unroll
        for (int k = 0; k < kPasses; ++k) {
            const unsigned long long vi = v0 + static_cast<unsigned long long>(k) * kThreads + threadIdx.x;
            live[k] = vi < vectors;
            if (!live[k]) continue;
            const unsigned long long at = begin + vi * VEC;
            gr[k] = load_vec<T, VEC>(g + at);
            mm[k] = load_vec<float, 4>(entry.first + at);
            vv[k] = load_vec<float, 4>(entry.second + at);
            ww[k] = load_vec<float, 4>(entry.master + at);
        }
#pragma unroll
        for (int k = 0; k < kPasses; ++k) {
            if (!live[k]) continue;
            const unsigned long long at = begin + (v0 + static_cast<unsigned long long>(k) * kThreads + threadIdx.x) * VEC;
            const vec_t<float, VEC> grad = vec_to_f32<T, VEC>(gr[k]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float m = mm[k][e], v = vv[k][e], w = ww[k][e];
                adamw_element(grad[e], m, v, w, h, bc1, bc2, clip);
                mm[k][e] = m;
                vv[k][e] = v;
                ww[k][e] = w;
            }
            store_vec<float, 4>(entry.first + at, mm[k]);
            store_vec<float, 4>(entry.second + at, vv[k]);
            store_vec<float, 4>(entry.master + at, ww[k]);
            store_vec<T, VEC>(p + at, vec_from_f32<T, VEC>(ww[k]));
        }
    }
    for (unsigned long long i = begin + vectors * VEC + threadIdx.x; i < end; i += kThreads) {
        float m = entry.first[i], v = entry.second[i], w = entry.master[i];
        adamw_element(to_f32(g[i]), m, v, w, h, bc1, bc2, clip);
        entry.first[i] = m;
        entry.second[i] = v;
        entry.master[i] = w;
        p[i] = from_f32<T>(w);
    }
}

__global__ __launch_bounds__(kThreads) void adamw_update_kernel(const DeviceEntry* __restrict__ entries,
                                                               const unsigned int* __restrict__ chunk_begin,
                                                               int entry_count,
                                                               const DeviceState* __restrict__ state) {
    if (state->non_finite != 0u) return;
    const Hyper h = state->hyper;
    const float bc1 = state->scalars[0], bc2 = state->scalars[1], clip = state->scalars[2];
    const int e = find_entry(chunk_begin, entry_count, blockIdx.x);
    const DeviceEntry entry = entries[e];
    const unsigned long long begin = static_cast<unsigned long long>(blockIdx.x - chunk_begin[e]) * kChunk;
    const unsigned long long end = begin + kChunk < entry.count ? begin + kChunk : entry.count;
    switch (entry.dtype) {
        case CGPTX_F16: update_chunk<f16_t>(entry, begin, end, h, bc1, bc2, clip); break;
        case CGPTX_BF16: update_chunk<bf16_t>(entry, begin, end, h, bc1, bc2, clip); break;
        default: update_chunk<float>(entry, begin, end, h, bc1, bc2, clip); break;
    }
}

__global__ void adamw_set_scalars_kernel(DeviceState* state, float bc1, float bc2) {
    state->scalars[0] = bc1;
    state->scalars[1] = bc2;
}

int validate_options(const cgptx_adamw_options* o, const char* name) {
    if (o == nullptr) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null options");
    if (!std::isfinite(o->learning_rate) || o->learning_rate < 0.0f || !std::isfinite(o->beta1) || o->beta1 < 0.0f ||
        o->beta1 >= 1.0f || !std::isfinite(o->beta2) || o->beta2 < 0.0f || o->beta2 >= 1.0f ||
        !std::isfinite(o->epsilon) || o->epsilon <= 0.0f || !std::isfinite(o->weight_decay) ||
        o->weight_decay < 0.0f || !std::isfinite(o->loss_scale) || o->loss_scale <= 0.0f ||
        o->max_grad_norm <= 0.0f || std::isnan(o->max_grad_norm))
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": invalid optimizer options");
    return CGPTX_OK;
}

int validate_entry(const cgptx_adamw_entry& e, const char* name) {
    if (e.parameter == nullptr || e.gradient == nullptr || e.master_parameter == nullptr ||
        e.first_moment == nullptr || e.second_moment == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null entry");
    if (!valid_dtype(e.dtype)) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": unsupported dtype");
    if (e.count == 0) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": empty tensor");
    return CGPTX_OK;
}

Hyper to_hyper(const cgptx_adamw_options& o) {
    return {o.learning_rate, o.beta1, o.beta2, o.epsilon, o.weight_decay, o.loss_scale, o.max_grad_norm};
}

}  // namespace
}  // namespace cgptx

struct cgptx_adamw_workspace {
    cgptx::DeviceState* state = nullptr;       // device
    cgptx::DeviceEntry* entries = nullptr;     // device
    unsigned int* chunk_begin = nullptr;       // device, entry_count + 1
    float* partial = nullptr;                  // device, total_chunks
    std::vector<cgptx_adamw_entry> bound;      // host copy of the bound entry list
    unsigned int total_chunks = 0;
    bool initialized = false;
};

namespace cgptx {
namespace {

int bind_entries(cgptx_adamw_workspace* ws, const cgptx_adamw_entry* entries, std::size_t entry_count,
                 hipStream_t stream) {
    std::vector<DeviceEntry> host(entry_count);
    std::vector<unsigned int> begin(entry_count + 1);
    unsigned long long chunks = 0;
    for (std::size_t i = 0; i < entry_count; ++i) {
        const auto& e = entries[i];
        host[i] = {e.parameter, e.gradient, e.master_parameter, e.first_moment, e.second_moment,
                   static_cast<unsigned long long>(e.count), e.dtype, 0};
        begin[i] = static_cast<unsigned int>(chunks);
        chunks += (e.count + kChunk - 1) / kChunk;
        if (chunks > 0x7fffffffull) return fail(CGPTX_OVERFLOW, "adamw: too many elements for one launch");
    }
    begin[entry_count] = static_cast<unsigned int>(chunks);
    if (ws->entries != nullptr) CGPTX_HIP(hipFree(ws->entries));
    if (ws->chunk_begin != nullptr) CGPTX_HIP(hipFree(ws->chunk_begin));
    if (ws->partial != nullptr) CGPTX_HIP(hipFree(ws->partial));
    CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->entries), entry_count * sizeof(DeviceEntry)));
    CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->chunk_begin), (entry_count + 1) * sizeof(unsigned int)));
    CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&ws->partial), chunks * sizeof(float)));
    // Pageable sources: these copies complete before hipMemcpyAsync returns control
    // to a later kernel on the same stream, and the vectors die at scope exit, so
    // use the synchronous form.
    CGPTX_HIP(hipStreamSynchronize(stream));
    CGPTX_HIP(hipMemcpy(ws->entries, host.data(), entry_count * sizeof(DeviceEntry), hipMemcpyHostToDevice));
    CGPTX_HIP(hipMemcpy(ws->chunk_begin, begin.data(), (entry_count + 1) * sizeof(unsigned int),
                        hipMemcpyHostToDevice));
    ws->total_chunks = static_cast<unsigned int>(chunks);
    ws->bound.assign(entries, entries + entry_count);
    return CGPTX_OK;
}

bool same_entries(const std::vector<cgptx_adamw_entry>& bound, const cgptx_adamw_entry* entries, std::size_t n) {
    if (bound.size() != n) return false;
    for (std::size_t i = 0; i < n; ++i) {
        const auto &a = bound[i], &b = entries[i];
        if (a.parameter != b.parameter || a.gradient != b.gradient || a.master_parameter != b.master_parameter ||
            a.first_moment != b.first_moment || a.second_moment != b.second_moment || a.count != b.count ||
            a.dtype != b.dtype)
            return false;
    }
    return true;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_adamw_workspace_create(cgptx_adamw_workspace** workspace) {
    using namespace cgptx;
    if (workspace == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "adamw_workspace_create: null output");
    auto* ws = new cgptx_adamw_workspace();
    if (int s = check_hip(hipMalloc(reinterpret_cast<void**>(&ws->state), sizeof(DeviceState)), "hipMalloc")) {
        delete ws;
        return s;
    }
    if (int s = check_hip(hipMemset(ws->state, 0, sizeof(DeviceState)), "hipMemset")) {
        (void)hipFree(ws->state);
        delete ws;
        return s;
    }
    *workspace = ws;
    return CGPTX_OK;
}

extern "C" int cgptx_adamw_workspace_destroy(cgptx_adamw_workspace* ws) {
    using namespace cgptx;
    if (ws == nullptr) return CGPTX_OK;
    (void)hipDeviceSynchronize();
    if (ws->state) (void)hipFree(ws->state);
    if (ws->entries) (void)hipFree(ws->entries);
    if (ws->chunk_begin) (void)hipFree(ws->chunk_begin);
    if (ws->partial) (void)hipFree(ws->partial);
    delete ws;
    return CGPTX_OK;
}

namespace cgptx {

// The two halves of adamw_step_many_async, for callers that record the update into a graph: the options travel to
// the device outside the recording (they change from step to step: the learning rate), the three launches inside.
int adamw_set_options(cgptx_adamw_workspace* ws, const cgptx_adamw_options* options, hipStream_t stream) {
    const char* name = "adamw_step_many_async";
    if (int s = validate_options(options, name)) return s;
    if (ws == nullptr) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null workspace");
    hipLaunchKernelGGL(adamw_set_hyper_kernel, dim3(1), dim3(1), 0, stream, ws->state, to_hyper(*options));
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

int adamw_enqueue(cgptx_adamw_workspace* ws, const cgptx_adamw_entry* entries, std::size_t entry_count,
                  std::uint64_t initial_step, hipStream_t stream) {
    const char* name = "adamw_step_many_async";
    if (ws == nullptr) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null workspace");
    if (entries == nullptr || entry_count == 0)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": empty parameter list");
    for (std::size_t i = 0; i < entry_count; ++i)
        if (int s = validate_entry(entries[i], name)) return s;
    if (!ws->initialized) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": the workspace has no entries bound yet");
    if (!same_entries(ws->bound, entries, entry_count))
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": workspace entries changed");
    (void)initial_step;
    const int n = static_cast<int>(entry_count);
    hipLaunchKernelGGL(adamw_stats_kernel, dim3((ws->total_chunks + kStatsChunks - 1) / kStatsChunks), dim3(kThreads), 0, stream,
                       ws->entries, ws->chunk_begin, n, ws->total_chunks, ws->partial, ws->state);
    CGPTX_LAUNCH_CHECK();
    hipLaunchKernelGGL(adamw_prepare_kernel, dim3(1), dim3(kPrepareThreads), 0, stream, ws->partial, ws->total_chunks,
                       ws->state, 1);
    CGPTX_LAUNCH_CHECK();
    hipLaunchKernelGGL(adamw_update_kernel, dim3(ws->total_chunks), dim3(kThreads), 0, stream, ws->entries,
                       ws->chunk_begin, n, ws->state);
    CGPTX_LAUNCH_CHECK();
    return CGPTX_OK;
}

// Binds the entry list on first use (device copies of the list: allocates and synchronises, so never under capture).
int adamw_bind(cgptx_adamw_workspace* ws, const cgptx_adamw_entry* entries, std::size_t entry_count,
               std::uint64_t initial_step, hipStream_t stream) {
    const char* name = "adamw_step_many_async";
    if (ws == nullptr) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null workspace");
    if (entries == nullptr || entry_count == 0)
        return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": empty parameter list");
    for (std::size_t i = 0; i < entry_count; ++i)
        if (int s = validate_entry(entries[i], name)) return s;
    if (ws->initialized) return CGPTX_OK;
    if (int s = bind_entries(ws, entries, entry_count, stream)) return s;
    DeviceState init{};
    init.step = initial_step;
    CGPTX_HIP(hipMemcpy(ws->state, &init, sizeof(init), hipMemcpyHostToDevice));
    ws->initialized = true;
    return CGPTX_OK;
}

}  // namespace cgptx

extern "C" int cgptx_adamw_step_many_async(cgptx_adamw_workspace* ws, const cgptx_adamw_entry* entries,
                                           size_t entry_count, const cgptx_adamw_options* options,
                                           uint64_t initial_step, cgptx_stream stream_) {
    using namespace cgptx;
    auto stream = static_cast<hipStream_t>(stream_);
    if (int s = validate_options(options, "adamw_step_many_async")) return s;
    if (int s = adamw_bind(ws, entries, entry_count, initial_step, stream)) return s;
    if (int s = adamw_set_options(ws, options, stream)) return s;
    return adamw_enqueue(ws, entries, entry_count, initial_step, stream);
}

extern "C" int cgptx_adamw_check(cgptx_adamw_workspace* ws, int* all_finite, uint64_t* step, cgptx_stream stream_) {
    using namespace cgptx;
    if (ws == nullptr || all_finite == nullptr || step == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "adamw_check: null argument");
    auto stream = static_cast<hipStream_t>(stream_);
    CGPTX_HIP(hipStreamSynchronize(stream));
    DeviceState host{};
    CGPTX_HIP(hipMemcpy(&host, ws->state, sizeof(host), hipMemcpyDeviceToHost));
    *all_finite = host.observed_non_finite == 0u ? 1 : 0;
    *step = host.step;
    const unsigned int zero = 0;
    CGPTX_HIP(hipMemcpy(&ws->state->observed_non_finite, &zero, sizeof(zero), hipMemcpyHostToDevice));
    return CGPTX_OK;
}

extern "C" int cgptx_adamw_step(void* parameter, const void* gradient, float* master_parameter, float* first_moment,
                                float* second_moment, size_t count, int dtype, const cgptx_adamw_options* options,
                                uint64_t next_step, int* updated, cgptx_stream stream_) {
    using namespace cgptx;
    const char* name = "adamw_step";
    if (int s = validate_options(options, name)) return s;
    if (updated == nullptr) return fail(CGPTX_INVALID_ARGUMENT, std::string(name) + ": null output flag");
    const cgptx_adamw_entry entry{parameter, gradient, master_parameter, first_moment, second_moment, count, dtype};
    if (int s = validate_entry(entry, name)) return s;
    if (next_step == 0) return fail(CGPTX_OVERFLOW, std::string(name) + ": step counter overflow");
    auto stream = static_cast<hipStream_t>(stream_);
    const unsigned long long chunks = (count + kChunk - 1) / kChunk;
    if (chunks > 0x7fffffffull) return fail(CGPTX_OVERFLOW, std::string(name) + ": tensor too large");
    // Scratch layout: DeviceState | DeviceEntry | chunk_begin[2] | partial[chunks]
    const std::size_t off_entry = 256, off_begin = 512, off_partial = 768;
    void* mem = nullptr;
    if (int s = scratch(stream, off_partial + chunks * sizeof(float), &mem)) return s;
    auto* base = static_cast<char*>(mem);
    auto* state = reinterpret_cast<DeviceState*>(base);
    auto* d_entry = reinterpret_cast<DeviceEntry*>(base + off_entry);
    auto* d_begin = reinterpret_cast<unsigned int*>(base + off_begin);
    auto* partial = reinterpret_cast<float*>(base + off_partial);
    const DeviceEntry h_entry{parameter, gradient, master_parameter, first_moment, second_moment,
                              static_cast<unsigned long long>(count), dtype, 0};
    const unsigned int h_begin[2] = {0u, static_cast<unsigned int>(chunks)};
    const Hyper h = to_hyper(*options);
    DeviceState init{};
    init.hyper = h;
    CGPTX_HIP(hipStreamSynchronize(stream));
    CGPTX_HIP(hipMemcpy(state, &init, sizeof(init), hipMemcpyHostToDevice));
    CGPTX_HIP(hipMemcpy(d_entry, &h_entry, sizeof(h_entry), hipMemcpyHostToDevice));
    CGPTX_HIP(hipMemcpy(d_begin, h_begin, sizeof(h_begin), hipMemcpyHostToDevice));
    hipLaunchKernelGGL(adamw_stats_kernel, dim3(static_cast<unsigned int>((chunks + kStatsChunks - 1) / kStatsChunks)),
                       dim3(kThreads), 0, stream, d_entry, d_begin, 1, static_cast<unsigned int>(chunks), partial, state);
    CGPTX_LAUNCH_CHECK();
    hipLaunchKernelGGL(adamw_prepare_kernel, dim3(1), dim3(kPrepareThreads), 0, stream, partial,
                       static_cast<unsigned int>(chunks), state, 0);
    CGPTX_LAUNCH_CHECK();
    // Bias corrections in double on the host, as adamw_step does (src/optim/adamw.cu:413-415).
    const float bc1 = static_cast<float>(1.0 - std::pow(static_cast<double>(h.beta1), static_cast<double>(next_step)));
    const float bc2 = static_cast<float>(1.0 - std::pow(static_cast<double>(h.beta2), static_cast<double>(next_step)));
    hipLaunchKernelGGL(adamw_set_scalars_kernel, dim3(1), dim3(1), 0, stream, state, bc1, bc2);
    CGPTX_LAUNCH_CHECK();
    hipLaunchKernelGGL(adamw_update_kernel, dim3(static_cast<unsigned int>(chunks)), dim3(kThreads), 0, stream,
                       d_entry, d_begin, 1, state);
    CGPTX_LAUNCH_CHECK();
    CGPTX_HIP(hipStreamSynchronize(stream));
    DeviceState result{};
    CGPTX_HIP(hipMemcpy(&result, state, sizeof(result), hipMemcpyDeviceToHost));
    *updated = result.non_finite == 0u ? 1 : 0;
    return CGPTX_OK;
}
