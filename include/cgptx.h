/*
 * cgptx.h — C-ABI of the MI355X (gfx950) training hot path.
 *
 * Every entry point takes plain device pointers, sizes, a dtype code and a
 * hipStream_t (passed as void*), enqueues work on that stream and returns a
 * status code. Nothing here throws, synchronises (unless stated) or owns a
 * caller tensor. Citations name the interface of B4rtekk1/CGPT that an entry
 * point stands in for (paths relative to the reference checkout).
 *
 * Scratch memory (row statistics, split-K partials, sort buffers) comes from
 * a per-(device, stream) arena that grows on the first eager call with a given
 * problem size. While a stream is being captured into a hipGraph the arena
 * cannot grow: a call that would need more scratch than an earlier eager call
 * reserved returns CGPTX_CAPTURE_ALLOC. Run each op once eagerly before
 * capture, exactly as the reference warms up before cudaStreamBeginCapture
 * (train/train.cpp:545-548).
 *
 * Threading: one host thread per stream, as in the reference.
 */
#ifndef CGPTX_H
#define CGPTX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage dtypes; numeric values follow enum class Dtype (include/core/dtype.h:12-21). */
enum { CGPTX_F16 = 0, CGPTX_BF16 = 1, CGPTX_F32 = 2 };

/* Status codes. The C++ layer maps INVALID_ARGUMENT to std::invalid_argument,
 * OVERFLOW to std::overflow_error and RUNTIME to the fatal path of
 * include/core/cuda_check.h:19-38. */
enum {
    CGPTX_OK = 0,
    CGPTX_INVALID_ARGUMENT = 1,
    CGPTX_OVERFLOW = 2,
    CGPTX_RUNTIME = 3,
    CGPTX_CAPTURE_ALLOC = 4
};

typedef void* cgptx_stream; /* hipStream_t */

/* Message of the last failing call on this host thread ("" if none). */
const char* cgptx_last_error(void);
/* Library version string. */
const char* cgptx_version(void);
/* Releases every scratch arena of the current device (synchronises the device). */
int cgptx_release_scratch(void);
/* Bytes of the scratch arena bound to (current device, stream): the largest request any operator has made on
 * that stream so far, rounded up to 1 MiB; 0 when the stream has none. For a train step it is dominated by the
 * logits chunk of the cut cross-entropy (rows x vocabulary in the storage dtype, up to 2 GiB - 1 MiB). */
size_t cgptx_scratch_bytes(cgptx_stream stream);

/* ------------------------------------------------------------------ backward */

/* rmsnorm_backward — include/ops/backward/rmsnorm_backward.h:21-29.
 * x, dy, dx: [rows, hidden]; weight, grad_weight: [hidden]; all of `dtype`.
 * dx = dy*w*r - x*(sum_j dy_j w_j x_j)*r^3/hidden, r = rsqrt(mean(x^2)+eps);
 * grad_weight_j = sum_rows dy*x*r. Both outputs are overwritten. */
int cgptx_rmsnorm_backward(void* grad_input, void* grad_weight,
                           const void* grad_output, const void* input,
                           const void* weight, size_t rows, size_t hidden,
                           float epsilon, int dtype, cgptx_stream stream);

/* rmsnorm_backward that allocates nothing. No counterpart in the reference: it is for callers that cannot
 * allocate device memory — code under hipGraph capture that has not run eagerly first, tight serving loops,
 * harnesses that forbid hipMalloc. Same arguments, kernels and results (bit for bit) as cgptx_rmsnorm_backward;
 * the partial sums of the weight gradient go to a 16 MiB block built into the library's device image (each GPU
 * the library runs on holds one until the process ends) instead of the per-stream arena. A shape that needs
 * more (4 bytes x hidden x the blocks resident on the device, at most a few thousand, for hidden sizes the row
 * kernel takes: multiples of 8 up to 2048 in 16-bit storage; else 4 bytes x rows + 1 KiB x hidden) returns
 * CGPTX_INVALID_ARGUMENT with both sizes in the message, before anything is launched. Calls no hipMalloc / hipFree. Every call on a GPU
 * shares that GPU's block: calls that overlap on one GPU (different streams or threads) race; calls on one
 * stream are ordered. */
int cgptx_rmsnorm_backward_static(void* grad_input, void* grad_weight,
                                  const void* grad_output, const void* input,
                                  const void* weight, size_t rows, size_t hidden,
                                  float epsilon, int dtype, cgptx_stream stream);

/* rope_backward — include/ops/backward/rope_backward.h:22-31.
 * q grads [batch, sequence, query_heads, head_dim], k grads [.., kv_heads, ..],
 * caches [cache_positions, rotary_dim/2]; adjacent pairs (2p, 2p+1) rotate by
 * the inverse angle; the tail past rotary_dim is copied. rotary_dim 0 = head_dim. */
int cgptx_rope_backward(void* grad_query, void* grad_key,
                        const void* grad_rotated_query,
                        const void* grad_rotated_key, const void* cos_cache,
                        const void* sin_cache, size_t batch, size_t sequence,
                        size_t query_heads, size_t kv_heads, size_t head_dim,
                        size_t rotary_dim, size_t position_offset,
                        size_t cache_positions, int dtype, cgptx_stream stream);

/* swiglu_backward (separate gate/up) — include/ops/backward/swiglu_backward.h:30-38. */
int cgptx_swiglu_backward(void* grad_gate, void* grad_up,
                          const void* grad_output, const void* gate,
                          const void* up, size_t count, int accumulate_gate,
                          int accumulate_up, int dtype, cgptx_stream stream);

/* swiglu_backward (packed [rows, 2*hidden] = [gate | up]) —
 * src/ops/backward/swiglu_backward.cu:830-883. */
int cgptx_swiglu_backward_packed(void* grad_gate_up, const void* grad_output,
                                 const void* gate_up, size_t rows,
                                 size_t hidden, int accumulate_gate_up,
                                 int dtype, cgptx_stream stream);

/* linear_backward — include/ops/backward/linear_backward.h:36-46.
 * dX[rows,in] = dY[rows,out]·W[out,in]; dW[out,in] = dYᵀ·X; db[out] = Σ_rows dY.
 * fp32 accumulation; each accumulate_* flag adds into the existing output.
 * Any of grad_input / grad_weight / grad_bias may be NULL to skip that product
 * (the reference always computes all three). */
int cgptx_linear_backward(void* grad_input, void* grad_weight, void* grad_bias,
                          const void* grad_output, const void* input,
                          const void* weight, size_t rows, size_t in_features,
                          size_t out_features, int accumulate_input,
                          int accumulate_weight, int accumulate_bias, int dtype,
                          cgptx_stream stream);

/* embedding_backward — include/ops/backward/embedding_backward.h:35-42.
 * dW[id_t,:] += dY[t,:]. Rows are summed in ascending token order with a
 * rounding to `dtype` after every add, which is the arithmetic of
 * src/ops/cpu/backward/embedding_backward_cpu.cpp:99-112, so the result is
 * deterministic. ids >= vocab are skipped (always; the reference leaves that
 * case undefined without bounds_check). */
int cgptx_embedding_backward(void* grad_weight, const void* grad_output,
                             const uint32_t* token_ids, size_t token_count,
                             size_t vocab, size_t hidden, int bounds_check,
                             int accumulate_weight, int dtype,
                             cgptx_stream stream);

/* cross_entropy_forward_backward — include/ops/cross_entropy.h:25-32.
 * loss[1] (fp32) = mean_r (logsumexp z_r − z_{r,y_r}) over rows with y_r < vocab;
 * gradient = (softmax − onehot)·gradient_scale/rows in `dtype`. */
int cgptx_cross_entropy_forward_backward(float* loss, void* gradient,
                                         const void* logits,
                                         const uint32_t* targets, size_t rows,
                                         size_t vocab, float gradient_scale,
                                         int dtype, cgptx_stream stream);

/* cross_entropy_forward — include/ops/cross_entropy.h:37-42. */
int cgptx_cross_entropy_forward(float* loss, const void* logits,
                                const uint32_t* targets, size_t rows,
                                size_t vocab, int dtype, cgptx_stream stream);

/* cut_cross_entropy_forward_backward — include/ops/cut_cross_entropy.h:25-33.
 * z = X·Cᵀ is never stored in full. The reference is F32-only with no gradient
 * scale; here any dtype is accepted, gradient_scale multiplies both gradients
 * (1.0 reproduces the reference) and accumulate_classifier adds into dC (needed
 * for tied embeddings). */
int cgptx_cut_cross_entropy_forward_backward(
    float* loss, void* input_gradient, void* classifier_gradient,
    const void* input, const void* classifier, const uint32_t* targets,
    size_t rows, size_t hidden, size_t vocab, float gradient_scale,
    int accumulate_classifier, int dtype, cgptx_stream stream);

/* flash_gqa_attention_backward_with_lse — include/ops/backward/attention_backward.h:57-70.
 * q, o, dO, dQ: [batch, query_sequence, query_heads, head_dim];
 * k, v, dK, dV: [batch, kv_sequence, kv_heads, head_dim];
 * logsumexp fp32 [batch, query_sequence, query_heads] = ln Σ exp(scale·q·k).
 * attention_scale <= 0 selects 1/sqrt(head_dim). Causal: key j visible to query
 * i iff j <= query_position_offset + i. */
int cgptx_flash_gqa_attention_backward_with_lse(
    void* grad_query, void* grad_key, void* grad_value, const void* grad_output,
    const void* output, const float* logsumexp, const void* query,
    const void* key, const void* value, size_t batch, size_t query_sequence,
    size_t kv_sequence, size_t query_heads, size_t kv_heads, size_t head_dim,
    float attention_scale, int causal, size_t query_position_offset,
    int accumulate_grads, int dtype, cgptx_stream stream);

/* flash_gqa_attention_backward — include/ops/backward/attention_backward.h:24-35.
 * Same without saved output/LSE: both are recomputed first. */
int cgptx_flash_gqa_attention_backward(
    void* grad_query, void* grad_key, void* grad_value, const void* grad_output,
    const void* query, const void* key, const void* value, size_t batch,
    size_t query_sequence, size_t kv_sequence, size_t query_heads,
    size_t kv_heads, size_t head_dim, float attention_scale, int causal,
    size_t query_position_offset, int accumulate_grads, int dtype,
    cgptx_stream stream);

/* ------------------------------------------------------------------- AdamW */

/* AdamWOptions — include/optim/adamw.h:12-27. */
typedef struct cgptx_adamw_options {
    float learning_rate;
    float beta1;
    float beta2;
    float epsilon;
    float weight_decay;
    float loss_scale;
    float max_grad_norm; /* +inf disables clipping */
} cgptx_adamw_options;

/* One parameter tensor of a batched update (AdamWBatchEntry + AdamWState,
 * include/optim/adamw.h:33-57). parameter/gradient are `dtype`; the three state
 * buffers are fp32. */
typedef struct cgptx_adamw_entry {
    void* parameter;
    const void* gradient;
    float* master_parameter;
    float* first_moment;
    float* second_moment;
    size_t count;
    int dtype;
} cgptx_adamw_entry;

typedef struct cgptx_adamw_workspace cgptx_adamw_workspace; /* AdamWWorkspace, adamw.h:60-84 */

int cgptx_adamw_workspace_create(cgptx_adamw_workspace** workspace);
int cgptx_adamw_workspace_destroy(cgptx_adamw_workspace* workspace);

/* adamw_step_many_async — include/optim/adamw.h:103-107 → src/optim/adamw.cu:276-346.
 * One global-norm AdamW update over all entries, fully on the device: gradient
 * statistics, non-finite check (skip everything, latch a sticky flag, do not
 * advance the step), bias correction, clipping, update. The first call binds the
 * workspace to this entry list and uploads initial_step; later calls must pass
 * the same list. Never synchronises. */
int cgptx_adamw_step_many_async(cgptx_adamw_workspace* workspace,
                                const cgptx_adamw_entry* entries,
                                size_t entry_count,
                                const cgptx_adamw_options* options,
                                uint64_t initial_step, cgptx_stream stream);

/* adamw_check — include/optim/adamw.h:114-115 → adamw.cu:348-359. Synchronises
 * the stream; *all_finite = 0 if any step since the last check saw NaN/Inf;
 * *step = device step counter; clears the sticky flag. */
int cgptx_adamw_check(cgptx_adamw_workspace* workspace, int* all_finite,
                      uint64_t* step, cgptx_stream stream);

/* adamw_step (single tensor, host-synchronous) — include/optim/adamw.h:131-136 →
 * adamw.cu:396-435. bias corrections come from the host in double as there;
 * *updated = 0 if the gradient held NaN/Inf (nothing is changed then). */
int cgptx_adamw_step(void* parameter, const void* gradient,
                     float* master_parameter, float* first_moment,
                     float* second_moment, size_t count, int dtype,
                     const cgptx_adamw_options* options, uint64_t next_step,
                     int* updated, cgptx_stream stream);

/* ------------------------------------------------------------------ forward */

/* rmsnorm_forward — include/ops/rmsnorm.h. y = x·rsqrt(mean x²+eps)·w. */
int cgptx_rmsnorm_forward(void* output, const void* input, const void* weight,
                          size_t rows, size_t hidden, float epsilon, int dtype,
                          cgptx_stream stream);

/* rope_forward (in place on q and k) — include/ops/rope.h:32-39. */
int cgptx_rope_forward(void* query, void* key, const void* cos_cache,
                       const void* sin_cache, size_t batch, size_t sequence,
                       size_t query_heads, size_t kv_heads, size_t head_dim,
                       size_t rotary_dim, size_t position_offset,
                       size_t cache_positions, int dtype, cgptx_stream stream);

/* swiglu_forward — include/ops/swiglu.h. out = silu(gate)·up. */
int cgptx_swiglu_forward(void* output, const void* gate, const void* up,
                         size_t count, int dtype, cgptx_stream stream);

/* swiglu_forward (packed input [rows, 2*hidden] = [gate | up]) — include/ops/swiglu.h:33-37,
 * src/ops/swiglu.cu:152-170. output is [rows, hidden]. */
int cgptx_swiglu_forward_packed(void* output, const void* gate_up, size_t rows,
                                size_t hidden, int dtype, cgptx_stream stream);

/* linear_forward — include/ops/linear.h. Y[rows,out] = X[rows,in]·W[out,in]ᵀ (+ bias[out]).
 * bias may be NULL. */
int cgptx_linear_forward(void* output, const void* input, const void* weight,
                         const void* bias, size_t rows, size_t in_features,
                         size_t out_features, int dtype, cgptx_stream stream);

/* The feed-forward's gate and up projections and its SwiGLU in one call — the sequence
 * linear_forward(gate), linear_forward(up), swiglu_forward(activated, gate, up) of
 * src/core/transformer_block.cu:586-590 with the concatenated layouts of include/ops/swiglu.h:33-37:
 * weight = [gate_proj; up_proj] ([2*hidden, in]), gate_up = [rows, 2*hidden] = [gate | up] (kept for the
 * backward pass), activated[rows, hidden] = silu(gate)·up from the rounded gate and up values. Large
 * aligned shapes run as one contraction whose epilogue writes all three; the rest as the two operators. */
int cgptx_linear_swiglu_forward(void* gate_up, void* activated, const void* input,
                                const void* weight, size_t rows, size_t in_features,
                                size_t hidden, int dtype, cgptx_stream stream);

/* The input gradient of the feed-forward's down projection and the SwiGLU gradient in one call — the
 * sequence linear_backward(down) (input gradient only), swiglu_backward of
 * src/core/transformer_block.cu:663-666 with the concatenated layouts of
 * src/ops/backward/swiglu_backward.cu:830-883: weight = down_proj ([out, hidden]), gate_up = the forward's
 * [rows, 2*hidden] = [gate | up], grad_gate_up = [rows, 2*hidden] = [dgate | dup], computed from
 * grad_output·weight rounded to the storage dtype. grad_activated ([rows, hidden]) is working memory: the
 * two-operator path writes the intermediate gradient there, the fused contraction (large aligned shapes)
 * leaves it untouched. */
int cgptx_linear_swiglu_backward(void* grad_gate_up, void* grad_activated, const void* grad_output,
                                 const void* weight, const void* gate_up, size_t rows,
                                 size_t hidden, size_t out_features, int dtype, cgptx_stream stream);

/* The weight gradients of `count` layers of one shape in one launch — `count` calls of linear_backward
 * (include/ops/backward/linear_backward.h:36-46) that ask for the weight gradient only, as
 * src/core/transformer_block.cu:660-745 makes them for every block of a model: layer j reads grad_output +
 * j * grad_output_stride ([rows, out_features]) and input + j * input_stride ([rows, in_features]), strides in
 * elements, and writes rows j * out_features .. of grad_weight ([count * out_features, in_features]). One launch
 * over all layers' tiles fills the chip without splitting the row sum of each product into partial tiles; shapes it
 * does not take (fp32 storage, out_features not a multiple of 256, unaligned tensors) run as `count` separate
 * weight gradients. */
int cgptx_linear_backward_weights_stacked(void* grad_weight, const void* grad_output, const void* input,
                                          size_t rows, size_t in_features, size_t out_features, size_t count,
                                          size_t grad_output_stride, size_t input_stride, int dtype,
                                          cgptx_stream stream);

/* embedding_forward — include/ops/embedding.h. out[t,:] = W[id_t,:]; ids >= vocab give a zero row. */
int cgptx_embedding_forward(void* output, const uint32_t* token_ids,
                            size_t token_count, const void* weight,
                            size_t vocab, size_t hidden, int dtype,
                            cgptx_stream stream);

/* flash_gqa_attention_forward_with_lse — include/ops/attention.h:70-78.
 * logsumexp may be NULL (flash_gqa_attention_forward, attention.h:47-54). */
int cgptx_flash_gqa_attention_forward(
    void* output, float* logsumexp, const void* query, const void* key,
    const void* value, size_t batch, size_t query_sequence, size_t kv_sequence,
    size_t query_heads, size_t kv_heads, size_t head_dim, float attention_scale,
    int causal, size_t query_position_offset, int dtype, cgptx_stream stream);

/* Residual helpers used by the block (src/core/transformer_block.cu:134-144, 242-248):
 * out = a + b, and out += b, elementwise over `count` values. */
int cgptx_add(void* output, const void* a, const void* b, size_t count,
              int dtype, cgptx_stream stream);

#ifdef __cplusplus
}
#endif
#endif /* CGPTX_H */
