/*
 * cgptx_train.h — C-ABI of the caller side of the hot path: one decoder model
 * (weights, gradients, AdamW state, activations) and its train step, composed
 * from the operators of cgptx.h in the order the reference composes them:
 *   forward   src/core/transformer_model.cu:195-241, src/core/transformer_block.cu:405-611
 *   backward  src/core/transformer_model.cu:336-381, src/core/transformer_block.cu:644-748
 *   step      train/train.cpp:536-556 (forward + loss + backward replayed from one
 *             captured graph; here the AdamW update is recorded with them)
 * The block is the reference's parallel-residual block with per-head QK-norm:
 *   out = x + Wo·Attn(rope(norm_q(Wq·n_a)), rope(norm_k(Wk·n_a)), Wv·n_a) + Wd·swiglu(Wg·n_f, Wu·n_f),
 *   n_a = RMSNorm_a(x), n_f = RMSNorm_f(x); embeddings are tied to the classifier.
 */
#ifndef CGPTX_TRAIN_H
#define CGPTX_TRAIN_H

#include "cgptx.h"

#ifdef __cplusplus
extern "C" {
#endif

/* TransformerModelOptions + TransformerBlockOptions (include/core/transformer_model.h,
 * include/core/transformer_block.h); the 104m preset is train/train.cpp:146-148. */
typedef struct cgptx_model_config {
    size_t vocabulary_size;
    size_t num_layers;
    size_t hidden_size;
    size_t intermediate_size;
    size_t num_query_heads;
    size_t num_kv_heads;
    size_t head_dim;
    size_t rotary_dim;
    float rms_epsilon;
    float rope_base;   /* 10000 in train/train.cpp:326 */
    int dtype;         /* storage dtype of weights, activations and gradients */
} cgptx_model_config;

enum { CGPTX_LOSS_DENSE = 0, CGPTX_LOSS_CUT = 1 };

typedef struct cgptx_model cgptx_model;

/* Allocates everything for a fixed [batch, sequence] step and initialises the weights from
 * `seed` with a counter-based generator: N(0, 0.02), o/down projections N(0, 0.02/sqrt(2L)),
 * norm weights 1 (the distribution of src/core/weight_initialization.cu:158-179). */
int cgptx_model_create(cgptx_model** model, const cgptx_model_config* config, size_t batch, size_t sequence,
                       uint64_t seed);
int cgptx_model_destroy(cgptx_model* model);

/* Copies `batch*sequence` input and target ids from host memory into the model's graph-stable
 * device buffers (data::upload_batch, src/data/dataset_loader.cpp:145-166). Synchronous. */
int cgptx_model_set_tokens(cgptx_model* model, const uint32_t* inputs, const uint32_t* targets);

/* data::Batch x 2 + data::upload_batch (include/data/dataset_loader.h:111-170 →
 * src/data/dataset_loader.cpp:120-166; train/train.cpp:463-465, 570-574): two page-locked host
 * slots for [batch, sequence] input and target ids, each with the event that says when the copies
 * out of it have finished. acquire hands out the slot to fill next and first waits until its last
 * upload has completed (Batch::wait_until_reusable); submit enqueues the two asynchronous copies
 * to the device buffers on `stream`, records the slot's event (Batch::mark_upload_complete) and
 * switches to the other slot. Nothing but acquire ever blocks the host. */
typedef struct cgptx_token_upload cgptx_token_upload;
int cgptx_token_upload_create(cgptx_token_upload** upload, size_t batch, size_t sequence);
int cgptx_token_upload_destroy(cgptx_token_upload* upload);
int cgptx_token_upload_acquire(cgptx_token_upload* upload, uint32_t** inputs, uint32_t** targets);
int cgptx_token_upload_submit(cgptx_token_upload* upload, uint32_t* device_inputs, uint32_t* device_targets,
                              cgptx_stream stream);
/* submit into the model's own token buffers, whose addresses a captured step keeps reading
 * (train/train.cpp:551-553 checks exactly that they never change). INVALID_ARGUMENT when the
 * upload's shape is not the model's ("Batch buffers do not match its declared shape"). */
int cgptx_model_upload_tokens(cgptx_model* model, cgptx_token_upload* upload, cgptx_stream stream);

/* The same upload for callers that own their batches (data::Batch / data::DeviceBatch,
 * include/data/dataset_loader.h:111-170): page-locked host blocks for the token vectors
 * (CudaHostAllocator::allocate / deallocate, include/data/dataset_loader.h:57-84; a request for 0 bytes
 * gives a valid block), device blocks for the destination (DeviceBuffer::allocate / release,
 * include/core/device_buffer.h:59-81), and the per-batch fence that says when the copies out of a host
 * batch have finished (Batch::upload_complete_: mark_upload_complete / wait_until_reusable,
 * src/data/dataset_loader.cpp:120-131). */
int cgptx_pinned_allocate(void** block, size_t bytes);
int cgptx_pinned_release(void* block);
int cgptx_device_allocate(void** block, size_t bytes);
int cgptx_device_release(void* block);
typedef struct cgptx_upload_fence cgptx_upload_fence;
/* Blocks the host until the copies recorded last on `fence` are done; a null fence has none. */
int cgptx_upload_fence_wait(cgptx_upload_fence* fence);
/* Does not wait; null is accepted. */
int cgptx_upload_fence_destroy(cgptx_upload_fence* fence);
/* data::upload_batch (src/data/dataset_loader.cpp:145-166) after its shape check: enqueues the copies of
 * `count` input and `count` target ids from page-locked host memory to the device buffers on `stream`
 * and records *fence behind them, creating the fence on first use. count == 0 only records. */
int cgptx_token_upload_async(uint32_t* device_inputs, uint32_t* device_targets, const uint32_t* inputs,
                             const uint32_t* targets, size_t count, cgptx_upload_fence** fence,
                             cgptx_stream stream);

/* Enqueues forward + loss + backward on `stream` (gradient of loss·loss_scale). With use_graph
 * the sequence is captured on first use (after one eager run) and replayed afterwards. */
int cgptx_model_forward_backward(cgptx_model* model, float loss_scale, int loss_mode, int use_graph,
                                 cgptx_stream stream);

/* Enqueues the global-norm AdamW update over all parameters (adamw_step_many_async). */
int cgptx_model_optimizer_step(cgptx_model* model, const cgptx_adamw_options* options, cgptx_stream stream);

/* forward_backward followed by optimizer_step (train/train.cpp:536-556). With use_graph the three launches of
 * the AdamW update are part of the recorded step: the options, which change from step to step (the learning rate),
 * are written to the device by one small launch ahead of the graph, and the update's kernels read them there — same
 * results as the eager step, bit for bit, including skipped (non-finite) steps. */
int cgptx_model_train_step(cgptx_model* model, const cgptx_adamw_options* options, int loss_mode, int use_graph,
                           cgptx_stream stream);

/* Synchronises `stream`; returns the last loss, whether all optimizer steps since the previous
 * call saw finite gradients, and the optimizer step count (adamw_check). */
int cgptx_model_status(cgptx_model* model, float* loss, int* all_finite, uint64_t* step, cgptx_stream stream);

/* Runs one eager forward + loss + backward with HIP events around every operator call on
 * `stream` and keeps the time per operator kind ("gemm_fwd", "gemm_dx", "gemm_dw", "attn_fwd",
 * "attn_bwd", "rmsnorm_bwd", ...), summed over the calls of that kind. Synchronises. */
int cgptx_model_profile(cgptx_model* model, float loss_scale, int loss_mode, cgptx_stream stream);
size_t cgptx_model_profile_count(const cgptx_model* model);
int cgptx_model_profile_entry(const cgptx_model* model, size_t index, const char** label, float* milliseconds);

/* The operator calls of the step when it runs as the reference's own call sequence (environment
 * CGPTX_FUSE=0: one public operator per call, forward in the order of src/core/transformer_block.cu:466-595,
 * backward in the order of :663-747 and src/core/transformer_model.cu:360-380). While recording is on, every
 * such step leaves the table of its calls: `op` is the operator's name in the headers under include/ops ("add" is the block's
 * residual helper, src/core/transformer_block.cu:134-144), `tensors` its device tensors in the operator's
 * argument order (outputs first; token ids and targets in their argument position), `dims` and `flags` its
 * sizes and accumulate / causal / bounds-check switches in the order of the operator's C-ABI entry point,
 * `scalar` its epsilon, attention scale or gradient scale. A caller written against those headers that walks
 * the table reproduces the step's results bit for bit. */
typedef struct cgptx_call_record {
    const char* op;
    const void* tensors[10];
    size_t dims[8];
    int flags[4];
    float scalar;
    int dtype;
} cgptx_call_record;
int cgptx_model_record_calls(cgptx_model* model, int enable);
size_t cgptx_model_call_count(const cgptx_model* model);
int cgptx_model_call(const cgptx_model* model, size_t index, cgptx_call_record* record);

/* Number of parameter tensors and, per index, name / device pointers / element count. Names follow
 * the checkpoint names of src/core/huggingface_export.cpp:362-378 where one exists. */
size_t cgptx_model_parameter_count(const cgptx_model* model);
int cgptx_model_parameter(const cgptx_model* model, size_t index, const char** name, void** parameter,
                          void** gradient, size_t* count);
/* Total number of parameters (tied embedding counted once). */
size_t cgptx_model_num_parameters(const cgptx_model* model);

/* The configuration and step shape the model was created with. */
int cgptx_model_describe(const cgptx_model* model, cgptx_model_config* config, size_t* batch, size_t* sequence);
/* Device pointers to the AdamW state of parameter `index`: fp32 master copy, first and second moment
 * (AdamWState, include/optim/adamw.h:45-58). */
int cgptx_model_optimizer_state(const cgptx_model* model, size_t index, float** master, float** first_moment,
                                float** second_moment);
/* Makes the optimizer continue from `step` completed steps (bias correction uses step + 1 next).
 * Synchronises the device. */
int cgptx_model_set_optimizer_step(cgptx_model* model, uint64_t step);

/* export_huggingface_model without the tokenizer files (include/core/huggingface_export.h →
 * src/core/huggingface_export.cpp:135-158, 180-225, 345-380): writes `config.json` (same keys) and
 * `model.safetensors` (same tensor names, order and layout; the tied classifier is written as
 * `lm_head.weight` too) into an existing directory. Synchronises the device. */
int cgptx_model_save_checkpoint(const cgptx_model* model, const char* directory, size_t max_position_embeddings);
/* load_huggingface_model (src/core/huggingface_export.cpp:400-430): reads `model.safetensors` from
 * `directory` into the model's weights; every tensor of the list must be present with the model's
 * dtype, shape and byte size (RUNTIME status otherwise, nothing is loaded partially into a tensor).
 * The fp32 master copies restart from the loaded values; moments and step are left alone. */
int cgptx_model_load_checkpoint(cgptx_model* model, const char* directory);
/* Optimizer state, which the reference does not save: `<name>.master`, `.exp_avg`, `.exp_avg_sq`
 * (fp32) and the step counter `step` (U64) in one safetensors file. `step` is the count
 * cgptx_model_status last reported. Loading also restores the step counter. */
int cgptx_model_save_optimizer(const cgptx_model* model, const char* path, uint64_t step);
int cgptx_model_load_optimizer(cgptx_model* model, const char* path, uint64_t* step);

/* Device pointer to a named tensor of the last step, for tests and for callers that run their own block code
 * on the saved state: "hidden.<l>" (input of block l; l = num_layers: the last block's output), "normalized",
 * "loss", "logits" (dense loss only), "rope.cos" / "rope.sin" ([sequence, rotary_dim/2]),
 * "layer.<l>.<name>" with name one of attention_norm_output, query_pre_norm, key_pre_norm, query, key, value,
 * attention_output, logsumexp (fp32), ffn_norm_output, gate_up ([rows, 2I] = [gate | up]; with CGPTX_FUSE=0 its two
 * halves are the separate [rows, I] gate and up tensors), activated; "grad.hidden.0" / "grad.hidden.1" (the
 * residual-stream gradients the first block's backward read and wrote). *count is in elements. Returns
 * INVALID_ARGUMENT for unknown names.
 *
 * Environment switches read at every enqueue (a recorded graph keeps what it was recorded with):
 * CGPTX_FUSE=0 runs the step as the reference's own call sequence, one public operator per call
 * (src/core/transformer_block.cu:466-595, 663-747); CGPTX_FUSE_QK=0, CGPTX_FUSE_NORMS=0, CGPTX_FUSE_SWIGLU=0 and
 * CGPTX_FUSE_DGAMMA=0 (the norm weight-gradient reductions after each pass instead of once per step) switch single
 * fusions of the default step off. */
int cgptx_model_activation(const cgptx_model* model, const char* name, void** data, size_t* count);

#ifdef __cplusplus
}
#endif
#endif /* CGPTX_TRAIN_H */
