// The caller side of the hot path: a decoder model and its train step composed
// from the cgptx_* operators, in the order of the reference's
// transformer_model_forward/backward (src/core/transformer_model.cu:195-241, 336-381),
// transformer_block_forward/backward (src/core/transformer_block.cu:405-611, 644-748)
// and the training loop (train/train.cpp:536-556).
//
// Differences from the reference's glue, none of which changes a result:
//   * no device-to-device copies: projections write straight into the buffers that
//     the backward pass reads (q/k before QK-norm, the layer inputs), and the output
//     projection's backward reads the incoming gradient in place;
//   * the attention-norm output is kept instead of being recomputed in the backward;
//   * bias gradients, which the reference computes into scratch and never uses
//     (the model has no biases), are not computed;
//   * forward + loss + backward, and in a train step the AdamW update behind them, are captured into
//     one hipGraph after one eager run; every scratch request was sized by that eager run, so replay
//     allocates nothing. The optimizer's options reach its kernels through device memory, written
//     ahead of each replay.
#include "cgptx_train.h"
#include "common.hpp"
#include "gemm.hpp"

#include <charconv>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

namespace cgptx {
namespace {

// ---- deterministic host-side initialisation ----------------------------------
inline std::uint64_t splitmix64(std::uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// Standard normal from (seed, tensor, index): Box–Muller on two counter-derived uniforms.
inline float normal_at(std::uint64_t seed, std::uint64_t tensor, std::uint64_t index) {
    const std::uint64_t a = splitmix64(seed ^ splitmix64(tensor * 0x100000001B3ull + 2 * index));
    const std::uint64_t b = splitmix64(seed ^ splitmix64(tensor * 0x100000001B3ull + 2 * index + 1));
    const double u1 = (static_cast<double>(a >> 11) + 1.0) / 9007199254740993.0;  // (0, 1)
    const double u2 = static_cast<double>(b >> 11) / 9007199254740992.0;          // [0, 1)
    return static_cast<float>(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
}

inline std::uint16_t to_bf16_bits(float x) {
    std::uint32_t b;
    std::memcpy(&b, &x, 4);
    return static_cast<std::uint16_t>((b + 0x7fffu + ((b >> 16) & 1u)) >> 16);
}

inline std::uint16_t to_f16_bits(float x) {
    const _Float16 h = static_cast<_Float16>(x);
    std::uint16_t bits;
    std::memcpy(&bits, &h, 2);
    return bits;
}

void convert_to_storage(const std::vector<float>& src, int dtype, std::vector<unsigned char>& dst) {
    if (dtype == CGPTX_F32) {
        dst.resize(src.size() * 4);
        std::memcpy(dst.data(), src.data(), dst.size());
        return;
    }
    dst.resize(src.size() * 2);
    auto* out = reinterpret_cast<std::uint16_t*>(dst.data());
    for (std::size_t i = 0; i < src.size(); ++i) out[i] = dtype == CGPTX_BF16 ? to_bf16_bits(src[i]) : to_f16_bits(src[i]);
}

struct Parameter {
    std::string name;
    void* value = nullptr;
    void* gradient = nullptr;
    float* master = nullptr;
    float* first = nullptr;
    float* second = nullptr;
    std::size_t count = 0;
};

struct LayerParameters {
    Parameter attention_norm, q, k, q_norm, k_norm, v, o, ffn_norm, gate, up, down;
};

struct LayerActivations {
    void *norm_a, *q_pre, *k_pre, *q, *k, *v, *attn_out, *norm_f, *gate_up, *act;  // gate_up: [rows, 2I] = [gate | up]
    float* lse;
};

}  // namespace
}  // namespace cgptx

struct cgptx_model {
    cgptx_model_config config{};
    std::size_t batch = 0, sequence = 0, rows = 0;
    std::vector<void*> allocations;
    cgptx::Parameter embedding, final_norm;
    std::vector<cgptx::LayerParameters> layers;
    std::vector<cgptx::LayerActivations> acts;
    std::vector<void*> hidden;  // num_layers + 1 buffers [rows, hidden]
    void* normalized = nullptr;
    void* logits = nullptr;       // dense loss only, allocated on first use
    void* grad_logits = nullptr;
    void *cos_cache = nullptr, *sin_cache = nullptr;
    std::uint32_t *tokens = nullptr, *targets = nullptr;
    float* loss = nullptr;
    // backward workspace
    void *d_normalized = nullptr, *grad_a = nullptr, *grad_b = nullptr, *d_act = nullptr, *d_gate_up = nullptr,
         *d_norm_in = nullptr, *d_norm_in_f = nullptr, *d_attn_out = nullptr, *d_q = nullptr,
         *d_k = nullptr, *d_v = nullptr, *d_q_pre = nullptr, *d_k_pre = nullptr;
    // Weight gradients of the projections for all layers at once, at the end of the backward pass (stacked_dw): what
    // those four launches read and write lies layer after layer in one block per tensor kind, and the backward pass
    // keeps every layer's output gradients instead of reusing one set of buffers.
    struct Stack {
        char* base = nullptr;
        std::size_t stride = 0;  // bytes from one layer to the next
        void* at(std::size_t layer) const { return base + layer * stride; }
    };
    bool stacked_dw = false;
    // The q and the output projection have one shape ([hidden, hidden], since hidden = query heads x head_dim), and so
    // have their inputs and output gradients: both projections of all layers form one stack of 2 x layers products —
    // slot l belongs to layer l's q projection, slot layers + l to its output projection.
    Stack q_o_gradients, kv_gradients, gate_up_gradients, down_gradients;  // [slots][out, in], no gaps
    Stack q_o_inputs;    // slot l: attention norm output, slot layers + l: attention output
    Stack norm_f_all, act_all;
    // slot l: dq of layer l; slot layers + l: the residual stream's gradient at layer l's output (slot 2 x layers: at
    // the first layer's input, read by the embedding's gradient)
    Stack q_o_output_gradients;
    Stack d_gate_up_all, d_k_all, d_v_all;
    std::size_t stacked_layers = 0;
    void* d_hidden_slot(std::size_t index) const {  // gradient of hidden[index]
        return index == 0 ? q_o_output_gradients.at(2 * stacked_layers) : q_o_output_gradients.at(stacked_layers + index - 1);
    }
    cgptx_adamw_workspace* optimizer = nullptr;
    std::uint64_t initial_step = 0;  // step count the optimizer workspace starts from when it is first used
    std::vector<cgptx_adamw_entry> entries;
    // captured graph
    // Recorded steps: [0] forward + loss + backward, [1] the same followed by the AdamW update.
    struct RecordedStep {
        hipGraphExec_t exec = nullptr;
        float loss_scale = 0.0f;
        int loss_mode = -1;
        hipStream_t stream = nullptr;
        std::uint64_t scratch_generation = 0;  // scratch arena block the recorded kernels point into
    };
    RecordedStep recorded[2];
    // weight-gradient reductions of the norm-backward passes, run as one pair of launches per step
    cgptx::ColumnReduceSink norm_reductions;
    cgptx::ColumnReduceEntry* norm_reduction_table = nullptr;       // device copy of the entries
    std::vector<cgptx::ColumnReduceEntry> norm_reduction_uploaded;  // what the device copy holds
    std::size_t norm_reduction_table_capacity = 0;                  // entries
    bool norm_reductions_resized = false;                           // the last pass grew the sink's memory
    // optional per-operator timing of one eager pass
    struct Timed {
        const char* label;
        hipEvent_t start, stop;
    };
    bool profiling = false;
    std::vector<Timed> timed;
    // optional table of the operator calls the reference call sequence makes (cgptx_model_record_calls)
    bool recording_calls = false;
    std::vector<cgptx_call_record> calls;
    std::vector<std::pair<std::string, float>> profile;  // label, milliseconds (summed per label)
};

namespace cgptx {
namespace {

int allocate(cgptx_model* m, void** out, std::size_t bytes) {
    CGPTX_HIP(hipMalloc(out, bytes));
    m->allocations.push_back(*out);
    return CGPTX_OK;
}

template <typename P>
int allocate_typed(cgptx_model* m, P** out, std::size_t bytes) {
    void* p = nullptr;
    if (int s = allocate(m, &p, bytes)) return s;
    *out = static_cast<P*>(p);
    return CGPTX_OK;
}

// kind: 0 = normal(0, stddev), 1 = ones
// value_slot / gradient_slot: storage inside a larger block (weights that one contraction reads as a
// single matrix), or null for an allocation of the parameter's own.
int make_parameter(cgptx_model* m, Parameter& p, const std::string& name, std::size_t count, int kind, float stddev,
                   std::uint64_t seed, std::uint64_t tensor_id, void* value_slot = nullptr,
                   void* gradient_slot = nullptr) {
    const std::size_t elem = dtype_size(m->config.dtype);
    p.name = name;
    p.count = count;
    p.value = value_slot;
    p.gradient = gradient_slot;
    if (p.value == nullptr) {
        if (int s = allocate(m, &p.value, count * elem)) return s;
    }
    if (p.gradient == nullptr) {
        if (int s = allocate(m, &p.gradient, count * elem)) return s;
    }
    if (int s = allocate_typed(m, &p.master, count * sizeof(float))) return s;
    if (int s = allocate_typed(m, &p.first, count * sizeof(float))) return s;
    if (int s = allocate_typed(m, &p.second, count * sizeof(float))) return s;
    std::vector<float> host(count);
    if (kind == 1) {
        for (auto& v : host) v = 1.0f;
    } else {
        for (std::size_t i = 0; i < count; ++i) host[i] = stddev * normal_at(seed, tensor_id, i);
    }
    std::vector<unsigned char> storage;
    convert_to_storage(host, m->config.dtype, storage);
    CGPTX_HIP(hipMemcpy(p.value, storage.data(), storage.size(), hipMemcpyHostToDevice));
    // The master copy is the stored (rounded) parameter widened to fp32, as AdamWState::for_parameter does.
    if (m->config.dtype != CGPTX_F32) {
        const auto* bits = reinterpret_cast<const std::uint16_t*>(storage.data());
        for (std::size_t i = 0; i < count; ++i) {
            if (m->config.dtype == CGPTX_BF16) {
                const std::uint32_t b = static_cast<std::uint32_t>(bits[i]) << 16;
                std::memcpy(&host[i], &b, 4);
            } else {
                _Float16 h;
                std::memcpy(&h, &bits[i], 2);
                host[i] = static_cast<float>(h);
            }
        }
    }
    CGPTX_HIP(hipMemcpy(p.master, host.data(), count * sizeof(float), hipMemcpyHostToDevice));
    CGPTX_HIP(hipMemset(p.first, 0, count * sizeof(float)));
    CGPTX_HIP(hipMemset(p.second, 0, count * sizeof(float)));
    CGPTX_HIP(hipMemset(p.gradient, 0, count * elem));
    return CGPTX_OK;
}

void collect(cgptx_model* m, std::vector<Parameter*>& out) {
    out.clear();
    out.push_back(&m->embedding);
    out.push_back(&m->final_norm);
    for (auto& l : m->layers) {
        for (Parameter* p : {&l.attention_norm, &l.q, &l.k, &l.q_norm, &l.k_norm, &l.v, &l.o, &l.ffn_norm, &l.gate,
                             &l.up, &l.down})
            out.push_back(p);
    }
}

#define CGPTX_TRY(expr)                     \
    do {                                    \
        if (int status_ = (expr)) return status_; \
    } while (0)

// Runs one operator call; when profiling, brackets it with events on the same stream. Labels are "kind" or
// "kind.part" (the contractions carry the projection they belong to: qkv, o, gate_up, down, classifier).
#define CGPTX_OP(label, expr)                                                   \
    do {                                                                        \
        cgptx_model::Timed t_{label, nullptr, nullptr};                         \
        if (m->profiling) {                                                     \
            CGPTX_HIP(hipEventCreate(&t_.start));                               \
            CGPTX_HIP(hipEventCreate(&t_.stop));                                \
            CGPTX_HIP(hipEventRecord(t_.start, stream));                        \
        }                                                                       \
        if (int status_ = (expr)) return status_;                               \
        if (m->profiling) {                                                     \
            CGPTX_HIP(hipEventRecord(t_.stop, stream));                         \
            m->timed.push_back(t_);                                             \
        }                                                                       \
    } while (0)

// linear_backward as two single-kernel calls so that each can be timed on its own.
int linear_backward_split(cgptx_model* m, void* dx, void* dw, const void* dy, const void* x, const void* w,
                          std::size_t rows, std::size_t in_features, std::size_t out_features, int accumulate_input,
                          int dt, hipStream_t stream, const char* dx_label, const char* dw_label) {
    auto* s = static_cast<cgptx_stream>(stream);
    CGPTX_OP(dx_label, cgptx_linear_backward(dx, nullptr, nullptr, dy, x, w, rows, in_features, out_features,
                                              accumulate_input, 0, 0, dt, s));
    CGPTX_OP(dw_label, cgptx_linear_backward(nullptr, dw, nullptr, dy, x, w, rows, in_features, out_features, 0, 0,
                                              0, dt, s));
    return CGPTX_OK;
}

// Y = X·Wᵀ + residual (accumulate: + Y): the block's residual additions ride in the projection's
// epilogue (fp32, one rounding) instead of taking two more passes over the hidden state.
int linear_forward_residual(void* out, const void* in, const void* w, const void* residual, bool accumulate,
                            std::size_t rows, std::size_t in_features, std::size_t out_features, int dt,
                            hipStream_t stream) {
    GemmArgs g;
    g.a = in;
    g.b = w;
    g.c = out;
    g.residual = residual;
    g.m = rows;
    g.n = out_features;
    g.k = in_features;
    g.lda = in_features;
    g.ldb = in_features;
    g.ldc = out_features;
    g.ldr = out_features;
    g.accumulate = accumulate;
    g.dtype = dt;
    return gemm(g, stream);
}

// The three buffers [rows, QW], [rows, KW], [rows, KW] as column segments of one [rows, QW + 2 KW] matrix.
GemmSegments qkv_segments(const void* q, const void* k, const void* v, std::size_t QW, std::size_t KW) {
    GemmSegments seg;
    seg.count = 3;
    seg.ptr[0] = q;
    seg.ptr[1] = k;
    seg.ptr[2] = v;
    seg.ld[0] = seg.cols[0] = QW;
    seg.ld[1] = seg.cols[1] = KW;
    seg.ld[2] = seg.cols[2] = KW;
    return seg;
}

// [q | k | v] = X·[Wq; Wk; Wv]ᵀ in one launch; qkv_weight is the shared [QW + 2 KW, H] block.
int qkv_forward(void* q, void* k, void* v, const void* x, const void* qkv_weight, std::size_t rows, std::size_t H,
                std::size_t QW, std::size_t KW, int dt, hipStream_t stream) {
    GemmArgs g;
    g.a = x;
    g.b = qkv_weight;
    g.c_segments = qkv_segments(q, k, v, QW, KW);
    g.m = rows;
    g.n = QW + 2 * KW;
    g.k = H;
    g.lda = H;
    g.ldb = H;
    g.dtype = dt;
    return gemm(g, stream);
}

// dX = [dq | dk | dv]·[Wq; Wk; Wv] in one launch.
int qkv_backward_input(void* dx, const void* dq, const void* dk, const void* dv, const void* qkv_weight,
                       std::size_t rows, std::size_t H, std::size_t QW, std::size_t KW, int dt, hipStream_t stream) {
    GemmArgs g;
    g.a_segments = qkv_segments(dq, dk, dv, QW, KW);
    g.b = qkv_weight;
    g.c = dx;
    g.m = rows;
    g.n = H;
    g.k = QW + 2 * KW;
    g.ldb = H;
    g.ldc = H;
    g.b_k_contiguous = false;
    g.dtype = dt;
    return gemm(g, stream);
}

// [dWq; dWk; dWv] = [dq | dk | dv]ᵀ·X in one launch.
int qkv_backward_weight(void* qkv_gradient, const void* dq, const void* dk, const void* dv, const void* x,
                        std::size_t rows, std::size_t H, std::size_t QW, std::size_t KW, int dt, hipStream_t stream) {
    GemmArgs g;
    g.a_segments = qkv_segments(dq, dk, dv, QW, KW);
    g.b = x;
    g.c = qkv_gradient;
    g.m = QW + 2 * KW;
    g.n = H;
    g.k = rows;
    g.ldb = H;
    g.ldc = H;
    g.a_k_contiguous = false;
    g.b_k_contiguous = false;
    g.dtype = dt;
    return gemm(g, stream);
}

// Whether the projections' weight gradients of all layers run as four launches at the end of the backward pass
// instead of four per layer (CGPTX_STACK_DW=0 keeps them per layer, for comparisons). One layer's weight
// gradients have far fewer tiles than the chip has compute units, so each of them splits its sum over the rows into
// partial tiles that a second launch adds up; the layers' tiles together fill the chip several times over and
// (almost) nothing is split. Needs 16-bit storage, tile-aligned weight shapes and at least two layers; costs the
// memory of every layer's output gradients.
bool stackable_weight_gradients(const cgptx_model_config& c, std::size_t rows) {
    const char* text = std::getenv("CGPTX_STACK_DW");  // read when the model is created
    if (text != nullptr && text[0] == '0') return false;
    const std::size_t H = c.hidden_size, I = c.intermediate_size;
    const std::size_t QW = c.num_query_heads * c.head_dim, KW = c.num_kv_heads * c.head_dim;
    return c.dtype != CGPTX_F32 && c.num_layers >= 2 && rows % 32 == 0 && H % 256 == 0 && QW % 256 == 0 && KW % 256 == 0 &&
           (2 * I) % 256 == 0 && I % 8 == 0;
}

// Rows j out .. of grad_weights = dY_jᵀ·X_j for every layer j: see cgptx_linear_backward_weights_stacked.
int stacked_weight_gradients(const cgptx_model::Stack& grad_weights, const void* dy, std::size_t dy_stride_bytes,
                             const cgptx_model::Stack& x, std::size_t rows, std::size_t in_features, std::size_t out_features,
                             std::size_t layers, int dt, hipStream_t stream) {
    const std::size_t elem = dtype_size(dt);
    return cgptx_linear_backward_weights_stacked(grad_weights.base, dy, x.base, rows, in_features, out_features, layers,
                                                 dy_stride_bytes / elem, x.stride / elem, dt, static_cast<cgptx_stream>(stream));
}

// [dWk; dWv] = [dk | dv]ᵀ·X for every layer in one launch (dk and dv lie in separate buffers).
int stacked_kv_weight_gradients(const cgptx_model* m, std::size_t rows, std::size_t H, std::size_t KW, int dt,
                                hipStream_t stream) {
    const std::size_t elem = dtype_size(dt);
    GemmArgs g;
    g.a_segments.count = 2;
    g.a_segments.ptr[0] = m->d_k_all.base;
    g.a_segments.ptr[1] = m->d_v_all.base;
    g.a_segments.ld[0] = g.a_segments.cols[0] = KW;
    g.a_segments.ld[1] = g.a_segments.cols[1] = KW;
    g.a_segment_batch_stride[0] = m->d_k_all.stride / elem;
    g.a_segment_batch_stride[1] = m->d_v_all.stride / elem;
    g.b = m->q_o_inputs.base;  // slots 0 .. layers - 1: the attention norm's output
    g.b_batch_stride = m->q_o_inputs.stride / elem;
    g.c = m->kv_gradients.base;
    g.batch_rows = 2 * KW;
    g.m = m->config.num_layers * 2 * KW;
    g.n = H;
    g.k = rows;
    g.ldb = H;
    g.ldc = H;
    g.a_k_contiguous = false;
    g.b_k_contiguous = false;
    g.dtype = dt;
    return gemm(g, stream);
}

// Whether the block's two norms run as one pass over the block input (CGPTX_FUSE_NORMS=0 keeps them
// separate, for comparisons).
bool fused_block_norms(const cgptx_model* m, const void* a, const void* b, const void* c, const void* d, const void* e) {
    const char* text = std::getenv("CGPTX_FUSE_NORMS");  // read per enqueue
    return (text == nullptr || text[0] != '0') && rmsnorm_dual_fusable(a, b, c, d, e, m->config.hidden_size, m->config.dtype);
}

// Whether the per-head norm and the rotary embedding of q or k run as one pass (CGPTX_FUSE_QK=0 keeps
// the separate operators, for comparisons).
bool fused_qk_norm_rope(const cgptx_model* m, const void* a, const void* b, const void* c, const void* weight) {
    const char* text = std::getenv("CGPTX_FUSE_QK");  // read per enqueue: a captured graph keeps what it was captured with
    const bool enabled = text == nullptr || text[0] != '0';
    return enabled && rmsnorm_rope_fusable(a, b, c, weight, m->cos_cache, m->sin_cache, m->config.head_dim,
                                           m->config.rotary_dim, m->config.dtype);
}

// Whether the gate/up projection also writes the SwiGLU product from its epilogue (CGPTX_FUSE_SWIGLU=0
// keeps the separate operator, for comparisons; shapes the fused kernel does not take run as the
// two operators either way).
bool fused_swiglu() {
    const char* text = std::getenv("CGPTX_FUSE_SWIGLU");  // read per enqueue
    return text == nullptr || text[0] != '0';
}

// Whether the down projection's input gradient also turns its result into the gradient of [gate | up] in its
// epilogue (CGPTX_FUSE_SWIGLU_GRAD=0 keeps the separate operator in the backward pass only, for comparisons).
bool fused_swiglu_gradient() {
    const char* text = std::getenv("CGPTX_FUSE_SWIGLU_GRAD");  // read per enqueue
    return text == nullptr || text[0] != '0';
}

// Whether the norm-backward passes of the step leave their weight-gradient reductions to one pair of launches at
// the end of the backward pass (CGPTX_FUSE_DGAMMA=0 keeps the two small launches after each pass, for comparisons:
// same additions in the same order, same bits).
cgptx::ColumnReduceSink* norm_reduction_sink(cgptx_model* m) {
    const char* text = std::getenv("CGPTX_FUSE_DGAMMA");  // read per enqueue
    return (text == nullptr || text[0] != '0') ? &m->norm_reductions : nullptr;
}

// Runs what the passes recorded. The entries are the same from pass to pass (same buffers, same shapes), so the
// device copy of the table is written once, by the first pass, outside any capture. The sink's memory and the
// table are sized when the model is created; should a pass still find the memory too small (it then reduced at
// once, from the arena), the memory grows here and the caller repeats the pass before recording it.
int finish_norm_reductions(cgptx_model* m, hipStream_t stream) {
    auto& sink = m->norm_reductions;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (stream != nullptr) CGPTX_HIP(hipStreamIsCapturing(stream, &capture));
    const bool capturing = capture != hipStreamCaptureStatusNone;
    // A recorded step holds the addresses of the table and of the sink's memory and the number of entries: it is
    // recorded again after any of them changes.
    auto drop_recorded_step = [&]() {
        for (auto& step : m->recorded) {
            if (step.exec != nullptr) (void)hipGraphExecDestroy(step.exec);
            step.exec = nullptr;
        }
    };
    if (!sink.entries.empty()) {
        if (!(sink.entries == m->norm_reduction_uploaded)) {
            if (capturing) return fail(CGPTX_RUNTIME, "model: the table of norm reductions changed under graph capture");
            CGPTX_HIP(hipStreamSynchronize(stream));  // earlier launches may still read the table
            drop_recorded_step();
            if (sink.entries.size() > m->norm_reduction_table_capacity) {
                if (m->norm_reduction_table != nullptr) CGPTX_HIP(hipFree(m->norm_reduction_table));
                m->norm_reduction_table = nullptr;
                CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&m->norm_reduction_table),
                                    sink.entries.size() * sizeof(ColumnReduceEntry)));
                m->norm_reduction_table_capacity = sink.entries.size();
            }
            CGPTX_HIP(hipMemcpy(m->norm_reduction_table, sink.entries.data(), sink.entries.size() * sizeof(ColumnReduceEntry),
                                hipMemcpyHostToDevice));
            m->norm_reduction_uploaded = sink.entries;
        }
        int max_hidden = 0, max_slices = 0;
        for (const ColumnReduceEntry& e : sink.entries) {
            max_hidden = std::max(max_hidden, e.hidden);
            max_slices = std::max(max_slices, e.slices);
        }
        if (int s = run_column_reductions(m->norm_reduction_table, static_cast<int>(sink.entries.size()), max_hidden,
                                          max_slices, stream))
            return s;
    }
    m->norm_reductions_resized = false;
    if (sink.wanted > sink.capacity && !capturing) {
        CGPTX_HIP(hipStreamSynchronize(stream));
        drop_recorded_step();
        if (sink.memory != nullptr) CGPTX_HIP(hipFree(sink.memory));
        sink.memory = nullptr;
        sink.capacity = 0;
        CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&sink.memory), sink.wanted));
        sink.capacity = sink.wanted;
        m->norm_reductions_resized = true;
    }
    return CGPTX_OK;
}

// CGPTX_FUSE=0: the step as the reference's own call sequence, one public operator per call — forward in the
// order of src/core/transformer_block.cu:466-595, backward in the order of :663-747 and
// src/core/transformer_model.cu:360-380 (separate q / k / v and gate / up projections with accumulating input
// gradients, separate SwiGLU and RoPE passes, residual additions as `add` calls). It is what a caller of
// include/ops/** executes, so its results are the yardstick for the fused step and for callers' own block code.
// The halves of the [rows, 2I] gate_up buffers serve as the separate [rows, I] gate and up tensors.
bool reference_call_sequence() {
    const char* text = std::getenv("CGPTX_FUSE");  // read per enqueue
    return text != nullptr && text[0] == '0';
}

// Adds one row to the model's call table (while cgptx_model_record_calls is on): the operator's name in
// include/ops/**, its tensors in the operator's argument order, its sizes and flags in the order of the C-ABI
// entry point, and its scalar (epsilon, attention scale or gradient scale).
void note_call(cgptx_model* m, const char* op, std::initializer_list<const void*> tensors,
               std::initializer_list<std::size_t> dims, std::initializer_list<int> flags = {}, float scalar = 0.0f) {
    if (!m->recording_calls) return;
    cgptx_call_record r{};
    r.op = op;
    std::size_t i = 0;
    for (const void* t : tensors) r.tensors[i++] = t;
    i = 0;
    for (std::size_t d : dims) r.dims[i++] = d;
    i = 0;
    for (int f : flags) r.flags[i++] = f;
    r.scalar = scalar;
    r.dtype = m->config.dtype;
    m->calls.push_back(r);
}

int enqueue_reference_sequence(cgptx_model* m, float loss_scale, int loss_mode, hipStream_t stream) {
    const auto& c = m->config;
    const int dt = c.dtype;
    const std::size_t N = m->rows, H = c.hidden_size, I = c.intermediate_size, V = c.vocabulary_size;
    const std::size_t HQ = c.num_query_heads, HKV = c.num_kv_heads, D = c.head_dim, B = m->batch, T = m->sequence;
    const std::size_t QW = HQ * D, KW = HKV * D, elem = dtype_size(dt);
    const float eps = c.rms_epsilon;
    auto* s = static_cast<cgptx_stream>(stream);
    auto second_half = [&](void* gate_up) { return static_cast<void*>(static_cast<char*>(gate_up) + N * I * elem); };
    m->calls.clear();

    // One public operator per call; each is entered in the call table before it is enqueued.
    auto norm_fwd = [&](void* out, const void* in, const void* w, std::size_t rows, std::size_t width) -> int {
        note_call(m, "rmsnorm_forward", {out, in, w}, {rows, width}, {}, eps);
        CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(out, in, w, rows, width, eps, dt, s));
        return CGPTX_OK;
    };
    auto norm_bwd = [&](void* dx, void* dw, const void* dy, const void* x, const void* w, std::size_t rows, std::size_t width) -> int {
        note_call(m, "rmsnorm_backward", {dx, dw, dy, x, w}, {rows, width}, {}, eps);
        CGPTX_OP("rmsnorm_bwd", cgptx_rmsnorm_backward(dx, dw, dy, x, w, rows, width, eps, dt, s));
        return CGPTX_OK;
    };
    auto project = [&](const char* label, void* out, const void* in, const void* w, std::size_t in_features, std::size_t out_features) -> int {
        note_call(m, "linear_forward", {out, in, w}, {N, in_features, out_features});
        CGPTX_OP(label, cgptx_linear_forward(out, in, w, nullptr, N, in_features, out_features, dt, s));
        return CGPTX_OK;
    };
    auto project_bwd = [&](const char* dx_label, const char* dw_label, void* dx, void* dw, const void* dy, const void* x, const void* w,
                           std::size_t in_features, std::size_t out_features, int accumulate_input) -> int {
        note_call(m, "linear_backward", {dx, dw, dy, x, w}, {N, in_features, out_features}, {accumulate_input});
        return linear_backward_split(m, dx, dw, dy, x, w, N, in_features, out_features, accumulate_input, dt, stream, dx_label, dw_label);
    };
    auto add = [&](void* out, const void* a, const void* b) -> int {
        note_call(m, "add", {out, a, b}, {N * H});
        CGPTX_OP("add", cgptx_add(out, a, b, N * H, dt, s));
        return CGPTX_OK;
    };

    note_call(m, "embedding_forward", {m->hidden[0], m->tokens, m->embedding.value}, {N, V, H});
    CGPTX_OP("embedding_fwd", cgptx_embedding_forward(m->hidden[0], m->tokens, N, m->embedding.value, V, H, dt, s));
    for (std::size_t l = 0; l < c.num_layers; ++l) {
        const auto& w = m->layers[l];
        const auto& a = m->acts[l];
        void *x = m->hidden[l], *out = m->hidden[l + 1];
        void *projected = m->d_norm_in, *ffn = m->d_norm_in_f;  // backward workspace, free during the forward pass
        void *gate = a.gate_up, *up = second_half(a.gate_up);
        CGPTX_TRY(norm_fwd(a.norm_a, x, w.attention_norm.value, N, H));
        CGPTX_TRY(project("gemm_fwd.qkv", a.q_pre, a.norm_a, w.q.value, H, QW));
        CGPTX_TRY(project("gemm_fwd.qkv", a.k_pre, a.norm_a, w.k.value, H, KW));
        CGPTX_TRY(project("gemm_fwd.qkv", a.v, a.norm_a, w.v.value, H, KW));
        CGPTX_TRY(norm_fwd(a.q, a.q_pre, w.q_norm.value, N * HQ, D));
        CGPTX_TRY(norm_fwd(a.k, a.k_pre, w.k_norm.value, N * HKV, D));
        note_call(m, "rope_forward", {a.q, a.k, m->cos_cache, m->sin_cache}, {B, T, HQ, HKV, D, c.rotary_dim, 0, T});
        CGPTX_OP("rope_fwd", cgptx_rope_forward(a.q, a.k, m->cos_cache, m->sin_cache, B, T, HQ, HKV, D, c.rotary_dim, 0, T, dt, s));
        note_call(m, "flash_gqa_attention_forward_with_lse", {a.attn_out, a.lse, a.q, a.k, a.v}, {B, T, T, HQ, HKV, D, 0}, {1});
        CGPTX_OP("attn_fwd", cgptx_flash_gqa_attention_forward(a.attn_out, a.lse, a.q, a.k, a.v, B, T, T, HQ, HKV, D, 0.0f, 1, 0, dt, s));
        CGPTX_TRY(project("gemm_fwd.o", projected, a.attn_out, w.o.value, QW, H));
        CGPTX_TRY(norm_fwd(a.norm_f, x, w.ffn_norm.value, N, H));
        CGPTX_TRY(project("gemm_fwd.gate_up", gate, a.norm_f, w.gate.value, H, I));
        CGPTX_TRY(project("gemm_fwd.gate_up", up, a.norm_f, w.up.value, H, I));
        note_call(m, "swiglu_forward", {a.act, gate, up}, {N * I});
        CGPTX_OP("swiglu_fwd", cgptx_swiglu_forward(a.act, gate, up, N * I, dt, s));
        CGPTX_TRY(project("gemm_fwd.down", ffn, a.act, w.down.value, I, H));
        CGPTX_TRY(add(out, x, projected));
        CGPTX_TRY(add(out, out, ffn));
    }
    void* last = m->hidden[c.num_layers];
    CGPTX_TRY(norm_fwd(m->normalized, last, m->final_norm.value, N, H));
    if (loss_mode == CGPTX_LOSS_CUT) {
        note_call(m, "cut_cross_entropy_forward_backward", {m->loss, m->d_normalized, m->embedding.gradient, m->normalized,
                                                            m->embedding.value, m->targets}, {N, H, V}, {}, loss_scale);
        CGPTX_OP("cut_ce", cgptx_cut_cross_entropy_forward_backward(m->loss, m->d_normalized, m->embedding.gradient, m->normalized,
                                                                    m->embedding.value, m->targets, N, H, V, loss_scale, 0, dt, s));
    } else {
        CGPTX_TRY(project("gemm_fwd.classifier", m->logits, m->normalized, m->embedding.value, H, V));
        note_call(m, "cross_entropy_forward_backward", {m->loss, m->grad_logits, m->logits, m->targets}, {N, V}, {}, loss_scale);
        CGPTX_OP("dense_ce", cgptx_cross_entropy_forward_backward(m->loss, m->grad_logits, m->logits, m->targets, N, V, loss_scale, dt, s));
        CGPTX_TRY(project_bwd("gemm_dx.classifier", "gemm_dw.classifier", m->d_normalized, m->embedding.gradient, m->grad_logits,
                              m->normalized, m->embedding.value, H, V, 0));
    }

    void *current = m->grad_a, *previous = m->grad_b;
    CGPTX_TRY(norm_bwd(current, m->final_norm.gradient, m->d_normalized, last, m->final_norm.value, N, H));
    for (std::size_t reverse = c.num_layers; reverse-- > 0;) {
        const auto& w = m->layers[reverse];
        const auto& a = m->acts[reverse];
        void* x = m->hidden[reverse];
        void *gate = a.gate_up, *up = second_half(a.gate_up);
        void *d_gate = m->d_gate_up, *d_up = second_half(m->d_gate_up);
        void* grad_residual = m->d_norm_in_f;
        CGPTX_TRY(project_bwd("gemm_dx.down", "gemm_dw.down", m->d_act, w.down.gradient, current, a.act, w.down.value, I, H, 0));
        note_call(m, "swiglu_backward", {d_gate, d_up, m->d_act, gate, up}, {N * I}, {0, 0});
        CGPTX_OP("swiglu_bwd", cgptx_swiglu_backward(d_gate, d_up, m->d_act, gate, up, N * I, 0, 0, dt, s));
        CGPTX_TRY(project_bwd("gemm_dx.gate_up", "gemm_dw.gate_up", m->d_norm_in, w.gate.gradient, d_gate, a.norm_f, w.gate.value, H, I, 0));
        CGPTX_TRY(project_bwd("gemm_dx.gate_up", "gemm_dw.gate_up", m->d_norm_in, w.up.gradient, d_up, a.norm_f, w.up.value, H, I, 1));
        CGPTX_TRY(norm_bwd(grad_residual, w.ffn_norm.gradient, m->d_norm_in, x, w.ffn_norm.value, N, H));
        CGPTX_TRY(add(previous, current, grad_residual));  // grad_input = grad_output + grad_residual
        CGPTX_TRY(project_bwd("gemm_dx.o", "gemm_dw.o", m->d_attn_out, w.o.gradient, current, a.attn_out, w.o.value, QW, H, 0));
        note_call(m, "flash_gqa_attention_backward_with_lse", {m->d_q, m->d_k, m->d_v, m->d_attn_out, a.attn_out, a.lse, a.q, a.k, a.v},
                  {B, T, T, HQ, HKV, D, 0}, {1, 0});
        CGPTX_OP("attn_bwd", cgptx_flash_gqa_attention_backward_with_lse(m->d_q, m->d_k, m->d_v, m->d_attn_out, a.attn_out, a.lse,
                                                                         a.q, a.k, a.v, B, T, T, HQ, HKV, D, 0.0f, 1, 0, 0, dt, s));
        note_call(m, "rope_backward", {m->d_q_pre, m->d_k_pre, m->d_q, m->d_k, m->cos_cache, m->sin_cache},
                  {B, T, HQ, HKV, D, c.rotary_dim, 0, T});
        CGPTX_OP("rope_bwd", cgptx_rope_backward(m->d_q_pre, m->d_k_pre, m->d_q, m->d_k, m->cos_cache, m->sin_cache, B, T, HQ, HKV, D,
                                                 c.rotary_dim, 0, T, dt, s));
        CGPTX_TRY(norm_bwd(m->d_q, w.q_norm.gradient, m->d_q_pre, a.q_pre, w.q_norm.value, N * HQ, D));
        CGPTX_TRY(norm_bwd(m->d_k, w.k_norm.gradient, m->d_k_pre, a.k_pre, w.k_norm.value, N * HKV, D));
        CGPTX_TRY(project_bwd("gemm_dx.qkv", "gemm_dw.qkv", m->d_norm_in, w.q.gradient, m->d_q, a.norm_a, w.q.value, H, QW, 0));
        CGPTX_TRY(project_bwd("gemm_dx.qkv", "gemm_dw.qkv", m->d_norm_in, w.k.gradient, m->d_k, a.norm_a, w.k.value, H, KW, 1));
        CGPTX_TRY(project_bwd("gemm_dx.qkv", "gemm_dw.qkv", m->d_norm_in, w.v.gradient, m->d_v, a.norm_a, w.v.value, H, KW, 1));
        CGPTX_TRY(norm_bwd(grad_residual, w.attention_norm.gradient, m->d_norm_in, x, w.attention_norm.value, N, H));
        CGPTX_TRY(add(previous, previous, grad_residual));
        std::swap(current, previous);
    }
    note_call(m, "embedding_backward", {m->embedding.gradient, current, m->tokens}, {N, V, H}, {1, 1});
    CGPTX_OP("embedding_bwd", cgptx_embedding_backward(m->embedding.gradient, current, m->tokens, N, V, H, 1, 1, dt, s));
    return CGPTX_OK;
}

int enqueue_forward_backward(cgptx_model* m, float loss_scale, int loss_mode, hipStream_t stream) {
    if (reference_call_sequence()) return enqueue_reference_sequence(m, loss_scale, loss_mode, stream);
    const auto& c = m->config;
    const int dt = c.dtype;
    const std::size_t N = m->rows, H = c.hidden_size, I = c.intermediate_size;
    const std::size_t HQ = c.num_query_heads, HKV = c.num_kv_heads, D = c.head_dim;
    const std::size_t QW = HQ * D, KW = HKV * D;
    const float eps = c.rms_epsilon;
    auto* s = static_cast<cgptx_stream>(stream);
    // One launch for the q/k/v projections needs 16-bit storage and segment widths the tiles respect.
    const bool fused_qkv = dt != CGPTX_F32 && QW % 256 == 0 && KW % 256 == 0 && H % 32 == 0 && N % 32 == 0;

    // ------------------------------------------------------------------ forward
    CGPTX_OP("embedding_fwd", cgptx_embedding_forward(m->hidden[0], m->tokens, N, m->embedding.value, c.vocabulary_size, H, dt, s));
    for (std::size_t l = 0; l < c.num_layers; ++l) {
        const auto& w = m->layers[l];
        const auto& a = m->acts[l];
        void* x = m->hidden[l];
        void* out = m->hidden[l + 1];
        // Both norms of the block read its input: one pass when the shape allows.
        const bool dual_norms = fused_block_norms(m, a.norm_a, a.norm_f, x, w.attention_norm.value, w.ffn_norm.value);
        if (dual_norms) {
            CGPTX_OP("rmsnorm_fwd", rmsnorm_forward_dual(a.norm_a, a.norm_f, x, w.attention_norm.value, w.ffn_norm.value, N, H, eps,
                                                         dt, stream));
        } else {
            CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(a.norm_a, x, w.attention_norm.value, N, H, eps, dt, s));
        }
        if (fused_qkv) {
            CGPTX_OP("gemm_fwd.qkv", qkv_forward(a.q_pre, a.k_pre, a.v, a.norm_a, w.q.value, N, H, QW, KW, dt, stream));
        } else {
            CGPTX_OP("gemm_fwd.qkv", cgptx_linear_forward(a.q_pre, a.norm_a, w.q.value, nullptr, N, H, QW, dt, s));
            CGPTX_OP("gemm_fwd.qkv", cgptx_linear_forward(a.k_pre, a.norm_a, w.k.value, nullptr, N, H, KW, dt, s));
            CGPTX_OP("gemm_fwd.qkv", cgptx_linear_forward(a.v, a.norm_a, w.v.value, nullptr, N, H, KW, dt, s));
        }
        if (fused_qk_norm_rope(m, a.q, a.q_pre, nullptr, w.q_norm.value) && fused_qk_norm_rope(m, a.k, a.k_pre, nullptr, w.k_norm.value)) {
            CGPTX_OP("rmsnorm_fwd", rmsnorm_rope_forward(a.q, a.q_pre, w.q_norm.value, m->cos_cache, m->sin_cache, N * HQ, D, HQ,
                                                         m->sequence, c.rotary_dim, 0, eps, dt, stream));
            CGPTX_OP("rmsnorm_fwd", rmsnorm_rope_forward(a.k, a.k_pre, w.k_norm.value, m->cos_cache, m->sin_cache, N * HKV, D, HKV,
                                                         m->sequence, c.rotary_dim, 0, eps, dt, stream));
        } else {
            CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(a.q, a.q_pre, w.q_norm.value, N * HQ, D, eps, dt, s));
            CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(a.k, a.k_pre, w.k_norm.value, N * HKV, D, eps, dt, s));
            CGPTX_OP("rope_fwd", cgptx_rope_forward(a.q, a.k, m->cos_cache, m->sin_cache, m->batch, m->sequence, HQ, HKV, D,
                                         c.rotary_dim, 0, m->sequence, dt, s));
        }
        CGPTX_OP("attn_fwd", cgptx_flash_gqa_attention_forward(a.attn_out, a.lse, a.q, a.k, a.v, m->batch, m->sequence,
                                                    m->sequence, HQ, HKV, D, 0.0f, 1, 0, dt, s));
        // out = x + attention_projection, then out += ffn_output (src/core/transformer_block.cu:594-595)
        CGPTX_OP("gemm_fwd.o", linear_forward_residual(out, a.attn_out, w.o.value, x, false, N, QW, H, dt, stream));
        if (!dual_norms) CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(a.norm_f, x, w.ffn_norm.value, N, H, eps, dt, s));
        if (fused_swiglu()) {
            CGPTX_OP("gemm_fwd.gate_up", cgptx_linear_swiglu_forward(a.gate_up, a.act, a.norm_f, w.gate.value, N, H, I, dt, s));
        } else {
            CGPTX_OP("gemm_fwd.gate_up", cgptx_linear_forward(a.gate_up, a.norm_f, w.gate.value, nullptr, N, H, 2 * I, dt, s));
            CGPTX_OP("swiglu_fwd", cgptx_swiglu_forward_packed(a.act, a.gate_up, N, I, dt, s));
        }
        CGPTX_OP("gemm_fwd.down", linear_forward_residual(out, a.act, w.down.value, nullptr, true, N, I, H, dt, stream));
    }
    void* last = m->hidden[c.num_layers];
    CGPTX_OP("rmsnorm_fwd", cgptx_rmsnorm_forward(m->normalized, last, m->final_norm.value, N, H, eps, dt, s));

    // --------------------------------------------------------- loss + classifier
    if (loss_mode == CGPTX_LOSS_CUT) {
        CGPTX_OP("cut_ce", cgptx_cut_cross_entropy_forward_backward(m->loss, m->d_normalized, m->embedding.gradient,
                                                           m->normalized, m->embedding.value, m->targets, N, H,
                                                           c.vocabulary_size, loss_scale, 0, dt, s));
    } else {
        CGPTX_OP("gemm_fwd.classifier", cgptx_linear_forward(m->logits, m->normalized, m->embedding.value, nullptr, N, H,
                                       c.vocabulary_size, dt, s));
        CGPTX_OP("dense_ce", cgptx_cross_entropy_forward_backward(m->loss, m->grad_logits, m->logits, m->targets, N,
                                                       c.vocabulary_size, loss_scale, dt, s));
        CGPTX_TRY(linear_backward_split(m, m->d_normalized, m->embedding.gradient, m->grad_logits, m->normalized, m->embedding.value, N, H, c.vocabulary_size, 0, dt, stream, "gemm_dx.classifier", "gemm_dw.classifier"));
    }

    // ----------------------------------------------------------------- backward
    // With the weight gradients left to the end, layer l keeps its output gradients: the residual stream's in slot
    // own slot (the slot of the block's input receives the block's input gradient), [dgate | dup], dq, dk and dv in slot l
    // of their stacks. Otherwise one set of buffers serves every layer.
    const bool stacked = m->stacked_dw && fused_qkv;
    void* current = stacked ? m->d_hidden_slot(c.num_layers) : m->grad_a;
    void* previous = stacked ? nullptr : m->grad_b;
    ColumnReduceSink* sink = norm_reduction_sink(m);
    m->norm_reductions.begin();
    CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_residual(current, m->final_norm.gradient, m->d_normalized, last, m->final_norm.value,
                                                      nullptr, N, H, eps, dt, stream, sink));
    for (std::size_t reverse = c.num_layers; reverse-- > 0;) {
        const auto& w = m->layers[reverse];
        const auto& a = m->acts[reverse];
        void* x = m->hidden[reverse];
        void* d_gate_up = stacked ? m->d_gate_up_all.at(reverse) : m->d_gate_up;
        void* d_q = stacked ? m->q_o_output_gradients.at(reverse) : m->d_q;
        void* d_k = stacked ? m->d_k_all.at(reverse) : m->d_k;
        void* d_v = stacked ? m->d_v_all.at(reverse) : m->d_v;
        if (stacked) previous = m->d_hidden_slot(reverse);
        if (fused_swiglu() && fused_swiglu_gradient()) {
            // The SwiGLU gradient rides in the epilogue of the down projection's input gradient.
            CGPTX_OP("gemm_dx.down", cgptx_linear_swiglu_backward(d_gate_up, m->d_act, current, w.down.value, a.gate_up, N, I, H, dt, s));
            if (!stacked)
                CGPTX_OP("gemm_dw.down", cgptx_linear_backward(nullptr, w.down.gradient, nullptr, current, a.act, w.down.value, N, I, H, 0, 0, 0, dt, s));
        } else {
            CGPTX_OP("gemm_dx.down", cgptx_linear_backward(m->d_act, nullptr, nullptr, current, a.act, w.down.value, N, I, H, 0, 0, 0, dt, s));
            if (!stacked)
                CGPTX_OP("gemm_dw.down", cgptx_linear_backward(nullptr, w.down.gradient, nullptr, current, a.act, w.down.value, N, I, H, 0, 0, 0, dt, s));
            CGPTX_OP("swiglu_bwd", cgptx_swiglu_backward_packed(d_gate_up, m->d_act, a.gate_up, N, I, 0, dt, s));
        }
        // The gradient of the residual stream collects the two norm branches: in one pass at the end of
        // the block when the shape allows (previous = current + d(ffn norm) + d(attention norm)), else as
        // they are produced (previous = current + d(ffn branch), later previous += d(attention branch)).
        const bool dual_norms = fused_block_norms(m, previous, m->d_norm_in, m->d_norm_in_f, x, current) &&
                                is_aligned16(w.attention_norm.value) && is_aligned16(w.ffn_norm.value);
        void* d_norm_f = dual_norms ? m->d_norm_in_f : m->d_norm_in;
        CGPTX_OP("gemm_dx.gate_up", cgptx_linear_backward(d_norm_f, nullptr, nullptr, d_gate_up, a.norm_f, w.gate.value, N, H, 2 * I, 0, 0, 0, dt, s));
        if (!stacked)
            CGPTX_OP("gemm_dw.gate_up", cgptx_linear_backward(nullptr, w.gate.gradient, nullptr, d_gate_up, a.norm_f, w.gate.value, N, H, 2 * I, 0, 0, 0, dt, s));
        if (!dual_norms) {
            CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_residual(previous, w.ffn_norm.gradient, m->d_norm_in, x, w.ffn_norm.value,
                                                              current, N, H, eps, dt, stream, sink));
        }
        CGPTX_OP("gemm_dx.o", cgptx_linear_backward(m->d_attn_out, nullptr, nullptr, current, a.attn_out, w.o.value, N, QW, H, 0, 0, 0, dt, s));
        if (!stacked)
            CGPTX_OP("gemm_dw.o", cgptx_linear_backward(nullptr, w.o.gradient, nullptr, current, a.attn_out, w.o.value, N, QW, H, 0, 0, 0, dt, s));
        CGPTX_OP("attn_bwd", cgptx_flash_gqa_attention_backward_with_lse(d_q, d_k, d_v, m->d_attn_out, a.attn_out,
                                                              a.lse, a.q, a.k, a.v, m->batch, m->sequence,
                                                              m->sequence, HQ, HKV, D, 0.0f, 1, 0, 0, dt, s));
        // In place over the attention gradients (a lane reads and writes the same elements).
        if (fused_qk_norm_rope(m, d_q, d_q, a.q_pre, w.q_norm.value) &&
            fused_qk_norm_rope(m, d_k, d_k, a.k_pre, w.k_norm.value)) {
            CGPTX_OP("rmsnorm_bwd", rmsnorm_rope_backward(d_q, w.q_norm.gradient, d_q, a.q_pre, w.q_norm.value, m->cos_cache,
                                                          m->sin_cache, N * HQ, D, HQ, m->sequence, c.rotary_dim, 0, eps, dt, stream, sink));
            CGPTX_OP("rmsnorm_bwd", rmsnorm_rope_backward(d_k, w.k_norm.gradient, d_k, a.k_pre, w.k_norm.value, m->cos_cache,
                                                          m->sin_cache, N * HKV, D, HKV, m->sequence, c.rotary_dim, 0, eps, dt, stream, sink));
        } else {
            CGPTX_OP("rope_bwd", cgptx_rope_backward(m->d_q_pre, m->d_k_pre, d_q, d_k, m->cos_cache, m->sin_cache, m->batch,
                                          m->sequence, HQ, HKV, D, c.rotary_dim, 0, m->sequence, dt, s));
            CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_residual(d_q, w.q_norm.gradient, m->d_q_pre, a.q_pre, w.q_norm.value, nullptr,
                                                              N * HQ, D, eps, dt, stream, sink));
            CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_residual(d_k, w.k_norm.gradient, m->d_k_pre, a.k_pre, w.k_norm.value, nullptr,
                                                              N * HKV, D, eps, dt, stream, sink));
        }
        if (fused_qkv) {
            CGPTX_OP("gemm_dx.qkv", qkv_backward_input(m->d_norm_in, d_q, d_k, d_v, w.q.value, N, H, QW, KW, dt, stream));
            if (!stacked)
                CGPTX_OP("gemm_dw.qkv", qkv_backward_weight(w.q.gradient, d_q, d_k, d_v, a.norm_a, N, H, QW, KW, dt, stream));
        } else {
            CGPTX_TRY(linear_backward_split(m, m->d_norm_in, w.q.gradient, d_q, a.norm_a, w.q.value, N, H, QW, 0, dt, stream, "gemm_dx.qkv", "gemm_dw.qkv"));
            CGPTX_TRY(linear_backward_split(m, m->d_norm_in, w.k.gradient, d_k, a.norm_a, w.k.value, N, H, KW, 1, dt, stream, "gemm_dx.qkv", "gemm_dw.qkv"));
            CGPTX_TRY(linear_backward_split(m, m->d_norm_in, w.v.gradient, d_v, a.norm_a, w.v.value, N, H, KW, 1, dt, stream, "gemm_dx.qkv", "gemm_dw.qkv"));
        }
        if (dual_norms) {
            CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_dual(previous, w.attention_norm.gradient, w.ffn_norm.gradient, m->d_norm_in,
                                                          m->d_norm_in_f, x, w.attention_norm.value, w.ffn_norm.value, current, N, H,
                                                          eps, dt, stream, sink));
        } else {
            CGPTX_OP("rmsnorm_bwd", rmsnorm_backward_residual(previous, w.attention_norm.gradient, m->d_norm_in, x,
                                                              w.attention_norm.value, previous, N, H, eps, dt, stream, sink));
        }
        if (stacked) current = previous;
        else std::swap(current, previous);
    }
    if (stacked) {
        // The down projection reads the residual stream's gradient at each block's output (slots layers .. of the q / output
        // stack); the q and output projections of all layers are one stack of 2 x layers products.
        const std::size_t L = c.num_layers;
        CGPTX_OP("gemm_dw.down", stacked_weight_gradients(m->down_gradients, m->d_hidden_slot(1), m->q_o_output_gradients.stride,
                                                          m->act_all, N, I, H, L, dt, stream));
        CGPTX_OP("gemm_dw.gate_up", stacked_weight_gradients(m->gate_up_gradients, m->d_gate_up_all.base, m->d_gate_up_all.stride,
                                                             m->norm_f_all, N, H, 2 * I, L, dt, stream));
        CGPTX_OP("gemm_dw.q_o", stacked_weight_gradients(m->q_o_gradients, m->q_o_output_gradients.base, m->q_o_output_gradients.stride,
                                                         m->q_o_inputs, N, H, H, 2 * L, dt, stream));
        CGPTX_OP("gemm_dw.kv", stacked_kv_weight_gradients(m, N, H, KW, dt, stream));
    }
    // Tied embedding: the classifier gradient is already in place; add the lookup's gradient
    // (src/core/transformer_model.cu:375-380).
    CGPTX_OP("embedding_bwd", cgptx_embedding_backward(m->embedding.gradient, current, m->tokens, N, c.vocabulary_size, H, 1, 1, dt, s));
    CGPTX_OP("rmsnorm_bwd", finish_norm_reductions(m, stream));
    return CGPTX_OK;
}

int validate_config(const cgptx_model_config& c, std::size_t batch, std::size_t sequence) {
    if (!valid_dtype(c.dtype)) return fail(CGPTX_INVALID_ARGUMENT, "model: unsupported dtype");
    if (c.vocabulary_size == 0 || c.num_layers == 0 || c.hidden_size == 0 || c.intermediate_size == 0 ||
        c.num_query_heads == 0 || c.num_kv_heads == 0 || c.head_dim == 0 || batch == 0 || sequence == 0)
        return fail(CGPTX_INVALID_ARGUMENT, "model: every dimension must be positive");
    if (c.num_query_heads % c.num_kv_heads != 0)
        return fail(CGPTX_INVALID_ARGUMENT, "model: query heads must be a multiple of kv heads");
    if (c.num_query_heads * c.head_dim != c.hidden_size)
        return fail(CGPTX_INVALID_ARGUMENT, "model: hidden_size must equal num_query_heads * head_dim");
    const std::size_t rotary = c.rotary_dim == 0 ? c.head_dim : c.rotary_dim;
    if ((rotary & 1) != 0 || rotary > c.head_dim || (c.head_dim & 1) != 0)
        return fail(CGPTX_INVALID_ARGUMENT, "model: head_dim and rotary_dim must be even, rotary_dim <= head_dim");
    if (c.head_dim > 128)  // the attention operators' limit (src/ops/backward/attention_backward.cu:1886-1887)
        return fail(CGPTX_INVALID_ARGUMENT, "model: head_dim must not exceed 128");
    if (!std::isfinite(c.rms_epsilon) || c.rms_epsilon <= 0.0f || !std::isfinite(c.rope_base) || c.rope_base <= 0.0f)
        return fail(CGPTX_INVALID_ARGUMENT, "model: invalid epsilon or rope base");
    return CGPTX_OK;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_model_destroy(cgptx_model* m) {
    if (m == nullptr) return CGPTX_OK;
    (void)hipDeviceSynchronize();
    for (auto& step : m->recorded)
        if (step.exec != nullptr) (void)hipGraphExecDestroy(step.exec);
    if (m->optimizer != nullptr) (void)cgptx_adamw_workspace_destroy(m->optimizer);
    for (void* p : m->allocations) (void)hipFree(p);
    if (m->norm_reductions.memory != nullptr) (void)hipFree(m->norm_reductions.memory);
    if (m->norm_reduction_table != nullptr) (void)hipFree(m->norm_reduction_table);
    delete m;
    return CGPTX_OK;
}

extern "C" int cgptx_model_create(cgptx_model** out, const cgptx_model_config* config, size_t batch, size_t sequence,
                                  uint64_t seed) {
    using namespace cgptx;
    if (out == nullptr || config == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_create: null argument");
    if (int s = validate_config(*config, batch, sequence)) return s;
    auto* m = new cgptx_model();
    m->config = *config;
    if (m->config.rotary_dim == 0) m->config.rotary_dim = m->config.head_dim;
    m->batch = batch;
    m->sequence = sequence;
    m->rows = batch * sequence;
    const auto& c = m->config;
    const std::size_t elem = dtype_size(c.dtype);
    const std::size_t N = m->rows, H = c.hidden_size, I = c.intermediate_size;
    const std::size_t QW = c.num_query_heads * c.head_dim, KW = c.num_kv_heads * c.head_dim;
    const float stddev = 0.02f;
    const float residual_stddev = stddev / std::sqrt(2.0f * static_cast<float>(c.num_layers));
    auto build = [&]() -> int {
        CGPTX_TRY(make_parameter(m, m->embedding, "model.embed_tokens.weight", c.vocabulary_size * H, 0, stddev, seed, 0));
        CGPTX_TRY(make_parameter(m, m->final_norm, "model.norm.weight", H, 1, 0.0f, seed, 1));
        m->layers.resize(c.num_layers);
        m->acts.resize(c.num_layers);
        m->stacked_dw = stackable_weight_gradients(c, N);
        if (m->stacked_dw) {
            const std::size_t L = c.num_layers;
            auto stack = [&](cgptx_model::Stack& st, std::size_t bytes, std::size_t count) -> int {
                st.stride = bytes;
                return allocate_typed(m, &st.base, bytes * count);
            };
            m->stacked_layers = L;
            CGPTX_TRY(stack(m->q_o_gradients, H * H * elem, 2 * L));
            CGPTX_TRY(stack(m->kv_gradients, 2 * KW * H * elem, L));
            CGPTX_TRY(stack(m->gate_up_gradients, 2 * I * H * elem, L));
            CGPTX_TRY(stack(m->down_gradients, H * I * elem, L));
            CGPTX_TRY(stack(m->q_o_inputs, N * H * elem, 2 * L));
            CGPTX_TRY(stack(m->norm_f_all, N * H * elem, L));
            CGPTX_TRY(stack(m->act_all, N * I * elem, L));
            CGPTX_TRY(stack(m->q_o_output_gradients, N * H * elem, 2 * L + 1));
            CGPTX_TRY(stack(m->d_gate_up_all, N * 2 * I * elem, L));
            CGPTX_TRY(stack(m->d_k_all, N * KW * elem, L));
            CGPTX_TRY(stack(m->d_v_all, N * KW * elem, L));
        }
        // A tensor of layer l: its slot in the stack of its kind, or an allocation of its own.
        auto place = [&](void** out, const cgptx_model::Stack& st, std::size_t l, std::size_t bytes) -> int {
            if (m->stacked_dw) {
                *out = st.at(l);
                return CGPTX_OK;
            }
            return allocate(m, out, bytes);
        };
        for (std::size_t l = 0; l < c.num_layers; ++l) {
            auto& w = m->layers[l];
            const std::string prefix = "model.layers." + std::to_string(l) + ".";
            const std::uint64_t id = 2 + l * 11;
            CGPTX_TRY(make_parameter(m, w.attention_norm, prefix + "input_layernorm.weight", H, 1, 0, seed, id));
            // q, k and v share one [QW + 2 KW, H] block of values: the three projections of the normalized input run as
            // one contraction whose output columns go to three buffers. Their gradients share such a block too when
            // every layer computes its own weight gradients; with the stacked launches q's lies in the q / output
            // stack and [k; v]'s in a stack of its own.
            char *qkv_value = nullptr, *q_gradient = nullptr, *k_gradient = nullptr, *v_gradient = nullptr;
            CGPTX_TRY(allocate_typed(m, &qkv_value, (QW + 2 * KW) * H * elem));
            if (m->stacked_dw) {
                q_gradient = static_cast<char*>(m->q_o_gradients.at(l));
                k_gradient = static_cast<char*>(m->kv_gradients.at(l));
                v_gradient = k_gradient + KW * H * elem;
            } else {
                CGPTX_TRY(allocate_typed(m, &q_gradient, (QW + 2 * KW) * H * elem));
                k_gradient = q_gradient + QW * H * elem;
                v_gradient = k_gradient + KW * H * elem;
            }
            CGPTX_TRY(make_parameter(m, w.q, prefix + "self_attn.q_proj.weight", QW * H, 0, stddev, seed, id + 1, qkv_value,
                                     q_gradient));
            CGPTX_TRY(make_parameter(m, w.k, prefix + "self_attn.k_proj.weight", KW * H, 0, stddev, seed, id + 2,
                                     qkv_value + QW * H * elem, k_gradient));
            CGPTX_TRY(make_parameter(m, w.q_norm, prefix + "self_attn.q_norm.weight", c.head_dim, 1, 0, seed, id + 3));
            CGPTX_TRY(make_parameter(m, w.k_norm, prefix + "self_attn.k_norm.weight", c.head_dim, 1, 0, seed, id + 4));
            CGPTX_TRY(make_parameter(m, w.v, prefix + "self_attn.v_proj.weight", KW * H, 0, stddev, seed, id + 5,
                                     qkv_value + (QW + KW) * H * elem, v_gradient));
            void* o_gradient = nullptr;
            if (m->stacked_dw) o_gradient = m->q_o_gradients.at(c.num_layers + l);
            CGPTX_TRY(make_parameter(m, w.o, prefix + "self_attn.o_proj.weight", H * QW, 0, residual_stddev, seed, id + 6, nullptr,
                                     o_gradient));
            CGPTX_TRY(make_parameter(m, w.ffn_norm, prefix + "post_attention_layernorm.weight", H, 1, 0, seed, id + 7));
            // gate and up share one [2I, H] block (values and gradients), so that the block's three
            // contractions with them each run as one [.., 2I] product on the packed activations.
            void *gate_up_value = nullptr, *gate_up_gradient = nullptr;
            CGPTX_TRY(allocate(m, &gate_up_value, 2 * I * H * elem));
            CGPTX_TRY(place(&gate_up_gradient, m->gate_up_gradients, l, 2 * I * H * elem));
            CGPTX_TRY(make_parameter(m, w.gate, prefix + "mlp.gate_proj.weight", I * H, 0, stddev, seed, id + 8,
                                     gate_up_value, gate_up_gradient));
            CGPTX_TRY(make_parameter(m, w.up, prefix + "mlp.up_proj.weight", I * H, 0, stddev, seed, id + 9,
                                     static_cast<char*>(gate_up_value) + I * H * elem,
                                     static_cast<char*>(gate_up_gradient) + I * H * elem));
            void* down_gradient = nullptr;
            if (m->stacked_dw) down_gradient = m->down_gradients.at(l);
            CGPTX_TRY(make_parameter(m, w.down, prefix + "mlp.down_proj.weight", H * I, 0, residual_stddev, seed, id + 10, nullptr,
                                     down_gradient));
            auto& a = m->acts[l];
            CGPTX_TRY(place(&a.norm_a, m->q_o_inputs, l, N * H * elem));
            CGPTX_TRY(allocate(m, &a.q_pre, N * QW * elem));
            CGPTX_TRY(allocate(m, &a.k_pre, N * KW * elem));
            CGPTX_TRY(allocate(m, &a.q, N * QW * elem));
            CGPTX_TRY(allocate(m, &a.k, N * KW * elem));
            CGPTX_TRY(allocate(m, &a.v, N * KW * elem));
            CGPTX_TRY(place(&a.attn_out, m->q_o_inputs, c.num_layers + l, N * QW * elem));
            CGPTX_TRY(allocate_typed(m, &a.lse, N * c.num_query_heads * sizeof(float)));
            CGPTX_TRY(place(&a.norm_f, m->norm_f_all, l, N * H * elem));
            CGPTX_TRY(allocate(m, &a.gate_up, N * 2 * I * elem));
            CGPTX_TRY(place(&a.act, m->act_all, l, N * I * elem));
        }
        m->hidden.resize(c.num_layers + 1);
        for (auto& h : m->hidden) CGPTX_TRY(allocate(m, &h, N * H * elem));
        CGPTX_TRY(allocate(m, &m->normalized, N * H * elem));
        CGPTX_TRY(allocate_typed(m, &m->tokens, N * sizeof(std::uint32_t)));
        CGPTX_TRY(allocate_typed(m, &m->targets, N * sizeof(std::uint32_t)));
        CGPTX_HIP(hipMemset(m->tokens, 0, N * sizeof(std::uint32_t)));
        CGPTX_HIP(hipMemset(m->targets, 0, N * sizeof(std::uint32_t)));
        CGPTX_TRY(allocate_typed(m, &m->loss, 256));
        CGPTX_HIP(hipMemset(m->loss, 0, 256));
        for (void** p : {&m->d_normalized, &m->grad_a, &m->grad_b, &m->d_norm_in, &m->d_norm_in_f})
            CGPTX_TRY(allocate(m, p, N * H * elem));
        CGPTX_TRY(allocate(m, &m->d_act, N * I * elem));
        CGPTX_TRY(allocate(m, &m->d_gate_up, N * 2 * I * elem));
        for (void** p : {&m->d_attn_out, &m->d_q, &m->d_q_pre}) CGPTX_TRY(allocate(m, p, N * QW * elem));
        for (void** p : {&m->d_k, &m->d_v, &m->d_k_pre}) CGPTX_TRY(allocate(m, p, N * KW * elem));
        // Rotary cache: theta = pos / base^(2i/rotary), cos/sin in float, stored in the model dtype
        // (train/train.cpp:322-333).
        const std::size_t pairs = c.rotary_dim / 2;
        std::vector<float> cosine(sequence * pairs), sine(sequence * pairs);
        for (std::size_t pos = 0; pos < sequence; ++pos) {
            for (std::size_t i = 0; i < pairs; ++i) {
                const float theta = static_cast<float>(pos) /
                                    std::pow(c.rope_base, 2.0f * static_cast<float>(i) / static_cast<float>(c.rotary_dim));
                cosine[pos * pairs + i] = std::cos(theta);
                sine[pos * pairs + i] = std::sin(theta);
            }
        }
        std::vector<unsigned char> storage;
        CGPTX_TRY(allocate(m, &m->cos_cache, sequence * pairs * elem));
        CGPTX_TRY(allocate(m, &m->sin_cache, sequence * pairs * elem));
        convert_to_storage(cosine, c.dtype, storage);
        CGPTX_HIP(hipMemcpy(m->cos_cache, storage.data(), storage.size(), hipMemcpyHostToDevice));
        convert_to_storage(sine, c.dtype, storage);
        CGPTX_HIP(hipMemcpy(m->sin_cache, storage.data(), storage.size(), hipMemcpyHostToDevice));
        // Memory for the weight-gradient partial sums of every norm-backward pass of a step, and the device table of
        // their reductions, sized here from the shapes: the first pass then finds room, defers its reductions and is
        // not repeated. Each pair of alternatives (per-head norms with or without the rotary embedding, the block's
        // two norms in one pass or two) is sized for the larger one; a pass that still asks for more than this grows
        // the memory when it ends, as before.
        {
            const std::size_t HQ = c.num_query_heads, HKV = c.num_kv_heads, D = c.head_dim;
            auto bytes = [&](NormPass pass, std::size_t rows, std::size_t width) {
                return rmsnorm_backward_sink_bytes(pass, rows, width, c.dtype);
            };
            const std::size_t heads = std::max(bytes(NormPass::with_rope, N * HQ, D) + bytes(NormPass::with_rope, N * HKV, D),
                                               bytes(NormPass::plain, N * HQ, D) + bytes(NormPass::plain, N * HKV, D));
            const std::size_t block = std::max(bytes(NormPass::dual, N, H), 2 * bytes(NormPass::plain, N, H));
            const std::size_t total = c.num_layers * (heads + block) + bytes(NormPass::plain, N, H);
            if (total != 0) {
                CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&m->norm_reductions.memory), total));
                m->norm_reductions.capacity = total;
            }
            m->norm_reduction_table_capacity = 4 * c.num_layers + 1;
            CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&m->norm_reduction_table),
                                m->norm_reduction_table_capacity * sizeof(ColumnReduceEntry)));
        }
        CGPTX_TRY(cgptx_adamw_workspace_create(&m->optimizer));
        std::vector<Parameter*> all;
        collect(m, all);
        for (Parameter* p : all)
            m->entries.push_back({p->value, p->gradient, p->master, p->first, p->second, p->count, c.dtype});
        return CGPTX_OK;
    };
    if (int s = build()) {
        const std::string message = cgptx_last_error();
        cgptx_model_destroy(m);
        return fail(s, message);
    }
    *out = m;
    return CGPTX_OK;
}

extern "C" int cgptx_model_set_tokens(cgptx_model* m, const uint32_t* inputs, const uint32_t* targets) {
    using namespace cgptx;
    if (m == nullptr || inputs == nullptr || targets == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "model_set_tokens: null argument");
    CGPTX_HIP(hipDeviceSynchronize());
    CGPTX_HIP(hipMemcpy(m->tokens, inputs, m->rows * sizeof(std::uint32_t), hipMemcpyHostToDevice));
    CGPTX_HIP(hipMemcpy(m->targets, targets, m->rows * sizeof(std::uint32_t), hipMemcpyHostToDevice));
    return CGPTX_OK;
}

// ---- token upload: two pinned host slots, one event each ------------------------------------------
struct cgptx_token_upload {
    std::size_t count = 0;                         // tokens per batch
    std::uint32_t* inputs[2] = {nullptr, nullptr};  // pinned
    std::uint32_t* targets[2] = {nullptr, nullptr};
    hipEvent_t copied[2] = {nullptr, nullptr};      // recorded after the copies out of a slot
    bool in_flight[2] = {false, false};
    int slot = 0;                                   // the one handed out by acquire
    bool acquired = false;
};

extern "C" int cgptx_token_upload_create(cgptx_token_upload** out, size_t batch, size_t sequence) {
    using namespace cgptx;
    clear_error();
    if (out == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "token_upload_create: null argument");
    if (batch != 0 && sequence > static_cast<std::size_t>(-1) / sizeof(std::uint32_t) / batch)
        return fail(CGPTX_OVERFLOW, "token_upload_create: batch size overflows");
    auto* u = new cgptx_token_upload();
    u->count = batch * sequence;
    const std::size_t bytes = std::max<std::size_t>(u->count, 1) * sizeof(std::uint32_t);
    int status = CGPTX_OK;
    for (int s = 0; s < 2 && status == CGPTX_OK; ++s) {
        // Allocated pinned (registering existing memory is not an option everywhere).
        status = check_hip(hipHostMalloc(reinterpret_cast<void**>(&u->inputs[s]), bytes, hipHostMallocDefault), "hipHostMalloc");
        if (status == CGPTX_OK)
            status = check_hip(hipHostMalloc(reinterpret_cast<void**>(&u->targets[s]), bytes, hipHostMallocDefault), "hipHostMalloc");
        if (status == CGPTX_OK) status = check_hip(hipEventCreateWithFlags(&u->copied[s], hipEventDisableTiming), "hipEventCreate");
    }
    if (status != CGPTX_OK) {
        cgptx_token_upload_destroy(u);
        return status;
    }
    *out = u;
    return CGPTX_OK;
}

extern "C" int cgptx_token_upload_destroy(cgptx_token_upload* u) {
    if (u == nullptr) return CGPTX_OK;
    for (int s = 0; s < 2; ++s) {
        if (u->copied[s] != nullptr) {
            if (u->in_flight[s]) (void)hipEventSynchronize(u->copied[s]);
            (void)hipEventDestroy(u->copied[s]);
        }
        if (u->inputs[s] != nullptr) (void)hipHostFree(u->inputs[s]);
        if (u->targets[s] != nullptr) (void)hipHostFree(u->targets[s]);
    }
    delete u;
    return CGPTX_OK;
}

extern "C" int cgptx_token_upload_acquire(cgptx_token_upload* u, uint32_t** inputs, uint32_t** targets) {
    using namespace cgptx;
    clear_error();
    if (u == nullptr || inputs == nullptr || targets == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "token_upload_acquire: null argument");
    // Batch::wait_until_reusable: the copies out of this slot, enqueued two submits ago, must be done
    // before the host writes it again.
    if (u->in_flight[u->slot]) {
        CGPTX_HIP(hipEventSynchronize(u->copied[u->slot]));
        u->in_flight[u->slot] = false;
    }
    *inputs = u->inputs[u->slot];
    *targets = u->targets[u->slot];
    u->acquired = true;
    return CGPTX_OK;
}

extern "C" int cgptx_token_upload_submit(cgptx_token_upload* u, uint32_t* device_inputs, uint32_t* device_targets,
                                         cgptx_stream stream_) {
    using namespace cgptx;
    clear_error();
    if (u == nullptr || device_inputs == nullptr || device_targets == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "token_upload_submit: null argument");
    if (!u->acquired) return fail(CGPTX_INVALID_ARGUMENT, "token_upload_submit: no slot was acquired");
    auto stream = static_cast<hipStream_t>(stream_);
    const std::size_t bytes = u->count * sizeof(std::uint32_t);
    if (bytes != 0) {
        CGPTX_HIP(hipMemcpyAsync(device_inputs, u->inputs[u->slot], bytes, hipMemcpyHostToDevice, stream));
        CGPTX_HIP(hipMemcpyAsync(device_targets, u->targets[u->slot], bytes, hipMemcpyHostToDevice, stream));
    }
    CGPTX_HIP(hipEventRecord(u->copied[u->slot], stream));  // Batch::mark_upload_complete
    u->in_flight[u->slot] = true;
    u->acquired = false;
    u->slot ^= 1;
    return CGPTX_OK;
}

extern "C" int cgptx_model_upload_tokens(cgptx_model* m, cgptx_token_upload* u, cgptx_stream stream) {
    using namespace cgptx;
    clear_error();
    if (m == nullptr || u == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_upload_tokens: null argument");
    if (u->count != m->rows)
        return fail(CGPTX_INVALID_ARGUMENT, "model_upload_tokens: batch buffers do not match the model's step shape");
    return cgptx_token_upload_submit(u, m->tokens, m->targets, stream);
}

// ---- caller-owned batches: pinned and device blocks, one fence per host batch ----------------------
struct cgptx_upload_fence {
    hipEvent_t copied = nullptr;
};

extern "C" int cgptx_pinned_allocate(void** block, size_t bytes) {
    using namespace cgptx;
    clear_error();
    if (block == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "pinned_allocate: null argument");
    *block = nullptr;
    CGPTX_HIP(hipHostMalloc(block, std::max<std::size_t>(bytes, 1), hipHostMallocDefault));
    return CGPTX_OK;
}

extern "C" int cgptx_pinned_release(void* block) {
    using namespace cgptx;
    clear_error();
    if (block != nullptr) CGPTX_HIP(hipHostFree(block));
    return CGPTX_OK;
}

extern "C" int cgptx_device_allocate(void** block, size_t bytes) {
    using namespace cgptx;
    clear_error();
    if (block == nullptr || bytes == 0) return fail(CGPTX_INVALID_ARGUMENT, "device_allocate: null argument or no bytes");
    *block = nullptr;
    CGPTX_HIP(hipMalloc(block, bytes));
    return CGPTX_OK;
}

extern "C" int cgptx_device_release(void* block) {
    using namespace cgptx;
    clear_error();
    if (block != nullptr) CGPTX_HIP(hipFree(block));
    return CGPTX_OK;
}

extern "C" int cgptx_upload_fence_wait(cgptx_upload_fence* fence) {
    using namespace cgptx;
    clear_error();
    if (fence != nullptr) CGPTX_HIP(hipEventSynchronize(fence->copied));
    return CGPTX_OK;
}

extern "C" int cgptx_upload_fence_destroy(cgptx_upload_fence* fence) {
    if (fence == nullptr) return CGPTX_OK;
    if (fence->copied != nullptr) (void)hipEventDestroy(fence->copied);
    delete fence;
    return CGPTX_OK;
}

extern "C" int cgptx_token_upload_async(uint32_t* device_inputs, uint32_t* device_targets, const uint32_t* inputs,
                                        const uint32_t* targets, size_t count, cgptx_upload_fence** fence,
                                        cgptx_stream stream_) {
    using namespace cgptx;
    clear_error();
    if (fence == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "token_upload_async: null fence slot");
    if (count != 0 && (device_inputs == nullptr || device_targets == nullptr || inputs == nullptr || targets == nullptr))
        return fail(CGPTX_INVALID_ARGUMENT, "token_upload_async: null buffer");
    if (count > static_cast<std::size_t>(-1) / sizeof(std::uint32_t))
        return fail(CGPTX_OVERFLOW, "token_upload_async: token count overflows");
    auto stream = static_cast<hipStream_t>(stream_);
    if (*fence == nullptr) {
        auto* created = new cgptx_upload_fence();
        if (int status = check_hip(hipEventCreateWithFlags(&created->copied, hipEventDisableTiming), "hipEventCreate")) {
            delete created;
            return status;
        }
        *fence = created;
    }
    const std::size_t bytes = count * sizeof(std::uint32_t);
    if (bytes != 0) {
        CGPTX_HIP(hipMemcpyAsync(device_inputs, inputs, bytes, hipMemcpyHostToDevice, stream));
        CGPTX_HIP(hipMemcpyAsync(device_targets, targets, bytes, hipMemcpyHostToDevice, stream));
    }
    CGPTX_HIP(hipEventRecord((*fence)->copied, stream));
    return CGPTX_OK;
}

namespace cgptx {
namespace {

// Forward + loss + backward and, with_optimizer, the three launches of the AdamW update behind them (its options
// are on the device already: adamw_set_options).
int enqueue_step(cgptx_model* m, float loss_scale, int loss_mode, bool with_optimizer, hipStream_t stream) {
    if (int s = enqueue_forward_backward(m, loss_scale, loss_mode, stream)) return s;
    if (!with_optimizer) return CGPTX_OK;
    return adamw_enqueue(m->optimizer, m->entries.data(), m->entries.size(), m->initial_step, stream);
}

int run_step(cgptx_model* m, float loss_scale, int loss_mode, int use_graph, bool with_optimizer, hipStream_t stream) {
    if (!std::isfinite(loss_scale) || loss_scale <= 0.0f)
        return fail(CGPTX_INVALID_ARGUMENT, "model_forward_backward: loss scale must be finite and positive");
    if (loss_mode != CGPTX_LOSS_DENSE && loss_mode != CGPTX_LOSS_CUT)
        return fail(CGPTX_INVALID_ARGUMENT, "model_forward_backward: unknown loss mode");
    if (loss_mode == CGPTX_LOSS_DENSE && m->logits == nullptr) {
        const std::size_t bytes = m->rows * m->config.vocabulary_size * dtype_size(m->config.dtype);
        if (int s = allocate(m, &m->logits, bytes)) return s;
        if (int s = allocate(m, &m->grad_logits, bytes)) return s;
    }
    if (!use_graph) return enqueue_step(m, loss_scale, loss_mode, with_optimizer, stream);
    if (stream == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "model_forward_backward: graph capture needs a non-default stream");
    cgptx_model::RecordedStep& step = m->recorded[with_optimizer ? 1 : 0];
    const bool have_graph = step.exec != nullptr && step.loss_scale == loss_scale && step.loss_mode == loss_mode &&
                            step.stream == stream &&
                            // The recorded kernels hold addresses inside the stream's scratch arena: a graph
                            // whose arena block has since been reallocated or released is recorded again.
                            step.scratch_generation == scratch_generation(stream);
    if (have_graph) {
        CGPTX_HIP(hipGraphLaunch(step.exec, stream));
        return CGPTX_OK;
    }
    // Eager run first: it sizes every scratch arena and does this call's work. Then record the
    // same sequence for the following calls.
    if (int s = enqueue_forward_backward(m, loss_scale, loss_mode, stream)) return s;
    if (m->norm_reductions_resized) {
        // The pass above sized the memory of the deferred norm reductions (and reduced at once): one more eager
        // pass records them and writes their table, which a capture cannot do.
        if (int s = enqueue_forward_backward(m, loss_scale, loss_mode, stream)) return s;
    }
    if (with_optimizer) {
        if (int s = adamw_enqueue(m->optimizer, m->entries.data(), m->entries.size(), m->initial_step, stream)) return s;
    }
    CGPTX_HIP(hipStreamSynchronize(stream));
    if (step.exec != nullptr) {
        CGPTX_HIP(hipGraphExecDestroy(step.exec));
        step.exec = nullptr;
    }
    CGPTX_HIP(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    const int status = enqueue_step(m, loss_scale, loss_mode, with_optimizer, stream);
    hipGraph_t graph = nullptr;
    const hipError_t end = hipStreamEndCapture(stream, &graph);
    if (status != CGPTX_OK) {
        if (graph != nullptr) (void)hipGraphDestroy(graph);
        return status;
    }
    CGPTX_HIP(end);
    const hipError_t inst = hipGraphInstantiate(&step.exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    CGPTX_HIP(inst);
    step.loss_scale = loss_scale;
    step.loss_mode = loss_mode;
    step.stream = stream;
    step.scratch_generation = scratch_generation(stream);
    return CGPTX_OK;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_model_forward_backward(cgptx_model* m, float loss_scale, int loss_mode, int use_graph,
                                            cgptx_stream stream_) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_forward_backward: null model");
    return run_step(m, loss_scale, loss_mode, use_graph, false, static_cast<hipStream_t>(stream_));
}

extern "C" int cgptx_model_optimizer_step(cgptx_model* m, const cgptx_adamw_options* options, cgptx_stream stream) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_optimizer_step: null model");
    return cgptx_adamw_step_many_async(m->optimizer, m->entries.data(), m->entries.size(), options, m->initial_step,
                                       stream);
}

// With use_graph the AdamW update is part of the recorded step: its options (the learning rate changes from step to
// step) are written to the device by one small launch ahead of the graph, and the update's kernels read them there.
extern "C" int cgptx_model_train_step(cgptx_model* m, const cgptx_adamw_options* options, int loss_mode,
                                      int use_graph, cgptx_stream stream_) {
    using namespace cgptx;
    if (m == nullptr || options == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_train_step: null argument");
    auto stream = static_cast<hipStream_t>(stream_);
    if (int s = adamw_bind(m->optimizer, m->entries.data(), m->entries.size(), m->initial_step, stream)) return s;
    if (int s = adamw_set_options(m->optimizer, options, stream)) return s;
    return run_step(m, options->loss_scale, loss_mode, use_graph, true, stream);
}

extern "C" int cgptx_model_status(cgptx_model* m, float* loss, int* all_finite, uint64_t* step,
                                  cgptx_stream stream_) {
    using namespace cgptx;
    if (m == nullptr || loss == nullptr || all_finite == nullptr || step == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "model_status: null argument");
    auto stream = static_cast<hipStream_t>(stream_);
    CGPTX_HIP(hipStreamSynchronize(stream));
    CGPTX_HIP(hipMemcpy(loss, m->loss, sizeof(float), hipMemcpyDeviceToHost));
    return cgptx_adamw_check(m->optimizer, all_finite, step, stream_);
}

extern "C" int cgptx_model_profile(cgptx_model* m, float loss_scale, int loss_mode, cgptx_stream stream_) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_profile: null model");
    auto stream = static_cast<hipStream_t>(stream_);
    if (int s = cgptx_model_forward_backward(m, loss_scale, loss_mode, 0, stream_)) return s;  // sizes scratch
    CGPTX_HIP(hipStreamSynchronize(stream));
    m->profiling = true;
    m->timed.clear();
    const int status = enqueue_forward_backward(m, loss_scale, loss_mode, stream);
    m->profiling = false;
    CGPTX_HIP(hipStreamSynchronize(stream));
    m->profile.clear();
    for (auto& t : m->timed) {
        float ms = 0.0f;
        if (status == CGPTX_OK) (void)hipEventElapsedTime(&ms, t.start, t.stop);
        (void)hipEventDestroy(t.start);
        (void)hipEventDestroy(t.stop);
        bool found = false;
        for (auto& entry : m->profile) {
            if (entry.first == t.label) {
                entry.second += ms;
                found = true;
            }
        }
        if (!found) m->profile.emplace_back(t.label, ms);
    }
    m->timed.clear();
    return status;
}

extern "C" int cgptx_model_record_calls(cgptx_model* m, int enable) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_record_calls: null model");
    m->recording_calls = enable != 0;
    if (!m->recording_calls) m->calls.clear();
    return CGPTX_OK;
}

extern "C" size_t cgptx_model_call_count(const cgptx_model* m) { return m == nullptr ? 0 : m->calls.size(); }

extern "C" int cgptx_model_call(const cgptx_model* m, size_t index, cgptx_call_record* record) {
    using namespace cgptx;
    if (m == nullptr || record == nullptr || index >= m->calls.size())
        return fail(CGPTX_INVALID_ARGUMENT, "model_call: null argument or index out of range");
    *record = m->calls[index];
    return CGPTX_OK;
}

extern "C" size_t cgptx_model_profile_count(const cgptx_model* m) { return m == nullptr ? 0 : m->profile.size(); }

extern "C" int cgptx_model_profile_entry(const cgptx_model* m, size_t index, const char** label, float* milliseconds) {
    using namespace cgptx;
    if (m == nullptr || index >= m->profile.size() || label == nullptr || milliseconds == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "model_profile_entry: index out of range");
    *label = m->profile[index].first.c_str();
    *milliseconds = m->profile[index].second;
    return CGPTX_OK;
}

extern "C" size_t cgptx_model_parameter_count(const cgptx_model* m) { return m == nullptr ? 0 : m->entries.size(); }

extern "C" int cgptx_model_parameter(const cgptx_model* m, size_t index, const char** name, void** parameter,
                                     void** gradient, size_t* count) {
    using namespace cgptx;
    if (m == nullptr || index >= m->entries.size())
        return fail(CGPTX_INVALID_ARGUMENT, "model_parameter: index out of range");
    std::vector<Parameter*> all;
    collect(const_cast<cgptx_model*>(m), all);
    if (name != nullptr) *name = all[index]->name.c_str();
    if (parameter != nullptr) *parameter = all[index]->value;
    if (gradient != nullptr) *gradient = all[index]->gradient;
    if (count != nullptr) *count = all[index]->count;
    return CGPTX_OK;
}

extern "C" int cgptx_model_describe(const cgptx_model* m, cgptx_model_config* config, size_t* batch, size_t* sequence) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_describe: null model");
    if (config != nullptr) *config = m->config;
    if (batch != nullptr) *batch = m->batch;
    if (sequence != nullptr) *sequence = m->sequence;
    return CGPTX_OK;
}

extern "C" int cgptx_model_optimizer_state(const cgptx_model* m, size_t index, float** master, float** first_moment,
                                           float** second_moment) {
    using namespace cgptx;
    if (m == nullptr || index >= m->entries.size())
        return fail(CGPTX_INVALID_ARGUMENT, "model_optimizer_state: index out of range");
    if (master != nullptr) *master = m->entries[index].master_parameter;
    if (first_moment != nullptr) *first_moment = m->entries[index].first_moment;
    if (second_moment != nullptr) *second_moment = m->entries[index].second_moment;
    return CGPTX_OK;
}

extern "C" int cgptx_model_set_optimizer_step(cgptx_model* m, uint64_t step) {
    using namespace cgptx;
    if (m == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_set_optimizer_step: null model");
    CGPTX_HIP(hipDeviceSynchronize());
    // The workspace reads its starting step when it is first used: a fresh one picks the new value up.
    if (int s = cgptx_adamw_workspace_destroy(m->optimizer)) return s;
    m->optimizer = nullptr;
    if (int s = cgptx_adamw_workspace_create(&m->optimizer)) return s;
    m->initial_step = step;
    return CGPTX_OK;
}

extern "C" size_t cgptx_model_num_parameters(const cgptx_model* m) {
    if (m == nullptr) return 0;
    size_t total = 0;
    for (const auto& e : m->entries) total += e.count;
    return total;
}

extern "C" int cgptx_model_activation(const cgptx_model* m, const char* name, void** data, size_t* count) {
    using namespace cgptx;
    if (m == nullptr || name == nullptr || data == nullptr || count == nullptr)
        return fail(CGPTX_INVALID_ARGUMENT, "model_activation: null argument");
    const std::string n(name);
    const std::size_t NH = m->rows * m->config.hidden_size;
    if (n == "normalized") { *data = m->normalized; *count = NH; return CGPTX_OK; }
    if (n == "loss") { *data = m->loss; *count = 1; return CGPTX_OK; }
    if (n == "rope.cos" || n == "rope.sin") {  // [sequence, rotary_dim / 2] in the storage dtype
        *data = n == "rope.cos" ? m->cos_cache : m->sin_cache;
        *count = m->sequence * (m->config.rotary_dim / 2);
        return CGPTX_OK;
    }
    if (n == "logits" && m->logits != nullptr) {
        *data = m->logits;
        *count = m->rows * m->config.vocabulary_size;
        return CGPTX_OK;
    }
    // Decimal index at [first, last) of the name; anything else is no index.
    auto index_at = [&](std::size_t first, std::size_t last, std::size_t* value) {
        const char* begin = n.data() + first;
        const char* end = n.data() + last;
        const auto parsed = std::from_chars(begin, end, *value);
        return first < last && parsed.ec == std::errc() && parsed.ptr == end;
    };
    if (n.rfind("hidden.", 0) == 0) {
        std::size_t l = 0;
        if (index_at(7, n.size(), &l) && l < m->hidden.size()) { *data = m->hidden[l]; *count = NH; return CGPTX_OK; }
    }
    // Gradient of the loss with respect to hidden.0 / hidden.1 as the last backward pass left them (the two
    // residual-stream gradient buffers alternate per block, so only the first block's pair survives a step).
    if (n == "grad.hidden.0" || n == "grad.hidden.1") {
        const bool even = m->config.num_layers % 2 == 0;  // d hidden[L] is in grad_a; each block switches buffers
        const bool in_a = (n == "grad.hidden.0") ? even : !even;
        *data = in_a ? m->grad_a : m->grad_b;
        *count = NH;
        return CGPTX_OK;
    }
    // Saved tensors of one block: "layer.<l>.<name>".
    if (n.rfind("layer.", 0) == 0) {
        const std::size_t dot = n.find('.', 6);
        if (dot != std::string::npos) {
            std::size_t l = m->acts.size();
            if (!index_at(6, dot, &l)) l = m->acts.size();
            const std::string what = n.substr(dot + 1);
            const auto& c = m->config;
            const std::size_t QW = m->rows * c.num_query_heads * c.head_dim, KW = m->rows * c.num_kv_heads * c.head_dim;
            const std::size_t NI = m->rows * c.intermediate_size;
            if (l < m->acts.size()) {
                const auto& a = m->acts[l];
                const struct { const char* name; void* ptr; std::size_t elements; } table[] = {
                    {"attention_norm_output", a.norm_a, NH}, {"query_pre_norm", a.q_pre, QW}, {"key_pre_norm", a.k_pre, KW},
                    {"query", a.q, QW}, {"key", a.k, KW}, {"value", a.v, KW}, {"attention_output", a.attn_out, QW},
                    {"logsumexp", a.lse, m->rows * c.num_query_heads}, {"ffn_norm_output", a.norm_f, NH},
                    {"gate_up", a.gate_up, 2 * NI}, {"activated", a.act, NI}};
                for (const auto& entry : table)
                    if (what == entry.name) { *data = entry.ptr; *count = entry.elements; return CGPTX_OK; }
            }
        }
    }
    return fail(CGPTX_INVALID_ARGUMENT, "model_activation: unknown activation " + n);
}
