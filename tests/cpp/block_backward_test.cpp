// Callers of include/ops/** get the library's results: two proofs against the headers only.
//
// (1) Compile-time: every operator wrapper is invocable with exactly the argument lists the reference's
//     block and model code pass (src/core/transformer_block.cu:466-595, 663-747, src/core/transformer_model.cu:
//     360-380): outputs, inputs, GEMM context, stream, options; defaults for the trailing ones; const saved
//     tensors reshaped in place through const_cast and passed on as const references.
// (2) Run-time: the library reports the operator calls of its own step when that step runs as the reference's
//     call sequence (CGPTX_FUSE=0, cgptx_model_record_calls). This program walks that table and makes every
//     call through the C++ wrapper of that operator, on Tensor views of the same buffers with all results
//     overwritten beforehand — eagerly, and from a HipGraph capture (include/core/hip_graph.h, the counterpart
//     of the CudaGraph train/train.cpp:536-548 uses). Every gradient must equal the library step's bit for bit.
// Built with hipcc by __graft_entry__.build(); run by tests/test_cpp_interface.py on the GPU.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "cgptx_train.h"
#include "core/hip_graph.h"
#include "ops/attention.h"
#include "ops/backward/attention_backward.h"
#include "ops/backward/embedding_backward.h"
#include "ops/backward/linear_backward.h"
#include "ops/backward/rmsnorm_backward.h"
#include "ops/backward/rope_backward.h"
#include "ops/backward/swiglu_backward.h"
#include "ops/cross_entropy.h"
#include "ops/cut_cross_entropy.h"
#include "ops/embedding.h"
#include "ops/linear.h"
#include "ops/rmsnorm.h"
#include "ops/rope.h"
#include "ops/swiglu.h"

namespace {

// ---- (1) argument lists -------------------------------------------------------------------------
using T = Tensor&;
using CT = const Tensor&;
using Ids = const bpe::TokenId*;
template <typename... Args>
using op = void (*)(Args...);
// Backward operators as the block calls them: with the stream and options, and with the defaults.
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, T, CT, CT, CT, const GemmContext&, hipStream_t,
                                                           const LinearBackwardOptions&>>(linear_backward)),
                                  T, T, T, CT, CT, CT, const GemmContext&, hipStream_t, const LinearBackwardOptions&>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, CT, CT, CT, float, hipStream_t>>(rmsnorm_backward)), T, T, CT, CT,
                                  CT, float, hipStream_t>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, CT, CT, CT, hipStream_t, const SwiGLUBackwardOptions&>>(swiglu_backward)),
                                  T, T, CT, CT, CT, hipStream_t, const SwiGLUBackwardOptions&>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, CT, CT, hipStream_t, const SwiGLUBackwardOptions&>>(swiglu_backward)), T,
                                  CT, CT, hipStream_t, const SwiGLUBackwardOptions&>);  // concatenated gate_up overload
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, CT, CT, CT, CT, hipStream_t, const RopeOptions&>>(rope_backward)), T,
                                  T, CT, CT, CT, CT, hipStream_t, RopeOptions>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, T, CT, CT, CT, CT, CT, CT, hipStream_t, const FlashAttentionOptions&,
                                                           bool>>(flash_gqa_attention_backward_with_lse)),
                                  T, T, T, CT, CT, CT, CT, CT, CT, hipStream_t, const FlashAttentionOptions&, bool>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, T, CT, CT, CT, CT, hipStream_t, const FlashAttentionOptions&, bool>>(
                                      flash_gqa_attention_backward)),
                                  T, T, T, CT, CT, CT, CT, hipStream_t, const FlashAttentionOptions&, bool>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, CT, Ids, std::size_t, hipStream_t, const EmbeddingBackwardOptions&>>(
                                      embedding_backward)),
                                  T, CT, Ids, std::size_t, hipStream_t, EmbeddingBackwardOptions>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, CT, Ids, std::size_t, hipStream_t, float>>(cross_entropy_forward_backward)),
                                  T, T, CT, Ids, std::size_t, hipStream_t, float>);
static_assert(std::is_invocable_v<decltype(static_cast<op<T, T, T, CT, CT, Ids, std::size_t, hipStream_t>>(
                                      cut_cross_entropy_forward_backward)),
                                  T, T, T, CT, CT, Ids, std::size_t, hipStream_t>);
// Trailing defaults: the stream, the options and the accumulate flag may be left out, as the reference's tests do.
template <typename... Args>
constexpr bool callable_linear_backward = requires(Args... a) { linear_backward(a...); };
static_assert(callable_linear_backward<T, T, T, CT, CT, CT, const GemmContext&>);
static_assert(callable_linear_backward<T, T, T, CT, CT, CT, const GemmContext&, hipStream_t>);
static_assert(requires(T a, CT b, float e) { rmsnorm_backward(a, a, b, b, b, e); });
static_assert(requires(T a, CT b) { swiglu_backward(a, a, b, b, b); });
static_assert(requires(T a, CT b) { rope_backward(a, a, b, b, b, b); });
static_assert(requires(T a, CT b) { flash_gqa_attention_backward_with_lse(a, a, a, b, b, b, b, b, b); });
static_assert(requires(T a, CT b, Ids ids) { embedding_backward(a, b, ids, std::size_t{1}); });
static_assert(requires(T a, CT b, Ids ids) { cross_entropy_forward_backward(a, a, b, ids, std::size_t{1}); });
// Option structs carry the reference's fields with its defaults (include/ops/backward/*.h, include/ops/attention.h).
static_assert(LinearBackwardOptions{}.compute_type == ComputeType::F32 && LinearBackwardOptions{}.workspace_bytes == (32ULL << 20) &&
              !LinearBackwardOptions{}.accumulate_input && !LinearBackwardOptions{}.accumulate_weight &&
              !LinearBackwardOptions{}.accumulate_bias);
static_assert(!SwiGLUBackwardOptions{}.accumulate_gate && !SwiGLUBackwardOptions{}.accumulate_up &&
              !SwiGLUBackwardOptions{}.accumulate_gate_up);
static_assert(EmbeddingBackwardOptions{}.bounds_check && !EmbeddingBackwardOptions{}.accumulate_weight);
static_assert(FlashAttentionOptions{}.causal && FlashAttentionOptions{}.attention_scale == 0.0F &&
              FlashAttentionOptions{}.query_position_offset == 0);
static_assert(RopeOptions{}.rotary_dim == 0 && RopeOptions{}.position_offset == 0);
// A saved (const) tensor is reshaped in place through const_cast and handed on as a const reference; reshape is
// metadata-only, so the view keeps its buffer.
static_assert(requires(const Tensor& saved) { const_cast<Tensor&>(saved).reshape({std::size_t{1}, std::size_t{1}}); });

// ---- (2) the call table, walked through the wrappers ---------------------------------------------
int failures = 0;
void expect(bool ok, const std::string& what) {
    if (!ok) {
        ++failures;
        std::printf("FAIL %s\n", what.c_str());
    }
}
void ok(int status, const char* what) {
    if (status != CGPTX_OK) throw std::runtime_error(std::string(what) + ": " + cgptx_last_error());
}
void check_hip(hipError_t status, const char* what) {
    if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
}
std::vector<std::uint8_t> bytes_of(const void* device, std::size_t bytes) {
    std::vector<std::uint8_t> host(bytes);
    check_hip(hipMemcpy(host.data(), device, bytes, hipMemcpyDeviceToHost), "hipMemcpy");
    return host;
}

struct Caller {
    hipStream_t stream;
    GemmContext gemm_context;
    std::map<std::size_t, Tensor> bias_scratch;  // linear_backward's bias gradient, which the block throws away

    static Dtype dtype_of(const cgptx_call_record& r) { return r.dtype == CGPTX_F16 ? Dtype::F16 : (r.dtype == CGPTX_BF16 ? Dtype::BF16 : Dtype::F32); }
    static Tensor view(const cgptx_call_record& r, int index, std::vector<std::size_t> shape) {
        return Tensor::device_view(std::move(shape), const_cast<void*>(r.tensors[index]), dtype_of(r));
    }
    static Tensor view_f32(const cgptx_call_record& r, int index, std::vector<std::size_t> shape) {
        return Tensor::device_view(std::move(shape), const_cast<void*>(r.tensors[index]), Dtype::F32);
    }
    static Ids ids(const cgptx_call_record& r, int index) { return static_cast<Ids>(r.tensors[index]); }

    void call(const cgptx_call_record& r) {
        const std::string name(r.op);
        const auto* d = r.dims;
        if (name == "embedding_forward") {
            Tensor out = view(r, 0, {d[0], d[2]});
            embedding_forward(out, ids(r, 1), d[0], view(r, 2, {d[1], d[2]}), stream);
        } else if (name == "rmsnorm_forward") {
            Tensor out = view(r, 0, {d[0], d[1]});
            rmsnorm_forward(out, view(r, 1, {d[0], d[1]}), view(r, 2, {d[1]}), r.scalar, stream);
        } else if (name == "linear_forward") {
            Tensor out = view(r, 0, {d[0], d[2]});
            linear_forward(out, view(r, 1, {d[0], d[1]}), view(r, 2, {d[2], d[1]}), gemm_context, stream);
        } else if (name == "rope_forward") {
            Tensor q = view(r, 0, {d[0], d[1], d[2], d[4]}), k = view(r, 1, {d[0], d[1], d[3], d[4]});
            rope_forward(q, k, view(r, 2, {d[7], d[5] / 2}), view(r, 3, {d[7], d[5] / 2}), stream, RopeOptions{d[5], d[6]});
        } else if (name == "flash_gqa_attention_forward_with_lse") {
            Tensor out = view(r, 0, {d[0], d[1], d[3], d[5]}), lse = view_f32(r, 1, {d[0], d[1], d[3]});
            flash_gqa_attention_forward_with_lse(out, lse, view(r, 2, {d[0], d[1], d[3], d[5]}), view(r, 3, {d[0], d[2], d[4], d[5]}),
                                                 view(r, 4, {d[0], d[2], d[4], d[5]}), stream, attention_options(r));
        } else if (name == "swiglu_forward") {
            Tensor out = view(r, 0, {d[0]});
            swiglu_forward(out, view(r, 1, {d[0]}), view(r, 2, {d[0]}), stream);
        } else if (name == "add") {  // the block's own residual helper, not an operator of include/ops
            ok(cgptx_add(const_cast<void*>(r.tensors[0]), r.tensors[1], r.tensors[2], d[0], r.dtype, stream), "add");
        } else if (name == "cross_entropy_forward_backward") {
            Tensor loss = view_f32(r, 0, {1}), gradient = view(r, 1, {d[0], d[1]});
            cross_entropy_forward_backward(loss, gradient, view(r, 2, {d[0], d[1]}), ids(r, 3), d[0], stream, r.scalar);
        } else if (name == "cut_cross_entropy_forward_backward") {
            if (r.scalar != 1.0f) throw std::runtime_error("cut_cross_entropy_forward_backward takes no gradient scale");
            Tensor loss = view_f32(r, 0, {1}), dx = view(r, 1, {d[0], d[1]}), dc = view(r, 2, {d[2], d[1]});
            cut_cross_entropy_forward_backward(loss, dx, dc, view(r, 3, {d[0], d[1]}), view(r, 4, {d[2], d[1]}), ids(r, 5), d[0], stream);
        } else if (name == "linear_backward") {
            Tensor dx = view(r, 0, {d[0], d[1]}), dw = view(r, 1, {d[2], d[1]});
            auto found = bias_scratch.find(d[2]);
            if (found == bias_scratch.end()) found = bias_scratch.emplace(d[2], Tensor({d[2]}, dtype_of(r))).first;
            LinearBackwardOptions options;
            options.accumulate_input = r.flags[0] != 0;
            linear_backward(dx, dw, found->second, view(r, 2, {d[0], d[2]}), view(r, 3, {d[0], d[1]}), view(r, 4, {d[2], d[1]}),
                            gemm_context, stream, options);
        } else if (name == "rmsnorm_backward") {
            Tensor dx = view(r, 0, {d[0], d[1]}), dw = view(r, 1, {d[1]});
            // The saved input is const for the caller and reshaped in place before the call, as the block does
            // with its q / k tensors before their per-head norm gradients.
            const Tensor saved = view(r, 3, {d[0] * d[1]});
            const_cast<Tensor&>(saved).reshape({d[0], d[1]});
            rmsnorm_backward(dx, dw, view(r, 2, {d[0], d[1]}), saved, view(r, 4, {d[1]}), r.scalar, stream);
        } else if (name == "swiglu_backward") {
            Tensor dg = view(r, 0, {d[0]}), du = view(r, 1, {d[0]});
            SwiGLUBackwardOptions options;
            options.accumulate_gate = r.flags[0] != 0;
            options.accumulate_up = r.flags[1] != 0;
            swiglu_backward(dg, du, view(r, 2, {d[0]}), view(r, 3, {d[0]}), view(r, 4, {d[0]}), stream, options);
        } else if (name == "flash_gqa_attention_backward_with_lse") {
            Tensor dq = view(r, 0, {d[0], d[1], d[3], d[5]}), dk = view(r, 1, {d[0], d[2], d[4], d[5]}),
                   dv = view(r, 2, {d[0], d[2], d[4], d[5]});
            flash_gqa_attention_backward_with_lse(dq, dk, dv, view(r, 3, {d[0], d[1], d[3], d[5]}), view(r, 4, {d[0], d[1], d[3], d[5]}),
                                                  view_f32(r, 5, {d[0], d[1], d[3]}), view(r, 6, {d[0], d[1], d[3], d[5]}),
                                                  view(r, 7, {d[0], d[2], d[4], d[5]}), view(r, 8, {d[0], d[2], d[4], d[5]}), stream,
                                                  attention_options(r), r.flags[1] != 0);
        } else if (name == "rope_backward") {
            Tensor dq = view(r, 0, {d[0], d[1], d[2], d[4]}), dk = view(r, 1, {d[0], d[1], d[3], d[4]});
            rope_backward(dq, dk, view(r, 2, {d[0], d[1], d[2], d[4]}), view(r, 3, {d[0], d[1], d[3], d[4]}),
                          view(r, 4, {d[7], d[5] / 2}), view(r, 5, {d[7], d[5] / 2}), stream, RopeOptions{d[5], d[6]});
        } else if (name == "embedding_backward") {
            Tensor dw = view(r, 0, {d[1], d[2]});
            EmbeddingBackwardOptions options;
            options.bounds_check = r.flags[0] != 0;
            options.accumulate_weight = r.flags[1] != 0;
            embedding_backward(dw, view(r, 1, {d[0], d[2]}), ids(r, 2), d[0], stream, options);
        } else {
            throw std::runtime_error("call table names an operator this caller does not know: " + name);
        }
    }
    static FlashAttentionOptions attention_options(const cgptx_call_record& r) {
        FlashAttentionOptions o{};
        o.num_query_heads = r.dims[3];
        o.num_kv_heads = r.dims[4];
        o.head_dim = r.dims[5];
        o.attention_scale = r.scalar;
        o.causal = r.flags[0] != 0;
        o.query_position_offset = r.dims[6];
        return o;
    }
};

}  // namespace

int main() {
    try {
        setenv("CGPTX_FUSE", "0", 1);  // the library step as the reference's call sequence
        constexpr std::size_t B = 2, T = 48, L = 2, H = 256, I = 512, HQ = 4, HKV = 2, D = 64, V = 512, N = B * T;
        cgptx_model_config config{};
        config.vocabulary_size = V;
        config.num_layers = L;
        config.hidden_size = H;
        config.intermediate_size = I;
        config.num_query_heads = HQ;
        config.num_kv_heads = HKV;
        config.head_dim = D;
        config.rotary_dim = D;
        config.rms_epsilon = 1e-5f;
        config.rope_base = 10000.0f;
        config.dtype = CGPTX_BF16;
        cgptx_model* model = nullptr;
        ok(cgptx_model_create(&model, &config, B, T, 11), "model_create");
        std::vector<std::uint32_t> tokens(N), targets(N);
        for (std::size_t i = 0; i < N; ++i) {
            tokens[i] = static_cast<std::uint32_t>((i * 37 + 11) % V);
            targets[i] = static_cast<std::uint32_t>((i * 101 + 5) % V);
        }
        ok(cgptx_model_set_tokens(model, tokens.data(), targets.data()), "set_tokens");
        hipStream_t stream = nullptr;
        check_hip(hipStreamCreate(&stream), "hipStreamCreate");
        ok(cgptx_model_record_calls(model, 1), "record_calls");
        ok(cgptx_model_forward_backward(model, 64.0f, CGPTX_LOSS_DENSE, 0, stream), "forward_backward");
        check_hip(hipStreamSynchronize(stream), "sync");

        // What the library step left: every parameter gradient, the gradient of the first hidden state, the loss.
        struct Result {
            std::string name;
            void* device;
            std::vector<std::uint8_t> want;
        };
        std::vector<Result> results;
        for (std::size_t i = 0; i < cgptx_model_parameter_count(model); ++i) {
            const char* name = nullptr;
            void *value = nullptr, *gradient = nullptr;
            std::size_t count = 0;
            ok(cgptx_model_parameter(model, i, &name, &value, &gradient, &count), "model_parameter");
            results.push_back({std::string("gradient of ") + name, gradient, bytes_of(gradient, count * 2)});
        }
        for (const char* name : {"grad.hidden.0", "loss"}) {
            void* data = nullptr;
            std::size_t count = 0;
            ok(cgptx_model_activation(model, name, &data, &count), name);
            const std::size_t bytes = std::string(name) == "loss" ? sizeof(float) : count * 2;
            results.push_back({name, data, bytes_of(data, bytes)});
        }

        std::vector<cgptx_call_record> table(cgptx_model_call_count(model));
        for (std::size_t i = 0; i < table.size(); ++i) ok(cgptx_model_call(model, i, &table[i]), "model_call");
        std::map<std::string, int> seen;
        for (const auto& r : table) ++seen[r.op];
        // Per block the reference makes 7 linear_backward calls (down, gate, up, o, q, k, v) and 4 norm gradients;
        // the model adds the classifier's and the final norm's.
        expect(seen["linear_backward"] == 7 * L + 1 && seen["rmsnorm_backward"] == 4 * L + 1 &&
                   seen["flash_gqa_attention_backward_with_lse"] == L && seen["rope_backward"] == L && seen["swiglu_backward"] == L &&
                   seen["embedding_backward"] == 1 && seen["cross_entropy_forward_backward"] == 1,
               "the call table holds the reference's backward calls");

        Caller caller{stream, GemmContext{}, {}};
        auto run = [&] {
            for (const auto& r : table) caller.call(r);
        };
        auto clear_outputs = [&] {
            for (const auto& r : results) check_hip(hipMemset(r.device, 0xFF, r.want.size()), "hipMemset");
        };
        auto compare = [&](const char* pass) {
            check_hip(hipStreamSynchronize(stream), "sync");
            for (const auto& r : results)
                expect(bytes_of(r.device, r.want.size()) == r.want, std::string(pass) + ": " + r.name + " differs from the library step");
        };

        clear_outputs();
        run();  // eager: also gives every operator its scratch memory
        compare("eager");

        HipGraph graph;
        graph.capture(stream, run);
        expect(graph.initialized(), "HipGraph::initialized after capture");
        for (int replay = 0; replay < 2; ++replay) {
            clear_outputs();
            graph.launch(stream);
            compare(replay == 0 ? "first graph replay" : "second graph replay");
        }

        // CudaGraph's error behaviour (src/core/cuda_graph.cu:86-146, 160-185).
        HipGraph empty;
        bool threw = false;
        try { empty.launch(stream); } catch (const std::logic_error&) { threw = true; }
        expect(threw, "launch without a graph throws std::logic_error");
        threw = false;
        try { empty.capture(stream, {}); } catch (const std::invalid_argument&) { threw = true; }
        expect(threw, "capture with an empty callback throws std::invalid_argument");
        threw = false;
        try { empty.capture(nullptr, [] {}); } catch (const std::invalid_argument&) { threw = true; }
        expect(threw, "capture on the null stream throws std::invalid_argument");
        threw = false;
        try { empty.instantiate(nullptr); } catch (const std::invalid_argument&) { threw = true; }
        expect(threw, "instantiate(nullptr) throws std::invalid_argument");
        threw = false;
        try { empty.capture(stream, [] { throw std::domain_error("from the callback"); }); } catch (const std::domain_error&) { threw = true; }
        expect(threw, "an exception from the capture callback is passed on");
        hipStreamCaptureStatus status = hipStreamCaptureStatusActive;
        check_hip(hipStreamIsCapturing(stream, &status), "hipStreamIsCapturing");
        expect(status == hipStreamCaptureStatusNone, "capture is ended after the callback threw");
        HipGraph moved = std::move(graph);
        expect(moved.initialized() && !graph.initialized(), "move leaves the source empty");
        clear_outputs();
        moved.launch(stream);
        compare("moved graph");

        // Typed host copies round to nearest even into the storage dtype and widen back exactly.
        Tensor half_tensor({4}, Dtype::F16), bf_tensor({4}, Dtype::BF16);
        const std::vector<float> values = {1.0f, -2.5f, 0.333333343f, 65504.0f};
        half_tensor.copy_from_host(values);
        bf_tensor.copy_from_host(values);
        std::vector<float> back(4);
        half_tensor.copy_to_host(back);
        expect(back[0] == 1.0f && back[1] == -2.5f && back[2] == 0.333251953125f && back[3] == 65504.0f, "F16 host copies");
        bf_tensor.copy_to_host(back);
        expect(back[0] == 1.0f && back[1] == -2.5f && back[2] == 0.333984375f && back[3] == 65536.0f, "BF16 host copies");
        const Tensor copy = bf_tensor;  // deep copy
        expect(copy.raw_data() != bf_tensor.raw_data() && copy.shape() == bf_tensor.shape(), "copy construction is deep");

        ok(cgptx_model_destroy(model), "model_destroy");
        check_hip(hipStreamDestroy(stream), "hipStreamDestroy");
    } catch (const std::exception& error) {
        std::printf("FAIL exception: %s\n", error.what());
        ++failures;
    }
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}
