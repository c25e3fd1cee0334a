// A caller shaped like the reference's transformer_block_backward (src/core/transformer_block.cu:644-748),
// written against include/ only: the same operator functions in the same order with the same argument
// order, the metadata-only reshapes of saved tensors through const_cast, the accumulate flags, and the
// block's own residual helper. It runs on the tensors a library step saved (a two-layer model stepped with
// CGPTX_FUSE=0, i.e. as the reference's call sequence), eagerly and from a HipGraph capture
// (include/core/hip_graph.h, the counterpart of the CudaGraph that train/train.cpp:536-548 uses), and every
// gradient it produces must equal the library step's bit for bit.
// Built with hipcc by __graft_entry__.build(); run by tests/test_cpp_interface.py on the GPU.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "cgptx_train.h"
#include "core/hip_graph.h"
#include "ops/backward/attention_backward.h"
#include "ops/backward/linear_backward.h"
#include "ops/backward/rmsnorm_backward.h"
#include "ops/backward/rope_backward.h"
#include "ops/backward/swiglu_backward.h"
#include "ops/rmsnorm.h"

namespace {

// The reference's option and workspace structs for one block (include/core/transformer_block.h), reduced to
// the members transformer_block_backward touches.
struct TransformerBlockOptions {
    std::size_t hidden_size, intermediate_size, num_query_heads, num_kv_heads, head_dim, rotary_dim;
    float rms_epsilon;
    bool causal = true;
    struct { ComputeType compute_type = ComputeType::F32; std::size_t workspace_bytes = 32ULL << 20; } linear_options;
};
struct TransformerBlockWeights {
    const Tensor &attention_norm, &q_projection, &k_projection, &q_norm, &k_norm, &v_projection, &o_projection, &ffn_norm,
        &gate_proj, &up_proj, &down_proj;
};
struct TransformerBlockGradients {
    Tensor &attention_norm, &q_projection, &k_projection, &q_norm, &k_norm, &v_projection, &o_projection, &ffn_norm,
        &gate_proj, &up_proj, &down_proj;
};
struct TransformerBlockWorkspace {
    Tensor norm, query_pre_norm, key_pre_norm, query, key, value, attention_output, attention_logsumexp, gate, up, activated;
};
struct TransformerBlockBackwardWorkspace {
    Tensor grad_activated, grad_gate, grad_up, grad_ffn_norm_input, grad_residual, grad_attention_projection,
        grad_attention_output, grad_query, grad_key, grad_value, grad_query_pre_rope, grad_key_pre_rope,
        attention_norm_output, grad_attention_norm_input, hidden_bias, intermediate_bias, kv_bias;
};

void check_hip(hipError_t status, const char* what) {
    if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
}

// a += b, the block's residual helper (src/core/transformer_block.cu:134-144).
void add_inplace(Tensor& a, const Tensor& b, hipStream_t stream) {
    cgptx_detail::check(cgptx_add(a.raw_data(), a.raw_data(), b.raw_data(), a.numel(), cgptx_detail::dtype_code(a.dtype()), stream));
}

void transformer_block_backward(Tensor& grad_input, const Tensor& grad_output, const Tensor& input,
                                const TransformerBlockWeights& weights, const TransformerBlockGradients gradients,
                                const TransformerBlockWorkspace& forward_workspace, TransformerBlockBackwardWorkspace& backward,
                                const Tensor& cos_cache, const Tensor& sin_cache, const GemmContext& gemm_context,
                                hipStream_t stream, const TransformerBlockOptions& options, const std::size_t position_offset) {
    if (input.shape() != grad_output.shape() || grad_input.shape() != input.shape() || input.dim() != 2)
        throw std::invalid_argument("transformer block backward: invalid input or output gradient");
    const std::size_t rows = input.size(0), hidden = options.hidden_size;
    const std::size_t batch = forward_workspace.query.size(0), sequence = forward_workspace.query.size(1);

    LinearBackwardOptions linear_options{options.linear_options.compute_type, options.linear_options.workspace_bytes};
    linear_backward(backward.grad_activated, gradients.down_proj, backward.hidden_bias, grad_output,
                    forward_workspace.activated, weights.down_proj, gemm_context, stream, linear_options);
    swiglu_backward(backward.grad_gate, backward.grad_up, backward.grad_activated, forward_workspace.gate,
                    forward_workspace.up, stream);
    linear_backward(backward.grad_ffn_norm_input, gradients.gate_proj, backward.intermediate_bias, backward.grad_gate,
                    forward_workspace.norm, weights.gate_proj, gemm_context, stream, linear_options);
    linear_options.accumulate_input = true;
    linear_backward(backward.grad_ffn_norm_input, gradients.up_proj, backward.intermediate_bias, backward.grad_up,
                    forward_workspace.norm, weights.up_proj, gemm_context, stream, linear_options);
    linear_options.accumulate_input = false;

    rmsnorm_backward(backward.grad_residual, gradients.ffn_norm, backward.grad_ffn_norm_input, input, weights.ffn_norm,
                     options.rms_epsilon, stream);

    check_hip(hipMemcpyAsync(grad_input.raw_data(), grad_output.raw_data(), grad_output.nbytes(), hipMemcpyDeviceToDevice, stream),
              "hipMemcpyAsync");
    add_inplace(grad_input, backward.grad_residual, stream);
    check_hip(hipMemcpyAsync(backward.grad_attention_projection.raw_data(), grad_output.raw_data(), grad_output.nbytes(),
                             hipMemcpyDeviceToDevice, stream),
              "hipMemcpyAsync");

    backward.grad_attention_output.reshape({rows, hidden});
    auto& saved_attention_output = const_cast<Tensor&>(forward_workspace.attention_output);
    saved_attention_output.reshape({rows, hidden});
    linear_backward(backward.grad_attention_output, gradients.o_projection, backward.hidden_bias,
                    backward.grad_attention_projection, saved_attention_output, weights.o_projection, gemm_context, stream,
                    linear_options);
    saved_attention_output.reshape({batch, sequence, options.num_query_heads, options.head_dim});
    backward.grad_attention_output.reshape({batch, sequence, options.num_query_heads, options.head_dim});
    FlashAttentionOptions attention_options{};
    attention_options.num_query_heads = options.num_query_heads;
    attention_options.num_kv_heads = options.num_kv_heads;
    attention_options.head_dim = options.head_dim;
    attention_options.causal = options.causal;
    attention_options.query_position_offset = position_offset;
    flash_gqa_attention_backward_with_lse(backward.grad_query, backward.grad_key, backward.grad_value,
                                          backward.grad_attention_output, forward_workspace.attention_output,
                                          forward_workspace.attention_logsumexp, forward_workspace.query, forward_workspace.key,
                                          forward_workspace.value, stream, attention_options);
    rope_backward(backward.grad_query_pre_rope, backward.grad_key_pre_rope, backward.grad_query, backward.grad_key, cos_cache,
                  sin_cache, stream, RopeOptions{options.rotary_dim, position_offset});

    backward.grad_query_pre_rope.reshape({batch * sequence * options.num_query_heads, options.head_dim});
    backward.grad_query.reshape({batch * sequence * options.num_query_heads, options.head_dim});
    auto& saved_query_pre_norm = const_cast<Tensor&>(forward_workspace.query_pre_norm);
    saved_query_pre_norm.reshape({batch * sequence * options.num_query_heads, options.head_dim});
    rmsnorm_backward(backward.grad_query, gradients.q_norm, backward.grad_query_pre_rope, saved_query_pre_norm, weights.q_norm,
                     options.rms_epsilon, stream);
    backward.grad_key_pre_rope.reshape({batch * sequence * options.num_kv_heads, options.head_dim});
    backward.grad_key.reshape({batch * sequence * options.num_kv_heads, options.head_dim});
    auto& saved_key_pre_norm = const_cast<Tensor&>(forward_workspace.key_pre_norm);
    saved_key_pre_norm.reshape({batch * sequence * options.num_kv_heads, options.head_dim});
    rmsnorm_backward(backward.grad_key, gradients.k_norm, backward.grad_key_pre_rope, saved_key_pre_norm, weights.k_norm,
                     options.rms_epsilon, stream);
    saved_query_pre_norm.reshape({batch, sequence, options.num_query_heads, options.head_dim});
    saved_key_pre_norm.reshape({batch, sequence, options.num_kv_heads, options.head_dim});

    rmsnorm_forward(backward.attention_norm_output, input, weights.attention_norm, options.rms_epsilon, stream);
    backward.grad_query.reshape({rows, options.num_query_heads * options.head_dim});
    backward.grad_key.reshape({rows, options.num_kv_heads * options.head_dim});
    backward.grad_value.reshape({rows, options.num_kv_heads * options.head_dim});
    linear_backward(backward.grad_attention_norm_input, gradients.q_projection, backward.hidden_bias, backward.grad_query,
                    backward.attention_norm_output, weights.q_projection, gemm_context, stream, linear_options);
    linear_options.accumulate_input = true;
    linear_backward(backward.grad_attention_norm_input, gradients.k_projection, backward.kv_bias, backward.grad_key,
                    backward.attention_norm_output, weights.k_projection, gemm_context, stream, linear_options);
    linear_backward(backward.grad_attention_norm_input, gradients.v_projection, backward.kv_bias, backward.grad_value,
                    backward.attention_norm_output, weights.v_projection, gemm_context, stream, linear_options);
    linear_options.accumulate_input = false;
    backward.grad_query_pre_rope.reshape({batch, sequence, options.num_query_heads, options.head_dim});
    backward.grad_key_pre_rope.reshape({batch, sequence, options.num_kv_heads, options.head_dim});
    backward.grad_value.reshape({batch, sequence, options.num_kv_heads, options.head_dim});
    backward.grad_query.reshape({batch, sequence, options.num_query_heads, options.head_dim});
    backward.grad_key.reshape({batch, sequence, options.num_kv_heads, options.head_dim});
    rmsnorm_backward(backward.grad_residual, gradients.attention_norm, backward.grad_attention_norm_input, input,
                     weights.attention_norm, options.rms_epsilon, stream);
    add_inplace(grad_input, backward.grad_residual, stream);
}

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
std::vector<std::uint8_t> bytes_of(const void* device, std::size_t bytes) {
    std::vector<std::uint8_t> host(bytes);
    check_hip(hipMemcpy(host.data(), device, bytes, hipMemcpyDeviceToHost), "hipMemcpy");
    return host;
}

}  // namespace

int main() {
    try {
        setenv("CGPTX_FUSE", "0", 1);  // the library step as the reference's call sequence
        constexpr std::size_t B = 2, T = 48, L = 2, H = 256, I = 512, HQ = 4, HKV = 2, D = 64, V = 512, N = B * T;
        constexpr Dtype dtype = Dtype::BF16;
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
        ok(cgptx_model_forward_backward(model, 64.0f, CGPTX_LOSS_DENSE, 0, stream), "forward_backward");
        check_hip(hipStreamSynchronize(stream), "sync");

        // The first block's weights and the gradients the library step computed for them.
        std::map<std::string, std::pair<void*, std::vector<std::uint8_t>>> parameters;  // short name -> (weight, gradient bytes)
        const std::string prefix = "model.layers.0.";
        for (std::size_t i = 0; i < cgptx_model_parameter_count(model); ++i) {
            const char* name = nullptr;
            void *value = nullptr, *gradient = nullptr;
            std::size_t count = 0;
            ok(cgptx_model_parameter(model, i, &name, &value, &gradient, &count), "model_parameter");
            const std::string full(name);
            if (full.rfind(prefix, 0) == 0) parameters[full.substr(prefix.size())] = {value, bytes_of(gradient, count * 2)};
        }
        auto named = [&](const char* name, std::vector<std::size_t> shape, Dtype t = dtype) {
            void* data = nullptr;
            std::size_t count = 0;
            ok(cgptx_model_activation(model, name, &data, &count), name);
            Tensor view = Tensor::device_view(std::move(shape), data, t);
            if (view.numel() != count) throw std::runtime_error(std::string(name) + ": unexpected size");
            return view;
        };
        auto weight = [&](const char* name, std::vector<std::size_t> shape) {
            return Tensor::device_view(std::move(shape), parameters.at(name).first, dtype);
        };
        const Tensor input = named("hidden.0", {N, H}), grad_output = named("grad.hidden.1", {N, H});
        const std::vector<std::uint8_t> want_grad_input = bytes_of(named("grad.hidden.0", {N, H}).raw_data(), N * H * 2);
        const Tensor cos_cache = named("rope.cos", {T, D / 2}), sin_cache = named("rope.sin", {T, D / 2});
        Tensor gate_up = named("layer.0.gate_up", {2, N, I});  // CGPTX_FUSE=0: [gate; up], each [N, I]
        TransformerBlockWorkspace forward{
            named("layer.0.ffn_norm_output", {N, H}),
            named("layer.0.query_pre_norm", {B, T, HQ, D}),
            named("layer.0.key_pre_norm", {B, T, HKV, D}),
            named("layer.0.query", {B, T, HQ, D}),
            named("layer.0.key", {B, T, HKV, D}),
            named("layer.0.value", {B, T, HKV, D}),
            named("layer.0.attention_output", {B, T, HQ, D}),
            named("layer.0.logsumexp", {B, T, HQ}, Dtype::F32),
            Tensor::device_view({N, I}, gate_up.raw_data(), dtype),
            Tensor::device_view({N, I}, static_cast<char*>(gate_up.raw_data()) + N * I * 2, dtype),
            named("layer.0.activated", {N, I})};
        const Tensor w_attention_norm = weight("input_layernorm.weight", {H}), w_q = weight("self_attn.q_proj.weight", {HQ * D, H}),
                     w_k = weight("self_attn.k_proj.weight", {HKV * D, H}), w_q_norm = weight("self_attn.q_norm.weight", {D}),
                     w_k_norm = weight("self_attn.k_norm.weight", {D}), w_v = weight("self_attn.v_proj.weight", {HKV * D, H}),
                     w_o = weight("self_attn.o_proj.weight", {H, HQ * D}), w_ffn_norm = weight("post_attention_layernorm.weight", {H}),
                     w_gate = weight("mlp.gate_proj.weight", {I, H}), w_up = weight("mlp.up_proj.weight", {I, H}),
                     w_down = weight("mlp.down_proj.weight", {H, I});
        const TransformerBlockWeights weights{w_attention_norm, w_q, w_k, w_q_norm, w_k_norm, w_v, w_o, w_ffn_norm, w_gate, w_up, w_down};
        auto fresh = [&](std::vector<std::size_t> shape) { return Tensor(std::move(shape), dtype); };
        Tensor g_attention_norm = fresh({H}), g_q = fresh({HQ * D, H}), g_k = fresh({HKV * D, H}), g_q_norm = fresh({D}),
               g_k_norm = fresh({D}), g_v = fresh({HKV * D, H}), g_o = fresh({H, HQ * D}), g_ffn_norm = fresh({H}),
               g_gate = fresh({I, H}), g_up = fresh({I, H}), g_down = fresh({H, I});
        const TransformerBlockGradients gradients{g_attention_norm, g_q, g_k, g_q_norm, g_k_norm, g_v, g_o, g_ffn_norm, g_gate, g_up, g_down};
        TransformerBlockBackwardWorkspace backward{
            fresh({N, I}), fresh({N, I}), fresh({N, I}), fresh({N, H}), fresh({N, H}), fresh({N, H}),
            fresh({B, T, HQ, D}), fresh({B, T, HQ, D}), fresh({B, T, HKV, D}), fresh({B, T, HKV, D}),
            fresh({B, T, HQ, D}), fresh({B, T, HKV, D}), fresh({N, H}), fresh({N, H}), fresh({H}), fresh({I}), fresh({HKV * D})};
        Tensor grad_input = fresh({N, H});
        const TransformerBlockOptions options{H, I, HQ, HKV, D, D, 1e-5f};
        const GemmContext gemm_context;
        const std::map<std::string, Tensor*> produced = {
            {"input_layernorm.weight", &g_attention_norm}, {"self_attn.q_proj.weight", &g_q}, {"self_attn.k_proj.weight", &g_k},
            {"self_attn.q_norm.weight", &g_q_norm}, {"self_attn.k_norm.weight", &g_k_norm}, {"self_attn.v_proj.weight", &g_v},
            {"self_attn.o_proj.weight", &g_o}, {"post_attention_layernorm.weight", &g_ffn_norm}, {"mlp.gate_proj.weight", &g_gate},
            {"mlp.up_proj.weight", &g_up}, {"mlp.down_proj.weight", &g_down}};
        auto clear_outputs = [&] {
            for (const auto& [name, tensor] : produced) check_hip(hipMemset(tensor->raw_data(), 0xFF, tensor->nbytes()), "hipMemset");
            check_hip(hipMemset(grad_input.raw_data(), 0xFF, grad_input.nbytes()), "hipMemset");
        };
        auto compare = [&](const char* pass) {
            check_hip(hipStreamSynchronize(stream), "sync");
            for (const auto& [name, tensor] : produced)
                expect(bytes_of(tensor->raw_data(), tensor->nbytes()) == parameters.at(name).second,
                       std::string(pass) + ": gradient of " + name + " differs from the library step");
            expect(bytes_of(grad_input.raw_data(), grad_input.nbytes()) == want_grad_input,
                   std::string(pass) + ": grad_input differs from the library step");
        };
        auto run = [&] {
            transformer_block_backward(grad_input, grad_output, input, weights, gradients, forward, backward, cos_cache, sin_cache,
                                       gemm_context, stream, options, 0);
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
