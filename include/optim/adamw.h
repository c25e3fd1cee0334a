// AdamW with global gradient clipping and loss-scale handling — reference: include/optim/adamw.h:13-136.
// adamw_step_many_async enqueues one fused update over all entries (skipped as a whole when any
// gradient is non-finite); adamw_check synchronises, reports whether the step was applied and
// brings the host-side step counters up to date.
#pragma once

#include <cstdint>
#include <limits>
#include <span>
#include <vector>

#include "core/status.h"
#include "core/tensor.h"

struct AdamWOptions {
    float learning_rate = 1.0e-3f;
    float beta1 = 0.9f;
    float beta2 = 0.999f;
    float epsilon = 1.0e-8f;
    float weight_decay = 1.0e-2f;
    float loss_scale = 1.0f;
    float max_grad_norm = std::numeric_limits<float>::infinity();
};

struct AdamWState {
    Tensor master_parameter;  // F32 copy of the stored parameter
    Tensor first_moment;
    Tensor second_moment;
    std::uint64_t step = 0;

    // Moments zero, master = the stored parameter widened to F32 (host round trip: set-up path).
    [[nodiscard]] static AdamWState for_parameter(const Tensor& parameter, hipStream_t stream = nullptr);
};

struct AdamWBatchEntry {
    Tensor* parameter = nullptr;
    const Tensor* gradient = nullptr;
    AdamWState* state = nullptr;
};

class AdamWWorkspace {
public:
    AdamWWorkspace() { cgptx_detail::check(cgptx_adamw_workspace_create(&handle_)); }
    AdamWWorkspace(const AdamWWorkspace&) = delete;
    AdamWWorkspace& operator=(const AdamWWorkspace&) = delete;
    AdamWWorkspace(AdamWWorkspace&& other) noexcept : handle_(other.handle_), states_(std::move(other.states_)) {
        other.handle_ = nullptr;
    }
    AdamWWorkspace& operator=(AdamWWorkspace&& other) noexcept {
        if (this != &other) {
            if (handle_ != nullptr) (void)cgptx_adamw_workspace_destroy(handle_);
            handle_ = other.handle_;
            states_ = std::move(other.states_);
            other.handle_ = nullptr;
        }
        return *this;
    }
    ~AdamWWorkspace() {
        if (handle_ != nullptr) (void)cgptx_adamw_workspace_destroy(handle_);
    }

private:
    friend void adamw_step_many_async(std::span<const AdamWBatchEntry>, const AdamWOptions&, AdamWWorkspace&, hipStream_t);
    friend bool adamw_check(AdamWWorkspace&, hipStream_t);
    cgptx_adamw_workspace* handle_ = nullptr;
    std::vector<AdamWState*> states_;
};

namespace cgptx_detail {
inline cgptx_adamw_options adamw_options(const AdamWOptions& o) {
    return {o.learning_rate, o.beta1, o.beta2, o.epsilon, o.weight_decay, o.loss_scale, o.max_grad_norm};
}
inline void validate_adamw_entry(const Tensor& parameter, const Tensor& gradient, const AdamWState& state) {
    require_device("adamw", {&parameter, &gradient, &state.master_parameter, &state.first_moment, &state.second_moment});
    if (gradient.dtype() != parameter.dtype() || gradient.numel() != parameter.numel() ||
        state.master_parameter.dtype() != Dtype::F32 || state.first_moment.dtype() != Dtype::F32 ||
        state.second_moment.dtype() != Dtype::F32 || state.master_parameter.numel() != parameter.numel() ||
        state.first_moment.numel() != parameter.numel() || state.second_moment.numel() != parameter.numel())
        throw std::invalid_argument("adamw: parameter, gradient and state do not match");
}
}  // namespace cgptx_detail

inline AdamWState AdamWState::for_parameter(const Tensor& parameter, hipStream_t stream) {
    if (parameter.device_type() != DeviceType::GPU) throw std::invalid_argument("AdamWState: parameter must live on the GPU");
    if (stream != nullptr && hipStreamSynchronize(stream) != hipSuccess) throw std::runtime_error("AdamWState: sync failed");
    AdamWState state;
    state.master_parameter = Tensor(parameter.shape(), DeviceType::GPU, Dtype::F32);
    state.first_moment = Tensor::zeros(parameter.shape(), DeviceType::GPU, stream, Dtype::F32);
    state.second_moment = Tensor::zeros(parameter.shape(), DeviceType::GPU, stream, Dtype::F32);
    const std::size_t count = parameter.numel();
    std::vector<std::uint8_t> raw(parameter.nbytes());
    parameter.copy_raw_to_host(raw);
    std::vector<float> wide(count);
    if (parameter.dtype() == Dtype::F32) {
        std::memcpy(wide.data(), raw.data(), raw.size());
    } else {
        const auto* bits = reinterpret_cast<const std::uint16_t*>(raw.data());
        for (std::size_t i = 0; i < count; ++i) {
            if (parameter.dtype() == Dtype::BF16) {
                const std::uint32_t word = static_cast<std::uint32_t>(bits[i]) << 16;
                std::memcpy(&wide[i], &word, 4);
            } else {
                wide[i] = cgptx_detail::half_bits_to_float(bits[i]);
            }
        }
    }
    state.master_parameter.copy_raw_from_host({reinterpret_cast<const std::uint8_t*>(wide.data()), count * sizeof(float)});
    return state;
}

inline void adamw_step_many_async(std::span<const AdamWBatchEntry> entries, const AdamWOptions& options,
                                  AdamWWorkspace& workspace, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    if (entries.empty()) throw std::invalid_argument("adamw_step_many_async: no entries");
    std::vector<cgptx_adamw_entry> raw;
    raw.reserve(entries.size());
    workspace.states_.clear();
    const std::uint64_t step = entries.front().state != nullptr ? entries.front().state->step : 0;
    for (const AdamWBatchEntry& e : entries) {
        if (e.parameter == nullptr || e.gradient == nullptr || e.state == nullptr)
            throw std::invalid_argument("adamw_step_many_async: null entry member");
        validate_adamw_entry(*e.parameter, *e.gradient, *e.state);
        if (e.state->step != step) throw std::invalid_argument("adamw_step_many_async: all states must be at the same step");
        raw.push_back({e.parameter->raw_data(), e.gradient->raw_data(), static_cast<float*>(e.state->master_parameter.raw_data()),
                       static_cast<float*>(e.state->first_moment.raw_data()),
                       static_cast<float*>(e.state->second_moment.raw_data()), e.parameter->numel(),
                       dtype_code(e.parameter->dtype())});
        workspace.states_.push_back(e.state);
    }
    const cgptx_adamw_options native = adamw_options(options);
    check(cgptx_adamw_step_many_async(workspace.handle_, raw.data(), raw.size(), &native, step, stream));
}

[[nodiscard]] inline bool adamw_check(AdamWWorkspace& workspace, hipStream_t stream = nullptr) {
    int all_finite = 0;
    std::uint64_t step = 0;
    cgptx_detail::check(cgptx_adamw_check(workspace.handle_, &all_finite, &step, stream));
    for (AdamWState* state : workspace.states_) state->step = step;
    return all_finite != 0;
}

[[nodiscard]] inline bool adamw_step(Tensor& parameter, const Tensor& gradient, AdamWState& state,
                                     const AdamWOptions& options = {}, hipStream_t stream = nullptr) {
    using namespace cgptx_detail;
    validate_adamw_entry(parameter, gradient, state);
    const cgptx_adamw_options native = adamw_options(options);
    int updated = 0;
    check(cgptx_adamw_step(parameter.raw_data(), gradient.raw_data(), static_cast<float*>(state.master_parameter.raw_data()),
                           static_cast<float*>(state.first_moment.raw_data()),
                           static_cast<float*>(state.second_moment.raw_data()), parameter.numel(),
                           dtype_code(parameter.dtype()), &native, state.step + 1, &updated, stream));
    if (updated != 0) ++state.step;
    return updated != 0;
}
