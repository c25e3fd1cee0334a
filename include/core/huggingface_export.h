// Checkpoints with the reference's names (include/core/huggingface_export.h →
// src/core/huggingface_export.cpp:135-158 config.json, 345-380 export, 400-430 load), over a model
// handle instead of a weight structure; the tokenizer files are not written. File problems throw
// std::runtime_error as there.
#pragma once

#include <cstddef>
#include <cstdint>
#include <filesystem>
#include <stdexcept>
#include <string>

#include "cgptx_train.h"

namespace cgptx_detail {
inline void check_io(const int status) {
    if (status == CGPTX_OK) return;
    const std::string message = cgptx_last_error();
    if (status == CGPTX_INVALID_ARGUMENT) throw std::invalid_argument(message);
    if (status == CGPTX_OVERFLOW) throw std::overflow_error(message);
    throw std::runtime_error(message);
}
}  // namespace cgptx_detail

/** Writes `config.json` and `model.safetensors` into `output_directory` (created if missing). */
inline void export_huggingface_model(const std::filesystem::path& output_directory, const cgptx_model* model,
                                     const std::size_t max_position_embeddings) {
    std::filesystem::create_directories(output_directory);
    cgptx_detail::check_io(cgptx_model_save_checkpoint(model, output_directory.string().c_str(), max_position_embeddings));
}

/** Loads `model.safetensors` from `input_directory` into the model's weights. */
inline void load_huggingface_model(const std::filesystem::path& input_directory, cgptx_model* model) {
    cgptx_detail::check_io(cgptx_model_load_checkpoint(model, input_directory.string().c_str()));
}

/** AdamW state (fp32 masters, moments, step), which the reference does not save. */
inline void save_optimizer_state(const std::filesystem::path& path, const cgptx_model* model, const std::uint64_t step) {
    cgptx_detail::check_io(cgptx_model_save_optimizer(model, path.string().c_str(), step));
}
inline std::uint64_t load_optimizer_state(const std::filesystem::path& path, cgptx_model* model) {
    std::uint64_t step = 0;
    cgptx_detail::check_io(cgptx_model_load_optimizer(model, path.string().c_str(), &step));
    return step;
}
