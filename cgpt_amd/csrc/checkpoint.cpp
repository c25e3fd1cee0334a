// Checkpoints of a model in the safetensors container, written against the public C-ABI only.
//
// Weights: `config.json` + `model.safetensors` with the tensor names, order, dtypes and config keys
// of the reference exporter (src/core/huggingface_export.cpp:135-158 write_config, 180-225
// write_safetensors, 362-378 the tensor list), so that either side reads the other's files; the
// tokenizer files the reference writes next to them are not produced here. The q/k/v and gate/up
// weights, which this model keeps in shared blocks, are written as the separate tensors of that list.
// Optimizer state (which the reference does not save): `<name>.master`, `<name>.exp_avg`,
// `<name>.exp_avg_sq` in fp32 plus the step counter, in a second safetensors file.
//
// File layout (safetensors): little-endian u64 header size, JSON header
// {"name":{"dtype":..,"shape":[..],"data_offsets":[begin,end]},...} padded with spaces to a
// multiple of 8, then the tensors' bytes. The reader takes any header of that grammar (keys in any
// order, a "__metadata__" object), not only the writer's own.
#include "common.hpp"
#include "cgptx_train.h"

#include <cstdint>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

namespace cgptx {
namespace {

struct Entry {
    std::string name;
    std::string dtype;
    std::vector<std::size_t> shape;
    const void* device = nullptr;  // source (writer)
    std::size_t bytes = 0;
    std::size_t begin = 0, end = 0;  // data offsets
};

const char* safetensors_dtype(int dtype) {
    switch (dtype) {
        case CGPTX_F16: return "F16";
        case CGPTX_BF16: return "BF16";
        case CGPTX_F32: return "F32";
        default: return nullptr;
    }
}

std::string json_string(const std::string& value) {
    std::string out = "\"";
    for (const char c : value) {
        switch (c) {
            case '"': out += "\\\""; break;
            case '\\': out += "\\\\"; break;
            case '\n': out += "\\n"; break;
            case '\r': out += "\\r"; break;
            case '\t': out += "\\t"; break;
            default: out += c; break;
        }
    }
    return out + "\"";
}

bool ends_with(const std::string& text, const std::string& suffix) {
    return text.size() >= suffix.size() && text.compare(text.size() - suffix.size(), suffix.size(), suffix) == 0;
}

// Shape of a parameter from its checkpoint name: [out, in] for projections, [V, H] for the
// embedding, [n] for norm weights.
std::vector<std::size_t> shape_of(const std::string& name, const cgptx_model_config& c, std::size_t count) {
    const std::size_t H = c.hidden_size, I = c.intermediate_size;
    const std::size_t QW = c.num_query_heads * c.head_dim, KW = c.num_kv_heads * c.head_dim;
    std::vector<std::size_t> shape;
    if (ends_with(name, "embed_tokens.weight") || name == "lm_head.weight") shape = {c.vocabulary_size, H};
    else if (ends_with(name, "q_proj.weight")) shape = {QW, H};
    else if (ends_with(name, "k_proj.weight") || ends_with(name, "v_proj.weight")) shape = {KW, H};
    else if (ends_with(name, "o_proj.weight")) shape = {H, QW};
    else if (ends_with(name, "gate_proj.weight") || ends_with(name, "up_proj.weight")) shape = {I, H};
    else if (ends_with(name, "down_proj.weight")) shape = {H, I};
    else shape = {count};
    std::size_t product = 1;
    for (const std::size_t d : shape) product *= d;
    if (product != count) shape = {count};
    return shape;
}

int write_file(const std::string& path, std::vector<Entry>& entries) {
    std::size_t offset = 0;
    for (Entry& e : entries) {
        if (e.bytes > static_cast<std::size_t>(-1) - offset) return fail(CGPTX_OVERFLOW, "checkpoint: offsets overflow");
        e.begin = offset;
        e.end = offset + e.bytes;
        offset = e.end;
    }
    std::ostringstream header;
    header << '{';
    for (std::size_t i = 0; i < entries.size(); ++i) {
        const Entry& e = entries[i];
        if (i != 0) header << ',';
        header << json_string(e.name) << ":{\"dtype\":" << json_string(e.dtype) << ",\"shape\":[";
        for (std::size_t d = 0; d < e.shape.size(); ++d) header << (d ? "," : "") << e.shape[d];
        header << "],\"data_offsets\":[" << e.begin << ',' << e.end << "]}";
    }
    header << '}';
    std::string text = header.str();
    while (text.size() % 8 != 0) text.push_back(' ');
    std::ofstream out(path, std::ios::binary);
    if (!out) return fail(CGPTX_RUNTIME, "checkpoint: cannot create " + path);
    const std::uint64_t size = text.size();
    out.write(reinterpret_cast<const char*>(&size), sizeof(size));
    out.write(text.data(), static_cast<std::streamsize>(text.size()));
    std::vector<char> host;
    for (const Entry& e : entries) {
        host.resize(e.bytes);
        if (e.bytes != 0) CGPTX_HIP(hipMemcpy(host.data(), e.device, e.bytes, hipMemcpyDeviceToHost));
        out.write(host.data(), static_cast<std::streamsize>(e.bytes));
    }
    out.flush();
    if (!out) return fail(CGPTX_RUNTIME, "checkpoint: cannot write " + path);
    return CGPTX_OK;
}

// ---- reader: a JSON parser for the header grammar ------------------------------------------------
struct Parser {
    const std::string& text;
    std::size_t at = 0;
    bool ok = true;

    void skip() {
        while (at < text.size() && (text[at] == ' ' || text[at] == '\n' || text[at] == '\r' || text[at] == '\t')) ++at;
    }
    bool take(char c) {
        skip();
        if (at < text.size() && text[at] == c) {
            ++at;
            return true;
        }
        return false;
    }
    std::string string() {
        std::string out;
        if (!take('"')) {
            ok = false;
            return out;
        }
        while (at < text.size() && text[at] != '"') {
            if (text[at] == '\\' && at + 1 < text.size()) {
                const char c = text[++at];
                out += c == 'n' ? '\n' : c == 'r' ? '\r' : c == 't' ? '\t' : c;
            } else {
                out += text[at];
            }
            ++at;
        }
        if (at >= text.size()) ok = false;
        ++at;
        return out;
    }
    std::size_t number() {
        skip();
        if (at >= text.size() || text[at] < '0' || text[at] > '9') {
            ok = false;
            return 0;
        }
        std::size_t value = 0;
        while (at < text.size() && text[at] >= '0' && text[at] <= '9') value = value * 10 + static_cast<std::size_t>(text[at++] - '0');
        return value;
    }
    std::vector<std::size_t> numbers() {
        std::vector<std::size_t> out;
        if (!take('[')) {
            ok = false;
            return out;
        }
        if (take(']')) return out;
        do out.push_back(number());
        while (ok && take(','));
        if (!take(']')) ok = false;
        return out;
    }
    // Skips any JSON value (for keys the reader has no use for).
    void skip_value() {
        skip();
        if (at >= text.size()) {
            ok = false;
            return;
        }
        const char c = text[at];
        if (c == '"') {
            string();
        } else if (c == '{' || c == '[') {
            const char close = c == '{' ? '}' : ']';
            ++at;
            if (take(close)) return;
            do {
                if (c == '{') {
                    string();
                    if (!take(':')) ok = false;
                }
                skip_value();
            } while (ok && take(','));
            if (!take(close)) ok = false;
        } else {
            while (at < text.size() && text[at] != ',' && text[at] != '}' && text[at] != ']') ++at;
        }
    }
};

int read_header(const std::string& path, std::ifstream& in, std::map<std::string, Entry>& entries, std::size_t& data_begin) {
    in.open(path, std::ios::binary);
    if (!in) return fail(CGPTX_RUNTIME, "checkpoint: cannot open " + path);
    std::uint64_t size = 0;
    in.read(reinterpret_cast<char*>(&size), sizeof(size));
    in.seekg(0, std::ios::end);
    const std::uint64_t file_size = static_cast<std::uint64_t>(in.tellg());
    if (!in || size == 0 || size > file_size - sizeof(size)) return fail(CGPTX_RUNTIME, "checkpoint: invalid header in " + path);
    std::string text(size, '\0');
    in.seekg(sizeof(size));
    in.read(text.data(), static_cast<std::streamsize>(size));
    if (!in) return fail(CGPTX_RUNTIME, "checkpoint: invalid header in " + path);
    data_begin = sizeof(size) + size;
    Parser p{text};
    if (!p.take('{')) return fail(CGPTX_RUNTIME, "checkpoint: invalid header in " + path);
    if (!p.take('}')) {
        do {
            const std::string name = p.string();
            if (!p.take(':')) p.ok = false;
            if (name == "__metadata__") {
                p.skip_value();
                continue;
            }
            Entry e;
            e.name = name;
            if (!p.take('{')) p.ok = false;
            do {
                const std::string key = p.string();
                if (!p.take(':')) p.ok = false;
                if (key == "dtype") e.dtype = p.string();
                else if (key == "shape") e.shape = p.numbers();
                else if (key == "data_offsets") {
                    const std::vector<std::size_t> offsets = p.numbers();
                    if (offsets.size() != 2 || offsets[1] < offsets[0]) p.ok = false;
                    else {
                        e.begin = offsets[0];
                        e.end = offsets[1];
                    }
                } else p.skip_value();
            } while (p.ok && p.take(','));
            if (!p.take('}')) p.ok = false;
            if (p.ok && e.end > file_size - data_begin) p.ok = false;
            entries[name] = e;
        } while (p.ok && p.take(','));
        if (!p.take('}')) p.ok = false;
    }
    if (!p.ok) return fail(CGPTX_RUNTIME, "checkpoint: invalid header in " + path);
    return CGPTX_OK;
}

int read_tensor(std::ifstream& in, std::size_t data_begin, const std::map<std::string, Entry>& entries,
                const std::string& name, const char* dtype, const std::vector<std::size_t>& shape, std::size_t bytes,
                std::vector<char>& host) {
    const auto found = entries.find(name);
    if (found == entries.end()) return fail(CGPTX_RUNTIME, "checkpoint: missing tensor " + name);
    const Entry& e = found->second;
    if (e.dtype != dtype) return fail(CGPTX_RUNTIME, "checkpoint: dtype mismatch for tensor " + name);
    if (e.shape != shape) return fail(CGPTX_RUNTIME, "checkpoint: shape mismatch for tensor " + name);
    if (e.end - e.begin != bytes) return fail(CGPTX_RUNTIME, "checkpoint: byte size mismatch for tensor " + name);
    host.resize(bytes);
    in.clear();
    in.seekg(static_cast<std::streamoff>(data_begin + e.begin));
    in.read(host.data(), static_cast<std::streamsize>(bytes));
    if (!in) return fail(CGPTX_RUNTIME, "checkpoint: cannot read tensor " + name);
    return CGPTX_OK;
}

float half_to_float(std::uint16_t h) {
    const std::uint32_t sign = static_cast<std::uint32_t>(h & 0x8000u) << 16;
    std::uint32_t exponent = (h >> 10) & 0x1Fu, mantissa = h & 0x3FFu, bits;
    if (exponent == 0) {
        if (mantissa == 0) {
            bits = sign;
        } else {
            int shift = 0;
            while ((mantissa & 0x400u) == 0) {
                mantissa <<= 1;
                ++shift;
            }
            bits = sign | static_cast<std::uint32_t>(113 - shift) << 23 | (mantissa & 0x3FFu) << 13;
        }
    } else if (exponent == 31) {
        bits = sign | 0x7F800000u | mantissa << 13;
    } else {
        bits = sign | (exponent + 112) << 23 | mantissa << 13;
    }
    float out;
    std::memcpy(&out, &bits, sizeof(out));
    return out;
}

// fp32 copy of `count` stored elements (what the optimizer keeps as master weights).
void widen(const std::vector<char>& stored, int dtype, std::size_t count, std::vector<float>& out) {
    out.resize(count);
    if (dtype == CGPTX_F32) {
        std::memcpy(out.data(), stored.data(), count * sizeof(float));
        return;
    }
    const auto* bits = reinterpret_cast<const std::uint16_t*>(stored.data());
    for (std::size_t i = 0; i < count; ++i) {
        if (dtype == CGPTX_BF16) {
            const std::uint32_t wide = static_cast<std::uint32_t>(bits[i]) << 16;
            std::memcpy(&out[i], &wide, sizeof(float));
        } else {
            out[i] = half_to_float(bits[i]);
        }
    }
}

struct Named {
    std::string name;
    void* value;
    std::size_t count;
    std::size_t index;
};

int parameters_of(const cgptx_model* model, std::vector<Named>& out) {
    const std::size_t n = cgptx_model_parameter_count(model);
    for (std::size_t i = 0; i < n; ++i) {
        const char* name = nullptr;
        void* value = nullptr;
        std::size_t count = 0;
        if (int s = cgptx_model_parameter(model, i, &name, &value, nullptr, &count)) return s;
        out.push_back({name, value, count, i});
    }
    return CGPTX_OK;
}

}  // namespace
}  // namespace cgptx

extern "C" int cgptx_model_save_checkpoint(const cgptx_model* model, const char* directory, size_t max_position_embeddings) {
    using namespace cgptx;
    clear_error();
    if (model == nullptr || directory == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_save_checkpoint: null argument");
    cgptx_model_config c{};
    if (int s = cgptx_model_describe(model, &c, nullptr, nullptr)) return s;
    const char* dtype = safetensors_dtype(c.dtype);
    if (dtype == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_save_checkpoint: unsupported dtype");
    CGPTX_HIP(hipDeviceSynchronize());
    const std::string base = std::string(directory) + "/";
    {
        std::ofstream config(base + "config.json");
        if (!config) return fail(CGPTX_RUNTIME, "checkpoint: cannot create " + base + "config.json");
        config.precision(9);
        config << "{\n"
               << "  \"architectures\": [\"CGPTForCausalLM\"],\n"
               << "  \"model_type\": \"cgpt\",\n"
               << "  \"torch_dtype\": \"" << (c.dtype == CGPTX_BF16 ? "bfloat16" : c.dtype == CGPTX_F16 ? "float16" : "float32") << "\",\n"
               << "  \"vocab_size\": " << c.vocabulary_size << ",\n"
               << "  \"hidden_size\": " << c.hidden_size << ",\n"
               << "  \"intermediate_size\": " << c.intermediate_size << ",\n"
               << "  \"num_hidden_layers\": " << c.num_layers << ",\n"
               << "  \"num_attention_heads\": " << c.num_query_heads << ",\n"
               << "  \"num_key_value_heads\": " << c.num_kv_heads << ",\n"
               << "  \"head_dim\": " << c.head_dim << ",\n"
               << "  \"max_position_embeddings\": " << max_position_embeddings << ",\n"
               << "  \"rms_norm_eps\": " << c.rms_epsilon << ",\n"
               << "  \"rope_theta\": " << std::fixed << c.rope_base << std::defaultfloat << ",\n"
               << "  \"use_parallel_residual\": true,\n"
               << "  \"tie_word_embeddings\": true\n"
               << "}\n";
        if (!config) return fail(CGPTX_RUNTIME, "checkpoint: cannot write " + base + "config.json");
    }
    std::vector<Named> parameters;
    if (int s = parameters_of(model, parameters)) return s;
    std::vector<Entry> entries;
    const std::size_t elem = c.dtype == CGPTX_F32 ? 4 : 2;
    for (const Named& p : parameters) {
        entries.push_back({p.name, dtype, shape_of(p.name, c, p.count), p.value, p.count * elem, 0, 0});
        // The reference's list has the (tied) classifier third, after the embedding and the final norm.
        if (p.name == "model.norm.weight") {
            const Named& embedding = parameters.front();
            entries.push_back({"lm_head.weight", dtype, shape_of("lm_head.weight", c, embedding.count), embedding.value,
                               embedding.count * elem, 0, 0});
        }
    }
    return write_file(base + "model.safetensors", entries);
}

extern "C" int cgptx_model_load_checkpoint(cgptx_model* model, const char* directory) {
    using namespace cgptx;
    clear_error();
    if (model == nullptr || directory == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_load_checkpoint: null argument");
    cgptx_model_config c{};
    if (int s = cgptx_model_describe(model, &c, nullptr, nullptr)) return s;
    const char* dtype = safetensors_dtype(c.dtype);
    if (dtype == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_load_checkpoint: unsupported dtype");
    std::ifstream in;
    std::map<std::string, Entry> entries;
    std::size_t data_begin = 0;
    if (int s = read_header(std::string(directory) + "/model.safetensors", in, entries, data_begin)) return s;
    std::vector<Named> parameters;
    if (int s = parameters_of(model, parameters)) return s;
    const std::size_t elem = c.dtype == CGPTX_F32 ? 4 : 2;
    CGPTX_HIP(hipDeviceSynchronize());
    std::vector<char> host;
    std::vector<float> wide;
    for (const Named& p : parameters) {
        if (int s = read_tensor(in, data_begin, entries, p.name, dtype, shape_of(p.name, c, p.count), p.count * elem, host)) return s;
        CGPTX_HIP(hipMemcpy(p.value, host.data(), host.size(), hipMemcpyHostToDevice));
        // The optimizer updates fp32 master copies: they restart from the loaded values.
        float* master = nullptr;
        if (int s = cgptx_model_optimizer_state(model, p.index, &master, nullptr, nullptr)) return s;
        if (master != nullptr) {
            widen(host, c.dtype, p.count, wide);
            CGPTX_HIP(hipMemcpy(master, wide.data(), wide.size() * sizeof(float), hipMemcpyHostToDevice));
        }
    }
    return CGPTX_OK;
}

extern "C" int cgptx_model_save_optimizer(const cgptx_model* model, const char* path, uint64_t step) {
    using namespace cgptx;
    clear_error();
    if (model == nullptr || path == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_save_optimizer: null argument");
    cgptx_model_config c{};
    if (int s = cgptx_model_describe(model, &c, nullptr, nullptr)) return s;
    CGPTX_HIP(hipDeviceSynchronize());
    std::vector<Named> parameters;
    if (int s = parameters_of(model, parameters)) return s;
    // The step counter travels as a one-element tensor at the front; its bytes come from a device
    // copy so that every entry is written the same way.
    std::uint64_t* device_step = nullptr;
    CGPTX_HIP(hipMalloc(reinterpret_cast<void**>(&device_step), sizeof(std::uint64_t)));
    int status = check_hip(hipMemcpy(device_step, &step, sizeof(step), hipMemcpyHostToDevice), "hipMemcpy");
    std::vector<Entry> entries;
    entries.push_back({"step", "U64", {1}, device_step, sizeof(std::uint64_t), 0, 0});
    for (const Named& p : parameters) {
        if (status != CGPTX_OK) break;
        float *master = nullptr, *first = nullptr, *second = nullptr;
        status = cgptx_model_optimizer_state(model, p.index, &master, &first, &second);
        const std::vector<std::size_t> shape = shape_of(p.name, c, p.count);
        entries.push_back({p.name + ".master", "F32", shape, master, p.count * sizeof(float), 0, 0});
        entries.push_back({p.name + ".exp_avg", "F32", shape, first, p.count * sizeof(float), 0, 0});
        entries.push_back({p.name + ".exp_avg_sq", "F32", shape, second, p.count * sizeof(float), 0, 0});
    }
    if (status == CGPTX_OK) status = write_file(path, entries);
    (void)hipFree(device_step);
    return status;
}

extern "C" int cgptx_model_load_optimizer(cgptx_model* model, const char* path, uint64_t* step) {
    using namespace cgptx;
    clear_error();
    if (model == nullptr || path == nullptr) return fail(CGPTX_INVALID_ARGUMENT, "model_load_optimizer: null argument");
    cgptx_model_config c{};
    if (int s = cgptx_model_describe(model, &c, nullptr, nullptr)) return s;
    std::ifstream in;
    std::map<std::string, Entry> entries;
    std::size_t data_begin = 0;
    if (int s = read_header(path, in, entries, data_begin)) return s;
    std::vector<Named> parameters;
    if (int s = parameters_of(model, parameters)) return s;
    CGPTX_HIP(hipDeviceSynchronize());
    std::vector<char> host;
    if (int s = read_tensor(in, data_begin, entries, "step", "U64", {1}, sizeof(std::uint64_t), host)) return s;
    std::uint64_t saved_step = 0;
    std::memcpy(&saved_step, host.data(), sizeof(saved_step));
    for (const Named& p : parameters) {
        float* state[3] = {nullptr, nullptr, nullptr};
        if (int s = cgptx_model_optimizer_state(model, p.index, &state[0], &state[1], &state[2])) return s;
        const char* suffix[3] = {".master", ".exp_avg", ".exp_avg_sq"};
        const std::vector<std::size_t> shape = shape_of(p.name, c, p.count);
        for (int k = 0; k < 3; ++k) {
            if (int s = read_tensor(in, data_begin, entries, p.name + suffix[k], "F32", shape, p.count * sizeof(float), host)) return s;
            CGPTX_HIP(hipMemcpy(state[k], host.data(), host.size(), hipMemcpyHostToDevice));
        }
    }
    if (int s = cgptx_model_set_optimizer_step(model, saved_step)) return s;
    if (step != nullptr) *step = saved_step;
    return CGPTX_OK;
}
