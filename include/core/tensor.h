// Dense row-major tensor handle of the operator interface: shape + storage dtype + one
// allocation in device memory (HIP) or host memory. Metadata-only reshape, owning or borrowed
// storage. Same members, argument orders and exceptions as the reference's
// include/core/tensor.h:20-345 for what the operators, src/core's blocks and the tests use:
// both constructors, device_view(shape, data, dtype), deep copies, data(), raw_data(), shape
// queries, reshape, typed and raw host copies, empty/zeros/ones/full. Tensor::eye is not provided.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <numeric>
#include <span>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "core/dtype.h"

// CUDA names the accelerator in the reference's callers; here it is the HIP device.
enum class DeviceType : std::uint8_t { CPU, GPU, CUDA = GPU };

class Tensor {
public:
    Tensor() = default;

    // Non-owning view of contiguous device memory (reference: Tensor::device_view, tensor.h:31-36).
    [[nodiscard]] static Tensor device_view(std::vector<std::size_t> shape, void* data, const Dtype dtype) {
        Tensor view;
        view.shape_ = std::move(shape);
        view.device_type_ = DeviceType::GPU;
        view.dtype_ = validate_dtype(dtype);
        view.element_count_ = count(view.shape_);
        view.data_ = data;
        view.owned_ = false;
        return view;
    }

    // Reference: tensor.h:45-60 (every dimension non-zero; throws std::invalid_argument otherwise).
    explicit Tensor(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                    const Dtype dtype = Dtype::F32)
        : shape_(std::move(shape)), device_type_(device_type), dtype_(validate_dtype(dtype)), element_count_(count(shape_)),
          owned_(true) {
        allocate();
    }

    // The data type before the device (reference: tensor.h:63-67).
    explicit Tensor(std::vector<std::size_t> shape, const Dtype dtype, const DeviceType device_type = DeviceType::GPU)
        : Tensor(std::move(shape), device_type, dtype) {}

    [[nodiscard]] static Tensor empty(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                                      const Dtype dtype = Dtype::F32) {
        return Tensor(std::move(shape), device_type, dtype);
    }

    // zeros / ones / full take the reference's argument order (tensor.h:231-256): the fill is enqueued on
    // `stream` for device tensors (host staging here, so the call returns with the copy issued).
    [[nodiscard]] static Tensor zeros(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                                      hipStream_t stream = nullptr, const Dtype dtype = Dtype::F32) {
        Tensor result(std::move(shape), device_type, dtype);
        if (result.nbytes() == 0) return result;
        if (device_type == DeviceType::GPU) {
            if (hipMemsetAsync(result.data_, 0, result.nbytes(), stream) != hipSuccess)
                throw std::runtime_error("Tensor: memset failed");
        } else {
            std::memset(result.data_, 0, result.nbytes());
        }
        return result;
    }
    [[nodiscard]] static Tensor full(std::vector<std::size_t> shape, const float value,
                                     const DeviceType device_type = DeviceType::GPU, hipStream_t stream = nullptr,
                                     const Dtype dtype = Dtype::F32) {
        (void)stream;
        Tensor result(std::move(shape), device_type, dtype);
        result.copy_from_host(std::vector<float>(result.numel(), value));
        return result;
    }
    [[nodiscard]] static Tensor ones(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                                     hipStream_t stream = nullptr, const Dtype dtype = Dtype::F32) {
        return full(std::move(shape), 1.0f, device_type, stream, dtype);
    }

    // Deep copies, as the reference's copy constructor and assignment (tensor.h:80-108). A copy of a view owns
    // its storage.
    Tensor(const Tensor& other)
        : shape_(other.shape_), device_type_(other.device_type_), dtype_(other.dtype_), element_count_(other.element_count_),
          owned_(true) {
        allocate();
        if (nbytes() == 0) return;
        if (device_type_ == DeviceType::GPU) {
            if (hipMemcpy(data_, other.data_, nbytes(), hipMemcpyDeviceToDevice) != hipSuccess)
                throw std::runtime_error("Tensor: device-to-device copy failed");
        } else {
            std::memcpy(data_, other.data_, nbytes());
        }
    }
    Tensor& operator=(const Tensor& other) {
        if (this == &other) return *this;
        Tensor copy(other);
        swap(copy);
        return *this;
    }
    Tensor(Tensor&& other) noexcept { swap(other); }
    Tensor& operator=(Tensor&& other) noexcept {
        if (this != &other) {
            release();
            swap(other);
        }
        return *this;
    }
    ~Tensor() { release(); }

    // F32 tensors only (reference: tensor.h:130-137).
    [[nodiscard]] float* data() {
        if (dtype_ != Dtype::F32) throw std::invalid_argument("Tensor::data requires F32 storage");
        return static_cast<float*>(data_);
    }
    [[nodiscard]] const float* data() const {
        if (dtype_ != Dtype::F32) throw std::invalid_argument("Tensor::data requires F32 storage");
        return static_cast<const float*>(data_);
    }
    [[nodiscard]] void* raw_data() noexcept { return data_; }
    [[nodiscard]] const void* raw_data() const noexcept { return data_; }
    [[nodiscard]] const std::vector<std::size_t>& shape() const noexcept { return shape_; }
    [[nodiscard]] std::size_t numel() const noexcept { return element_count_; }
    [[nodiscard]] std::size_t nbytes() const noexcept { return element_count_ * dtype_size(dtype_); }
    [[nodiscard]] std::size_t dim() const noexcept { return shape_.size(); }
    [[nodiscard]] DeviceType device_type() const noexcept { return device_type_; }
    [[nodiscard]] Dtype dtype() const noexcept { return dtype_; }
    [[nodiscard]] std::size_t size(const std::size_t axis) const {
        if (axis >= shape_.size()) throw std::out_of_range("Tensor::size: axis out of range");
        return shape_[axis];
    }

    // Metadata only; the element count must not change.
    void reshape(std::vector<std::size_t> new_shape) {
        if (count(new_shape) != element_count_) throw std::invalid_argument("Tensor::reshape: element count differs");
        shape_ = std::move(new_shape);
    }

    // F32 host values into the tensor's storage dtype (round to nearest even) and back, synchronously
    // (reference: tensor.h:268-274, src/core/tensor.cu:156-246).
    void copy_from_host(std::span<const float> source) {
        if (source.size() != numel()) throw std::invalid_argument("Tensor: invalid input size");
        if (dtype_ == Dtype::F32) {
            copy_raw_from_host({reinterpret_cast<const std::uint8_t*>(source.data()), nbytes()});
            return;
        }
        std::vector<std::uint16_t> converted(source.size());
        for (std::size_t i = 0; i < source.size(); ++i)
            converted[i] = dtype_ == Dtype::F16 ? cgptx_detail::float_to_half_bits(source[i])
                                                : cgptx_detail::float_to_bf16_bits(source[i]);
        copy_raw_from_host({reinterpret_cast<const std::uint8_t*>(converted.data()), nbytes()});
    }
    void copy_to_host(std::span<float> destination) const {
        if (destination.size() != numel()) throw std::invalid_argument("Tensor: invalid output size");
        if (dtype_ == Dtype::F32) {
            copy_raw_to_host({reinterpret_cast<std::uint8_t*>(destination.data()), nbytes()});
            return;
        }
        std::vector<std::uint16_t> stored(destination.size());
        copy_raw_to_host({reinterpret_cast<std::uint8_t*>(stored.data()), nbytes()});
        for (std::size_t i = 0; i < stored.size(); ++i)
            destination[i] = dtype_ == Dtype::F16 ? cgptx_detail::half_bits_to_float(stored[i])
                                                  : cgptx_detail::bf16_bits_to_float(stored[i]);
    }

    void copy_raw_from_host(std::span<const std::uint8_t> source) {
        if (source.size() != nbytes()) throw std::invalid_argument("Tensor::copy_raw_from_host: size differs");
        if (source.empty()) return;
        if (device_type_ == DeviceType::GPU) {
            if (hipMemcpy(data_, source.data(), source.size(), hipMemcpyHostToDevice) != hipSuccess)
                throw std::runtime_error("Tensor: host-to-device copy failed");
        } else {
            std::memcpy(data_, source.data(), source.size());
        }
    }
    void copy_raw_to_host(std::span<std::uint8_t> destination) const {
        if (destination.size() != nbytes()) throw std::invalid_argument("Tensor::copy_raw_to_host: size differs");
        if (destination.empty()) return;
        if (device_type_ == DeviceType::GPU) {
            if (hipMemcpy(destination.data(), data_, destination.size(), hipMemcpyDeviceToHost) != hipSuccess)
                throw std::runtime_error("Tensor: device-to-host copy failed");
        } else {
            std::memcpy(destination.data(), data_, destination.size());
        }
    }

    void swap(Tensor& other) noexcept {
        std::swap(shape_, other.shape_);
        std::swap(device_type_, other.device_type_);
        std::swap(dtype_, other.dtype_);
        std::swap(element_count_, other.element_count_);
        std::swap(data_, other.data_);
        std::swap(owned_, other.owned_);
    }

private:
    // Product of the dimensions; an empty shape or a zero dimension is an error (reference: tensor.h:318-335).
    static std::size_t count(const std::vector<std::size_t>& shape) {
        if (shape.empty()) throw std::invalid_argument("Tensor shape cannot be empty");
        std::size_t total = 1;
        for (const std::size_t extent : shape) {
            if (extent == 0) throw std::invalid_argument("Tensor dimension cannot be zero");
            if (total > static_cast<std::size_t>(-1) / extent) throw std::overflow_error("Tensor element count overflows");
            total *= extent;
        }
        return total;
    }
    static Dtype validate_dtype(const Dtype dtype) {
        if (!is_floating_point(dtype)) throw std::invalid_argument("Tensor: storage dtype must be F16, BF16 or F32");
        return dtype;
    }
    void allocate() {
        const std::size_t bytes = nbytes();
        if (bytes == 0) return;
        if (device_type_ == DeviceType::GPU) {
            if (hipMalloc(&data_, bytes) != hipSuccess) throw std::runtime_error("Tensor: device allocation failed");
        } else if (device_type_ == DeviceType::CPU) {
            data_ = ::operator new(bytes);
        } else {
            throw std::invalid_argument("Tensor: invalid device type");
        }
    }
    void release() noexcept {
        if (owned_ && data_ != nullptr) {
            if (device_type_ == DeviceType::GPU) (void)hipFree(data_);
            else ::operator delete(data_);
        }
        data_ = nullptr;
        owned_ = false;
    }

    std::vector<std::size_t> shape_;
    DeviceType device_type_ = DeviceType::GPU;
    Dtype dtype_ = Dtype::F32;
    std::size_t element_count_ = 0;
    void* data_ = nullptr;
    bool owned_ = false;
};

namespace cgptx_detail {

inline void require_device(const char* op, std::initializer_list<const Tensor*> tensors) {
    for (const Tensor* t : tensors)
        if (t->device_type() != DeviceType::GPU)
            throw std::invalid_argument(std::string(op) + ": all tensors must live on the GPU");
}
inline void require_same_dtype(const char* op, const Tensor& first, std::initializer_list<const Tensor*> others) {
    for (const Tensor* t : others)
        if (t->dtype() != first.dtype()) throw std::invalid_argument(std::string(op) + ": tensors must share one dtype");
}
inline void require_same_shape(const char* op, const Tensor& first, std::initializer_list<const Tensor*> others) {
    for (const Tensor* t : others)
        if (t->shape() != first.shape()) throw std::invalid_argument(std::string(op) + ": tensor shapes differ");
}

}  // namespace cgptx_detail
