// Dense row-major tensor handle of the operator interface: shape + storage dtype + one
// allocation in device memory (HIP) or host memory. Metadata-only reshape, owning or borrowed
// storage. Mirrors what the operators and their callers use of the reference's
// include/core/tensor.h:20-300 (construction, device_view, raw_data, shape queries, reshape, raw
// host copies); factories such as eye/full are not part of this path.
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

    Tensor(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU, const Dtype dtype = Dtype::F32)
        : shape_(std::move(shape)), device_type_(device_type), dtype_(dtype), element_count_(count(shape_)), owned_(true) {
        const std::size_t bytes = nbytes();
        if (bytes == 0) return;
        if (device_type_ == DeviceType::GPU) {
            if (hipMalloc(&data_, bytes) != hipSuccess) throw std::runtime_error("Tensor: device allocation failed");
        } else {
            data_ = ::operator new(bytes);
        }
    }

    // Non-owning view of device memory (reference: Tensor::device_view, tensor.h:32-40).
    [[nodiscard]] static Tensor device_view(void* data, std::vector<std::size_t> shape, const Dtype dtype) {
        Tensor view;
        view.shape_ = std::move(shape);
        view.device_type_ = DeviceType::GPU;
        view.dtype_ = dtype;
        view.element_count_ = count(view.shape_);
        view.data_ = data;
        view.owned_ = false;
        return view;
    }

    [[nodiscard]] static Tensor empty(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                                      const Dtype dtype = Dtype::F32) {
        return Tensor(std::move(shape), device_type, dtype);
    }

    [[nodiscard]] static Tensor zeros(std::vector<std::size_t> shape, const DeviceType device_type = DeviceType::GPU,
                                      const Dtype dtype = Dtype::F32) {
        Tensor result(std::move(shape), device_type, dtype);
        if (result.nbytes() == 0) return result;
        if (device_type == DeviceType::GPU) {
            if (hipMemset(result.data_, 0, result.nbytes()) != hipSuccess) throw std::runtime_error("Tensor: memset failed");
        } else {
            std::memset(result.data_, 0, result.nbytes());
        }
        return result;
    }

    Tensor(const Tensor&) = delete;
    Tensor& operator=(const Tensor&) = delete;
    Tensor(Tensor&& other) noexcept { swap(other); }
    Tensor& operator=(Tensor&& other) noexcept {
        if (this != &other) {
            release();
            swap(other);
        }
        return *this;
    }
    ~Tensor() { release(); }

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
    static std::size_t count(const std::vector<std::size_t>& shape) {
        return std::accumulate(shape.begin(), shape.end(), std::size_t{1}, [](std::size_t a, std::size_t b) { return a * b; });
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
