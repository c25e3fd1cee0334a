// The device half of the reference's data path (include/data/dataset_loader.h:53-170,
// src/data/dataset_loader.cpp:120-166): a training batch in page-locked host memory, its device
// twin, and the asynchronous upload between them. Same names, fields and error behaviour; the
// stream is a hipStream_t. The loader that fills batches from a token file is not part of this
// library.
#pragma once

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstddef>
#include <new>
#include <stdexcept>
#include <utility>
#include <vector>

#include "core/status.h"
#include "core/token_id.h"

namespace data {

namespace detail {
inline void hip_check(const hipError_t error, const char* what) {
    if (error == hipSuccess) return;
    std::fprintf(stderr, "%s: %s\n", what, hipGetErrorString(error));
    std::exit(EXIT_FAILURE);
}
}  // namespace detail

/** Allocator of page-locked host memory (CudaHostAllocator in the reference). */
template <typename T>
class HipHostAllocator {
public:
    using value_type = T;
    HipHostAllocator() noexcept = default;
    template <typename U>
    HipHostAllocator(const HipHostAllocator<U>&) noexcept {}
    [[nodiscard]] T* allocate(const std::size_t count) {
        if (count > static_cast<std::size_t>(-1) / sizeof(T)) throw std::bad_array_new_length();
        void* pointer = nullptr;
        detail::hip_check(hipHostMalloc(&pointer, std::max<std::size_t>(count, 1) * sizeof(T), hipHostMallocDefault),
                          "hipHostMalloc");
        return static_cast<T*>(pointer);
    }
    void deallocate(T* pointer, std::size_t) noexcept { (void)hipHostFree(pointer); }
    template <typename U>
    friend constexpr bool operator==(const HipHostAllocator&, const HipHostAllocator<U>&) noexcept {
        return true;
    }
};

using HostTokenVector = std::vector<bpe::TokenId, HipHostAllocator<bpe::TokenId>>;

/** Device memory that grows on request and keeps its address otherwise (DeviceBuffer in the reference). */
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    DeviceBuffer(DeviceBuffer&& other) noexcept { swap(other); }
    DeviceBuffer& operator=(DeviceBuffer&& other) noexcept {
        swap(other);
        return *this;
    }
    ~DeviceBuffer() {
        if (data_ != nullptr) (void)hipFree(data_);
    }
    void allocate(const std::size_t bytes) {
        if (data_ != nullptr) detail::hip_check(hipFree(data_), "hipFree");
        data_ = nullptr;
        bytes_ = 0;
        if (bytes != 0) detail::hip_check(hipMalloc(&data_, bytes), "hipMalloc");
        bytes_ = bytes;
    }
    [[nodiscard]] void* data() const noexcept { return data_; }
    [[nodiscard]] std::size_t bytes() const noexcept { return bytes_; }

private:
    void swap(DeviceBuffer& other) noexcept {
        std::swap(data_, other.data_);
        std::swap(bytes_, other.bytes_);
    }
    void* data_ = nullptr;
    std::size_t bytes_ = 0;
};

/** Host-side training batch in page-locked memory, with the event that guards its reuse. */
struct Batch {
    HostTokenVector input_ids;   // [batch_size, sequence_length]
    HostTokenVector target_ids;  // input_ids shifted by one token
    std::size_t batch_size = 0;
    std::size_t sequence_length = 0;

    Batch() = default;
    ~Batch() {
        if (upload_complete_ != nullptr) (void)hipEventDestroy(upload_complete_);
    }
    Batch(const Batch& other)
        : input_ids(other.input_ids), target_ids(other.target_ids), batch_size(other.batch_size),
          sequence_length(other.sequence_length) {}
    Batch& operator=(const Batch& other) {
        if (this != &other) {
            wait_until_reusable();
            input_ids = other.input_ids;
            target_ids = other.target_ids;
            batch_size = other.batch_size;
            sequence_length = other.sequence_length;
        }
        return *this;
    }
    Batch(Batch&& other) noexcept
        : input_ids(std::move(other.input_ids)), target_ids(std::move(other.target_ids)), batch_size(other.batch_size),
          sequence_length(other.sequence_length), upload_complete_(std::exchange(other.upload_complete_, nullptr)) {}
    Batch& operator=(Batch&& other) noexcept {
        if (this != &other) {
            if (upload_complete_ != nullptr) {
                (void)hipEventSynchronize(upload_complete_);
                (void)hipEventDestroy(upload_complete_);
            }
            input_ids = std::move(other.input_ids);
            target_ids = std::move(other.target_ids);
            batch_size = other.batch_size;
            sequence_length = other.sequence_length;
            upload_complete_ = std::exchange(other.upload_complete_, nullptr);
        }
        return *this;
    }

    [[nodiscard]] std::size_t token_count() const noexcept { return batch_size * sequence_length; }
    [[nodiscard]] bool empty() const noexcept { return token_count() == 0; }

    /** Waits until the last asynchronous upload no longer reads this batch. */
    void wait_until_reusable() const {
        if (upload_complete_ != nullptr) detail::hip_check(hipEventSynchronize(upload_complete_), "hipEventSynchronize");
    }
    /** Records the event that marks host-buffer reuse as safe. */
    void mark_upload_complete(const hipStream_t stream) const {
        if (upload_complete_ == nullptr)
            detail::hip_check(hipEventCreateWithFlags(&upload_complete_, hipEventDisableTiming), "hipEventCreate");
        detail::hip_check(hipEventRecord(upload_complete_, stream), "hipEventRecord");
    }

private:
    mutable hipEvent_t upload_complete_ = nullptr;
};

/** Device-side destination of a batch; the buffers grow only when needed, so their addresses
 *  stay valid for a captured graph as long as the batch shape does not grow. */
struct DeviceBatch {
    DeviceBuffer input_ids;
    DeviceBuffer target_ids;
    std::size_t batch_size = 0;
    std::size_t sequence_length = 0;
};

/** Asynchronously uploads a host batch; throws std::invalid_argument if the batch buffers do not
 *  match its declared shape. */
inline void upload_batch(const Batch& batch, DeviceBatch& destination, const hipStream_t stream = nullptr) {
    batch.wait_until_reusable();
    const std::size_t count = batch.token_count();
    if (batch.input_ids.size() != count || batch.target_ids.size() != count)
        throw std::invalid_argument("Batch buffers do not match its declared shape");
    const std::size_t bytes = count * sizeof(bpe::TokenId);
    if (destination.input_ids.bytes() < bytes) destination.input_ids.allocate(bytes);
    if (destination.target_ids.bytes() < bytes) destination.target_ids.allocate(bytes);
    if (bytes != 0) {
        detail::hip_check(hipMemcpyAsync(destination.input_ids.data(), batch.input_ids.data(), bytes, hipMemcpyHostToDevice, stream),
                          "hipMemcpyAsync");
        detail::hip_check(hipMemcpyAsync(destination.target_ids.data(), batch.target_ids.data(), bytes, hipMemcpyHostToDevice, stream),
                          "hipMemcpyAsync");
    }
    batch.mark_upload_complete(stream);
    destination.batch_size = batch.batch_size;
    destination.sequence_length = batch.sequence_length;
}

}  // namespace data
