// The device half of the reference's data path: a training batch in page-locked host memory, its
// device twin, and the asynchronous upload between them — the declarations of
// include/data/dataset_loader.h:53-170 (CudaHostAllocator, HostTokenVector, Batch, DeviceBatch,
// upload_batch; behaviour: src/data/dataset_loader.cpp:82-166) over the library's upload entry points
// (cgptx_pinned_*, cgptx_device_*, cgptx_upload_fence_*, cgptx_token_upload_async in cgptx_train.h).
// The stream is a hipStream_t. The loader that cuts batches out of a token file is not part of this
// library.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <limits>
#include <new>
#include <stdexcept>
#include <type_traits>
#include <utility>
#include <vector>

#include "cgptx_train.h"
#include "core/status.h"
#include "core/token_id.h"

namespace data {

/** Standard-library allocator over the library's page-locked host memory (the reference's
 *  CudaHostAllocator): a vector built on it can be the source of an asynchronous upload. */
template <typename T>
struct PinnedHostAllocator {
    using value_type = T;
    using is_always_equal = std::true_type;

    constexpr PinnedHostAllocator() noexcept = default;
    template <typename Other>
    constexpr PinnedHostAllocator(const PinnedHostAllocator<Other>&) noexcept {}

    [[nodiscard]] T* allocate(const std::size_t elements) {
        if (elements > std::numeric_limits<std::size_t>::max() / sizeof(T)) throw std::bad_array_new_length();
        void* block = nullptr;
        if (cgptx_pinned_allocate(&block, elements * sizeof(T)) != CGPTX_OK) throw std::bad_alloc();
        return static_cast<T*>(block);
    }
    void deallocate(T* block, std::size_t) noexcept { (void)cgptx_pinned_release(block); }
};
template <typename A, typename B>
constexpr bool operator==(const PinnedHostAllocator<A>&, const PinnedHostAllocator<B>&) noexcept {
    return true;
}
template <typename T>
using HipHostAllocator = PinnedHostAllocator<T>;

using HostTokenVector = std::vector<bpe::TokenId, PinnedHostAllocator<bpe::TokenId>>;

/** Device memory that is replaced only on request, so its address survives re-uploads of the same
 *  shape (what DeviceBatch needs of include/core/device_buffer.h). */
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(const std::size_t bytes) { allocate(bytes); }
    DeviceBuffer(DeviceBuffer&& other) noexcept : block_(other.block_), bytes_(other.bytes_) { other.forget(); }
    DeviceBuffer& operator=(DeviceBuffer&& other) noexcept {
        if (this != &other) {
            release();
            block_ = other.block_;
            bytes_ = other.bytes_;
            other.forget();
        }
        return *this;
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    ~DeviceBuffer() { release(); }

    /** The replacement is obtained before the old block is given back; 0 bytes just releases. */
    void allocate(const std::size_t bytes) {
        void* fresh = nullptr;
        if (bytes != 0) cgptx_detail::check(cgptx_device_allocate(&fresh, bytes));
        release();
        block_ = fresh;
        bytes_ = bytes;
    }
    void release() noexcept {
        if (block_ != nullptr) (void)cgptx_device_release(block_);
        forget();
    }
    [[nodiscard]] void* data() noexcept { return block_; }
    [[nodiscard]] const void* data() const noexcept { return block_; }
    [[nodiscard]] std::size_t bytes() const noexcept { return bytes_; }
    [[nodiscard]] bool empty() const noexcept { return block_ == nullptr; }

private:
    void forget() noexcept {
        block_ = nullptr;
        bytes_ = 0;
    }
    void* block_ = nullptr;
    std::size_t bytes_ = 0;
};

struct DeviceBatch;

namespace detail {
/** The library's upload fence of one batch. A copy of a batch starts without one (nothing reads the copy's
 *  buffers yet); assigning to a batch first waits for the uploads that still read its buffers. */
class ReuseGuard {
public:
    ReuseGuard() = default;
    ReuseGuard(const ReuseGuard&) noexcept {}
    ReuseGuard(ReuseGuard&& other) noexcept : fence_(std::exchange(other.fence_, nullptr)) {}
    ReuseGuard& operator=(const ReuseGuard& other) {
        if (this != &other) wait();
        return *this;
    }
    ReuseGuard& operator=(ReuseGuard&& other) noexcept {
        if (this != &other) {
            (void)cgptx_upload_fence_wait(fence_);
            (void)cgptx_upload_fence_destroy(fence_);
            fence_ = std::exchange(other.fence_, nullptr);
        }
        return *this;
    }
    ~ReuseGuard() { (void)cgptx_upload_fence_destroy(fence_); }

    void wait() const { cgptx_detail::check(cgptx_upload_fence_wait(fence_)); }
    [[nodiscard]] cgptx_upload_fence** slot() noexcept { return &fence_; }

private:
    cgptx_upload_fence* fence_ = nullptr;
};
}  // namespace detail

/** Host-side training batch in page-locked memory for asynchronous uploads. */
struct Batch {
private:
    // Declared first: member-wise assignment then waits for pending uploads before the token vectors
    // below are overwritten.
    mutable detail::ReuseGuard reuse_;

public:
    HostTokenVector input_ids;   // [batch_size, sequence_length]
    HostTokenVector target_ids;  // input_ids shifted by one token
    std::size_t batch_size = 0;
    std::size_t sequence_length = 0;

    Batch() = default;
    Batch(const Batch& other) = default;             // deep copy, no upload pending on the copy
    Batch& operator=(const Batch& other) = default;  // waits, then deep copy
    Batch(Batch&& other) noexcept = default;
    Batch& operator=(Batch&& other) noexcept = default;
    /** Ends only after pending uploads have stopped reading the token vectors, which are freed next. */
    ~Batch() { (void)cgptx_upload_fence_wait(*reuse_.slot()); }

    [[nodiscard]] std::size_t token_count() const noexcept { return batch_size * sequence_length; }
    [[nodiscard]] bool empty() const noexcept { return token_count() == 0; }
    /** Waits until the last asynchronous upload no longer reads this batch. */
    void wait_until_reusable() const { reuse_.wait(); }

private:
    friend void upload_batch(const Batch&, DeviceBatch&, hipStream_t);
};

/** Reusable device storage for a host-side Batch. */
struct DeviceBatch {
    DeviceBuffer input_ids;
    DeviceBuffer target_ids;
    std::size_t batch_size = 0;
    std::size_t sequence_length = 0;
};

/** Enqueues the upload of both token arrays on `stream`. Destination buffers grow only when needed, so a
 *  captured graph that reads them stays valid while the batch shape does not grow; the host batch stays in
 *  use until the copies have completed (wait_until_reusable). Throws std::invalid_argument when the batch
 *  buffers do not match its declared shape. */
inline void upload_batch(const Batch& batch, DeviceBatch& destination, const hipStream_t stream = nullptr) {
    batch.wait_until_reusable();
    const std::size_t tokens = batch.token_count();
    if (tokens != batch.input_ids.size() || tokens != batch.target_ids.size())
        throw std::invalid_argument("Batch buffers do not match its declared shape");
    for (DeviceBuffer* buffer : {&destination.input_ids, &destination.target_ids})
        if (buffer->bytes() < tokens * sizeof(bpe::TokenId)) buffer->allocate(tokens * sizeof(bpe::TokenId));
    cgptx_detail::check(cgptx_token_upload_async(static_cast<bpe::TokenId*>(destination.input_ids.data()),
                                                 static_cast<bpe::TokenId*>(destination.target_ids.data()),
                                                 batch.input_ids.data(), batch.target_ids.data(), tokens,
                                                 batch.reuse_.slot(), stream));
    destination.batch_size = batch.batch_size;
    destination.sequence_length = batch.sequence_length;
}

}  // namespace data
