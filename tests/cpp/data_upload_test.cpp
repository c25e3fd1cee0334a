// Drives include/data/dataset_loader.h the way train/train.cpp:463-465, 570-574 drives the reference's:
// two page-locked batches uploaded alternately into one DeviceBatch, the device bits read back after each,
// host buffers rewritten only after wait_until_reusable, plus the declared copy / move / error behaviour
// (src/data/dataset_loader.cpp:82-166). Built with hipcc by __graft_entry__.build(); run by
// tests/test_cpp_interface.py on the GPU.
#include <cstdio>
#include <numeric>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "data/dataset_loader.h"

namespace {

int failures = 0;
void expect(bool ok, const std::string& what) {
    if (!ok) {
        ++failures;
        std::printf("FAIL %s\n", what.c_str());
    }
}
void hip_ok(hipError_t status, const char* what) {
    if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
}
std::vector<bpe::TokenId> read_back(const data::DeviceBuffer& buffer, std::size_t count, hipStream_t stream) {
    std::vector<bpe::TokenId> host(count);
    hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize");
    hip_ok(hipMemcpy(host.data(), buffer.data(), count * sizeof(bpe::TokenId), hipMemcpyDeviceToHost), "hipMemcpy");
    return host;
}
void fill(data::Batch& batch, std::size_t rows, std::size_t length, bpe::TokenId first) {
    batch.batch_size = rows;
    batch.sequence_length = length;
    batch.input_ids.resize(rows * length);
    batch.target_ids.resize(rows * length);
    std::iota(batch.input_ids.begin(), batch.input_ids.end(), first);
    std::iota(batch.target_ids.begin(), batch.target_ids.end(), first + 1);  // inputs shifted by one token
}
bool equal(const std::vector<bpe::TokenId>& device, const data::HostTokenVector& host) {
    return device.size() == host.size() && std::equal(device.begin(), device.end(), host.begin());
}

// The declarations callers rely on.
static_assert(std::is_same_v<data::HostTokenVector::value_type, bpe::TokenId>);
static_assert(std::is_invocable_v<decltype(&data::upload_batch), const data::Batch&, data::DeviceBatch&, hipStream_t>);
static_assert(std::is_copy_constructible_v<data::Batch> && std::is_copy_assignable_v<data::Batch>);
static_assert(std::is_nothrow_move_constructible_v<data::Batch> && std::is_nothrow_move_assignable_v<data::Batch>);
static_assert(!std::is_copy_constructible_v<data::DeviceBuffer> && std::is_nothrow_move_constructible_v<data::DeviceBuffer>);
static_assert(std::is_same_v<decltype(data::Batch::batch_size), std::size_t> &&
              std::is_same_v<decltype(data::Batch::sequence_length), std::size_t>);

}  // namespace

int main() {
    try {
        hipStream_t stream = nullptr;
        hip_ok(hipStreamCreate(&stream), "hipStreamCreate");
        constexpr std::size_t rows = 4, length = 96, count = rows * length;
        data::Batch slots[2];
        data::DeviceBatch device;
        expect(slots[0].empty() && slots[0].token_count() == 0, "a new batch is empty");
        slots[0].wait_until_reusable();  // nothing pending: returns at once

        // Two batches through one device batch, alternating host slots as the training loop does.
        const void* first_address = nullptr;
        for (int step = 0; step < 6; ++step) {
            data::Batch& batch = slots[step & 1];
            batch.wait_until_reusable();  // the upload issued two steps ago has left this slot
            fill(batch, rows, length, static_cast<bpe::TokenId>(1000 * step + 7));
            data::upload_batch(batch, device, stream);
            if (step == 0) first_address = device.input_ids.data();
            expect(device.input_ids.data() == first_address, "device buffers keep their address while the shape does not grow");
            expect(device.batch_size == rows && device.sequence_length == length, "device batch takes the shape");
            expect(equal(read_back(device.input_ids, count, stream), batch.input_ids), "input ids arrive bit for bit, step " + std::to_string(step));
            expect(equal(read_back(device.target_ids, count, stream), batch.target_ids), "target ids arrive bit for bit, step " + std::to_string(step));
        }
        expect(device.input_ids.bytes() == count * sizeof(bpe::TokenId), "device buffer holds exactly one batch");

        // A smaller batch reuses the buffers, a larger one replaces them.
        data::Batch small;
        fill(small, 2, 8, 5);
        data::upload_batch(small, device, stream);
        expect(device.input_ids.data() == first_address && device.batch_size == 2 && device.sequence_length == 8,
               "a smaller batch reuses the device buffers");
        expect(equal(read_back(device.target_ids, 16, stream), small.target_ids), "smaller batch arrives");
        data::Batch large;
        fill(large, 8, 128, 9);
        data::upload_batch(large, device, stream);
        expect(device.input_ids.bytes() == 8 * 128 * sizeof(bpe::TokenId), "a larger batch grows the device buffers");
        expect(equal(read_back(device.input_ids, 8 * 128, stream), large.input_ids), "larger batch arrives");

        // Declared shape and buffers must agree.
        data::Batch wrong;
        fill(wrong, 2, 8, 1);
        wrong.sequence_length = 9;
        bool threw = false;
        try { data::upload_batch(wrong, device, stream); } catch (const std::invalid_argument&) { threw = true; }
        expect(threw, "a batch whose buffers do not match its shape throws std::invalid_argument");

        // An empty batch uploads nothing and still becomes reusable.
        data::Batch nothing;
        data::upload_batch(nothing, device, stream);
        nothing.wait_until_reusable();
        expect(device.batch_size == 0 && device.sequence_length == 0, "an empty batch gives an empty device batch");

        // Copies are deep and independent of pending uploads; moves carry buffers and the pending upload along.
        data::upload_batch(large, device, stream);
        data::Batch copy = large;
        expect(copy.input_ids.data() != large.input_ids.data() && equal({copy.input_ids.begin(), copy.input_ids.end()}, large.input_ids),
               "copy construction is deep");
        copy.wait_until_reusable();
        const bpe::TokenId* moved_from = large.input_ids.data();
        data::Batch moved = std::move(large);
        expect(moved.input_ids.data() == moved_from && large.input_ids.empty(), "move construction takes the buffers");
        moved.wait_until_reusable();
        small = moved;  // waits for small's own pending upload, then deep copy
        expect(small.token_count() == moved.token_count() && small.input_ids.data() != moved.input_ids.data(), "copy assignment is deep");
        small = std::move(moved);
        expect(small.input_ids.data() == moved_from, "move assignment takes the buffers");
        data::upload_batch(small, device, stream);  // destroyed below with the upload possibly still pending

        hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize");
        device = data::DeviceBatch{};
        expect(device.input_ids.empty() && device.target_ids.bytes() == 0, "move assignment of an empty device batch releases");
    } catch (const std::exception& error) {
        std::printf("FAIL exception: %s\n", error.what());
        ++failures;
    }
    std::printf("%d failure(s)\n", failures);
    return failures == 0 ? 0 : 1;
}
