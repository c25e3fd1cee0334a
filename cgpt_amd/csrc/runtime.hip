// Status reporting and the per-stream scratch arena behind every entry point.
#include "common.hpp"

#include <map>
#include <mutex>
#include <utility>

namespace cgptx {
namespace {

thread_local std::string g_last_error;

struct Arena {
    void* data = nullptr;
    std::size_t bytes = 0;
    std::uint64_t generation = 0;  // value of g_generation when this block was allocated
};

std::mutex g_arena_mutex;
std::map<std::pair<int, hipStream_t>, Arena> g_arenas;
std::uint64_t g_generation = 0;  // bumped by every allocation; a released arena reads as generation 0

}  // namespace

int fail(int code, const std::string& message) {
    g_last_error = message;
    return code;
}

void clear_error() { g_last_error.clear(); }

int check_hip(hipError_t error, const char* what) {
    if (error == hipSuccess) return CGPTX_OK;
    return fail(CGPTX_RUNTIME, std::string(what) + ": " + hipGetErrorString(error));
}

int scratch(hipStream_t stream, std::size_t bytes, void** out) {
    int device = 0;
    CGPTX_HIP(hipGetDevice(&device));
    std::lock_guard<std::mutex> lock(g_arena_mutex);
    Arena& arena = g_arenas[{device, stream}];
    if (arena.bytes < bytes) {
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if (stream != nullptr) CGPTX_HIP(hipStreamIsCapturing(stream, &capture));
        if (capture != hipStreamCaptureStatusNone) {
            return fail(CGPTX_CAPTURE_ALLOC,
                        "scratch arena would have to grow during stream capture; run the op once eagerly first");
        }
        // Round up so that small variations in problem size do not reallocate.
        const std::size_t rounded = (bytes + (std::size_t{1} << 20) - 1) & ~((std::size_t{1} << 20) - 1);
        void* fresh = nullptr;
        CGPTX_HIP(hipMalloc(&fresh, rounded));
        if (arena.data != nullptr) {
            // hipFree waits for outstanding work that may still read the old block.
            CGPTX_HIP(hipFree(arena.data));
        }
        arena.data = fresh;
        arena.bytes = rounded;
        arena.generation = ++g_generation;
    }
    *out = arena.data;
    return CGPTX_OK;
}

std::uint64_t scratch_generation(hipStream_t stream) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_arena_mutex);
    const auto it = g_arenas.find({device, stream});
    return it == g_arenas.end() ? 0 : it->second.generation;
}

int compute_units() {
    static int cached = [] {
        int device = 0;
        int count = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0) {
            count = 256;
        }
        return count;
    }();
    return cached;
}

}  // namespace cgptx

extern "C" const char* cgptx_last_error(void) { return cgptx::g_last_error.c_str(); }

extern "C" const char* cgptx_version(void) { return "cgptx 0.1 (gfx950)"; }

extern "C" size_t cgptx_scratch_bytes(cgptx_stream stream) {
    using namespace cgptx;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    std::lock_guard<std::mutex> lock(g_arena_mutex);
    const auto it = g_arenas.find({device, static_cast<hipStream_t>(stream)});
    return it == g_arenas.end() ? 0 : it->second.bytes;
}

extern "C" int cgptx_release_scratch(void) {
    using namespace cgptx;
    int device = 0;
    CGPTX_HIP(hipGetDevice(&device));
    CGPTX_HIP(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lock(g_arena_mutex);
    for (auto it = g_arenas.begin(); it != g_arenas.end();) {
        if (it->first.first == device) {
            if (it->second.data != nullptr) CGPTX_HIP(hipFree(it->second.data));
            it = g_arenas.erase(it);
        } else {
            ++it;
        }
    }
    return CGPTX_OK;
}
