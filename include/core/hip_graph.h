// RAII wrapper around stream capture and an executable hipGraph: records a fixed sequence of work
// submitted to a stream and replays it with one launch. Counterpart of the reference's CudaGraph
// (include/core/cuda_graph.h:17-93, src/core/cuda_graph.cu:86-210): same members, same exceptions
// (std::invalid_argument for an empty callback, a null stream or a null graph; std::runtime_error when
// capture, instantiation, launch or upload fails; std::logic_error when there is nothing to launch).
//
// The recorded work keeps the device addresses used during capture: tensors, and the operators' scratch
// memory, must stay where they are while the executable graph is in use. Run the sequence once eagerly
// before capturing it (as train/train.cpp:545-548 does) so that every operator has its scratch memory;
// an operator that would have to allocate during capture makes capture() throw std::runtime_error.
#pragma once

#include <hip/hip_runtime_api.h>

#include <functional>
#include <stdexcept>
#include <string>
#include <utility>

class HipGraph {
public:
    HipGraph() noexcept = default;
    HipGraph(const HipGraph&) = delete;
    HipGraph& operator=(const HipGraph&) = delete;
    HipGraph(HipGraph&& other) noexcept
        : graph_(std::exchange(other.graph_, nullptr)), executable_(std::exchange(other.executable_, nullptr)) {}
    HipGraph& operator=(HipGraph&& other) noexcept {
        if (this != &other) {
            reset();
            graph_ = std::exchange(other.graph_, nullptr);
            executable_ = std::exchange(other.executable_, nullptr);
        }
        return *this;
    }
    ~HipGraph() noexcept { reset(); }

    // Captures what capture_body enqueues on `stream` and instantiates it. The previous graph is destroyed
    // first. If the callback throws, capture is ended, the abandoned graph destroyed and the exception
    // passed on.
    void capture(hipStream_t stream, const std::function<void()>& capture_body,
                 const hipStreamCaptureMode mode = hipStreamCaptureModeThreadLocal) {
        if (!capture_body) throw std::invalid_argument("HipGraph::capture: capture callback is empty");
        if (stream == nullptr) throw std::invalid_argument("HipGraph::capture: stream must not be null");
        reset();
        check(hipStreamBeginCapture(stream, mode), "hipStreamBeginCapture");
        try {
            capture_body();
        } catch (...) {
            hipGraph_t abandoned = nullptr;
            if (hipStreamEndCapture(stream, &abandoned) != hipSuccess) (void)hipGetLastError();
            if (abandoned != nullptr) (void)hipGraphDestroy(abandoned);
            throw;
        }
        hipGraph_t captured = nullptr;
        check(hipStreamEndCapture(stream, &captured), "hipStreamEndCapture");
        if (captured == nullptr) throw std::runtime_error("HipGraph::capture: the runtime returned an empty graph");
        try {
            instantiate(captured);
        } catch (...) {
            (void)hipGraphDestroy(captured);
            throw;
        }
    }

    // Takes ownership of `graph` on success.
    void instantiate(hipGraph_t graph) {
        if (graph == nullptr) throw std::invalid_argument("HipGraph::instantiate: graph is null");
        hipGraphExec_t executable = nullptr;
        check(hipGraphInstantiate(&executable, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
        reset();
        graph_ = graph;
        executable_ = executable;
    }

    void launch(hipStream_t stream) const {
        if (executable_ == nullptr) throw std::logic_error("HipGraph::launch: no executable graph");
        check(hipGraphLaunch(executable_, stream), "hipGraphLaunch");
    }

    void upload(hipStream_t stream) const {
        if (executable_ == nullptr) throw std::logic_error("HipGraph::upload: no executable graph");
        check(hipGraphUpload(executable_, stream), "hipGraphUpload");
    }

    void reset() noexcept {
        if (executable_ != nullptr) (void)hipGraphExecDestroy(executable_);
        if (graph_ != nullptr) (void)hipGraphDestroy(graph_);
        executable_ = nullptr;
        graph_ = nullptr;
    }

    [[nodiscard]] bool initialized() const noexcept { return executable_ != nullptr; }
    [[nodiscard]] hipGraph_t graph() const noexcept { return graph_; }
    [[nodiscard]] hipGraphExec_t executable() const noexcept { return executable_; }

private:
    static void check(const hipError_t status, const char* what) {
        if (status != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(status));
    }

    hipGraph_t graph_ = nullptr;
    hipGraphExec_t executable_ = nullptr;
};
