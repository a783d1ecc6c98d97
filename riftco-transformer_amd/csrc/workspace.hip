// Per-stream scratch memory for kernels that exchange partial results between
// workgroups (the small-batch forward and the split-K dense matmul).
//
// One buffer of kStreamWorkspaceBytes per (device, stream), allocated on first
// use and kept until the process ends: calls on one stream are ordered, so
// they can share it; calls on different streams get different buffers.  If
// the stream is recording a graph, the allocation is made in the relaxed
// capture mode (it is not part of the graph and outlives it).

#include "kernels.hpp"

#include <map>
#include <mutex>
#include <utility>

namespace rthip {

hipError_t stream_workspace(hipStream_t stream, float** out) {
    static std::mutex guard;
    static std::map<std::pair<int, hipStream_t>, float*> buffers;
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) {
        return status;
    }
    const std::pair<int, hipStream_t> key(device, stream);
    const std::lock_guard<std::mutex> lock(guard);
    const auto found = buffers.find(key);
    if (found != buffers.end()) {
        *out = found->second;
        return hipSuccess;
    }
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    status = hipThreadExchangeStreamCaptureMode(&mode);
    if (status != hipSuccess) {
        return status;
    }
    void* fresh = nullptr;
    status = hipMalloc(&fresh, kStreamWorkspaceBytes);
    const hipError_t restored = hipThreadExchangeStreamCaptureMode(&mode);
    if (status != hipSuccess) {
        return status;
    }
    // kept even if the capture mode could not be restored: the buffer exists
    buffers.emplace(key, static_cast<float*>(fresh));
    if (restored != hipSuccess) {
        return restored;
    }
    *out = static_cast<float*>(fresh);
    return hipSuccess;
}

}  // namespace rthip
