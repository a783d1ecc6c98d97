// Per-stream scratch memory for kernels that exchange partial results between
// workgroups (the small-batch forward and input backward, the tiled GEMM's
// leftover tiles, the split-K dense matmul) and for the few status words the
// quantizer and the payload check hand back to the host.
//
// One buffer of kStreamWorkspaceBytes (+ kStatusWords status words) per
// (device, stream), allocated on first use and kept until
// release_stream_workspaces: calls on one stream are ordered on the device,
// so they can share it; calls on different streams get different buffers.
// If the stream is recording a graph, the allocation is made in the relaxed
// capture mode (it is not part of the graph and outlives it).
//
// A call that uses the buffer issues more than one launch (partial results,
// then their sum).  Two host threads may launch on the same stream at once,
// and the device would then run A's partials, B's partials, A's sum, B's sum:
// A's sum would read B's partial results.  A lease therefore holds the
// buffer's mutex until every launch of the call has been enqueued, which
// makes the stream order A, A, B, B.  (A graph captured from one stream and
// replayed on another while the first still runs eager work is not covered:
// the graph names the capture stream's buffer.)

#include "kernels.hpp"

#include <map>
#include <memory>
#include <mutex>
#include <utility>

namespace rthip {
namespace {

struct Workspace {
    float* data = nullptr;
    std::mutex busy;
};

struct Registry {
    std::mutex guard;
    std::map<std::pair<int, hipStream_t>, std::unique_ptr<Workspace>> buffers;
};

Registry& registry() {
    static Registry* const instance = new Registry;  // never destroyed
    return *instance;
}

}  // namespace

hipError_t lease_stream_workspace(hipStream_t stream, WorkspaceLease* lease) {
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) {
        return status;
    }
    Registry& all = registry();
    Workspace* workspace = nullptr;
    {
        // `busy` is taken while `guard` is still held (the order in which
        // release_stream_workspaces takes them): a release that runs between
        // the lookup and the lease cannot free the buffer under the caller.
        const std::pair<int, hipStream_t> key(device, stream);
        const std::lock_guard<std::mutex> lock(all.guard);
        const auto found = all.buffers.find(key);
        if (found != all.buffers.end()) {
            workspace = found->second.get();
        } else {
            hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
            status = hipThreadExchangeStreamCaptureMode(&mode);
            if (status != hipSuccess) {
                return status;
            }
            void* fresh = nullptr;
            status = hipMalloc(&fresh, kStreamWorkspaceBytes +
                                           kStatusWords * sizeof(std::uint64_t));
            const hipError_t restored =
                hipThreadExchangeStreamCaptureMode(&mode);
            if (status != hipSuccess) {
                return status;
            }
            // kept even if the capture mode could not be restored: the
            // buffer exists
            auto entry = std::make_unique<Workspace>();
            entry->data = static_cast<float*>(fresh);
            workspace = entry.get();
            all.buffers.emplace(key, std::move(entry));
            if (restored != hipSuccess) {
                return restored;
            }
        }
        lease->lock_ = std::unique_lock<std::mutex>(workspace->busy);
    }
    lease->data_ = workspace->data;
    return hipSuccess;
}

hipError_t release_stream_workspaces(hipStream_t stream, bool every_stream) {
    int device = 0;
    hipError_t status = hipGetDevice(&device);
    if (status != hipSuccess) {
        return status;
    }
    Registry& all = registry();
    const std::lock_guard<std::mutex> lock(all.guard);
    for (auto entry = all.buffers.begin(); entry != all.buffers.end();) {
        if (entry->first.first != device ||
            (!every_stream && entry->first.second != stream)) {
            ++entry;
            continue;
        }
        {
            // waits for a call that is still enqueueing
            const std::lock_guard<std::mutex> busy(entry->second->busy);
            // hipFree waits for the device to finish with the memory
            const hipError_t freed = hipFree(entry->second->data);
            if (freed != hipSuccess && status == hipSuccess) {
                status = freed;
            }
        }
        entry = all.buffers.erase(entry);
    }
    return status;
}

}  // namespace rthip
