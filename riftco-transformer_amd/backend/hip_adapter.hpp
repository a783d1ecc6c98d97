// The `hip` backend adapter: MI355X implementation of the storage and packed
// NF4 linear capabilities of riftco-transformer's BackendAdapter
// (src/core/backend/adapter.hpp:57-80), next to the reference's CPU, Metal,
// CUDA and TPU adapters.
#pragma once

#if defined(RIFTCO_TRANSFORMER_IN_TREE)
#include "core/backend/adapter.hpp"
#else
#include "interface.hpp"
#endif

#include <cstddef>
#include <cstdint>
#include <memory>
#include <span>
#include <vector>

namespace riftco_transformer::backend_detail {

// ExecutionBackend::Hip.  Spelled as a cast so that this file also compiles
// against a reference tree whose enum has not gained the enumerator yet.
inline constexpr ExecutionBackend kHipBackend =
    static_cast<ExecutionBackend>(4);

// Process-lifetime singleton, like cpu_backend_adapter()
// (src/core/backend/adapters/cpu/adapter.cpp:368-371).
[[nodiscard]] const BackendAdapter& hip_backend_adapter() noexcept;

// A checkpoint's packed model state (src/c_api/model_state.cpp:34-113,
// 166-300) and the hip backend.
//
// hip_load_packed_model_state is what rt_model_packed_state_load
// (src/c_api/model_state.cpp:343-376) does up to the point where the model
// takes the weights -- parse, QuantizedWeight::from_packed_nf4 for every
// entry, nothing returned unless all entries are valid -- except that each
// payload array is copied from `state` straight into HBM and the content
// rules of require_canonical_payload are checked there by a kernel, instead
// of being copied into vectors, scanned on the host and copied again.
// Exceptions and messages are the reference's.
struct HipPackedWeight {
    std::vector<std::size_t> shape;
    std::size_t block_size = 0;
    std::unique_ptr<QuantizedWeightStorage> storage;
};
[[nodiscard]] std::vector<HipPackedWeight> hip_load_packed_model_state(
    std::span<const std::uint8_t> state);

// packed_model_state_bytes (src/c_api/model_state.cpp:34-113) for weights that
// live in hip storage: the arrays are read from HBM into their place in the
// result.
struct HipPackedWeightSource {
    std::span<const std::size_t> shape;
    std::size_t block_size = 0;
    const QuantizedWeightStorage* storage = nullptr;
};
[[nodiscard]] std::vector<std::uint8_t> hip_packed_model_state_bytes(
    std::span<const HipPackedWeightSource> weights);

// Several packed linears applied to ONE input -- the query, key and value
// projections of an attention block
// (src/model/decoder_only_transformer.cpp:406-419) -- in one call: every
// request must name the same input storage and agree in rows, input width,
// block size and scale encoding; outputs are what one
// quantized_linear_forward per request writes, bit for bit, but decode-sized
// inputs go out as one kernel launch per four weights.  Like the capability
// call it stands in for, it expects requests that the dispatcher has already
// validated (dispatch_quantized_linear_forward's checks, once per request).
void hip_quantized_linear_forward_group(
    std::span<const QuantizedLinearForwardRequest> requests);

// Linear::forward of a layer that holds a packed weight, an optional bias and
// a low-rank adapter (src/nn/linear.cpp:147-172 with LowRankAdapter::forward,
// src/nn/low_rank_adapter.cpp:126-151), and the backward pass the reference's
// autograd runs through it (src/core/autograd/operations.cpp:176-194,252-277,
// 480-492; src/nn/quantized_linear.cpp:60-80), each as ONE call on hip
// storage.  A maintainer wraps the pair in a custom-gradient node whose
// closure keeps `input` and `reduced`:
//
//   forward   output = input.deq(W)^T (+ bias) + scale * (input.A^T).B^T,
//             reduced = input.A^T
//   backward  input_gradient  = upstream.deq(W) + ((upstream * scale).B).A
//             lora_a_gradient = ((upstream * scale).B)^T . input
//             lora_b_gradient = (upstream * scale)^T . reduced
//
// Gradients are written, not added to what the storages hold; the reference
// adds them to a node's gradient afterwards (Variable::accumulate_gradient,
// src/core/autograd/graph.cpp:218-242).  Sizes are checked against
// `dimensions` and `rank`; a rank outside [1, min(input, output width)] or a
// scale that is not finite and positive is refused with the messages of
// LowRankAdapter's constructor (src/nn/low_rank_adapter.cpp:27-62).
struct QuantizedLinearAdapterForwardRequest {
    const TensorStorage& input;
    const QuantizedWeightStorage& weight;
    const TensorStorage* bias;  // [output_width] or null
    const TensorStorage& lora_a;  // [rank, input_width]
    const TensorStorage& lora_b;  // [output_width, rank]
    std::size_t rank;
    float scale;  // alpha / rank
    TensorStorage& reduced;  // [rows, rank]
    TensorStorage& output;   // [rows, output_width]
    QuantizedLinearDimensions dimensions;
};
void hip_quantized_linear_adapter_forward(
    const QuantizedLinearAdapterForwardRequest& request);

struct QuantizedLinearAdapterBackwardRequest {
    const TensorStorage& upstream;  // [rows, output_width]
    const TensorStorage& input;     // [rows, input_width]
    const TensorStorage& reduced;   // [rows, rank], from the forward
    const QuantizedWeightStorage& weight;
    const TensorStorage& lora_a;
    const TensorStorage& lora_b;
    std::size_t rank;
    float scale;
    TensorStorage& input_gradient;   // [rows, input_width]
    TensorStorage& lora_a_gradient;  // [rank, input_width]
    TensorStorage& lora_b_gradient;  // [output_width, rank]
    QuantizedLinearDimensions dimensions;
};
void hip_quantized_linear_adapter_backward(
    const QuantizedLinearAdapterBackwardRequest& request);

// Callers that were NOT changed get the same launches: quantized_linear_forward
// calls of up to 128 rows that follow each other on the same input are held
// back and launched together (at most four weights per launch) as soon as a
// call arrives that does not belong to them, another operation of the adapter
// runs, host code reads a tensor, or a device buffer is released.  This is
// the default and implies the queued execution of
// RIFTCO_TRANSFORMER_HIP_ASYNC=1; RIFTCO_TRANSFORMER_HIP_MERGE=0 turns it off.
// requests: forwards that went through the merge; launches: kernel launches
// they became.  Both stay zero while merging is off.
struct HipForwardMergeStatistics {
    std::uint64_t requests = 0;
    std::uint64_t launches = 0;
};
[[nodiscard]] HipForwardMergeStatistics hip_forward_merge_statistics() noexcept;

// Optional extension implemented by hip weight storage: the O(#blocks) scale
// validation that the dispatcher runs before every launch
// (src/core/backend/nn/quantized_linear/dispatch.cpp:98-151) only has to run
// once for storage that can never change.
// (A reference tree whose dispatcher has been taught to consult it declares
// the interface itself, beside QuantizedWeightStorage, and says so.)
#ifndef RIFTCO_TRANSFORMER_HAS_SCALE_VALIDATION_MEMO
class ScaleValidationMemo {
public:
    virtual ~ScaleValidationMemo() = default;
    [[nodiscard]] virtual bool scales_validated() const noexcept = 0;
    virtual void mark_scales_validated() const noexcept = 0;
};
#endif

}  // namespace riftco_transformer::backend_detail
