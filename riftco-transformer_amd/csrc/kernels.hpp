// Host-callable launchers of the packed NF4 linear kernels.  Each launcher
// only enqueues work on `stream`; shape preconditions are checked by the
// matching *_supports() predicate, which the C ABI consults before launching.
#pragma once

#include "lora_epilogue.hpp"
#include "nf4_decode.hpp"

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <mutex>

namespace rthip {

// One forward (activations = x, result = y) or input-backward
// (activations = dy, result = dx) problem.  The weight is row-major
// [output_width, input_width] in both directions.
struct LinearProblem {
    const float* activations;
    Nf4WeightView weight;
    const float* bias;  // forward only, may be null
    float* result;
    std::size_t rows;
    std::size_t input_width;
    std::size_t output_width;
    unsigned block_shift;  // log2(block_size)
    // low-rank adapter term added in the epilogue (lora.reduced == nullptr:
    // none); forward: reduced . B^T, input backward: d_reduced . A
    LoraEpilogue lora{nullptr, nullptr, 0U, 0.0F};
    // Memory for partial results that the caller brings (a launcher that
    // needs more than scratch_bytes fails with hipErrorOutOfMemory); null:
    // the launcher leases the stream workspace.
    float* scratch = nullptr;
    std::size_t scratch_bytes = 0;
};

// nf4_generic.hip
void launch_generic_forward(const LinearProblem& problem, hipStream_t stream);
hipError_t launch_generic_input_backward(const LinearProblem& problem,
                                         hipStream_t stream);
void launch_dequantize(const Nf4WeightView& weight, float* out,
                       std::size_t element_count, unsigned block_shift,
                       hipStream_t stream);
void launch_fill(float* out, float value, std::size_t count,
                 hipStream_t stream);

// nf4_gemv.hip -- forward only, small row counts.
constexpr std::size_t kGemvMaxRows = 4;
bool gemv_forward_supports(const LinearProblem& problem);
void launch_gemv_forward(const LinearProblem& problem, hipStream_t stream);
// Up to kGemvGroupMax weights applied to the same activations in ONE launch
// (the projections of a layer that share their input).  Every output equals,
// bit for bit, what launch_gemv_forward writes for that member alone.
constexpr std::size_t kGemvGroupMax = 4;
bool gemv_group_supports(const LinearProblem* problems, std::size_t count);
void launch_gemv_group(const LinearProblem* problems, std::size_t count,
                       hipStream_t stream);
// nf4_gemv1.hip -- the same product for ONE row of x (the decode step of a
// model), built around the launch's start and the bytes in flight: `count`
// weights that gemv_group_supports accepts, each of which
// gemv1_forward_supports accepts.  launch_gemv_forward / launch_gemv_group
// route here by themselves.
bool gemv1_forward_supports(const LinearProblem& problem);
// Up to kGemvGroupMax members, each accepted by gemv1_forward_supports, that
// share x, row count, row width and scale encoding; every member may carry its
// own adapter term.
bool gemv1_group_supports(const LinearProblem* problems, std::size_t count);
void launch_gemv1_forward(const LinearProblem* problems, std::size_t count,
                          hipStream_t stream);
// The name of the instance that launch would run, as a profiler prints it
// without its namespace ("gemv1_forward_kernel<1, 8, 2, 4, false, false, 4>").
void gemv1_kernel_name(const LinearProblem* problems, std::size_t count,
                       char* name, std::size_t capacity);

// workspace.hip -- scratch memory shared by the kernels that pass partial
// results between workgroups; one fixed-size buffer per (device, stream),
// followed by kStatusWords 64-bit words for verdicts that go back to the host.
constexpr std::size_t kStreamWorkspaceBytes = std::size_t{64} << 20;
constexpr std::size_t kStatusWords = 8;
// The buffer, and the exclusive right to enqueue launches that use it: hold
// the lease until the call's last launch is enqueued (two threads that launch
// on one stream must not interleave their partial-result and sum kernels).
class WorkspaceLease {
public:
    float* data() const { return data_; }
    // the status words behind the float area (reset them with a kernel)
    std::uint64_t* status_words() const {
        return reinterpret_cast<std::uint64_t*>(
            reinterpret_cast<char*>(data_) + kStreamWorkspaceBytes);
    }

private:
    friend hipError_t lease_stream_workspace(hipStream_t, WorkspaceLease*);
    float* data_ = nullptr;
    std::unique_lock<std::mutex> lock_;
};
hipError_t lease_stream_workspace(hipStream_t stream, WorkspaceLease* lease);
// Frees the buffer of `stream` (or of every stream) on the current device,
// after the device has finished with it.
hipError_t release_stream_workspaces(hipStream_t stream, bool every_stream);

// nf4_skinny.hip -- forward only, up to 64 rows, decode straight into MFMA
// operands.  Shapes whose output tiles are shared between workgroups use a
// per-stream workspace that is allocated on first use, so the launcher can
// fail.
// nf4_resident.hip: up to 128 rows in groups of 16, x resident in registers
constexpr std::size_t kResidentMaxRows = 128;
bool resident_forward_supports(const LinearProblem& problem);
hipError_t launch_resident_forward(const LinearProblem& problem,
                                   hipStream_t stream);
// Up to kResidentGroupMax weights applied to the same activations in ONE
// launch; every output equals, bit for bit, what launch_resident_forward
// writes for that member alone.
constexpr std::size_t kResidentGroupMax = 4;
bool resident_group_supports(const LinearProblem* problems, std::size_t count);
hipError_t launch_resident_group(const LinearProblem* problems,
                                 std::size_t count, hipStream_t stream);

constexpr std::size_t kSkinnyMaxRows = 64;
bool skinny_forward_supports(const LinearProblem& problem);
hipError_t launch_skinny_forward(const LinearProblem& problem,
                                 hipStream_t stream);

// nf4_small_backward.hip -- input backward for up to 64 rows: the weight is
// walked as it lies in memory, a lane owning eight columns of a weight row.
// Uses the stream workspace when the weight rows are cut into chunks.
constexpr std::size_t kSmallBackwardMaxRows = 64;
bool small_input_backward_supports(const LinearProblem& problem);
hipError_t launch_small_input_backward(const LinearProblem& problem,
                                       hipStream_t stream);
// Bytes of partial sums the launch above writes outside dx (0: none).
std::size_t small_input_backward_scratch_bytes(const LinearProblem& problem);

// nf4_stream_backward.hip -- input backward for up to four rows: the weight
// is streamed as it lies in memory, a lane owning sixteen columns, the
// products on the 4 x 4 x 1 matrix instruction.  Uses the stream workspace
// when the weight rows are cut into ranges.
constexpr std::size_t kStreamBackwardMaxRows = 4;
bool stream_input_backward_supports(const LinearProblem& problem);
hipError_t launch_stream_input_backward(const LinearProblem& problem,
                                        hipStream_t stream);

// lora_backward.hip -- the adapter's gradients: d_reduced = (dy * scale) . B
// (always), dB = ((dy * scale)^T . reduced) when d_b is not null and
// dA = (d_reduced^T . x) when d_a is not null.
struct LoraBackwardProblem {
    const float* upstream;     // dy [rows, output_width]
    const float* activations;  // x [rows, input_width] (dA only)
    const float* reduced;      // x . A^T [rows, rank] (dB only)
    const float* b;            // [output_width, rank]
    float* d_reduced;          // [rows, rank]
    float* d_a;                // [rank, input_width] or null
    float* d_b;                // [output_width, rank] or null
    std::size_t rows;
    std::size_t input_width;
    std::size_t output_width;
    std::size_t rank;
    float scale;
};
hipError_t launch_lora_backward(const LoraBackwardProblem& problem,
                                hipStream_t stream);

// lora.hip -- reduced[rows, rank] = x A^T, the input of the adapter epilogue.
void launch_lora_reduce(const float* x, const float* a, float* reduced,
                        std::size_t rows, std::size_t input_width,
                        std::size_t rank, hipStream_t stream);
// The same for several adapters on one x: one launch per four of them while
// the products are few (the one-workgroup-per-output kernel), else one launch
// each; every product equals launch_lora_reduce's
// bit for bit.
constexpr std::size_t kLoraReduceGroupMax = 4;
struct LoraReduceItem {
    const float* a;   // [rank, input_width]
    float* reduced;   // [rows, rank]
    std::size_t rank;
};
void launch_lora_reduce_group(const float* x, const LoraReduceItem* items,
                              std::size_t count, std::size_t rows,
                              std::size_t input_width, hipStream_t stream);

// dense_matmul.hip -- out[b] = left[b] [rows, shared] * right[b] [shared,
// columns], plain fp32.
hipError_t launch_dense_matmul(const float* left, const float* right,
                               float* out, std::size_t batch_count,
                               std::size_t rows, std::size_t shared,
                               std::size_t columns, hipStream_t stream);

// nf4_quantize.hip -- the quantizer.  fp32_scales always receives the block
// scales; scale_codes == nullptr means plain fp32 scales, otherwise the
// scales are double-quantised into scale_codes / second_level / *offset.
// status is a device word the kernels OR error bits into (1: non-finite
// source value, 2: the scale mean is not finite).
struct QuantizeProblem {
    const float* values;
    std::size_t element_count;
    unsigned block_shift;
    std::uint8_t* codes;
    float* fp32_scales;
    std::uint8_t* scale_codes;
    float* second_level;
    unsigned second_level_shift;
    float* offset;     // device
    unsigned* status;  // device, zeroed by the caller
};
void launch_quantize(const QuantizeProblem& problem, hipStream_t stream);

// nf4_check.hip: content rules of a canonical payload.  words is a device
// array of three 64-bit words that the launch initialises and fills;
// classify_payload reads a host copy of it.
enum class PayloadViolation {
    None,
    UnusedNibble,
    SecondLevelScale,
    BlockScale,
    ZeroBlockCode,
};
void launch_check_payload(const Nf4WeightView& weight,
                          std::size_t element_count, unsigned block_shift,
                          std::size_t second_level_count,
                          unsigned long long* words, hipStream_t stream);
PayloadViolation classify_payload(const unsigned long long words[3]);

// nf4_mfma.hip
bool mfma_forward_supports(const LinearProblem& problem);
hipError_t launch_mfma_forward(const LinearProblem& problem,
                               hipStream_t stream);
// Leading 128-wide tile columns of a forward's output that go out as 256-row
// tiles in a launch of their own (0: none; all of them: one launch).
unsigned mfma_forward_tall_tile_columns(std::size_t rows,
                                        std::size_t output_width);
bool mfma_input_backward_supports(const LinearProblem& problem);
hipError_t launch_mfma_input_backward(const LinearProblem& problem,
                                      hipStream_t stream);

}  // namespace rthip
