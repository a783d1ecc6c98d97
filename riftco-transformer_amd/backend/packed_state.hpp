// The packed model state of a checkpoint ("RTNF4S1"): every packed NF4 Linear
// weight of a model in one byte string.  Reader and writer of the format the
// reference defines in src/c_api/model_state.cpp:34-113 (writer) and :166-300
// (reader), with the same checks, exception types and messages.
//
// Unlike the reference's reader, which copies every payload array into a
// vector, parsing here only produces views into the caller's bytes: the hip
// backend copies each array from there straight into device memory.
#pragma once

#include <cstddef>
#include <cstdint>
#include <span>
#include <vector>

namespace riftco_transformer::backend_detail {

// One weight of a packed model state.  The fp32 arrays are viewed as the
// little-endian bytes they are stored as (they need not be aligned).
struct PackedWeightView {
    std::vector<std::size_t> shape;  // rank two
    std::size_t block_size = 0;
    std::span<const std::uint8_t> packed_codes;
    std::span<const std::uint8_t> block_scale_bytes;         // 4 per scale
    bool double_quantized = false;
    std::span<const std::uint8_t> scale_codes;
    std::span<const std::uint8_t> second_level_scale_bytes;  // 4 per scale
    std::size_t scale_block_size = 0;
    float offset = 0.0F;
};

// parse_packed_model_state (src/c_api/model_state.cpp:166-300): the container
// only; whether an entry is a valid NF4 weight is decided by
// require_payload_lengths below and by the content check on the device.
[[nodiscard]] std::vector<PackedWeightView> parse_packed_model_state(
    std::span<const std::uint8_t> bytes);

// The checks of QuantizedWeight::from_packed_nf4 that need no payload data
// (src/core/quantization/quantized_weight.cpp:339-352 with :16-35, :48-53 and
// the length checks of :102-147): supported block sizes, a positive shape
// whose element count is addressable, and array lengths that match it.
// Returns the element count.
std::size_t require_payload_lengths(const PackedWeightView& weight);

// Size of, and offsets into, the bytes that packed_model_state_bytes
// (src/c_api/model_state.cpp:34-113) writes for one weight.
struct PackedWeightLayout {
    std::size_t header = 0;         // offset of the entry's first byte
    std::size_t packed_codes = 0;   // offsets of the four arrays
    std::size_t block_scales = 0;
    std::size_t scale_codes = 0;
    std::size_t second_level_scales = 0;
    std::size_t end = 0;
};

// Appends the header of one entry (everything up to and including the
// dimensions) to `output`, reserves zeroed room for its arrays and says where
// they go.  Array lengths are element counts.
PackedWeightLayout append_packed_weight_header(
    std::vector<std::uint8_t>& output, std::span<const std::size_t> shape,
    std::size_t block_size, std::size_t packed_code_count,
    std::size_t block_scale_count, bool double_quantized,
    std::size_t scale_code_count, std::size_t second_level_scale_count,
    std::size_t scale_block_size, float offset);

// Magic and weight count: the first sixteen bytes.
void append_packed_state_prologue(std::vector<std::uint8_t>& output,
                                  std::size_t weight_count);

}  // namespace riftco_transformer::backend_detail
