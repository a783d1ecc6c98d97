// TEST INFRASTRUCTURE ONLY.  A C-callable wrapper around the reference's own
// reader of the packed model state (parse_packed_model_state,
// src/c_api/model_state.cpp:166-300), compiled from the reference's sources
// where they lie under /root/reference (recipe: oracle/Makefile, target _ref,
// output _ref/libstateref.so).  Only that function is reachable from the
// exported symbols; the rest of its translation unit (the model-level entry
// points) is dropped by the linker's section garbage collection, so no model
// code is built or linked.  Nothing of the reference is copied here.

#include "internal/model_state.hpp"

#include <cstring>
#include <string>

namespace {

using riftco_transformer::PackedLinearWeightState;

thread_local std::vector<PackedLinearWeightState> g_parsed;
thread_local std::string g_message;

}  // namespace

#define STATEREF_API extern "C" __attribute__((visibility("default")))

// 0 ok, 1 invalid_argument, 3 overflow_error, 255 anything else.
STATEREF_API int stateref_parse(const std::uint8_t* bytes, std::size_t size) {
    g_parsed.clear();
    g_message.clear();
    try {
        g_parsed = riftco_transformer::c_api::detail::parse_packed_model_state(
            std::span<const std::uint8_t>(bytes, size));
        return 0;
    } catch (const std::invalid_argument& error) {
        g_message = error.what();
        return 1;
    } catch (const std::overflow_error& error) {
        g_message = error.what();
        return 3;
    } catch (const std::exception& error) {
        g_message = error.what();
        return 255;
    }
}

STATEREF_API const char* stateref_message() { return g_message.c_str(); }

STATEREF_API std::size_t stateref_weight_count() { return g_parsed.size(); }

// header[0..8] = dimension 0, dimension 1, block size, packed code bytes,
// fp32 block scales, scale codes, second-level scales, second-level block
// size, nested flag; *offset_bits = bit pattern of the offset.
STATEREF_API int stateref_weight_header(std::size_t index,
                                        std::uint64_t* header,
                                        std::uint32_t* offset_bits) {
    if (index >= g_parsed.size() || g_parsed[index].shape.size() != 2) {
        return 1;
    }
    const auto& weight = g_parsed[index];
    const auto& nested = weight.payload.double_quantized_scales;
    header[0] = weight.shape[0];
    header[1] = weight.shape[1];
    header[2] = weight.block_size;
    header[3] = weight.payload.packed_codes.size();
    header[4] = weight.payload.block_scales.size();
    header[5] = nested ? nested->scale_codes.size() : 0;
    header[6] = nested ? nested->second_level_scales.size() : 0;
    header[7] = nested ? nested->scale_block_size : 0;
    header[8] = nested ? 1 : 0;
    const float offset = nested ? nested->offset : 0.0F;
    std::memcpy(offset_bits, &offset, sizeof(offset));
    return 0;
}

// Copies the four payload arrays (sizes as reported by the header; a pointer
// may be NULL when its count is zero).
STATEREF_API int stateref_weight_payload(std::size_t index,
                                         std::uint8_t* packed_codes,
                                         float* block_scales,
                                         std::uint8_t* scale_codes,
                                         float* second_level_scales) {
    if (index >= g_parsed.size()) {
        return 1;
    }
    const auto& payload = g_parsed[index].payload;
    const auto copy = [](auto* destination, const auto& source) {
        if (!source.empty()) {
            std::memcpy(destination, source.data(),
                        source.size() * sizeof(source[0]));
        }
    };
    copy(packed_codes, payload.packed_codes);
    copy(block_scales, payload.block_scales);
    if (payload.double_quantized_scales) {
        copy(scale_codes, payload.double_quantized_scales->scale_codes);
        copy(second_level_scales,
             payload.double_quantized_scales->second_level_scales);
    }
    return 0;
}
