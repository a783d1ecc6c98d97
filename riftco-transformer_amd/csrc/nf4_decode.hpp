// Device-side NF4 decode shared by every kernel of the packed linear path.
//
// Semantics restated from the reference (paths under /root/reference):
//   codebook literals      src/core/quantization/nf4.cpp:14-31
//   nibble order           src/core/quantization/nf4.cpp:70-75
//   block-scale decode     src/core/backend/nn/quantized_linear/storage.hpp:46-65
//   weight decode          src/core/backend/nn/quantized_linear/reference/operations.cpp:32-45
//
// Bit-exactness rules kept here: the scale decode uses a correctly rounded
// division, a separately rounded multiply and a separately rounded add (no
// fused multiply-add), and a weight is codebook[code] * scale in one rounded
// multiply.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace rthip {

// Description of one packed weight in device memory; the six values the
// C ABI receives (include/rthip.h).
struct Nf4WeightView {
    const std::uint8_t* codes;
    const void* primary_scales;     // float[blocks] or uint8[blocks]
    const float* secondary_scales;  // float[groups] for double quantisation
    int encoding;                   // 0 = fp32 absmax, 1 = double-quantised uint8
    unsigned second_level_shift;    // log2(second-level block)
    float offset;
};

__device__ __constant__ const float kNf4Codebook[16] = {
    -1.0F,
    -0.6961928009986877F,
    -0.5250730514526367F,
    -0.39491748809814453F,
    -0.28444138169288635F,
    -0.18477343022823334F,
    -0.09105003625154495F,
    0.0F,
    0.07958029955625534F,
    0.16093020141124725F,
    0.24611230194568634F,
    0.33791524171829224F,
    0.44070982933044434F,
    0.5626170039176941F,
    0.7229568362236023F,
    1.0F,
};

// Copies the codebook into a 16-float LDS table.  Sixteen consecutive dwords
// sit in sixteen different banks, so a per-lane lookup never conflicts: lanes
// with equal codes broadcast, lanes with different codes hit different banks.
__device__ __forceinline__ void load_codebook_to_lds(float* table) {
    if (threadIdx.x < 16) {
        table[threadIdx.x] = kNf4Codebook[threadIdx.x];
    }
}

// Block scale of a double-quantised weight.  Every operation below must round
// on its own: the pragma keeps the compiler from contracting the multiply and
// the add into one fused multiply-add, and plain operators are used because
// only code written inside this scope is covered by it.  Division of fp32 is
// correctly rounded in HIP by default.
// The part after the division: factor = (float)(code - 128) / 127.0F.
__device__ __forceinline__ float double_quantized_scale_from_factor(
    float factor, float second_level, float offset
) {
#pragma clang fp contract(off)
    const float delta = second_level * factor;
    constexpr float kMaxFinite = 0x1.fffffep+127F;
    if (delta > 0.0F && offset > kMaxFinite - delta) {
        return kMaxFinite;
    }
    const float reconstructed = offset + delta;
    return reconstructed > 0.0F ? reconstructed : 0.0F;
}

__device__ __forceinline__ float decode_double_quantized_scale(
    std::uint8_t scale_code, float second_level, float offset
) {
#pragma clang fp contract(off)
    const int centered = static_cast<int>(scale_code) - 128;
    const float factor = static_cast<float>(centered) / 127.0F;
    return double_quantized_scale_from_factor(factor, second_level, offset);
}

template <bool kDoubleQuantized>
__device__ __forceinline__ float load_block_scale(
    const Nf4WeightView& weight, std::size_t block
) {
    if constexpr (!kDoubleQuantized) {
        return static_cast<const float*>(weight.primary_scales)[block];
    } else {
        const std::uint8_t code =
            static_cast<const std::uint8_t*>(weight.primary_scales)[block];
        const float second =
            weight.secondary_scales[block >> weight.second_level_shift];
        return decode_double_quantized_scale(code, second, weight.offset);
    }
}

// Runtime-encoding form for the shape-agnostic kernels.
__device__ __forceinline__ float load_block_scale_any(
    const Nf4WeightView& weight, std::size_t block
) {
    return weight.encoding == 0 ? load_block_scale<false>(weight, block)
                                : load_block_scale<true>(weight, block);
}

__device__ __forceinline__ unsigned unpack_code(
    const std::uint8_t* codes, std::size_t flat_index
) {
    const unsigned packed = codes[flat_index >> 1];
    return (flat_index & 1U) == 0U ? (packed & 0x0FU) : (packed >> 4U);
}

}  // namespace rthip
