// Pieces of the decode-sized forward kernel (nf4_gemv.hip) that do not depend
// on its template parameters: the description of the weights of a launch,
// buffer descriptors and moves between lanes.
#pragma once

#include "kernels.hpp"

#include <cstdint>

namespace rthip {
namespace {

constexpr int kWave = 64;
constexpr int kRowLanes = 16;      // lanes of one DPP row

typedef unsigned uint2_vec __attribute__((ext_vector_type(2)));

// value of lane (l ^ kXor) within the 16-lane DPP row, vector ALU only.
template <int kXor>
__device__ __forceinline__ float dpp_xor(float value) {
    const int bits = __builtin_bit_cast(int, value);
    int moved;
    if constexpr (kXor == 1) {
        moved = __builtin_amdgcn_update_dpp(0, bits, 0xB1, 0xF, 0xF, false);
    } else if constexpr (kXor == 2) {
        moved = __builtin_amdgcn_update_dpp(0, bits, 0x4E, 0xF, 0xF, false);
    } else if constexpr (kXor == 4) {
        // lanes 0-3 and 8-11 read four lanes up, the others four lanes down
        moved = __builtin_amdgcn_update_dpp(0, bits, 0x104, 0xF, 0x5, false);
        moved =
            __builtin_amdgcn_update_dpp(moved, bits, 0x114, 0xF, 0xA, false);
    } else {
        static_assert(kXor == 8);
        moved = __builtin_amdgcn_update_dpp(0, bits, 0x128, 0xF, 0xF, false);
    }
    return __builtin_bit_cast(float, moved);
}

// v_permlane16_swap_b32 / v_permlane32_swap_b32: exchanges between two
// registers across lanes on the vector ALU -- the LDS crossbar (ds_bpermute,
// what __shfl_xor compiles to) and its round trip are not involved.  With the
// wavefront's four 16-lane rows written r0 r1 r2 r3:
//     swap_rows:   a = a0 a1 a2 a3, b = b0 b1 b2 b3  ->  a = a0 b0 a2 b2,
//                                                        b = a1 b1 a3 b3
//     swap_halves: a = a0 a1 a2 a3, b = b0 b1 b2 b3  ->  a = a0 a1 b0 b1,
//                                                        b = a2 a3 b2 b3
// Written as assembly because the compiler's builtins return the FIRST result
// twice when both operands hold the same value (seen with ROCm 7.2: the add
// below became v_add v1, v1, v1).  The instruction may not directly follow a
// vector ALU write of its operands: two wait states, hence the s_nop, which
// the compiler's hazard pass would add for the builtin but not for assembly.
__device__ __forceinline__ void swap_rows(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1"
                 : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_halves(float& a, float& b) {
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1"
                 : "+v"(a), "+v"(b));
}

// Sum of `value` over the wavefront's four rows, in every lane: lane l ends
// with value(l) + value(l ^ 16) + (the same of lanes l ^ 32 and l ^ 48).
// Bit-identical to value += shfl_xor(value, 16); value += shfl_xor(value, 32).
__device__ __forceinline__ float sum_over_rows(float value) {
    float twin = value;
    swap_rows(value, twin);  // rows 0 0 2 2 of value and rows 1 1 3 3
    value += twin;
    twin = value;
    swap_halves(value, twin);  // the lower half twice and the upper half twice
    return value + twin;
}

template <int kXor, int kHalf, int kValues>
__device__ __forceinline__ void transposed_step(float (&values)[kValues],
                                                unsigned lane) {
    if constexpr (kHalf >= 1) {
        // Lanes with bit kXor set keep the upper half of the values and hand
        // the lower half to their partner, and vice versa.
        const bool upper = (lane & kXor) != 0;
#pragma unroll
        for (int j = 0; j < kHalf; ++j) {
            float low = values[j];
            float high = values[j + kHalf];
            // Keep the two operands as plain registers: without this the
            // selects below are rewritten into a dynamically indexed read of
            // `values`, which costs a compare/select chain over the array.
            asm volatile("" : "+v"(low), "+v"(high));
            const float keep = upper ? high : low;
            const float send = upper ? low : high;
            values[j] = keep + dpp_xor<kXor>(send);
        }
    } else {
        values[0] += dpp_xor<kXor>(values[0]);
    }
}

// Sum over each 16-lane DPP row of kValues per-lane values.  On return every
// lane holds the row total of value `slot_of_lane(lane)`.
template <int kValues>
__device__ __forceinline__ float transposed_row_sum(float (&values)[kValues],
                                                    unsigned lane) {
    static_assert((kValues & (kValues - 1)) == 0 && kValues <= kRowLanes);
    transposed_step<1, kValues / 2>(values, lane);
    transposed_step<2, kValues / 4>(values, lane);
    transposed_step<4, kValues / 8>(values, lane);
    transposed_step<8, kValues / 16>(values, lane);
    return values[0];
}

// Which value a lane ends up holding after transposed_row_sum: lane bit s
// selected the upper half at step s.
template <int kValues>
__device__ __forceinline__ unsigned slot_of_lane(unsigned lane) {
    unsigned slot = 0;
    unsigned bit = 1;
#pragma unroll
    for (int half = kValues / 2; half >= 1; half /= 2) {
        if (lane & bit) {
            slot += half;
        }
        bit *= 2;
    }
    return slot;
}

// One weight of a launch.  A launch covers up to kGemvGroupMax weights that
// are applied to the same x (the q/k/v or gate/up projections of a layer):
// their row batches are numbered one member after the other, and member m owns
// batches first_batch .. first_batch + ceil(output_width / kRows) - 1.  Unused
// members carry first_batch = 0xFFFFFFFF.
struct GemvMember {
    const std::uint8_t* codes;
    const void* primary_scales;
    const float* secondary_scales;
    const float* bias;
    float* y;
    unsigned output_width;
    unsigned first_batch;
    unsigned secondary_bytes;  // extent of the second-level scale table
    float offset;
};
struct GemvGroup {
    GemvMember member[kGemvGroupMax];
};
static_assert(kGemvGroupMax == 4, "member selection is written for four");

// Field `field` of member m, m per lane (the epilogue): a chain of selects
// over kernel arguments.
#define RTHIP_MEMBER(m, field)                                              \
    (!kGrouped || (m) == 0                                                  \
         ? group.member[0].field                                            \
         : ((m) == 1 ? group.member[1].field                                \
                     : ((m) == 2 ? group.member[2].field                    \
                                 : group.member[3].field)))

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_buffer(const void* base,
                                                             unsigned bytes) {
    // Raw (untyped, stride 0) buffer with range checking on `bytes`.
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0,
                                             static_cast<int>(bytes),
                                             0x00020000);
}

}  // namespace
}  // namespace rthip
