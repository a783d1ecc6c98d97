// The (low nibble, high nibble) -> (level, level) pair table that the decode
// GEMV and the small-batch kernel use to turn one code BYTE into two fp32
// codebook levels with one ds_read_b64.
//
// Layout: entry-major with 32 interleaved replicas; replica k of entry e sits
// at byte e * 256 + k * 8 and lane l reads replica l % 32.  An entry's 256
// bytes span all 64 LDS banks of the CU, so the 32 lanes served per clock
// always touch 32 different bank pairs whatever their codes are (16 replicas
// in 128 bytes measured 2 conflict cycles per 64-lane read), and an entry's
// address is (byte << 8) | ((l % 32) << 3): ONE
// v_perm_b32 that drops the code byte into bits 8..15 above the lane's fixed
// low byte.  Levels are the literals of src/core/quantization/nf4.cpp:14-31
// (under /root/reference), built from instruction immediates so that the build
// cannot stall behind the streaming loads.
#pragma once

#include <hip/hip_runtime.h>

namespace rthip {

constexpr int kReplicas = 32;      // interleaved copies of the pair table
constexpr int kEntryStride = 256;  // bytes between table entries
constexpr int kPairTableBytes = 256 * kEntryStride;

// codebook[n] selected with compare/select on instruction literals (no memory
// access, so it cannot stall behind the streaming loads).
__device__ __forceinline__ float codebook_literal(unsigned n) {
    const float lo0 = (n & 1U) ? -0.6961928009986877F : -1.0F;
    const float lo1 = (n & 1U) ? -0.39491748809814453F : -0.5250730514526367F;
    const float lo2 = (n & 1U) ? -0.18477343022823334F : -0.28444138169288635F;
    const float lo3 = (n & 1U) ? 0.0F : -0.09105003625154495F;
    const float hi0 = (n & 1U) ? 0.16093020141124725F : 0.07958029955625534F;
    const float hi1 = (n & 1U) ? 0.33791524171829224F : 0.24611230194568634F;
    const float hi2 = (n & 1U) ? 0.5626170039176941F : 0.44070982933044434F;
    const float hi3 = (n & 1U) ? 1.0F : 0.7229568362236023F;
    const float a = (n & 2U) ? lo1 : lo0;
    const float b = (n & 2U) ? lo3 : lo2;
    const float c = (n & 2U) ? hi1 : hi0;
    const float d = (n & 2U) ? hi3 : hi2;
    const float low = (n & 4U) ? b : a;
    const float high = (n & 4U) ? d : c;
    return (n & 8U) ? high : low;
}

// Level of nibble 4 * quarter + i (i is a compile-time constant).
template <int kIndex>
__device__ __forceinline__ float level_in_quarter(unsigned quarter) {
    constexpr float kLevels[16] = {
        -1.0F, -0.6961928009986877F, -0.5250730514526367F,
        -0.39491748809814453F, -0.28444138169288635F, -0.18477343022823334F,
        -0.09105003625154495F, 0.0F, 0.07958029955625534F,
        0.16093020141124725F, 0.24611230194568634F, 0.33791524171829224F,
        0.44070982933044434F, 0.5626170039176941F, 0.7229568362236023F, 1.0F};
    const float low = (quarter & 1U) ? kLevels[4 + kIndex] : kLevels[kIndex];
    const float high =
        (quarter & 1U) ? kLevels[12 + kIndex] : kLevels[8 + kIndex];
    return (quarter & 2U) ? high : low;
}

// Builds the replicated pair table with all kThreads threads of the
// workgroup.  A thread fills two neighbouring replicas (one 16-byte store) of
// 2048 / kThreads consecutive entries, in groups of four that share a high
// nibble and a low-nibble quarter.  Eight consecutive lanes write the 128
// bytes of one entry, which is what the LDS takes per clock.
template <int kThreads>
__device__ __forceinline__ void build_pair_table(char* table) {
    // at most 512 threads build (four entries each); the others skip
    constexpr int kBuilders = kThreads > 512 ? 512 : kThreads;
    constexpr int kEntries = 256 * (kReplicas / 2) / kBuilders;  // per thread
    static_assert(kEntries >= 4 && kEntries % 4 == 0);
    if (kBuilders < kThreads && threadIdx.x >= kBuilders) {
        return;
    }
    const unsigned replica_pair = threadIdx.x % (kReplicas / 2);
    const unsigned first_entry = (threadIdx.x / (kReplicas / 2)) * kEntries;
    char* slot = table + replica_pair * sizeof(float4);
#pragma unroll
    for (int group = 0; group < kEntries / 4; ++group) {
        const unsigned entry = first_entry + 4 * group;
        const float high_level = codebook_literal(entry >> 4);
        const unsigned quarter = (entry >> 2) & 3U;
        float4* target =
            reinterpret_cast<float4*>(slot + entry * kEntryStride);
        constexpr int kStep = kEntryStride / sizeof(float4);
        const float low0 = level_in_quarter<0>(quarter);
        const float low1 = level_in_quarter<1>(quarter);
        const float low2 = level_in_quarter<2>(quarter);
        const float low3 = level_in_quarter<3>(quarter);
        target[0 * kStep] = make_float4(low0, high_level, low0, high_level);
        target[1 * kStep] = make_float4(low1, high_level, low1, high_level);
        target[2 * kStep] = make_float4(low2, high_level, low2, high_level);
        target[3 * kStep] = make_float4(low3, high_level, low3, high_level);
    }
}

// The lane's fixed low address byte.
__device__ __forceinline__ unsigned pair_table_lane_bits(unsigned lane) {
    return (lane % kReplicas) * sizeof(float2);  // < 256
}

// (level[low nibble], level[high nibble]) of byte `byte` (0..3) of `word`.
__device__ __forceinline__ float2 pair_table_lookup(const char* table,
                                                    unsigned word, int byte,
                                                    unsigned lane_bits) {
    // v_perm_b32 selector: (byte b of the code word) << 8 | lane_bits
    const unsigned selector = 0x0C0C0400U + (static_cast<unsigned>(byte) << 8);
    const unsigned address = __builtin_amdgcn_perm(word, lane_bits, selector);
    return *reinterpret_cast<const float2*>(table + address);
}

}  // namespace rthip
