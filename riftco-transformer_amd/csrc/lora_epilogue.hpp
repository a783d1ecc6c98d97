// The low-rank adapter term of a Linear's forward, fused into the epilogue of
// the packed-weight kernels:
//     y[m, n] = (acc[m, n] + bias[n]) + scale * sum_j reduced[m, j] * B[n, j]
// restating LowRankAdapter::forward (src/nn/low_rank_adapter.cpp:126-151, under
// /root/reference) as Linear::forward composes it (src/nn/linear.cpp:165-172):
// `reduced` = x A^T is produced beforehand by the kernel in lora.hip, the sum
// over the rank runs in ascending j in fp32 like the reference's matmul
// (src/core/backend/adapters/cpu/adapter.cpp:158-203), the scale multiplies
// that sum, and the result is added to the biased base output.
#pragma once

#include <hip/hip_runtime.h>

namespace rthip {

struct LoraEpilogue {
    const float* reduced;  // [rows, rank], null when there is no adapter
    const float* b;        // [output_width, rank]
    unsigned rank;
    float scale;
};

// term[i] = scale * sum_j reduced_rows[i][j] * b_row[j] for kCount outputs that
// share one row of B.  Every pointer must be readable for `rank` floats.
template <int kCount>
__device__ __forceinline__ void lora_terms(
    float (&term)[kCount], const float* __restrict__ b_row,
    const float* const (&reduced_rows)[kCount], unsigned rank, float scale
) {
#pragma unroll
    for (int i = 0; i < kCount; ++i) {
        term[i] = 0.0F;
    }
    unsigned j = 0;
    if (rank % 4 == 0) {  // uniform: rows are then 16-byte aligned
        for (; j < rank; j += 4) {
            const float4 b = *reinterpret_cast<const float4*>(b_row + j);
#pragma unroll
            for (int i = 0; i < kCount; ++i) {
                const float4 r =
                    *reinterpret_cast<const float4*>(reduced_rows[i] + j);
                term[i] += r.x * b.x;
                term[i] += r.y * b.y;
                term[i] += r.z * b.z;
                term[i] += r.w * b.w;
            }
        }
    }
    for (; j < rank; ++j) {
        const float b = b_row[j];
#pragma unroll
        for (int i = 0; i < kCount; ++i) {
            term[i] += reduced_rows[i][j] * b;
        }
    }
#pragma unroll
    for (int i = 0; i < kCount; ++i) {
        term[i] *= scale;
    }
}

// One output.
__device__ __forceinline__ float lora_term(const LoraEpilogue& lora,
                                           unsigned m, unsigned n) {
    float term[1];
    const float* const rows[1] = {lora.reduced +
                                  static_cast<std::size_t>(m) * lora.rank};
    lora_terms<1>(term, lora.b + static_cast<std::size_t>(n) * lora.rank, rows,
                  lora.rank, lora.scale);
    return term[0];
}

}  // namespace rthip
