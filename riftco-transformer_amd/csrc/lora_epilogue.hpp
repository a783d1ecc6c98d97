// The low-rank adapter term of a Linear's forward, fused into the epilogue of
// the packed-weight kernels:
//     y[m, n] = (acc[m, n] + bias[n]) + scale * sum_j reduced[m, j] * B[n, j]
// restating LowRankAdapter::forward (src/nn/low_rank_adapter.cpp:126-151, under
// /root/reference) as Linear::forward composes it (src/nn/linear.cpp:165-172):
// `reduced` = x A^T is produced beforehand by the kernel in lora.hip, the sum
// over the rank runs in ascending j in fp32 like the reference's matmul
// (src/core/backend/adapters/cpu/adapter.cpp:158-203), the scale multiplies
// that sum, and the result is added to the biased base output.
//
// The input backward uses the same epilogue for the adapter's share of dx,
//     dx[m, i] = acc[m, i] + sum_j d_reduced[m, j] * A[j, i]
// (matmul's closure for its left operand, src/core/autograd/operations.cpp:
// 252-277, met with the base gradient by Variable::accumulate_gradient,
// src/core/autograd/graph.cpp:218-242): `reduced` is then d_reduced, `b` is
// A [rank, input_width] read down a column (row stride 1, rank stride
// input_width) and the scale is one.
#pragma once

#include <hip/hip_runtime.h>

namespace rthip {

struct LoraEpilogue {
    const float* reduced;  // [rows, rank], null when there is no adapter
    // the second factor: element j of output column n is
    // b[n * row_stride + j * rank_stride]
    const float* b;
    unsigned rank;
    float scale;
    unsigned row_stride = 0;   // forward: rank; input backward: 1
    unsigned rank_stride = 1;  // forward: 1;    input backward: input_width
};

// term[i] = scale * sum_j reduced_rows[i][j] * b_row[j * rank_stride] for
// kCount outputs that share one output column.  Every reduced pointer must be
// readable for `rank` floats.
template <int kCount>
__device__ __forceinline__ void lora_terms(
    float (&term)[kCount], const float* __restrict__ b_row,
    const float* const (&reduced_rows)[kCount], unsigned rank, float scale,
    unsigned rank_stride
) {
#pragma unroll
    for (int i = 0; i < kCount; ++i) {
        term[i] = 0.0F;
    }
    unsigned j = 0;
    if (rank_stride != 1) {  // uniform: a column of A
        if (rank % 4 == 0) {
            for (; j < rank; j += 4) {
                float b[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    b[e] = b_row[static_cast<std::size_t>(j + e) * rank_stride];
                }
#pragma unroll
                for (int i = 0; i < kCount; ++i) {
                    const float4 r =
                        *reinterpret_cast<const float4*>(reduced_rows[i] + j);
                    term[i] += r.x * b[0];
                    term[i] += r.y * b[1];
                    term[i] += r.z * b[2];
                    term[i] += r.w * b[3];
                }
            }
        }
        for (; j < rank; ++j) {
            const float b = b_row[static_cast<std::size_t>(j) * rank_stride];
#pragma unroll
            for (int i = 0; i < kCount; ++i) {
                term[i] += reduced_rows[i][j] * b;
            }
        }
    } else if (rank % 4 == 0) {  // uniform: rows are then 16-byte aligned
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
    lora_terms<1>(term,
                  lora.b + static_cast<std::size_t>(n) * lora.row_stride, rows,
                  lora.rank, lora.scale, lora.rank_stride);
    return term[0];
}

}  // namespace rthip
