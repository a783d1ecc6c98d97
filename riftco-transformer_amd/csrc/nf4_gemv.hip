// Streaming GEMV for decode-sized row counts (rows <= 4):
//     y[r, o] = sum_i x[r, i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81) for the
// HBM-bound case, where the only traffic that matters is the packed codes and
// their scales, each read exactly once.
//
// Work split.  A workgroup of four wavefronts owns kRows consecutive weight
// rows.  The contraction axis is cut into 16-weight segments (8 bytes of
// codes); thread t owns segments t, t + 256, ... of EVERY row, so
//   * a wavefront's loads of one row are 512 contiguous bytes,
//   * the x values a thread needs never change: they are loaded once into
//     registers and reused for all rows (x costs no LDS or cache bandwidth in
//     the row loop),
//   * a segment lies inside one quantisation block (block sizes are powers of
//     two >= 32 and the row width is a multiple of 16), so a thread applies
//     one scale per segment:  acc += scale * sum_i x_i * codebook[c_i].
// All loads of a workgroup's rows are issued before the first use, which
// keeps ~32 KB per CU in flight.  Nibble -> fp32 goes through a 16-entry LDS
// table (conflict-free by construction).  Row sums are reduced across the
// wavefront with shuffles and across the four wavefronts through LDS.

#include "kernels.hpp"
#include "nf4_decode.hpp"

namespace rthip {
namespace {

constexpr int kThreads = 256;
constexpr int kWave = 64;
constexpr int kWaves = kThreads / kWave;
constexpr int kSegment = 16;  // weights per thread per row visit

__device__ __forceinline__ float wave_sum(float value) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        value += __shfl_xor(value, offset, kWave);
    }
    return value;
}

template <int kX, int kSegments, int kRows, bool kDoubleQuantized>
__global__ __launch_bounds__(kThreads) void gemv_forward_kernel(
    const float* __restrict__ x, Nf4WeightView weight,
    const float* __restrict__ bias, float* __restrict__ y,
    unsigned input_width, unsigned output_width, unsigned block_shift
) {
    __shared__ float table[16];
    __shared__ float partial[kWaves][kRows][kX];
    load_codebook_to_lds(table);

    const unsigned thread = threadIdx.x;
    const unsigned segment_count = input_width / kSegment;

    // This thread's slice of x, resident for the whole kernel.
    float xs[kX][kSegments][kSegment];
#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
        const unsigned segment = thread + kThreads * j;
        const bool valid = segment < segment_count;
#pragma unroll
        for (int r = 0; r < kX; ++r) {
            const float4* source = reinterpret_cast<const float4*>(
                x + static_cast<std::size_t>(r) * input_width +
                static_cast<std::size_t>(segment) * kSegment);
#pragma unroll
            for (int q = 0; q < kSegment / 4; ++q) {
                const float4 v =
                    valid ? source[q] : make_float4(0.0F, 0.0F, 0.0F, 0.0F);
                xs[r][j][4 * q + 0] = v.x;
                xs[r][j][4 * q + 1] = v.y;
                xs[r][j][4 * q + 2] = v.z;
                xs[r][j][4 * q + 3] = v.w;
            }
        }
    }

    const unsigned first_row = blockIdx.x * kRows;

    // Issue every load of this workgroup's rows before any use.
    uint2 codes[kRows][kSegments];
    float scales[kRows][kSegments];
#pragma unroll
    for (int row = 0; row < kRows; ++row) {
        const unsigned o = first_row + row;
#pragma unroll
        for (int j = 0; j < kSegments; ++j) {
            const unsigned segment = thread + kThreads * j;
            const bool valid = segment < segment_count && o < output_width;
            const std::size_t flat =
                static_cast<std::size_t>(o) * input_width +
                static_cast<std::size_t>(segment) * kSegment;
            // An absent segment decodes to code 7 (0.0) with scale 0.
            codes[row][j] = valid
                ? *reinterpret_cast<const uint2*>(weight.codes + (flat >> 1))
                : make_uint2(0x77777777U, 0x77777777U);
            scales[row][j] = valid
                ? load_block_scale<kDoubleQuantized>(weight,
                                                     flat >> block_shift)
                : 0.0F;
        }
    }

    __syncthreads();  // codebook table visible

    float acc[kRows][kX];
#pragma unroll
    for (int row = 0; row < kRows; ++row) {
#pragma unroll
        for (int r = 0; r < kX; ++r) {
            acc[row][r] = 0.0F;
        }
#pragma unroll
        for (int j = 0; j < kSegments; ++j) {
            float sums[kX];
#pragma unroll
            for (int r = 0; r < kX; ++r) {
                sums[r] = 0.0F;
            }
            const unsigned words[2] = {codes[row][j].x, codes[row][j].y};
#pragma unroll
            for (int w = 0; w < 2; ++w) {
#pragma unroll
                for (int n = 0; n < 8; ++n) {
                    const float level = table[(words[w] >> (4 * n)) & 0xFU];
#pragma unroll
                    for (int r = 0; r < kX; ++r) {
                        sums[r] += xs[r][j][8 * w + n] * level;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < kX; ++r) {
                acc[row][r] += sums[r] * scales[row][j];
            }
        }
    }

    const unsigned wave = thread / kWave;
    const unsigned lane = thread % kWave;
#pragma unroll
    for (int row = 0; row < kRows; ++row) {
#pragma unroll
        for (int r = 0; r < kX; ++r) {
            const float total = wave_sum(acc[row][r]);
            if (lane == 0) {
                partial[wave][row][r] = total;
            }
        }
    }
    __syncthreads();

    if (thread < kRows * kX) {
        const unsigned row = thread / kX;
        const unsigned r = thread % kX;
        const unsigned o = first_row + row;
        if (o < output_width) {
            float total = 0.0F;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                total += partial[w][row][r];
            }
            if (bias != nullptr) {
                total += bias[o];
            }
            y[static_cast<std::size_t>(r) * output_width + o] = total;
        }
    }
}

template <int kX, int kSegments, bool kDoubleQuantized>
void launch_instance(const LinearProblem& p, hipStream_t stream) {
    // Fewer rows per workgroup when a thread carries more state.
    constexpr int kRows = (kX * kSegments <= 2) ? 8 : 4;
    const unsigned blocks =
        static_cast<unsigned>((p.output_width + kRows - 1) / kRows);
    gemv_forward_kernel<kX, kSegments, kRows, kDoubleQuantized>
        <<<blocks, kThreads, 0, stream>>>(
            p.activations, p.weight, p.bias, p.result,
            static_cast<unsigned>(p.input_width),
            static_cast<unsigned>(p.output_width), p.block_shift);
}

template <int kX, bool kDoubleQuantized>
void launch_segments(const LinearProblem& p, hipStream_t stream) {
    const std::size_t per_thread =
        (p.input_width / kSegment + kThreads - 1) / kThreads;
    switch (per_thread) {
    case 1: launch_instance<kX, 1, kDoubleQuantized>(p, stream); break;
    case 2: launch_instance<kX, 2, kDoubleQuantized>(p, stream); break;
    case 3: launch_instance<kX, 3, kDoubleQuantized>(p, stream); break;
    default: launch_instance<kX, 4, kDoubleQuantized>(p, stream); break;
    }
}

template <bool kDoubleQuantized>
void launch_rows(const LinearProblem& p, hipStream_t stream) {
    switch (p.rows) {
    case 1: launch_segments<1, kDoubleQuantized>(p, stream); break;
    case 2: launch_segments<2, kDoubleQuantized>(p, stream); break;
    case 3: launch_segments<3, kDoubleQuantized>(p, stream); break;
    default: launch_segments<4, kDoubleQuantized>(p, stream); break;
    }
}

}  // namespace

bool gemv_forward_supports(const LinearProblem& p) {
    constexpr std::size_t kMaxWidth =
        static_cast<std::size_t>(kSegment) * kThreads * 4;
    // x rows times segments per thread bounds the register-resident x slice.
    const std::size_t per_thread =
        (p.input_width / kSegment + kThreads - 1) / kThreads;
    return p.rows >= 1 && p.rows <= kGemvMaxRows &&
           p.rows * per_thread <= 8 &&
           p.input_width % kSegment == 0 && p.input_width <= kMaxWidth &&
           p.output_width < (1ULL << 31) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 8 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

void launch_gemv_forward(const LinearProblem& p, hipStream_t stream) {
    if (p.weight.encoding == 0) {
        launch_rows<false>(p, stream);
    } else {
        launch_rows<true>(p, stream);
    }
}

}  // namespace rthip
