// Forward product for small batches (4 < rows <= 64):
//     y[r, o] = sum_i x[r, i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81) where
// the weight stream still dominates but there are enough rows to feed the
// matrix cores.
//
// With so few rows every decoded weight is used by ONE tile of x, so staging
// weights through LDS buys nothing: each lane decodes its weights straight into
// the register layout of the MFMA B operand.  x, on the other hand, is shared
// by all wavefronts and is staged through LDS with coalesced loads.
//
//   * v_mfma_f32_16x16x4_f32: A is x[16 rows][4 k], B is W^T[4 k][16 weight
//     rows].  Lane l feeds weight row l % 16 and the k-quarter l / 16.
//   * A workgroup of eight wavefronts owns 16 consecutive weight rows.  The
//     contraction advances in rounds of 512: the workgroup copies
//     x[rows][512] into LDS (row stride padded so that the 16 rows of a
//     fragment read hit distinct banks), then wavefront w handles the 64
//     contraction values [64 w, 64 w + 64) of the round.  There a lane loads
//     8 code bytes (16 weights of its row in its quarter), reads 16 x values per
//     16-row block from LDS, and issues 16 MFMAs per block; MFMA j contracts
//     k = 16 q + j over the four quarters q -- any assignment of k to lanes is
//     valid as long as A and B agree.
//   * The next round's x (in registers) and code bytes are loaded while the
//     current round computes.
//   * Decode: nibble -> level through a 16-entry LDS table (sixteen dwords sit
//     in sixteen banks, so the lookup is conflict-free), times the block scale
//     in one rounded multiply.
//   * The eight partial tiles are added through LDS in a fixed order, so
//     results do not depend on scheduling.

#include "kernels.hpp"
#include "nf4_decode.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uint2_vec __attribute__((ext_vector_type(2)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kTileN = 16;    // weight rows per workgroup
constexpr int kGroup = 64;    // contraction values per wavefront per round
constexpr int kChunk = 16;    // weights per lane per round
constexpr int kRound = kGroup * kWaves;  // 512 contraction values
constexpr int kStride = kRound + 4;      // padded x row stride in floats

// kBlocks: 16-row blocks of x (rows <= 16 * kBlocks).
template <int kBlocks, bool kDoubleQuantized>
__global__ __launch_bounds__(kThreads) void skinny_forward_kernel(
    const float* __restrict__ x, Nf4WeightView weight,
    const float* __restrict__ bias, float* __restrict__ y, unsigned rows,
    unsigned input_width, unsigned output_width, unsigned block_shift
) {
    constexpr int kRows = 16 * kBlocks;
    // float4 loads per thread to copy one round of x
    constexpr int kCopies = kRows * (kRound / 4) / kThreads;  // 4 * kBlocks
    extern __shared__ __attribute__((aligned(16))) float shared[];
    float* x_tile = shared;                                   // kRows * kStride
    float* table = x_tile + kRows * kStride;                  // 16
    float* partial = table + 16;  // (kWaves - 1) * kBlocks * 4 * 64

    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % 64;
    const unsigned wave = thread / 64;
    const unsigned quarter = lane / 16;
    const unsigned n = blockIdx.x * kTileN + lane % 16;
    const std::size_t weight_row =
        static_cast<std::size_t>(min(n, output_width - 1)) * input_width;
    const unsigned round_count = (input_width + kRound - 1) / kRound;

    load_codebook_to_lds(table);

    // Copy plan: thread t moves float4 (t + 512 c) of the [kRows][128] tile.
    const auto load_x = [&](float4 (&staged)[kCopies], unsigned round) {
#pragma unroll
        for (int c = 0; c < kCopies; ++c) {
            const unsigned index = thread + kThreads * c;
            const unsigned row = index / (kRound / 4);
            const unsigned k = round * kRound + (index % (kRound / 4)) * 4;
            staged[c] = (row < rows && k < input_width)
                ? *reinterpret_cast<const float4*>(
                      x + static_cast<std::size_t>(row) * input_width + k)
                : make_float4(0.0F, 0.0F, 0.0F, 0.0F);
        }
    };
    const auto store_x = [&](const float4 (&staged)[kCopies]) {
#pragma unroll
        for (int c = 0; c < kCopies; ++c) {
            const unsigned index = thread + kThreads * c;
            const unsigned row = index / (kRound / 4);
            const unsigned column = (index % (kRound / 4)) * 4;
            *reinterpret_cast<float4*>(x_tile + row * kStride + column) =
                staged[c];
        }
    };
    struct Codes {
        uint2_vec codes;
        float scale;
    };
    const auto load_codes = [&](Codes& staged, unsigned round) {
        const unsigned k = round * kRound + wave * kGroup + quarter * kChunk;
        if (k < input_width) {
            const std::size_t flat = weight_row + k;
            staged.codes = *reinterpret_cast<const uint2_vec*>(
                weight.codes + (flat >> 1));
            staged.scale = load_block_scale<kDoubleQuantized>(
                weight, flat >> block_shift);
        } else {
            staged.codes = uint2_vec{0x77777777U, 0x77777777U};
            staged.scale = 0.0F;
        }
    };

    floatx4 acc[kBlocks];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
        acc[b] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
    }

    // Code bytes run kDepth rounds ahead of their use (a ring of register
    // sets, indexed statically by unrolling the round loop): every round is
    // only 4 KB per workgroup, and without a deep queue of requests the stream
    // would be paced by one memory latency per round.
    constexpr int kDepth = 4;
    float4 x_staged[kCopies];
    Codes ring[kDepth];
    load_x(x_staged, 0);
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        load_codes(ring[d], d);
    }

    // This lane's fragment of the x tile: row lane % 16 of each block, sixteen
    // consecutive values at 64 * wave + 16 * quarter.
    const float* fragment =
        x_tile + (lane % 16) * kStride + wave * kGroup + quarter * kChunk;

    const auto run_round = [&](Codes& slot, unsigned round) {
        __syncthreads();  // the previous round's fragment reads are done
        store_x(x_staged);
        __syncthreads();
        if (round + 1 < round_count) {
            load_x(x_staged, round + 1);
        }

        float w[kChunk];
        {
#pragma clang fp contract(off)
            const unsigned words[2] = {slot.codes.x, slot.codes.y};
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int nibble = 0; nibble < 8; ++nibble) {
                    w[8 * half + nibble] =
                        table[(words[half] >> (4 * nibble)) & 0xFU] *
                        slot.scale;
                }
            }
        }
        // refill this slot for the round kDepth ahead
        load_codes(slot, round + kDepth);
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
            float4 a[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                a[q] = *reinterpret_cast<const float4*>(
                    fragment + b * 16 * kStride + 4 * q);
            }
            const float values[16] = {a[0].x, a[0].y, a[0].z, a[0].w,
                                      a[1].x, a[1].y, a[1].z, a[1].w,
                                      a[2].x, a[2].y, a[2].z, a[2].w,
                                      a[3].x, a[3].y, a[3].z, a[3].w};
#pragma unroll
            for (int j = 0; j < kChunk; ++j) {
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                    values[j], w[j], acc[b], 0, 0, 0);
            }
        }
    };

    for (unsigned round = 0; round < round_count; round += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (round + d < round_count) {  // uniform across the workgroup
                run_round(ring[d], round + d);
            }
        }
    }

    // Wavefronts 1..7 park their tiles; wavefront 0 adds them in order.
    if (wave != 0) {
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                partial[(((wave - 1) * kBlocks + b) * 4 + r) * 64 + lane] =
                    acc[b][r];
            }
        }
    }
    __syncthreads();
    if (wave == 0 && n < output_width) {
        const float addend = bias != nullptr ? bias[n] : 0.0F;
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // accumulator element r of lane l is x row 4 * (l / 16) + r
                const unsigned m = 16 * b + 4 * quarter + r;
                if (m < rows) {
                    float sum = acc[b][r];
#pragma unroll
                    for (int other = 0; other < kWaves - 1; ++other) {
                        sum += partial[((other * kBlocks + b) * 4 + r) * 64 +
                                       lane];
                    }
                    y[static_cast<std::size_t>(m) * output_width + n] =
                        sum + addend;
                }
            }
        }
    }
}

template <int kBlocks, bool kDoubleQuantized>
void launch_instance(const LinearProblem& p, hipStream_t stream) {
    constexpr std::size_t kSharedBytes =
        (static_cast<std::size_t>(16 * kBlocks) * kStride + 16 +
         (kWaves - 1) * kBlocks * 4 * 64) *
        sizeof(float);
    const auto kernel = skinny_forward_kernel<kBlocks, kDoubleQuantized>;
    // More than the default 64 KB of LDS for the larger tiles.
    static const hipError_t configured = hipFuncSetAttribute(
        reinterpret_cast<const void*>(kernel),
        hipFuncAttributeMaxDynamicSharedMemorySize,
        static_cast<int>(kSharedBytes));
    static_cast<void>(configured);
    const unsigned grid =
        static_cast<unsigned>((p.output_width + kTileN - 1) / kTileN);
    kernel<<<grid, kThreads, kSharedBytes, stream>>>(
        p.activations, p.weight, p.bias, p.result,
        static_cast<unsigned>(p.rows), static_cast<unsigned>(p.input_width),
        static_cast<unsigned>(p.output_width), p.block_shift);
}

template <int kBlocks>
void launch_blocks(const LinearProblem& p, hipStream_t stream) {
    if (p.weight.encoding == 0) {
        launch_instance<kBlocks, false>(p, stream);
    } else {
        launch_instance<kBlocks, true>(p, stream);
    }
}

}  // namespace

bool skinny_forward_supports(const LinearProblem& p) {
    constexpr std::size_t kLimit = 1ULL << 31;
    return p.rows >= 1 && p.rows <= kSkinnyMaxRows &&
           p.input_width % kChunk == 0 && p.input_width < kLimit &&
           p.output_width < kLimit &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 8 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

void launch_skinny_forward(const LinearProblem& p, hipStream_t stream) {
    const std::size_t blocks = (p.rows + 15) / 16;
    switch (blocks) {
    case 1: launch_blocks<1>(p, stream); break;
    case 2: launch_blocks<2>(p, stream); break;
    case 3: launch_blocks<3>(p, stream); break;
    default: launch_blocks<4>(p, stream); break;
    }
}

}  // namespace rthip
