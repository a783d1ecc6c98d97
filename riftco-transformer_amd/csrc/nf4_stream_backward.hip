// Input backward for decode-sized row counts (rows <= 4):
//     dx[r, i] = sum_o dy[r, o] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_input_backward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:83-115) for
// the case where the packed bytes, not the arithmetic, set the pace.
//
// The weight is streamed exactly as it lies in memory, like the forward GEMV
// does: a lane owns sixteen consecutive columns (one 8-byte load of codes per
// weight row), a wavefront 1024, and the contraction runs over the weight
// rows a wavefront visits.  What differs from the forward product is that a
// lane's outputs are its own columns -- nothing is ever summed across lanes --
// and that the products fit the smallest matrix instruction without moving a
// byte between lanes:
//
//   v_mfma_f32_4x4x1_f32 works on sixteen independent blocks of four lanes,
//   D[i][j] += A[i] * B[j] with A[i] taken from lane 4 b + i, B[j] from lane
//   4 b + j, and D[.][j] kept by lane 4 b + j.  Here
//       B[j] = codebook level of ONE weight of lane 4 b + j   (row o, a column)
//       A[i] = dy[i, o] * scale(o, block)                      (upstream row i)
//   so D[i][j] gathers dx[i, column of lane 4 b + j]: all sixteen products
//   of a block are wanted, one instruction per weight serves up to four rows
//   of dy, and a lane needs sixteen accumulators (one per column, four rows
//   each).  The four lanes of a block hold 64 consecutive columns starting
//   at a multiple of 64, i.e. weights of ONE quantisation block (block sizes
//   of at least 64, rows that start on block boundaries), which is why the
//   scale may ride on A.  Sixteen instructions in a row write sixteen
//   different accumulators: no instruction waits for the one before.
//
// Decode is the GEMV's: a code byte indexes the replicated pair table in LDS
// (nf4_pair_table.hpp), lookups run one weight row ahead of the matrix
// instructions that consume them.
//
// Work split.  Column groups of 1024 times ranges of weight rows: a workgroup
// of eight wavefronts owns one column group and one range; its wavefronts
// take the range's four-row chunks in turn (four rows: one 16-byte load of
// dy), keep two chunks in flight, and add their accumulators through LDS in
// wavefront order.  With more than one range the sums go to the stream
// workspace and stream_backward_sum_kernel adds the ranges in ascending
// order: no atomics, the result does not depend on timing.

#include "kernels.hpp"
#include "launch_config.hpp"
#include "gemv_shared.hpp"
#include "nf4_decode.hpp"
#include "nf4_pair_table.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uint4_vec __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kLaneColumns = 16;                    // one 8-byte load of codes
constexpr int kWaveColumns = kWave * kLaneColumns;  // 1024
constexpr int kChunkRows = 4;                       // one 16-byte load of dy
constexpr int kDepth = 3;                           // chunks held per wavefront
constexpr unsigned kRejected = 0x80000000U;         // fails every range check
constexpr unsigned kComputeUnits = 256;
constexpr int kMaxRows = 4;                         // rows of dy
// staging of the wavefronts' sums: a lane's columns, padded
constexpr int kStageLane = kLaneColumns + 1;
constexpr int kStageWave = kWave * kStageLane;
constexpr int kStageBytes = kMaxRows * kWaves * kStageWave * 4;

struct StreamBackwardPlan {
    unsigned column_groups;     // ceil(I / 1024)
    unsigned row_ranges;        // pieces of the weight rows
    unsigned chunks_per_range;  // four-row chunks per piece
    unsigned chunk_count;       // O / 4
};

// One chunk of a wavefront: four weight rows of its 1024 columns.
template <bool kDoubleQuantized>
struct Chunk {
    uint2_vec codes[kChunkRows];
    float scale[kChunkRows];      // fp32 scale, or the second-level scale
    unsigned scale_code[kDoubleQuantized ? kChunkRows : 1];
    floatx4 upstream;             // dy[lane % 4][4 rows of the chunk]
};

// kMatrix: products on the matrix instruction (up to four rows of dy);
// otherwise one row of dy on the vector ALU, where sixteen multiply-adds take
// half the time of sixteen matrix instructions.
template <bool kDoubleQuantized, bool kMatrix>
__global__ __launch_bounds__(kThreads) void stream_backward_kernel(
    const float* __restrict__ dy, Nf4WeightView weight,
    float* __restrict__ target, unsigned rows, unsigned input_width,
    unsigned output_width, unsigned block_shift, StreamBackwardPlan plan
) {
    extern __shared__ __attribute__((aligned(256))) char lds[];
    char* const table = lds;
    float* const stage = reinterpret_cast<float*>(lds);  // after the loop

    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const unsigned lane = threadIdx.x % kWave;
    const unsigned group = blockIdx.x % plan.column_groups;
    const unsigned range = blockIdx.x / plan.column_groups;
    const unsigned column = group * kWaveColumns + lane * kLaneColumns;
    const bool lane_valid = column < input_width;
    // the A operand's row of a block; without the matrix instruction every
    // lane multiplies by row 0
    const unsigned upstream_row = kMatrix ? lane % 4 : 0U;

    const unsigned first_chunk = range * plan.chunks_per_range;
    const unsigned end_chunk =
        min(first_chunk + plan.chunks_per_range, plan.chunk_count);
    // chunks first_chunk + wave, + kWaves, ... belong to this wavefront
    const unsigned my_chunks =
        end_chunk > first_chunk + wave
            ? (end_chunk - first_chunk - wave + kWaves - 1) / kWaves
            : 0U;

    const unsigned row_code_bytes = input_width / 2;
    const unsigned row_blocks = input_width >> block_shift;
    const unsigned lane_block = column >> block_shift;
    const unsigned block_total = output_width * row_blocks;
    // per-lane offsets; a lane past the row end never touches memory
    const unsigned code_lane = lane_valid ? column / 2 : kRejected;
    const unsigned scale_lane =
        lane_valid ? lane_block * (kDoubleQuantized ? 1U : 4U) : kRejected;
    const unsigned upstream_lane =
        upstream_row < rows ? upstream_row * output_width * 4U : kRejected;

    using Held = Chunk<kDoubleQuantized>;
    Held ring[kDepth];
    const auto request = [&](Held& chunk, unsigned index) {
        // The scalar offset of a buffer load is not range-checked, so a chunk
        // that does not exist gets descriptors of extent zero instead.
        const bool exists = index < my_chunks;
        const unsigned row0 =
            (first_chunk + wave + index * kWaves) * kChunkRows;
        const __amdgpu_buffer_rsrc_t code_buffer = make_buffer(
            weight.codes, exists ? output_width * row_code_bytes : 0U);
        const __amdgpu_buffer_rsrc_t scale_buffer = make_buffer(
            weight.primary_scales,
            exists ? block_total * (kDoubleQuantized ? 1U : 4U) : 0U);
        const __amdgpu_buffer_rsrc_t upstream_buffer =
            make_buffer(dy, exists ? rows * output_width * 4U : 0U);
        chunk.upstream = __builtin_bit_cast(
            floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                         upstream_buffer, upstream_lane,
                         exists ? row0 * 4U : 0U, 0));
#pragma unroll
        for (int r = 0; r < kChunkRows; ++r) {
            const unsigned row = row0 + r;
            chunk.codes[r] = __builtin_amdgcn_raw_buffer_load_b64(
                code_buffer, code_lane, exists ? row * row_code_bytes : 0U,
                0);
            if constexpr (!kDoubleQuantized) {
                chunk.scale[r] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               scale_buffer, scale_lane,
                               exists ? row * row_blocks * 4U : 0U, 0));
            } else {
                chunk.scale_code[r] = __builtin_amdgcn_raw_buffer_load_b8(
                    scale_buffer, scale_lane, exists ? row * row_blocks : 0U,
                    0);
                const __amdgpu_buffer_rsrc_t second_buffer = make_buffer(
                    weight.secondary_scales,
                    exists ? (((block_total - 1) >>
                               weight.second_level_shift) +
                              1) * 4U
                           : 0U);
                const unsigned second =
                    lane_valid ? ((row * row_blocks + lane_block) >>
                                  weight.second_level_shift) * 4U
                               : kRejected;
                chunk.scale[r] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               second_buffer, second, 0, 0));
            }
        }
    };
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) {
        request(ring[d], d);
    }

    build_pair_table<kThreads>(table);
    // (code - 128) / 127 of a nested scale, once per code: the division of
    // decode_double_quantized_scale leaves the loop
    __shared__ float factor[kDoubleQuantized ? 256 : 1];
    if constexpr (kDoubleQuantized) {
        if (threadIdx.x < 256) {
            factor[threadIdx.x] =
                static_cast<float>(static_cast<int>(threadIdx.x) - 128) /
                127.0F;
        }
    }
    __syncthreads();
    const unsigned lane_bits = pair_table_lane_bits(lane);

    float2 levels[2][8];
    const auto look_up = [&](const uint2_vec& word, float2 (&out)[8]) {
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            out[b] = pair_table_lookup(table, word.x, b, lane_bits);
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            out[4 + b] = pair_table_lookup(table, word.y, b, lane_bits);
        }
    };

    // acc[k][i]: dx[i, column + k] over the weight rows seen so far
    // (without the matrix instruction only acc[k][0] is used)
    floatx4 acc[kLaneColumns];
#pragma unroll
    for (int k = 0; k < kLaneColumns; ++k) {
        acc[k] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
    }

    look_up(ring[0].codes[0], levels[0]);
    const unsigned turns = (my_chunks + kDepth - 1) / kDepth;
    for (unsigned turn = 0; turn < turns; ++turn) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            request(ring[(d + kDepth - 1) % kDepth],
                    turn * kDepth + d + kDepth - 1);
            const Held& current = ring[d];
#pragma unroll
            for (int r = 0; r < kChunkRows; ++r) {
                __builtin_amdgcn_sched_barrier(0);
                // the lookups of the next weight row go out first
                look_up(r + 1 < kChunkRows
                            ? current.codes[r + 1]
                            : ring[(d + 1) % kDepth].codes[0],
                        levels[(r + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
                float scale;
                if constexpr (kDoubleQuantized) {
                    scale = double_quantized_scale_from_factor(
                        factor[current.scale_code[r] & 0xFFU],
                        current.scale[r], weight.offset);
                } else {
                    scale = current.scale[r];
                }
                const float a = current.upstream[r] * scale;
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    const float2 pair = levels[r & 1][p];
                    if constexpr (kMatrix) {
                        acc[2 * p] = __builtin_amdgcn_mfma_f32_4x4x1f32(
                            a, pair.x, acc[2 * p], 0, 0, 0);
                        acc[2 * p + 1] = __builtin_amdgcn_mfma_f32_4x4x1f32(
                            a, pair.y, acc[2 * p + 1], 0, 0, 0);
                    } else {
                        acc[2 * p][0] += a * pair.x;
                        acc[2 * p + 1][0] += a * pair.y;
                    }
                }
            }
        }
    }

    // The wavefronts' sums, added in wavefront order (the table's memory is
    // free once every wavefront has left the loop).  A lane's sixteen columns
    // are stored seventeen floats apart from the next lane's: the stores of a
    // wavefront and the loads of the adding threads then meet no bank
    // conflict.
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kMaxRows; ++r) {
        if (static_cast<unsigned>(r) < rows) {
            float* const mine =
                stage + (r * kWaves + wave) * kStageWave + lane * kStageLane;
#pragma unroll
            for (int k = 0; k < kLaneColumns; ++k) {
                mine[k] = acc[k][r];
            }
        }
    }
    __syncthreads();
    for (unsigned c = threadIdx.x; c < kWaveColumns * rows; c += kThreads) {
        const unsigned r = c / kWaveColumns;
        const unsigned in_group = c % kWaveColumns;
        const float* const first =
            stage + r * kWaves * kStageWave +
            (in_group / kLaneColumns) * kStageLane + in_group % kLaneColumns;
        float sum = 0.0F;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            sum += first[w * kStageWave];
        }
        const unsigned out_column = group * kWaveColumns + in_group;
        if (out_column < input_width) {
            target[(static_cast<std::size_t>(range) * rows + r) *
                       input_width +
                   out_column] = sum;
        }
    }
}

// dx[e] = sum over the ranges, ascending, of partial[range][e].  A block
// owns 32 consecutive elements; its eight groups of 32 threads each add one
// contiguous eighth of the ranges (every load of a thread is issued before
// the first is used: one memory round trip, not one per range), and the
// eight sums are added in group order.
constexpr int kSumElements = 32;
constexpr int kSumSlices = 8;
constexpr unsigned kMaxRanges = 256;
__global__ __launch_bounds__(kSumElements * kSumSlices)
void stream_backward_sum_kernel(
    const float* __restrict__ partial, float* __restrict__ dx,
    unsigned elements, unsigned ranges, unsigned input_width,
    LoraEpilogue lora
) {
    __shared__ float slices[kSumSlices][kSumElements];
    const unsigned in_block = threadIdx.x % kSumElements;
    const unsigned slice = threadIdx.x / kSumElements;
    const unsigned element = blockIdx.x * kSumElements + in_block;
    const unsigned per_slice = (ranges + kSumSlices - 1) / kSumSlices;
    const unsigned first = slice * per_slice;
    const unsigned last = min(first + per_slice, ranges);
    float sum = 0.0F;
    if (element < elements && first < last) {
        constexpr int kHeld = kMaxRanges / kSumSlices;
        float parts[kHeld];
#pragma unroll
        for (int i = 0; i < kHeld; ++i) {
            // (ranges past the slice's last re-read its last, not added)
            const unsigned range = min(first + i, last - 1);
            parts[i] =
                partial[static_cast<std::size_t>(range) * elements + element];
        }
#pragma unroll
        for (int i = 0; i < kHeld; ++i) {
            if (first + i < last) {
                sum += parts[i];
            }
        }
    }
    slices[slice][in_block] = sum;
    __syncthreads();
    if (slice == 0 && element < elements) {
        float total = slices[0][in_block];
#pragma unroll
        for (int other = 1; other < kSumSlices; ++other) {
            total += slices[other][in_block];
        }
        if (lora.reduced != nullptr) {  // uniform
            total += lora_term(lora, element / input_width,
                               element % input_width);
        }
        dx[element] = total;
    }
}

StreamBackwardPlan plan_for(const LinearProblem& p) {
    StreamBackwardPlan plan{};
    plan.column_groups = static_cast<unsigned>(
        (p.input_width + kWaveColumns - 1) / kWaveColumns);
    plan.chunk_count = static_cast<unsigned>(p.output_width / kChunkRows);
    // one workgroup per compute unit; every wavefront gets at least two
    // chunks where the weight has that many
    unsigned ranges = kComputeUnits / plan.column_groups;
    const unsigned useful = (plan.chunk_count + 2 * kWaves - 1) / (2 * kWaves);
    ranges = ranges < useful ? ranges : useful;
    const std::size_t per_range = p.rows * p.input_width * sizeof(float);
    if (ranges > kStreamWorkspaceBytes / per_range) {
        ranges = static_cast<unsigned>(kStreamWorkspaceBytes / per_range);
    }
    ranges = ranges > kMaxRanges ? kMaxRanges : ranges;
    ranges = ranges < 1 ? 1 : ranges;
    plan.chunks_per_range = (plan.chunk_count + ranges - 1) / ranges;
    plan.row_ranges =
        (plan.chunk_count + plan.chunks_per_range - 1) / plan.chunks_per_range;
    return plan;
}

template <bool kDoubleQuantized, bool kMatrix>
hipError_t launch_instance(const LinearProblem& p, hipStream_t stream) {
    const StreamBackwardPlan plan = plan_for(p);
    float* target = p.result;
    WorkspaceLease lease;  // held until both launches are enqueued
    // (an adapter term is added by the second kernel, which then runs for
    // a single range too)
    const bool two_kernels = plan.row_ranges > 1 || p.lora.reduced != nullptr;
    if (two_kernels) {
        if (const hipError_t status = lease_stream_workspace(stream, &lease);
            status != hipSuccess) {
            return status;
        }
        target = lease.data();
    }
    const auto kernel = stream_backward_kernel<kDoubleQuantized, kMatrix>;
    // the table, and after the loop the staging area in the same memory
    constexpr int kSharedBytes =
        kStageBytes > kPairTableBytes ? kStageBytes : kPairTableBytes;
    static_assert(kSharedBytes <= 160 * 1024);
    static std::atomic<std::uint64_t> served{0};
    if (const hipError_t error = allow_dynamic_lds(
            reinterpret_cast<const void*>(kernel), kSharedBytes, served);
        error != hipSuccess) {
        return error;
    }
    kernel<<<plan.column_groups * plan.row_ranges, kThreads, kSharedBytes,
             stream>>>(p.activations, p.weight, target,
                       static_cast<unsigned>(p.rows),
                       static_cast<unsigned>(p.input_width),
                       static_cast<unsigned>(p.output_width), p.block_shift,
                       plan);
    if (two_kernels) {
        const unsigned elements =
            static_cast<unsigned>(p.rows * p.input_width);
        stream_backward_sum_kernel<<<(elements + kSumElements - 1) /
                                         kSumElements,
                                     kSumElements * kSumSlices, 0, stream>>>(
            target, p.result, elements, plan.row_ranges,
            static_cast<unsigned>(p.input_width), p.lora);
    }
    return hipSuccess;
}

template <bool kDoubleQuantized>
hipError_t launch_encoding(const LinearProblem& p, hipStream_t stream) {
    return p.rows == 1 ? launch_instance<kDoubleQuantized, false>(p, stream)
                       : launch_instance<kDoubleQuantized, true>(p, stream);
}

}  // namespace

bool stream_input_backward_supports(const LinearProblem& p) {
    return p.rows >= 1 && p.rows <= kStreamBackwardMaxRows &&
           // four lanes of a matrix block share one scale
           p.block_shift >= 6 &&
           p.input_width % (std::size_t{1} << p.block_shift) == 0 &&
           p.input_width % kLaneColumns == 0 &&
           p.output_width % kChunkRows == 0 &&
           p.output_width * p.input_width < (1ULL << 32) &&
           p.rows * p.output_width * sizeof(float) < (1ULL << 31) &&
           p.rows * p.input_width * sizeof(float) < (1ULL << 31) &&
           // with an adapter term the partial sums always pass through the
           // stream workspace, even where the weight is a single range
           (p.lora.reduced == nullptr ||
            p.rows * p.input_width * sizeof(float) <= kStreamWorkspaceBytes) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 8 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.result) % 4 == 0;
}

hipError_t launch_stream_input_backward(const LinearProblem& p,
                                        hipStream_t stream) {
    return p.weight.encoding == 0 ? launch_encoding<false>(p, stream)
                                  : launch_encoding<true>(p, stream);
}

}  // namespace rthip
