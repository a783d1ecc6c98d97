// Input backward for up to 64 rows:
//     dx[m, i] = sum_o dy[m, o] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_input_backward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:83-115) for
// row counts at which the 128-row tiles of the GEMM are mostly empty.
//
// The contraction runs over weight ROWS, the outputs over weight columns, so
// the packed weight is walked exactly as it lies in memory and never
// transposed:
//
//   * v_mfma_f32_16x16x4_f32 with A = dy [16 rows][4 weight rows] and
//     B = W [4 weight rows][16 columns].  Lane l supplies dy row l % 16 and
//     weight row l / 16 of the step.  Which 16 columns an instruction covers is
//     free as long as the accumulator is read back the same way, so a lane
//     owns EIGHT consecutive columns -- one 4-byte load of codes, the 16 lanes
//     of a weight row reading 64 contiguous bytes -- and feeds eight
//     instructions with eight accumulators: instruction t multiplies column
//     8 (l % 16) + t of every lane's run.
//   * A workgroup of eight wavefronts owns 128 columns and a chunk of weight
//     rows, which it walks 128 rows at a time: wavefront w takes rows
//     16 w .. 16 w + 15 of those, and in sub-step j (0..3) of the walk its lane
//     quarter k multiplies weight row 16 w + 4 k + j.  Any assignment of rows
//     to (sub-step, quarter) is valid as long as A and B agree; this one makes
//     the four dy values a lane needs for the four sub-steps CONTIGUOUS (one
//     16-byte load per row group instead of four scattered 4-byte ones -- with
//     those, the dy traffic through L1, not the matrix instructions, set the
//     pace).  (tile, chunk) units are numbered so that an XCD gets a
//     contiguous run of them: neighbouring column tiles, which share 128-byte
//     lines of the packed rows, go through the same L2.
//   * The loads of a walk step (four codes words, four scales, the dy values)
//     are issued one or two walk steps ahead and carry no branch; scheduling
//     barriers keep them where they are written, because the wait counts in
//     front of every operand are exact only if the order of the loads is the
//     same on every path into the loop.  Nested scales are decoded by the
//     step that consumes them.  Decode as everywhere: a code byte indexes the
//     replicated pair table in LDS, each level times its block scale in one
//     rounded multiply.
//   * At the end the eight wavefronts park their partial sums in LDS, row
//     group by row group, and the workgroup adds them in wavefront order.  With
//     one chunk that is dx; otherwise it is the chunk's partial sum, written to
//     the stream workspace, and a second kernel adds the chunks in ascending
//     order.  Nothing depends on scheduling.

#include "kernels.hpp"
#include "launch_config.hpp"
#include "nf4_decode.hpp"
#include "backward_split.hpp"
#include "nf4_pair_table.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kLaneColumns = 8;    // of which a lane owns this many
constexpr int kStepRows = 4;       // weight rows per matrix instruction
constexpr int kSubSteps = 4;       // matrix-instruction steps per walk step
static_assert(kWalkRows == kWaves * kStepRows * kSubSteps);
// Register slots for walk steps (steps in flight + 1): fewer when there are
// more row groups, which is when a step lasts longer and registers are scarce.
constexpr int ring_depth(int blocks) { return blocks <= 2 ? 3 : 2; }
constexpr unsigned kRejectedOffset = 0x80000000U;  // fails every range check
// parked[wavefront][instruction][lane]: one accumulator (four floats) each
constexpr std::size_t kParkingBytes =
    static_cast<std::size_t>(kWaves) * kLaneColumns * 64 * sizeof(floatx4);

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base,
                                                            std::size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// kBlocks: groups of 16 dy rows (1..4).
template <int kBlocks, bool kDoubleQuantized>
__global__ __launch_bounds__(kThreads) void small_backward_kernel(
    const float* __restrict__ dy, Nf4WeightView weight,
    float* __restrict__ out, unsigned rows, unsigned input_width,
    unsigned output_width, unsigned block_shift, BackwardSplit split
) {
    constexpr int kDepth = ring_depth(kBlocks);
    __shared__ __attribute__((aligned(256))) char table[kPairTableBytes];
    extern __shared__ __attribute__((aligned(16))) char shared[];
    floatx4* parked = reinterpret_cast<floatx4*>(shared);

    // XCD x gets units [x * units_per_xcd, (x + 1) * units_per_xcd).
    const unsigned unit =
        (blockIdx.x % 8) * split.units_per_xcd + blockIdx.x / 8;
    if (blockIdx.x / 8 >= split.units_per_xcd ||
        unit >= split.column_tiles * split.chunks) {
        return;  // the whole workgroup, before any barrier
    }
    const unsigned tile = unit % split.column_tiles;
    const unsigned chunk = unit / split.column_tiles;

    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const unsigned lane_row = lane % 16;     // dy row within a group of 16
    const unsigned step_row = lane / 16;     // weight row within a step
    const unsigned column0 =
        tile * kTileColumns + lane_row * kLaneColumns;  // first of my eight
    const unsigned chunk_begin = chunk * split.chunk_rows;
    const unsigned chunk_end =
        min(chunk_begin + split.chunk_rows, output_width);

    const std::size_t elements =
        static_cast<std::size_t>(output_width) * input_width;  // < 2^32
    const std::size_t block_total =
        (elements + (std::size_t{1} << block_shift) - 1) >> block_shift;
    const __amdgpu_buffer_rsrc_t code_buffer =
        raw_buffer(weight.codes, elements / 2);
    const __amdgpu_buffer_rsrc_t primary_buffer = raw_buffer(
        weight.primary_scales, block_total * (kDoubleQuantized ? 1 : 4));
    const __amdgpu_buffer_rsrc_t secondary_buffer = raw_buffer(
        weight.secondary_scales,
        kDoubleQuantized
            ? (((block_total - 1) >> weight.second_level_shift) + 1) * 4
            : 0);
    const __amdgpu_buffer_rsrc_t dy_buffer = raw_buffer(
        dy, static_cast<std::size_t>(rows) * output_width * sizeof(float));

    // One walk step's operands of a lane, as loaded: sub-step j multiplies
    // weight row first + j.  scales: block scales (fp32 encoding) or
    // second-level scales with their codes in scale_codes.
    struct Staged {
        unsigned codes[kSubSteps];  // eight nibbles each
        float scales[kSubSteps];
        unsigned scale_codes[kDoubleQuantized ? kSubSteps : 1];
        floatx4 upstream[kBlocks];  // dy[row][first .. first + 3]
    };
    // Weight rows past the chunk and dy rows past `rows` read as zeros: their
    // offsets carry bit 31, which fails every range check (all three arrays
    // are shorter than 2^31 bytes) and touches no memory.  The bit is OR-ed or
    // added in, never selected: a select in front of a load tends to become
    // two loads under a branch.  Lanes whose columns lie past the row end
    // re-read the row's last eight columns; what they compute is not written.
    const unsigned my_column =
        min(column0, input_width - static_cast<unsigned>(kLaneColumns));
    unsigned upstream_base[kBlocks];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
        const unsigned m = 16 * b + lane_row;
        upstream_base[b] =
            m < rows ? m * output_width * static_cast<unsigned>(sizeof(float))
                     : kRejectedOffset;
    }
    // first weight row of this lane in walk step 0
    const unsigned my_first_row =
        chunk_begin + wave * (kStepRows * kSubSteps) + step_row * kSubSteps;
    const auto load = [&](Staged& staged, unsigned walk_step) {
        const unsigned first = my_first_row + walk_step * kWalkRows;
        // (chunk ends are multiples of four, like `first`)
        const unsigned reject = first < chunk_end ? 0U : kRejectedOffset;
#pragma unroll
        for (int j = 0; j < kSubSteps; ++j) {
            const unsigned flat = (first + j) * input_width + my_column;
            staged.codes[j] = __builtin_amdgcn_raw_buffer_load_b32(
                code_buffer, (flat >> 1) | reject, 0, 0);
            const unsigned block = flat >> block_shift;
            if constexpr (!kDoubleQuantized) {
                staged.scales[j] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               primary_buffer, (block * 4) | reject, 0, 0));
            } else {
                staged.scale_codes[j] = __builtin_amdgcn_raw_buffer_load_b8(
                    primary_buffer, block | reject, 0, 0);
                staged.scales[j] = __builtin_bit_cast(
                    float,
                    __builtin_amdgcn_raw_buffer_load_b32(
                        secondary_buffer,
                        ((block >> weight.second_level_shift) * 4) | reject,
                        0, 0));
            }
        }
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
            // (first * 4 < 2^31, so a rejected base stays rejected)
            staged.upstream[b] = __builtin_bit_cast(
                floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                             dy_buffer,
                             (upstream_base[b] +
                              first * static_cast<unsigned>(sizeof(float))) |
                                 reject,
                             0, 0));
        }
    };

    const unsigned steps =
        (chunk_end - chunk_begin + kWalkRows - 1) / kWalkRows;  // >= 1
    // kDepth register slots: walk step s lives in slot s % kDepth and is
    // requested kDepth - 1 steps before it is used.
    Staged ring[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) {
        load(ring[d], d);
        // Step by step, as in the loop: the wait counts at the loop head
        // must hold for both ways into it, and loads grouped by kind here
        // would make every turn of the ring drain most of what is in flight.
        __builtin_amdgcn_sched_barrier(0);
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
    const unsigned lane_bits = pair_table_lane_bits(lane);
    __syncthreads();

    floatx4 acc[kBlocks][kLaneColumns];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
        for (int t = 0; t < kLaneColumns; ++t) {
            acc[b][t] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
        }
    }

    // Sub-step j: the eight weights are decoded into eight registers BEFORE
    // the matrix instructions are issued, and the table lookups of sub-step
    // j + 1 are requested in between.  Left to itself the compiler decodes
    // one weight at a time into ONE register, right in front of the
    // instruction that reads it -- and every such write then waits until the
    // matrix instruction in flight has read that register (30 % of the
    // matrix pipe's rate instead of 90 %).
    float2 raw[4];
    const auto issue_lookups = [&](const Staged& staged, int j) {
#pragma unroll
        for (int byte = 0; byte < 4; ++byte) {
            raw[byte] =
                pair_table_lookup(table, staged.codes[j], byte, lane_bits);
        }
    };
    const auto compute = [&](const Staged& staged) {
        issue_lookups(staged, 0);
#pragma unroll
        for (int j = 0; j < kSubSteps; ++j) {
            float w[kLaneColumns];
            {
#pragma clang fp contract(off)
                float scale = staged.scales[j];
                if constexpr (kDoubleQuantized) {
                    scale = double_quantized_scale_from_factor(
                        factor[staged.scale_codes[j] & 0xFFU],
                        staged.scales[j], weight.offset);
                }
#pragma unroll
                for (int byte = 0; byte < 4; ++byte) {
                    w[2 * byte] = raw[byte].x * scale;
                    w[2 * byte + 1] = raw[byte].y * scale;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (j + 1 < kSubSteps) {
                issue_lookups(staged, j + 1);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < kLaneColumns; ++t) {
#pragma unroll
                for (int b = 0; b < kBlocks; ++b) {
                    acc[b][t] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        staged.upstream[b][j], w[t], acc[b][t], 0, 0, 0);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // Static ring slots.  Whole turns of the ring run without a single
    // branch: a branch around a step's arithmetic would leave that step's
    // loads pending on the path that skips it, and every later reuse of their
    // registers would then wait for loads that are long done.  (Loads past the
    // chunk have rejected offsets and touch no memory.)  The last, partial
    // turn needs no loads any more -- its operands are already on their way.
    unsigned step = 0;
    for (; step + kDepth <= steps; step += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            load(ring[(d + kDepth - 1) % kDepth], step + d + kDepth - 1);
            // (the scheduler would otherwise collect the loads of the whole
            // turn at its end)
            __builtin_amdgcn_sched_barrier(0);
            compute(ring[d]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) {
        if (step + d < steps) {  // uniform
            compute(ring[d]);
        }
    }

    // Accumulator element r of instruction t, lane l, row group b is
    // dx[16 b + 4 (l / 16) + r][tile column 8 (l % 16) + t], summed over this
    // wavefront's weight rows.  Thread (t', l') adds the eight wavefronts'
    // accumulators of instruction t' and lane l' -- one 16-byte LDS read each,
    // consecutive lanes reading consecutive addresses -- and writes the four
    // elements to their four output rows.
    float* const target =
        out + static_cast<std::size_t>(chunk) * rows * input_width;
    const unsigned sum_lane = thread % 64;
    const unsigned sum_instruction = thread / 64;  // 0..7
    const unsigned sum_column = tile * kTileColumns +
                                (sum_lane % 16) * kLaneColumns +
                                sum_instruction;
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
        for (int t = 0; t < kLaneColumns; ++t) {
            parked[(wave * kLaneColumns + t) * 64 + lane] = acc[b][t];
        }
        __syncthreads();
        floatx4 sum = parked[sum_instruction * 64 + sum_lane];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) {  // wavefront order
            sum += parked[(w * kLaneColumns + sum_instruction) * 64 + sum_lane];
        }
        if (sum_column < input_width) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const unsigned m = 16 * b + 4 * (sum_lane / 16) + r;
                if (m < rows) {
                    target[static_cast<std::size_t>(m) * input_width +
                           sum_column] = sum[r];
                }
            }
        }
        __syncthreads();  // the parking space is free again
    }
}

// dx[e] = sum over chunks, ascending, of partial[chunk][e].  The loads of all
// chunks are issued before the first addition (a loop over a run-time chunk
// count would wait for them one after the other).
__global__ __launch_bounds__(256) void small_backward_sum_kernel(
    const float* __restrict__ partial, float* __restrict__ dx,
    unsigned elements, unsigned chunks, unsigned input_width,
    LoraEpilogue lora
) {
    const unsigned element = blockIdx.x * blockDim.x + threadIdx.x;
    if (element >= elements) {
        return;
    }
    float parts[kMaxChunks];
#pragma unroll
    for (unsigned chunk = 0; chunk < kMaxChunks; ++chunk) {
        // (chunks past the last one re-read the last one and are not added)
        const unsigned source = chunk < chunks ? chunk : chunks - 1;
        parts[chunk] =
            partial[static_cast<std::size_t>(source) * elements + element];
    }
    float sum = parts[0];
#pragma unroll
    for (unsigned chunk = 1; chunk < kMaxChunks; ++chunk) {
        if (chunk < chunks) {
            sum += parts[chunk];
        }
    }
    if (lora.reduced != nullptr) {  // uniform
        sum += lora_term(lora, element / input_width, element % input_width);
    }
    dx[element] = sum;
}

template <int kBlocks, bool kDoubleQuantized>
hipError_t launch_instance(const LinearProblem& p, hipStream_t stream) {
    const BackwardSplit split = split_weight_rows(
        p.rows, p.input_width, p.output_width, kStreamWorkspaceBytes);
    float* target = p.result;
    WorkspaceLease lease;  // held until both launches are enqueued
    // (an adapter term is added by the second kernel, which then runs for
    // a single chunk too)
    const bool two_kernels = split.chunks > 1 || p.lora.reduced != nullptr;
    if (two_kernels) {
        if (p.scratch != nullptr) {
            // the caller's memory; the split is the one the stream
            // workspace would get, so the sums are the same bit for bit
            if (static_cast<std::size_t>(split.chunks) * p.rows *
                    p.input_width * sizeof(float) >
                p.scratch_bytes) {
                return hipErrorOutOfMemory;
            }
            target = p.scratch;
        } else {
            if (const hipError_t status =
                    lease_stream_workspace(stream, &lease);
                status != hipSuccess) {
                return status;
            }
            target = lease.data();
        }
    }
    const auto kernel = small_backward_kernel<kBlocks, kDoubleQuantized>;
    // More than the default 64 KB of LDS (table + parking space).
    static std::atomic<std::uint64_t> served{0};
    if (const hipError_t error = allow_dynamic_lds(
            reinterpret_cast<const void*>(kernel), kParkingBytes, served);
        error != hipSuccess) {
        return error;
    }
    kernel<<<split.units_per_xcd * 8, kThreads, kParkingBytes, stream>>>(
        p.activations, p.weight, target, static_cast<unsigned>(p.rows),
        static_cast<unsigned>(p.input_width),
        static_cast<unsigned>(p.output_width), p.block_shift, split);
    if (two_kernels) {
        const unsigned elements =
            static_cast<unsigned>(p.rows * p.input_width);
        small_backward_sum_kernel<<<(elements + 255) / 256, 256, 0, stream>>>(
            target, p.result, elements, split.chunks,
            static_cast<unsigned>(p.input_width), p.lora);
    }
    return hipSuccess;
}

template <bool kDoubleQuantized>
hipError_t launch_blocks(const LinearProblem& p, hipStream_t stream) {
    switch ((p.rows + 15) / 16) {
    case 1: return launch_instance<1, kDoubleQuantized>(p, stream);
    case 2: return launch_instance<2, kDoubleQuantized>(p, stream);
    case 3: return launch_instance<3, kDoubleQuantized>(p, stream);
    default: return launch_instance<4, kDoubleQuantized>(p, stream);
    }
}

}  // namespace

bool small_input_backward_supports(const LinearProblem& p) {
    return p.rows >= 1 && p.rows <= kSmallBackwardMaxRows &&
           // a lane's eight columns: one aligned 4-byte load inside one block
           p.input_width % kLaneColumns == 0 &&
           // a lane's four dy values: one aligned 16-byte load
           p.output_width % kSubSteps == 0 &&
           p.output_width * p.input_width < (1ULL << 32) &&
           // bit 31 of a byte offset means "rejected"
           p.rows * p.output_width * sizeof(float) < (1ULL << 31) &&
           p.rows * p.input_width * sizeof(float) < (1ULL << 32) &&
           // with an adapter term the partial sums always pass through the
           // workspace, even where the weight rows are a single chunk
           (p.lora.reduced == nullptr ||
            p.rows * p.input_width * sizeof(float) <=
                (p.scratch != nullptr ? p.scratch_bytes
                                      : kStreamWorkspaceBytes)) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 4 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.result) % 4 == 0;
}

std::size_t small_input_backward_scratch_bytes(const LinearProblem& p) {
    // the split never depends on who brings the memory
    const BackwardSplit split = split_weight_rows(
        p.rows, p.input_width, p.output_width, kStreamWorkspaceBytes);
    return split.chunks > 1 ? static_cast<std::size_t>(split.chunks) *
                                  p.rows * p.input_width * sizeof(float)
                            : 0;
}

hipError_t launch_small_input_backward(const LinearProblem& p,
                                       hipStream_t stream) {
    return p.weight.encoding == 0 ? launch_blocks<false>(p, stream)
                                  : launch_blocks<true>(p, stream);
}

}  // namespace rthip
