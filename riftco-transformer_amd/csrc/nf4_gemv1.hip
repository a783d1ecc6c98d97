// Decode GEMV for one to four rows of x:
//     y[m][o] = sum_i x[m][i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81) for
// the case the decode step of a model is made of (one row; two to four rows
// reuse every load and lookup and add multiply-adds).  A launch of 9 to 50 MB
// lasts three to ten microseconds, and what bounds it besides the bytes is
// the compute unit's vector-memory pipeline: it takes one load instruction of
// a wavefront every ~6 clocks when a lane loads 4 bytes, but only every ~28
// clocks when a lane loads 8 or 16 (measured on MI355X, eight wavefronts per
// CU), so a kernel whose lanes fetch 8 code bytes plus one scale per weight row
// spends more time issuing loads than the bytes take to arrive.  Hence:
//
// * A lane owns 8 consecutive weights of a row (one 4-byte load); the 512
//   threads of a workgroup span 4096 columns and take kSegments such stripes
//   of wider rows.  A wavefront's load of a row is 256 contiguous bytes, the
//   workgroup's 2 KB.  The thread's slice of x (8 values per stripe) stays in
//   registers; x costs the CU 16 KB of loads per launch.
// * The block scale is applied AFTER the sum over the block's lanes, not per
//   lane: with block size 64 the 8 lanes of a block first add their sums of
//   x[i] * level(code) for the kRows rows of a batch (8, or fewer for rows
//   wider than 4096 weights; a transposed butterfly of DPP moves: afterwards
//   lane l holds the block's sum for row slot(l)), then each lane multiplies
//   by the ONE scale it needs -- block l / 8 of row slot(l) -- which it
//   loaded itself.  One scale load per batch
//   and lane instead of one per row, no movement of scales between lanes, and
//   a nested (double-quantised) scale costs one decode per lane and batch.
// * One buffer descriptor per array covers the whole weight; a load's offset
//   is (row offset, scalar) + (lane offset, fixed).  Rows past the output
//   width and batches past the last one lie past the arrays' ends, where the
//   hardware's range check returns zeros without touching memory, so nothing
//   branches on bounds and no per-row descriptors are built.
//
// Work split.  One persistent workgroup per CU; batch b of kRows consecutive
// weight rows goes to workgroup b % gridDim.x.  Requests: batch 0, then x,
// then -- after the table build -- the further batches of the ring; batch
// i + kDepth - 1 is requested when batch i is about to be multiplied.  A
// compute unit keeps about 32 KB of loads in flight (the size of its vector
// L1: beyond that the issue of further loads blocks), and the memory system
// serves a burst from all CUs at once badly -- the first bytes of a launch
// that requests 64 KB per CU up front arrive later than the LAST bytes of one
// that requests 16 KB at a time -- so a batch is 9 to 25 KB per CU and the ring
// is two deep.  The step exists in two compiled copies, with and without a
// batch left to request, and nothing on the vector ALU stands between a
// step's start and its loads (see load_batch): the compiler's wait counts are
// exact only along straight-line code.
//
// Decode is the (low nibble, high nibble) pair table in LDS of nf4_gemv.hip
// (which serves block sizes other than 64, output widths that are no multiple
// of eight and rows wider than 12288 weights).  Row
// sums: transposed butterfly inside each 16-lane DPP row, across the
// wavefront's four rows with v_permlane swaps, the eight wavefront partials
// parked in LDS and added in wavefront order after ONE barrier at the end.  A
// grouped launch equals its members' separate launches bit for bit: a batch is
// always multiplied by the same lanes in the same order.

#include "kernels.hpp"
#include "nf4_decode.hpp"
#include "nf4_pair_table.hpp"
#include "gemv_shared.hpp"

#include <cstdio>
#include <type_traits>

namespace rthip {
namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
constexpr int kSegment = 8;  // weights per thread per row visit
constexpr unsigned kBlockShift = 6;  // the block size this kernel is built for
constexpr unsigned kBlockLanes = (1U << kBlockShift) / kSegment;
constexpr int kMaxRows = 8;  // weight rows per batch: 8, 4 or 2
static_assert(kBlockLanes == kMaxRows, "a block's lanes hold a row sum each");
constexpr unsigned kComputeUnits = 256;
// Row sums a wavefront may park in LDS before the final barrier.
constexpr unsigned kParkedRows = 512;

typedef float float4_vec __attribute__((ext_vector_type(4)));

// What the loads of a member's batches need.
struct OneRowSource {
    const std::uint8_t* codes;
    const void* primary_scales;
    const float* secondary_scales;
    unsigned code_bytes;       // extent of the code array
    unsigned primary_bytes;    // extent of the block-scale array
    unsigned secondary_bytes;  // extent of the second-level scale table
    float offset;
    unsigned first_batch;
};
// What the final sums of a member need.
struct OneRowTarget {
    float* y;
    const float* bias;
    unsigned output_width;
    unsigned first_batch;
    LoraEpilogue lora;  // the member's adapter term (reduced == null: none)
};
// Members 1 ... of a grouped launch (member 0's source is passed as plain
// kernel arguments, see the kernel), and every member's target.
template <int kMembers>
struct OneRowRest {
    OneRowTarget target[kMembers];
    OneRowSource source[kMembers > 1 ? kMembers - 1 : 1];
    unsigned member_first_batch[kMembers + 1];  // [kMembers] = 0xFFFFFFFF
};

template <int kRows, int kSegments, bool kDoubleQuantized>
struct RowBatch {
    unsigned codes[kRows][kSegments];
    // fp32 scales: the scale itself; nested: the second-level scale
    float scales[kSegments];
    unsigned scale_codes[kDoubleQuantized ? kSegments : 1];
    float offset;  // of the member the batch belongs to (uniform)
};

// kWholeGroups (nested scales): every batch starts on a second-level group
// boundary, so a lane's second-level scale sits at a fixed offset from the
// batch's first one.
// kX: rows of x held per thread (1, 2 or 4; three rows run as four with an
// empty fourth).
template <int kX, int kSegments, int kRows, int kDepth, int kLook,
          bool kDoubleQuantized, bool kWholeGroups, int kMembers>
__global__ __launch_bounds__(kThreads) void gemv1_forward_kernel(
    // The first 14 dwords are preloaded into scalar registers when the
    // wavefront is created (the file is compiled with
    // -amdgpu-kernarg-preload-count): what the first loads need, so that they
    // do not wait for a read of the argument block from memory.
    const float* __restrict__ x, const std::uint8_t* __restrict__ codes,
    const void* __restrict__ primary_scales, unsigned input_width,
    unsigned code_bytes, unsigned primary_bytes, unsigned iterations,
    const float* __restrict__ secondary_scales, unsigned secondary_bytes,
    float offset_of_scales,
    // read from memory
    unsigned second_level_shift, unsigned batch_count, unsigned x_rows,
    const OneRowRest<kMembers> rest
) {
    constexpr bool kGrouped = kMembers > 1;
    constexpr unsigned kMaxIterations = kParkedRows / (kRows * kX);
    static_assert(kRows == 8 || kRows == 4 || kRows == 2);
    static_assert(kX == 1 || kX == 2 || kX == 4);
    __shared__ __attribute__((aligned(256))) char table[kPairTableBytes];
    __shared__ float partial[kMaxIterations][kWaves][kRows][kX];
    // Nested scales: (code - 128) / 127 for every scale code, so that a
    // scale costs its lane one LDS read, a multiply and an add instead of a
    // correctly rounded division (the same quotients, hence the same scales
    // bit for bit as decode_double_quantized_scale).
    __shared__ float factor[kDoubleQuantized ? 256 : 1];

    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % kWave;
    const unsigned wave = __builtin_amdgcn_readfirstlane(thread / kWave);
    const unsigned segment_count = input_width / kSegment;
    const unsigned row_code_bytes = input_width / 2;
    const unsigned row_blocks = input_width >> kBlockShift;
    // the row of a batch whose block sum this lane ends up holding
    const unsigned my_row = slot_of_lane<kRows>(lane);

    // Where this thread's stripes sit inside a row.  A stripe past the row
    // end reads stripe 0 again (any in-range bytes will do: its x is zero).
    unsigned code_offset[kSegments];
    // of the scale of (my_row, this stripe's block), from the batch's first
    // scale: in bytes for fp32 scales, in blocks (= bytes) for nested ones
    unsigned scale_offset[kSegments];
#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
        const unsigned segment = thread + kThreads * j;
        const unsigned kept = segment < segment_count ? segment : 0U;
        code_offset[j] = kept * (kSegment / 2);
        scale_offset[j] = (my_row * row_blocks + kept / kBlockLanes) *
                          (kDoubleQuantized ? 1U : 4U);
    }
    // (nested scales, whole groups) of this lane's second-level scale, from
    // the batch's first one, in bytes
    unsigned second_offset[kSegments];
#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
        second_offset[j] = (scale_offset[j] >> second_level_shift) * 4;
    }

    // The member whose batches are being REQUESTED.  A workgroup's batch
    // numbers only grow, so the member only moves forward; its fields live in
    // scalar registers and are re-read in the rare step that crosses into the
    // next member (a uniform branch without any vector memory access in it).
    unsigned member_index = 0;
    OneRowSource member{codes, primary_scales, secondary_scales, code_bytes,
                        primary_bytes, secondary_bytes, offset_of_scales, 0U};
    unsigned member_end = kGrouped ? rest.member_first_batch[1] : ~0U;
    const auto seek_member = [&](unsigned batch_index) {
        if constexpr (kGrouped) {
            while (batch_index >= member_end) {
                member = rest.source[member_index];
                ++member_index;
                member_end = rest.member_first_batch[member_index + 1];
            }
        }
    };

    // The loads of a batch are issued without ANY vector instruction in front
    // of them: per-lane offsets are fixed registers, everything that changes
    // from batch to batch is scalar -- a descriptor that starts at the
    // batch's first row (extent: what is left of the array, zero for batches
    // past the last one) -- and a row's offset inside its batch is a scalar
    // that never changes.  A vector instruction that computes an address
    // may be given a register of the ring slot being refilled, and the
    // compiler then waits for loads it believes pending in that register --
    // in effect for the batch that is about to be multiplied -- before it
    // issues the new loads, which serialises request and arrival.
    using Batch = RowBatch<kRows, kSegments, kDoubleQuantized>;
    const auto load_batch = [&](Batch& batch, unsigned batch_index) {
        seek_member(batch_index);
        const unsigned first_row = (batch_index - member.first_batch) * kRows;
        batch.offset = member.offset;
        const unsigned code_start =
            min(first_row * row_code_bytes, member.code_bytes);
        const unsigned code_left = member.code_bytes - code_start;
        const __amdgpu_buffer_rsrc_t code_buffer =
            make_buffer(member.codes + code_start, code_left);
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            // scalar, the same for every batch (output widths are multiples
            // of kRows: a batch has all of its rows or none)
            const unsigned row_start =
                static_cast<unsigned>(row) * row_code_bytes;
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                batch.codes[row][j] = __builtin_amdgcn_raw_buffer_load_b32(
                    code_buffer, code_offset[j], row_start, 0);
            }
        }
        const unsigned first_block = first_row * row_blocks;
        constexpr unsigned kScaleBytes = kDoubleQuantized ? 1 : 4;
        const unsigned scale_start =
            min(first_block * kScaleBytes, member.primary_bytes);
        const __amdgpu_buffer_rsrc_t primary_buffer = make_buffer(
            static_cast<const char*>(member.primary_scales) + scale_start,
            member.primary_bytes - scale_start);
#pragma unroll
        for (int j = 0; j < kSegments; ++j) {
            if constexpr (!kDoubleQuantized) {
                batch.scales[j] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               primary_buffer, scale_offset[j], 0, 0));
            } else {
                batch.scale_codes[j] = __builtin_amdgcn_raw_buffer_load_b8(
                    primary_buffer, scale_offset[j], 0, 0);
            }
        }
        if constexpr (kDoubleQuantized && kWholeGroups) {
            const unsigned second_start =
                min((first_block >> second_level_shift) * 4,
                    member.secondary_bytes);
            const __amdgpu_buffer_rsrc_t secondary_buffer = make_buffer(
                reinterpret_cast<const char*>(member.secondary_scales) +
                    second_start,
                member.secondary_bytes - second_start);
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                batch.scales[j] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               secondary_buffer, second_offset[j], 0, 0));
            }
        } else if constexpr (kDoubleQuantized) {
            // The second-level scale's index needs a shift of the block
            // number, a vector instruction: its result is kept alive past
            // the load, so it cannot share a register with the load's
            // destination (see above).
            const __amdgpu_buffer_rsrc_t secondary_buffer = make_buffer(
                member.secondary_scales, member.secondary_bytes);
            unsigned second[kSegments];
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                second[j] = ((first_block + scale_offset[j]) >>
                             second_level_shift) * 4;
            }
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                batch.scales[j] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               secondary_buffer, second[j], 0, 0));
            }
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                asm volatile("" ::"v"(second[j]));
            }
        }
    };

    // Batch b goes to workgroup b % gridDim.x.
    const unsigned stride = gridDim.x;
    const unsigned first_batch = blockIdx.x;

    Batch ring[kDepth];
    load_batch(ring[0], first_batch);

    // This thread's slice of x, resident for the whole kernel; stripes past
    // the row end and rows past x_rows read as zero (range check).
    float xs[kX][kSegments][kSegment];
#pragma unroll
    for (int r = 0; r < kX; ++r) {
        const bool row_exists = static_cast<unsigned>(r) < x_rows;
        const __amdgpu_buffer_rsrc_t x_buffer = make_buffer(
            x + (row_exists ? static_cast<unsigned>(r) * input_width : 0U),
            row_exists ? input_width * 4U : 0U);
#pragma unroll
        for (int j = 0; j < kSegments; ++j) {
            const unsigned first = (thread + kThreads * j) * (kSegment * 4);
#pragma unroll
            for (int q = 0; q < kSegment / 4; ++q) {
                // (the whole vector is cast at once: a bit cast of ONE
                // element of an ext-vector reads element 0 whatever the
                // element is)
                const float4_vec v = __builtin_bit_cast(
                    float4_vec, __builtin_amdgcn_raw_buffer_load_b128(
                                    x_buffer, first + q * 16, 0, 0));
                xs[r][j][4 * q + 0] = v.x;
                xs[r][j][4 * q + 1] = v.y;
                xs[r][j][4 * q + 2] = v.z;
                xs[r][j][4 * q + 3] = v.w;
            }
        }
    }

    build_pair_table<kThreads>(table);
    if constexpr (kDoubleQuantized) {
        if (thread < 256) {
            factor[thread] =
                static_cast<float>(static_cast<int>(thread) - 128) / 127.0F;
        }
    }

#pragma unroll
    for (int d = 1; d < kDepth - 1; ++d) {
        load_batch(ring[d], first_batch + d * stride);
    }
    __syncthreads();

    const unsigned lane_bits = pair_table_lane_bits(lane);

    const auto step = [&](const Batch& current, Batch& refill,
                          unsigned iteration, auto refill_exists) {
        constexpr bool kRefill = decltype(refill_exists)::value;
        const unsigned batch_index = first_batch + iteration * stride;
        unsigned step_lane_bits = lane_bits;
        if constexpr (kRefill) {
            load_batch(refill, batch_index + (kDepth - 1) * stride);
            // keeps the lookups' address arithmetic of the two copies of the
            // step apart (hoisted above the branch it would drag the wait for
            // the current codes in front of the new loads)
            asm volatile("" : "+v"(step_lane_bits)::"memory");
        }

        // Table lookups run kLook - 1 weight rows ahead of the multiply-adds
        // that consume them, which keeps the LDS queue deep enough to stream.
        float2 levels[kLook][kSegments][4];
        const auto look_up = [&](int row) {
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    levels[row % kLook][j][b] = pair_table_lookup(
                        table, current.codes[row][j], b, step_lane_bits);
                }
            }
        };
#pragma unroll
        for (int row = 0; row < kLook - 1; ++row) {
            look_up(row);
        }
        float acc[kX][kSegments][kRows];
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            if (row + kLook - 1 < kRows) {
                look_up(row + kLook - 1);
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                float even[kX];
                float odd[kX];
#pragma unroll
                for (int r = 0; r < kX; ++r) {
                    even[r] = 0.0F;
                    odd[r] = 0.0F;
                }
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const float2 pair = levels[row % kLook][j][p];
#pragma unroll
                    for (int r = 0; r < kX; ++r) {
                        even[r] += xs[r][j][2 * p] * pair.x;
                        odd[r] += xs[r][j][2 * p + 1] * pair.y;
                    }
                }
#pragma unroll
                for (int r = 0; r < kX; ++r) {
                    acc[r][j][row] = even[r] + odd[r];
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // Block sums (8 lanes), times the block's scale, then the stripes, the
        // 16-lane DPP row and the wavefront's four rows.
        float scale[kSegments];
#pragma unroll
        for (int j = 0; j < kSegments; ++j) {
            scale[j] = current.scales[j];
            if constexpr (kDoubleQuantized) {
                scale[j] = double_quantized_scale_from_factor(
                    factor[current.scale_codes[j] & 0xFFU], scale[j],
                    current.offset);
            }
        }
#pragma unroll
        for (int r = 0; r < kX; ++r) {
            float total = 0.0F;
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                // after log2(kRows) transposed steps a lane holds ONE row's
                // sum over kRows lanes; plain steps take it to the block's 8
                // lanes
                transposed_step<1, kRows / 2>(acc[r][j], lane);
                transposed_step<2, kRows / 4>(acc[r][j], lane);
                transposed_step<4, kRows / 8>(acc[r][j], lane);
                total += acc[r][j][0] * scale[j];
            }
            total += dpp_xor<8>(total);
            total = sum_over_rows(total);
            if (lane < kRows) {
                partial[iteration][wave][my_row][r] = total;
            }
        }
    };

    // The ring is walked with static slot numbers.  The last kDepth - 1 steps
    // have nothing left to request; they run the copy of the step that issues
    // no loads.
    for (unsigned iteration = 0; iteration < iterations;
         iteration += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            if (iteration + d < iterations) {
                Batch& refill = ring[(d + kDepth - 1) % kDepth];
                if (iteration + d + kDepth - 1 < iterations) {
                    step(ring[d], refill, iteration + d, std::true_type{});
                } else {
                    step(ring[d], refill, iteration + d, std::false_type{});
                }
            }
        }
    }

    // The only barrier after the table build: every batch of this workgroup
    // has been parked.  The eight wavefront partials of a row are added in
    // wavefront order.
    __syncthreads();
    for (unsigned index = thread; index < iterations * kRows * kX;
         index += kThreads) {
        const unsigned iteration = index / (kRows * kX);
        const unsigned value = index / kX % kRows;
        const unsigned r = index % kX;
        const unsigned batch_index = first_batch + iteration * stride;
        // the member's target per lane: a chain of selects over kernel
        // arguments
        OneRowTarget target = rest.target[0];
        if constexpr (kGrouped) {
#pragma unroll
            for (int k = 1; k < kMembers; ++k) {
                if (batch_index >= rest.target[k].first_batch) {
                    target = rest.target[k];
                }
            }
        }
        const unsigned o = (batch_index - target.first_batch) * kRows + value;
        if (batch_index < batch_count && o < target.output_width &&
            r < x_rows) {
            float sum = 0.0F;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                sum += partial[iteration][w][value][r];
            }
            if (target.bias != nullptr) {
                sum += target.bias[o];
            }
            if (target.lora.reduced != nullptr) {
                sum += lora_term(target.lora, r, o);
            }
            target.y[r * target.output_width + o] = sum;
        }
    }
}

#ifndef RTHIP_GEMV1_DEPTH
#define RTHIP_GEMV1_DEPTH 2
#endif
#ifndef RTHIP_GEMV1_LOOK
#define RTHIP_GEMV1_LOOK 4
#endif
#ifndef RTHIP_GEMV1_WIDE_ROWS
#define RTHIP_GEMV1_WIDE_ROWS 4
#endif

std::size_t segments_per_thread(const LinearProblem& p) {
    return (p.input_width / kSegment + kThreads - 1) / kThreads;
}

// What to do with the instance that serves a call: launch it, or only write
// its name (as a profiler prints it) into `name`.
struct Request {
    hipStream_t stream;
    char* name;
    std::size_t capacity;
};

template <int kX, int kSegments, bool kDoubleQuantized, int kMembers>
void launch_instance(const LinearProblem* problems, std::size_t count,
                     const Request& request) {
    constexpr int kDepth = RTHIP_GEMV1_DEPTH;
    // A compute unit keeps about 32 KB of loads in flight (its vector L1):
    // a batch should stay well below that, so wider rows take fewer of them.
    // (With four rows of x and three stripes the thread's slice of x alone
    // is 96 registers: two weight rows per batch.)
    constexpr int kRows =
        kSegments == 1 ? 8
                       : (kSegments == 2 ? 4
                                         : (kX == 4 ? 2 : RTHIP_GEMV1_WIDE_ROWS));
    constexpr int kLook = kSegments == 1 ? (kX == 4 ? 2 : RTHIP_GEMV1_LOOK) : 2;
    constexpr unsigned kMaxIterations = kParkedRows / (kRows * kX);
    const LinearProblem& first = problems[0];
    OneRowRest<kMembers> rest{};
    OneRowSource sources[kMembers];
    unsigned batch_count = 0;
    for (std::size_t m = 0; m < static_cast<std::size_t>(kMembers); ++m) {
        OneRowSource& source = sources[m];
        OneRowTarget& target = rest.target[m];
        rest.member_first_batch[m] = m < count ? batch_count : ~0U;
        target.first_batch = rest.member_first_batch[m];
        source = OneRowSource{};
        source.first_batch = rest.member_first_batch[m];
        if (m >= count) {
            continue;
        }
        const LinearProblem& p = problems[m];
        const std::size_t weights = p.output_width * p.input_width;
        const std::size_t block_count = weights >> kBlockShift;
        source.codes = p.weight.codes;
        source.primary_scales = p.weight.primary_scales;
        source.secondary_scales = p.weight.secondary_scales;
        source.code_bytes = static_cast<unsigned>(weights / 2);
        source.primary_bytes = static_cast<unsigned>(
            kDoubleQuantized ? block_count : block_count * 4);
        source.secondary_bytes =
            kDoubleQuantized
                ? static_cast<unsigned>(
                      (((block_count - 1) >> p.weight.second_level_shift) + 1) *
                      4)
                : 0U;
        source.offset = p.weight.offset;
        target.y = p.result;
        target.bias = p.bias;
        target.lora = p.lora;
        target.output_width = static_cast<unsigned>(p.output_width);
        batch_count += static_cast<unsigned>(p.output_width / kRows);
    }
    rest.member_first_batch[kMembers] = ~0U;
    for (int m = 1; m < kMembers; ++m) {
        rest.source[m - 1] = sources[m];
    }
    // One workgroup per CU; more when a workgroup would otherwise need more
    // batches than its LDS parking space holds.
    unsigned blocks = batch_count < kComputeUnits ? batch_count : kComputeUnits;
    if ((batch_count + blocks - 1) / blocks > kMaxIterations) {
        blocks = (batch_count + kMaxIterations - 1) / kMaxIterations;
    }
    const unsigned iterations = (batch_count + blocks - 1) / blocks;
    const OneRowSource& head = sources[0];
    const auto launch = [&](auto whole_groups) {
        constexpr bool kWhole = decltype(whole_groups)::value;
        if (request.name != nullptr) {
            std::snprintf(request.name, request.capacity,
                          "gemv1_forward_kernel<%d, %d, %d, %d, %d, %s, %s, %d>",
                          kX, kSegments, kRows, kDepth, kLook,
                          kDoubleQuantized ? "true" : "false",
                          kWhole ? "true" : "false", kMembers);
            return;
        }
        gemv1_forward_kernel<kX, kSegments, kRows, kDepth, kLook,
                             kDoubleQuantized, kWhole, kMembers>
            <<<blocks, kThreads, 0, request.stream>>>(
                first.activations, head.codes, head.primary_scales,
                static_cast<unsigned>(first.input_width), head.code_bytes,
                head.primary_bytes, iterations, head.secondary_scales,
                head.secondary_bytes, head.offset,
                first.weight.second_level_shift, batch_count,
                static_cast<unsigned>(first.rows), rest);
    };
    if constexpr (kDoubleQuantized) {
        const std::size_t batch_blocks =
            kRows * (first.input_width >> kBlockShift);
        if (batch_blocks % (std::size_t{1} << first.weight.second_level_shift)
            == 0) {
            launch(std::true_type{});
            return;
        }
    }
    launch(std::false_type{});
}

template <int kX, bool kDoubleQuantized, int kMembers>
void launch_segments(const LinearProblem* problems, std::size_t count,
                     const Request& request) {
    switch (segments_per_thread(problems[0])) {
    case 1:
        launch_instance<kX, 1, kDoubleQuantized, kMembers>(problems, count,
                                                           request);
        break;
    case 2:
        launch_instance<kX, 2, kDoubleQuantized, kMembers>(problems, count,
                                                           request);
        break;
    default:
        launch_instance<kX, 3, kDoubleQuantized, kMembers>(problems, count,
                                                           request);
        break;
    }
}

template <bool kDoubleQuantized, int kMembers>
void launch_rows(const LinearProblem* problems, std::size_t count,
                 const Request& request) {
    switch (problems[0].rows) {
    case 1:
        launch_segments<1, kDoubleQuantized, kMembers>(problems, count,
                                                       request);
        break;
    case 2:
        launch_segments<2, kDoubleQuantized, kMembers>(problems, count,
                                                       request);
        break;
    default:
        launch_segments<4, kDoubleQuantized, kMembers>(problems, count,
                                                       request);
        break;
    }
}

template <int kMembers>
void launch_encoding(const LinearProblem* problems, std::size_t count,
                     const Request& stream) {
    if (problems[0].weight.encoding == 0) {
        launch_rows<false, kMembers>(problems, count, stream);
    } else {
        launch_rows<true, kMembers>(problems, count, stream);
    }
}

}  // namespace

bool gemv1_forward_supports(const LinearProblem& p) {
    constexpr std::size_t kMaxWidth =
        static_cast<std::size_t>(kSegment) * kThreads * 3;
    // Offsets are 32-bit and run up to a few batches past an array's end.
    constexpr std::size_t kMaxBytes = std::size_t{1} << 31;
    const std::size_t weights = p.output_width * p.input_width;
    return p.rows >= 1 && p.rows <= kGemvMaxRows &&
           p.block_shift == kBlockShift &&
           p.output_width % kMaxRows == 0 &&
           p.input_width % (std::size_t{1} << kBlockShift) == 0 &&
           p.input_width <= kMaxWidth && weights / 2 < kMaxBytes &&
           p.rows * p.output_width < (1ULL << 32) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 4 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

bool gemv1_group_supports(const LinearProblem* problems, std::size_t count) {
    if (count < 1 || count > kGemvGroupMax) {
        return false;
    }
    const LinearProblem& first = problems[0];
    std::size_t batches = 0;
    for (std::size_t m = 0; m < count; ++m) {
        const LinearProblem& p = problems[m];
        if (!gemv1_forward_supports(p) || p.activations != first.activations ||
            p.rows != first.rows || p.input_width != first.input_width ||
            p.weight.encoding != first.weight.encoding ||
            p.weight.second_level_shift != first.weight.second_level_shift) {
            return false;
        }
        batches += (p.output_width + 1) / 2;  // at least two rows per batch
    }
    return batches < (1ULL << 31);
}

void launch_gemv1_forward(const LinearProblem* problems, std::size_t count,
                          hipStream_t stream) {
    const Request request{stream, nullptr, 0};
    if (count == 1) {
        launch_encoding<1>(problems, count, request);
    } else {
        launch_encoding<static_cast<int>(kGemvGroupMax)>(problems, count,
                                                         request);
    }
}

void gemv1_kernel_name(const LinearProblem* problems, std::size_t count,
                       char* name, std::size_t capacity) {
    const Request request{nullptr, name, capacity};
    if (count == 1) {
        launch_encoding<1>(problems, count, request);
    } else {
        launch_encoding<static_cast<int>(kGemvGroupMax)>(problems, count,
                                                         request);
    }
}

}  // namespace rthip
