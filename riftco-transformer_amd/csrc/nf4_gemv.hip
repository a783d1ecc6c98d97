// Streaming GEMV for decode-sized row counts (rows <= 4):
//     y[r, o] = sum_i x[r, i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81) for the
// HBM-bound case, where the only traffic that matters is the packed codes and
// their scales, each read exactly once.
//
// Work split.  One persistent workgroup per CU holds kTeams teams of four
// wavefronts.  A team owns batches of kRows consecutive weight rows; the
// contraction axis is cut into 16-weight segments (8 bytes of codes) and thread
// t of a team owns segments t, t + 256, ... of EVERY row, so
//   * a wavefront's loads of one row are 512 contiguous bytes,
//   * the x values a thread needs never change: they are loaded once into
//     registers and reused for all rows,
//   * a segment lies inside one quantisation block (block sizes are powers of
//     two >= 32 and the row width is a multiple of 16), so a thread applies
//     one scale per segment:  acc += scale * sum_i x_i * codebook[c_i].
// The loads of batch b + 1 are issued before batch b is computed, and the
// wavefronts never wait for each other inside the loop, so HBM requests are in
// flight for the whole life of the workgroup.  Nothing may branch around
// those loads or sit between them and the work they overlap with: the
// compiler's wait counts are exact only along straight-line code, and a
// uniform `if` around the loads makes every wait for the CURRENT batch wait
// for the just-issued loads as well.  Hence the two compiled copies of the
// step (with and without a batch left to request) and the deferred decode of
// nested scales.
//
// Groups.  One launch can cover up to kGemvGroupMax weights that share x (the
// query/key/value or gate/up projections of a layer): their batches are
// numbered one weight after the other and dealt exactly like the batches of a
// single weight, so every output is computed by the same lanes in the same
// order as in a launch of its own, and the launch's fixed cost is paid once.
//
// Decode.  Nibble -> fp32 is a table lookup in LDS, 4 bytes of table per
// weight.  Nibbles are decoded two at a time -- a code BYTE indexes a table of
// (codebook[low nibble], codebook[high nibble]) pairs, one ds_read_b64 per two
// weights -- and everything else is kept off the LDS.  The table is stored
// entry-major with 32 interleaved replicas (nf4_pair_table.hpp): replica k of
// entry e sits at byte e * 256 + k * 8, lane l reads replica l % 32, so a
// lookup never meets a bank conflict whatever the codes are, and an entry's
// address is (byte << 8) | ((l % 32) << 3): ONE v_perm_b32 that drops the code
// byte into bits 8..15 above the lane's fixed low byte.  The table is built
// from instruction literals while the first loads are in flight.
//
// Weight bytes and scales are fetched with buffer loads through per-row
// descriptors (built with scalar instructions): the per-lane offset is a
// constant, so stepping to the next row costs no vector arithmetic, and the
// hardware range check turns reads past the row end into zeros.  Nothing branches on data or on bounds:
// segments past the row end carry x = 0 and rows past the output width are
// computed on whatever was read and never written.
//
// Reduction.  Row sums are reduced inside each 16-lane DPP row with a transposed
// butterfly of DPP moves (vector ALU only), then across the four rows of the
// wavefront; the four wavefront partials per team and batch are parked in LDS,
// and after ONE barrier at the end of the kernel the team adds them up and
// writes y.

#include "kernels.hpp"
#include "nf4_decode.hpp"
#include "nf4_pair_table.hpp"
#include "gemv_shared.hpp"

#include <type_traits>

namespace rthip {
namespace {

constexpr int kWorkgroupThreads = 512;
// Four teams: a workgroup of sixteen wavefronts (teams stay 256 threads wide).
constexpr int workgroup_threads(int teams) {
    return teams == 4 ? 2 * kWorkgroupThreads : kWorkgroupThreads;
}
constexpr int kSegment = 16;       // weights per thread per row visit
constexpr unsigned kComputeUnits = 256;
// Row totals a team may park in LDS before the final barrier, per wavefront.
constexpr unsigned kParkedValues = 512;
#ifndef RTHIP_GEMV_TEAMS
#define RTHIP_GEMV_TEAMS 2
#endif
#ifndef RTHIP_GEMV_ROWS
#define RTHIP_GEMV_ROWS 4
#endif
#ifndef RTHIP_GEMV_DEPTH
#define RTHIP_GEMV_DEPTH 2
#endif

// Shared scale loads per batch (nested scale encoding): a load covers 64
// (row, block) pairs and a wavefront's part of a row spans at most 32 blocks
// (block size 32), so two-row batches need one load and four-row batches two.
constexpr int scale_loads(int rows) { return rows * 32 > 64 ? 2 : 1; }

// kShared false: scales[row][j] is the scale of this lane's weights of row
// `row`.  kShared true: scale_codes[q][j] / scales[q][j] are the scale code
// and the second-level scale of ONE (row, block) pair per lane and load, as
// loaded; the step that consumes the batch decodes them, and the lanes that
// need a scale fetch it from the lane that holds it (see scale_of below).
template <int kRows, int kSegments, bool kShared>
struct RowBatch {
    uint2_vec codes[kRows][kSegments];
    float scales[kShared ? scale_loads(kRows) : kRows][kSegments];
    unsigned scale_codes[kShared ? scale_loads(kRows) : 1]
                        [kShared ? kSegments : 1];
    float offset;  // of the member the batch belongs to (uniform)
};

static_assert(RTHIP_GEMV_ROWS <= 4, "two scale loads cover four rows");

// kX: x rows held per thread (1, 2 or 4; a 3-row call runs as 4 with a zero
// row).  kSegments: segments per thread.  kRows: weight rows per batch.
// kTeams: teams per workgroup (2 teams of four wavefronts, or 1 team of eight
// for rows so wide that four wavefronts' threads could not hold their x).
// kGrouped: more than one member (a single weight compiles to the same code as
// before: every member selection folds to member 0).
template <int kX, int kSegments, int kRows, int kTeams, int kDepth,
          bool kDoubleQuantized, bool kGrouped>
__global__ __launch_bounds__(workgroup_threads(kTeams)) void gemv_forward_kernel(
    const float* __restrict__ x, GemvGroup group, unsigned second_level_shift,
    unsigned x_rows, unsigned input_width, unsigned block_shift,
    unsigned batch_count, unsigned iterations, LoraEpilogue lora
) {
    constexpr int kThreads = workgroup_threads(kTeams);
    // threads that share one weight row
    constexpr int kTeamThreads = kThreads / kTeams;
    constexpr int kTeamWaves = kTeamThreads / kWave;
    constexpr int kValues = kRows * kX;
    constexpr unsigned kMaxIterations = kParkedValues / kValues;
    __shared__ __attribute__((aligned(256))) char table[kPairTableBytes];
    __shared__ float partial[kTeams][kMaxIterations][kTeamWaves][kValues];

    const unsigned team =
        __builtin_amdgcn_readfirstlane(threadIdx.x / kTeamThreads);
    const unsigned thread = threadIdx.x % kTeamThreads;  // within the team
    const unsigned lane = thread % kWave;
    const unsigned segment_count = input_width / kSegment;

    // The hardware range check covers the per-lane offset only, not the
    // scalar offset, so every weight row gets descriptors of its own: base at
    // the row's first code byte / first scale, extent one row (zero for rows
    // past the output width).  They are built with a few scalar instructions
    // per row; lanes past the row end then read zeros instead of memory
    // beyond the payload.
    const unsigned row_code_bytes = input_width / 2;
    const unsigned row_blocks = input_width >> block_shift;
    // The member that the batches being REQUESTED belong to.  A team's batch
    // numbers only grow, so the member only moves forward: its fields live in
    // scalar registers and are re-read from the kernel arguments in the rare
    // step that crosses into the next member (a uniform branch without any
    // vector memory access in it, so the wait counts around it stay exact).
    // Batches past the last one stay with the last member, where their rows
    // lie past its output width.
    unsigned member_index = 0;
    GemvMember member = group.member[0];
    unsigned member_end = kGrouped ? group.member[1].first_batch : 0xFFFFFFFFU;
    const auto seek_member = [&](unsigned batch_index) {
        if constexpr (kGrouped) {
            while (batch_index >= member_end) {
                ++member_index;
                member = group.member[member_index];
                member_end = member_index + 1 < kGemvGroupMax
                                 ? group.member[member_index + 1].first_batch
                                 : 0xFFFFFFFFU;
            }
        }
    };
    // Plain fp32 scales are loaded by the lane that uses them, one per row
    // and stripe.  For the nested encoding that would mean two loads and a
    // decode (with a division) per row, which nearly doubles the kernel's
    // work, so those are shared: a wavefront's 64 segments of a row span 1024
    // weights = P = max(1, 1024 / B) quantisation blocks, the kRows rows of a
    // batch need only kRows x P scales per wavefront, lane l of load q fetches
    // and decodes the scale of row q x (64 / P) + l / P, block l % P of the
    // wavefront's range, and the lanes that own weights of that block read it
    // from lane l with one ds_bpermute: one decode per lane and batch instead
    // of kRows.  (Sharing plain fp32 scales the same way measured 2-4 %
    // slower than loading them: the ds_bpermute costs more than the load it
    // replaces.)  These loads go through a descriptor of the member's whole
    // scale array.
    // lanes per block (log2), blocks per wavefront-row (log2), rows per load
    const unsigned lanes_shift = block_shift - 4;
    const unsigned p_shift = lanes_shift < 6 ? 6 - lanes_shift : 0;
    const unsigned rows_per_load = 64U >> p_shift;
    const unsigned my_row = lane >> p_shift;          // within a load
    const unsigned my_block = lane & ((1U << p_shift) - 1);
    // lane that holds the scale of MY weights of row r of a load
    const unsigned my_source =
        (lanes_shift < 6 ? (lane >> lanes_shift) : 0U) * 4;  // byte address
    const unsigned wave_in_team = thread / kWave;

    // Per-lane constants: where this thread's segments sit inside a row.  The
    // row width is a multiple of the block size, so a row starts on a block
    // boundary and (row block) + (segment block) is the flat block index.
    unsigned segment_weights[kSegments];
#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
        segment_weights[j] = (thread + kTeamThreads * j) * kSegment;
    }

    using Batch = RowBatch<kRows, kSegments, kDoubleQuantized>;
    constexpr int kScaleLoads = scale_loads(kRows);
    const auto load_batch = [&](Batch& batch, unsigned batch_index) {
        seek_member(batch_index);
        const unsigned output_width = member.output_width;
        const std::uint8_t* const codes = member.codes;
        const void* const primary_scales = member.primary_scales;
        const unsigned first_row = (batch_index - member.first_batch) * kRows;
        batch.offset = member.offset;
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            const unsigned o = first_row + row;  // scalar
            const bool row_valid = o < output_width;
            const std::size_t row_start =
                static_cast<std::size_t>(o) * input_width;
            const __amdgpu_buffer_rsrc_t code_row = make_buffer(
                codes + (row_start >> 1), row_valid ? row_code_bytes : 0U);
            const __amdgpu_buffer_rsrc_t scale_row = make_buffer(
                static_cast<const float*>(primary_scales) +
                    (row_start >> block_shift),
                row_valid && !kDoubleQuantized ? row_blocks * 4 : 0U);
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                batch.codes[row][j] = __builtin_amdgcn_raw_buffer_load_b64(
                    code_row, segment_weights[j] >> 1, 0, 0);
                if constexpr (!kDoubleQuantized) {
                    batch.scales[row][j] = __builtin_bit_cast(
                        float,
                        __builtin_amdgcn_raw_buffer_load_b32(
                            scale_row,
                            (segment_weights[j] >> block_shift) * 4, 0, 0));
                }
            }
        }
        if constexpr (!kDoubleQuantized) {
            return;
        }
        const unsigned block_total =
            (output_width * input_width) >> block_shift;  // < 2^32 / 32
        const __amdgpu_buffer_rsrc_t primary_buffer =
            make_buffer(primary_scales, block_total);
        const __amdgpu_buffer_rsrc_t secondary_buffer =
            make_buffer(member.secondary_scales, member.secondary_bytes);
        // Every load is always issued (a second one is needed for block size
        // 32 only; otherwise every lane's offset is the rejected one and no
        // memory is touched): a branch here would sit between these loads
        // and the waits of the step that issued them.
#pragma unroll
        for (int q = 0; q < kScaleLoads; ++q) {
            const unsigned row_in_batch = q * rows_per_load + my_row;
            const unsigned o = first_row + row_in_batch;
            const bool mine = row_in_batch < static_cast<unsigned>(kRows) &&
                              o < output_width;
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                // first weight of this wavefront's segments of stripe j
                const unsigned wave_first =
                    (wave_in_team * kWave + kTeamThreads * j) * kSegment;
                const unsigned block =
                    o * row_blocks + (wave_first >> block_shift) + my_block;
                batch.scale_codes[q][j] = __builtin_amdgcn_raw_buffer_load_b8(
                    primary_buffer, mine ? block : 0x80000000U, 0, 0);
                batch.scales[q][j] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               secondary_buffer,
                               mine ? (block >> second_level_shift) * 4
                                    : 0x80000000U,
                               0, 0));
            }
        }
    };
    // The scale of this lane's weights of row `row` (of the batch), stripe j.
    // held: this lane's decoded (row, block) scales of the batch.
    const auto scale_of = [&](const Batch& batch,
                              const float (&held)[kScaleLoads][kSegments],
                              int row, int j) {
        if constexpr (!kDoubleQuantized) {
            return batch.scales[row][j];
        } else {
            const unsigned q = static_cast<unsigned>(row) / rows_per_load;
            const unsigned row_in_load =
                static_cast<unsigned>(row) % rows_per_load;
            return __builtin_bit_cast(
                float, __builtin_amdgcn_ds_bpermute(
                           static_cast<int>(((row_in_load << p_shift) * 4) +
                                            my_source),
                           __builtin_bit_cast(
                               int, q == 0 ? held[0][j]
                                           : held[kScaleLoads - 1][j])));
        }
    };

    // Batches are dealt round-robin: iteration i of workgroup g, team t takes
    // batch (i * gridDim.x + g) * kTeams + t.
    const unsigned stride = gridDim.x * kTeams;
    const unsigned first_batch = blockIdx.x * kTeams + team;

    // A ring of register batches: batch i lives in slot i % kDepth and is
    // requested kDepth - 1 batches before it is used.  (Loads past the last
    // batch are range-checked to zero by the buffer descriptor.)
    Batch ring[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d) {
        load_batch(ring[d], first_batch + d * stride);
    }

    // This thread's slice of x, resident for the whole kernel.  Segments past
    // the row end and rows past x_rows read as zero.  The loads are issued
    // here and consumed only after the table is built, so that their latency
    // and the build overlap.
    float xs[kX][kSegments][kSegment];
    bool x_valid[kX][kSegments];
#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
        const bool segment_valid = thread + kTeamThreads * j < segment_count;
        const unsigned clamped =
            min(thread + kTeamThreads * j, segment_count - 1) * kSegment;
#pragma unroll
        for (int r = 0; r < kX; ++r) {
            x_valid[r][j] =
                segment_valid && static_cast<unsigned>(r) < x_rows;
            const unsigned source_row =
                min(static_cast<unsigned>(r), x_rows - 1);
            const float4* source = reinterpret_cast<const float4*>(
                x + source_row * input_width + clamped);
#pragma unroll
            for (int q = 0; q < kSegment / 4; ++q) {
                const float4 v = source[q];
                xs[r][j][4 * q + 0] = v.x;
                xs[r][j][4 * q + 1] = v.y;
                xs[r][j][4 * q + 2] = v.z;
                xs[r][j][4 * q + 3] = v.w;
            }
        }
    }

    build_pair_table<kThreads>(table);
    __syncthreads();

#pragma unroll
    for (int j = 0; j < kSegments; ++j) {
#pragma unroll
        for (int r = 0; r < kX; ++r) {
#pragma unroll
            for (int i = 0; i < kSegment; ++i) {
                xs[r][j][i] = x_valid[r][j] ? xs[r][j][i] : 0.0F;
            }
        }
    }

    const unsigned lane_bits = pair_table_lane_bits(lane);

    // One batch: refill the slot freed by the previous batch, compute
    // `current`, reduce, park.
    // kRefill: whether a batch kDepth - 1 steps ahead exists.  It is a
    // compile-time property of the call, not a branch around the loads: with
    // a branch, the compiler's wait counts must assume the path WITHOUT the
    // new loads, so every wait for the current batch would also wait for the
    // loads just issued and nothing would be prefetched.
    const auto step = [&](const Batch& current, Batch& refill,
                          unsigned iteration, auto refill_exists) {
        constexpr bool kRefill = decltype(refill_exists)::value;
        const unsigned batch_index = first_batch + iteration * stride;
        // The table address bits pass through an empty asm in the copy that
        // loads: the lookups' address arithmetic is otherwise identical in
        // both copies, gets hoisted above the branch between them, and drags
        // the wait for the current codes in front of the new loads.
        unsigned step_lane_bits = lane_bits;
        if constexpr (kRefill) {
            load_batch(refill, batch_index + (kDepth - 1) * stride);
            asm volatile("" : "+v"(step_lane_bits)::"memory");
        }

        // Table lookups run one weight row ahead of the multiply-adds that
        // consume them: a row's 8 * kSegments ds_read_b64 are all in flight
        // while the previous row is accumulated, which keeps the LDS queue
        // deep enough to stream at its full rate.
        float2 levels[2][kSegments][8];
        const auto look_up = [&](int row, float2 (&out)[kSegments][8]) {
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                const unsigned words[2] = {current.codes[row][j].x,
                                           current.codes[row][j].y};
#pragma unroll
                for (int w = 0; w < 2; ++w) {
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        out[j][4 * w + b] =
                            pair_table_lookup(table, words[w], b,
                                              step_lane_bits);
                    }
                }
            }
        };

        // Nested scales are decoded here, a step after they were requested.
        float held[kScaleLoads][kSegments];
        if constexpr (kDoubleQuantized) {
            const float scale_offset = current.offset;
#pragma unroll
            for (int q = 0; q < kScaleLoads; ++q) {
#pragma unroll
                for (int j = 0; j < kSegments; ++j) {
                    held[q][j] = decode_double_quantized_scale(
                        static_cast<std::uint8_t>(current.scale_codes[q][j]),
                        current.scales[q][j], scale_offset);
                }
            }
        }

        float acc[kValues];
        look_up(0, levels[0]);
#pragma unroll
        for (int row = 0; row < kRows; ++row) {
            if (row + 1 < kRows) {
                look_up(row + 1, levels[(row + 1) & 1]);
            }
            __builtin_amdgcn_sched_barrier(0);
            float row_acc[kX];
#pragma unroll
            for (int r = 0; r < kX; ++r) {
                row_acc[r] = 0.0F;
            }
            float row_scale[kSegments];
#pragma unroll
            for (int j = 0; j < kSegments; ++j) {
                row_scale[j] = scale_of(current, held, row, j);
            }
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
                for (int p = 0; p < 8; ++p) {
                    const float2 pair = levels[row & 1][j][p];
#pragma unroll
                    for (int r = 0; r < kX; ++r) {
                        even[r] += xs[r][j][2 * p] * pair.x;
                        odd[r] += xs[r][j][2 * p + 1] * pair.y;
                    }
                }
#pragma unroll
                for (int r = 0; r < kX; ++r) {
                    row_acc[r] += (even[r] + odd[r]) * row_scale[j];
                }
            }
#pragma unroll
            for (int r = 0; r < kX; ++r) {
                acc[row * kX + r] = row_acc[r];
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // Totals of each 16-lane DPP row, then of the wavefront's four rows;
        // the wavefront parks them and nobody waits here.
        float total = transposed_row_sum<kValues>(acc, lane);
        total = sum_over_rows(total);
        if (lane < kValues) {
            partial[team][iteration][thread / kWave]
                   [slot_of_lane<kValues>(lane)] = total;
        }
    };

    // Walk the ring with static slot numbers (no register copies).  The last
    // kDepth - 1 steps have nothing left to request; they run the copy of the
    // step that issues no loads.
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
    // has been parked.  Each team adds up its four wavefront partials per
    // value and writes y.
    __syncthreads();
    for (unsigned index = thread; index < iterations * kValues;
         index += kTeamThreads) {
        const unsigned iteration = index / kValues;
        const unsigned value = index % kValues;
        const unsigned batch_index = first_batch + iteration * stride;
        // which member the batch belongs to: per lane here
        const unsigned m =
            !kGrouped
                ? 0U
                : (batch_index >= group.member[1].first_batch ? 1U : 0U) +
                      (batch_index >= group.member[2].first_batch ? 1U : 0U) +
                      (batch_index >= group.member[3].first_batch ? 1U : 0U);
        const unsigned output_width = RTHIP_MEMBER(m, output_width);
        const unsigned o =
            (batch_index - RTHIP_MEMBER(m, first_batch)) * kRows + value / kX;
        const unsigned r = value % kX;
        if (batch_index < batch_count && o < output_width && r < x_rows) {
            float sum = 0.0F;
#pragma unroll
            for (int wave = 0; wave < kTeamWaves; ++wave) {
                sum += partial[team][iteration][wave][value];
            }
            const float* const bias = RTHIP_MEMBER(m, bias);
            if (bias != nullptr) {
                sum += bias[o];
            }
            if (!kGrouped && lora.reduced != nullptr) {
                sum += lora_term(lora, r, o);
            }
            float* const y = RTHIP_MEMBER(m, y);
            y[r * output_width + o] = sum;
        }
    }
}

std::size_t segments_per_thread(const LinearProblem& p,
                                std::size_t team_threads) {
    return (p.input_width / kSegment + team_threads - 1) / team_threads;
}

// x rows held per thread (a 3-row call runs as 4 with a zero row).
std::size_t held_rows(const LinearProblem& p) {
    return p.rows == 3 ? 4 : p.rows;
}

// What a thread keeps in registers grows with both the x rows it holds (its
// slice of x: held rows x segments x 16 values) and the segments it takes of a
// weight row (the looked-up levels of two rows: 32 values per segment).  These
// combinations fit the 256 registers without spills: one x row with up to four
// segments, two with up to three, four with up to two.
constexpr bool fits_registers(std::size_t held, std::size_t segments) {
    return segments >= 1 && (held == 1   ? segments <= 4
                             : held == 2 ? segments <= 3
                                         : segments <= 2);
}
// Two teams of 256 threads per workgroup measured best; rows too wide for
// that get one team of 512 (half the segments per thread): four rows of x
// from 8192 weights per row on, two from 12288, one from 16384 to 32768.
bool wide_team(const LinearProblem& p) {
    return !fits_registers(held_rows(p), segments_per_thread(p, 256));
}

// The weights of one launch: `count` problems that share activations, row
// count, row width, block size and scale encoding.
struct Launch {
    const LinearProblem* problems;
    std::size_t count;
};

// Launches that read this many bytes of codes or more run sixteen wavefronts
// per workgroup instead of eight: a long run gains from the fuller issue
// slots (32000 x 4096: 17.2 -> 16.8 us, nested scales 19.6 -> 17.9 us), a
// short one loses more at its start (4096 x 4096: 4.7 -> 5.2 us; two
// 11008 x 4096 in one launch: 12.9 -> 14.3 us).
constexpr std::size_t kLargeLaunchBytes = std::size_t{60} << 20;

template <int kX, int kSegments, bool kDoubleQuantized, bool kGrouped,
          bool kWide = false, bool kLarge = false>
void launch_instance(const Launch& launch, hipStream_t stream) {
    // Two teams (eight wavefronts) per workgroup measured best on MI355X; a
    // thread that carries more x rows or segments takes fewer weight rows per
    // batch so that its registers fit.
    constexpr bool kLight = kX * kSegments == 1;
    static_assert(!kLarge || (kX * kSegments == 1 && !kWide));
    constexpr int kTeams =
        kWide ? 1 : (kLarge ? 4 : (kLight ? RTHIP_GEMV_TEAMS : 2));
    // Rows of three and more segments per thread (wider than 8192 weights)
    // also take two: a 4096 x 11008 weight has only two four-row batches per
    // team, and the multiply of the last one is exposed (9.3 -> 8.6 us).
    constexpr int kRows =
        kLight ? RTHIP_GEMV_ROWS
               : (kX * kSegments <= 4 && kSegments < 3 ? 4 : 2);
    constexpr int kDepth = kLight ? RTHIP_GEMV_DEPTH : 2;
    constexpr unsigned kMaxIterations = kParkedValues / (kRows * kX);
    const LinearProblem& first = launch.problems[0];
    GemvGroup group{};
    unsigned batch_count = 0;
    for (std::size_t m = 0; m < kGemvGroupMax; ++m) {
        GemvMember& member = group.member[m];
        if (m >= launch.count) {
            member.first_batch = 0xFFFFFFFFU;
            continue;
        }
        const LinearProblem& p = launch.problems[m];
        const std::size_t block_count =
            (p.output_width * p.input_width) >> p.block_shift;
        member.codes = p.weight.codes;
        member.primary_scales = p.weight.primary_scales;
        member.secondary_scales = p.weight.secondary_scales;
        member.bias = p.bias;
        member.y = p.result;
        member.output_width = static_cast<unsigned>(p.output_width);
        member.first_batch = batch_count;
        member.secondary_bytes =
            kDoubleQuantized
                ? static_cast<unsigned>(
                      (((block_count - 1) >> p.weight.second_level_shift) + 1) *
                      4)
                : 0U;
        member.offset = p.weight.offset;
        batch_count +=
            static_cast<unsigned>((p.output_width + kRows - 1) / kRows);
    }
    const unsigned team_groups = (batch_count + kTeams - 1) / kTeams;
    // One workgroup per CU; more when a team would otherwise need more
    // batches than its LDS parking space holds.
    unsigned blocks = team_groups < kComputeUnits ? team_groups : kComputeUnits;
    if ((team_groups + blocks - 1) / blocks > kMaxIterations) {
        blocks = (team_groups + kMaxIterations - 1) / kMaxIterations;
    }
    const unsigned iterations = (team_groups + blocks - 1) / blocks;
    gemv_forward_kernel<kX, kSegments, kRows, kTeams, kDepth, kDoubleQuantized,
                        kGrouped><<<blocks, workgroup_threads(kTeams), 0, stream>>>(
        first.activations, group, first.weight.second_level_shift,
        static_cast<unsigned>(first.rows),
        static_cast<unsigned>(first.input_width), first.block_shift,
        batch_count, iterations, first.lora);
}

// One instance per (x rows, segments) pair that fits; the others are never
// compiled.
template <int kX, int kSegments, bool kDoubleQuantized, bool kGrouped,
          bool kWide>
void launch_fitting(const Launch& launch, hipStream_t stream) {
    if constexpr (fits_registers(kX, kSegments)) {
        launch_instance<kX, kSegments, kDoubleQuantized, kGrouped, kWide>(
            launch, stream);
    }
}

template <int kX, bool kDoubleQuantized, bool kGrouped>
void launch_segments(const Launch& launch, hipStream_t stream) {
    const LinearProblem& p = launch.problems[0];
    if (wide_team(p)) {
        // one 512-thread team per weight row
        switch (segments_per_thread(p, 512)) {
        case 2:
            launch_fitting<kX, 2, kDoubleQuantized, kGrouped, true>(launch,
                                                                    stream);
            break;
        case 3:
            launch_fitting<kX, 3, kDoubleQuantized, kGrouped, true>(launch,
                                                                    stream);
            break;
        default:
            launch_fitting<kX, 4, kDoubleQuantized, kGrouped, true>(launch,
                                                                    stream);
            break;
        }
        return;
    }
    switch (segments_per_thread(p, 256)) {
    case 1:
        if constexpr (kX == 1) {
            std::size_t code_bytes = 0;
            for (std::size_t m = 0; m < launch.count; ++m) {
                code_bytes += launch.problems[m].output_width *
                              launch.problems[m].input_width / 2;
            }
            if (code_bytes >= kLargeLaunchBytes) {
                launch_instance<1, 1, kDoubleQuantized, kGrouped, false, true>(
                    launch, stream);
                break;
            }
        }
        launch_instance<kX, 1, kDoubleQuantized, kGrouped>(launch, stream);
        break;
    case 2:
        launch_fitting<kX, 2, kDoubleQuantized, kGrouped, false>(launch,
                                                                 stream);
        break;
    case 3:
        launch_fitting<kX, 3, kDoubleQuantized, kGrouped, false>(launch,
                                                                 stream);
        break;
    default:
        launch_fitting<kX, 4, kDoubleQuantized, kGrouped, false>(launch,
                                                                 stream);
        break;
    }
}

template <bool kDoubleQuantized, bool kGrouped>
void launch_rows(const Launch& launch, hipStream_t stream) {
    switch (launch.problems[0].rows) {
    case 1: launch_segments<1, kDoubleQuantized, kGrouped>(launch, stream); break;
    case 2: launch_segments<2, kDoubleQuantized, kGrouped>(launch, stream); break;
    default: launch_segments<4, kDoubleQuantized, kGrouped>(launch, stream); break;
    }
}

template <bool kGrouped>
void launch_encoding(const Launch& launch, hipStream_t stream) {
    if (launch.problems[0].weight.encoding == 0) {
        launch_rows<false, kGrouped>(launch, stream);
    } else {
        launch_rows<true, kGrouped>(launch, stream);
    }
}

}  // namespace

bool gemv_forward_supports(const LinearProblem& p) {
    constexpr std::size_t kMaxWidth =
        static_cast<std::size_t>(kSegment) * 512 * 4;
    return p.rows >= 1 && p.rows <= kGemvMaxRows &&
           // the registers must hold a thread's share, with two teams of 256
           // threads or one team of 512 (then at least two segments each)
           (!wide_team(p) ||
            (segments_per_thread(p, 512) >= 2 &&
             fits_registers(held_rows(p), segments_per_thread(p, 512)))) &&
           p.input_width % kSegment == 0 && p.input_width <= kMaxWidth &&
           // rows start on block boundaries (scalar row offset into scales)
           p.input_width % (std::size_t{1} << p.block_shift) == 0 &&
           p.output_width * p.input_width < (1ULL << 32) &&
           p.rows * p.input_width < (1ULL << 32) &&
           p.rows * p.output_width < (1ULL << 32) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 8 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

void launch_gemv_forward(const LinearProblem& p, hipStream_t stream) {
    if (gemv1_forward_supports(p)) {  // one row of x: the kernel of its own
        launch_gemv1_forward(&p, 1, stream);
        return;
    }
    launch_encoding<false>(Launch{&p, 1}, stream);
}

bool gemv_group_supports(const LinearProblem* problems, std::size_t count) {
    if (count < 1 || count > kGemvGroupMax) {
        return false;
    }
    const LinearProblem& first = problems[0];
    std::size_t batches = 0;
    for (std::size_t m = 0; m < count; ++m) {
        const LinearProblem& p = problems[m];
        if (!gemv_forward_supports(p) || p.activations != first.activations ||
            p.rows != first.rows || p.input_width != first.input_width ||
            p.block_shift != first.block_shift ||
            p.weight.encoding != first.weight.encoding ||
            p.weight.second_level_shift != first.weight.second_level_shift ||
            p.lora.reduced != nullptr) {
            return false;
        }
        batches += (p.output_width + 1) / 2;  // at least two rows per batch
    }
    return batches < (1ULL << 31);
}

void launch_gemv_group(const LinearProblem* problems, std::size_t count,
                       hipStream_t stream) {
    if (count == 1) {
        launch_gemv_forward(problems[0], stream);
        return;
    }
    // Members that the one-row kernel takes go to it together, the others
    // stay with this file's kernel: either way a member's output is what its
    // launch alone writes, bit for bit.
    LinearProblem one_row[kGemvGroupMax];
    LinearProblem other[kGemvGroupMax];
    std::size_t one_row_count = 0;
    std::size_t other_count = 0;
    for (std::size_t m = 0; m < count; ++m) {
        if (gemv1_forward_supports(problems[m])) {
            one_row[one_row_count++] = problems[m];
        } else {
            other[other_count++] = problems[m];
        }
    }
    if (one_row_count != 0) {
        launch_gemv1_forward(one_row, one_row_count, stream);
    }
    if (other_count == 1) {
        launch_encoding<false>(Launch{other, 1}, stream);
    } else if (other_count > 1) {
        launch_encoding<true>(Launch{other, other_count}, stream);
    }
}

}  // namespace rthip
