// Forward product for up to 128 rows when a row of the weight is short enough
// for x to live in registers (row width 1024, 2048, 3072 or 4096):
//     y[r, o] = sum_i x[r, i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81).
//
// The small-batch kernel of nf4_skinny.hip stages x through LDS slab by slab,
// which costs two workgroup barriers per 256 contraction values; with 16 rows
// those barriers and the copies take longer than the matrix instructions.
// Here the contraction axis is cut ACROSS the eight wavefronts of a workgroup
// instead: wavefront w owns contraction values [w I/8, (w+1) I/8) of every
// weight row, its 16 x I/8 slice of x is loaded into registers once (I/32
// values per lane, at most 128; coalesced loads passed through a per-wavefront
// LDS area) and stays there, and a workgroup streams 16-row tiles of the weight
// with no barrier and no LDS traffic for x in the loop -- the structure of the
// GEMV, with matrix instructions instead of lane sums.  What it pays for this
// is that every workgroup reads all of x (256 KB for 16 x 4096) once.
//
//   * v_mfma_f32_16x16x4_f32: A is x[16 rows][4 k], B is W^T[4 k][16 weight
//     rows].  Lane l supplies x row l % 16, weight row l % 16 and contraction
//     quarter q = l / 16.  The 128 values of contraction group g of a wavefront
//     are dealt to the quarters in runs of 32: lane (n, q) owns
//         k = w I/8 + 128 g + 32 q + [0, 32)
//     of weight row n (one 16-byte load; the four lanes of a row read 64
//     contiguous bytes) and the same k of x row n.  Any assignment of k to
//     (quarter, instruction) is valid as long as A and B agree.
//   * Decode as everywhere: a code byte indexes the replicated pair table in
//     LDS (one v_perm_b32 + one ds_read_b64 per two weights), each level times
//     its block scale in one rounded multiply.  The lookups of the next 16
//     weights are issued before the 16 matrix instructions of the current
//     ones.
//   * Tiles are dealt round-robin to one persistent workgroup per compute
//     unit; the codes of tile t + 1 are requested before tile t is computed.
//   * More than 16 rows of x are handled as up to eight row groups of 16: a
//     workgroup holds ONE row group for its whole life, and the work items
//     (tile, row group) are numbered so that the row groups of a tile go to
//     workgroups eight apart in the grid -- the same XCD, in the same round of
//     the dispatch -- which read the tile's weights at about the same time, so
//     the weights come from HBM once and from that XCD's L2 for the others.
//   * A wavefront parks its 16 x 16 partial tile in LDS; every four tiles
//     (and at the end) the workgroup meets at a barrier, adds the eight
//     partial tiles of each parked output tile in wavefront order and writes y
//     with bias and adapter term.  Nothing depends on scheduling.
//   * Several weights that share x (the query, key and value projections; the
//     gate and up projections) can run as ONE launch: their tiles, each
//     weight's padded to a multiple of eight, are numbered one after the other
//     and dealt exactly as one weight's tiles are, so every output is computed
//     by the same lanes in the same order as in a launch of its own -- bit
//     for bit the same -- while the launch, the table and the x slice are
//     paid for once (at 16 rows of 4096 the x slice alone is a quarter of a
//     single launch).  The member a tile belongs to is looked up per tile
//     from the kernel arguments (scalar work, a few dozen instructions).

#include "kernels.hpp"
#include "launch_config.hpp"
#include "nf4_decode.hpp"
#include "nf4_pair_table.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;
constexpr int kWaves = 8;
constexpr int kTileRows = 16;        // weight rows per tile
constexpr int kGroupWeights = 128;   // contraction values per wavefront group
constexpr int kLaneWeights = 32;     // of which one lane owns this many
constexpr unsigned kComputeUnits = 256;
constexpr unsigned kParkTiles = 4;  // tiles a workgroup parks between flushes
// Per-wavefront LDS area that x passes through on its way into registers:
// [16 rows][128 values], rows padded by four floats.
constexpr unsigned kStagingStride = kGroupWeights + 4;
constexpr unsigned kStagingFloats = kTileRows * kStagingStride;
constexpr std::size_t kStagingBytes =
    static_cast<std::size_t>(kWaves) * kStagingFloats * sizeof(float);
constexpr unsigned kRejectedOffset = 0x80000000U;  // fails every range check

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base,
                                                            std::size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// The weights of one launch.  Tiles are numbered member after member, each
// member's count padded to a multiple of eight; first_tile of the slots past
// `count` is the total.
struct ResidentMember {
    Nf4WeightView weight;
    const float* bias;
    float* y;
    unsigned output_width;
    LoraEpilogue lora;  // the member's adapter term (reduced == null: none)
};
struct ResidentGroup {
    ResidentMember member[kResidentGroupMax];
    unsigned first_tile[kResidentGroupMax + 1];
    unsigned count;
};

// kGroups: contraction groups per wavefront; the row width is 1024 * kGroups.
// kGrouped: more than one member (otherwise member 0 is used throughout and
// nothing is looked up per tile).
template <int kGroups, bool kDoubleQuantized, bool kGrouped>
__global__ __launch_bounds__(kThreads) void resident_forward_kernel(
    const float* __restrict__ x, ResidentGroup group, unsigned rows,
    unsigned block_shift, unsigned row_groups, unsigned iterations
) {
    constexpr unsigned kInputWidth = 1024U * kGroups;
    constexpr int kSubChunks = 2 * kGroups;  // 16 weights each
    // The table is a static array so that its LDS address is a compile-time
    // constant (zero) that folds into the lookups; the rest is sized at
    // launch.
    __shared__ __attribute__((aligned(256))) char table[kPairTableBytes];
    extern __shared__ __attribute__((aligned(256))) char shared[];
    // parked[iteration][wavefront][lane]: accumulator of that lane
    floatx4* parked = reinterpret_cast<floatx4*>(shared);

    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const unsigned quarter = lane / 16;
    const unsigned lane_row = lane % 16;
    // first contraction value of this lane in group 0
    const unsigned k_base =
        wave * (kInputWidth / kWaves) + quarter * kLaneWeights;
    // Work item w = blockIdx.x + i * gridDim.x of iteration i is tile
    // 8 (w / (8 G)) + w % 8 and row group (w / 8) % G.  The grid is a multiple
    // of 8 G, so the row group is the same in every iteration.
    const unsigned row_base = (blockIdx.x / 8) % row_groups * kTileRows;
    const unsigned rows_here = min(rows - row_base, 16U);
    const auto tile_of = [&](unsigned iteration) {
        const unsigned item = blockIdx.x + iteration * gridDim.x;
        return item / (8 * row_groups) * 8 + item % 8;
    };

    const __amdgpu_buffer_rsrc_t x_buffer = raw_buffer(
        x, static_cast<std::size_t>(rows) * kInputWidth * sizeof(float));

    // What the loads of one member need (all of it scalar).
    struct Source {
        __amdgpu_buffer_rsrc_t codes, primary, secondary;
        float offset;
        unsigned second_level_shift;
        unsigned output_width;
        unsigned first_tile;
    };
    const auto source_of = [&](unsigned m) {
        const ResidentMember& member = group.member[m];
        const std::size_t elements =
            static_cast<std::size_t>(member.output_width) *
            kInputWidth;  // < 2^32
        const std::size_t block_total =
            (elements + (std::size_t{1} << block_shift) - 1) >> block_shift;
        Source source;
        source.codes = raw_buffer(member.weight.codes, elements / 2);
        source.primary =
            raw_buffer(member.weight.primary_scales,
                       block_total * (kDoubleQuantized ? 1 : 4));
        source.secondary = raw_buffer(
            member.weight.secondary_scales,
            kDoubleQuantized
                ? (((block_total - 1) >> member.weight.second_level_shift) +
                   1) * 4
                : 0);
        source.offset = member.weight.offset;
        source.second_level_shift = member.weight.second_level_shift;
        source.output_width = member.output_width;
        source.first_tile = kGrouped ? group.first_tile[m] : 0U;
        return source;
    };
    // The member that owns a tile (tiles past the last one: the last member,
    // whose row check then fails).
    const auto member_of = [&](unsigned tile) {
        unsigned m = 0;
        if constexpr (kGrouped) {
#pragma unroll
            for (unsigned next = 1; next < kResidentGroupMax; ++next) {
                if (next < group.count && tile >= group.first_tile[next]) {
                    m = next;
                }
            }
        }
        return m;
    };
    const Source only = source_of(0);  // (unused code when kGrouped)

    struct Codes {
        uintx4 codes[kGroups];  // 32 nibbles each
        float scales[kGroups];
    };
    // Tiles past the workgroup's last one, and weight rows past the output
    // width, read as zeros.
    const auto load_codes = [&](Codes& staged, unsigned tile) {
        Source source = only;
        if constexpr (kGrouped) {
            source = source_of(member_of(tile));
        }
        // (a tile is never below its member's first; padding tiles and
        // tiles past the last member fail the row check)
        const unsigned n = (tile - source.first_tile) * kTileRows + lane_row;
        // Real offsets stay below 2^31; lanes with nothing to read get bit 31
        // set, which the range check rejects.  (One value, kept opaque: a
        // select per load invites the compiler to branch around the loads,
        // and its wait counts are exact only on straight-line code.)
        unsigned reject = n < source.output_width ? 0U : kRejectedOffset;
        asm volatile("" : "+v"(reject));
        const unsigned flat = n * kInputWidth + k_base;
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
            const unsigned first = flat + kGroupWeights * g;
            staged.codes[g] = __builtin_bit_cast(
                uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                            source.codes, (first >> 1) | reject, 0, 0));
            const unsigned block = first >> block_shift;
            if constexpr (!kDoubleQuantized) {
                staged.scales[g] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               source.primary, (block * 4) | reject, 0, 0));
            } else {
                const std::uint8_t scale_code =
                    __builtin_amdgcn_raw_buffer_load_b8(
                        source.primary, block | reject, 0, 0);
                const float second = __builtin_bit_cast(
                    float,
                    __builtin_amdgcn_raw_buffer_load_b32(
                        source.secondary,
                        ((block >> source.second_level_shift) * 4) | reject,
                        0, 0));
                // Lanes with nothing to read decode (0, 0.0) into the
                // offset: finite, and never written.
                staged.scales[g] = decode_double_quantized_scale(
                    scale_code, second, source.offset);
            }
        }
    };

    Codes ring[2];
    load_codes(ring[0], tile_of(0));

    // This lane's slice of x: row lane % 16, resident for the whole kernel.
    // A lane's values are 128 contiguous bytes of one x row, and the 16 rows
    // of a wavefront lie a whole row apart, so loading them directly would
    // touch 64 cache lines per instruction.  Each wavefront therefore reads
    // its [16 rows][128] piece of group g with coalesced loads (two x rows per
    // instruction, 512 contiguous bytes each), passes it through a private
    // LDS area and picks up its own values from there.  Rows past `rows` read
    // as zero.
    float* staging =
        reinterpret_cast<float*>(shared) + wave * kStagingFloats;
    float xs[kGroups][kLaneWeights];
    {
        // chunk c = lane + 64 j of the piece: row c / 32, floats 4 (c % 32)
        const unsigned piece_row = lane / 32;
        const unsigned piece_column = (lane % 32) * 4;
        const auto load_piece = [&](floatx4 (&piece)[8], int g) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const unsigned row = piece_row + 2 * j;
                piece[j] = __builtin_bit_cast(
                    floatx4,
                    __builtin_amdgcn_raw_buffer_load_b128(
                        x_buffer,
                        row < rows_here
                            ? ((row_base + row) * kInputWidth +
                               wave * (kInputWidth / kWaves) +
                               kGroupWeights * g + piece_column) *
                                  static_cast<unsigned>(sizeof(float))
                            : kRejectedOffset,
                        0, 0));
            }
        };
        // All pieces are requested at once (their registers are free until
        // xs fills up), so the slice costs one round trip to L2, not one per
        // group.
        floatx4 pieces[kGroups][8];
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
            load_piece(pieces[g], g);
        }
#pragma unroll
        for (int g = 0; g < kGroups; ++g) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                *reinterpret_cast<floatx4*>(
                    staging + (piece_row + 2 * j) * kStagingStride +
                    piece_column) = pieces[g][j];
            }
            // (LDS operations of one wavefront complete in order)
#pragma unroll
            for (int v = 0; v < kLaneWeights / 4; ++v) {
                const floatx4 values = *reinterpret_cast<const floatx4*>(
                    staging + lane_row * kStagingStride +
                    quarter * kLaneWeights + 4 * v);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    xs[g][4 * v + e] = values[e];
                }
            }
        }
    }

    build_pair_table<kThreads>(table);
    const unsigned lane_bits = pair_table_lane_bits(lane);
    // The table is built, and every wavefront is done with its staging area,
    // which the parked tiles reuse.
    __syncthreads();

    // Sub-chunk s of a tile: 16 weights = two code words of group s / 2.
    float2 raw[8];
    const auto issue_lookups = [&](const Codes& codes, int s) {
        const unsigned words[2] = {codes.codes[s / 2][2 * (s % 2)],
                                   codes.codes[s / 2][2 * (s % 2) + 1]};
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int byte = 0; byte < 4; ++byte) {
                raw[4 * half + byte] =
                    pair_table_lookup(table, words[half], byte, lane_bits);
            }
        }
    };

    const auto compute = [&](const Codes& current, const Codes& next,
                             unsigned iteration) {
        floatx4 acc = {0.0F, 0.0F, 0.0F, 0.0F};
#pragma unroll
        for (int s = 0; s < kSubChunks; ++s) {
            float w[16];
            {
#pragma clang fp contract(off)
                const float scale = current.scales[s / 2];
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    w[2 * p] = raw[p].x * scale;
                    w[2 * p + 1] = raw[p].y * scale;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (s + 1 < kSubChunks) {
                issue_lookups(current, s + 1);
            } else {
                issue_lookups(next, 0);  // the next tile's first
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(
                    xs[s / 2][16 * (s % 2) + i], w[i], acc, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        parked[((iteration % kParkTiles) * kWaves + wave) * 64 + lane] = acc;
    };

    // Adds the eight wavefront partials of the tiles parked since the last
    // flush, in wavefront order, and writes y with bias and adapter term.
    // Accumulator element r of lane l is x row 4 (l / 16) + r and weight row
    // l % 16 of the tile.
    const auto flush = [&](unsigned first_iteration, unsigned count) {
        __syncthreads();  // every wavefront has parked these tiles
        for (unsigned index = thread; index < count * 256;
             index += kThreads) {
            const unsigned iteration = first_iteration + index / 256;
            const unsigned m_row = (index % 256) / 16;
            const unsigned column = index % 16;
            const unsigned tile = tile_of(iteration);
            // (a wavefront's 64 outputs belong to one tile)
            const unsigned m = kGrouped ? __builtin_amdgcn_readfirstlane(
                                              member_of(tile))
                                        : 0U;
            const ResidentMember& member = group.member[m];
            const unsigned first_tile = kGrouped ? group.first_tile[m] : 0U;
            const unsigned n = (tile - first_tile) * kTileRows + column;
            if (n >= member.output_width || m_row >= rows_here) {
                continue;
            }
            const float* source =
                reinterpret_cast<const float*>(
                    parked + (iteration % kParkTiles) * kWaves * 64 +
                    (m_row / 4) * 16 + column) +
                m_row % 4;
            float sum = 0.0F;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                sum += source[w * 64 * 4];  // wavefront order
            }
            if (member.bias != nullptr) {
                sum += member.bias[n];
            }
            if (member.lora.reduced != nullptr) {
                sum += lora_term(member.lora, row_base + m_row, n);
            }
            member.y[static_cast<std::size_t>(row_base + m_row) *
                         member.output_width +
                     n] = sum;
        }
        __syncthreads();  // the parking slots are free again
    };

    issue_lookups(ring[0], 0);
    for (unsigned iteration = 0; iteration < iterations; iteration += 2) {
        load_codes(ring[1], tile_of(iteration + 1));
        compute(ring[0], ring[1], iteration);
        if (iteration + 1 < iterations) {  // uniform
            load_codes(ring[0], tile_of(iteration + 2));
            compute(ring[1], ring[0], iteration + 1);
        }
        // The only barriers after the table build: one pair per kParkTiles
        // tiles.
        const unsigned done = min(iteration + 2, iterations);
        if (done % kParkTiles == 0 || done == iterations) {  // uniform
            const unsigned first = (done - 1) / kParkTiles * kParkTiles;
            flush(first, done - first);
        }
    }
}

template <int kGroups, bool kDoubleQuantized, bool kGrouped>
hipError_t launch_instance(const LinearProblem* problems, std::size_t count,
                           hipStream_t stream) {
    const LinearProblem& p = problems[0];
    ResidentGroup group{};
    unsigned tiles = 0;  // each member's padded to a multiple of eight
    for (std::size_t m = 0; m < kResidentGroupMax; ++m) {
        group.first_tile[m] = tiles;
        if (m < count) {
            const LinearProblem& member = problems[m];
            group.member[m].weight = member.weight;
            group.member[m].bias = member.bias;
            group.member[m].y = member.result;
            group.member[m].output_width =
                static_cast<unsigned>(member.output_width);
            group.member[m].lora = member.lora;
            tiles += static_cast<unsigned>(
                (member.output_width + kTileRows - 1) / kTileRows + 7) / 8 * 8;
        }
    }
    group.first_tile[kResidentGroupMax] = tiles;
    group.count = static_cast<unsigned>(count);
    const unsigned row_groups =
        static_cast<unsigned>((p.rows + kTileRows - 1) / kTileRows);
    // Work items (tile, row group).  One workgroup per compute unit, rounded
    // down to a multiple of 8 x row groups so that a workgroup keeps its row
    // group.
    const unsigned items = tiles * row_groups;
    const unsigned granule = 8 * row_groups;
    unsigned groups = kComputeUnits / granule * granule;
    if (groups > items) {
        groups = items;
    }
    const unsigned iterations = (items + groups - 1) / groups;
    const std::size_t shared_bytes = kStagingBytes;
    const auto kernel =
        resident_forward_kernel<kGroups, kDoubleQuantized, kGrouped>;
    // More than the default 64 KB of LDS.
    static_assert(kStagingBytes >=
                  kParkTiles * kWaves * 64 * sizeof(floatx4));
    static std::atomic<std::uint64_t> served{0};
    if (const hipError_t error = allow_dynamic_lds(
            reinterpret_cast<const void*>(kernel), kStagingBytes, served);
        error != hipSuccess) {
        return error;
    }
    kernel<<<groups, kThreads, shared_bytes, stream>>>(
        p.activations, group, static_cast<unsigned>(p.rows), p.block_shift,
        row_groups, iterations);
    return hipSuccess;
}

template <int kGroups>
hipError_t launch_groups(const LinearProblem* problems, std::size_t count,
                         hipStream_t stream) {
    const bool nested = problems[0].weight.encoding != 0;
    if (count == 1) {
        return nested ? launch_instance<kGroups, true, false>(problems, 1,
                                                              stream)
                      : launch_instance<kGroups, false, false>(problems, 1,
                                                               stream);
    }
    return nested
               ? launch_instance<kGroups, true, true>(problems, count, stream)
               : launch_instance<kGroups, false, true>(problems, count,
                                                       stream);
}

hipError_t launch_width(const LinearProblem* problems, std::size_t count,
                        hipStream_t stream) {
    switch (problems[0].input_width / 1024) {
    case 1: return launch_groups<1>(problems, count, stream);
    case 2: return launch_groups<2>(problems, count, stream);
    case 3: return launch_groups<3>(problems, count, stream);
    default: return launch_groups<4>(problems, count, stream);
    }
}

}  // namespace

bool resident_forward_supports(const LinearProblem& p) {
    return p.rows >= 1 && p.rows <= kResidentMaxRows &&
           p.input_width % 1024 == 0 && p.input_width <= 4096 &&
           // 32-bit flat weight indices; byte offsets into x, the codes and
           // the scales all stay below the rejected offset
           p.output_width * p.input_width < (1ULL << 32) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 16 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

hipError_t launch_resident_forward(const LinearProblem& p,
                                   hipStream_t stream) {
    return launch_width(&p, 1, stream);
}

bool resident_group_supports(const LinearProblem* problems,
                             std::size_t count) {
    if (count < 1 || count > kResidentGroupMax) {
        return false;
    }
    const LinearProblem& first = problems[0];
    std::size_t tiles = 0;
    for (std::size_t m = 0; m < count; ++m) {
        const LinearProblem& p = problems[m];
        if (!resident_forward_supports(p) ||
            p.activations != first.activations || p.rows != first.rows ||
            p.input_width != first.input_width ||
            p.block_shift != first.block_shift ||
            p.weight.encoding != first.weight.encoding) {
            return false;
        }
        tiles += (p.output_width + kTileRows - 1) / kTileRows + 8;
    }
    // tile numbers times row groups stay far inside 32 bits
    return tiles < (1ULL << 26);
}

hipError_t launch_resident_group(const LinearProblem* problems,
                                 std::size_t count, hipStream_t stream) {
    return launch_width(problems, count, stream);
}

}  // namespace rthip
