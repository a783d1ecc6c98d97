// Forward product for small batches (4 < rows <= 64):
//     y[r, o] = sum_i x[r, i] * codebook[code(o, i)] * scale(o, i / B)
// restating reference_quantized_linear_forward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81) where
// the weight stream still matters but there are enough rows to feed the matrix
// cores.
//
// With so few rows every decoded weight is used by ONE tile of x, so staging
// weights through LDS buys nothing: each lane decodes its weights straight into
// the register layout of the MFMA B operand, and every weight is decoded
// exactly once.  x, on the other hand, is needed by every weight row; what
// bounds a naive kernel is the L2 traffic of re-reading it.  So:
//
//   * v_mfma_f32_16x16x4_f32: A is x[16 rows][4 k], B is W^T[4 k][16 weight
//     rows].  Lane l feeds x row l % 16, weight row l % 16 and the k-quarter
//     l / 16.
//   * A workgroup of eight wavefronts owns a tile of 128 weight rows, 16 per
//     wavefront, and all eight walk the contraction axis together in slabs
//     of 256.  The x tile of a slab ([rows][256] floats) is copied to LDS
//     once and read by all eight wavefronts, which divides the L2 traffic for
//     x by eight compared with one 16-row tile per workgroup.
//   * In a slab a lane owns 64 consecutive weights of its row (two 16-byte
//     loads; a wavefront reads 128 contiguous bytes of each of its 16 rows)
//     and, per 16-row block of x, the 64 matching x values from LDS.  MFMA j
//     of the slab contracts k = 64 q + j over the four quarters q -- any
//     assignment of k to lanes is valid as long as A and B agree.
//   * Decode: code byte -> two levels through the replicated pair table (one
//     v_perm_b32 + one ds_read_b64 per two weights), times the block scale in
//     one rounded multiply each.
//   * Work split ("stream-K"): the (tile, slab) pairs, tile-major, are dealt
//     in equal contiguous runs to one workgroup per compute unit, so that every
//     unit carries the same load whatever the shape.  A workgroup that covers a
//     whole tile writes y directly.  Otherwise it writes a partial tile to a
//     workspace slot and a second small kernel adds the partial tiles of each
//     output tile in ascending workgroup order (plus bias), so results do not
//     depend on scheduling.
//   * The code bytes of the next two slabs and the x tile of the next slab
//     are in flight while the current slab computes.  Every load is a raw
//     buffer load whose range check (on the per-lane offset) returns zeros for
//     lanes with nothing to read, so nothing in the loop is predicated.

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
constexpr int kTileN = 16 * kWaves;  // weight rows per workgroup
constexpr int kSlab = 256;          // contraction values per slab
constexpr int kChunk = kSlab / 4;   // weights per lane per slab
constexpr int kStride = kSlab + 4;  // padded x row stride in LDS (floats)
constexpr int kDepth = 2;            // slabs the code bytes run ahead
constexpr unsigned kComputeUnits = 256;
constexpr unsigned kSlotsPerGroup = 2;  // partial tiles one workgroup may write
// Offset that the range checks always reject (every buffer is smaller).
constexpr unsigned kRejectedOffset = 0x80000000U;

// How the (tile, slab) units are dealt to the workgroups: the first
// `remainder` workgroups take quotient + 1 units, the others quotient.
struct UnitSplit {
    unsigned slabs;  // slabs per tile
    unsigned quotient;
    unsigned remainder;

    __host__ __device__ unsigned begin(unsigned group) const {
        return group * quotient + (group < remainder ? group : remainder);
    }
    __host__ __device__ unsigned owner(unsigned unit) const {
        const unsigned boundary = remainder * (quotient + 1);
        return unit < boundary ? unit / (quotient + 1)
                               : remainder + (unit - boundary) / quotient;
    }
};

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base,
                                                            std::size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// kBlocks: 16-row blocks of x (rows <= 16 * kBlocks).  kScales: block scales
// per 64-weight lane chunk (2 for block size 32, else 1).  kTwoLevel: the
// matrix instructions' sums are folded into a second accumulator after every
// slab (see `total` below).
template <int kBlocks, int kScales, bool kDoubleQuantized, bool kTwoLevel>
__global__ __launch_bounds__(kThreads) void skinny_forward_kernel(
    const float* __restrict__ x, Nf4WeightView weight,
    const float* __restrict__ bias, float* __restrict__ y,
    float* __restrict__ workspace, unsigned rows, unsigned input_width,
    unsigned output_width, unsigned block_shift, UnitSplit split,
    LoraEpilogue lora
) {
    constexpr int kRows = 16 * kBlocks;
    // float4 copies per thread to move one x tile
    constexpr int kCopies = kRows * (kSlab / 4) / kThreads;  // 2 * kBlocks
    // The table is a static array so that its LDS address is a compile-time
    // constant (zero) that folds into the lookups; the x tile is sized at
    // launch.
    __shared__ __attribute__((aligned(256))) char table[kPairTableBytes];
    extern __shared__ __attribute__((aligned(256))) char shared[];
    float* x_tile = reinterpret_cast<float*>(shared);

    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(thread / 64);
    const unsigned quarter = lane / 16;
    const unsigned group = blockIdx.x;
    const unsigned unit_begin = split.begin(group);
    const unsigned unit_count = split.begin(group + 1) - unit_begin;

    const std::size_t elements =
        static_cast<std::size_t>(output_width) * input_width;  // < 2^32
    const std::size_t block_total =
        (elements + (std::size_t{1} << block_shift) - 1) >> block_shift;
    const __amdgpu_buffer_rsrc_t x_buffer = raw_buffer(
        x, static_cast<std::size_t>(rows) * input_width * sizeof(float));
    const __amdgpu_buffer_rsrc_t code_buffer =
        raw_buffer(weight.codes, elements / 2);
    const __amdgpu_buffer_rsrc_t primary_buffer = raw_buffer(
        weight.primary_scales, block_total * (kDoubleQuantized ? 1 : 4));
    const __amdgpu_buffer_rsrc_t secondary_buffer = raw_buffer(
        weight.secondary_scales,
        kDoubleQuantized
            ? (((block_total - 1) >> weight.second_level_shift) + 1) * 4
            : 0);

    // A position on the unit axis, advanced one slab at a time with scalar
    // arithmetic only.  Positions past the workgroup's run have left == 0 and
    // make every load return zeros.
    struct Cursor {
        unsigned tile;
        unsigned slab;
        unsigned left;  // units of the run not yet passed, this one included
    };
    const auto advance = [&](Cursor& c) {
        c.slab += 1;
        if (c.slab == split.slabs) {
            c.slab = 0;
            c.tile += 1;
        }
        c.left = c.left > 0 ? c.left - 1 : 0;
    };
    Cursor compute_cursor;
    compute_cursor.tile = unit_begin / split.slabs;
    compute_cursor.slab = unit_begin - compute_cursor.tile * split.slabs;
    compute_cursor.left = unit_count;
    Cursor x_cursor = compute_cursor;
    Cursor code_cursor = compute_cursor;

    // -- x tile: global -> registers -> LDS -----------------------------------
    // Thread t moves float4 (t + 512 i) of the [kRows][64 float4] tile.
    unsigned x_source[kCopies];  // byte offset inside x for slab 0
#pragma unroll
    for (int i = 0; i < kCopies; ++i) {
        const unsigned index = thread + kThreads * i;
        const unsigned row = index / (kSlab / 4);
        const unsigned column = (index % (kSlab / 4)) * 4;
        x_source[i] = row < rows ? (row * input_width + column) *
                                       static_cast<unsigned>(sizeof(float))
                                 : kRejectedOffset;
    }
    // kThreads is a multiple of the tile's float4 columns, so a thread's
    // column is the same for all of its copies.
    const unsigned x_column = (thread % (kSlab / 4)) * 4;
    const auto load_x = [&](floatx4 (&staged)[kCopies], const Cursor& c) {
        const unsigned k0 = c.slab * kSlab;
        const bool valid = c.left > 0 && k0 + x_column < input_width;
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            // (a rejected row stays rejected: 2^31 plus a small offset)
            staged[i] = __builtin_bit_cast(
                floatx4,
                __builtin_amdgcn_raw_buffer_load_b128(
                    x_buffer,
                    valid ? x_source[i] +
                                k0 * static_cast<unsigned>(sizeof(float))
                          : kRejectedOffset,
                    0, 0));
        }
    };
    const auto store_x = [&](const floatx4 (&staged)[kCopies]) {
#pragma unroll
        for (int i = 0; i < kCopies; ++i) {
            const unsigned index = thread + kThreads * i;
            const unsigned row = index / (kSlab / 4);
            *reinterpret_cast<floatx4*>(x_tile + row * kStride + x_column) =
                staged[i];
        }
    };

    // -- weights: global -> registers -----------------------------------------
    struct Codes {
        uintx4 codes[2];  // 64 nibbles
        float scales[kScales];
    };
    const unsigned lane_row = wave * 16 + lane % 16;  // within the tile
    const auto load_codes = [&](Codes& staged, const Cursor& c) {
        const unsigned n = c.tile * kTileN + lane_row;
        const unsigned k = c.slab * kSlab + quarter * kChunk;
        const bool valid = c.left > 0 && n < output_width && k < input_width;
        const unsigned flat = n * input_width + k;
        const unsigned code_offset = valid ? flat >> 1 : kRejectedOffset;
        staged.codes[0] = __builtin_bit_cast(
            uintx4, __builtin_amdgcn_raw_buffer_load_b128(code_buffer,
                                                          code_offset, 0, 0));
        staged.codes[1] = __builtin_bit_cast(
            uintx4, __builtin_amdgcn_raw_buffer_load_b128(
                        code_buffer, code_offset + 16, 0, 0));
#pragma unroll
        for (int h = 0; h < kScales; ++h) {
            const unsigned block =
                (flat + (kChunk / kScales) * h) >> block_shift;
            if constexpr (!kDoubleQuantized) {
                staged.scales[h] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               primary_buffer,
                               valid ? block * 4 : kRejectedOffset, 0, 0));
            } else {
                const std::uint8_t scale_code =
                    __builtin_amdgcn_raw_buffer_load_b8(
                        primary_buffer, valid ? block : kRejectedOffset, 0, 0);
                const float second = __builtin_bit_cast(
                    float,
                    __builtin_amdgcn_raw_buffer_load_b32(
                        secondary_buffer,
                        valid ? (block >> weight.second_level_shift) * 4
                              : kRejectedOffset,
                        0, 0));
                // Lanes with nothing to read decode (0, 0.0) into the
                // offset: finite, and multiplied by x = 0 or never written.
                staged.scales[h] = decode_double_quantized_scale(
                    scale_code, second, weight.offset);
            }
        }
    };

    // Two-level accumulation: the matrix instructions add into `acc` for one
    // slab (64 instructions, 256 contraction values), then `acc` is folded
    // into `total`.  One fp32 chain over 7000 and more contraction values
    // drifts as far as the CPU's sequential sum (1.0-1.7e-5 of an output's
    // K-normalised scale measured on 28672 x 8192 and 16384 x 20480); chains
    // of a slab stay an order of magnitude below that (1.5-1.8e-6).  Without
    // kTwoLevel `total` is not kept (with four blocks of x its registers do
    // not fit beside the rest); the launcher asks for that only where a
    // workgroup's run of slabs is short.
    floatx4 acc[kBlocks];
    floatx4 total[kTwoLevel ? kBlocks : 1];
    const auto clear_accumulators = [&]() {
#pragma unroll
        for (int b = 0; b < kBlocks; ++b) {
            acc[b] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
            if constexpr (kTwoLevel) {
                total[b] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
            }
        }
    };
    const auto fold_accumulators = [&]() {
        if constexpr (kTwoLevel) {
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
                total[b] += acc[b];
                acc[b] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
            }
        }
    };
    // a run's sums, once its last slab has been folded
    const auto sums = [&](int b) -> const floatx4& {
        if constexpr (kTwoLevel) {
            return total[b];
        } else {
            return acc[b];
        }
    };
    clear_accumulators();

    // Where an output tile goes once its last slab of this run is done.
    // Accumulator element r of lane l in block b is x row 16 b + 4 (l / 16) + r
    // and weight row l % 16 of the wavefront.
    const auto flush = [&](unsigned tile, bool whole_tile, unsigned slot) {
        const unsigned n = tile * kTileN + lane_row;
        if (whole_tile) {
            if (n < output_width) {
                const float addend = bias != nullptr ? bias[n] : 0.0F;
#pragma unroll
                for (int b = 0; b < kBlocks; ++b) {
                    float term[4] = {0.0F, 0.0F, 0.0F, 0.0F};
                    if (lora.reduced != nullptr) {  // uniform
                        const float* reduced_rows[4];
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const unsigned m =
                                min(16U * b + 4 * quarter + r, rows - 1);
                            reduced_rows[r] =
                                lora.reduced +
                                static_cast<std::size_t>(m) * lora.rank;
                        }
                        lora_terms<4>(
                            term,
                            lora.b + static_cast<std::size_t>(n) *
                                         lora.row_stride,
                            reduced_rows, lora.rank, lora.scale,
                            lora.rank_stride);
                    }
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const unsigned m = 16 * b + 4 * quarter + r;
                        if (m < rows) {
                            y[static_cast<std::size_t>(m) * output_width + n] =
                                (sums(b)[r] + addend) + term[r];
                        }
                    }
                }
            }
        } else {
            // slot layout: [kRows][kTileN] floats
            float* target =
                workspace + static_cast<std::size_t>(slot) * kRows * kTileN;
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const unsigned m = 16 * b + 4 * quarter + r;
                    target[m * kTileN + lane_row] = sums(b)[r];
                }
            }
        }
    };

    const unsigned first_tile = compute_cursor.tile;
    unsigned segment_first_slab = compute_cursor.slab;

    floatx4 x_staged[kCopies];
    Codes ring[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
        load_codes(ring[d], code_cursor);
        advance(code_cursor);
    }
    load_x(x_staged, x_cursor);
    advance(x_cursor);

    build_pair_table<kThreads>(table);
    const unsigned lane_bits = pair_table_lane_bits(lane);

    // This lane's fragment of the x tile: row lane % 16 of each block, 64
    // consecutive values at 64 * quarter.
    const float* fragment = x_tile + (lane % 16) * kStride + quarter * kChunk;

    // The inner loop is software-pipelined by hand so that no LDS latency is
    // exposed to the matrix pipe: the table lookups of sub-chunk c + 1 and the
    // x fragment of the next (sub-chunk, block) stage are issued BEFORE the
    // matrix instructions of the current stage, and the lookups of a slab's
    // first sub-chunk are issued at the end of the previous slab.
    float2 raw[8];  // levels of the sub-chunk being looked up
    const auto issue_lookups = [&](const Codes& codes, int c) {
        const unsigned words[2] = {codes.codes[c / 2][2 * (c % 2)],
                                   codes.codes[c / 2][2 * (c % 2) + 1]};
#pragma unroll
        for (int half = 0; half < 2; ++half) {
#pragma unroll
            for (int byte = 0; byte < 4; ++byte) {
                raw[4 * half + byte] =
                    pair_table_lookup(table, words[half], byte, lane_bits);
            }
        }
    };
    const auto issue_fragment = [&](floatx4 (&a)[4], int c, int b) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            a[v] = *reinterpret_cast<const floatx4*>(
                fragment + b * 16 * kStride + 16 * c + 4 * v);
        }
    };

    __syncthreads();  // the table is built
    issue_lookups(ring[0], 0);

    for (unsigned step = 0; step < unit_count; ++step) {
        __syncthreads();  // the previous slab's fragment reads are done
        store_x(x_staged);
        __syncthreads();
        // (the previous slab's matrix instructions finished long ago: the
        // fold waits for nothing)
        fold_accumulators();
        load_x(x_staged, x_cursor);
        advance(x_cursor);

        const Codes current = ring[0];
#pragma unroll
        for (int d = 0; d + 1 < kDepth; ++d) {
            ring[d] = ring[d + 1];
        }
        load_codes(ring[kDepth - 1], code_cursor);
        advance(code_cursor);

        floatx4 a[2][4];
        issue_fragment(a[0], 0, 0);
        // Four sub-chunks of 16 contraction values, kBlocks stages each.
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float w[16];
            {
#pragma clang fp contract(off)
                const float scale = current.scales[c * kScales / 4];
#pragma unroll
                for (int p = 0; p < 8; ++p) {
                    w[2 * p] = raw[p].x * scale;
                    w[2 * p + 1] = raw[p].y * scale;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (c + 1 < 4) {
                issue_lookups(current, c + 1);
            } else {
                issue_lookups(ring[0], 0);  // the next slab's first
            }
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
                constexpr int kStages = 4 * kBlocks;
                const int stage = c * kBlocks + b;
                if (stage + 1 < kStages) {
                    issue_fragment(a[(stage + 1) % 2], (stage + 1) / kBlocks,
                                   (stage + 1) % kBlocks);
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                            a[stage % 2][v][e], w[4 * v + e], acc[b], 0, 0,
                            0);
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        // End of this run's part of the tile?
        const bool tile_done = compute_cursor.slab + 1 == split.slabs;
        if (tile_done || step + 1 == unit_count) {  // uniform
            const bool whole_tile = segment_first_slab == 0 && tile_done;
            const unsigned slot =
                group * kSlotsPerGroup +
                (compute_cursor.tile == first_tile ? 0U : 1U);
            fold_accumulators();
            flush(compute_cursor.tile, whole_tile, slot);
            clear_accumulators();
            segment_first_slab = 0;
        }
        advance(compute_cursor);
    }
}

// Adds the partial tiles of every output tile that more than one workgroup
// worked on, in ascending workgroup order, plus bias.  One thread per output
// element: blockIdx.x is the tile, blockIdx.y a slab of 256 elements of it.
template <int kBlocks>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(
    const float* __restrict__ workspace, const float* __restrict__ bias,
    float* __restrict__ y, unsigned rows, unsigned output_width,
    UnitSplit split, LoraEpilogue lora
) {
    constexpr int kRows = 16 * kBlocks;
    constexpr int kBatch = 8;  // partial tiles fetched together
    const unsigned tile = blockIdx.x;
    const unsigned first_unit = tile * split.slabs;
    const unsigned first_group = split.owner(first_unit);
    const unsigned last_group = split.owner(first_unit + split.slabs - 1);
    if (first_group == last_group) {
        return;  // written directly by its only workgroup
    }
    const unsigned index = blockIdx.y * blockDim.x + threadIdx.x;
    const unsigned m = index / kTileN;
    const unsigned column = index % kTileN;
    const unsigned n = tile * kTileN + column;
    if (m >= rows || n >= output_width) {
        return;
    }
    const float* source = workspace + m * kTileN + column;
    float sum = 0.0F;
    for (unsigned group = first_group; group <= last_group; group += kBatch) {
        float part[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            const unsigned g = group + j;
            // A workgroup's slot 0 holds the first tile of its run.
            const unsigned slot =
                g * kSlotsPerGroup +
                (tile == split.begin(g) / split.slabs ? 0U : 1U);
            part[j] = g <= last_group
                          ? source[static_cast<std::size_t>(slot) * kRows *
                                   kTileN]
                          : 0.0F;
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
            sum += part[j];  // ascending workgroup order
        }
    }
    if (bias != nullptr) {
        sum += bias[n];
    }
    if (lora.reduced != nullptr) {
        sum += lora_term(lora, m, n);
    }
    y[static_cast<std::size_t>(m) * output_width + n] = sum;
}

// Partial tiles of the largest case: two slots of [64][128] floats per
// workgroup.
constexpr std::size_t kWorkspaceBytes =
    static_cast<std::size_t>(kComputeUnits) * kSlotsPerGroup * 64 * kTileN *
    sizeof(float);
static_assert(kWorkspaceBytes <= kStreamWorkspaceBytes);

// Slabs a workgroup may chain in ONE accumulator (1536 contraction values:
// rounding stays below 5e-6 of an output's scale; runs of 8 slabs measured
// 6.0e-6 on 5000 x 12352, runs of 13.5 slabs 7.6e-6).
constexpr unsigned kSingleChainSlabs = 6;

// The split of (tile, slab) units over the workgroups.
struct LaunchSplit {
    UnitSplit split;
    unsigned tiles;
    unsigned groups;
};
LaunchSplit split_units(const LinearProblem& p) {
    LaunchSplit launch;
    launch.tiles =
        static_cast<unsigned>((p.output_width + kTileN - 1) / kTileN);
    launch.split.slabs =
        static_cast<unsigned>((p.input_width + kSlab - 1) / kSlab);
    const unsigned units = launch.tiles * launch.split.slabs;
    // One workgroup per compute unit; with at least that many tiles, one
    // workgroup per tile (no partial tiles at all).
    launch.groups =
        launch.tiles >= kComputeUnits
            ? launch.tiles
            : (units < kComputeUnits ? units : kComputeUnits);
    launch.split.quotient = units / launch.groups;
    launch.split.remainder = units % launch.groups;
    return launch;
}

template <int kBlocks, int kScales, bool kDoubleQuantized, bool kTwoLevel>
hipError_t launch_instance(const LinearProblem& p, hipStream_t stream) {
    constexpr std::size_t kSharedBytes =
        static_cast<std::size_t>(16 * kBlocks) * kStride * sizeof(float);
    const auto kernel =
        skinny_forward_kernel<kBlocks, kScales, kDoubleQuantized, kTwoLevel>;
    // More than the default 64 KB of LDS.
    static std::atomic<std::uint64_t> served{0};
    if (const hipError_t error = allow_dynamic_lds(
            reinterpret_cast<const void*>(kernel), kSharedBytes, served);
        error != hipSuccess) {
        return error;
    }
    const LaunchSplit launch = split_units(p);
    const UnitSplit& split = launch.split;
    const unsigned tiles = launch.tiles;
    const unsigned groups = launch.groups;
    const bool partial_tiles = groups != tiles;
    WorkspaceLease lease;  // held until both launches are enqueued
    if (partial_tiles) {
        const hipError_t status = lease_stream_workspace(stream, &lease);
        if (status != hipSuccess) {
            return status;
        }
    }
    float* const workspace = lease.data();
    kernel<<<groups, kThreads, kSharedBytes, stream>>>(
        p.activations, p.weight, p.bias, p.result, workspace,
        static_cast<unsigned>(p.rows), static_cast<unsigned>(p.input_width),
        static_cast<unsigned>(p.output_width), p.block_shift, split, p.lora);
    if (partial_tiles) {
        const dim3 reduce_grid(
            tiles, static_cast<unsigned>((p.rows * kTileN + 255) / 256));
        skinny_reduce_kernel<kBlocks><<<reduce_grid, 256, 0, stream>>>(
            workspace, p.bias, p.result, static_cast<unsigned>(p.rows),
            static_cast<unsigned>(p.output_width), split, p.lora);
    }
    return hipSuccess;
}

template <int kBlocks, bool kTwoLevel>
hipError_t launch_encoding(const LinearProblem& p, hipStream_t stream) {
    const bool two_scales = p.block_shift == 5;  // block size 32
    if (p.weight.encoding == 0) {
        return two_scales
                   ? launch_instance<kBlocks, 2, false, kTwoLevel>(p, stream)
                   : launch_instance<kBlocks, 1, false, kTwoLevel>(p, stream);
    }
    return two_scales
               ? launch_instance<kBlocks, 2, true, kTwoLevel>(p, stream)
               : launch_instance<kBlocks, 1, true, kTwoLevel>(p, stream);
}

template <int kBlocks>
hipError_t launch_blocks(const LinearProblem& p, hipStream_t stream) {
    if constexpr (kBlocks == 4) {
        // the second accumulator costs four blocks of x spilled registers
        // (4096 x 11008 at 64 rows: 64.5 -> 69.4 us): kept for long runs only
        const LaunchSplit launch = split_units(p);
        const unsigned longest_run =
            std::min(launch.split.quotient + 1, launch.split.slabs);
        if (longest_run <= kSingleChainSlabs) {
            return launch_encoding<4, false>(p, stream);
        }
    }
    return launch_encoding<kBlocks, true>(p, stream);
}

}  // namespace

bool skinny_forward_supports(const LinearProblem& p) {
    return p.rows >= 1 && p.rows <= kSkinnyMaxRows &&
           // a lane's 64-weight chunk never straddles a row end, and lies in
           // one quantisation block (two for block size 32)
           p.input_width % kChunk == 0 &&
           // 32-bit flat weight indices; byte offsets into x, the codes and
           // the scales all stay below the rejected offset
           p.output_width * p.input_width < (1ULL << 32) &&
           p.rows * p.input_width * sizeof(float) < kRejectedOffset &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 16 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

hipError_t launch_skinny_forward(const LinearProblem& p, hipStream_t stream) {
    const std::size_t blocks = (p.rows + 15) / 16;
    switch (blocks) {
    case 1: return launch_blocks<1>(p, stream);
    case 2: return launch_blocks<2>(p, stream);
    case 3: return launch_blocks<3>(p, stream);
    default: return launch_blocks<4>(p, stream);
    }
}

}  // namespace rthip
