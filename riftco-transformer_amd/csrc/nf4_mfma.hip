// LDS-tiled fp32 MFMA GEMM with NF4 dequantisation fused into the tile load,
// for prefill / training row counts.  Two products over the same packed
// weight W [output_width, input_width]:
//
//   forward         y [M, O] = x  [M, I] * deq(W)^T     (contract over I)
//   input backward  dx[M, I] = dy [M, O] * deq(W)       (contract over O)
//
// restating reference_quantized_linear_forward / _input_backward
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-115).
// The fp32 weight never exists in HBM: packed nibbles and block scales are
// read straight from global memory (buffer loads: a lane's offset is fixed for
// a whole tile, the step is a scalar offset), decoded in registers
// (codebook[code] * scale, one rounded multiply) and written to the LDS tile
// the matrix cores read.
//
// Tiling.  A workgroup of four wavefronts computes a 128 x 128 output tile in
// steps of 32 along the contraction (or eight wavefronts a 256 x 128 tile,
// see Tile); each wavefront owns a 64 x 64 part as 2 x 2 blocks of
// v_mfma_f32_32x32x2_f32.  Both LDS tiles are laid out
// [row-or-column][contraction] with a padded stride of 36 floats, so that one
// ds_read_b128 per lane fetches four consecutive contraction values; lanes
// 0-31 take offsets 0..3 and lanes 32-63 offsets 4..7 of each group of eight,
// which the four MFMAs of the group consume as (k, k+4) pairs -- any pairing is
// valid because both operands use the same one.  There are two such pairs of
// tiles: step t multiplies from one pair, writes the tiles of step t + 1 --
// whose operands are in registers by then -- into the other between its two
// halves of matrix instructions, and then requests the operands of step t + 2
// into the freed registers, so a step has one barrier and its loads have a
// whole step to arrive.
//
// Work split.  Output tiles are dealt to workgroups whole while they fill the
// device evenly (two workgroups per compute unit).  What is left over -- 1376
// tiles on 512 places leave 352 -- would occupy the device for a whole further
// round at 69 % occupancy, so those tiles are cut along the contraction
// instead: their (tile, step) units are dealt in equal contiguous runs to as
// many workgroups as there are places, a workgroup whose run covers a whole
// tile writes it as usual, the others write partial tiles to the stream's
// workspace and a second kernel adds the parts of each tile in ascending
// workgroup order (plus bias).  Nothing depends on timing.
//
// A low-rank adapter's term, s * (x A^T) . B^T, is not an epilogue: after a
// tile's last step its rows of x A^T and its columns of B pass through the
// same LDS tiles and the same matrix instructions, 32 of the rank at a time.
//
// The two directions share everything except the weight-tile loader: forward
// reads 128 weight rows x 32 contiguous columns, backward reads 32 weight rows
// (the contraction) x 128 contiguous columns and transposes while writing LDS.

#include "gemv_shared.hpp"
#include "kernels.hpp"
#include "launch_config.hpp"
#include "nf4_decode.hpp"
#include "tile_plan.hpp"

#include <algorithm>

namespace rthip {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned uintx2 __attribute__((ext_vector_type(2)));

constexpr int kTileN = 128;       // output columns per workgroup
constexpr int kTileK = 32;        // contraction per step
constexpr int kStride = 36;       // padded LDS row stride in floats
constexpr unsigned kFlushSteps = 8;  // steps per first-level accumulation

// The two tile shapes.  Tall: 256 output rows per workgroup of eight
// wavefronts, one workgroup per compute unit -- a weight tile is decoded once
// per 256 rows of x.  Otherwise 128 rows per workgroup of four wavefronts, two
// workgroups per compute unit.  A wavefront owns 64 x 64 in both.
template <bool kTall>
struct Tile {
    static constexpr int kThreads = kTall ? 512 : 256;
    static constexpr int kTileM = kTall ? 256 : 128;  // output rows
    // weights decoded per thread per step (the 128 x 32 weight tile over the
    // workgroup's threads), and the 32-bit words of codes they come in
    static constexpr int kChunk = kTileN * kTileK / kThreads;
    static constexpr int kWords = kChunk / 8;
    static constexpr int kWorkgroupsPerUnit = kTall ? 1 : 2;
    // workgroups the device holds at once
    static constexpr unsigned kPlaces = kTall ? 256 : 512;
    static constexpr unsigned kActivationFloats = kTileM * kStride;
    static constexpr unsigned kBufferFloats = (kTileM + kTileN) * kStride;
    // LDS of a workgroup: two buffers x (activation tile + weight tile)
    static constexpr std::size_t kTileBytes =
        std::size_t{2} * kBufferFloats * sizeof(float);
};

struct GemmShape {
    unsigned rows;         // M
    unsigned contraction;  // I (forward) or O (backward)
    unsigned columns;      // O (forward) or I (backward)
    unsigned input_width;  // I: the weight's row length
};


// Registers holding one step's global loads of a thread.
template <bool kTall>
struct Staged {
    float4 a[4];
    unsigned codes[Tile<kTall>::kWords];
    // fp32 scales: the block scale; nested: the second-level scale, with the
    // block's scale code beside it (decoded when the tile is written)
    float scale;
    unsigned scale_code;
};

template <bool kTall>
__device__ __forceinline__ void store_activation_tile(
    const Staged<kTall>& staged, float* __restrict__ tile
) {
    const unsigned thread = threadIdx.x;
    const unsigned column = (thread % 8) * 4;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const unsigned row = thread / 8 + (Tile<kTall>::kThreads / 8) * pass;
        *reinterpret_cast<float4*>(tile + row * kStride + column) =
            staged.a[pass];
    }
}

template <bool kTall>
__device__ __forceinline__ void decode_chunk(
    const Staged<kTall>& staged, const float* __restrict__ table, float scale,
    float (&out)[Tile<kTall>::kChunk]
) {
#pragma clang fp contract(off)
#pragma unroll
    for (int w = 0; w < Tile<kTall>::kWords; ++w) {
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            out[8 * w + n] =
                table[(staged.codes[w] >> (4 * n)) & 0xFU] * scale;
        }
    }
}

// table: the sixteen levels, followed for nested scales by the 256 factors
// (code - 128) / 127.
template <bool kTall, bool kDoubleQuantized, bool kBackward>
__device__ __forceinline__ void store_weight_tile(
    const Staged<kTall>& staged, const float* __restrict__ table, float offset,
    float* __restrict__ tile
) {
    constexpr unsigned kChunk = Tile<kTall>::kChunk;
    constexpr unsigned kPerRow = kTileK / kChunk;
    const unsigned thread = threadIdx.x;
    float decoded[kChunk];
    float scale = staged.scale;
    if constexpr (kDoubleQuantized) {
        scale = double_quantized_scale_from_factor(
            table[16 + staged.scale_code], staged.scale, offset);
    }
    decode_chunk<kTall>(staged, table, scale, decoded);
    if constexpr (!kBackward) {
        float* destination =
            tile + (thread / kPerRow) * kStride + (thread % kPerRow) * kChunk;
#pragma unroll
        for (int q = 0; q < static_cast<int>(kChunk) / 4; ++q) {
            *reinterpret_cast<float4*>(destination + 4 * q) = make_float4(
                decoded[4 * q], decoded[4 * q + 1], decoded[4 * q + 2],
                decoded[4 * q + 3]);
        }
    } else {
        // tile[column][contraction]: transpose while writing.
        float* destination =
            tile + ((thread / 32) * kChunk) * kStride + thread % 32;
#pragma unroll
        for (int i = 0; i < static_cast<int>(kChunk); ++i) {
            destination[i * kStride] = decoded[i];
        }
    }
}

// One segment: contraction values [k_begin, k_end) of the output tile at
// (row0, col0).  `partial` null: the segment is the whole contraction and the
// tile goes to `result` with bias; otherwise the tile's partial sums go to
// `partial`.  The segment that starts at 0 includes the adapter term.
template <bool kTall, bool kDoubleQuantized, bool kBackward>
__device__ __forceinline__ void gemm_segment(
    const float* __restrict__ activations, const Nf4WeightView& weight,
    const float* __restrict__ bias, float* __restrict__ result,
    float* __restrict__ partial, const GemmShape& shape, unsigned block_shift,
    const LoraEpilogue& lora, float* __restrict__ tiles,
    const float* __restrict__ table, unsigned row0, unsigned col0,
    unsigned k_begin, unsigned k_end
) {
    const unsigned thread = threadIdx.x;
    const unsigned lane = thread % 64;
    const unsigned wave = thread / 64;
    const unsigned wave_m = wave / 2;
    const unsigned wave_n = wave % 2;
    // tiles: [buffer][activations | weights][row or column][k], two buffers.
    // A step computes from one buffer while the next step's tiles are written
    // into the other, so the writes need no barrier of their own.
    constexpr unsigned kTileFloats = Tile<kTall>::kActivationFloats;
    constexpr unsigned kBufferFloats = Tile<kTall>::kBufferFloats;
    const unsigned a_offset =
        (wave_m * 64 + lane % 32) * kStride + 4 * (lane / 32);
    const unsigned b_offset = kTileFloats +
        (wave_n * 64 + lane % 32) * kStride + 4 * (lane / 32);

    // Two-level accumulation: the matrix cores add into `acc` for
    // kFlushSteps steps (256 contraction values), then `acc` is folded into
    // `total` and cleared.  One long fp32 chain over K = 11008 drifts about as
    // far as the CPU's sequential sum (~1e-5 of an output's standard
    // deviation); chains of 256 stay an order of magnitude below that.
    floatx16 acc[2][2];
    floatx16 total[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0.0F;
                total[i][j][e] = 0.0F;
            }
        }
    }
    unsigned steps_since_flush = 0;

    // Every load of a step is a buffer load whose per-lane offset is fixed for
    // the whole segment and whose scalar offset advances with the step: no
    // vector address arithmetic in the loop, and what lies outside -- rows of
    // the activations past the last one, weight rows or columns past the
    // weight -- is past a descriptor's extent (or carries an offset that is),
    // where the hardware returns zeros: nothing branches on bounds.  (Garbage
    // in columns past the output width is never stored.)
    constexpr unsigned kTileRows = Tile<kTall>::kTileM;
    constexpr unsigned kChunk = Tile<kTall>::kChunk;
    constexpr unsigned kOutside = 0xFFFFFFFFU;
    const unsigned tile_rows = min(shape.rows - row0, kTileRows);
    const __amdgpu_buffer_rsrc_t a_buffer = make_buffer(
        activations + static_cast<std::size_t>(row0) * shape.contraction,
        static_cast<std::size_t>(tile_rows) * shape.contraction *
            sizeof(float));
    unsigned a_lane[4];
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const unsigned row = thread / 8 + (Tile<kTall>::kThreads / 8) * pass;
        a_lane[pass] = static_cast<unsigned>(
            (row * shape.contraction + (thread % 8) * 4) * sizeof(float));
    }
    const unsigned weights = shape.input_width *
        (kBackward ? shape.contraction : shape.columns);
    const unsigned block_count = ((weights - 1U) >> block_shift) + 1U;
    const __amdgpu_buffer_rsrc_t code_buffer =
        make_buffer(weight.codes, weights / 2);
    const __amdgpu_buffer_rsrc_t primary_buffer = make_buffer(
        weight.primary_scales,
        kDoubleQuantized ? block_count : block_count * sizeof(float));
    const __amdgpu_buffer_rsrc_t secondary_buffer = make_buffer(
        weight.secondary_scales,
        kDoubleQuantized
            ? (((block_count - 1U) >> weight.second_level_shift) + 1U) *
                  sizeof(float)
            : 0);
    // the thread's chunk at step 0 of the weight: its flat index, or nothing
    unsigned chunk_flat;
    bool chunk_inside;
    if constexpr (!kBackward) {
        constexpr unsigned kPerRow = kTileK / kChunk;
        const unsigned n = col0 + thread / kPerRow;
        chunk_inside = n < shape.columns;
        chunk_flat = n * shape.input_width + (thread % kPerRow) * kChunk;
    } else {
        const unsigned column = col0 + (thread / 32) * kChunk;
        chunk_inside = column < shape.columns;
        chunk_flat = (thread % 32) * shape.input_width + column;
    }
    const unsigned code_lane = chunk_inside ? chunk_flat / 2 : kOutside;

    Staged<kTall> staged;
    const auto load_step = [&](unsigned k) {
        // scalar: where the step starts in x (bytes) and in the weight (flat)
        const unsigned a_step = k * static_cast<unsigned>(sizeof(float));
        const unsigned weight_step = kBackward ? k * shape.input_width : k;
#pragma unroll
        for (int pass = 0; pass < 4; ++pass) {
            const floatx4 loaded = __builtin_bit_cast(
                floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                             a_buffer, a_lane[pass], a_step, 0));
            staged.a[pass] =
                make_float4(loaded.x, loaded.y, loaded.z, loaded.w);
        }
        if constexpr (Tile<kTall>::kWords == 2) {
            const uintx2 both = __builtin_bit_cast(
                uintx2, __builtin_amdgcn_raw_buffer_load_b64(
                            code_buffer, code_lane, weight_step / 2, 0));
            staged.codes[0] = both.x;
            staged.codes[1] = both.y;
        } else {
            staged.codes[0] = __builtin_amdgcn_raw_buffer_load_b32(
                code_buffer, code_lane, weight_step / 2, 0);
        }
        const unsigned block = chunk_inside
            ? (chunk_flat + weight_step) >> block_shift
            : kOutside / 4;
        if constexpr (kDoubleQuantized) {
            staged.scale_code = __builtin_amdgcn_raw_buffer_load_b8(
                primary_buffer, block, 0, 0);
            staged.scale = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(
                           secondary_buffer,
                           (block >> weight.second_level_shift) * 4, 0, 0));
        } else {
            staged.scale = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(
                           primary_buffer, block * 4, 0, 0));
        }
    };
    const auto store_step = [&](unsigned buffer) {
        float* const target = tiles + buffer * kBufferFloats;
        store_activation_tile<kTall>(staged, target);
        store_weight_tile<kTall, kDoubleQuantized, kBackward>(
            staged, table, weight.offset, target + kTileFloats);
    };
    // Matrix instructions of contraction values [kk, kk + 8) of the step.
    const auto multiply = [&](const float* a_fragment,
                              const float* b_fragment, int kk) {
        float4 a[2];
        float4 b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            a[i] = *reinterpret_cast<const float4*>(
                a_fragment + i * 32 * kStride + kk);
            b[i] = *reinterpret_cast<const float4*>(
                b_fragment + i * 32 * kStride + kk);
        }
        const float a_values[2][4] = {{a[0].x, a[0].y, a[0].z, a[0].w},
                                      {a[1].x, a[1].y, a[1].z, a[1].w}};
        const float b_values[2][4] = {{b[0].x, b[0].y, b[0].z, b[0].w},
                                      {b[1].x, b[1].y, b[1].z, b[1].w}};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                        a_values[i][s], b_values[j][s], acc[i][j], 0, 0, 0);
                }
            }
        }
    };

    load_step(k_begin);
    __syncthreads();  // nobody still reads the tiles of an earlier segment
    store_step(0);
    if (k_begin + kTileK < k_end) {
        load_step(k_begin + kTileK);
    }
    __syncthreads();

    unsigned buffer = 0;
    for (unsigned k0 = k_begin; k0 < k_end; k0 += kTileK) {
        const float* const a_fragment =
            tiles + buffer * kBufferFloats + a_offset;
        const float* const b_fragment =
            tiles + buffer * kBufferFloats + b_offset;
        // (the wavefront is given priority while it issues matrix
        // instructions: the other workgroup's wavefront on the SIMD is then
        // the one that waits with its decode and tile writes; 0.3-0.9 %)
        __builtin_amdgcn_s_setprio(1);
        multiply(a_fragment, b_fragment, 0);
        multiply(a_fragment, b_fragment, 8);
        __builtin_amdgcn_s_setprio(0);

        // The next step's tiles go into the other buffer while this step's
        // matrix instructions run, and once the staging registers are free
        // they take the loads of the step after that, which then have a
        // whole step to arrive.
        const unsigned next = k0 + kTileK;
        if (next < k_end) {  // uniform
            store_step(buffer ^ 1U);
            if (next + kTileK < k_end) {
                load_step(next + kTileK);
            }
        }

        __builtin_amdgcn_s_setprio(1);
        multiply(a_fragment, b_fragment, 16);
        multiply(a_fragment, b_fragment, 24);
        __builtin_amdgcn_s_setprio(0);

        if (++steps_since_flush == kFlushSteps) {
            steps_since_flush = 0;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int j = 0; j < 2; ++j) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        total[i][j][e] += acc[i][j][e];
                        acc[i][j][e] = 0.0F;
                    }
                }
            }
        }
        // One barrier per step: the other buffer is complete, and this one
        // may be overwritten.
        __syncthreads();
        buffer ^= 1U;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                total[i][j][e] += acc[i][j][e];
            }
        }
    }

    // The adapter term is a few more, short, steps on the matrix cores: the
    // tile's rows of `reduced` take the place of the activation tile, the
    // tile's columns of the second factor that of the weight tile, 32 of the
    // rank at a time (contraction values past the rank are zeros); the
    // products land in `acc`, which the fold above has left free, and are
    // folded into `total` times the adapter's scale.  The segment that starts
    // the contraction carries the term, so a tile whose steps are shared
    // between workgroups gets it exactly once.
    if (lora.reduced != nullptr && k_begin == 0) {  // uniform
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    acc[i][j][e] = 0.0F;
                }
            }
        }
        float* const reduced_tile = tiles;
        float* const factor_tile = tiles + kTileFloats;
        for (unsigned first = 0; first < lora.rank;
             first += static_cast<unsigned>(kTileK)) {
            const unsigned count =
                min(lora.rank - first, static_cast<unsigned>(kTileK));
            const unsigned padded = (count + 7U) & ~7U;
            if (first != 0) {
                __syncthreads();  // the tiles of the 32 before have been read
            }
            // (every wavefront is past the last step's barrier: buffer 0 is
            // free)
            for (unsigned index = thread; index < kTileRows * padded;
                 index += Tile<kTall>::kThreads) {
                const unsigned r = index / padded;
                const unsigned j = index % padded;
                float value = 0.0F;
                if (row0 + r < shape.rows && j < count) {
                    value = lora.reduced[static_cast<std::size_t>(row0 + r) *
                                             lora.rank +
                                         first + j];
                }
                reduced_tile[r * kStride + j] = value;
            }
            for (unsigned index = thread; index < kTileN * padded;
                 index += Tile<kTall>::kThreads) {
                const unsigned c = index / padded;
                const unsigned j = index % padded;
                float value = 0.0F;
                if (col0 + c < shape.columns && j < count) {
                    value =
                        lora.b[static_cast<std::size_t>(col0 + c) *
                                   lora.row_stride +
                               static_cast<std::size_t>(first + j) *
                                   lora.rank_stride];
                }
                factor_tile[c * kStride + j] = value;
            }
            __syncthreads();
#pragma unroll
            for (int kk = 0; kk < static_cast<int>(kTileK); kk += 8) {
                if (static_cast<unsigned>(kk) < padded) {  // uniform
                    multiply(tiles + a_offset, tiles + b_offset, kk);
                }
            }
        }
        // (a following segment of this workgroup meets a barrier before it
        // writes the tiles)
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    total[i][j][e] += lora.scale * acc[i][j][e];
                }
            }
        }
    }

    // Accumulator element e of lane l is output row 8*(e/4) + 4*(l/32) + e%4,
    // column l%32 of its 32 x 32 block.
    if (partial != nullptr) {  // uniform; layout [tile rows][kTileN]
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const unsigned column = wave_n * 64 + j * 32 + lane % 32;
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const unsigned row = wave_m * 64 + i * 32 + 8 * (e / 4) +
                                         4 * (lane / 32) + e % 4;
                    partial[row * kTileN + column] = total[i][j][e];
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const unsigned column = col0 + wave_n * 64 + j * 32 + lane % 32;
            if (column >= shape.columns) {
                continue;
            }
            float addend = 0.0F;
            if constexpr (!kBackward) {
                if (bias != nullptr) {
                    addend = bias[column];
                }
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const unsigned row = row0 + wave_m * 64 + i * 32 +
                                     8 * (e / 4) + 4 * (lane / 32) + e % 4;
                if (row < shape.rows) {
                    result[static_cast<std::size_t>(row) * shape.columns +
                           column] = total[i][j][e] + addend;
                }
            }
        }
    }
}

template <bool kTall, bool kDoubleQuantized, bool kBackward>
__global__ __launch_bounds__(Tile<kTall>::kThreads,
                             Tile<kTall>::kWorkgroupsPerUnit)
void mfma_gemm_kernel(
    const float* __restrict__ activations, Nf4WeightView weight,
    const float* __restrict__ bias, float* __restrict__ result,
    float* __restrict__ workspace, GemmShape shape, TilePlan plan,
    unsigned block_shift, LoraEpilogue lora
) {
    constexpr unsigned kTileM = Tile<kTall>::kTileM;
    // two buffers of an activation and a weight tile each: more than the 64
    // KB a static array may have, so sized at launch
    extern __shared__ __attribute__((aligned(16))) float tiles[];
    __shared__ float table[kDoubleQuantized ? 16 + 256 : 16];
    load_codebook_to_lds(table);
    if constexpr (kDoubleQuantized) {
        if (threadIdx.x < 256) {
            // the division of decode_double_quantized_scale, once per code
            table[16 + threadIdx.x] =
                static_cast<float>(static_cast<int>(threadIdx.x) - 128) /
                127.0F;
        }
    }

    // A whole tile, or a run of (tile, step) units: one or two segments,
    // each inside one tile.
    const bool whole = blockIdx.x < plan.whole_tiles;
    const unsigned group = whole ? 0U : blockIdx.x - plan.whole_tiles;
    const unsigned first_tile = whole ? blockIdx.x : plan.whole_tiles;
    unsigned unit = whole ? 0U : plan.begin(group);
    const unsigned unit_end = whole ? plan.steps : plan.begin(group + 1);
    for (unsigned segment = 0; unit < unit_end; ++segment) {
        const unsigned tile_in_run = unit / plan.steps;
        const unsigned first_step = unit - tile_in_run * plan.steps;
        const unsigned segment_steps =
            min(unit_end - unit, plan.steps - first_step);
        const unsigned tile = first_tile + tile_in_run;
        float* const partial =
            segment_steps == plan.steps
                ? nullptr
                : workspace +
                      static_cast<std::size_t>(group * 2 + segment) * kTileM *
                          kTileN;
        gemm_segment<kTall, kDoubleQuantized, kBackward>(
            activations, weight, bias, result, partial, shape, block_shift,
            lora, tiles, table, plan.tile_row(tile) * kTileM,
            plan.tile_column(tile) * kTileN, first_step * kTileK,
            (first_step + segment_steps) * kTileK);
        unit += segment_steps;
    }
}

// Adds the parts of every unit-dealt tile that more than one workgroup worked
// on, in ascending workgroup order, plus bias (the adapter term is in the
// part that starts the contraction).  One thread
// per output element: blockIdx.x is the tile among the unit-dealt ones,
// blockIdx.y a run of 256 elements of it.
template <unsigned kTileM>
__global__ __launch_bounds__(256) void gemm_parts_kernel(
    const float* __restrict__ workspace, const float* __restrict__ bias,
    float* __restrict__ result, GemmShape shape, TilePlan plan
) {
    const unsigned dealt_tile = blockIdx.x;
    const unsigned first_unit = dealt_tile * plan.steps;
    const unsigned first_group = plan.owner(first_unit);
    const unsigned last_group = plan.owner(first_unit + plan.steps - 1);
    if (first_group == last_group) {
        return;  // written directly by its only workgroup
    }
    const unsigned tile = plan.whole_tiles + dealt_tile;
    const unsigned index = blockIdx.y * blockDim.x + threadIdx.x;
    const unsigned m = index / kTileN;
    const unsigned c = index % kTileN;
    const unsigned row = plan.tile_row(tile) * kTileM + m;
    const unsigned column = plan.tile_column(tile) * kTileN + c;
    if (row >= shape.rows || column >= shape.columns) {
        return;
    }
    const float* source = workspace + m * kTileN + c;
    float sum = 0.0F;
    for (unsigned group = first_group; group <= last_group; ++group) {
        sum += source[static_cast<std::size_t>(plan.slot(group, dealt_tile)) *
                      kTileM * kTileN];
    }
    if (bias != nullptr) {
        sum += bias[column];
    }
    result[static_cast<std::size_t>(row) * shape.columns + column] = sum;
}

// Tile columns [first_tile_n, first_tile_n + tiles_n) of the output.
template <bool kTall, bool kDoubleQuantized, bool kBackward>
hipError_t launch_tiles(const LinearProblem& p, const GemmShape& shape,
                        unsigned first_tile_n, unsigned tiles_n,
                        hipStream_t stream) {
    constexpr unsigned kTileM = Tile<kTall>::kTileM;
    constexpr unsigned kThreads = Tile<kTall>::kThreads;
    constexpr std::size_t kTileBytes = Tile<kTall>::kTileBytes;
    const auto kernel = mfma_gemm_kernel<kTall, kDoubleQuantized, kBackward>;
    const unsigned tiles_m = (shape.rows + kTileM - 1) / kTileM;
    const unsigned tiles = tiles_m * tiles_n;
    TilePlan plan;
    plan.tiles_n = tiles_n;
    plan.first_tile_n = first_tile_n;
    plan.steps = (shape.contraction + kTileK - 1) / kTileK;
    const unsigned groups =
        plan_tiles(plan, tiles, kTileM * kTileN * sizeof(float),
                   kStreamWorkspaceBytes, Tile<kTall>::kPlaces);
    WorkspaceLease lease;  // held until both launches are enqueued
    if (groups != 0) {
        if (const hipError_t status = lease_stream_workspace(stream, &lease);
            status != hipSuccess) {
            return status;
        }
    }
    float* const workspace = lease.data();
    static std::atomic<std::uint64_t> served{0};
    if (const hipError_t error = allow_dynamic_lds(
            reinterpret_cast<const void*>(kernel), kTileBytes, served);
        error != hipSuccess) {
        return error;
    }
    kernel<<<plan.whole_tiles + groups, kThreads, kTileBytes, stream>>>(
        p.activations, p.weight, p.bias, p.result, workspace, shape, plan,
        p.block_shift, p.lora);
    if (groups != 0) {
        const dim3 grid(tiles - plan.whole_tiles, kTileM * kTileN / 256);
        gemm_parts_kernel<kTileM><<<grid, 256, 0, stream>>>(
            workspace, p.bias, p.result, shape, plan);
    }
    return hipSuccess;
}

// The tall tile halves the decode work per product but leaves a compute unit
// one workgroup, whose barriers nothing covers.  Measured at 2048 rows: the
// forward wins where its tiles fill the device in whole rounds (4096 x 4096:
// 123-124 -> 127-128 TFLOP/s) and is level where leftover tiles are dealt in
// runs (all of 11008 x 4096 in tall tiles); the input backward, whose weight
// tile is written transposed word by word, loses (W 11008 x 4096: 119 ->
// 116).  So: forward, whole rounds -- and an output whose tile columns do not
// come out in whole rounds is cut in two launches: as many tile columns as
// fill whole rounds in tall tiles, the rest in square ones.
//
// Returns the number of leading tile columns that tall tiles take.
unsigned tall_tile_columns(const GemmShape& shape) {
    constexpr unsigned kTallRows = Tile<true>::kTileM;
    constexpr unsigned kPlaces = Tile<true>::kPlaces;
    if (shape.rows < kTallRows) {
        return 0;
    }
    const unsigned tiles_m = (shape.rows + kTallRows - 1) / kTallRows;
    const unsigned last_row_fill = shape.rows - (tiles_m - 1) * kTallRows;
    if (last_row_fill <= kTallRows / 2) {
        return 0;
    }
    // tile columns per whole round: the least n with tiles_m * n a multiple
    // of the places
    unsigned common = tiles_m;
    for (unsigned other = kPlaces; other != 0;) {
        const unsigned rest = common % other;
        common = other;
        other = rest;
    }
    const unsigned period = kPlaces / common;
    const unsigned tiles_n = (shape.columns + kTileN - 1) / kTileN;
    const unsigned tall = tiles_n / period * period;
    // a second launch is worth it when tall tiles take at least half
    return tall * 2 >= tiles_n ? tall : 0;
}

template <bool kDoubleQuantized, bool kBackward>
hipError_t launch_encoding(const LinearProblem& p, const GemmShape& shape,
                           hipStream_t stream) {
    const unsigned tiles_n = (shape.columns + kTileN - 1) / kTileN;
    if constexpr (!kBackward) {
        const unsigned tall = tall_tile_columns(shape);
        if (tall != 0) {
            if (const hipError_t status =
                    launch_tiles<true, kDoubleQuantized, false>(p, shape, 0,
                                                                tall, stream);
                status != hipSuccess || tall == tiles_n) {
                return status;
            }
            return launch_tiles<false, kDoubleQuantized, false>(
                p, shape, tall, tiles_n - tall, stream);
        }
    }
    return launch_tiles<false, kDoubleQuantized, kBackward>(p, shape, 0,
                                                            tiles_n, stream);
}

template <bool kBackward>
hipError_t launch(const LinearProblem& p, hipStream_t stream) {
    GemmShape shape;
    shape.rows = static_cast<unsigned>(p.rows);
    shape.input_width = static_cast<unsigned>(p.input_width);
    if constexpr (!kBackward) {
        shape.contraction = static_cast<unsigned>(p.input_width);
        shape.columns = static_cast<unsigned>(p.output_width);
    } else {
        shape.contraction = static_cast<unsigned>(p.output_width);
        shape.columns = static_cast<unsigned>(p.input_width);
    }
    return p.weight.encoding == 0
               ? launch_encoding<false, kBackward>(p, shape, stream)
               : launch_encoding<true, kBackward>(p, shape, stream);
}

bool common_supports(const LinearProblem& p) {
    constexpr std::size_t kLimit = 1ULL << 31;
    return p.rows >= 1 && p.rows < kLimit && p.input_width < kLimit &&
           p.output_width < kLimit &&
           // tile and (tile, step) unit counts stay 32-bit
           ((p.rows + Tile<false>::kTileM - 1) / Tile<false>::kTileM) *
                   ((std::max(p.input_width, p.output_width) + kTileN - 1) /
                    kTileN) <
               (1ULL << 24) &&
           // 32-bit flat weight indices and byte offsets inside a tile's rows
           // of the activations (buffer loads)
           p.output_width * p.input_width < (1ULL << 32) &&
           std::max(p.input_width, p.output_width) < (1ULL << 22) &&
           reinterpret_cast<std::uintptr_t>(p.weight.codes) % 8 == 0 &&
           reinterpret_cast<std::uintptr_t>(p.activations) % 16 == 0;
}

}  // namespace

unsigned mfma_forward_tall_tile_columns(std::size_t rows,
                                        std::size_t output_width) {
    GemmShape shape{};
    shape.rows = static_cast<unsigned>(rows);
    shape.columns = static_cast<unsigned>(output_width);
    return tall_tile_columns(shape);
}

bool mfma_forward_supports(const LinearProblem& p) {
    // Contraction over the row width in steps of 32; a 16-weight chunk must
    // sit inside one quantisation block (true for every supported block size
    // once the row width is a multiple of 16).
    return common_supports(p) && p.input_width % kTileK == 0;
}

hipError_t launch_mfma_forward(const LinearProblem& p, hipStream_t stream) {
    return launch<false>(p, stream);
}

bool mfma_input_backward_supports(const LinearProblem& p) {
    // Contraction over weight rows in steps of 32; output columns in chunks
    // of 16 within a row.
    return common_supports(p) && p.output_width % kTileK == 0 &&
           p.input_width % Tile<false>::kChunk == 0;
}

hipError_t launch_mfma_input_backward(const LinearProblem& p,
                                      hipStream_t stream) {
    return launch<true>(p, stream);
}

}  // namespace rthip
