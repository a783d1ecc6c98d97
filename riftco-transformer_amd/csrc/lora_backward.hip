// The backward pass of a low-rank adapter: what the reference's autograd
// computes for LowRankAdapter::forward (src/nn/low_rank_adapter.cpp:126-151
// under /root/reference) out of the closures of operator*, matmul and
// transpose_2d (src/core/autograd/operations.cpp:176-194,252-277,480-492):
//
//     scaled    = dy * scale                        [rows, output_width]
//     d_reduced = scaled . B                        [rows, rank]
//     dB        = (reduced^T . scaled)^T            [output_width, rank]
//     dA        = (x^T . d_reduced)^T               [rank, input_width]
//
// (the adapter's share of dx, d_reduced . A, is added in the epilogue of the
// packed-weight input backward, lora_epilogue.hpp).  Every product is rounded
// to fp32 and summed in fp32; `scaled` is rounded once per element as the
// reference's elementwise multiply does and never stored.
//
// Two kernels, both on v_mfma_f32_16x16x4_f32 with sixteen wavefronts per
// workgroup that split the contraction and add their tiles through LDS in
// wavefront order, so results do not depend on timing:
//
//  * contract_columns_kernel: d_reduced.  A workgroup owns 16 rows of dy and a
//    slice of the output columns; dy is read once with 16-byte loads, B (small,
//    from L2) with 4-byte loads.  Few rows: the columns are cut into slices so
//    that the device is full, slices go to the stream workspace and
//    sum_slices_kernel adds them in ascending order.
//  * contract_rows_kernel: dB and dA, out[n, j] = sum_m left[m, n] * right[m, j]
//    with (left, right) = (scaled, reduced) or (x, d_reduced).  A workgroup
//    owns 32 columns of `left`, which is read once with 8-byte loads (four
//    rows of 128 contiguous bytes per instruction), and writes its tile of the
//    result as [n, j] (dB) or [j, n] (dA).
//
// Lanes that have nothing to read get an offset the buffer range check
// rejects and read zeros.  Shapes these kernels do not take (odd widths,
// more than 2 GiB per operand) go to one-thread-per-output kernels.

#include "kernels.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kWaves = 16;
constexpr int kThreads = 64 * kWaves;
constexpr unsigned kRejectedOffset = 0x80000000U;
constexpr unsigned kComputeUnits = 256;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base,
                                                            std::size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// ---- d_reduced[m, j] = sum_o (dy[m, o] * scale) * B[o, j] -----------------

// kBlocks: 16-wide blocks of the rank handled by one workgroup (1, 2 or 4).
// gridDim = (row tiles of 16, column slices, rank chunks of 16 * kBlocks).
template <int kBlocks>
__global__ __launch_bounds__(kThreads) void contract_columns_kernel(
    const float* __restrict__ dy, const float* __restrict__ b,
    float* __restrict__ target, unsigned rows, unsigned output_width,
    unsigned rank, float scale, unsigned slice_columns
) {
    __shared__ float partial[kWaves][kBlocks][4][64];

    const unsigned lane = threadIdx.x % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const unsigned quarter = lane / 16;
    const unsigned row = blockIdx.x * 16 + lane % 16;  // of dy
    const unsigned first_slot = blockIdx.z * 16 * kBlocks;

    const __amdgpu_buffer_rsrc_t dy_buffer = raw_buffer(
        dy, static_cast<std::size_t>(rows) * output_width * sizeof(float));
    const __amdgpu_buffer_rsrc_t b_buffer = raw_buffer(
        b, static_cast<std::size_t>(output_width) * rank * sizeof(float));

    // This workgroup's columns, cut into one span per wavefront (multiples
    // of 16 columns).
    const unsigned slice_begin = blockIdx.y * slice_columns;
    const unsigned slice_end = min(slice_begin + slice_columns, output_width);
    const unsigned span = ((slice_columns + 16 * kWaves - 1) / (16 * kWaves)) * 16;
    const unsigned span_begin = min(slice_begin + wave * span, slice_end);
    const unsigned span_end = min(span_begin + span, slice_end);

    const bool row_valid = row < rows;
    const unsigned row_bytes = row * output_width * 4U;
    bool slot_valid[kBlocks];
    unsigned slot_bytes[kBlocks];
#pragma unroll
    for (int block = 0; block < kBlocks; ++block) {
        const unsigned j = first_slot + 16 * block + lane % 16;
        slot_valid[block] = j < rank;
        slot_bytes[block] = j * 4U;
    }

    floatx4 acc[kBlocks];
#pragma unroll
    for (int block = 0; block < kBlocks; ++block) {
        acc[block] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
    }
    // Two steps of 16 columns per trip, their loads in flight together;
    // steps past the span read zeros.
    constexpr int kUnroll = 2;
    for (unsigned o0 = span_begin; o0 < span_end; o0 += 16 * kUnroll) {
        floatx4 upstream[kUnroll];
        float factor[kUnroll][kBlocks][4];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            // the output width is a multiple of 4 and so is every span
            // boundary: a float4 lies inside or outside as a whole
            const unsigned o = o0 + 16 * u + 4 * quarter;
            const bool column_valid = o < span_end;
            upstream[u] = __builtin_bit_cast(
                floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                             dy_buffer,
                             row_valid && column_valid ? row_bytes + o * 4U
                                                       : kRejectedOffset,
                             0, 0));
#pragma unroll
            for (int block = 0; block < kBlocks; ++block) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    factor[u][block][e] = __builtin_bit_cast(
                        float, __builtin_amdgcn_raw_buffer_load_b32(
                                   b_buffer,
                                   slot_valid[block] && column_valid
                                       ? (o + e) * rank * 4U + slot_bytes[block]
                                       : kRejectedOffset,
                                   0, 0));
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float scaled = upstream[u][e] * scale;
#pragma unroll
                for (int block = 0; block < kBlocks; ++block) {
                    acc[block] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        scaled, factor[u][block][e], acc[block], 0, 0, 0);
                }
            }
        }
    }

#pragma unroll
    for (int block = 0; block < kBlocks; ++block) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            partial[wave][block][r][lane] = acc[block][r];
        }
    }
    __syncthreads();
    // Accumulator element r of lane l is dy row 4 * (l / 16) + r, rank slot
    // l % 16 of its block.  Thread t adds up element t of the tile.
    float* const out =
        target + static_cast<std::size_t>(blockIdx.y) * rows * rank;
    for (unsigned index = threadIdx.x; index < kBlocks * 256U;
         index += kThreads) {
        const unsigned block = index / 256;
        const unsigned r = (index / 64) % 4;
        const unsigned l = index % 64;
        float sum = 0.0F;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            sum += partial[w][block][r][l];
        }
        const unsigned m = blockIdx.x * 16 + 4 * (l / 16) + r;
        const unsigned j = first_slot + 16 * block + l % 16;
        if (m < rows && j < rank) {
            out[static_cast<std::size_t>(m) * rank + j] = sum;
        }
    }
}

// out[e] = sum over slices, ascending, of slices[s][e].
__global__ __launch_bounds__(256) void sum_slices_kernel(
    const float* __restrict__ slices, float* __restrict__ out,
    unsigned elements, unsigned count
) {
    const unsigned element = blockIdx.x * blockDim.x + threadIdx.x;
    if (element >= elements) {
        return;
    }
    float sum = 0.0F;
    unsigned s = 0;
    for (; s + 4 <= count; s += 4) {  // four loads in flight
        float part[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            part[i] = slices[static_cast<std::size_t>(s + i) * elements +
                             element];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sum += part[i];
        }
    }
    for (; s < count; ++s) {
        sum += slices[static_cast<std::size_t>(s) * elements + element];
    }
    out[element] = sum;
}

// Any shape: one thread per d_reduced[m, j].
__global__ __launch_bounds__(256) void contract_columns_generic_kernel(
    const float* __restrict__ dy, const float* __restrict__ b,
    float* __restrict__ d_reduced, std::size_t rows,
    std::size_t output_width, std::size_t rank, float scale
) {
    const std::size_t index =
        static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= rows * rank) {
        return;
    }
    const float* upstream = dy + (index / rank) * output_width;
    const float* column = b + index % rank;
    float sum = 0.0F;
    for (std::size_t o = 0; o < output_width; ++o) {
        sum += (upstream[o] * scale) * column[o * rank];
    }
    d_reduced[index] = sum;
}

// ---- out[n, j] = sum_m (left[m, n] * scale) * right[m, j] -----------------

// kBlocks: 1 or 2; kTransposed: the result is stored [j, n] (dA) instead of
// [n, j] (dB).  gridDim = (column tiles of 32, rank chunks).
template <int kBlocks, bool kTransposed>
__global__ __launch_bounds__(kThreads) void contract_rows_kernel(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, unsigned rows, unsigned width, unsigned rank,
    float scale
) {
    __shared__ float partial[kWaves][2][kBlocks][4][64];

    const unsigned lane = threadIdx.x % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const unsigned quarter = lane / 16;
    const unsigned column = blockIdx.x * 32 + 2 * (lane % 16);  // and + 1
    const unsigned first_slot = blockIdx.y * 16 * kBlocks;

    const __amdgpu_buffer_rsrc_t left_buffer = raw_buffer(
        left, static_cast<std::size_t>(rows) * width * sizeof(float));
    const __amdgpu_buffer_rsrc_t right_buffer = raw_buffer(
        right, static_cast<std::size_t>(rows) * rank * sizeof(float));

    // Rows are dealt to the wavefronts in spans that are multiples of 4.
    const unsigned span = ((rows + 4 * kWaves - 1) / (4 * kWaves)) * 4;
    const unsigned span_begin = min(wave * span, rows);
    const unsigned span_end = min(span_begin + span, rows);

    // the width is even: a float2 lies inside or outside as a whole
    const bool column_valid = column < width;
    bool slot_valid[kBlocks];
    unsigned slot_bytes[kBlocks];
#pragma unroll
    for (int block = 0; block < kBlocks; ++block) {
        const unsigned j = first_slot + 16 * block + lane % 16;
        slot_valid[block] = j < rank;
        slot_bytes[block] = j * 4U;
    }

    floatx4 acc[2][kBlocks];
#pragma unroll
    for (int e = 0; e < 2; ++e) {
#pragma unroll
        for (int block = 0; block < kBlocks; ++block) {
            acc[e][block] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
        }
    }
    constexpr int kUnroll = 4;  // steps of four rows per trip
    for (unsigned m0 = span_begin; m0 < span_end; m0 += 4 * kUnroll) {
        floatx2 first[kUnroll];
        float second[kUnroll][kBlocks];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const unsigned m = m0 + 4 * u + quarter;
            const bool row_valid = m < span_end;
            first[u] = __builtin_bit_cast(
                floatx2, __builtin_amdgcn_raw_buffer_load_b64(
                             left_buffer,
                             row_valid && column_valid
                                 ? (m * width + column) * 4U
                                 : kRejectedOffset,
                             0, 0));
#pragma unroll
            for (int block = 0; block < kBlocks; ++block) {
                second[u][block] = __builtin_bit_cast(
                    float, __builtin_amdgcn_raw_buffer_load_b32(
                               right_buffer,
                               row_valid && slot_valid[block]
                                   ? m * rank * 4U + slot_bytes[block]
                                   : kRejectedOffset,
                               0, 0));
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const float scaled = first[u][e] * scale;
#pragma unroll
                for (int block = 0; block < kBlocks; ++block) {
                    acc[e][block] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        scaled, second[u][block], acc[e][block], 0, 0, 0);
                }
            }
        }
    }

#pragma unroll
    for (int e = 0; e < 2; ++e) {
#pragma unroll
        for (int block = 0; block < kBlocks; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                partial[wave][e][block][r][lane] = acc[e][block][r];
            }
        }
    }
    __syncthreads();
    // Accumulator element r of lane l, column half e: column
    // 2 * (4 * (l / 16) + r) + e of the tile, rank slot l % 16 of its block.
    for (unsigned index = threadIdx.x; index < 2U * kBlocks * 256U;
         index += kThreads) {
        const unsigned e = index / (kBlocks * 256);
        const unsigned block = (index / 256) % kBlocks;
        const unsigned r = (index / 64) % 4;
        const unsigned l = index % 64;
        float sum = 0.0F;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            sum += partial[w][e][block][r][l];
        }
        const unsigned n = blockIdx.x * 32 + 2 * (4 * (l / 16) + r) + e;
        const unsigned j = first_slot + 16 * block + l % 16;
        if (n < width && j < rank) {
            if constexpr (kTransposed) {
                out[static_cast<std::size_t>(j) * width + n] = sum;
            } else {
                out[static_cast<std::size_t>(n) * rank + j] = sum;
            }
        }
    }
}

// Any shape: one thread per output, neighbouring threads neighbouring columns
// of `left`.
__global__ __launch_bounds__(256) void contract_rows_generic_kernel(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, std::size_t rows, std::size_t width,
    std::size_t rank, float scale, bool transposed
) {
    const std::size_t index =
        static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= width * rank) {
        return;
    }
    const std::size_t n = index % width;
    const std::size_t j = index / width;
    float sum = 0.0F;
    for (std::size_t m = 0; m < rows; ++m) {
        sum += (left[m * width + n] * scale) * right[m * rank + j];
    }
    out[transposed ? j * width + n : n * rank + j] = sum;
}

bool aligned(const void* pointer, std::size_t bytes) {
    return reinterpret_cast<std::uintptr_t>(pointer) % bytes == 0;
}

template <bool kTransposed>
void launch_contract_rows(const float* left, const float* right, float* out,
                          std::size_t rows, std::size_t width,
                          std::size_t rank, float scale, hipStream_t stream) {
    const bool tiled =
        width % 2 == 0 && rows * width * sizeof(float) < kRejectedOffset &&
        rows * rank * sizeof(float) < kRejectedOffset &&
        (rank + 31) / 32 <= 65535 && aligned(left, 8) && aligned(right, 4);
    if (!tiled) {
        const std::size_t outputs = width * rank;
        contract_rows_generic_kernel<<<
            static_cast<unsigned>((outputs + 255) / 256), 256, 0, stream>>>(
            left, right, out, rows, width, rank, scale, kTransposed);
        return;
    }
    const unsigned tiles = static_cast<unsigned>((width + 31) / 32);
    const auto m = static_cast<unsigned>(rows);
    const auto n = static_cast<unsigned>(width);
    const auto k = static_cast<unsigned>(rank);
    if (rank <= 16) {
        contract_rows_kernel<1, kTransposed>
            <<<dim3(tiles, 1), kThreads, 0, stream>>>(left, right, out, m, n,
                                                      k, scale);
    } else {  // (two blocks: the wavefronts' tiles fill the 64 KB of LDS)
        const unsigned chunks = static_cast<unsigned>((rank + 31) / 32);
        contract_rows_kernel<2, kTransposed>
            <<<dim3(tiles, chunks), kThreads, 0, stream>>>(left, right, out,
                                                           m, n, k, scale);
    }
}

hipError_t launch_contract_columns(const float* dy, const float* b,
                                   float* d_reduced, std::size_t rows,
                                   std::size_t output_width, std::size_t rank,
                                   float scale, hipStream_t stream) {
    const std::size_t row_tiles = (rows + 15) / 16;
    const bool tiled =
        output_width % 4 == 0 &&
        rows * output_width * sizeof(float) < kRejectedOffset &&
        output_width * rank * sizeof(float) < kRejectedOffset &&
        row_tiles < (1ULL << 31) && (rank + 63) / 64 <= 65535 &&
        aligned(dy, 16) && aligned(b, 4);
    if (!tiled) {
        const std::size_t outputs = rows * rank;
        contract_columns_generic_kernel<<<
            static_cast<unsigned>((outputs + 255) / 256), 256, 0, stream>>>(
            dy, b, d_reduced, rows, output_width, rank, scale);
        return hipSuccess;
    }
    // Slices of the columns, multiples of 256 (16 per wavefront), so that
    // about two workgroups per compute unit exist; bounded by the workspace.
    const std::size_t widest = (output_width + 255) / 256;
    std::size_t slices = (2 * kComputeUnits + row_tiles - 1) / row_tiles;
    slices = slices < widest ? slices : widest;
    const std::size_t slice_bytes = rows * rank * sizeof(float);
    if (slices > kStreamWorkspaceBytes / slice_bytes) {
        slices = kStreamWorkspaceBytes / slice_bytes;
    }
    slices = slices < 1 ? 1 : slices;
    slices = slices > 65535 ? 65535 : slices;
    const std::size_t slice_columns =
        ((output_width + slices - 1) / slices + 255) / 256 * 256;
    slices = (output_width + slice_columns - 1) / slice_columns;

    float* target = d_reduced;
    WorkspaceLease lease;  // held until both launches are enqueued
    if (slices > 1) {
        if (const hipError_t status = lease_stream_workspace(stream, &lease);
            status != hipSuccess) {
            return status;
        }
        target = lease.data();
    }
    const auto m = static_cast<unsigned>(rows);
    const auto n = static_cast<unsigned>(output_width);
    const auto k = static_cast<unsigned>(rank);
    const auto columns = static_cast<unsigned>(slice_columns);
    const auto tiles = static_cast<unsigned>(row_tiles);
    const auto count = static_cast<unsigned>(slices);
    if (rank <= 16) {
        contract_columns_kernel<1><<<dim3(tiles, count, 1), kThreads, 0,
                                     stream>>>(dy, b, target, m, n, k, scale,
                                               columns);
    } else if (rank <= 32) {
        contract_columns_kernel<2><<<dim3(tiles, count, 1), kThreads, 0,
                                     stream>>>(dy, b, target, m, n, k, scale,
                                               columns);
    } else {
        const unsigned chunks = static_cast<unsigned>((rank + 63) / 64);
        contract_columns_kernel<4><<<dim3(tiles, count, chunks), kThreads, 0,
                                     stream>>>(dy, b, target, m, n, k, scale,
                                               columns);
    }
    if (slices > 1) {
        const unsigned elements = static_cast<unsigned>(rows * rank);
        sum_slices_kernel<<<(elements + 255) / 256, 256, 0, stream>>>(
            target, d_reduced, elements, count);
    }
    return hipSuccess;
}

}  // namespace

hipError_t launch_lora_backward(const LoraBackwardProblem& p,
                                hipStream_t stream) {
    if (const hipError_t status = launch_contract_columns(
            p.upstream, p.b, p.d_reduced, p.rows, p.output_width, p.rank,
            p.scale, stream);
        status != hipSuccess) {
        return status;
    }
    if (p.d_b != nullptr) {
        launch_contract_rows<false>(p.upstream, p.reduced, p.d_b, p.rows,
                                    p.output_width, p.rank, p.scale, stream);
    }
    if (p.d_a != nullptr) {
        launch_contract_rows<true>(p.activations, p.d_reduced, p.d_a, p.rows,
                                   p.input_width, p.rank, 1.0F, stream);
    }
    return hipSuccess;
}

}  // namespace rthip
