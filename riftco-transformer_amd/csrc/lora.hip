// reduced[m, j] = sum_k x[m, k] * A[j, k]: the first product of a low-rank
// adapter, matmul(x, transpose(A)) in LowRankAdapter::forward
// (src/nn/low_rank_adapter.cpp:140-143 under /root/reference).  A is
// [rank, input_width]; the result is tiny ([rows, rank]) and is consumed by
// the epilogue of the packed-weight kernels (lora_epilogue.hpp).
//
// Few outputs (up to 64 rows, or up to about 6000 outputs per sixteen adapter
// rows): one workgroup per output element (lora_reduce_rows_kernel).  Beyond
// that x is read exactly once: a workgroup of sixteen wavefronts owns
// 16 rows of x and up to 64 adapter rows; the contraction axis is cut into
// sixteen spans,
// one per wavefront, which each run v_mfma_f32_16x16x4_f32 over their span
// (A operand: x[16 rows][4 k]; B operand: A^T[4 k][16 adapter rows]) from
// 16-byte loads, and the sixteen partial tiles are added through LDS in
// wavefront order.
//
// Loads are raw buffer loads; lanes past the last row, the last adapter row or
// the row end get an offset the range check rejects and read zeros.

#include "kernels.hpp"

namespace rthip {
namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 16;
constexpr int kThreads = 64 * kWaves;
constexpr unsigned kRejectedOffset = 0x80000000U;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t raw_buffer(const void* base,
                                                            std::size_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(
        const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}

// kBlocks: 16-row blocks of A handled by one workgroup (1, 2 or 4).
template <int kBlocks>
__global__ __launch_bounds__(kThreads) void lora_reduce_kernel(
    const float* __restrict__ x, const float* __restrict__ a,
    float* __restrict__ reduced, unsigned rows, unsigned input_width,
    unsigned rank, unsigned rows_per_group
) {
    __shared__ float partial[kWaves][kBlocks][4][64];

    const unsigned lane = threadIdx.x % 64;
    const unsigned wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64);
    const unsigned quarter = lane / 16;
    // (a workgroup takes 16 rows of x, or 8 or 4 when that leaves compute
    // units without one: the other rows of its tile are then zeros)
    const unsigned row = blockIdx.x * rows_per_group + lane % 16;  // of x
    const unsigned first_adapter_row = blockIdx.y * 16 * kBlocks;

    const __amdgpu_buffer_rsrc_t x_buffer = raw_buffer(
        x, static_cast<std::size_t>(rows) * input_width * sizeof(float));
    const __amdgpu_buffer_rsrc_t a_buffer = raw_buffer(
        a, static_cast<std::size_t>(rank) * input_width * sizeof(float));

    // Spans are multiples of 16 contraction values.
    const unsigned span = ((input_width + 16 * kWaves - 1) / (16 * kWaves)) * 16;
    const unsigned span_begin = wave * span;
    const unsigned span_end = min(span_begin + span, input_width);

    const bool row_valid = lane % 16 < rows_per_group && row < rows;
    const unsigned x_row_bytes = row * input_width * 4U;
    bool adapter_valid[kBlocks];
    unsigned a_row_bytes[kBlocks];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
        const unsigned j = first_adapter_row + 16 * b + lane % 16;
        adapter_valid[b] = j < rank;
        a_row_bytes[b] = j * input_width * 4U;
    }

    floatx4 acc[kBlocks];
#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
        acc[b] = floatx4{0.0F, 0.0F, 0.0F, 0.0F};
    }
    // Four steps of 16 contraction values per trip, so that their loads are
    // in flight together; steps past the span read zeros.
    constexpr int kUnroll = 4;
    for (unsigned k0 = span_begin; k0 < span_end; k0 += 16 * kUnroll) {
        floatx4 xv[kUnroll];
        floatx4 av[kUnroll][kBlocks];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const unsigned k = k0 + 16 * u + 4 * quarter;
            // spans and the row width are multiples of 4, so a float4 lies
            // inside or outside as a whole
            const bool column_valid = k < span_end;
            xv[u] = __builtin_bit_cast(
                floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                             x_buffer,
                             row_valid && column_valid ? x_row_bytes + k * 4U
                                                       : kRejectedOffset,
                             0, 0));
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
                av[u][b] = __builtin_bit_cast(
                    floatx4, __builtin_amdgcn_raw_buffer_load_b128(
                                 a_buffer,
                                 adapter_valid[b] && column_valid
                                     ? a_row_bytes[b] + k * 4U
                                     : kRejectedOffset,
                                 0, 0));
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(
                        xv[u][e], av[u][b][e], acc[b], 0, 0, 0);
                }
            }
        }
    }

#pragma unroll
    for (int b = 0; b < kBlocks; ++b) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            partial[wave][b][r][lane] = acc[b][r];
        }
    }
    __syncthreads();
    // Accumulator element r of lane l is x row 4 * (l / 16) + r, adapter row
    // l % 16 of its block.  Thread t adds up element t of the tile.
    for (unsigned index = threadIdx.x; index < kBlocks * 256U;
         index += kThreads) {
        const unsigned b = index / 256;
        const unsigned r = (index / 64) % 4;
        const unsigned l = index % 64;
        float sum = 0.0F;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            sum += partial[w][b][r][l];
        }
        const unsigned row_in_group = 4 * (l / 16) + r;
        const unsigned m = blockIdx.x * rows_per_group + row_in_group;
        const unsigned j = first_adapter_row + 16 * b + l % 16;
        if (row_in_group < rows_per_group && m < rows && j < rank) {
            reduced[static_cast<std::size_t>(m) * rank + j] = sum;
        }
    }
}

// Few rows (decode and small batches): one workgroup per output element, so
// that the product takes one memory round trip however small it is.  Thread t
// takes float4 chunks t, t + 256, ...; the 256 partial sums are added with
// DPP-free shuffles inside each wavefront and then in wavefront order.
constexpr int kDotThreads = 256;

__device__ __forceinline__ void reduce_one_output(
    const float* __restrict__ x, const float* __restrict__ a,
    float* __restrict__ reduced, unsigned input_width, unsigned rank,
    unsigned j, unsigned m
) {
    __shared__ float wave_sums[kDotThreads / 64];
    const float4* x_row = reinterpret_cast<const float4*>(
        x + static_cast<std::size_t>(m) * input_width);
    const float4* a_row = reinterpret_cast<const float4*>(
        a + static_cast<std::size_t>(j) * input_width);
    const unsigned chunks = input_width / 4;
    float sum = 0.0F;
    constexpr int kUnroll = 4;
    for (unsigned c0 = threadIdx.x; c0 < chunks; c0 += kDotThreads * kUnroll) {
        float4 xv[kUnroll];
        float4 av[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const unsigned c = c0 + kDotThreads * u;
            const bool valid = c < chunks;
            const unsigned clamped = valid ? c : 0;
            xv[u] = x_row[clamped];
            av[u] = valid ? a_row[clamped] : make_float4(0.0F, 0.0F, 0.0F, 0.0F);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            sum += xv[u].x * av[u].x;
            sum += xv[u].y * av[u].y;
            sum += xv[u].z * av[u].z;
            sum += xv[u].w * av[u].w;
        }
    }
#pragma unroll
    for (int offset = 32; offset >= 1; offset /= 2) {
        sum += __shfl_xor(sum, offset, 64);
    }
    if (threadIdx.x % 64 == 0) {
        wave_sums[threadIdx.x / 64] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.0F;
#pragma unroll
        for (int w = 0; w < kDotThreads / 64; ++w) {
            total += wave_sums[w];
        }
        reduced[static_cast<std::size_t>(m) * rank + j] = total;
    }
}

__global__ __launch_bounds__(kDotThreads) void lora_reduce_rows_kernel(
    const float* __restrict__ x, const float* __restrict__ a,
    float* __restrict__ reduced, unsigned input_width, unsigned rank
) {
    reduce_one_output(x, a, reduced, input_width, rank, blockIdx.x,
                      blockIdx.y);
}

// The same for up to four adapters on one x in one launch (the query and
// value projections of a decoder block): blockIdx.z is the adapter.
struct ReduceItems {
    const float* a[kLoraReduceGroupMax];
    float* reduced[kLoraReduceGroupMax];
    unsigned rank[kLoraReduceGroupMax];
};

__global__ __launch_bounds__(kDotThreads) void lora_reduce_rows_group_kernel(
    const float* __restrict__ x, const ReduceItems items, unsigned input_width
) {
    const unsigned item = blockIdx.z;
    const unsigned rank = items.rank[item];
    if (blockIdx.x >= rank) {  // uniform
        return;
    }
    // (selects over kernel arguments: indexing them by a register would put
    // the array into scratch memory)
    const float* a = items.a[0];
    float* reduced = items.reduced[0];
#pragma unroll
    for (unsigned k = 1; k < kLoraReduceGroupMax; ++k) {
        if (item == k) {
            a = items.a[k];
            reduced = items.reduced[k];
        }
    }
    reduce_one_output(x, a, reduced, input_width, rank, blockIdx.x,
                      blockIdx.y);
}

// Any shape and alignment: one wavefront per output.
__global__ __launch_bounds__(256) void lora_reduce_generic_kernel(
    const float* __restrict__ x, const float* __restrict__ a,
    float* __restrict__ reduced, std::size_t rows, std::size_t input_width,
    std::size_t rank
) {
    const std::size_t output =
        (static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x) / 64;
    const unsigned lane = threadIdx.x % 64;
    if (output >= rows * rank) {
        return;
    }
    const float* x_row = x + (output / rank) * input_width;
    const float* a_row = a + (output % rank) * input_width;
    float sum = 0.0F;
    for (std::size_t k = lane; k < input_width; k += 64) {
        sum += x_row[k] * a_row[k];
    }
#pragma unroll
    for (int offset = 32; offset >= 1; offset /= 2) {
        sum += __shfl_xor(sum, offset, 64);
    }
    if (lane == 0) {
        reduced[output] = sum;
    }
}

}  // namespace

// One workgroup per output element pays while there are few outputs: about
// 3 us plus 1.25 us per thousand outputs of 4096 values, against 12 us and
// more per sixteen adapter rows for the kernel above (measured: rank 16 up to
// 384 rows, rank 64 likewise, rank 4 far beyond).
static bool reduce_by_outputs(std::size_t rows, std::size_t rank) {
    return rows <= 65535 && rank <= 65535 &&
           (rows <= 64 || rows * rank <= 6144 * ((rank + 15) / 16));
}

void launch_lora_reduce(const float* x, const float* a, float* reduced,
                        std::size_t rows, std::size_t input_width,
                        std::size_t rank, hipStream_t stream) {
    const bool tiled =
        input_width % 4 == 0 &&
        rows * input_width * sizeof(float) < kRejectedOffset &&
        rank * input_width * sizeof(float) < kRejectedOffset &&
        (rows + 3) / 4 < (1ULL << 31) && (rank + 63) / 64 <= 65535 &&
        reinterpret_cast<std::uintptr_t>(x) % 16 == 0 &&
        reinterpret_cast<std::uintptr_t>(a) % 16 == 0;
    if (!tiled) {
        const std::size_t waves = rows * rank;
        const unsigned blocks = static_cast<unsigned>((waves + 3) / 4);
        lora_reduce_generic_kernel<<<blocks, 256, 0, stream>>>(
            x, a, reduced, rows, input_width, rank);
        return;
    }
    if (reduce_by_outputs(rows, rank)) {
        lora_reduce_rows_kernel<<<dim3(static_cast<unsigned>(rank),
                                       static_cast<unsigned>(rows)),
                                  kDotThreads, 0, stream>>>(
            x, a, reduced, static_cast<unsigned>(input_width),
            static_cast<unsigned>(rank));
        return;
    }
    const auto r = static_cast<unsigned>(rows);
    const auto i = static_cast<unsigned>(input_width);
    const auto k = static_cast<unsigned>(rank);
    const unsigned chunks =
        rank <= 32 ? 1U : static_cast<unsigned>((rank + 63) / 64);
    // x comes in through the compute units that hold a workgroup: fewer rows
    // per workgroup while the grid is smaller than the device
    unsigned rows_per_group = 16;
    while (rows_per_group > 4 &&
           (rows + rows_per_group - 1) / rows_per_group * chunks < 256) {
        rows_per_group /= 2;
    }
    const unsigned row_tiles = static_cast<unsigned>(
        (rows + rows_per_group - 1) / rows_per_group);
    if (rank <= 16) {
        lora_reduce_kernel<1><<<dim3(row_tiles, 1), kThreads, 0, stream>>>(
            x, a, reduced, r, i, k, rows_per_group);
    } else if (rank <= 32) {
        lora_reduce_kernel<2><<<dim3(row_tiles, 1), kThreads, 0, stream>>>(
            x, a, reduced, r, i, k, rows_per_group);
    } else {
        lora_reduce_kernel<4><<<dim3(row_tiles, chunks), kThreads, 0, stream>>>(
            x, a, reduced, r, i, k, rows_per_group);
    }
}


void launch_lora_reduce_group(const float* x, const LoraReduceItem* items,
                              std::size_t count, std::size_t rows,
                              std::size_t input_width, hipStream_t stream) {
    std::size_t next = 0;
    while (next < count) {
        const std::size_t run =
            count - next < kLoraReduceGroupMax ? count - next
                                               : kLoraReduceGroupMax;
        bool together = run > 1 && input_width % 4 == 0 &&
                        rows * input_width * sizeof(float) < kRejectedOffset &&
                        reinterpret_cast<std::uintptr_t>(x) % 16 == 0;
        unsigned widest = 0;
        ReduceItems group{};
        for (std::size_t k = 0; k < run; ++k) {
            const LoraReduceItem& item = items[next + k];
            together = together && reduce_by_outputs(rows, item.rank) &&
                       item.rank * input_width * sizeof(float) <
                           kRejectedOffset &&
                       reinterpret_cast<std::uintptr_t>(item.a) % 16 == 0;
            group.a[k] = item.a;
            group.reduced[k] = item.reduced;
            group.rank[k] = static_cast<unsigned>(item.rank);
            widest = widest < group.rank[k] ? group.rank[k] : widest;
        }
        if (together) {
            lora_reduce_rows_group_kernel<<<
                dim3(widest, static_cast<unsigned>(rows),
                     static_cast<unsigned>(run)),
                kDotThreads, 0, stream>>>(x, group,
                                          static_cast<unsigned>(input_width));
        } else {
            for (std::size_t k = 0; k < run; ++k) {
                const LoraReduceItem& item = items[next + k];
                launch_lora_reduce(x, item.a, item.reduced, rows, input_width,
                                   item.rank, stream);
            }
        }
        next += run;
    }
}

}  // namespace rthip
