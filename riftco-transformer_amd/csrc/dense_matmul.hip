// Dense fp32 matmul  out[b] [M, N] = left[b] [M, K] * right[b] [K, N]
// (row-major, batched), restating BackendAdapter::matmul as the CPU adapter
// computes it (src/core/backend/adapters/cpu/adapter.cpp:158-203 under
// /root/reference).  In a QLoRA layer this is every product that is not the
// packed one: the adapter's x A^T, (.) B^T and their gradients.
//
// Tiling is the one of the packed GEMM (nf4_mfma.hip): a workgroup of four
// wavefronts computes a 128 x 128 output tile in steps of 32 along K, each
// wavefront owns a 64 x 64 quadrant as 2 x 2 blocks of v_mfma_f32_32x32x2_f32,
// both LDS tiles are [row-or-column][k] with a padded stride of 36 floats and
// are read with one ds_read_b128 per lane per four MFMAs, global loads of step
// t + 1 are issued before the MFMAs of step t, and accumulation is two-level
// (chains of 256 contraction values folded into a second accumulator).
// The right operand is [K, N]: a step reads 32 of its rows x 128 contiguous
// columns and transposes while writing LDS.  All edges (M, N, K not multiples
// of the tile) are handled by zero-filling; only K % 4 == 0, N % 4 == 0 and
// 16-byte aligned pointers are required -- other shapes take the plain kernel
// below, which is also the exact restatement of the reference loop (one fp32
// accumulator per output, ascending k).
//
// Narrow products (an adapter's x A^T, its gradients) have few output tiles and
// a long contraction; they would occupy a handful of compute units.  For a
// single matrix with fewer than 128 tiles the contraction is therefore cut
// into slices, one workgroup per (tile, slice) writes its partial tile to the
// stream's workspace, and a second kernel adds the slices in ascending order.
//
// A large single matrix whose tile count does not fill the device evenly
// (2048 x 11008 is 1376 tiles on 512 places) has its leftover tiles cut along
// the contraction and dealt in equal runs to the workgroups that would
// otherwise idle (tile_plan.hpp), as the packed GEMM does.

#include "kernels.hpp"
#include "tile_plan.hpp"

namespace rthip {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kTileM = 128;
constexpr int kTileN = 128;
constexpr int kTileK = 32;
constexpr int kStride = 36;
constexpr unsigned kFlushSteps = 8;

struct MatmulShape {
    unsigned rows;     // M
    unsigned shared;   // K
    unsigned columns;  // N
    // 0: blockIdx.z is the batch.  Otherwise blockIdx.z is a slice of this
    // many contraction values and `out` is the workspace of partial results.
    unsigned slice;
};

struct Staged {
    float4 left[4];
    float4 right[4];
};

__device__ __forceinline__ float4 zero4() {
    return make_float4(0.0F, 0.0F, 0.0F, 0.0F);
}

// left tile: rows row0..row0+127, 32 contraction values from k0.  Thread t
// takes float4 column t % 8 of rows t / 8 + 32 * pass.
__device__ __forceinline__ void load_left(Staged& staged,
                                          const float* __restrict__ left,
                                          const MatmulShape& shape,
                                          unsigned row0, unsigned k0) {
    const unsigned thread = threadIdx.x;
    const unsigned k = k0 + (thread % 8) * 4;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const unsigned row = row0 + thread / 8 + 32 * pass;
        staged.left[pass] =
            row < shape.rows && k < shape.shared
                ? *reinterpret_cast<const float4*>(
                      left + static_cast<std::size_t>(row) * shape.shared + k)
                : zero4();
    }
}

// right tile: contraction rows k0..k0+31, columns col0..col0+127.  Thread t
// takes 16 consecutive columns (t / 32) * 16 of row k0 + t % 32.
__device__ __forceinline__ void load_right(Staged& staged,
                                           const float* __restrict__ right,
                                           const MatmulShape& shape,
                                           unsigned col0, unsigned k0) {
    const unsigned thread = threadIdx.x;
    const unsigned k = k0 + thread % 32;
    const unsigned column = col0 + (thread / 32) * 16;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        staged.right[q] =
            k < shape.shared && column + 4 * q < shape.columns
                ? *reinterpret_cast<const float4*>(
                      right + static_cast<std::size_t>(k) * shape.columns +
                      column + 4 * q)
                : zero4();
    }
}

__device__ __forceinline__ void store_tiles(const Staged& staged,
                                            float* __restrict__ left_tile,
                                            float* __restrict__ right_tile) {
    const unsigned thread = threadIdx.x;
#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        *reinterpret_cast<float4*>(left_tile +
                                   (thread / 8 + 32 * pass) * kStride +
                                   (thread % 8) * 4) = staged.left[pass];
    }
    // tile[column][k]: transpose while writing.
    float* destination =
        right_tile + ((thread / 32) * 16) * kStride + thread % 32;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        destination[(4 * q + 0) * kStride] = staged.right[q].x;
        destination[(4 * q + 1) * kStride] = staged.right[q].y;
        destination[(4 * q + 2) * kStride] = staged.right[q].z;
        destination[(4 * q + 3) * kStride] = staged.right[q].w;
    }
}

// Contraction values [k_begin, k_end) of the output tile at (row0, col0).
// `partial` null: the result goes to `out` ([rows][columns]); otherwise the
// 128 x 128 sums go to `partial` ([kTileM][kTileN]).
__device__ __forceinline__ void matmul_segment(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, float* __restrict__ partial,
    const MatmulShape& shape, float* __restrict__ left_tile,
    float* __restrict__ right_tile, unsigned row0, unsigned col0,
    unsigned k_begin, unsigned k_end
) {
    const unsigned lane = threadIdx.x % 64;
    const unsigned wave = threadIdx.x / 64;
    const unsigned wave_m = wave / 2;
    const unsigned wave_n = wave % 2;

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

    // (loads past k_end of a slice are not masked: slices are multiples of
    // the step, so only the last slice ends inside a step, at the matrix edge)
    Staged staged;
    load_left(staged, left, shape, row0, k_begin);
    load_right(staged, right, shape, col0, k_begin);

    const float* left_fragment =
        left_tile + (wave_m * 64 + lane % 32) * kStride + 4 * (lane / 32);
    const float* right_fragment =
        right_tile + (wave_n * 64 + lane % 32) * kStride + 4 * (lane / 32);

    for (unsigned k0 = k_begin; k0 < k_end; k0 += kTileK) {
        __syncthreads();  // previous step's fragment reads are done
        store_tiles(staged, left_tile, right_tile);
        __syncthreads();

        const unsigned next = k0 + kTileK;
        if (next < k_end) {
            load_left(staged, left, shape, row0, next);
            load_right(staged, right, shape, col0, next);
        }

#pragma unroll
        for (int kk = 0; kk < kTileK; kk += 8) {
            float4 a[2];
            float4 b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = *reinterpret_cast<const float4*>(
                    left_fragment + i * 32 * kStride + kk);
                b[i] = *reinterpret_cast<const float4*>(
                    right_fragment + i * 32 * kStride + kk);
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
                            a_values[i][s], b_values[j][s], acc[i][j], 0, 0,
                            0);
                    }
                }
            }
        }

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
    }

    // Accumulator element e of lane l is output row 8*(e/4) + 4*(l/32) + e%4,
    // column l%32 of its 32 x 32 block.
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const unsigned tile_column = wave_n * 64 + j * 32 + lane % 32;
            const unsigned column = col0 + tile_column;
            if (partial == nullptr && column >= shape.columns) {
                continue;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const unsigned tile_row = wave_m * 64 + i * 32 + 8 * (e / 4) +
                                          4 * (lane / 32) + e % 4;
                const float value = total[i][j][e] + acc[i][j][e];
                if (partial != nullptr) {  // uniform
                    partial[tile_row * kTileN + tile_column] = value;
                } else if (row0 + tile_row < shape.rows) {
                    out[static_cast<std::size_t>(row0 + tile_row) *
                            shape.columns +
                        column] = value;
                }
            }
        }
    }
}

// One whole tile per workgroup; blockIdx.z is the batch or, for a sliced
// contraction, the slice.
__global__ __launch_bounds__(kThreads, 2) void dense_matmul_kernel(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, MatmulShape shape
) {
    __shared__ __attribute__((aligned(16))) float left_tile[kTileM * kStride];
    __shared__ __attribute__((aligned(16))) float right_tile[kTileN * kStride];
    unsigned k_begin = 0;
    unsigned k_end = shape.shared;
    if (shape.slice == 0) {
        const std::size_t batch = blockIdx.z;
        left += batch * shape.rows * shape.shared;
        right += batch * shape.shared * shape.columns;
        out += batch * shape.rows * shape.columns;
    } else {
        k_begin = blockIdx.z * shape.slice;
        k_end = min(k_begin + shape.slice, shape.shared);
        out += static_cast<std::size_t>(blockIdx.z) * shape.rows *
               shape.columns;
    }
    matmul_segment(left, right, out, nullptr, shape, left_tile, right_tile,
                   blockIdx.y * kTileM, blockIdx.x * kTileN, k_begin, k_end);
}

// A single matrix covered according to a TilePlan: whole tiles first, then
// runs of (tile, step) units.
__global__ __launch_bounds__(kThreads, 2) void dense_matmul_planned_kernel(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, float* __restrict__ workspace, MatmulShape shape,
    TilePlan plan
) {
    __shared__ __attribute__((aligned(16))) float left_tile[kTileM * kStride];
    __shared__ __attribute__((aligned(16))) float right_tile[kTileN * kStride];
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
        matmul_segment(left, right, out, partial, shape, left_tile,
                       right_tile, (tile / plan.tiles_n) * kTileM,
                       (tile % plan.tiles_n) * kTileN, first_step * kTileK,
                       min((first_step + segment_steps) * kTileK,
                           shape.shared));
        unit += segment_steps;
    }
}

// Adds the parts of every unit-dealt tile that more than one workgroup worked
// on, in ascending workgroup order.  blockIdx.x is the tile among the
// unit-dealt ones, blockIdx.y a run of 256 elements of it.
__global__ __launch_bounds__(256) void matmul_parts_kernel(
    const float* __restrict__ workspace, float* __restrict__ out,
    MatmulShape shape, TilePlan plan
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
    const unsigned row = (tile / plan.tiles_n) * kTileM + m;
    const unsigned column = (tile % plan.tiles_n) * kTileN + c;
    if (row >= shape.rows || column >= shape.columns) {
        return;
    }
    const float* source = workspace + m * kTileN + c;
    float sum = 0.0F;
    for (unsigned group = first_group; group <= last_group; ++group) {
        sum += source[static_cast<std::size_t>(plan.slot(group, dealt_tile)) *
                      kTileM * kTileN];
    }
    out[static_cast<std::size_t>(row) * shape.columns + column] = sum;
}

// out[i] = sum over slices of partial[slice][i], ascending.
__global__ __launch_bounds__(256) void add_slices_kernel(
    const float* __restrict__ partial, float* __restrict__ out,
    unsigned count, unsigned slices
) {
    const unsigned index = blockIdx.x * blockDim.x + threadIdx.x;
    if (index >= count) {
        return;
    }
    float sum = 0.0F;
    for (unsigned s = 0; s < slices; ++s) {
        sum += partial[static_cast<std::size_t>(s) * count + index];
    }
    out[index] = sum;
}

// Any shape: one thread per output, one fp32 accumulator, ascending k --
// the reference loop itself.  Neighbouring threads take neighbouring columns.
__global__ __launch_bounds__(256) void plain_matmul_kernel(
    const float* __restrict__ left, const float* __restrict__ right,
    float* __restrict__ out, std::size_t batch_count, std::size_t rows,
    std::size_t shared, std::size_t columns
) {
    const std::size_t per_batch = rows * columns;
    const std::size_t count = batch_count * per_batch;
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    for (std::size_t index =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        const std::size_t batch = index / per_batch;
        const std::size_t row = (index % per_batch) / columns;
        const std::size_t column = index % columns;
        const float* a = left + (batch * rows + row) * shared;
        const float* b = right + batch * shared * columns + column;
        float sum = 0.0F;
        for (std::size_t k = 0; k < shared; ++k) {
            sum += a[k] * b[k * columns];
        }
        out[index] = sum;
    }
}

}  // namespace

hipError_t launch_dense_matmul(const float* left, const float* right,
                               float* out, std::size_t batch_count,
                               std::size_t rows, std::size_t shared,
                               std::size_t columns, hipStream_t stream) {
    constexpr std::size_t kLimit = 1ULL << 31;
    const std::size_t tiles_m = (rows + kTileM - 1) / kTileM;
    const std::size_t tiles_n = (columns + kTileN - 1) / kTileN;
    const bool tiled =
        shared % 4 == 0 && columns % 4 == 0 && rows < kLimit &&
        shared < kLimit && columns < kLimit && tiles_m <= 65535 &&
        batch_count <= 65535 &&
        // a matrix-core tile pays off once there is a tile's worth of work
        rows * columns >= 1024 &&
        reinterpret_cast<std::uintptr_t>(left) % 16 == 0 &&
        reinterpret_cast<std::uintptr_t>(right) % 16 == 0;
    if (tiled) {
        MatmulShape shape;
        shape.rows = static_cast<unsigned>(rows);
        shape.shared = static_cast<unsigned>(shared);
        shape.columns = static_cast<unsigned>(columns);
        shape.slice = 0;
        const std::size_t tiles = tiles_m * tiles_n;
        const std::size_t steps = (shared + kTileK - 1) / kTileK;
        // Slices: enough workgroups for the device, at least four steps each,
        // and partial results that fit the workspace.
        std::size_t slices = 1;
        if (batch_count == 1 && tiles < 128 && steps >= 8) {
            slices = (256 + tiles - 1) / tiles;
            if (slices > steps / 4) {
                slices = steps / 4;
            }
            const std::size_t fit =
                kStreamWorkspaceBytes / (rows * columns * sizeof(float));
            if (slices > fit) {
                slices = fit;
            }
        }
        if (slices > 1) {
            const std::size_t steps_per_slice = (steps + slices - 1) / slices;
            shape.slice = static_cast<unsigned>(steps_per_slice * kTileK);
            slices = (shared + shape.slice - 1) / shape.slice;
            WorkspaceLease lease;  // held until both launches are enqueued
            if (const hipError_t status =
                    lease_stream_workspace(stream, &lease);
                status != hipSuccess) {
                return status;
            }
            float* const workspace = lease.data();
            const dim3 grid(static_cast<unsigned>(tiles_n),
                            static_cast<unsigned>(tiles_m),
                            static_cast<unsigned>(slices));
            dense_matmul_kernel<<<grid, kThreads, 0, stream>>>(
                left, right, workspace, shape);
            const unsigned count = static_cast<unsigned>(rows * columns);
            add_slices_kernel<<<(count + 255) / 256, 256, 0, stream>>>(
                workspace, out, count, static_cast<unsigned>(slices));
            return hipSuccess;
        }
        if (batch_count == 1 && tiles < (1ULL << 24)) {
            TilePlan plan;
            plan.tiles_n = static_cast<unsigned>(tiles_n);
            plan.steps = static_cast<unsigned>(steps);
            const unsigned groups = plan_tiles(
                plan, static_cast<unsigned>(tiles),
                kTileM * kTileN * sizeof(float), kStreamWorkspaceBytes);
            if (groups != 0) {
                WorkspaceLease lease;
                if (const hipError_t status =
                        lease_stream_workspace(stream, &lease);
                    status != hipSuccess) {
                    return status;
                }
                float* const workspace = lease.data();
                dense_matmul_planned_kernel<<<plan.whole_tiles + groups,
                                              kThreads, 0, stream>>>(
                    left, right, out, workspace, shape, plan);
                const dim3 parts(static_cast<unsigned>(tiles) -
                                     plan.whole_tiles,
                                 kTileM * kTileN / 256);
                matmul_parts_kernel<<<parts, 256, 0, stream>>>(workspace, out,
                                                               shape, plan);
                return hipSuccess;
            }
        }
        const dim3 grid(static_cast<unsigned>(tiles_n),
                        static_cast<unsigned>(tiles_m),
                        static_cast<unsigned>(batch_count));
        dense_matmul_kernel<<<grid, kThreads, 0, stream>>>(left, right, out,
                                                           shape);
        return hipSuccess;
    }
    const std::size_t outputs = batch_count * rows * columns;
    std::size_t blocks = (outputs + 255) / 256;
    if (blocks > 65535 * 16) {
        blocks = 65535 * 16;
    }
    if (blocks == 0) {
        blocks = 1;
    }
    plain_matmul_kernel<<<static_cast<unsigned>(blocks), 256, 0, stream>>>(
        left, right, out, batch_count, rows, shared, columns);
    return hipSuccess;
}

}  // namespace rthip
