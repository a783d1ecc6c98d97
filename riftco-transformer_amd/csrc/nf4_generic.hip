// Shape-agnostic kernels of the packed NF4 linear path: any row width, any
// supported block size, odd element counts, blocks that straddle weight rows
// (the [33 x 33], block 32 layout of
// tests/core/backend/test_quantized_linear_backend.cpp:127-169).  They decode
// one nibble and one scale per multiply like the reference loops
// (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-115) and
// are the fallback when the streaming GEMV and the MFMA GEMM do not apply.
// Also here: the device dequantiser used to check decode bit-exactness and a
// fill kernel for freshly made tensor storage.

#include "kernels.hpp"
#include "nf4_decode.hpp"

namespace rthip {
namespace {

constexpr int kWave = 64;

__device__ __forceinline__ float wave_sum(float value) {
#pragma unroll
    for (int offset = kWave / 2; offset > 0; offset >>= 1) {
        value += __shfl_xor(value, offset, kWave);
    }
    return value;
}

__device__ __forceinline__ float decode_weight_any(
    const Nf4WeightView& weight, unsigned block_shift, std::size_t flat_index
) {
    return kNf4Codebook[unpack_code(weight.codes, flat_index)] *
           load_block_scale_any(weight, flat_index >> block_shift);
}

// Rows of x (forward) or dy (backward) that share one decode of a weight.
constexpr int kRowGroup = 8;

// One wavefront per (weight row o, group of eight rows of x): lanes stride the
// contraction so that neighbouring lanes read neighbouring nibbles and inputs,
// and a weight is decoded once for the eight products it enters.  Items are
// numbered group-major, so consecutive wavefronts walk consecutive weight
// rows.
__global__ __launch_bounds__(256) void generic_forward_kernel(
    const float* __restrict__ x, Nf4WeightView weight,
    const float* __restrict__ bias, float* __restrict__ y,
    std::size_t rows, std::size_t input_width, std::size_t output_width,
    unsigned block_shift, LoraEpilogue lora
) {
    const std::size_t waves_per_block = blockDim.x / kWave;
    const std::size_t wave =
        static_cast<std::size_t>(blockIdx.x) * waves_per_block +
        threadIdx.x / kWave;
    const std::size_t wave_stride =
        static_cast<std::size_t>(gridDim.x) * waves_per_block;
    const unsigned lane = threadIdx.x % kWave;
    const std::size_t groups = (rows + kRowGroup - 1) / kRowGroup;
    const std::size_t item_count = groups * output_width;

    for (std::size_t item = wave; item < item_count; item += wave_stride) {
        const std::size_t first_row = item / output_width * kRowGroup;
        const std::size_t column = item % output_width;
        const std::size_t here =
            rows - first_row < kRowGroup ? rows - first_row : kRowGroup;
        const float* input = x + first_row * input_width;
        const std::size_t weight_offset = column * input_width;
        float total[kRowGroup];
#pragma unroll
        for (int r = 0; r < kRowGroup; ++r) {
            total[r] = 0.0F;
        }
        if (here == 1) {  // uniform: one row, no per-row tests in the loop
            for (std::size_t i = lane; i < input_width; i += kWave) {
                total[0] += input[i] * decode_weight_any(weight, block_shift,
                                                         weight_offset + i);
            }
        } else {
            for (std::size_t i = lane; i < input_width; i += kWave) {
                const float w =
                    decode_weight_any(weight, block_shift, weight_offset + i);
#pragma unroll
                for (int r = 0; r < kRowGroup; ++r) {
                    if (static_cast<std::size_t>(r) < here) {  // uniform
                        total[r] += input[r * input_width + i] * w;
                    }
                }
            }
        }
#pragma unroll
        for (int r = 0; r < kRowGroup; ++r) {
            total[r] = wave_sum(total[r]);
        }
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < kRowGroup; ++r) {
                if (static_cast<std::size_t>(r) >= here) {
                    continue;
                }
                const std::size_t row = first_row + r;
                float value =
                    bias != nullptr ? total[r] + bias[column] : total[r];
                if (lora.reduced != nullptr) {
                    value += lora_term(lora, static_cast<unsigned>(row),
                                       static_cast<unsigned>(column));
                }
                y[row * output_width + column] = value;
            }
        }
    }
}

// Input backward.  A block owns 256 neighbouring columns of dx (neighbouring
// threads walk neighbouring nibbles of the same weight row, so code bytes and
// scales are shared within a wavefront), one chunk of the weight rows and one
// group of eight rows of dy, whose values are the same for every thread; a
// weight is decoded once for the eight products it enters.  gridDim = (column
// tiles, chunks of weight rows, row groups).  With one chunk the sums go
// straight to dx; otherwise to `target`, [chunk][rows][input_width], and
// generic_backward_sum_kernel adds the chunks in ascending order.
constexpr unsigned kBackwardColumns = 256;

__global__ __launch_bounds__(kBackwardColumns)
void generic_input_backward_kernel(
    const float* __restrict__ dy, Nf4WeightView weight,
    float* __restrict__ target, std::size_t rows, std::size_t input_width,
    std::size_t output_width, unsigned block_shift,
    std::size_t chunk_rows, LoraEpilogue lora
) {
    const std::size_t column =
        static_cast<std::size_t>(blockIdx.x) * kBackwardColumns + threadIdx.x;
    const std::size_t first = blockIdx.y * chunk_rows;
    const std::size_t last =
        first + chunk_rows < output_width ? first + chunk_rows : output_width;
    if (column >= input_width) {
        return;
    }
    const std::size_t groups = (rows + kRowGroup - 1) / kRowGroup;
    for (std::size_t group = blockIdx.z; group < groups;
         group += gridDim.z) {
        const std::size_t first_row = group * kRowGroup;
        const std::size_t here =
            rows - first_row < kRowGroup ? rows - first_row : kRowGroup;
        const float* upstream = dy + first_row * output_width;
        // Two levels of sums (runs of 64 weight rows folded into a second
        // accumulator): one fp32 chain over thousands of rows drifts like
        // the CPU's sequential sum.
        float total[kRowGroup];
#pragma unroll
        for (int r = 0; r < kRowGroup; ++r) {
            total[r] = 0.0F;
        }
        for (std::size_t run = first; run < last; run += 64) {
            const std::size_t run_end = run + 64 < last ? run + 64 : last;
            float partial[kRowGroup];
#pragma unroll
            for (int r = 0; r < kRowGroup; ++r) {
                partial[r] = 0.0F;
            }
            for (std::size_t o = run; o < run_end; ++o) {
                const float w = decode_weight_any(weight, block_shift,
                                                  o * input_width + column);
#pragma unroll
                for (int r = 0; r < kRowGroup; ++r) {
                    if (static_cast<std::size_t>(r) < here) {  // uniform
                        partial[r] += upstream[r * output_width + o] * w;
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < kRowGroup; ++r) {
                total[r] += partial[r];
            }
        }
        float* out = target + (static_cast<std::size_t>(blockIdx.y) * rows +
                               first_row) * input_width + column;
#pragma unroll
        for (int r = 0; r < kRowGroup; ++r) {
            if (static_cast<std::size_t>(r) < here) {
                float value = total[r];
                if (gridDim.y == 1 && lora.reduced != nullptr) {
                    value += lora_term(lora,
                                       static_cast<unsigned>(first_row + r),
                                       static_cast<unsigned>(column));
                }
                out[r * input_width] = value;
            }
        }
    }
}

// dx[e] = sum over chunks, ascending, of partial[chunk][e] (+ adapter term).
__global__ __launch_bounds__(256) void generic_backward_sum_kernel(
    const float* __restrict__ partial, float* __restrict__ dx,
    std::size_t elements, std::size_t chunks, std::size_t input_width,
    LoraEpilogue lora
) {
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    for (std::size_t element =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         element < elements; element += stride) {
        float sum = 0.0F;
        for (std::size_t chunk = 0; chunk < chunks; ++chunk) {
            sum += partial[chunk * elements + element];
        }
        if (lora.reduced != nullptr) {
            sum += lora_term(lora,
                             static_cast<unsigned>(element / input_width),
                             static_cast<unsigned>(element % input_width));
        }
        dx[element] = sum;
    }
}

// out[j] = scale(j / B) * codebook[code(j)]: one rounded multiply, the form of
// QuantizedWeight::dequantize (src/core/quantization/quantized_weight.cpp:462-465).
__global__ __launch_bounds__(256) void dequantize_kernel(
    Nf4WeightView weight, float* __restrict__ out, std::size_t element_count,
    unsigned block_shift
) {
#pragma clang fp contract(off)
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    for (std::size_t index =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < element_count; index += stride) {
        const float scale =
            load_block_scale_any(weight, index >> block_shift);
        out[index] = scale * kNf4Codebook[unpack_code(weight.codes, index)];
    }
}

__global__ __launch_bounds__(256) void fill_kernel(
    float* __restrict__ out, float value, std::size_t count
) {
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    for (std::size_t index =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        out[index] = value;
    }
}

unsigned grid_for(std::size_t work_items, std::size_t items_per_block) {
    // Enough blocks to cover the work once, capped at a few waves of the
    // 256-CU device; the kernels grid-stride over the remainder.
    constexpr std::size_t kMaxBlocks = 256 * 32;
    std::size_t blocks = (work_items + items_per_block - 1) / items_per_block;
    if (blocks < 1) {
        blocks = 1;
    }
    return static_cast<unsigned>(blocks < kMaxBlocks ? blocks : kMaxBlocks);
}

}  // namespace

void launch_generic_forward(const LinearProblem& p, hipStream_t stream) {
    const std::size_t items =
        (p.rows + kRowGroup - 1) / kRowGroup * p.output_width;
    generic_forward_kernel<<<grid_for(items, 4), 256, 0, stream>>>(
        p.activations, p.weight, p.bias, p.result, p.rows, p.input_width,
        p.output_width, p.block_shift, p.lora);
}

hipError_t launch_generic_input_backward(const LinearProblem& p,
                                         hipStream_t stream) {
    const std::size_t tiles =
        (p.input_width + kBackwardColumns - 1) / kBackwardColumns;
    const std::size_t groups = (p.rows + kRowGroup - 1) / kRowGroup;
    // Chunks of weight rows so that about two blocks per compute unit exist
    // (at least sixteen weight rows each), as far as the workspace holds
    // their sums.  Row groups beyond the grid's third dimension are walked
    // by a loop in the kernel.
    constexpr std::size_t kWantedBlocks = 512;
    std::size_t chunks = (kWantedBlocks + tiles * groups - 1) / (tiles * groups);
    const std::size_t most = (p.output_width + 15) / 16;
    chunks = chunks < most ? chunks : most;
    const std::size_t per_chunk = p.rows * p.input_width * sizeof(float);
    if (chunks > kStreamWorkspaceBytes / per_chunk) {
        chunks = kStreamWorkspaceBytes / per_chunk;
    }
    chunks = chunks < 1 ? 1 : (chunks > 65535 ? 65535 : chunks);
    const std::size_t chunk_rows = (p.output_width + chunks - 1) / chunks;
    chunks = (p.output_width + chunk_rows - 1) / chunk_rows;
    if (tiles > 0x7FFFFFFFULL) {
        return hipErrorInvalidValue;
    }
    float* target = p.result;
    WorkspaceLease lease;  // held until both launches are enqueued
    if (chunks > 1) {
        if (const hipError_t status = lease_stream_workspace(stream, &lease);
            status != hipSuccess) {
            return status;
        }
        target = lease.data();
    }
    const dim3 grid(static_cast<unsigned>(tiles),
                    static_cast<unsigned>(chunks),
                    static_cast<unsigned>(groups < 65535 ? groups : 65535));
    generic_input_backward_kernel<<<grid, kBackwardColumns, 0, stream>>>(
        p.activations, p.weight, target, p.rows, p.input_width,
        p.output_width, p.block_shift, chunk_rows, p.lora);
    if (chunks > 1) {
        const std::size_t elements = p.rows * p.input_width;
        generic_backward_sum_kernel<<<grid_for(elements, 256), 256, 0,
                                      stream>>>(
            target, p.result, elements, chunks, p.input_width, p.lora);
    }
    return hipSuccess;
}

void launch_dequantize(const Nf4WeightView& weight, float* out,
                       std::size_t element_count, unsigned block_shift,
                       hipStream_t stream) {
    dequantize_kernel<<<grid_for(element_count, 256), 256, 0, stream>>>(
        weight, out, element_count, block_shift);
}

void launch_fill(float* out, float value, std::size_t count,
                 hipStream_t stream) {
    fill_kernel<<<grid_for(count, 256), 256, 0, stream>>>(out, value, count);
}

}  // namespace rthip
