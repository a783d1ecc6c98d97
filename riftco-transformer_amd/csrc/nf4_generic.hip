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

// One wavefront per output element y[r, o]; lanes stride the contraction so
// that neighbouring lanes read neighbouring nibbles and inputs.
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
    const std::size_t output_count = rows * output_width;

    for (std::size_t output_index = wave; output_index < output_count;
         output_index += wave_stride) {
        const std::size_t row = output_index / output_width;
        const std::size_t column = output_index % output_width;
        const float* input = x + row * input_width;
        const std::size_t weight_offset = column * input_width;
        float total = 0.0F;
        for (std::size_t i = lane; i < input_width; i += kWave) {
            total += input[i] *
                     decode_weight_any(weight, block_shift, weight_offset + i);
        }
        total = wave_sum(total);
        if (lane == 0) {
            float value = bias != nullptr ? total + bias[column] : total;
            if (lora.reduced != nullptr) {
                value += lora_term(lora, static_cast<unsigned>(row),
                                   static_cast<unsigned>(column));
            }
            y[output_index] = value;
        }
    }
}

// One thread per dx[r, i]; neighbouring threads walk neighbouring columns of
// the same weight row, so code bytes and scales are shared within a wave.
__global__ __launch_bounds__(256) void generic_input_backward_kernel(
    const float* __restrict__ dy, Nf4WeightView weight,
    float* __restrict__ dx, std::size_t rows, std::size_t input_width,
    std::size_t output_width, unsigned block_shift, LoraEpilogue lora
) {
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    const std::size_t gradient_count = rows * input_width;
    for (std::size_t index =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < gradient_count; index += stride) {
        const std::size_t row = index / input_width;
        const std::size_t column = index % input_width;
        const float* upstream = dy + row * output_width;
        // Eight interleaved partial sums: shorter rounding walks than one
        // long chain, and independent multiply-adds in flight.
        float partial[8] = {0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F, 0.0F};
        std::size_t o = 0;
        for (; o + 8 <= output_width; o += 8) {
#pragma unroll
            for (int lane = 0; lane < 8; ++lane) {
                partial[lane] += upstream[o + lane] *
                    decode_weight_any(weight, block_shift,
                                      (o + lane) * input_width + column);
            }
        }
        for (; o < output_width; ++o) {
            partial[o % 8] += upstream[o] *
                decode_weight_any(weight, block_shift,
                                  o * input_width + column);
        }
        const float total =
            ((partial[0] + partial[1]) + (partial[2] + partial[3])) +
            ((partial[4] + partial[5]) + (partial[6] + partial[7]));
        dx[index] = lora.reduced == nullptr
                        ? total
                        : total + lora_term(lora, static_cast<unsigned>(row),
                                            static_cast<unsigned>(column));
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
    const std::size_t outputs = p.rows * p.output_width;
    generic_forward_kernel<<<grid_for(outputs, 4), 256, 0, stream>>>(
        p.activations, p.weight, p.bias, p.result, p.rows, p.input_width,
        p.output_width, p.block_shift, p.lora);
}

void launch_generic_input_backward(const LinearProblem& p,
                                   hipStream_t stream) {
    const std::size_t gradients = p.rows * p.input_width;
    generic_input_backward_kernel<<<grid_for(gradients, 256), 256, 0,
                                    stream>>>(
        p.activations, p.weight, p.result, p.rows, p.input_width,
        p.output_width, p.block_shift, p.lora);
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
