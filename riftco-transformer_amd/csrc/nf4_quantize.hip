// The NF4 quantizer on the device: pack_nf4 and double_quantize_scales of the
// reference (src/core/quantization/quantized_weight.cpp:176-206 and :208-254,
// nearest_nf4_code src/core/quantization/nf4.cpp:55-68, under /root/reference),
// bit for bit.
//
//   block scale   s_b = max |w| over the block (fp32; max is order-free)
//   code          7 for a zero block, else the codebook entry nearest to w / s_b
//                 -- the reference's linear scan with a strict '<', so the
//                 lowest index wins a tie; the division is correctly rounded
//   packing       even flat index in the low nibble, an unused high nibble of
//                 the last byte stays zero
//   double quantisation of the scales
//                 offset = (float)(sum of the scales in double, in index
//                 order, / count);  per group of C scales t = max |s - offset|,
//                 code = 128 + clamp(round-half-away(127 (s - offset) / t)),
//                 every operation rounded on its own
//
// The one step whose result depends on evaluation order is the double sum.
// It is evaluated in parallel only when that provably cannot matter: the
// scales are non-negative fp32 values, so if count * max < 2^53 * (smallest
// unit in the last place among the non-zero scales), every partial sum in
// every order is exactly representable and all orders give the same double.
// Otherwise one thread adds the scales in index order, as the reference does.

#include "kernels.hpp"
#include "nf4_decode.hpp"

#include <cfloat>

namespace rthip {
namespace {

// Bits of the status word the kernels report through.
constexpr unsigned kNonFiniteSource = 1U;
constexpr unsigned kOffsetOverflow = 2U;

__device__ __forceinline__ unsigned nearest_code(float normalized) {
    unsigned best_code = 0;
    float best_distance = fabsf(normalized - kNf4Codebook[0]);
#pragma unroll
    for (unsigned code = 1; code < 16; ++code) {
        const float distance = fabsf(normalized - kNf4Codebook[code]);
        if (distance < best_distance) {
            best_distance = distance;
            best_code = code;
        }
    }
    return best_code;
}

// One wavefront per quantisation block: scale = max |w|.
__global__ __launch_bounds__(256) void block_scale_kernel(
    const float* __restrict__ values, std::size_t element_count,
    unsigned block_shift, std::size_t block_count, float* __restrict__ scales,
    unsigned* __restrict__ status
) {
    const std::size_t waves_per_grid =
        static_cast<std::size_t>(gridDim.x) * (blockDim.x / 64);
    const unsigned lane = threadIdx.x % 64;
    const std::size_t block_size = std::size_t{1} << block_shift;
    bool bad = false;
    for (std::size_t block =
             static_cast<std::size_t>(blockIdx.x) * (blockDim.x / 64) +
             threadIdx.x / 64;
         block < block_count; block += waves_per_grid) {
        const std::size_t begin = block << block_shift;
        const std::size_t end = begin + block_size < element_count
                                    ? begin + block_size
                                    : element_count;
        float scale = 0.0F;
        for (std::size_t index = begin + lane; index < end; index += 64) {
            const float value = values[index];
            bad = bad || !isfinite(value);
            const float magnitude = fabsf(value);
            scale = scale < magnitude ? magnitude : scale;
        }
#pragma unroll
        for (int offset = 32; offset >= 1; offset /= 2) {
            const float other = __shfl_xor(scale, offset, 64);
            scale = scale < other ? other : scale;
        }
        if (lane == 0) {
            scales[block] = scale;
        }
    }
    if (bad) {
        atomicOr(status, kNonFiniteSource);
    }
}

// One thread per eight consecutive weights (four code bytes); eight weights
// never straddle a block because block sizes are multiples of 32.
__global__ __launch_bounds__(256) void encode_kernel(
    const float* __restrict__ values, std::size_t element_count,
    unsigned block_shift, const float* __restrict__ scales,
    std::uint8_t* __restrict__ codes
) {
    const std::size_t group_count = (element_count + 7) / 8;
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    for (std::size_t group =
             static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         group < group_count; group += stride) {
        const std::size_t first = group * 8;
        const float scale = scales[first >> block_shift];
        unsigned packed = 0;
#pragma unroll
        for (unsigned i = 0; i < 8; ++i) {
            const std::size_t index = first + i;
            unsigned code = 0;  // an unused nibble stays zero
            if (index < element_count) {
                code = scale == 0.0F ? 7U : nearest_code(values[index] / scale);
            }
            packed |= code << (4 * i);
        }
        const std::size_t byte_count = (element_count + 1) / 2;
        const std::size_t first_byte = group * 4;
        if (first_byte + 4 <= byte_count) {
            // four-byte groups start at multiples of four bytes
            *reinterpret_cast<unsigned*>(codes + first_byte) = packed;
        } else {
            for (unsigned i = 0; first_byte + i < byte_count; ++i) {
                codes[first_byte + i] =
                    static_cast<std::uint8_t>((packed >> (8 * i)) & 0xFFU);
            }
        }
    }
}

// offset = (float)(sum of the scales in double / count), by ONE workgroup.
constexpr int kMeanThreads = 1024;

__global__ __launch_bounds__(kMeanThreads) void scale_mean_kernel(
    const float* __restrict__ scales, std::size_t count,
    float* __restrict__ offset_out, unsigned* __restrict__ status
) {
    __shared__ double sums[kMeanThreads];
    __shared__ int largest_exponent[kMeanThreads];
    __shared__ int smallest_ulp[kMeanThreads];

    // exponent of a value's unit in the last place; INT_MAX for zero
    double sum = 0.0;
    int top = INT_MIN;
    int ulp = INT_MAX;
    for (std::size_t index = threadIdx.x; index < count;
         index += kMeanThreads) {
        const float value = scales[index];
        sum += static_cast<double>(value);
        if (value != 0.0F) {
            const unsigned bits = __float_as_uint(value);
            const int biased = static_cast<int>((bits >> 23) & 0xFFU);
            const int exponent = (biased == 0 ? 1 : biased) - 127;
            top = max(top, exponent);
            ulp = min(ulp, exponent - 23);
        }
    }
    sums[threadIdx.x] = sum;
    largest_exponent[threadIdx.x] = top;
    smallest_ulp[threadIdx.x] = ulp;
    __syncthreads();
    for (int width = kMeanThreads / 2; width >= 1; width /= 2) {
        if (static_cast<int>(threadIdx.x) < width) {
            sums[threadIdx.x] += sums[threadIdx.x + width];
            largest_exponent[threadIdx.x] =
                max(largest_exponent[threadIdx.x],
                    largest_exponent[threadIdx.x + width]);
            smallest_ulp[threadIdx.x] = min(smallest_ulp[threadIdx.x],
                                            smallest_ulp[threadIdx.x + width]);
        }
        __syncthreads();
    }
    if (threadIdx.x != 0) {
        return;
    }
    double total = sums[0];
    if (largest_exponent[0] != INT_MIN) {
        // every value < 2^(top + 1), so any partial sum < count * 2^(top + 1)
        // <= 2^(count_bits + top + 1); exact in double while that stays
        // <= 2^53 * 2^ulp.
        int count_bits = 0;
        while ((std::size_t{1} << count_bits) < count) {
            ++count_bits;
        }
        const bool order_free =
            count_bits + largest_exponent[0] + 1 <= 53 + smallest_ulp[0];
        if (!order_free) {
            total = 0.0;
            for (std::size_t index = 0; index < count; ++index) {
                total += static_cast<double>(scales[index]);
            }
        }
    }
    const float offset =
        static_cast<float>(total / static_cast<double>(count));
    *offset_out = offset;
    if (!isfinite(offset)) {
        atomicOr(status, kOffsetOverflow);
    }
}

// One wavefront per group of second-level-block scales.
__global__ __launch_bounds__(256) void scale_encode_kernel(
    const float* __restrict__ scales, std::size_t count, unsigned group_shift,
    std::size_t group_count, const float* __restrict__ offset_pointer,
    std::uint8_t* __restrict__ scale_codes, float* __restrict__ second_level
) {
#pragma clang fp contract(off)
    const float offset = *offset_pointer;
    const std::size_t waves_per_grid =
        static_cast<std::size_t>(gridDim.x) * (blockDim.x / 64);
    const unsigned lane = threadIdx.x % 64;
    const std::size_t group_size = std::size_t{1} << group_shift;
    for (std::size_t group =
             static_cast<std::size_t>(blockIdx.x) * (blockDim.x / 64) +
             threadIdx.x / 64;
         group < group_count; group += waves_per_grid) {
        const std::size_t begin = group << group_shift;
        const std::size_t end =
            begin + group_size < count ? begin + group_size : count;
        float absmax = 0.0F;
        for (std::size_t index = begin + lane; index < end; index += 64) {
            const float distance = fabsf(scales[index] - offset);
            absmax = absmax < distance ? distance : absmax;
        }
#pragma unroll
        for (int step = 32; step >= 1; step /= 2) {
            const float other = __shfl_xor(absmax, step, 64);
            absmax = absmax < other ? other : absmax;
        }
        if (lane == 0) {
            second_level[group] = absmax;
        }
        for (std::size_t index = begin + lane; index < end; index += 64) {
            unsigned code = 128;
            if (absmax != 0.0F) {
                const float normalized = (scales[index] - offset) / absmax;
                const float scaled = normalized * 127.0F;
                const float rounded = scaled >= 0.0F ? floorf(scaled + 0.5F)
                                                     : ceilf(scaled - 0.5F);
                int centered = static_cast<int>(rounded);
                centered =
                    centered < -127 ? -127 : (centered > 127 ? 127 : centered);
                code = static_cast<unsigned>(centered + 128);
            }
            scale_codes[index] = static_cast<std::uint8_t>(code);
        }
    }
}

unsigned grid_for(std::size_t items, std::size_t per_block) {
    constexpr std::size_t kMaxBlocks = 256 * 32;
    std::size_t blocks = (items + per_block - 1) / per_block;
    if (blocks == 0) {
        blocks = 1;
    }
    return static_cast<unsigned>(blocks < kMaxBlocks ? blocks : kMaxBlocks);
}

}  // namespace

void launch_quantize(const QuantizeProblem& p, hipStream_t stream) {
    const std::size_t block_count =
        (p.element_count + (std::size_t{1} << p.block_shift) - 1) >>
        p.block_shift;
    block_scale_kernel<<<grid_for(block_count, 4), 256, 0, stream>>>(
        p.values, p.element_count, p.block_shift, block_count, p.fp32_scales,
        p.status);
    encode_kernel<<<grid_for((p.element_count + 7) / 8, 256), 256, 0,
                    stream>>>(p.values, p.element_count, p.block_shift,
                              p.fp32_scales, p.codes);
    if (p.scale_codes == nullptr) {
        return;
    }
    scale_mean_kernel<<<1, kMeanThreads, 0, stream>>>(
        p.fp32_scales, block_count, p.offset, p.status);
    const std::size_t group_count =
        (block_count + (std::size_t{1} << p.second_level_shift) - 1) >>
        p.second_level_shift;
    scale_encode_kernel<<<grid_for(group_count, 4), 256, 0, stream>>>(
        p.fp32_scales, block_count, p.second_level_shift, group_count,
        p.offset, p.scale_codes, p.second_level);
}

}  // namespace rthip
