// The content rules of a canonical packed NF4 payload, checked where the
// payload lives: require_canonical_payload of the reference
// (src/core/quantization/quantized_weight.cpp:102-174 under /root/reference)
// without its array-length checks, which need no device.
//
//   1  an unused high nibble (odd element count) must be zero
//   2  second-level scales must be finite and non-negative
//   3  every decoded block scale must be finite and non-negative
//   4  a block whose fp32 scale is zero must hold code 7 only (nested scales
//      may round a small scale to zero; their codes stay as they are)
//
// The reference walks the blocks in order and stops at the first that breaks
// rule 3 or 4, so which of the two it reports depends on the lowest offending
// block: each rule keeps the minimum block index that breaks it.

#include "kernels.hpp"
#include "nf4_decode.hpp"

namespace rthip {
namespace {

constexpr unsigned long long kNoBlock = ~0ULL;

__global__ void check_reset_kernel(unsigned long long* words) {
    if (threadIdx.x == 0) {
        words[0] = 0;         // bit 0: rule 1, bit 1: rule 2
        words[1] = kNoBlock;  // lowest block breaking rule 3
        words[2] = kNoBlock;  // lowest block breaking rule 4
    }
}

__device__ __forceinline__ bool valid_scale(float scale) {
    return isfinite(scale) && !(scale < 0.0F);
}

// True if elements [begin, end) all have code 7.  begin is even (block sizes
// are); end is odd only at the end of a weight with an odd element count.
__device__ bool all_zero_codes(const std::uint8_t* __restrict__ codes,
                               std::size_t begin, std::size_t end) {
    std::size_t byte = begin / 2;
    const std::size_t full_end = end / 2;  // bytes with both nibbles inside
    bool good = true;
    while (byte < full_end &&
           reinterpret_cast<std::uintptr_t>(codes + byte) % 4 != 0) {
        good = good && codes[byte] == 0x77U;
        ++byte;
    }
    for (; byte + 4 <= full_end; byte += 4) {
        good = good &&
               *reinterpret_cast<const unsigned*>(codes + byte) == 0x77777777U;
    }
    for (; byte < full_end; ++byte) {
        good = good && codes[byte] == 0x77U;
    }
    if (end % 2 != 0) {
        good = good && (codes[full_end] & 0x0FU) == 7U;
    }
    return good;
}

__global__ __launch_bounds__(256) void check_payload_kernel(
    Nf4WeightView weight, std::size_t element_count, unsigned block_shift,
    std::size_t block_count, std::size_t second_level_count,
    unsigned long long* __restrict__ words
) {
    const std::size_t stride =
        static_cast<std::size_t>(gridDim.x) * blockDim.x;
    const std::size_t first =
        static_cast<std::size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (first == 0 && element_count % 2 != 0 &&
        (weight.codes[element_count / 2] & 0xF0U) != 0U) {
        atomicOr(&words[0], 1ULL);
    }
    for (std::size_t group = first; group < second_level_count;
         group += stride) {
        if (!valid_scale(weight.secondary_scales[group])) {
            atomicOr(&words[0], 2ULL);
        }
    }
    for (std::size_t block = first; block < block_count; block += stride) {
        const float scale = load_block_scale_any(weight, block);
        if (!valid_scale(scale)) {
            atomicMin(&words[1], static_cast<unsigned long long>(block));
        } else if (scale == 0.0F && weight.encoding == 0) {
            const std::size_t begin = block << block_shift;
            const std::size_t size = std::size_t{1} << block_shift;
            const std::size_t end =
                begin + size < element_count ? begin + size : element_count;
            if (!all_zero_codes(weight.codes, begin, end)) {
                atomicMin(&words[2], static_cast<unsigned long long>(block));
            }
        }
    }
}

}  // namespace

void launch_check_payload(const Nf4WeightView& weight,
                          std::size_t element_count, unsigned block_shift,
                          std::size_t second_level_count,
                          unsigned long long* words, hipStream_t stream) {
    const std::size_t block_count =
        (element_count + (std::size_t{1} << block_shift) - 1) >> block_shift;
    std::size_t groups = (block_count + 255) / 256;
    if (groups > 256 * 16) {
        groups = 256 * 16;
    }
    if (groups == 0) {
        groups = 1;
    }
    check_reset_kernel<<<1, 64, 0, stream>>>(words);
    check_payload_kernel<<<static_cast<unsigned>(groups), 256, 0, stream>>>(
        weight, element_count, block_shift, block_count, second_level_count,
        words);
}

PayloadViolation classify_payload(const unsigned long long words[3]) {
    if ((words[0] & 1ULL) != 0ULL) {
        return PayloadViolation::UnusedNibble;
    }
    if ((words[0] & 2ULL) != 0ULL) {
        return PayloadViolation::SecondLevelScale;
    }
    if (words[1] == kNoBlock && words[2] == kNoBlock) {
        return PayloadViolation::None;
    }
    return words[1] < words[2] ? PayloadViolation::BlockScale
                               : PayloadViolation::ZeroBlockCode;
}

}  // namespace rthip
