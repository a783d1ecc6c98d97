#include "packed_state.hpp"

#include <algorithm>
#include <array>
#include <bit>
#include <cstring>
#include <limits>
#include <stdexcept>
#include <string>

namespace riftco_transformer::backend_detail {
namespace {

static_assert(std::endian::native == std::endian::little,
              "the packed state stores little-endian values and the payload "
              "arrays are copied as they are");
static_assert(sizeof(std::size_t) == sizeof(std::uint64_t));

constexpr std::array<std::uint8_t, 8> kMagic{'R', 'T', 'N', 'F',
                                             '4', 'S', '1', '\0'};
// Seven counts, offset, flags and two dimensions.
constexpr std::size_t kMinimumEntryBytes = 80;
constexpr std::size_t kSizeMax = std::numeric_limits<std::size_t>::max();

class Cursor {
public:
    explicit Cursor(std::span<const std::uint8_t> bytes) : rest_(bytes) {}

    std::span<const std::uint8_t> take(std::size_t count,
                                       const char* description) {
        if (count > rest_.size()) {
            throw std::invalid_argument(
                std::string("truncated packed model state: ") + description);
        }
        const auto result = rest_.first(count);
        rest_ = rest_.subspan(count);
        return result;
    }
    std::uint32_t u32(const char* description) {
        std::uint32_t value = 0;
        std::memcpy(&value, take(4, description).data(), 4);
        return value;
    }
    std::uint64_t u64(const char* description) {
        std::uint64_t value = 0;
        std::memcpy(&value, take(8, description).data(), 8);
        return value;
    }
    [[nodiscard]] std::size_t remaining() const noexcept {
        return rest_.size();
    }

private:
    std::span<const std::uint8_t> rest_;
};

void append_u32(std::vector<std::uint8_t>& output, std::uint32_t value) {
    std::uint8_t bytes[4];
    std::memcpy(bytes, &value, 4);
    output.insert(output.end(), bytes, bytes + 4);
}

void append_u64(std::vector<std::uint8_t>& output, std::uint64_t value) {
    std::uint8_t bytes[8];
    std::memcpy(bytes, &value, 8);
    output.insert(output.end(), bytes, bytes + 8);
}

bool block_size_supported(std::size_t block_size) noexcept {
    return block_size >= 32 && block_size <= 4096 &&
           std::has_single_bit(block_size);
}

void require_supported_block_size(std::size_t block_size) {
    if (!block_size_supported(block_size)) {
        throw std::invalid_argument(
            "NF4 block size must be one of "
            "32, 64, 128, 256, 512, 1024, 2048, or 4096");
    }
}

std::size_t ceil_divide(std::size_t value, std::size_t divisor) noexcept {
    return value / divisor + static_cast<std::size_t>(value % divisor != 0);
}

}  // namespace

std::vector<PackedWeightView> parse_packed_model_state(
    std::span<const std::uint8_t> bytes
) {
    Cursor cursor(bytes);
    const auto magic = cursor.take(kMagic.size(), "magic");
    if (!std::equal(magic.begin(), magic.end(), kMagic.begin())) {
        throw std::invalid_argument("unknown packed model state format");
    }
    const std::uint64_t count = cursor.u64("weight count");
    if (count == 0 || count > cursor.remaining() / kMinimumEntryBytes) {
        throw std::invalid_argument(
            "packed model state weight count is inconsistent with its size");
    }
    std::vector<PackedWeightView> result;
    result.reserve(count);
    for (std::uint64_t index = 0; index < count; ++index) {
        const std::uint64_t rank = cursor.u64("rank");
        if (rank != 2) {
            throw std::invalid_argument(
                "packed decoder Linear weights must have rank two");
        }
        PackedWeightView weight;
        weight.block_size = cursor.u64("block size");
        const std::uint64_t packed_count = cursor.u64("packed code count");
        const std::uint64_t block_scale_count =
            cursor.u64("block scale count");
        const std::uint64_t scale_code_count = cursor.u64("scale code count");
        const std::uint64_t second_scale_count =
            cursor.u64("second-level scale count");
        const std::uint64_t scale_block_size = cursor.u64("scale block size");
        const std::uint32_t offset_bits = cursor.u32("scale offset");
        const std::uint32_t flags = cursor.u32("flags");
        if (flags > 1U) {
            throw std::invalid_argument(
                "packed model state has unknown flags");
        }
        weight.double_quantized = flags == 1U;
        if ((!weight.double_quantized &&
             (scale_code_count != 0 || second_scale_count != 0 ||
              scale_block_size != 0 || offset_bits != 0U)) ||
            (weight.double_quantized &&
             (block_scale_count != 0 || scale_block_size == 0))) {
            throw std::invalid_argument(
                "packed model state has inconsistent NF4 scale metadata");
        }

        std::size_t required = rank * sizeof(std::uint64_t);
        const auto add_required = [&required](std::size_t value,
                                              std::size_t element_size) {
            if (value > (kSizeMax - required) / element_size) {
                throw std::overflow_error(
                    "packed model state entry size exceeds addressable "
                    "memory");
            }
            required += value * element_size;
        };
        add_required(packed_count, 1);
        add_required(block_scale_count, sizeof(float));
        add_required(scale_code_count, 1);
        add_required(second_scale_count, sizeof(float));
        if (required > cursor.remaining()) {
            throw std::invalid_argument(
                "truncated packed model state: weight payload");
        }

        for (std::uint64_t dimension = 0; dimension < rank; ++dimension) {
            weight.shape.push_back(cursor.u64("dimension"));
        }
        weight.packed_codes = cursor.take(packed_count, "packed codes");
        weight.block_scale_bytes =
            cursor.take(block_scale_count * sizeof(float), "block scale");
        if (weight.double_quantized) {
            weight.scale_codes = cursor.take(scale_code_count, "scale codes");
            weight.second_level_scale_bytes = cursor.take(
                second_scale_count * sizeof(float), "second-level scale");
            weight.scale_block_size = scale_block_size;
            weight.offset = std::bit_cast<float>(offset_bits);
        }
        result.push_back(std::move(weight));
    }
    if (cursor.remaining() != 0) {
        throw std::invalid_argument(
            "packed model state contains trailing bytes");
    }
    return result;
}

std::size_t require_payload_lengths(const PackedWeightView& weight) {
    require_supported_block_size(weight.block_size);
    std::size_t count = 1;
    for (const std::size_t dimension : weight.shape) {
        if (dimension == 0) {
            throw std::invalid_argument(
                "quantized weight dimensions must be greater than zero");
        }
        if (count > kSizeMax / dimension) {
            throw std::overflow_error(
                "quantized weight shape exceeds addressable size");
        }
        count *= dimension;
    }
    if (count > kSizeMax / sizeof(float)) {
        throw std::overflow_error(
            "quantized weight FP32 equivalent exceeds addressable size");
    }
    const std::size_t blocks = ceil_divide(count, weight.block_size);
    if (weight.packed_codes.size() != ceil_divide(count, 2)) {
        throw std::invalid_argument(
            "NF4 packed byte count does not match the weight shape");
    }
    const std::size_t block_scales =
        weight.block_scale_bytes.size() / sizeof(float);
    if (!weight.double_quantized) {
        if (block_scales != blocks) {
            throw std::invalid_argument(
                "NF4 scale count does not match the weight shape and block "
                "size");
        }
        return count;
    }
    if (block_scales != 0) {
        throw std::invalid_argument(
            "double-quantized NF4 payload must not retain FP32 block scales");
    }
    require_supported_block_size(weight.scale_block_size);
    if (weight.scale_codes.size() != blocks) {
        throw std::invalid_argument(
            "double-quantized NF4 scale-code count does not match the weight");
    }
    if (weight.second_level_scale_bytes.size() / sizeof(float) !=
        ceil_divide(blocks, weight.scale_block_size)) {
        throw std::invalid_argument(
            "double-quantized NF4 second-level scale count is invalid");
    }
    return count;
}

void append_packed_state_prologue(std::vector<std::uint8_t>& output,
                                  std::size_t weight_count) {
    output.insert(output.end(), kMagic.begin(), kMagic.end());
    append_u64(output, weight_count);
}

PackedWeightLayout append_packed_weight_header(
    std::vector<std::uint8_t>& output, std::span<const std::size_t> shape,
    std::size_t block_size, std::size_t packed_code_count,
    std::size_t block_scale_count, bool double_quantized,
    std::size_t scale_code_count, std::size_t second_level_scale_count,
    std::size_t scale_block_size, float offset
) {
    PackedWeightLayout layout;
    layout.header = output.size();
    append_u64(output, shape.size());
    append_u64(output, block_size);
    append_u64(output, packed_code_count);
    append_u64(output, block_scale_count);
    append_u64(output, double_quantized ? scale_code_count : 0);
    append_u64(output, double_quantized ? second_level_scale_count : 0);
    append_u64(output, double_quantized ? scale_block_size : 0);
    append_u32(output,
               std::bit_cast<std::uint32_t>(double_quantized ? offset : 0.0F));
    append_u32(output, double_quantized ? 1U : 0U);
    for (const std::size_t dimension : shape) {
        append_u64(output, dimension);
    }
    layout.packed_codes = output.size();
    layout.block_scales = layout.packed_codes + packed_code_count;
    layout.scale_codes =
        layout.block_scales + block_scale_count * sizeof(float);
    layout.second_level_scales =
        layout.scale_codes + (double_quantized ? scale_code_count : 0);
    layout.end =
        layout.second_level_scales +
        (double_quantized ? second_level_scale_count * sizeof(float) : 0);
    output.resize(layout.end, 0);
    return layout;
}

}  // namespace riftco_transformer::backend_detail
