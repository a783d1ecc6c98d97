// Stand-alone statement of the slice of riftco-transformer's backend interface
// that the packed NF4 linear path touches, for building and testing the `hip`
// adapter outside the reference tree.  Names, signatures, value semantics and
// error behaviour match the reference so that hip_adapter.cpp compiles
// unchanged against either this header or the reference's own
// (define RIFTCO_TRANSFORMER_IN_TREE for the latter).
//
// What each declaration mirrors (paths under /root/reference):
//   ExecutionBackend ............ include/riftco_transformer/core/backend.hpp:13-18
//                                 (+ Hip = 4, appended; 0..3 keep their values)
//   TensorStorage ............... src/core/backend/storage.hpp:15-31
//   Nf4ScaleEncoding, Nf4ScaleStorageData, Nf4ScaleStorageView,
//   decode_nf4_block_scale, nf4_scale_payload_bytes,
//   QuantizedWeightStorage ...... src/core/backend/nn/quantized_linear/storage.hpp:13-108
//   QuantizedLinearDimensions and the two request structs
//                                 src/core/backend/nn/quantized_linear/contracts.hpp:10-34
//   StorageCapability ........... src/core/backend/adapter.hpp:33-46
//   QuantizedStorageCapability,
//   QuantizedLinearCapability ... src/core/backend/nn/quantized_linear/capability.hpp:16-50
//   BackendAdapter .............. src/core/backend/adapter.hpp:57-80, restricted
//                                 to the capability bases named above
#pragma once

#include <cstddef>
#include <cstdint>
#include <limits>
#include <memory>
#include <span>
#include <stdexcept>
#include <string_view>
#include <vector>

namespace riftco_transformer {

enum class ExecutionBackend : std::uint8_t {
    Cpu = 0,
    Metal = 1,
    Cuda = 2,
    Tpu = 3,
    Hip = 4,
};

namespace backend_detail {

class TensorStorage {
public:
    virtual ~TensorStorage() = default;
    [[nodiscard]] virtual ExecutionBackend backend() const noexcept = 0;
    [[nodiscard]] virtual std::size_t size() const noexcept = 0;
    [[nodiscard]] virtual std::span<float> data() noexcept = 0;
    [[nodiscard]] virtual std::span<const float> data() const noexcept = 0;
    [[nodiscard]] virtual void* native_handle() noexcept = 0;
    [[nodiscard]] virtual const void* native_handle() const noexcept = 0;
    [[nodiscard]] virtual std::unique_ptr<TensorStorage> clone() const = 0;
};

enum class Nf4ScaleEncoding : std::uint8_t {
    Float32 = 0,
    DoubleQuantizedUInt8 = 1,
};

struct Nf4ScaleStorageData {
    Nf4ScaleEncoding encoding = Nf4ScaleEncoding::Float32;
    std::vector<float> fp32_scales;
    std::vector<std::uint8_t> quantized_scales;
    std::vector<float> second_level_scales;
    std::size_t second_level_block_size = 0;
    float offset = 0.0F;
};

struct Nf4ScaleStorageView {
    Nf4ScaleEncoding encoding = Nf4ScaleEncoding::Float32;
    std::span<const float> fp32_scales;
    std::span<const std::uint8_t> quantized_scales;
    std::span<const float> second_level_scales;
    std::size_t second_level_block_size = 0;
    float offset = 0.0F;

    [[nodiscard]] std::size_t scale_count() const noexcept {
        return encoding == Nf4ScaleEncoding::Float32 ? fp32_scales.size()
                                                     : quantized_scales.size();
    }
};

// offset + second_level[index / C] * ((code - 128) / 127), clamped to
// [0, FLT_MAX]; three separately rounded fp32 operations.
[[nodiscard]] inline float decode_nf4_block_scale(
    const Nf4ScaleStorageView& scales, std::size_t index
) noexcept {
    if (scales.encoding == Nf4ScaleEncoding::Float32) {
        return scales.fp32_scales[index];
    }
    const int centered = static_cast<int>(scales.quantized_scales[index]) - 128;
    const float factor = static_cast<float>(centered) / 127.0F;
    const float delta =
        scales.second_level_scales[index / scales.second_level_block_size] *
        factor;
    constexpr float kMax = std::numeric_limits<float>::max();
    if (delta > 0.0F && scales.offset > kMax - delta) {
        return kMax;
    }
    const float value = scales.offset + delta;
    return value > 0.0F ? value : 0.0F;
}

[[nodiscard]] inline std::size_t nf4_scale_payload_bytes(
    const Nf4ScaleStorageView& scales
) noexcept {
    if (scales.encoding == Nf4ScaleEncoding::Float32) {
        return scales.fp32_scales.size() * sizeof(float);
    }
    return scales.quantized_scales.size() +
           scales.second_level_scales.size() * sizeof(float) + sizeof(float);
}

class QuantizedWeightStorage {
public:
    virtual ~QuantizedWeightStorage() = default;
    [[nodiscard]] virtual ExecutionBackend backend() const noexcept = 0;
    [[nodiscard]] virtual std::span<const std::uint8_t> packed_codes()
        const noexcept = 0;
    [[nodiscard]] virtual Nf4ScaleStorageView scale_storage()
        const noexcept = 0;
    [[nodiscard]] virtual const void* packed_codes_native_handle()
        const noexcept = 0;
    [[nodiscard]] virtual const void* primary_scales_native_handle()
        const noexcept = 0;
    [[nodiscard]] virtual const void* secondary_scales_native_handle()
        const noexcept = 0;
    [[nodiscard]] virtual std::size_t resident_payload_bytes()
        const noexcept = 0;
};

struct QuantizedLinearDimensions {
    std::size_t rows;
    std::size_t input_width;
    std::size_t output_width;
    std::size_t block_size;
};

struct QuantizedLinearForwardRequest {
    const TensorStorage& input;
    const QuantizedWeightStorage& weight;
    TensorStorage& output;
    QuantizedLinearDimensions dimensions;
};

struct QuantizedLinearInputBackwardRequest {
    const TensorStorage& upstream;
    const QuantizedWeightStorage& weight;
    TensorStorage& input_gradient;
    QuantizedLinearDimensions dimensions;
};

class StorageCapability {
public:
    virtual ~StorageCapability() = default;
    [[nodiscard]] virtual std::unique_ptr<TensorStorage> make_storage(
        std::size_t element_count, float fill_value) const = 0;
    [[nodiscard]] virtual std::unique_ptr<TensorStorage> make_storage(
        std::vector<float> values) const = 0;
};

class QuantizedStorageCapability {
public:
    virtual ~QuantizedStorageCapability() = default;
    [[nodiscard]] virtual std::unique_ptr<QuantizedWeightStorage>
    make_nf4_weight_storage(std::vector<std::uint8_t>,
                            Nf4ScaleStorageData) const {
        throw std::runtime_error(
            "NF4 weight storage is unsupported by this execution backend");
    }
};

class QuantizedLinearCapability {
public:
    virtual ~QuantizedLinearCapability() = default;
    virtual void quantized_linear_forward(
        const QuantizedLinearForwardRequest&) const {
        throw std::runtime_error(
            "quantized linear is unsupported by this execution backend");
    }
    virtual void quantized_linear_input_backward(
        const QuantizedLinearInputBackwardRequest&) const {
        throw std::runtime_error(
            "quantized linear backward is unsupported by this execution "
            "backend");
    }
};

class BackendAdapter : public StorageCapability,
                       public QuantizedStorageCapability,
                       public QuantizedLinearCapability {
public:
    ~BackendAdapter() override = default;
    [[nodiscard]] virtual std::string_view name() const noexcept = 0;
    [[nodiscard]] virtual bool is_available() const noexcept = 0;
    [[nodiscard]] virtual std::string_view unavailability_reason()
        const noexcept {
        return {};
    }
};

}  // namespace backend_detail
}  // namespace riftco_transformer
