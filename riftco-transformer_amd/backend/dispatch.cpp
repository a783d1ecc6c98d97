#include "dispatch.hpp"

#include <cmath>
#include <initializer_list>
#include <limits>
#include <stdexcept>
#include <string>

namespace riftco_transformer {
namespace backend_detail {
namespace {

// A recognised backend that this stand-alone build does not carry; keeps
// numeric identities 0..3 meaningful (names, "unavailable" errors) without
// pretending to implement them.
class AbsentBackendAdapter final : public BackendAdapter {
public:
    explicit AbsentBackendAdapter(std::string_view name) noexcept
        : name_(name) {}
    [[nodiscard]] std::string_view name() const noexcept override {
        return name_;
    }
    [[nodiscard]] bool is_available() const noexcept override { return false; }
    [[nodiscard]] std::string_view unavailability_reason()
        const noexcept override {
        return "support was not compiled into this build";
    }
    [[nodiscard]] std::unique_ptr<TensorStorage> make_storage(
        std::size_t, float) const override {
        unavailable();
    }
    [[nodiscard]] std::unique_ptr<TensorStorage> make_storage(
        std::vector<float>) const override {
        unavailable();
    }

private:
    [[noreturn]] void unavailable() const {
        throw std::runtime_error(std::string(name_) +
                                 " execution backend is unavailable");
    }
    std::string_view name_;
};

const BackendAdapter& require_backend_adapter(ExecutionBackend backend) {
    const BackendAdapter* adapter = find_backend_adapter(backend);
    if (adapter == nullptr) {
        throw std::invalid_argument("unknown execution backend");
    }
    if (!adapter->is_available()) {
        std::string message =
            std::string(adapter->name()) + " execution backend is unavailable";
        const std::string_view reason = adapter->unavailability_reason();
        if (!reason.empty()) {
            message += ": ";
            message += reason;
        }
        throw std::runtime_error(message);
    }
    return *adapter;
}

std::size_t checked_product(std::initializer_list<std::size_t> factors) {
    std::size_t result = 1;
    for (const std::size_t factor : factors) {
        if (factor == 0) {
            throw std::invalid_argument(
                "quantized linear dimensions must be positive");
        }
        if (result > std::numeric_limits<std::size_t>::max() / factor) {
            throw std::overflow_error(
                "quantized linear size exceeds addressable storage");
        }
        result *= factor;
    }
    return result;
}

std::size_t checked_payload_bytes(std::size_t packed_code_count,
                                  const Nf4ScaleStorageView& scales) {
    constexpr std::size_t kMax = std::numeric_limits<std::size_t>::max();
    const bool nested =
        scales.encoding == Nf4ScaleEncoding::DoubleQuantizedUInt8;
    const std::size_t float_count = nested ? scales.second_level_scales.size()
                                           : scales.fp32_scales.size();
    if (float_count > kMax / sizeof(float)) {
        throw std::overflow_error(
            "NF4 scale storage exceeds addressable memory");
    }
    std::size_t scale_bytes = float_count * sizeof(float);
    if (nested) {
        if (scale_bytes > kMax - sizeof(float) ||
            scales.quantized_scales.size() >
                kMax - sizeof(float) - scale_bytes) {
            throw std::overflow_error(
                "double-quantized NF4 scale storage exceeds addressable "
                "memory");
        }
        scale_bytes += sizeof(float) + scales.quantized_scales.size();
    }
    if (packed_code_count > kMax - scale_bytes) {
        throw std::overflow_error(
            "NF4 weight storage exceeds addressable memory");
    }
    return packed_code_count + scale_bytes;
}

bool nf4_block_size_supported(std::size_t block_size) noexcept {
    // src/core/quantization/nf4.cpp:39-53
    for (std::size_t candidate = 32; candidate <= 4096; candidate *= 2) {
        if (block_size == candidate) {
            return true;
        }
    }
    return false;
}

void require_finite_nonnegative(std::span<const float> scales) {
    for (const float scale : scales) {
        if (!std::isfinite(scale) || scale < 0.0F) {
            throw std::invalid_argument(
                "NF4 block scales must be finite and non-negative");
        }
    }
}

// `deep` covers the per-element checks (O(#blocks)); the representation checks
// always run.
void require_scale_storage(const Nf4ScaleStorageView& scales,
                           std::size_t expected_count, bool deep) {
    switch (scales.encoding) {
    case Nf4ScaleEncoding::Float32:
        if (scales.fp32_scales.size() != expected_count ||
            !scales.quantized_scales.empty() ||
            !scales.second_level_scales.empty() ||
            scales.second_level_block_size != 0 || scales.offset != 0.0F) {
            throw std::invalid_argument(
                "legacy NF4 scale storage has an invalid representation");
        }
        if (deep) {
            require_finite_nonnegative(scales.fp32_scales);
        }
        return;
    case Nf4ScaleEncoding::DoubleQuantizedUInt8:
        if (!scales.fp32_scales.empty() ||
            scales.quantized_scales.size() != expected_count ||
            scales.second_level_block_size == 0 ||
            !nf4_block_size_supported(scales.second_level_block_size) ||
            !std::isfinite(scales.offset) || scales.offset < 0.0F) {
            throw std::invalid_argument(
                "double-quantized NF4 scale storage has an invalid "
                "representation");
        }
        if (scales.second_level_scales.size() !=
            1 + (expected_count - 1) / scales.second_level_block_size) {
            throw std::invalid_argument(
                "double-quantized NF4 second-level scale count is invalid");
        }
        if (deep) {
            require_finite_nonnegative(scales.second_level_scales);
            for (std::size_t index = 0; index < expected_count; ++index) {
                if (!std::isfinite(decode_nf4_block_scale(scales, index))) {
                    throw std::invalid_argument(
                        "double-quantized NF4 scale reconstruction is "
                        "nonfinite");
                }
            }
        }
        return;
    }
    throw std::invalid_argument("unknown NF4 scale encoding");
}

bool tensor_storage_aliases(const TensorStorage& left,
                            const TensorStorage& right) noexcept {
    if (&left == &right) {
        return true;
    }
    const void* left_handle = left.native_handle();
    return left_handle != nullptr && left_handle == right.native_handle();
}

void require_tensor_storage(const TensorStorage& storage,
                            ExecutionBackend backend,
                            std::size_t expected_size) {
    if (storage.backend() != backend) {
        throw std::invalid_argument(
            "quantized linear tensor storage does not match its backend");
    }
    // size() is the contract here; the reference also compares
    // data().size(), which for hip storage would force a device read-back of
    // a tensor nobody on the host is going to look at.
    if (storage.size() != expected_size) {
        throw std::logic_error(
            "quantized linear tensor storage size does not match dimensions");
    }
}

void require_weight_separate_from_output(const QuantizedWeightStorage& weight,
                                         const TensorStorage& output) {
    const void* handle = output.native_handle();
    if (handle == nullptr) {
        return;
    }
    if (handle == weight.packed_codes_native_handle() ||
        handle == weight.primary_scales_native_handle() ||
        handle == weight.secondary_scales_native_handle()) {
        throw std::invalid_argument(
            "quantized linear weight and output storage must not alias");
    }
}

void require_weight_storage(const QuantizedWeightStorage& weight,
                            ExecutionBackend backend,
                            const QuantizedLinearDimensions& dimensions) {
    if (weight.backend() != backend) {
        throw std::invalid_argument(
            "quantized linear weight storage does not match its backend");
    }
    if (dimensions.block_size == 0) {
        throw std::invalid_argument(
            "NF4 block size must be greater than zero");
    }
    const std::size_t logical_size =
        checked_product({dimensions.output_width, dimensions.input_width});
    const std::size_t expected_codes = logical_size / 2 + logical_size % 2;
    const std::size_t expected_scales =
        1 + (logical_size - 1) / dimensions.block_size;
    if (weight.packed_codes().size() != expected_codes) {
        throw std::logic_error(
            "NF4 packed-code count does not match weight dimensions");
    }
    // Immutable hip storage remembers a successful deep validation.
    const auto* memo = dynamic_cast<const ScaleValidationMemo*>(&weight);
    const bool deep = memo == nullptr || !memo->scales_validated();
    const auto scales = weight.scale_storage();
    require_scale_storage(scales, expected_scales, deep);
    if (deep && memo != nullptr) {
        memo->mark_scales_validated();
    }
    if (weight.resident_payload_bytes() <
        checked_payload_bytes(expected_codes, scales)) {
        throw std::logic_error(
            "NF4 resident payload is smaller than its packed storage");
    }
}

void require_dimensions(const QuantizedLinearDimensions& dimensions) {
    static_cast<void>(checked_product(
        {dimensions.rows, dimensions.input_width, dimensions.output_width}));
    if (dimensions.block_size == 0) {
        throw std::invalid_argument(
            "NF4 block size must be greater than zero");
    }
}

}  // namespace

const BackendAdapter* find_backend_adapter(ExecutionBackend backend) noexcept {
    static const AbsentBackendAdapter cpu("cpu");
    static const AbsentBackendAdapter metal("metal");
    static const AbsentBackendAdapter cuda("cuda");
    static const AbsentBackendAdapter tpu("tpu");
    switch (static_cast<std::uint8_t>(backend)) {
    case 0: return &cpu;
    case 1: return &metal;
    case 2: return &cuda;
    case 3: return &tpu;
    case 4: return &hip_backend_adapter();
    default: return nullptr;
    }
}

std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::size_t element_count, float fill_value
) {
    auto storage = require_backend_adapter(backend).make_storage(
        element_count, fill_value);
    if (storage == nullptr || storage->backend() != backend ||
        storage->size() != element_count) {
        throw std::logic_error(
            "backend adapter returned invalid tensor storage");
    }
    return storage;
}

std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::vector<float> values
) {
    const std::size_t expected = values.size();
    auto storage =
        require_backend_adapter(backend).make_storage(std::move(values));
    if (storage == nullptr || storage->backend() != backend ||
        storage->size() != expected) {
        throw std::logic_error(
            "backend adapter returned invalid tensor storage");
    }
    return storage;
}

std::unique_ptr<QuantizedWeightStorage> make_nf4_weight_storage(
    ExecutionBackend backend, std::vector<std::uint8_t> packed_codes,
    Nf4ScaleStorageData scales
) {
    const BackendAdapter& adapter = require_backend_adapter(backend);
    if (packed_codes.empty()) {
        throw std::invalid_argument(
            "NF4 packed-code storage must not be empty");
    }
    const std::size_t packed_count = packed_codes.size();
    const Nf4ScaleStorageView input_view{
        scales.encoding,
        scales.fp32_scales,
        scales.quantized_scales,
        scales.second_level_scales,
        scales.second_level_block_size,
        scales.offset,
    };
    const std::size_t scale_count = input_view.scale_count();
    if (scale_count == 0) {
        throw std::invalid_argument("NF4 scale storage must not be empty");
    }
    // The one deep validation of this payload: here, on host vectors, before
    // anything is uploaded.
    require_scale_storage(input_view, scale_count, true);
    const std::size_t expected_payload =
        checked_payload_bytes(packed_count, input_view);
    const auto encoding = input_view.encoding;
    const auto second_level_count = input_view.second_level_scales.size();
    const auto second_level_block = input_view.second_level_block_size;
    const float offset = input_view.offset;

    auto storage = adapter.make_nf4_weight_storage(std::move(packed_codes),
                                                   std::move(scales));
    if (storage == nullptr) {
        throw std::logic_error(
            "backend adapter returned null NF4 weight storage");
    }
    const auto stored = storage->scale_storage();
    if (storage->backend() != backend ||
        storage->packed_codes().size() != packed_count ||
        stored.encoding != encoding || stored.scale_count() != scale_count ||
        stored.second_level_scales.size() != second_level_count ||
        stored.second_level_block_size != second_level_block ||
        stored.offset != offset ||
        storage->resident_payload_bytes() < expected_payload) {
        throw std::logic_error(
            "backend adapter returned invalid NF4 weight storage");
    }
    require_scale_storage(stored, scale_count, false);
    if (const auto* memo =
            dynamic_cast<const ScaleValidationMemo*>(storage.get())) {
        memo->mark_scales_validated();
    }
    return storage;
}

void dispatch_quantized_linear_forward(
    ExecutionBackend backend, const QuantizedLinearForwardRequest& request
) {
    const BackendAdapter& adapter = require_backend_adapter(backend);
    require_dimensions(request.dimensions);
    const std::size_t input_size = checked_product(
        {request.dimensions.rows, request.dimensions.input_width});
    const std::size_t output_size = checked_product(
        {request.dimensions.rows, request.dimensions.output_width});
    require_tensor_storage(request.input, backend, input_size);
    require_tensor_storage(request.output, backend, output_size);
    require_weight_storage(request.weight, backend, request.dimensions);
    if (tensor_storage_aliases(request.input, request.output)) {
        throw std::invalid_argument(
            "quantized linear input and output must not alias");
    }
    require_weight_separate_from_output(request.weight, request.output);
    adapter.quantized_linear_forward(request);
}

void dispatch_quantized_linear_input_backward(
    ExecutionBackend backend,
    const QuantizedLinearInputBackwardRequest& request
) {
    const BackendAdapter& adapter = require_backend_adapter(backend);
    require_dimensions(request.dimensions);
    const std::size_t upstream_size = checked_product(
        {request.dimensions.rows, request.dimensions.output_width});
    const std::size_t gradient_size = checked_product(
        {request.dimensions.rows, request.dimensions.input_width});
    require_tensor_storage(request.upstream, backend, upstream_size);
    require_tensor_storage(request.input_gradient, backend, gradient_size);
    require_weight_storage(request.weight, backend, request.dimensions);
    if (tensor_storage_aliases(request.upstream, request.input_gradient)) {
        throw std::invalid_argument(
            "quantized linear upstream and input gradient must not alias");
    }
    require_weight_separate_from_output(request.weight,
                                        request.input_gradient);
    adapter.quantized_linear_input_backward(request);
}

}  // namespace backend_detail

bool execution_backend_available(ExecutionBackend backend) noexcept {
    const auto* adapter = backend_detail::find_backend_adapter(backend);
    return adapter != nullptr && adapter->is_available();
}

std::string_view execution_backend_unavailability_reason(
    ExecutionBackend backend
) noexcept {
    const auto* adapter = backend_detail::find_backend_adapter(backend);
    if (adapter == nullptr || adapter->is_available()) {
        return {};
    }
    return adapter->unavailability_reason();
}

std::string_view execution_backend_name(ExecutionBackend backend) {
    const auto* adapter = backend_detail::find_backend_adapter(backend);
    if (adapter == nullptr) {
        throw std::invalid_argument("unknown execution backend");
    }
    return adapter->name();
}

}  // namespace riftco_transformer
