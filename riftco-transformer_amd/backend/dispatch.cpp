// Stand-alone registry and packed-NF4 dispatch for the `hip` adapter.
//
// What is contract here -- which conditions are rejected, in which order, with
// which exception type and message -- follows the reference dispatcher
// (src/core/backend/nn/quantized_linear/dispatch.cpp:18-370) and registry
// (src/core/backend/registry.cpp:83-141), because callers and tests observe
// it.  How it is done is this file's own: a call is described once
// (`LinearCall`, for both directions), its findings are data (`Finding`:
// exception kind + message) produced by small audit functions and thrown in
// one place, the weight's geometry is derived once per call, and the
// O(#blocks) pass over the scale values runs once per immutable weight
// (`ScaleValidationMemo`) instead of once per call.

#include "dispatch.hpp"

#include <array>
#include <cmath>
#include <limits>
#include <optional>
#include <stdexcept>
#include <string>

namespace riftco_transformer {
namespace backend_detail {
namespace {

// ---- findings ----------------------------------------------------------

enum class Kind { Argument, Logic, Overflow };

struct Finding {
    Kind kind;
    const char* message;
};

using Verdict = std::optional<Finding>;

[[noreturn]] void raise(const Finding& finding) {
    switch (finding.kind) {
    case Kind::Argument: throw std::invalid_argument(finding.message);
    case Kind::Overflow: throw std::overflow_error(finding.message);
    case Kind::Logic: break;
    }
    throw std::logic_error(finding.message);
}

void settle(const Verdict& verdict) {
    if (verdict) {
        raise(*verdict);
    }
}

constexpr Finding kNoDimensions{Kind::Argument,
                                "quantized linear dimensions must be positive"};
constexpr Finding kTooLarge{Kind::Overflow,
                            "quantized linear size exceeds addressable storage"};
constexpr Finding kNoBlockSize{Kind::Argument,
                               "NF4 block size must be greater than zero"};

// ---- sizes ---------------------------------------------------------------

// a * b, or the finding that says why not (zero factors are findings too:
// every product taken here is a tensor or weight extent).
Verdict multiply(std::size_t a, std::size_t b, std::size_t* product) {
    if (a == 0 || b == 0) {
        return kNoDimensions;
    }
    if (__builtin_mul_overflow(a, b, product)) {
        return kTooLarge;
    }
    return std::nullopt;
}

// Element counts a request implies.
struct Extents {
    std::size_t source = 0;   // rows x (input or output width)
    std::size_t target = 0;
    std::size_t weight = 0;   // output_width x input_width
    std::size_t code_bytes = 0;
    std::size_t blocks = 0;
};

// The bytes a scale storage occupies next to `code_bytes` of codes: fp32
// scales, or scale codes + second-level scales + the offset.
Verdict payload_bytes(std::size_t code_bytes, const Nf4ScaleStorageView& scales,
                      std::size_t* bytes) {
    const bool nested =
        scales.encoding == Nf4ScaleEncoding::DoubleQuantizedUInt8;
    const std::size_t floats = nested ? scales.second_level_scales.size()
                                      : scales.fp32_scales.size();
    std::size_t total = 0;
    if (__builtin_mul_overflow(floats, sizeof(float), &total)) {
        return Finding{Kind::Overflow,
                       "NF4 scale storage exceeds addressable memory"};
    }
    if (nested &&
        (__builtin_add_overflow(total, sizeof(float), &total) ||
         __builtin_add_overflow(total, scales.quantized_scales.size(),
                                &total))) {
        return Finding{Kind::Overflow,
                       "double-quantized NF4 scale storage exceeds "
                       "addressable memory"};
    }
    if (__builtin_add_overflow(total, code_bytes, &total)) {
        return Finding{Kind::Overflow,
                       "NF4 weight storage exceeds addressable memory"};
    }
    *bytes = total;
    return std::nullopt;
}

// ---- scale storage -------------------------------------------------------

bool power_of_two_block(std::size_t size) noexcept {
    // the format's block sizes: 32, 64, ..., 4096
    // (src/core/quantization/nf4.cpp:39-53)
    return size >= 32 && size <= 4096 && (size & (size - 1)) == 0;
}

bool sound(float scale) noexcept { return std::isfinite(scale) && scale >= 0.0F; }

constexpr Finding kBadScaleValue{
    Kind::Argument, "NF4 block scales must be finite and non-negative"};

// Which arrays are present, how long, and the scalar fields: O(1).
Verdict audit_scale_layout(const Nf4ScaleStorageView& scales,
                           std::size_t expected) {
    const std::size_t groups =
        scales.second_level_block_size == 0
            ? 0
            : 1 + (expected - 1) / scales.second_level_block_size;
    switch (scales.encoding) {
    case Nf4ScaleEncoding::Float32: {
        const bool plain = scales.fp32_scales.size() == expected &&
                           scales.quantized_scales.empty() &&
                           scales.second_level_scales.empty() &&
                           scales.second_level_block_size == 0 &&
                           scales.offset == 0.0F;
        if (!plain) {
            return Finding{Kind::Argument,
                           "legacy NF4 scale storage has an invalid "
                           "representation"};
        }
        return std::nullopt;
    }
    case Nf4ScaleEncoding::DoubleQuantizedUInt8: {
        const bool nested =
            scales.fp32_scales.empty() &&
            scales.quantized_scales.size() == expected &&
            power_of_two_block(scales.second_level_block_size) &&
            sound(scales.offset);
        if (!nested) {
            return Finding{Kind::Argument,
                           "double-quantized NF4 scale storage has an "
                           "invalid representation"};
        }
        if (scales.second_level_scales.size() != groups) {
            return Finding{Kind::Argument,
                           "double-quantized NF4 second-level scale count "
                           "is invalid"};
        }
        return std::nullopt;
    }
    }
    return Finding{Kind::Argument, "unknown NF4 scale encoding"};
}

// Every stored value and, for nested scales, every reconstruction:
// O(#blocks).  Only meaningful after audit_scale_layout has passed.
Verdict audit_scale_values(const Nf4ScaleStorageView& scales,
                           std::size_t expected) {
    const bool nested =
        scales.encoding == Nf4ScaleEncoding::DoubleQuantizedUInt8;
    for (const float value :
         nested ? scales.second_level_scales : scales.fp32_scales) {
        if (!sound(value)) {
            return kBadScaleValue;
        }
    }
    if (nested) {
        for (std::size_t block = 0; block < expected; ++block) {
            if (!std::isfinite(decode_nf4_block_scale(scales, block))) {
                return Finding{Kind::Argument,
                               "double-quantized NF4 scale reconstruction "
                               "is nonfinite"};
            }
        }
    }
    return std::nullopt;
}

// ---- one call, either direction -------------------------------------------

struct LinearCall {
    const TensorStorage& source;  // x, or the upstream gradient
    const TensorStorage& target;  // y, or the input gradient
    const QuantizedWeightStorage& weight;
    const QuantizedLinearDimensions& dimensions;
    std::size_t source_width;
    std::size_t target_width;
    const char* alias_message;
};

Verdict measure(const LinearCall& call, Extents* extents) {
    const QuantizedLinearDimensions& d = call.dimensions;
    // all three together first, as the reference's require_dimensions does
    std::size_t all = 0;
    if (Verdict bad = multiply(d.rows, d.input_width, &all)) {
        return bad;
    }
    if (Verdict bad = multiply(all, d.output_width, &all)) {
        return bad;
    }
    if (d.block_size == 0) {
        return kNoBlockSize;
    }
    if (Verdict bad = multiply(d.rows, call.source_width, &extents->source)) {
        return bad;
    }
    if (Verdict bad = multiply(d.rows, call.target_width, &extents->target)) {
        return bad;
    }
    if (Verdict bad =
            multiply(d.output_width, d.input_width, &extents->weight)) {
        return bad;
    }
    extents->code_bytes = extents->weight / 2 + extents->weight % 2;
    extents->blocks = 1 + (extents->weight - 1) / d.block_size;
    return std::nullopt;
}

Verdict audit_tensor(const TensorStorage& storage, ExecutionBackend backend,
                     std::size_t elements) {
    if (storage.backend() != backend) {
        return Finding{Kind::Argument,
                       "quantized linear tensor storage does not match its "
                       "backend"};
    }
    // size() is the contract; the reference also compares data().size(),
    // which for hip storage would force a device read-back of a tensor that
    // nobody on the host is going to look at.
    if (storage.size() != elements) {
        return Finding{Kind::Logic,
                       "quantized linear tensor storage size does not match "
                       "dimensions"};
    }
    return std::nullopt;
}

Verdict audit_weight(const QuantizedWeightStorage& weight,
                     ExecutionBackend backend, const Extents& extents) {
    if (weight.backend() != backend) {
        return Finding{Kind::Argument,
                       "quantized linear weight storage does not match its "
                       "backend"};
    }
    if (weight.packed_codes().size() != extents.code_bytes) {
        return Finding{Kind::Logic,
                       "NF4 packed-code count does not match weight "
                       "dimensions"};
    }
    const Nf4ScaleStorageView scales = weight.scale_storage();
    if (Verdict bad = audit_scale_layout(scales, extents.blocks)) {
        return bad;
    }
    // An immutable weight whose values have been read once needs no second
    // reading.
    const auto* memo = dynamic_cast<const ScaleValidationMemo*>(&weight);
    if (memo == nullptr || !memo->scales_validated()) {
        if (Verdict bad = audit_scale_values(scales, extents.blocks)) {
            return bad;
        }
        if (memo != nullptr) {
            memo->mark_scales_validated();
        }
    }
    std::size_t logical = 0;
    if (Verdict bad = payload_bytes(extents.code_bytes, scales, &logical)) {
        return bad;
    }
    if (weight.resident_payload_bytes() < logical) {
        return Finding{Kind::Logic,
                       "NF4 resident payload is smaller than its packed "
                       "storage"};
    }
    return std::nullopt;
}

bool same_memory(const TensorStorage& a, const TensorStorage& b) noexcept {
    const void* const handle = a.native_handle();
    return &a == &b || (handle != nullptr && handle == b.native_handle());
}

bool writes_into(const TensorStorage& target,
                 const QuantizedWeightStorage& weight) noexcept {
    const void* const handle = target.native_handle();
    if (handle == nullptr) {
        return false;
    }
    const std::array<const void*, 3> arrays{
        weight.packed_codes_native_handle(),
        weight.primary_scales_native_handle(),
        weight.secondary_scales_native_handle()};
    for (const void* array : arrays) {
        if (array == handle) {
            return true;
        }
    }
    return false;
}

Verdict vet(const LinearCall& call, ExecutionBackend backend) {
    Extents extents;
    if (Verdict bad = measure(call, &extents)) {
        return bad;
    }
    if (Verdict bad = audit_tensor(call.source, backend, extents.source)) {
        return bad;
    }
    if (Verdict bad = audit_tensor(call.target, backend, extents.target)) {
        return bad;
    }
    if (Verdict bad = audit_weight(call.weight, backend, extents)) {
        return bad;
    }
    if (same_memory(call.source, call.target)) {
        return Finding{Kind::Argument, call.alias_message};
    }
    if (writes_into(call.target, call.weight)) {
        return Finding{Kind::Argument,
                       "quantized linear weight and output storage must not "
                       "alias"};
    }
    return std::nullopt;
}

// ---- registry --------------------------------------------------------------

// A recognised backend that this stand-alone build does not carry: keeps the
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
        refuse();
    }
    [[nodiscard]] std::unique_ptr<TensorStorage> make_storage(
        std::vector<float>) const override {
        refuse();
    }

private:
    [[noreturn]] void refuse() const {
        throw std::runtime_error(std::string(name_) +
                                 " execution backend is unavailable");
    }
    std::string_view name_;
};

// The adapter of an available backend; otherwise the reference's two
// errors: unknown identity, or "<name> execution backend is unavailable[:
// reason]".
const BackendAdapter& usable_adapter(ExecutionBackend backend) {
    const BackendAdapter* const adapter = find_backend_adapter(backend);
    if (adapter == nullptr) {
        throw std::invalid_argument("unknown execution backend");
    }
    if (adapter->is_available()) {
        return *adapter;
    }
    std::string message(adapter->name());
    message += " execution backend is unavailable";
    if (const std::string_view reason = adapter->unavailability_reason();
        !reason.empty()) {
        message.append(": ").append(reason);
    }
    throw std::runtime_error(message);
}

template <typename Make>
std::unique_ptr<TensorStorage> checked_tensor(ExecutionBackend backend,
                                              std::size_t elements,
                                              Make&& make) {
    std::unique_ptr<TensorStorage> storage = make(usable_adapter(backend));
    if (storage == nullptr || storage->backend() != backend ||
        storage->size() != elements) {
        throw std::logic_error(
            "backend adapter returned invalid tensor storage");
    }
    return storage;
}

}  // namespace

const BackendAdapter* find_backend_adapter(ExecutionBackend backend) noexcept {
    static const AbsentBackendAdapter absent[4] = {
        AbsentBackendAdapter("cpu"), AbsentBackendAdapter("metal"),
        AbsentBackendAdapter("cuda"), AbsentBackendAdapter("tpu")};
    const auto identity = static_cast<std::uint8_t>(backend);
    if (identity < 4) {
        return &absent[identity];
    }
    return identity == 4 ? &hip_backend_adapter() : nullptr;
}

std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::size_t element_count, float fill_value
) {
    return checked_tensor(backend, element_count,
                          [&](const BackendAdapter& adapter) {
                              return adapter.make_storage(element_count,
                                                          fill_value);
                          });
}

std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::vector<float> values
) {
    const std::size_t elements = values.size();
    return checked_tensor(backend, elements,
                          [&](const BackendAdapter& adapter) {
                              return adapter.make_storage(std::move(values));
                          });
}

std::unique_ptr<QuantizedWeightStorage> make_nf4_weight_storage(
    ExecutionBackend backend, std::vector<std::uint8_t> packed_codes,
    Nf4ScaleStorageData scales
) {
    const BackendAdapter& adapter = usable_adapter(backend);
    if (packed_codes.empty()) {
        throw std::invalid_argument(
            "NF4 packed-code storage must not be empty");
    }
    // What the caller hands over, noted before the vectors are moved away.
    const Nf4ScaleStorageView given{
        scales.encoding,           scales.fp32_scales,
        scales.quantized_scales,   scales.second_level_scales,
        scales.second_level_block_size, scales.offset};
    const std::size_t code_bytes = packed_codes.size();
    const std::size_t blocks = given.scale_count();
    if (blocks == 0) {
        throw std::invalid_argument("NF4 scale storage must not be empty");
    }
    // The one full reading of this payload's scales: here, on host vectors,
    // before anything is uploaded.
    settle(audit_scale_layout(given, blocks));
    settle(audit_scale_values(given, blocks));
    std::size_t logical = 0;
    settle(payload_bytes(code_bytes, given, &logical));
    const Nf4ScaleEncoding encoding = given.encoding;
    const std::size_t groups = given.second_level_scales.size();
    const std::size_t group_size = given.second_level_block_size;
    const float offset = given.offset;

    std::unique_ptr<QuantizedWeightStorage> storage =
        adapter.make_nf4_weight_storage(std::move(packed_codes),
                                        std::move(scales));
    if (storage == nullptr) {
        throw std::logic_error(
            "backend adapter returned null NF4 weight storage");
    }
    // The adapter must hand back what it was given.
    const Nf4ScaleStorageView kept = storage->scale_storage();
    const bool faithful =
        storage->backend() == backend &&
        storage->packed_codes().size() == code_bytes &&
        kept.encoding == encoding && kept.scale_count() == blocks &&
        kept.second_level_scales.size() == groups &&
        kept.second_level_block_size == group_size && kept.offset == offset &&
        storage->resident_payload_bytes() >= logical;
    if (!faithful) {
        throw std::logic_error(
            "backend adapter returned invalid NF4 weight storage");
    }
    settle(audit_scale_layout(kept, blocks));
    if (const auto* memo =
            dynamic_cast<const ScaleValidationMemo*>(storage.get())) {
        memo->mark_scales_validated();  // same bytes as `given`
    } else {
        settle(audit_scale_values(kept, blocks));
    }
    return storage;
}

void dispatch_quantized_linear_forward(
    ExecutionBackend backend, const QuantizedLinearForwardRequest& request
) {
    const BackendAdapter& adapter = usable_adapter(backend);
    settle(vet(LinearCall{request.input, request.output, request.weight,
                          request.dimensions, request.dimensions.input_width,
                          request.dimensions.output_width,
                          "quantized linear input and output must not alias"},
               backend));
    adapter.quantized_linear_forward(request);
}

void dispatch_quantized_linear_input_backward(
    ExecutionBackend backend,
    const QuantizedLinearInputBackwardRequest& request
) {
    const BackendAdapter& adapter = usable_adapter(backend);
    settle(vet(LinearCall{request.upstream, request.input_gradient,
                          request.weight, request.dimensions,
                          request.dimensions.output_width,
                          request.dimensions.input_width,
                          "quantized linear upstream and input gradient "
                          "must not alias"},
               backend));
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
    const bool has_reason = adapter != nullptr && !adapter->is_available();
    return has_reason ? adapter->unavailability_reason() : std::string_view{};
}

std::string_view execution_backend_name(ExecutionBackend backend) {
    if (const auto* adapter = backend_detail::find_backend_adapter(backend)) {
        return adapter->name();
    }
    throw std::invalid_argument("unknown execution backend");
}

}  // namespace riftco_transformer
