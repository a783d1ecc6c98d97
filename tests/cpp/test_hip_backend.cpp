// Tests of the `hip` backend adapter through the same entry points the
// reference's own backend test uses (make_nf4_weight_storage,
// dispatch_quantized_linear_forward / _input_backward), against the CPU oracle.
// Counterparts (paths under /root/reference):
//   accelerator oracle loop, memory accounting, edge layout
//       tests/core/backend/test_quantized_linear_backend.cpp:382-453
//   unavailable backend must reject packed transfer   :472-499
//   backend identity / unknown ids
//       tests/core/backend/test_backend.cpp:172-240
//   byte-preserving transfer   tests/core/test_quantization.cpp:400-435
//   packed model state: copy -> load -> copy is byte-identical, a truncated
//   state is refused      tests/abi/test_c_api.c:3267-3302
//
// Plain main(), as the reference's tests are.  Modes:
//   test_hip_backend                 run against whatever runtime the adapter
//                                    loads (RIFTCO_TRANSFORMER_HIP_LIBRARY)
//   test_hip_backend --expect-unavailable
//                                    the runtime must be unavailable and the
//                                    adapter must fail the documented way
//   test_hip_backend --parse-state FILE...
//                                    prints, per file, what the packed model
//                                    state reader makes of it (no runtime)
// RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP=1 turns "unavailable" into a failure.

#include "../../riftco-transformer_amd/backend/dispatch.hpp"
#include "../../riftco-transformer_amd/backend/packed_state.hpp"

extern "C" {
#include "../../oracle/nf4_oracle.h"
}

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <iterator>
#include <limits>
#include <new>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace {

using riftco_transformer::ExecutionBackend;
namespace backend = riftco_transformer::backend_detail;

constexpr ExecutionBackend kHip = backend::kHipBackend;
constexpr std::size_t kEdgeWidth = 33;

void require(bool condition, const std::string& message) {
    if (!condition) {
        throw std::runtime_error(message);
    }
}

template <typename Exception, typename Function>
void require_throws(Function&& function, const std::string& message,
                    std::string_view fragment = {}) {
    try {
        function();
    } catch (const Exception& error) {
        if (!fragment.empty() &&
            std::string(error.what()).find(fragment) == std::string::npos) {
            throw std::runtime_error(message + ": wrong message: " +
                                     error.what());
        }
        return;
    } catch (const std::exception& error) {
        throw std::runtime_error(message + ": wrong exception: " +
                                 error.what());
    }
    throw std::runtime_error(message + ": nothing was thrown");
}

// |a - e| <= 3e-5 * max(1, |a|, |e|): the reference's tolerance
// (test_quantized_linear_backend.cpp:46-70).
void require_close(std::span<const float> actual,
                   const std::vector<float>& expected,
                   const std::string& message, float tolerance = 3.0e-5F) {
    require(actual.size() == expected.size(), message + ": size mismatch");
    for (std::size_t index = 0; index < expected.size(); ++index) {
        const float scale = std::max(
            {1.0F, std::fabs(actual[index]), std::fabs(expected[index])});
        if (!std::isfinite(actual[index]) ||
            std::fabs(actual[index] - expected[index]) > tolerance * scale) {
            throw std::runtime_error(
                message + " at flat index " + std::to_string(index) +
                ": expected " + std::to_string(expected[index]) + ", got " +
                std::to_string(actual[index]));
        }
    }
}

// ---- fixtures: the integer-formula tensors of the reference test ---------

std::vector<float> aligned_weight() {  // :89-100
    std::vector<float> values(3 * 32);
    for (std::size_t i = 0; i < values.size(); ++i) {
        values[i] = static_cast<float>(static_cast<int>(i % 19) - 9) * 0.1375F;
    }
    values[0] = -2.0F;
    values[31] = 1.75F;
    values[32] = 3.0F;
    values.back() = -4.0F;
    return values;
}

std::vector<float> aligned_input() {  // :102-109
    std::vector<float> values(2 * 32);
    for (std::size_t i = 0; i < values.size(); ++i) {
        values[i] = static_cast<float>(static_cast<int>(i % 11) - 5) * 0.2F;
    }
    return values;
}

std::vector<float> aligned_upstream() {  // :111-124
    return {0.25F, -0.75F, 1.5F, -1.0F, 0.5F, 0.125F};
}

std::vector<float> edge_weight() {  // :126-142
    std::vector<float> values(kEdgeWidth * kEdgeWidth);
    for (std::size_t i = 0; i < values.size(); ++i) {
        values[i] = static_cast<float>(static_cast<int>(i % 37) - 18) * 0.0625F;
    }
    values[0] = -3.0F;
    values[31] = 2.5F;
    values[32] = -2.75F;
    values[1023] = 4.0F;
    values[1024] = -4.5F;
    values.back() = 5.0F;
    return values;
}

std::vector<float> edge_input() {  // :144-155
    std::vector<float> values(2 * kEdgeWidth);
    for (std::size_t i = 0; i < values.size(); ++i) {
        values[i] = static_cast<float>(static_cast<int>(i % 17) - 8) * 0.125F;
    }
    return values;
}

std::vector<float> edge_upstream() {  // :157-168
    std::vector<float> values(2 * kEdgeWidth);
    for (std::size_t i = 0; i < values.size(); ++i) {
        values[i] = static_cast<float>(static_cast<int>(i % 13) - 6) * 0.075F;
    }
    return values;
}

// A deterministic pseudo-normal filler for the larger layer.
std::vector<float> pseudo_normal(std::size_t count, float sigma,
                                 std::uint32_t seed) {
    std::vector<float> values(count);
    std::uint32_t state = seed * 2654435761U + 12345U;
    for (float& value : values) {
        float sum = 0.0F;
        for (int k = 0; k < 4; ++k) {
            state = state * 1664525U + 1013904223U;
            sum += static_cast<float>(state >> 8) / 16777216.0F - 0.5F;
        }
        value = sum * 1.7320508F * sigma;
    }
    return values;
}

// ---- a packed weight on the host, quantised by the oracle ----------------

struct HostWeight {
    std::size_t output_width;
    std::size_t input_width;
    std::size_t block_size;
    std::vector<std::uint8_t> codes;
    backend::Nf4ScaleStorageData scales;

    [[nodiscard]] nf4o_scales view() const {
        nf4o_scales result{};
        result.encoding = static_cast<int32_t>(scales.encoding);
        result.fp32_scales = scales.fp32_scales.data();
        result.fp32_count = scales.fp32_scales.size();
        result.quantized_scales = scales.quantized_scales.data();
        result.quantized_count = scales.quantized_scales.size();
        result.second_level = scales.second_level_scales.data();
        result.second_level_count = scales.second_level_scales.size();
        result.second_level_block = scales.second_level_block_size;
        result.offset = scales.offset;
        return result;
    }
    [[nodiscard]] std::size_t logical_bytes() const {
        const nf4o_scales v = view();
        return codes.size() + nf4o_scale_payload_bytes(&v);
    }
};

HostWeight quantize(const std::vector<float>& dense, std::size_t output_width,
                    std::size_t input_width, std::size_t block_size,
                    bool double_quantized, std::size_t second_level_block) {
    HostWeight weight{output_width, input_width, block_size, {}, {}};
    const std::size_t count = dense.size();
    weight.codes.resize(nf4o_packed_byte_count(count));
    std::vector<float> block_scales(nf4o_block_count(count, block_size));
    require(nf4o_quantize(dense.data(), count, block_size, weight.codes.data(),
                          block_scales.data()) == NF4O_OK,
            "oracle quantizer failed");
    if (!double_quantized) {
        weight.scales.fp32_scales = std::move(block_scales);
        return weight;
    }
    weight.scales.encoding = backend::Nf4ScaleEncoding::DoubleQuantizedUInt8;
    weight.scales.quantized_scales.resize(block_scales.size());
    weight.scales.second_level_scales.resize(
        nf4o_block_count(block_scales.size(), second_level_block));
    weight.scales.second_level_block_size = second_level_block;
    require(nf4o_double_quantize_scales(
                block_scales.data(), block_scales.size(), second_level_block,
                weight.scales.quantized_scales.data(),
                weight.scales.second_level_scales.data(),
                &weight.scales.offset) == NF4O_OK,
            "oracle double quantizer failed");
    return weight;
}

std::unique_ptr<backend::QuantizedWeightStorage> to_hip(
    const HostWeight& weight
) {
    return backend::make_nf4_weight_storage(kHip, weight.codes, weight.scales);
}

std::vector<float> hip_forward(const std::vector<float>& input,
                               const backend::QuantizedWeightStorage& storage,
                               const HostWeight& weight) {
    const std::size_t rows = input.size() / weight.input_width;
    auto source = backend::make_tensor_storage(kHip, input);
    auto target =
        backend::make_tensor_storage(kHip, rows * weight.output_width, 0.0F);
    backend::dispatch_quantized_linear_forward(
        kHip, {*source, storage, *target,
               {rows, weight.input_width, weight.output_width,
                weight.block_size}});
    const auto data = std::as_const(*target).data();
    return {data.begin(), data.end()};
}

std::vector<float> hip_input_backward(
    const std::vector<float>& upstream,
    const backend::QuantizedWeightStorage& storage, const HostWeight& weight
) {
    const std::size_t rows = upstream.size() / weight.output_width;
    auto source = backend::make_tensor_storage(kHip, upstream);
    auto target =
        backend::make_tensor_storage(kHip, rows * weight.input_width, 0.0F);
    backend::dispatch_quantized_linear_input_backward(
        kHip, {*source, storage, *target,
               {rows, weight.input_width, weight.output_width,
                weight.block_size}});
    const auto data = std::as_const(*target).data();
    return {data.begin(), data.end()};
}

std::vector<float> oracle_forward(const std::vector<float>& input,
                                  const HostWeight& weight) {
    const std::size_t rows = input.size() / weight.input_width;
    std::vector<float> output(rows * weight.output_width);
    const nf4o_scales scales = weight.view();
    nf4o_linear_forward(input.data(), weight.codes.data(), &scales,
                        output.data(), rows, weight.input_width,
                        weight.output_width, weight.block_size);
    return output;
}

std::vector<float> oracle_input_backward(const std::vector<float>& upstream,
                                         const HostWeight& weight) {
    const std::size_t rows = upstream.size() / weight.output_width;
    std::vector<float> gradient(rows * weight.input_width);
    const nf4o_scales scales = weight.view();
    nf4o_linear_input_backward(upstream.data(), weight.codes.data(), &scales,
                               gradient.data(), rows, weight.input_width,
                               weight.output_width, weight.block_size);
    return gradient;
}

// ---- tests ---------------------------------------------------------------

void test_identity() {
    using riftco_transformer::execution_backend_name;
    require(static_cast<int>(ExecutionBackend::Cpu) == 0 &&
                static_cast<int>(ExecutionBackend::Metal) == 1 &&
                static_cast<int>(ExecutionBackend::Cuda) == 2 &&
                static_cast<int>(ExecutionBackend::Tpu) == 3 &&
                static_cast<int>(ExecutionBackend::Hip) == 4,
            "backend identities must keep their numeric values");
    require(execution_backend_name(ExecutionBackend::Cpu) == "cpu" &&
                execution_backend_name(ExecutionBackend::Metal) == "metal" &&
                execution_backend_name(ExecutionBackend::Cuda) == "cuda" &&
                execution_backend_name(ExecutionBackend::Tpu) == "tpu" &&
                execution_backend_name(kHip) == "hip",
            "backend names");
    const auto unknown = static_cast<ExecutionBackend>(0xFF);
    require(!riftco_transformer::execution_backend_available(unknown),
            "an unknown backend is not available");
    require(riftco_transformer::execution_backend_unavailability_reason(unknown)
                .empty(),
            "an unknown backend has no diagnostic");
    require_throws<std::invalid_argument>(
        [&] { static_cast<void>(execution_backend_name(unknown)); },
        "naming an unknown backend must throw", "unknown execution backend");
    require(backend::find_backend_adapter(unknown) == nullptr,
            "the registry must not invent adapters");
    require(&backend::hip_backend_adapter() ==
                backend::find_backend_adapter(kHip),
            "the registry serves the process-lifetime hip adapter");
    require(backend::hip_backend_adapter().name() == "hip", "adapter name");
}

void test_unavailable() {
    require(!riftco_transformer::execution_backend_available(kHip),
            "the hip backend should be unavailable in this mode");
    require(!riftco_transformer::execution_backend_unavailability_reason(kHip)
                 .empty(),
            "an unavailable hip backend must say why");
    for (const bool double_quantized : {false, true}) {
        const HostWeight weight =
            quantize(aligned_weight(), 3, 32, 32, double_quantized, 32);
        require_throws<std::runtime_error>(
            [&] { static_cast<void>(to_hip(weight)); },
            "an unavailable backend must reject packed weight transfer",
            "unavailable");
    }
    require_throws<std::runtime_error>(
        [&] {
            static_cast<void>(backend::make_tensor_storage(kHip, 4, 0.0F));
        },
        "an unavailable backend must reject tensor storage", "unavailable");
}

void require_memory_accounting(const backend::QuantizedWeightStorage& storage,
                               const HostWeight& weight,
                               const std::string& description) {
    const std::size_t logical = weight.logical_bytes();
    const std::size_t fp32_equivalent =
        weight.output_width * weight.input_width * sizeof(float);
    const bool mirrored = std::getenv("FAKE_RTHIP_NO_BAR") != nullptr;
    require(storage.resident_payload_bytes() ==
                (mirrored ? 2 * logical - (weight.scales.encoding ==
                                                   backend::Nf4ScaleEncoding::
                                                       DoubleQuantizedUInt8
                                               ? sizeof(float)
                                               : 0)
                          : logical),
            description + ": resident bytes must equal the logical payload "
                          "when HBM is host-visible");
    require(logical < fp32_equivalent,
            description + ": packed storage must stay below fp32 size");
    const auto scales = storage.scale_storage();
    if (weight.scales.encoding == backend::Nf4ScaleEncoding::Float32) {
        require(!scales.fp32_scales.empty() &&
                    scales.quantized_scales.empty() &&
                    scales.second_level_scales.empty() &&
                    scales.offset == 0.0F,
                description + ": legacy NF4 keeps only fp32 block scales");
    } else {
        require(scales.fp32_scales.empty() &&
                    !scales.quantized_scales.empty() &&
                    !scales.second_level_scales.empty(),
                description + ": double quantisation keeps encoded scales");
    }
}

void require_byte_preserving(const backend::QuantizedWeightStorage& storage,
                             const HostWeight& weight,
                             const std::string& description) {
    const auto codes = storage.packed_codes();
    require(codes.size() == weight.codes.size() &&
                std::equal(codes.begin(), codes.end(), weight.codes.begin()),
            description + ": packed codes must survive the transfer");
    const auto scales = storage.scale_storage();
    const auto same_floats = [](std::span<const float> a,
                                const std::vector<float>& b) {
        // (memcmp must not see the null pointers of two empty arrays)
        return a.size() == b.size() &&
               (b.empty() ||
                std::memcmp(a.data(), b.data(), b.size() * sizeof(float)) ==
                    0);
    };
    require(same_floats(scales.fp32_scales, weight.scales.fp32_scales) &&
                same_floats(scales.second_level_scales,
                            weight.scales.second_level_scales) &&
                scales.quantized_scales.size() ==
                    weight.scales.quantized_scales.size() &&
                std::equal(scales.quantized_scales.begin(),
                           scales.quantized_scales.end(),
                           weight.scales.quantized_scales.begin()) &&
                scales.second_level_block_size ==
                    weight.scales.second_level_block_size &&
                scales.offset == weight.scales.offset &&
                scales.encoding == weight.scales.encoding,
            description + ": scales must survive the transfer bit for bit");
    require(storage.backend() == kHip, description + ": backend identity");
    require(storage.packed_codes_native_handle() != nullptr &&
                storage.primary_scales_native_handle() != nullptr &&
                (storage.secondary_scales_native_handle() != nullptr) ==
                    (weight.scales.encoding ==
                     backend::Nf4ScaleEncoding::DoubleQuantizedUInt8),
            description + ": native handles");
}

void run_accelerator_oracle(const std::vector<float>& dense,
                            std::size_t output_width, std::size_t input_width,
                            const std::vector<float>& input,
                            const std::vector<float>& upstream,
                            bool double_quantized, bool edge_layout) {
    const std::string description =
        std::string("hip") + (double_quantized ? " double-quantized" : "") +
        " NF4 " + (edge_layout ? "edge" : "aligned") + " fixture";
    const HostWeight weight = quantize(dense, output_width, input_width, 32,
                                       double_quantized, 32);
    if (edge_layout) {
        // odd element count, partial last block, two second-level groups
        require(weight.codes.size() == (kEdgeWidth * kEdgeWidth + 1) / 2 &&
                    (weight.codes.back() & 0xF0U) == 0,
                description + ": canonical odd packed-code tail");
        require(nf4o_block_count(kEdgeWidth * kEdgeWidth, 32) == 35,
                description + ": partial last block");
        if (double_quantized) {
            require(weight.scales.second_level_scales.size() == 2,
                    description + ": two second-level groups");
        }
    }
    const auto storage = to_hip(weight);
    require_byte_preserving(*storage, weight, description);
    require_memory_accounting(*storage, weight, description);
    require_close(hip_forward(input, *storage, weight),
                  oracle_forward(input, weight),
                  description + " forward must match the CPU oracle");
    require_close(hip_input_backward(upstream, *storage, weight),
                  oracle_input_backward(upstream, weight),
                  description + " input backward must match the CPU oracle");
    // the frozen weight is untouched by execution
    require_byte_preserving(*storage, weight, description + " after use");
}

void test_accelerator_oracle() {
    for (const bool double_quantized : {false, true}) {
        run_accelerator_oracle(aligned_weight(), 3, 32, aligned_input(),
                               aligned_upstream(), double_quantized, false);
        run_accelerator_oracle(edge_weight(), kEdgeWidth, kEdgeWidth,
                               edge_input(), edge_upstream(), double_quantized,
                               true);
    }
}

void test_transformer_sized_layer() {
    // [768 x 256], block 64: rows 1 (decode kernel) and 16 (tiled kernel).
    const std::vector<float> dense = pseudo_normal(768 * 256, 0.02F, 1);
    for (const bool double_quantized : {false, true}) {
        const HostWeight weight =
            quantize(dense, 768, 256, 64, double_quantized, 256);
        const auto storage = to_hip(weight);
        require_memory_accounting(*storage, weight, "layer");
        for (const std::size_t rows : {std::size_t{1}, std::size_t{16}}) {
            const auto input = pseudo_normal(rows * 256, 1.0F, 2);
            const auto upstream = pseudo_normal(rows * 768, 0.01F, 3);
            require_close(hip_forward(input, *storage, weight),
                          oracle_forward(input, weight), "layer forward");
            require_close(hip_input_backward(upstream, *storage, weight),
                          oracle_input_backward(upstream, weight),
                          "layer input backward");
        }
    }
}

void test_forward_group() {
    // Three projections of one input (the query/key/value pattern), through
    // hip_quantized_linear_forward_group: bit for bit what one dispatch per
    // projection writes.
    namespace detail = riftco_transformer::backend_detail;
    const std::size_t widths[] = {96, 64, 130};
    for (const bool double_quantized : {false, true}) {
        std::vector<HostWeight> weights;
        std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> storages;
        for (std::size_t m = 0; m < 3; ++m) {
            weights.push_back(quantize(
                pseudo_normal(widths[m] * 256, 0.02F, 40 + m), widths[m], 256,
                64, double_quantized, 256));
            storages.push_back(to_hip(weights.back()));
        }
        for (const std::size_t rows : {std::size_t{1}, std::size_t{3},
                                       std::size_t{9}}) {
            const auto input = pseudo_normal(rows * 256, 1.0F, 50 + rows);
            auto source = backend::make_tensor_storage(kHip, input);
            std::vector<std::unique_ptr<backend::TensorStorage>> targets;
            std::vector<backend::QuantizedLinearForwardRequest> requests;
            for (std::size_t m = 0; m < 3; ++m) {
                targets.push_back(backend::make_tensor_storage(
                    kHip, rows * widths[m], 0.0F));
                requests.push_back({*source, *storages[m], *targets[m],
                                    {rows, 256, widths[m], 64}});
            }
            detail::hip_quantized_linear_forward_group(requests);
            for (std::size_t m = 0; m < 3; ++m) {
                const auto data = std::as_const(*targets[m]).data();
                const std::vector<float> together(data.begin(), data.end());
                const std::vector<float> alone =
                    hip_forward(input, *storages[m], weights[m]);
                require(together.size() == alone.size() &&
                            std::memcmp(together.data(), alone.data(),
                                        alone.size() * sizeof(float)) == 0,
                        "a grouped forward must equal the separate one");
            }
        }
        // requests that do not belong together are refused
        const auto input = pseudo_normal(256, 1.0F, 60);
        auto source = backend::make_tensor_storage(kHip, input);
        auto other_source = backend::make_tensor_storage(kHip, input);
        auto target_a = backend::make_tensor_storage(kHip, widths[0], 0.0F);
        auto target_b = backend::make_tensor_storage(kHip, widths[1], 0.0F);
        const std::vector<backend::QuantizedLinearForwardRequest> mixed = {
            {*source, *storages[0], *target_a, {1, 256, widths[0], 64}},
            {*other_source, *storages[1], *target_b, {1, 256, widths[1], 64}}};
        require_throws<std::invalid_argument>(
            [&] { detail::hip_quantized_linear_forward_group(mixed); },
            "a group over two inputs", "share their input");
        require_throws<std::invalid_argument>(
            [&] { detail::hip_quantized_linear_forward_group({}); },
            "an empty group", "at least one request");
    }
}

void test_adapter_layer() {
    // A layer with a packed weight, a bias and a rank-3 adapter: the fused
    // forward and backward of backend/hip_adapter.hpp against the CPU
    // restatement of the reference's autograd (pinned to the compiled
    // reference's own Linear bit for bit).
    namespace detail = riftco_transformer::backend_detail;
    const std::size_t out_w = 40, in_w = 256, rank = 3;
    const float scale = 8.0F / 3.0F;
    const auto a_values = pseudo_normal(rank * in_w, 0.05F, 71);
    const auto b_values = pseudo_normal(out_w * rank, 0.05F, 72);
    const auto bias_values = pseudo_normal(out_w, 0.01F, 73);
    for (const bool double_quantized : {false, true}) {
        const HostWeight weight =
            quantize(pseudo_normal(out_w * in_w, 0.02F, 70), out_w, in_w, 64,
                     double_quantized, 32);
        const auto storage = to_hip(weight);
        const nf4o_scales scales = weight.view();
        for (const std::size_t rows : {std::size_t{1}, std::size_t{9}}) {
            const auto x = pseudo_normal(rows * in_w, 1.0F, 74 + rows);
            const auto dy = pseudo_normal(rows * out_w, 0.01F, 75 + rows);
            std::vector<float> want_y(rows * out_w), want_dx(rows * in_w),
                want_da(rank * in_w), want_db(out_w * rank);
            nf4o_lora_linear_forward(
                x.data(), weight.codes.data(), &scales, bias_values.data(),
                a_values.data(), b_values.data(), rank, scale, want_y.data(),
                rows, in_w, out_w, 64);
            nf4o_lora_linear_backward(
                dy.data(), x.data(), weight.codes.data(), &scales,
                a_values.data(), b_values.data(), rank, scale, want_dx.data(),
                want_da.data(), want_db.data(), rows, in_w, out_w, 64);

            auto input = backend::make_tensor_storage(kHip, x);
            auto upstream = backend::make_tensor_storage(kHip, dy);
            auto lora_a = backend::make_tensor_storage(kHip, a_values);
            auto lora_b = backend::make_tensor_storage(kHip, b_values);
            auto bias = backend::make_tensor_storage(kHip, bias_values);
            auto reduced =
                backend::make_tensor_storage(kHip, rows * rank, 0.0F);
            auto output =
                backend::make_tensor_storage(kHip, rows * out_w, 0.0F);
            const backend::QuantizedLinearDimensions dimensions{rows, in_w,
                                                                out_w, 64};
            detail::hip_quantized_linear_adapter_forward(
                {*input, *storage, bias.get(), *lora_a, *lora_b, rank, scale,
                 *reduced, *output, dimensions});
            require_close(std::as_const(*output).data(), want_y,
                          "adapter forward");
            auto dx = backend::make_tensor_storage(kHip, rows * in_w, 7.0F);
            auto da = backend::make_tensor_storage(kHip, rank * in_w, 7.0F);
            auto db = backend::make_tensor_storage(kHip, out_w * rank, 7.0F);
            detail::hip_quantized_linear_adapter_backward(
                {*upstream, *input, *reduced, *storage, *lora_a, *lora_b, rank,
                 scale, *dx, *da, *db, dimensions});
            require_close(std::as_const(*dx).data(), want_dx,
                          "adapter backward, input gradient");
            require_close(std::as_const(*da).data(), want_da,
                          "adapter backward, A gradient");
            require_close(std::as_const(*db).data(), want_db,
                          "adapter backward, B gradient");

            // what a request may not carry
            require_throws<std::invalid_argument>(
                [&] {
                    detail::hip_quantized_linear_adapter_forward(
                        {*input, *storage, nullptr, *lora_a, *lora_b, 0,
                         scale, *reduced, *output, dimensions});
                },
                "rank zero", "LoRA rank must be in");
            require_throws<std::invalid_argument>(
                [&] {
                    detail::hip_quantized_linear_adapter_forward(
                        {*input, *storage, nullptr, *lora_a, *lora_b, rank,
                         -1.0F, *reduced, *output, dimensions});
                },
                "negative scale", "finite and positive");
            require_throws<std::invalid_argument>(
                [&] {
                    detail::hip_quantized_linear_adapter_backward(
                        {*upstream, *input, *reduced, *storage, *lora_a,
                         *lora_b, rank, scale, *dx, *db, *db, dimensions});
                },
                "an A gradient of the wrong size", "A gradient");
            require_throws<std::invalid_argument>(
                [&] {
                    detail::hip_quantized_linear_adapter_forward(
                        {*input, *storage, lora_a.get(), *lora_a, *lora_b,
                         rank, scale, *reduced, *output, dimensions});
                },
                "a bias of the wrong size", "bias");
        }
    }
}

void test_one_value_tensors() {
    // make_tensor_storage(count, value) writes the value where it is first
    // needed: read by host code, read by a kernel (as the input of a
    // forward), cloned, or never (an output that a kernel overwrites).
    const std::size_t in_w = 256, out_w = 64;
    const HostWeight weight = quantize(
        pseudo_normal(out_w * in_w, 0.02F, 301), out_w, in_w, 64, false, 256);
    const auto storage = to_hip(weight);
    {
        auto tensor = backend::make_tensor_storage(kHip, 5, 3.5F);
        const auto values = std::as_const(*tensor).data();
        require(values.size() == 5 && values[0] == 3.5F && values[4] == 3.5F,
                "a one-value tensor read by host code");
        tensor->data()[2] = 1.0F;  // host write, then a device read
        auto copy = tensor->clone();
        require(std::as_const(*copy).data()[2] == 1.0F &&
                    std::as_const(*copy).data()[3] == 3.5F,
                "a clone of a one-value tensor that host code changed");
    }
    {
        auto input = backend::make_tensor_storage(kHip, in_w, 0.25F);
        auto output = backend::make_tensor_storage(kHip, out_w, 9.0F);
        backend::dispatch_quantized_linear_forward(
            kHip, {*input, *storage, *output, {1, in_w, out_w, 64}});
        require_close(std::as_const(*output).data(),
                      oracle_forward(std::vector<float>(in_w, 0.25F), weight),
                      "a one-value tensor read by a kernel first");
        // the input still reads as its value on the host
        require(std::as_const(*input).data()[in_w - 1] == 0.25F,
                "a one-value tensor read by a kernel, then by host code");
    }
    {
        auto untouched = backend::make_tensor_storage(kHip, 3, -2.0F);
        auto copy = untouched->clone();
        require(std::as_const(*copy).data()[1] == -2.0F,
                "a clone of a one-value tensor nobody has read");
    }
}

void test_merged_adapter_forwards() {
    // A decoder whose query and value projections carry adapters: q (adapter,
    // bias), k (plain, through the dispatcher), v (adapter) on one input, then
    // a dependent layer whose input is q's output.  Unless
    // RIFTCO_TRANSFORMER_HIP_MERGE=0 the first three are one launch (their
    // x.A^T products go out at once) and the dependent one is launched only
    // after them.
    namespace detail = riftco_transformer::backend_detail;
    const char* option = std::getenv("RIFTCO_TRANSFORMER_HIP_MERGE");
    const bool merging = option == nullptr || std::string_view(option) != "0";
    const std::size_t in_w = 256, out_w = 256, rank = 4;
    const float scale = 0.5F;
    for (const bool double_quantized : {false, true}) {
        std::vector<HostWeight> weights;
        std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> storages;
        for (std::size_t m = 0; m < 4; ++m) {
            weights.push_back(quantize(
                pseudo_normal(out_w * in_w, 0.02F, 170 + m), out_w, in_w, 64,
                double_quantized, 32));
            storages.push_back(to_hip(weights.back()));
        }
        const auto a_values = pseudo_normal(rank * in_w, 0.05F, 181);
        const auto b_values = pseudo_normal(out_w * rank, 0.05F, 182);
        const auto bias_values = pseudo_normal(out_w, 0.01F, 183);
        for (const std::size_t rows : {std::size_t{1}, std::size_t{4},
                                       std::size_t{9}}) {
            const auto x = pseudo_normal(rows * in_w, 1.0F, 184 + rows);
            auto input = backend::make_tensor_storage(kHip, x);
            auto lora_a = backend::make_tensor_storage(kHip, a_values);
            auto lora_b = backend::make_tensor_storage(kHip, b_values);
            auto bias = backend::make_tensor_storage(kHip, bias_values);
            std::vector<std::unique_ptr<backend::TensorStorage>> outputs;
            std::vector<std::unique_ptr<backend::TensorStorage>> products;
            for (std::size_t m = 0; m < 4; ++m) {
                outputs.push_back(
                    backend::make_tensor_storage(kHip, rows * out_w, 0.0F));
                products.push_back(
                    backend::make_tensor_storage(kHip, rows * rank, 0.0F));
            }
            const backend::QuantizedLinearDimensions dimensions{rows, in_w,
                                                                out_w, 64};
            const auto before = detail::hip_forward_merge_statistics();
            detail::hip_quantized_linear_adapter_forward(
                {*input, *storages[0], bias.get(), *lora_a, *lora_b, rank,
                 scale, *products[0], *outputs[0], dimensions});
            backend::dispatch_quantized_linear_forward(
                kHip, {*input, *storages[1], *outputs[1], dimensions});
            detail::hip_quantized_linear_adapter_forward(
                {*input, *storages[2], nullptr, *lora_a, *lora_b, rank, scale,
                 *products[2], *outputs[2], dimensions});
            // reads q's output: what is held back goes out first
            detail::hip_quantized_linear_adapter_forward(
                {*outputs[0], *storages[3], nullptr, *lora_a, *lora_b, rank,
                 scale, *products[3], *outputs[3], dimensions});
            const auto after_calls = detail::hip_forward_merge_statistics();

            std::vector<float> want_q(rows * out_w), want_k, want_v(rows * out_w),
                want_next(rows * out_w);
            const nf4o_scales scales_q = weights[0].view();
            nf4o_lora_linear_forward(
                x.data(), weights[0].codes.data(), &scales_q,
                bias_values.data(), a_values.data(), b_values.data(), rank,
                scale, want_q.data(), rows, in_w, out_w, 64);
            want_k = oracle_forward(x, weights[1]);
            const nf4o_scales scales_v = weights[2].view();
            nf4o_lora_linear_forward(
                x.data(), weights[2].codes.data(), &scales_v, nullptr,
                a_values.data(), b_values.data(), rank, scale, want_v.data(),
                rows, in_w, out_w, 64);
            const nf4o_scales scales_next = weights[3].view();
            nf4o_lora_linear_forward(
                want_q.data(), weights[3].codes.data(), &scales_next, nullptr,
                a_values.data(), b_values.data(), rank, scale,
                want_next.data(), rows, in_w, out_w, 64);
            require_close(std::as_const(*outputs[0]).data(), want_q,
                          "merged adapter forward, first member");
            require_close(std::as_const(*outputs[1]).data(), want_k,
                          "merged adapter forward, plain member");
            require_close(std::as_const(*outputs[2]).data(), want_v,
                          "merged adapter forward, third member");
            require_close(std::as_const(*outputs[3]).data(), want_next,
                          "a layer that reads a held-back output");
            // x.A^T is the saved activation of the backward
            std::vector<float> want_product(rows * rank);
            nf4o_matmul_nt(x.data(), a_values.data(), want_product.data(),
                           rows, in_w, rank);
            require_close(std::as_const(*products[2]).data(), want_product,
                          "the reduced buffer of a merged member");
            if (merging) {
                require(after_calls.requests - before.requests == 4 &&
                            after_calls.launches - before.launches == 1,
                        "three forwards on one input are held back until the "
                        "dependent one arrives: one launch so far");
                const auto after = detail::hip_forward_merge_statistics();
                require(after.launches - before.launches == 2,
                        "reading the outputs launches the dependent one");
            }
        }
    }
}

void test_merged_forwards() {
    // The decoder's pattern, unchanged callers: three projections of one
    // input and then one of another, each through the dispatcher.  Results are
    // those of the CPU oracle in every mode; unless
    // RIFTCO_TRANSFORMER_HIP_MERGE=0 the four requests become two launches,
    // and what is held back is launched before anything can observe it.
    namespace detail = riftco_transformer::backend_detail;
    const char* option = std::getenv("RIFTCO_TRANSFORMER_HIP_MERGE");
    const bool merging = option == nullptr || std::string_view(option) != "0";
    const std::size_t widths[] = {96, 64, 130};
    for (const bool double_quantized : {false, true}) {
        std::vector<HostWeight> weights;
        std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> storages;
        for (std::size_t m = 0; m < 3; ++m) {
            weights.push_back(quantize(
                pseudo_normal(widths[m] * 256, 0.02F, 70 + m), widths[m], 256,
                64, double_quantized, 256));
            storages.push_back(to_hip(weights.back()));
        }
        for (const std::size_t rows : {std::size_t{1}, std::size_t{4}}) {
            const auto input = pseudo_normal(rows * 256, 1.0F, 80 + rows);
            const auto other_input = pseudo_normal(rows * 256, 1.0F, 90 + rows);
            auto source = backend::make_tensor_storage(kHip, input);
            auto other_source = backend::make_tensor_storage(kHip, other_input);
            std::vector<std::unique_ptr<backend::TensorStorage>> targets;
            for (std::size_t m = 0; m < 3; ++m) {
                targets.push_back(backend::make_tensor_storage(
                    kHip, rows * widths[m], 0.0F));
            }
            auto other_target =
                backend::make_tensor_storage(kHip, rows * widths[0], 0.0F);
            const auto before = detail::hip_forward_merge_statistics();
            for (std::size_t m = 0; m < 3; ++m) {
                backend::dispatch_quantized_linear_forward(
                    kHip, {*source, *storages[m], *targets[m],
                           {rows, 256, widths[m], 64}});
            }
            backend::dispatch_quantized_linear_forward(
                kHip, {*other_source, *storages[0], *other_target,
                       {rows, 256, widths[0], 64}});
            // twice into the same output: the second call must find the
            // first one launched, not share a launch with it
            backend::dispatch_quantized_linear_forward(
                kHip, {*other_source, *storages[0], *other_target,
                       {rows, 256, widths[0], 64}});
            for (std::size_t m = 0; m < 3; ++m) {
                const auto data = std::as_const(*targets[m]).data();
                require_close({data.begin(), data.end()},
                              oracle_forward(input, weights[m]),
                              "a forward that may have been merged must match "
                              "the CPU oracle");
            }
            const auto data = std::as_const(*other_target).data();
            require_close({data.begin(), data.end()},
                          oracle_forward(other_input, weights[0]),
                          "two forwards into one output, one after the other");
            const auto after = detail::hip_forward_merge_statistics();
            if (merging) {
                require(after.requests - before.requests == 5 &&
                            after.launches - before.launches == 3,
                        "five forwards (three sharing an input, two into one "
                        "output) must become three launches");
            } else {
                require(after.requests == 0 && after.launches == 0,
                        "nothing is merged once merging is turned off");
            }
        }
        // a tensor that is released while a launch that writes it is held
        // back: the launch goes out first (no write into recycled memory)
        const auto input = pseudo_normal(256, 1.0F, 99);
        auto source = backend::make_tensor_storage(kHip, input);
        auto kept = backend::make_tensor_storage(kHip, widths[1], 0.0F);
        {
            auto dropped = backend::make_tensor_storage(kHip, widths[0], 0.0F);
            backend::dispatch_quantized_linear_forward(
                kHip, {*source, *storages[0], *dropped,
                       {1, 256, widths[0], 64}});
        }
        auto recycled = backend::make_tensor_storage(kHip, widths[0], 7.0F);
        backend::dispatch_quantized_linear_forward(
            kHip, {*source, *storages[1], *kept, {1, 256, widths[1], 64}});
        const auto untouched = std::as_const(*recycled).data();
        for (const float value : untouched) {
            require(value == 7.0F,
                    "a held-back launch must not write into a buffer that "
                    "was released and handed out again");
        }
        const auto data = std::as_const(*kept).data();
        require_close({data.begin(), data.end()},
                      oracle_forward(input, weights[1]),
                      "forward after a released output");
    }
}

void test_tensor_storage() {
    auto filled = backend::make_tensor_storage(kHip, 5, 1.5F);
    require(filled->backend() == kHip && filled->size() == 5 &&
                filled->native_handle() != nullptr,
            "filled tensor storage identity");
    for (const float value : std::as_const(*filled).data()) {
        require(value == 1.5F, "fill value must reach the host view");
    }
    auto copy = filled->clone();
    filled->data()[2] = -7.0F;  // a host write through the mutable span
    require(std::as_const(*copy).data()[2] == 1.5F &&
                copy->native_handle() != filled->native_handle(),
            "a clone owns separate storage");

    // a host write must be seen by the next kernel that reads the tensor
    const HostWeight weight = quantize(aligned_weight(), 3, 32, 32, false, 32);
    const auto storage = to_hip(weight);
    std::vector<float> input = aligned_input();
    auto source = backend::make_tensor_storage(kHip, input);
    auto target = backend::make_tensor_storage(kHip, 2 * 3, 0.0F);
    source->data()[5] = 3.25F;
    input[5] = 3.25F;
    backend::dispatch_quantized_linear_forward(
        kHip, {*source, *storage, *target, {2, 32, 3, 32}});
    require_close(std::as_const(*target).data(), oracle_forward(input, weight),
                  "kernels must see host writes made through data()");
}

void test_dispatch_validation() {
    const HostWeight weight = quantize(aligned_weight(), 3, 32, 32, false, 32);
    const auto storage = to_hip(weight);
    auto input = backend::make_tensor_storage(kHip, aligned_input());
    auto output = backend::make_tensor_storage(kHip, 2 * 3, 0.0F);
    const backend::QuantizedLinearDimensions good{2, 32, 3, 32};

    {
        // a square weight, so that one tensor fits both roles
        const HostWeight square = quantize(pseudo_normal(32 * 32, 0.02F, 9),
                                           32, 32, 32, false, 32);
        const auto square_storage = to_hip(square);
        require_throws<std::invalid_argument>(
            [&] {
                backend::dispatch_quantized_linear_forward(
                    kHip,
                    {*input, *square_storage, *input, {2, 32, 32, 32}});
            },
            "input and output must not alias", "must not alias");
        require_throws<std::invalid_argument>(
            [&] {
                backend::dispatch_quantized_linear_input_backward(
                    kHip,
                    {*input, *square_storage, *input, {2, 32, 32, 32}});
            },
            "upstream and gradient must not alias", "must not alias");
    }
    require_throws<std::invalid_argument>(
        [&] {
            backend::dispatch_quantized_linear_forward(
                kHip, {*input, *storage, *output, {0, 32, 3, 32}});
        },
        "zero rows must be rejected", "positive");
    require_throws<std::logic_error>(
        [&] {
            backend::dispatch_quantized_linear_forward(
                kHip, {*input, *storage, *output, {3, 32, 3, 32}});
        },
        "tensor size must match the dimensions");
    require_throws<std::logic_error>(
        [&] {
            backend::dispatch_quantized_linear_forward(
                kHip, {*input, *storage, *output, {2, 16, 3, 32}});
        },
        "tensor/weight size must match the dimensions");
    require_throws<std::invalid_argument>(
        [&] {
            backend::dispatch_quantized_linear_forward(
                static_cast<ExecutionBackend>(0xFF),
                {*input, *storage, *output, good});
        },
        "unknown backend", "unknown execution backend");
    require_throws<std::runtime_error>(
        [&] {
            backend::dispatch_quantized_linear_forward(
                ExecutionBackend::Cuda, {*input, *storage, *output, good});
        },
        "a backend that is not part of the build is unavailable",
        "cuda execution backend is unavailable");

    // storage construction validates the payload before anything is uploaded
    require_throws<std::invalid_argument>(
        [&] {
            static_cast<void>(backend::make_nf4_weight_storage(
                kHip, {}, weight.scales));
        },
        "empty codes", "must not be empty");
    require_throws<std::invalid_argument>(
        [&] {
            backend::Nf4ScaleStorageData scales = weight.scales;
            scales.fp32_scales[1] = -1.0F;
            static_cast<void>(backend::make_nf4_weight_storage(
                kHip, weight.codes, std::move(scales)));
        },
        "negative scale", "finite and non-negative");
    require_throws<std::invalid_argument>(
        [&] {
            backend::Nf4ScaleStorageData scales = weight.scales;
            scales.offset = 1.0F;
            static_cast<void>(backend::make_nf4_weight_storage(
                kHip, weight.codes, std::move(scales)));
        },
        "legacy representation with an offset", "invalid representation");
    require_throws<std::invalid_argument>(
        [&] {
            backend::Nf4ScaleStorageData scales;
            scales.encoding = backend::Nf4ScaleEncoding::DoubleQuantizedUInt8;
            scales.quantized_scales = {128, 128, 128};
            scales.second_level_scales = {0.0F};
            scales.second_level_block_size = 48;
            static_cast<void>(backend::make_nf4_weight_storage(
                kHip, weight.codes, std::move(scales)));
        },
        "unsupported second-level block", "invalid representation");
}

// ---- packed model state ---------------------------------------------------

std::vector<std::uint8_t> state_of(
    const std::vector<const HostWeight*>& weights,
    const std::vector<std::unique_ptr<backend::QuantizedWeightStorage>>&
        storages
) {
    std::vector<std::vector<std::size_t>> shapes;
    std::vector<backend::HipPackedWeightSource> sources;
    for (const HostWeight* weight : weights) {
        shapes.push_back({weight->output_width, weight->input_width});
    }
    for (std::size_t index = 0; index < weights.size(); ++index) {
        sources.push_back({shapes[index], weights[index]->block_size,
                           storages[index].get()});
    }
    return backend::hip_packed_model_state_bytes(sources);
}

// What the oracle says about one parsed entry after `damage` was applied.
std::string oracle_verdict(const backend::PackedWeightView& entry) {
    std::vector<float> fp32(entry.block_scale_bytes.size() / 4);
    if (!fp32.empty()) {
        std::memcpy(fp32.data(), entry.block_scale_bytes.data(),
                    entry.block_scale_bytes.size());
    }
    std::vector<float> second(entry.second_level_scale_bytes.size() / 4);
    if (!second.empty()) {
        std::memcpy(second.data(), entry.second_level_scale_bytes.data(),
                    entry.second_level_scale_bytes.size());
    }
    nf4o_scales scales{};
    scales.encoding = entry.double_quantized ? 1 : 0;
    scales.fp32_scales = fp32.data();
    scales.fp32_count = fp32.size();
    scales.quantized_scales = entry.scale_codes.data();
    scales.quantized_count = entry.scale_codes.size();
    scales.second_level = second.data();
    scales.second_level_count = second.size();
    scales.second_level_block = entry.scale_block_size;
    scales.offset = entry.offset;
    const char* message = "";
    const int status = nf4o_validate_payload(
        entry.shape[0] * entry.shape[1], entry.block_size,
        entry.packed_codes.data(), entry.packed_codes.size(), &scales,
        &message);
    return status == NF4O_OK ? std::string() : std::string(message);
}

void test_packed_model_state() {
    // Three weights as a model would hold them: fp32 scales with an odd
    // element count, nested scales, and a larger nested one with whole zero
    // rows (zero-scale blocks).
    const HostWeight edge = quantize(edge_weight(), kEdgeWidth, kEdgeWidth, 32,
                                     false, 32);
    const HostWeight nested_edge = quantize(edge_weight(), kEdgeWidth,
                                            kEdgeWidth, 32, true, 32);
    std::vector<float> dense = pseudo_normal(96 * 256, 0.02F, 7);
    std::fill(dense.begin() + 256, dense.begin() + 3 * 256, 0.0F);
    const HostWeight zero_rows = quantize(dense, 96, 256, 64, false, 32);
    const HostWeight nested_rows = quantize(dense, 96, 256, 64, true, 256);
    const std::vector<const HostWeight*> weights{&edge, &nested_edge,
                                                 &zero_rows, &nested_rows};
    std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> storages;
    for (const HostWeight* weight : weights) {
        storages.push_back(to_hip(*weight));
    }

    // copy -> load -> copy is byte-identical (tests/abi/test_c_api.c:3284-3302)
    const std::vector<std::uint8_t> state = state_of(weights, storages);
    const auto entries = backend::parse_packed_model_state(state);
    require(entries.size() == weights.size(), "packed state entry count");
    for (std::size_t index = 0; index < weights.size(); ++index) {
        const HostWeight& weight = *weights[index];
        const auto& entry = entries[index];
        require(entry.shape == std::vector<std::size_t>{weight.output_width,
                                                        weight.input_width} &&
                    entry.block_size == weight.block_size,
                "packed state shape and block size");
        require(std::equal(entry.packed_codes.begin(),
                           entry.packed_codes.end(), weight.codes.begin(),
                           weight.codes.end()),
                "packed state codes must be the stored bytes");
        require(oracle_verdict(entry).empty(),
                "a written state must hold canonical payloads");
    }
    auto loaded = backend::hip_load_packed_model_state(state);
    require(loaded.size() == weights.size(), "loaded weight count");
    std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> restored;
    for (std::size_t index = 0; index < loaded.size(); ++index) {
        const HostWeight& weight = *weights[index];
        require(loaded[index].shape ==
                        std::vector<std::size_t>{weight.output_width,
                                                 weight.input_width} &&
                    loaded[index].block_size == weight.block_size,
                "loaded shape and block size");
        require(loaded[index].storage != nullptr &&
                    loaded[index].storage->backend() == kHip,
                "loaded storage must be hip storage");
        require_byte_preserving(*loaded[index].storage, weight,
                                "loaded packed state");
        restored.push_back(std::move(loaded[index].storage));
    }
    require(state_of(weights, restored) == state,
            "copy -> load -> copy must be byte-identical");

    // a restored weight computes what the original does
    const std::vector<float> input = edge_input();
    require(hip_forward(input, *restored[1], nested_edge) ==
                hip_forward(input, *storages[1], nested_edge),
            "a restored weight must compute like the original");
    require_close(hip_forward(input, *restored[0], edge),
                  oracle_forward(input, edge), "restored forward");

    // a truncated state is refused (tests/abi/test_c_api.c:3289-3293)
    require_throws<std::invalid_argument>(
        [&] {
            static_cast<void>(backend::hip_load_packed_model_state(
                std::span(state).first(state.size() - 1)));
        },
        "a truncated packed state must be refused",
        "truncated packed model state");
    require_throws<std::invalid_argument>(
        [&] {
            std::vector<std::uint8_t> other = state;
            other[6] = '2';
            static_cast<void>(backend::hip_load_packed_model_state(other));
        },
        "an unknown format must be refused",
        "unknown packed model state format");

    // Damaged payloads: the loader must throw std::invalid_argument with the
    // message the oracle's require_canonical_payload gives for the same bytes.
    // A patch overwrites bytes of one array of one entry: 0 codes, 1 block
    // scales, 2 scale codes, 3 second-level scales, 4 the entry's header
    // (offset in bytes from its start).
    struct Patch {
        std::size_t entry;
        int array;
        std::size_t offset;
        std::vector<std::uint8_t> bytes;
    };
    struct Damage {
        const char* name;
        std::vector<Patch> patches;
    };
    const auto f32 = [](float value) {
        std::vector<std::uint8_t> bytes(4);
        std::memcpy(bytes.data(), &value, 4);
        return bytes;
    };
    const auto u64 = [](std::uint64_t value) {
        std::vector<std::uint8_t> bytes(8);
        std::memcpy(bytes.data(), &value, 8);
        return bytes;
    };
    const float infinity = std::numeric_limits<float>::infinity();
    const float nan = std::numeric_limits<float>::quiet_NaN();
    const std::vector<Damage> damages{
        {"unused nibble", {{0, 0, edge.codes.size() - 1, {0xF7}}}},
        {"negative scale", {{0, 1, 4 * 5, f32(-1.0F)}}},
        {"infinite scale", {{0, 1, 4 * 30, f32(infinity)}}},
        {"nan scale", {{2, 1, 4 * 100, f32(nan)}}},
        {"zero block with a code", {{2, 0, 128 + 17, {0x78}}}},
        {"zero block with a code, last byte", {{2, 0, 3 * 128 - 1, {0x87}}}},
        {"zeroed scale of a used block", {{2, 1, 4 * 200, f32(0.0F)}}},
        // the lowest offending block decides which rule is reported
        {"bad scale below a bad zero block",
         {{2, 1, 4 * 2, f32(-2.0F)}, {2, 0, 128 + 17, {0x78}}}},
        {"bad zero block below a bad scale",
         {{2, 1, 4 * 300, f32(-2.0F)}, {2, 0, 128 + 17, {0x78}}}},
        // the unused nibble is reported before anything else
        {"unused nibble and a bad scale",
         {{0, 0, edge.codes.size() - 1, {0xF7}}, {0, 1, 0, f32(nan)}}},
        {"nested: second-level nan", {{1, 3, 0, f32(nan)}}},
        {"nested: second-level negative", {{3, 3, 0, f32(-1.0F)}}},
        {"nested: offset infinite", {{1, 4, 56, f32(infinity)}}},
        {"nested: offset negative", {{3, 4, 56, f32(-0.5F)}}},
        {"nested: offset before second-level scales",
         {{3, 4, 56, f32(nan)}, {3, 3, 0, f32(nan)}}},
        {"nested: unused nibble",
         {{1, 0, nested_edge.codes.size() - 1, {0xF7}}}},
        {"block size", {{0, 4, 8, u64(48)}}},
        {"second-level block size", {{1, 4, 48, u64(48)}}},
        {"rows", {{2, 4, 64, u64(95)}}},
        {"zero rows", {{2, 4, 64, u64(0)}}},
        {"huge shape", {{2, 4, 64, u64(1ULL << 63)}}},
        {"block size and scale count", {{2, 4, 8, u64(128)}}},
    };
    for (const Damage& damage : damages) {
        std::vector<std::uint8_t> damaged = state;
        for (const Patch& patch : damage.patches) {
            const auto views = backend::parse_packed_model_state(damaged);
            const auto& view = views[patch.entry];
            const std::uint8_t* base = nullptr;
            switch (patch.array) {
            case 0: base = view.packed_codes.data(); break;
            case 1: base = view.block_scale_bytes.data(); break;
            case 2: base = view.scale_codes.data(); break;
            case 3: base = view.second_level_scale_bytes.data(); break;
            default:
                // the entry's header starts 64 + 16 bytes before its codes
                base = view.packed_codes.data() - 80;
                break;
            }
            const std::size_t position =
                static_cast<std::size_t>(base - damaged.data()) +
                patch.offset;
            std::copy(patch.bytes.begin(), patch.bytes.end(),
                      damaged.begin() + static_cast<std::ptrdiff_t>(position));
        }
        // The expected outcome: the length rules first (host), then the
        // oracle's verdict on the content.
        std::string expected;
        bool overflow = false;
        const auto views = backend::parse_packed_model_state(damaged);
        for (const auto& view : views) {
            try {
                static_cast<void>(backend::require_payload_lengths(view));
            } catch (const std::overflow_error& error) {
                expected = error.what();
                overflow = true;
            } catch (const std::invalid_argument& error) {
                expected = error.what();
            }
            if (expected.empty()) {
                expected = oracle_verdict(view);
            }
            if (!expected.empty()) {
                break;
            }
        }
        require(!expected.empty(),
                std::string("damage must be detectable: ") + damage.name);
        try {
            static_cast<void>(backend::hip_load_packed_model_state(damaged));
            throw std::runtime_error(std::string("damaged state accepted: ") +
                                     damage.name);
        } catch (const std::overflow_error& error) {
            require(overflow && expected == error.what(),
                    std::string(damage.name) + ": " + error.what() +
                        " instead of " + expected);
        } catch (const std::invalid_argument& error) {
            require(!overflow && expected == error.what(),
                    std::string(damage.name) + ": " + error.what() +
                        " instead of " + expected);
        }
    }

    // The committed fixture, which the reference's own reader accepted.
    if (const char* golden = std::getenv("RIFTCO_TRANSFORMER_TEST_GOLDEN")) {
        std::ifstream file(std::string(golden) + "/packed_state.bin",
                           std::ios::binary);
        require(file.good(), "tests/golden/packed_state.bin must be readable");
        const std::vector<std::uint8_t> fixture(
            (std::istreambuf_iterator<char>(file)),
            std::istreambuf_iterator<char>());
        auto golden_weights = backend::hip_load_packed_model_state(fixture);
        require(golden_weights.size() == 3, "fixture weight count");
        std::vector<backend::HipPackedWeightSource> sources;
        for (const auto& weight : golden_weights) {
            sources.push_back(
                {weight.shape, weight.block_size, weight.storage.get()});
        }
        require(backend::hip_packed_model_state_bytes(sources) == fixture,
                "the fixture must survive load -> copy byte for byte");
        // its first two entries are the edge weight, as quantised above
        require(std::equal(edge.codes.begin(), edge.codes.end(),
                           golden_weights[0].storage->packed_codes().begin()),
                "fixture codes must equal the oracle quantizer's");
    }
}

void test_out_of_memory_maps_to_bad_alloc() {
    // Only the fake runtime can be told to fail an allocation.
    if (std::getenv("FAKE_RTHIP_CAN_FAIL") == nullptr) {
        return;
    }
    setenv("FAKE_RTHIP_OUT_OF_MEMORY", "1", 1);
    require_throws<std::bad_alloc>(
        [&] {
            // larger than anything the adapter's buffer pool keeps, so the
            // request always reaches the runtime
            static_cast<void>(backend::make_tensor_storage(
                kHip, (std::size_t{1} << 26) + 1, 0.0F));
        },
        "device out-of-memory must surface as std::bad_alloc");
    unsetenv("FAKE_RTHIP_OUT_OF_MEMORY");
}


// One line per file: "ok <entries>", "ValueError <message>" or
// "OverflowError <message>" -- the vocabulary of the Python oracle.
int parse_states(int count, char** paths) {
    for (int index = 0; index < count; ++index) {
        std::ifstream file(paths[index], std::ios::binary);
        if (!file.good()) {
            std::cerr << "cannot read " << paths[index] << '\n';
            return 1;
        }
        const std::vector<std::uint8_t> bytes(
            (std::istreambuf_iterator<char>(file)),
            std::istreambuf_iterator<char>());
        try {
            const std::size_t entries =
                backend::parse_packed_model_state(bytes).size();
            std::cout << "ok " << entries << '\n';
        } catch (const std::invalid_argument& error) {
            std::cout << "ValueError " << error.what() << '\n';
        } catch (const std::overflow_error& error) {
            std::cout << "OverflowError " << error.what() << '\n';
        }
    }
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    try {
        if (argc >= 2 && std::string_view(argv[1]) == "--parse-state") {
            return parse_states(argc - 2, argv + 2);
        }
        const bool expect_unavailable =
            argc == 2 && std::string_view(argv[1]) == "--expect-unavailable";
        if (argc > 2 || (argc == 2 && !expect_unavailable)) {
            throw std::invalid_argument(
                "usage: test_hip_backend [--expect-unavailable]");
        }
        test_identity();
        const bool available =
            riftco_transformer::execution_backend_available(kHip);
        if (expect_unavailable) {
            test_unavailable();
            std::cout << "hip backend tests passed (unavailable path: "
                      << riftco_transformer::
                             execution_backend_unavailability_reason(kHip)
                      << ")\n";
            return 0;
        }
        if (!available) {
            const char* required =
                std::getenv("RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP");
            require(required == nullptr || std::string_view(required) != "1",
                    "hip backend tests require an available backend: " +
                        std::string(riftco_transformer::
                                        execution_backend_unavailability_reason(
                                            kHip)));
            test_unavailable();
            std::cout << "hip backend tests passed (backend unavailable)\n";
            return 0;
        }
        test_accelerator_oracle();
        test_transformer_sized_layer();
        test_forward_group();
        test_adapter_layer();
        test_one_value_tensors();
        test_merged_forwards();
        test_merged_adapter_forwards();
        test_tensor_storage();
        test_dispatch_validation();
        test_packed_model_state();
        test_out_of_memory_maps_to_bad_alloc();
        std::cout << "hip backend tests passed\n";
        return 0;
    } catch (const std::exception& error) {
        std::cerr << "hip backend test failure: " << error.what() << '\n';
        return 1;
    }
}
