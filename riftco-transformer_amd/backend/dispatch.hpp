// Stand-alone backend registry and the packed-NF4 dispatch entry points, for
// using and testing the `hip` adapter outside the reference tree.  Validation
// rules, exception types and messages restate
// src/core/backend/nn/quantized_linear/dispatch.cpp:18-370 and
// src/core/backend/registry.cpp:83-141; inside the reference tree those files
// are used instead and only gain the `hip` cases.
#pragma once

#include "hip_adapter.hpp"

#include <string_view>

namespace riftco_transformer {

// include/riftco_transformer/core/backend.hpp:20-34
[[nodiscard]] bool execution_backend_available(ExecutionBackend backend) noexcept;
[[nodiscard]] std::string_view execution_backend_unavailability_reason(
    ExecutionBackend backend) noexcept;
[[nodiscard]] std::string_view execution_backend_name(ExecutionBackend backend);

namespace backend_detail {

// src/core/backend/adapter.hpp:99-112
[[nodiscard]] const BackendAdapter* find_backend_adapter(
    ExecutionBackend backend) noexcept;
[[nodiscard]] std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::size_t element_count, float fill_value);
[[nodiscard]] std::unique_ptr<TensorStorage> make_tensor_storage(
    ExecutionBackend backend, std::vector<float> values);

// src/core/backend/nn/quantized_linear/dispatch.hpp:12-27
[[nodiscard]] std::unique_ptr<QuantizedWeightStorage> make_nf4_weight_storage(
    ExecutionBackend backend, std::vector<std::uint8_t> packed_codes,
    Nf4ScaleStorageData scales);
void dispatch_quantized_linear_forward(
    ExecutionBackend backend, const QuantizedLinearForwardRequest& request);
void dispatch_quantized_linear_input_backward(
    ExecutionBackend backend,
    const QuantizedLinearInputBackwardRequest& request);

}  // namespace backend_detail
}  // namespace riftco_transformer
