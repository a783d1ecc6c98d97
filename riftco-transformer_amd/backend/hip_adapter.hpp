// The `hip` backend adapter: MI355X implementation of the storage and packed
// NF4 linear capabilities of riftco-transformer's BackendAdapter
// (src/core/backend/adapter.hpp:57-80), next to the reference's CPU, Metal,
// CUDA and TPU adapters.
#pragma once

#if defined(RIFTCO_TRANSFORMER_IN_TREE)
#include "core/backend/adapter.hpp"
#else
#include "interface.hpp"
#endif

namespace riftco_transformer::backend_detail {

// ExecutionBackend::Hip.  Spelled as a cast so that this file also compiles
// against a reference tree whose enum has not gained the enumerator yet.
inline constexpr ExecutionBackend kHipBackend =
    static_cast<ExecutionBackend>(4);

// Process-lifetime singleton, like cpu_backend_adapter()
// (src/core/backend/adapters/cpu/adapter.cpp:368-371).
[[nodiscard]] const BackendAdapter& hip_backend_adapter() noexcept;

// Optional extension implemented by hip weight storage: the O(#blocks) scale
// validation that the dispatcher runs before every launch
// (src/core/backend/nn/quantized_linear/dispatch.cpp:98-151) only has to run
// once for storage that can never change.
class ScaleValidationMemo {
public:
    virtual ~ScaleValidationMemo() = default;
    [[nodiscard]] virtual bool scales_validated() const noexcept = 0;
    virtual void mark_scales_validated() const noexcept = 0;
};

}  // namespace riftco_transformer::backend_detail
