// Function table over the kernel C ABI (include/rthip.h), bound at run time.
//
// The adapter never links librthip.so: it opens it on first use, the way the
// reference's TPU adapter opens its PJRT plugin
// (src/core/backend/adapters/tpu/runtime.hpp:59-67), so that a build of the
// host library does not need ROCm and so that tests can substitute a host-only
// implementation of the same ABI.
//
//   RIFTCO_TRANSFORMER_HIP_LIBRARY             path of the library to open
//                                              (default: librthip.so beside
//                                              this shared object, then the
//                                              loader's search path)
//   RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN  when set to 1, a library that
//                                              exports rthip_test_plugin_marker
//                                              is refused (hardware gates)
#pragma once

#include "../../include/rthip.h"

#include <string>

namespace riftco_transformer::backend_detail {

struct HipRuntime {
    bool available = false;
    bool host_visible_memory = false;
    std::string reason;       // why unavailable
    std::string description;  // device description when available

    decltype(&rthip_last_error) last_error = nullptr;
    decltype(&rthip_malloc) malloc = nullptr;
    decltype(&rthip_free) free = nullptr;
    decltype(&rthip_copy_to_device) copy_to_device = nullptr;
    decltype(&rthip_copy_to_host) copy_to_host = nullptr;
    decltype(&rthip_fill_f32) fill_f32 = nullptr;
    decltype(&rthip_stream_synchronize) stream_synchronize = nullptr;
    decltype(&rthip_nf4_linear_forward) nf4_linear_forward = nullptr;
    decltype(&rthip_nf4_linear_forward_group) nf4_linear_forward_group =
        nullptr;
    decltype(&rthip_nf4_linear_input_backward) nf4_linear_input_backward =
        nullptr;
    decltype(&rthip_nf4_dequantize) nf4_dequantize = nullptr;
    decltype(&rthip_matmul) matmul = nullptr;
    decltype(&rthip_nf4_lora_linear_forward) nf4_lora_linear_forward =
        nullptr;
    decltype(&rthip_nf4_lora_linear_forward_group)
        nf4_lora_linear_forward_group = nullptr;
    decltype(&rthip_lora_backward) lora_backward = nullptr;
    decltype(&rthip_nf4_lora_linear_input_backward)
        nf4_lora_linear_input_backward = nullptr;
    decltype(&rthip_nf4_check_payload) nf4_check_payload = nullptr;
};

// Process-lifetime runtime; loading happens once, on the first call.
[[nodiscard]] const HipRuntime& hip_runtime() noexcept;

}  // namespace riftco_transformer::backend_detail
