// The C ABI's backend identity with the hip backend added: compiled against
// the scratch copy of the reference in which include/riftco_transformer/c_api.h
// defines RT_BACKEND_HIP ((rt_backend)4) and src/c_api/bridge.cpp maps it in
// both directions (checked_backend, :5-41; c_backend, :43-56).
//
// With RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP=1 in the environment an unavailable
// backend is a failure; otherwise the check of the refusal runs instead: the
// bridge must throw BackendUnavailable that names the backend and the reason.
#include "internal/bridge.hpp"

#include "riftco_transformer/core/backend.hpp"

#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <string_view>

namespace {

namespace bridge = riftco_transformer::c_api::detail;
using riftco_transformer::ExecutionBackend;

void require(bool condition, const std::string& message) {
    if (!condition) {
        throw std::runtime_error(message);
    }
}

void test_numeric_identity() {
    require(RT_BACKEND_HIP == static_cast<rt_backend>(4),
            "RT_BACKEND_HIP is 4");
    require(static_cast<rt_backend>(ExecutionBackend::Hip) == RT_BACKEND_HIP,
            "the C constant equals the native enumerator");
    require(bridge::c_backend(ExecutionBackend::Hip) == RT_BACKEND_HIP,
            "native -> C");
    // the neighbours keep their values
    require(bridge::c_backend(ExecutionBackend::Tpu) == RT_BACKEND_TPU &&
                bridge::c_backend(ExecutionBackend::Cpu) == RT_BACKEND_CPU,
            "existing backends are unchanged");
    require(bridge::checked_backend(RT_BACKEND_CPU) == ExecutionBackend::Cpu,
            "C -> native for the CPU backend");
}

void test_unknown_values_are_still_rejected() {
    bool rejected = false;
    try {
        static_cast<void>(bridge::checked_backend(static_cast<rt_backend>(5)));
    } catch (const std::invalid_argument&) {
        rejected = true;
    }
    require(rejected, "backend 5 is unknown");
}

void test_hip_selection(bool required) {
    const bool available =
        riftco_transformer::execution_backend_available(ExecutionBackend::Hip);
    require(available || !required,
            "the hip backend is required here but unavailable: " +
                std::string(riftco_transformer::
                                execution_backend_unavailability_reason(
                                    ExecutionBackend::Hip)));
    if (available) {
        require(bridge::checked_backend(RT_BACKEND_HIP) ==
                    ExecutionBackend::Hip,
                "C -> native for the hip backend");
        std::cout << "hip backend selected through the C ABI\n";
        return;
    }
    bool refused = false;
    try {
        static_cast<void>(bridge::checked_backend(RT_BACKEND_HIP));
    } catch (const bridge::BackendUnavailable& error) {
        const std::string_view message = error.what();
        refused = message.find("hip execution backend is unavailable") !=
                  std::string_view::npos;
    }
    require(refused, "an unavailable hip backend is refused by name");
    std::cout << "hip backend refused through the C ABI (unavailable)\n";
}

}  // namespace

int main() {
    try {
        const char* gate = std::getenv("RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP");
        test_numeric_identity();
        test_unknown_values_are_still_rejected();
        test_hip_selection(gate != nullptr && std::string_view(gate) == "1");
        std::cout << "C ABI backend identity tests passed\n";
        return 0;
    } catch (const std::exception& error) {
        std::cerr << "C ABI backend identity test failure: " << error.what()
                  << '\n';
        return 1;
    }
}
