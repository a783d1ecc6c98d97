#include "hip_runtime.hpp"

#include <dlfcn.h>

#include <cstdlib>
#include <cstring>
#include <mutex>

namespace riftco_transformer::backend_detail {
namespace {

template <typename Function>
bool bind(void* library, const char* name, Function& target,
          std::string& reason) {
    target = reinterpret_cast<Function>(dlsym(library, name));
    if (target == nullptr) {
        reason = std::string("runtime library does not export ") + name;
        return false;
    }
    return true;
}

std::string default_library_path() {
    Dl_info info{};
    if (dladdr(reinterpret_cast<const void*>(&default_library_path), &info) !=
            0 &&
        info.dli_fname != nullptr) {
        const std::string self(info.dli_fname);
        const std::size_t slash = self.rfind('/');
        if (slash != std::string::npos) {
            return self.substr(0, slash + 1) + "librthip.so";
        }
    }
    return "librthip.so";
}

void load(HipRuntime& runtime) {
    const char* configured = std::getenv("RIFTCO_TRANSFORMER_HIP_LIBRARY");
    const std::string path = configured != nullptr && configured[0] != '\0'
        ? std::string(configured)
        : default_library_path();
    void* library = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
    if (library == nullptr && configured == nullptr) {
        library = dlopen("librthip.so", RTLD_NOW | RTLD_LOCAL);
    }
    if (library == nullptr) {
        const char* error = dlerror();
        runtime.reason = "cannot load the HIP runtime library " + path + ": " +
                         (error != nullptr ? error : "unknown loader error");
        return;
    }
    const char* reject =
        std::getenv("RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN");
    if (reject != nullptr && std::strcmp(reject, "1") == 0 &&
        dlsym(library, "rthip_test_plugin_marker") != nullptr) {
        runtime.reason = "the configured HIP runtime library is a test "
                         "plugin and test plugins are rejected";
        return;
    }

    decltype(&rthip_abi_version) abi_version = nullptr;
    decltype(&rthip_device_count) device_count = nullptr;
    decltype(&rthip_device_description) device_description = nullptr;
    decltype(&rthip_device_memory_host_visible) host_visible = nullptr;
    std::string& reason = runtime.reason;
    if (!bind(library, "rthip_abi_version", abi_version, reason) ||
        !bind(library, "rthip_last_error", runtime.last_error, reason) ||
        !bind(library, "rthip_device_count", device_count, reason) ||
        !bind(library, "rthip_device_description", device_description,
              reason) ||
        !bind(library, "rthip_device_memory_host_visible", host_visible,
              reason) ||
        !bind(library, "rthip_malloc", runtime.malloc, reason) ||
        !bind(library, "rthip_free", runtime.free, reason) ||
        !bind(library, "rthip_copy_to_device", runtime.copy_to_device,
              reason) ||
        !bind(library, "rthip_copy_to_host", runtime.copy_to_host, reason) ||
        !bind(library, "rthip_fill_f32", runtime.fill_f32, reason) ||
        !bind(library, "rthip_stream_synchronize", runtime.stream_synchronize,
              reason) ||
        !bind(library, "rthip_nf4_linear_forward", runtime.nf4_linear_forward,
              reason) ||
        !bind(library, "rthip_nf4_linear_forward_group",
              runtime.nf4_linear_forward_group, reason) ||
        !bind(library, "rthip_nf4_linear_input_backward",
              runtime.nf4_linear_input_backward, reason) ||
        !bind(library, "rthip_nf4_dequantize", runtime.nf4_dequantize,
              reason) ||
        !bind(library, "rthip_matmul", runtime.matmul, reason) ||
        !bind(library, "rthip_nf4_lora_linear_forward",
              runtime.nf4_lora_linear_forward, reason) ||
        !bind(library, "rthip_nf4_lora_linear_forward_group",
              runtime.nf4_lora_linear_forward_group, reason) ||
        !bind(library, "rthip_lora_backward", runtime.lora_backward,
              reason) ||
        !bind(library, "rthip_nf4_lora_linear_input_backward",
              runtime.nf4_lora_linear_input_backward, reason) ||
        !bind(library, "rthip_nf4_check_payload", runtime.nf4_check_payload,
              reason)) {
        return;
    }
    if ((abi_version() >> 16) != RTHIP_ABI_VERSION_MAJOR) {
        runtime.reason = "the HIP runtime library has an incompatible ABI "
                         "major version";
        return;
    }
    int32_t count = 0;
    if (device_count(&count) != RTHIP_OK || count <= 0) {
        runtime.reason = runtime.last_error();
        if (runtime.reason.empty()) {
            runtime.reason = "no MI355X device is visible";
        }
        return;
    }
    char description[256] = "";
    if (device_description(description, sizeof(description)) == RTHIP_OK) {
        runtime.description = description;
    }
    int32_t visible = 0;
    runtime.host_visible_memory =
        host_visible(&visible) == RTHIP_OK && visible != 0;
    runtime.available = true;
    runtime.reason.clear();
}

}  // namespace

const HipRuntime& hip_runtime() noexcept {
    static HipRuntime runtime;
    static std::once_flag once;
    std::call_once(once, [] {
        try {
            load(runtime);
        } catch (...) {
            runtime.available = false;
            runtime.reason = "loading the HIP runtime library failed";
        }
    });
    return runtime;
}

}  // namespace riftco_transformer::backend_detail
