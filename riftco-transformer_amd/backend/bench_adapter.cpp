// Per-call latency of the packed linear forward THROUGH the backend adapter:
// make_tensor_storage for the output (what src/nn/quantized_linear.cpp:41 does
// for every forward), dispatch_quantized_linear_forward with its validation,
// the kernel, and whatever synchronisation the adapter performs.  Prints one
// line per shape; the environment selects the adapter options
// (RIFTCO_TRANSFORMER_HIP_POOL, RIFTCO_TRANSFORMER_HIP_ASYNC).
//
//   bench_adapter [calls]

#include "dispatch.hpp"

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

namespace {

namespace backend = riftco_transformer::backend_detail;
using riftco_transformer::ExecutionBackend;

constexpr ExecutionBackend kHip = static_cast<ExecutionBackend>(4);

double seconds_since(std::chrono::steady_clock::time_point begin) {
    return std::chrono::duration<double>(std::chrono::steady_clock::now() -
                                         begin)
        .count();
}

}  // namespace

int main(int argc, char** argv) {
    const int calls = argc > 1 ? std::atoi(argv[1]) : 2000;
    if (!riftco_transformer::execution_backend_available(kHip)) {
        std::fprintf(stderr, "hip backend unavailable: %s\n",
                     std::string(riftco_transformer::
                                     execution_backend_unavailability_reason(
                                         kHip))
                         .c_str());
        return 2;
    }
    std::mt19937 random(5);
    struct Shape {
        const char* name;
        std::size_t out_w, in_w;
    };
    for (const Shape shape : {Shape{"q_proj 4096x4096", 4096, 4096},
                              Shape{"gate_proj 11008x4096", 11008, 4096}}) {
        const std::size_t count = shape.out_w * shape.in_w;
        std::vector<std::uint8_t> codes(count / 2);
        for (auto& byte : codes) {
            byte = static_cast<std::uint8_t>(random() & 0xFFU);
        }
        backend::Nf4ScaleStorageData scales;
        scales.fp32_scales.assign(count / 64, 0.05F);
        const auto weight =
            backend::make_nf4_weight_storage(kHip, std::move(codes),
                                             std::move(scales));
        std::vector<float> x(shape.in_w);
        for (auto& value : x) {
            value = static_cast<float>(random() % 2001) / 1000.0F - 1.0F;
        }
        const auto input = backend::make_tensor_storage(kHip, x);
        const backend::QuantizedLinearDimensions dimensions{
            1, shape.in_w, shape.out_w, 64};
        double checksum = 0.0;
        for (int phase = 0; phase < 2; ++phase) {  // 0: warm-up
            const int repeats = phase == 0 ? 20 : calls;
            const auto begin = std::chrono::steady_clock::now();
            std::unique_ptr<backend::TensorStorage> output;
            for (int call = 0; call < repeats; ++call) {
                output = backend::make_tensor_storage(kHip, shape.out_w, 0.0F);
                backend::dispatch_quantized_linear_forward(
                    kHip, {*input, *weight, *output, dimensions});
            }
            // one host read at the end, as a caller that samples a token does
            checksum += std::as_const(*output).data()[0];
            if (phase == 1) {
                std::printf("%-22s %8.2f us per call (%d calls, checksum "
                            "%.6g)\n",
                            shape.name, seconds_since(begin) / repeats * 1e6,
                            repeats, checksum);
            }
        }
    }
    return 0;
}
