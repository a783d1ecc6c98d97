// Per-call latency of the packed linear forward THROUGH the backend adapter:
// make_tensor_storage for the output (what src/nn/quantized_linear.cpp:41 does
// for every forward), dispatch_quantized_linear_forward with its validation,
// the kernel, and whatever synchronisation the adapter performs.  Prints one
// line per shape; the environment selects the adapter options
// (RIFTCO_TRANSFORMER_HIP_POOL, RIFTCO_TRANSFORMER_HIP_ASYNC).
//
//   bench_adapter [calls]
//   bench_adapter --packed-state [repeats]
//       restoring one Llama-7B layer (seven projections, block 64) from a
//       checkpoint's packed model state into HBM, and writing it back:
//       hip_load_packed_model_state / hip_packed_model_state_bytes

#include "dispatch.hpp"
#include "packed_state.hpp"

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <string_view>
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

int bench_packed_state(int repeats) {
    struct Shape {
        std::size_t out_w, in_w;
    };
    const Shape layer[] = {{4096, 4096},  {4096, 4096},  {4096, 4096},
                           {4096, 4096},  {11008, 4096}, {11008, 4096},
                           {4096, 11008}};
    std::mt19937 random(9);
    for (const bool nested : {false, true}) {
        std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> weights;
        std::vector<std::vector<std::size_t>> shapes;
        for (const Shape shape : layer) {
            const std::size_t count = shape.out_w * shape.in_w;
            std::vector<std::uint8_t> codes(count / 2);
            for (auto& byte : codes) {
                byte = static_cast<std::uint8_t>(random() & 0xFFU);
            }
            backend::Nf4ScaleStorageData scales;
            if (nested) {
                scales.encoding =
                    backend::Nf4ScaleEncoding::DoubleQuantizedUInt8;
                scales.quantized_scales.resize(count / 64);
                for (auto& code : scales.quantized_scales) {
                    code = static_cast<std::uint8_t>(random() & 0xFFU);
                }
                scales.second_level_scales.assign(count / 64 / 256, 0.01F);
                scales.second_level_block_size = 256;
                scales.offset = 0.05F;
            } else {
                scales.fp32_scales.assign(count / 64, 0.05F);
            }
            weights.push_back(backend::make_nf4_weight_storage(
                kHip, std::move(codes), std::move(scales)));
            shapes.push_back({shape.out_w, shape.in_w});
        }
        std::vector<backend::HipPackedWeightSource> sources;
        for (std::size_t index = 0; index < weights.size(); ++index) {
            sources.push_back({shapes[index], 64, weights[index].get()});
        }
        double write_seconds = 0.0;
        double parse_seconds = 0.0;
        double load_seconds = 0.0;
        std::vector<std::uint8_t> state;
        for (int repeat = -1; repeat < repeats; ++repeat) {  // -1: warm-up
            auto begin = std::chrono::steady_clock::now();
            state = backend::hip_packed_model_state_bytes(sources);
            const double wrote = seconds_since(begin);
            begin = std::chrono::steady_clock::now();
            const auto views = backend::parse_packed_model_state(state);
            const double parsed = seconds_since(begin);
            begin = std::chrono::steady_clock::now();
            const auto loaded = backend::hip_load_packed_model_state(state);
            const double restored = seconds_since(begin);
            if (loaded.size() != views.size()) {
                return 1;
            }
            if (repeat >= 0) {
                write_seconds += wrote;
                parse_seconds += parsed;
                load_seconds += restored;
            }
        }
        const double megabytes = static_cast<double>(state.size()) / 1e6;
        std::printf(
            "packed state, %s scales: %.1f MB; load %.2f ms (%.1f GB/s, of "
            "which parsing %.3f ms); write %.2f ms (%.1f GB/s)\n",
            nested ? "nested" : "fp32", megabytes,
            load_seconds / repeats * 1e3,
            megabytes / 1e3 / (load_seconds / repeats),
            parse_seconds / repeats * 1e3, write_seconds / repeats * 1e3,
            megabytes / 1e3 / (write_seconds / repeats));
    }
    return 0;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc > 1 && std::string_view(argv[1]) == "--packed-state") {
        if (!riftco_transformer::execution_backend_available(kHip)) {
            std::fprintf(stderr, "hip backend unavailable\n");
            return 2;
        }
        return bench_packed_state(argc > 2 ? std::atoi(argv[2]) : 5);
    }
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
    // The decoder's pattern (src/model/decoder_only_transformer.cpp:406-419):
    // three projections of one input per step, outputs alive together.
    {
        constexpr std::size_t width = 4096;
        std::vector<std::unique_ptr<backend::QuantizedWeightStorage>> weights;
        for (int m = 0; m < 3; ++m) {
            std::vector<std::uint8_t> codes(width * width / 2);
            for (auto& byte : codes) {
                byte = static_cast<std::uint8_t>(random() & 0xFFU);
            }
            backend::Nf4ScaleStorageData scales;
            scales.fp32_scales.assign(width * width / 64, 0.05F);
            weights.push_back(backend::make_nf4_weight_storage(
                kHip, std::move(codes), std::move(scales)));
        }
        std::vector<float> x(width);
        for (auto& value : x) {
            value = static_cast<float>(random() % 2001) / 1000.0F - 1.0F;
        }
        const auto input = backend::make_tensor_storage(kHip, x);
        const backend::QuantizedLinearDimensions dimensions{1, width, width,
                                                            64};
        double checksum = 0.0;
        for (int phase = 0; phase < 2; ++phase) {  // 0: warm-up
            const int repeats = phase == 0 ? 20 : calls;
            const auto begin = std::chrono::steady_clock::now();
            std::unique_ptr<backend::TensorStorage> outputs[3];
            for (int call = 0; call < repeats; ++call) {
                for (auto& output : outputs) {
                    output = backend::make_tensor_storage(kHip, width, 0.0F);
                }
                for (int m = 0; m < 3; ++m) {
                    backend::dispatch_quantized_linear_forward(
                        kHip, {*input, *weights[m], *outputs[m], dimensions});
                }
            }
            checksum += std::as_const(*outputs[2]).data()[0];
            if (phase == 1) {
                const auto merged =
                    backend::hip_forward_merge_statistics();
                std::printf("q/k/v 3 x 4096x4096    %8.2f us per projection "
                            "(%d steps, checksum %.6g; merged %llu requests "
                            "into %llu launches)\n",
                            seconds_since(begin) / (3.0 * repeats) * 1e6,
                            repeats, checksum,
                            static_cast<unsigned long long>(merged.requests),
                            static_cast<unsigned long long>(merged.launches));
            }
        }
        // The same block with unmerged rank-16 adapters on the query and value
        // projections (what Linear::forward of such a layer calls on hip).
        namespace detail = riftco_transformer::backend_detail;
        constexpr std::size_t rank = 16;
        std::vector<float> a_values(rank * width), b_values(width * rank);
        for (auto& value : a_values) {
            value = static_cast<float>(random() % 2001) / 20000.0F - 0.05F;
        }
        for (auto& value : b_values) {
            value = static_cast<float>(random() % 2001) / 20000.0F - 0.05F;
        }
        const auto lora_a = backend::make_tensor_storage(kHip, a_values);
        const auto lora_b = backend::make_tensor_storage(kHip, b_values);
        for (int phase = 0; phase < 2; ++phase) {  // 0: warm-up
            const int repeats = phase == 0 ? 20 : calls;
            const auto before = backend::hip_forward_merge_statistics();
            const auto begin = std::chrono::steady_clock::now();
            std::unique_ptr<backend::TensorStorage> outputs[3];
            std::unique_ptr<backend::TensorStorage> products[3];
            for (int call = 0; call < repeats; ++call) {
                for (int m = 0; m < 3; ++m) {
                    outputs[m] = backend::make_tensor_storage(kHip, width, 0.0F);
                    products[m] = backend::make_tensor_storage(kHip, rank, 0.0F);
                }
                for (int m = 0; m < 3; ++m) {
                    if (m == 1) {
                        backend::dispatch_quantized_linear_forward(
                            kHip,
                            {*input, *weights[m], *outputs[m], dimensions});
                    } else {
                        detail::hip_quantized_linear_adapter_forward(
                            {*input, *weights[m], nullptr, *lora_a, *lora_b,
                             rank, 2.0F, *products[m], *outputs[m],
                             dimensions});
                    }
                }
            }
            checksum += std::as_const(*outputs[2]).data()[0];
            if (phase == 1) {
                const auto merged = backend::hip_forward_merge_statistics();
                std::printf("q/k/v, adapters on q,v %8.2f us per projection "
                            "(%d steps, checksum %.6g; %llu requests in %llu "
                            "launches)\n",
                            seconds_since(begin) / (3.0 * repeats) * 1e6,
                            repeats, checksum,
                            static_cast<unsigned long long>(
                                merged.requests - before.requests),
                            static_cast<unsigned long long>(
                                merged.launches - before.launches));
            }
        }
    }
    return 0;
}
