// The adapter driven from several host threads at once.  Its methods are
// const and callable from any thread, and the reference selects backends per
// thread (src/core/backend/registry.cpp:17-18; its own test of that:
// tests/core/backend/test_backend.cpp:355-395), so two threads may hold the
// same weight, the same input tensor and the same buffer pool at the same
// moment.  Built with -fsanitize=thread against the host-only test runtime
// (make -C tests/cpp sanitize); what is checked is that every result equals
// the single-threaded one, and that the sanitizer reports no race in
//   * the pool that recycles device buffers (storages created and released
//     in a loop on every thread),
//   * the lazily synchronised host copy of a tensor that several threads read
//     (data() const) while others use it as a kernel input,
//   * the validated-once flag of a weight that every thread dispatches on,
//   * the list of held-back forwards (RIFTCO_TRANSFORMER_HIP_MERGE=1) and the
//     queued execution (RIFTCO_TRANSFORMER_HIP_ASYNC=1).

#include "../../riftco-transformer_amd/backend/dispatch.hpp"

#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <exception>
#include <iostream>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

namespace {

using riftco_transformer::ExecutionBackend;
namespace backend = riftco_transformer::backend_detail;
constexpr ExecutionBackend kHip = backend::kHipBackend;

constexpr std::size_t kOutputWidth = 48;
constexpr std::size_t kInputWidth = 128;
constexpr std::size_t kBlock = 32;
constexpr std::size_t kRows = 3;
constexpr int kThreads = 4;
constexpr int kRounds = 60;

void require(bool condition, const std::string& message) {
    if (!condition) {
        throw std::runtime_error(message);
    }
}

std::unique_ptr<backend::QuantizedWeightStorage> make_weight(bool nested) {
    std::vector<std::uint8_t> codes(kOutputWidth * kInputWidth / 2);
    for (std::size_t i = 0; i < codes.size(); ++i) {
        codes[i] = static_cast<std::uint8_t>((i * 73 + 19) & 0xFF);
    }
    const std::size_t blocks = kOutputWidth * kInputWidth / kBlock;
    backend::Nf4ScaleStorageData scales;
    if (!nested) {
        for (std::size_t b = 0; b < blocks; ++b) {
            scales.fp32_scales.push_back(0.125F + 0.015625F * (b % 13));
        }
    } else {
        scales.encoding = backend::Nf4ScaleEncoding::DoubleQuantizedUInt8;
        for (std::size_t b = 0; b < blocks; ++b) {
            scales.quantized_scales.push_back(
                static_cast<std::uint8_t>(40 + (b * 7) % 200));
        }
        scales.second_level_block_size = 64;
        scales.second_level_scales.assign((blocks + 63) / 64, 0.25F);
        scales.offset = 0.5F;
    }
    return backend::make_nf4_weight_storage(kHip, std::move(codes),
                                            std::move(scales));
}

std::vector<float> make_values(std::size_t count, int salt) {
    std::vector<float> values(count);
    for (std::size_t i = 0; i < count; ++i) {
        values[i] = static_cast<float>(
                        static_cast<int>((i * 31 + salt * 17) % 23) - 11) *
                    0.0625F;
    }
    return values;
}

std::vector<float> forward(const backend::TensorStorage& input,
                           const backend::QuantizedWeightStorage& weight) {
    const auto output =
        backend::make_tensor_storage(kHip, kRows * kOutputWidth, 0.0F);
    backend::dispatch_quantized_linear_forward(
        kHip, {input, weight, *output,
               backend::QuantizedLinearDimensions{kRows, kInputWidth,
                                                  kOutputWidth, kBlock}});
    const auto values = static_cast<const backend::TensorStorage&>(*output)
                            .data();
    return {values.begin(), values.end()};
}

std::vector<float> backward(const backend::TensorStorage& upstream,
                            const backend::QuantizedWeightStorage& weight) {
    const auto gradient =
        backend::make_tensor_storage(kHip, kRows * kInputWidth, 0.0F);
    backend::dispatch_quantized_linear_input_backward(
        kHip, {upstream, weight, *gradient,
               backend::QuantizedLinearDimensions{kRows, kInputWidth,
                                                  kOutputWidth, kBlock}});
    const auto values = static_cast<const backend::TensorStorage&>(*gradient)
                            .data();
    return {values.begin(), values.end()};
}

void same(const std::vector<float>& got, const std::vector<float>& want,
          const std::string& what) {
    require(got.size() == want.size(), what + ": size");
    for (std::size_t i = 0; i < got.size(); ++i) {
        // the same kernel on the same bytes: bit for bit
        require(got[i] == want[i] || (std::isnan(got[i]) && std::isnan(want[i])),
                what + ": element " + std::to_string(i) + " differs");
    }
}

}  // namespace

int main() {
    try {
        require(riftco_transformer::execution_backend_available(kHip),
                "the hip backend must be available (test runtime)");
        for (const bool nested : {false, true}) {
            const auto weight = make_weight(nested);
            // one input and one upstream tensor that every thread reads
            const auto shared_input = backend::make_tensor_storage(
                kHip, make_values(kRows * kInputWidth, 1));
            const auto shared_upstream = backend::make_tensor_storage(
                kHip, make_values(kRows * kOutputWidth, 2));
            const std::vector<float> expected_forward =
                forward(*shared_input, *weight);
            const std::vector<float> expected_backward =
                backward(*shared_upstream, *weight);

            // a second weight that no thread has dispatched on yet: the
            // validated-once flag is first set under contention
            const auto fresh_weight = make_weight(nested);

            // Per round, tensors whose FIRST synchronisation happens under
            // contention: one that only HBM holds (a kernel wrote it; the
            // first host read downloads it) and one that only the host holds
            // (written through data(); the first kernel uploads it).
            std::vector<std::unique_ptr<backend::TensorStorage>> device_only;
            std::vector<std::unique_ptr<backend::TensorStorage>> host_only;
            for (int round = 0; round < kRounds; ++round) {
                auto produced = backend::make_tensor_storage(
                    kHip, kRows * kOutputWidth, 0.0F);
                backend::dispatch_quantized_linear_forward(
                    kHip, {*shared_input, *weight, *produced,
                           backend::QuantizedLinearDimensions{
                               kRows, kInputWidth, kOutputWidth, kBlock}});
                device_only.push_back(std::move(produced));
                auto written = backend::make_tensor_storage(
                    kHip, kRows * kInputWidth, 0.0F);
                const std::vector<float> values =
                    make_values(kRows * kInputWidth, 1);
                const auto span = written->data();
                std::copy(values.begin(), values.end(), span.begin());
                host_only.push_back(std::move(written));
            }
            std::vector<std::atomic<int>> arrived(kRounds);

            std::atomic<int> ready{0};
            std::vector<std::exception_ptr> failures(kThreads);
            std::vector<std::thread> threads;
            for (int t = 0; t < kThreads; ++t) {
                threads.emplace_back([&, t] {
                    try {
                        ++ready;
                        while (ready.load() < kThreads) {
                        }
                        for (int round = 0; round < kRounds; ++round) {
                            ++arrived[round];
                            while (arrived[round].load() < kThreads) {
                            }
                            {
                                const auto seen = static_cast<
                                    const backend::TensorStorage&>(
                                    *device_only[round]).data();
                                same({seen.begin(), seen.end()},
                                     expected_forward,
                                     "first host read of a kernel's output");
                            }
                            same(forward(*host_only[round], *weight),
                                 expected_forward,
                                 "first launch on a host-written tensor");
                            same(forward(*shared_input, *weight),
                                 expected_forward, "shared input forward");
                            same(forward(*shared_input, *fresh_weight),
                                 expected_forward, "fresh weight forward");
                            same(backward(*shared_upstream, *weight),
                                 expected_backward, "shared upstream backward");
                            // a tensor of the thread's own, written through
                            // the host span and read back after a launch
                            auto own = backend::make_tensor_storage(
                                kHip, kRows * kInputWidth, 0.0F);
                            const std::vector<float> values =
                                make_values(kRows * kInputWidth, 1);
                            const auto span = own->data();
                            std::copy(values.begin(), values.end(),
                                      span.begin());
                            same(forward(*own, *weight), expected_forward,
                                 "own input forward");
                            // host reads of the shared tensors while other
                            // threads launch on them
                            const auto seen =
                                static_cast<const backend::TensorStorage&>(
                                    *shared_input)
                                    .data();
                            require(seen.size() == kRows * kInputWidth &&
                                        seen[5] == values[5],
                                    "shared input host read");
                        }
                    } catch (...) {
                        failures[t] = std::current_exception();
                    }
                });
            }
            for (std::thread& thread : threads) {
                thread.join();
            }
            for (const std::exception_ptr& failure : failures) {
                if (failure) {
                    std::rethrow_exception(failure);
                }
            }
        }
        std::cout << "hip backend thread tests passed\n";
        return 0;
    } catch (const std::exception& error) {
        std::cerr << "hip backend thread test failure: " << error.what()
                  << '\n';
        return 1;
    }
}
