// The fused Linear of tests/in_tree/apply_hip_backend.py (a packed weight and
// a low-rank adapter on the hip backend: ONE custom-gradient node) against
// the reference's own composition of the same layer on the CPU backend
// (src/nn/linear.cpp:147-172): forward values, the gradients of the input,
// of both adapter matrices and of the bias, and the shape of the autograd
// graph.  Compiled against the edited scratch copy of the reference.
//
// With RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP=1 in the environment an unavailable
// backend is a failure; otherwise the program reports that it skipped.
#include "riftco_transformer/core/autograd.hpp"
#include "riftco_transformer/core/backend.hpp"
#include "riftco_transformer/nn/linear.hpp"

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdlib>
#include <iostream>
#include <memory>
#include <random>
#include <stdexcept>
#include <string>
#include <string_view>
#include <utility>
#include <vector>

namespace {

using riftco_transformer::ExecutionBackend;
using riftco_transformer::Linear;
using riftco_transformer::Tensor;
using riftco_transformer::Variable;

constexpr std::size_t kInputWidth = 192;
constexpr std::size_t kOutputWidth = 40;
constexpr std::size_t kRank = 4;
constexpr float kTolerance = 2.0e-5F;

void require(bool condition, const std::string& message) {
    if (!condition) {
        throw std::runtime_error(message);
    }
}

std::vector<float> wave(std::size_t count, float frequency, float amplitude) {
    std::vector<float> values(count);
    for (std::size_t index = 0; index < count; ++index) {
        values[index] = amplitude *
            std::sin(frequency * static_cast<float>(index) + 0.25F);
    }
    return values;
}

void require_close(const Tensor& actual, const Tensor& expected,
                   const std::string& what) {
    require(actual.shape() == expected.shape(), what + ": shape");
    float largest = 0.0F;
    for (std::size_t index = 0; index < expected.numel(); ++index) {
        largest = std::max(largest, std::fabs(expected.flat(index)));
    }
    for (std::size_t index = 0; index < expected.numel(); ++index) {
        const float difference =
            std::fabs(actual.flat(index) - expected.flat(index));
        require(std::isfinite(actual.flat(index)) &&
                    difference <= kTolerance * std::max(1.0F, largest),
                what + " at " + std::to_string(index) + ": expected " +
                    std::to_string(expected.flat(index)) + ", got " +
                    std::to_string(actual.flat(index)));
    }
}

// A packed layer with an adapter whose B is not the zero it starts as.
std::unique_ptr<Linear> make_layer(bool with_bias, bool double_quantized) {
    Tensor weight({kOutputWidth, kInputWidth},
                  wave(kOutputWidth * kInputWidth, 0.37F, 0.05F),
                  ExecutionBackend::Cpu);
    auto layer = with_bias
        ? std::make_unique<Linear>(
              std::move(weight),
              Tensor({kOutputWidth}, wave(kOutputWidth, 1.3F, 0.1F),
                     ExecutionBackend::Cpu))
        : std::make_unique<Linear>(std::move(weight));
    if (double_quantized) {
        layer->quantize_weight_nf4_double_quantized(64, 256);
    } else {
        layer->quantize_weight_nf4(64);
    }
    std::mt19937 random(2024U);
    layer->attach_lora(kRank, 8.0F, random);
    auto adapters = layer->lora_parameters();
    require(adapters.size() == 2, "A and B");
    bool found_b = false;
    for (auto& adapter : adapters) {
        if (adapter.name.find("lora_b") != std::string::npos) {
            adapter.parameter->set_value(
                Tensor(adapter.parameter->value().shape(),
                       wave(adapter.parameter->value().numel(), 0.91F, 0.2F),
                       ExecutionBackend::Cpu));
            found_b = true;
        }
    }
    require(found_b, "the adapter's B is named lora_b");
    return layer;
}

struct Outcome {
    Tensor output;
    Tensor input_gradient;
    std::vector<Tensor> parameter_gradients;
    std::size_t graph_nodes;
};

Outcome run(Linear& layer, const Tensor::Shape& shape,
            ExecutionBackend backend) {
    std::size_t count = 1;
    for (const std::size_t extent : shape) {
        count *= extent;
    }
    const Variable input(Tensor(shape, wave(count, 0.113F, 1.0F), backend),
                         true);
    const Variable output = layer.forward(input);
    Tensor::Shape upstream_shape = shape;
    upstream_shape.back() = kOutputWidth;
    output.backward(Tensor(upstream_shape,
                           wave(count / kInputWidth * kOutputWidth, 0.71F,
                                0.5F),
                           backend));
    Outcome outcome{output.value().to(ExecutionBackend::Cpu),
                    input.gradient().to(ExecutionBackend::Cpu),
                    {},
                    output.graph_statistics().node_count};
    auto parameters = layer.lora_parameters();
    for (const auto& named : layer.parameters()) {
        parameters.push_back(named);
    }
    for (const auto& named : parameters) {
        outcome.parameter_gradients.push_back(
            named.parameter->gradient().to(ExecutionBackend::Cpu));
        named.parameter->zero_gradient();
    }
    return outcome;
}

void compare(bool with_bias, bool double_quantized,
             const Tensor::Shape& shape) {
    const std::string label =
        std::string(with_bias ? "bias" : "no bias") +
        (double_quantized ? ", nested scales" : ", fp32 scales") + ", " +
        std::to_string(shape.size()) + "-d input";
    const auto on_cpu = make_layer(with_bias, double_quantized);
    const auto on_hip = make_layer(with_bias, double_quantized);
    on_hip->to(ExecutionBackend::Hip);
    const Outcome expected = run(*on_cpu, shape, ExecutionBackend::Cpu);
    const Outcome actual = run(*on_hip, shape, ExecutionBackend::Hip);
    require_close(actual.output, expected.output, label + ": forward");
    require_close(actual.input_gradient, expected.input_gradient,
                  label + ": input gradient");
    require(actual.parameter_gradients.size() ==
                expected.parameter_gradients.size() &&
                actual.parameter_gradients.size() ==
                    (with_bias ? 3U : 2U),
            label + ": parameter count");
    for (std::size_t index = 0; index < actual.parameter_gradients.size();
         ++index) {
        require_close(actual.parameter_gradients[index],
                      expected.parameter_gradients[index],
                      label + ": parameter gradient " +
                          std::to_string(index));
    }
    // the fused node and its leaves: input, A, B (and the bias)
    require(actual.graph_nodes == (with_bias ? 5U : 4U),
            label + ": the hip layer is one graph node, found " +
                std::to_string(actual.graph_nodes));
    require(expected.graph_nodes > actual.graph_nodes,
            label + ": the reference composition has more nodes");
}

}  // namespace

int main() {
    try {
        const char* gate = std::getenv("RIFTCO_TRANSFORMER_TEST_REQUIRE_HIP");
        const bool required =
            gate != nullptr && std::string_view(gate) == "1";
        if (!riftco_transformer::execution_backend_available(
                ExecutionBackend::Hip)) {
            require(!required, "the hip backend is required but unavailable");
            std::cout << "fused Linear tests skipped: hip is unavailable\n";
            return 0;
        }
        for (const bool with_bias : {false, true}) {
            for (const bool double_quantized : {false, true}) {
                compare(with_bias, double_quantized, {5, kInputWidth});
                compare(with_bias, double_quantized, {2, 3, kInputWidth});
                compare(with_bias, double_quantized, {1, kInputWidth});
            }
        }
        std::cout << "fused Linear tests passed\n";
        return 0;
    } catch (const std::exception& error) {
        std::cerr << "fused Linear test failure: " << error.what() << '\n';
        return 1;
    }
}
