// TEST INFRASTRUCTURE ONLY.  A C-callable wrapper around the *compiled
// reference itself*: this file is linked against objects built from the
// reference's own sources where they lie under /root/reference (recipe:
// oracle/Makefile, target _ref) and exposes its CPU backend through plain C
// signatures, so that the restatement in nf4_oracle.c can be diffed against
// it and so that it can serve as the timed CPU baseline.  Nothing of the
// reference is copied here; only its public and internal headers are included.
//
// Entry points used (reference file:line):
//   QuantizedWeight::quantize_nf4 / quantize_nf4_double_quantized /
//   from_packed_nf4 / copy_payload_to_host / dequantize
//       include/riftco_transformer/core/quantized_weight.hpp:69-111
//   dispatch_quantized_linear_forward / _input_backward
//       src/core/backend/nn/quantized_linear/dispatch.hpp:19-27
//   tensor_ops::matmul / transpose_2d / scale / add / broadcast_to
//       include/riftco_transformer/core/tensor_ops.hpp:12-36
//   require_scale_storage, reached through dispatch_quantized_linear_forward
//       src/core/backend/nn/quantized_linear/dispatch.cpp:98-154,203-242
//   Linear (packed weight, attach_lora, forward) and Variable::backward
//       include/riftco_transformer/nn/linear.hpp:16-60,
//       include/riftco_transformer/core/autograd.hpp:31-50

#include "core/backend/adapter.hpp"
#include "core/backend/nn/quantized_linear/dispatch.hpp"
#include "riftco_transformer/core/backend.hpp"
#include "riftco_transformer/core/quantized_weight.hpp"
#include "riftco_transformer/core/tensor.hpp"
#include "riftco_transformer/core/tensor_ops.hpp"
#include "riftco_transformer/nn/linear.hpp"

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <exception>
#include <optional>
#include <random>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace {

using riftco_transformer::ExecutionBackend;
using riftco_transformer::Nf4DoubleQuantizedScales;
using riftco_transformer::Nf4Payload;
using riftco_transformer::QuantizedWeight;
using riftco_transformer::Tensor;
namespace backend = riftco_transformer::backend_detail;

thread_local std::string g_last_error;

// 0 ok, 1 invalid_argument, 2 logic_error, 3 overflow_error, 4 runtime_error,
// 255 anything else -- the first three match nf4_oracle.h's status codes.
template <typename Function> int guarded(Function&& function) noexcept {
    try {
        function();
        g_last_error.clear();
        return 0;
    } catch (const std::invalid_argument& error) {
        g_last_error = error.what();
        return 1;
    } catch (const std::overflow_error& error) {
        g_last_error = error.what();
        return 3;
    } catch (const std::logic_error& error) {
        g_last_error = error.what();
        return 2;
    } catch (const std::runtime_error& error) {
        g_last_error = error.what();
        return 4;
    } catch (const std::exception& error) {
        g_last_error = error.what();
        return 255;
    }
}

Nf4Payload make_payload(
    const std::uint8_t* codes, std::size_t code_bytes, int encoding,
    const float* fp32_scales, std::size_t fp32_count,
    const std::uint8_t* scale_codes, std::size_t scale_code_count,
    const float* second_level, std::size_t second_level_count,
    std::size_t second_level_block, float offset
) {
    Nf4Payload payload;
    payload.packed_codes.assign(codes, codes + code_bytes);
    if (fp32_count != 0) {
        payload.block_scales.assign(fp32_scales, fp32_scales + fp32_count);
    }
    if (encoding == 1) {
        Nf4DoubleQuantizedScales nested;
        nested.scale_codes.assign(scale_codes, scale_codes + scale_code_count);
        nested.second_level_scales.assign(
            second_level, second_level + second_level_count);
        nested.scale_block_size = second_level_block;
        nested.offset = offset;
        payload.double_quantized_scales = std::move(nested);
    }
    return payload;
}

}  // namespace

extern "C" {

const char* nf4ref_last_error(void) { return g_last_error.c_str(); }

// Quantizes values[output_width*input_width] with the reference quantizer.
// encoding 0: fills fp32_scales.  encoding 1: fills scale_codes, second_level
// and *offset.  Buffers are sized by the caller from the block counts.
int nf4ref_quantize(
    const float* values, std::size_t output_width, std::size_t input_width,
    std::size_t block_size, int encoding, std::size_t second_level_block,
    std::uint8_t* codes, float* fp32_scales, std::uint8_t* scale_codes,
    float* second_level, float* offset
) {
    return guarded([&] {
        const std::size_t count = output_width * input_width;
        Tensor source(
            {output_width, input_width},
            std::vector<float>(values, values + count),
            ExecutionBackend::Cpu
        );
        const QuantizedWeight weight = encoding == 1
            ? QuantizedWeight::quantize_nf4_double_quantized(
                  source, block_size, second_level_block)
            : QuantizedWeight::quantize_nf4(source, block_size);
        const Nf4Payload payload = weight.copy_payload_to_host();
        std::copy(payload.packed_codes.begin(), payload.packed_codes.end(),
                  codes);
        if (encoding == 1) {
            const auto& nested = *payload.double_quantized_scales;
            std::copy(nested.scale_codes.begin(), nested.scale_codes.end(),
                      scale_codes);
            std::copy(nested.second_level_scales.begin(),
                      nested.second_level_scales.end(), second_level);
            *offset = nested.offset;
        } else {
            std::copy(payload.block_scales.begin(), payload.block_scales.end(),
                      fp32_scales);
        }
    });
}

// Validates and imports a packed payload exactly as a checkpoint load would
// (QuantizedWeight::from_packed_nf4), then runs mode 0 = dequantize,
// 1 = forward, 2 = input backward on the reference CPU backend.
int nf4ref_run(
    int mode, const float* activations, float* result, std::size_t rows,
    std::size_t input_width, std::size_t output_width, std::size_t block_size,
    const std::uint8_t* codes, std::size_t code_bytes, int encoding,
    const float* fp32_scales, std::size_t fp32_count,
    const std::uint8_t* scale_codes, std::size_t scale_code_count,
    const float* second_level, std::size_t second_level_count,
    std::size_t second_level_block, float offset
) {
    return guarded([&] {
        const QuantizedWeight weight = QuantizedWeight::from_packed_nf4(
            {output_width, input_width}, block_size,
            make_payload(codes, code_bytes, encoding, fp32_scales, fp32_count,
                         scale_codes, scale_code_count, second_level,
                         second_level_count, second_level_block, offset),
            ExecutionBackend::Cpu
        );
        if (mode == 0) {
            const Tensor dense = weight.dequantize();
            const auto data = dense.data();
            std::copy(data.begin(), data.end(), result);
            return;
        }
        const std::size_t in_width = mode == 1 ? input_width : output_width;
        const std::size_t out_width = mode == 1 ? output_width : input_width;
        const Tensor source(
            {rows, in_width},
            std::vector<float>(activations, activations + rows * in_width),
            ExecutionBackend::Cpu
        );
        Tensor target({rows, out_width}, ExecutionBackend::Cpu);
        const backend::QuantizedLinearDimensions dimensions{
            rows, input_width, output_width, block_size};
        if (mode == 1) {
            backend::dispatch_quantized_linear_forward(
                ExecutionBackend::Cpu,
                {backend::tensor_storage(source),
                 backend::quantized_weight_storage(weight),
                 backend::tensor_storage(target), dimensions});
        } else {
            backend::dispatch_quantized_linear_input_backward(
                ExecutionBackend::Cpu,
                {backend::tensor_storage(source),
                 backend::quantized_weight_storage(weight),
                 backend::tensor_storage(target), dimensions});
        }
        const auto data = target.data();
        std::copy(data.begin(), data.end(), result);
    });
}

// Byte accounting of QuantizedWeight::memory_usage() for a quantized tensor of
// element_count zeros-free synthetic values is not needed; this reports the
// nine counters for an imported payload instead (out[9], order of the struct
// in include/riftco_transformer/core/quantized_weight.hpp:52-65).
int nf4ref_memory_usage(
    std::size_t input_width, std::size_t output_width, std::size_t block_size,
    const std::uint8_t* codes, std::size_t code_bytes, int encoding,
    const float* fp32_scales, std::size_t fp32_count,
    const std::uint8_t* scale_codes, std::size_t scale_code_count,
    const float* second_level, std::size_t second_level_count,
    std::size_t second_level_block, float offset, std::size_t* out
) {
    return guarded([&] {
        const QuantizedWeight weight = QuantizedWeight::from_packed_nf4(
            {output_width, input_width}, block_size,
            make_payload(codes, code_bytes, encoding, fp32_scales, fp32_count,
                         scale_codes, scale_code_count, second_level,
                         second_level_count, second_level_block, offset),
            ExecutionBackend::Cpu
        );
        const auto usage = weight.memory_usage();
        out[0] = usage.packed_code_bytes;
        out[1] = usage.scale_bytes;
        out[2] = usage.logical_payload_bytes;
        out[3] = usage.resident_payload_bytes;
        out[4] = usage.fp32_equivalent_bytes;
        out[5] = usage.fp32_scale_bytes;
        out[6] = usage.scale_code_bytes;
        out[7] = usage.second_level_scale_bytes;
        out[8] = usage.scale_offset_bytes;
    });
}

// out[rows, columns] = left[rows, shared] x right[shared, columns] through
// tensor_ops::matmul on the CPU backend.
int nf4ref_matmul(
    const float* left, const float* right, float* out, std::size_t rows,
    std::size_t shared, std::size_t columns
) {
    return guarded([&] {
        const Tensor a({rows, shared},
                       std::vector<float>(left, left + rows * shared),
                       ExecutionBackend::Cpu);
        const Tensor b({shared, columns},
                       std::vector<float>(right, right + shared * columns),
                       ExecutionBackend::Cpu);
        const Tensor c = riftco_transformer::tensor_ops::matmul(a, b);
        const auto data = c.data();
        std::copy(data.begin(), data.end(), out);
    });
}

// The forward of a Linear that holds a packed weight, an optional bias and a
// low-rank adapter, composed from the reference's own tensor operations in
// the order of src/nn/linear.cpp:147-172 and
// src/nn/low_rank_adapter.cpp:126-151 (the autograd wrappers those files use
// call exactly these operations for their forward values).
int nf4ref_lora_linear_forward(
    const float* x, const float* bias_or_null, const float* lora_a,
    const float* lora_b, std::size_t rank, float lora_scale, float* y,
    std::size_t rows, std::size_t input_width, std::size_t output_width,
    std::size_t block_size, const std::uint8_t* codes, std::size_t code_bytes,
    int encoding, const float* fp32_scales, std::size_t fp32_count,
    const std::uint8_t* scale_codes, std::size_t scale_code_count,
    const float* second_level, std::size_t second_level_count,
    std::size_t second_level_block, float offset
) {
    namespace ops = riftco_transformer::tensor_ops;
    return guarded([&] {
        const QuantizedWeight weight = QuantizedWeight::from_packed_nf4(
            {output_width, input_width}, block_size,
            make_payload(codes, code_bytes, encoding, fp32_scales, fp32_count,
                         scale_codes, scale_code_count, second_level,
                         second_level_count, second_level_block, offset),
            ExecutionBackend::Cpu
        );
        const Tensor input({rows, input_width},
                           std::vector<float>(x, x + rows * input_width),
                           ExecutionBackend::Cpu);
        Tensor projected({rows, output_width}, ExecutionBackend::Cpu);
        backend::dispatch_quantized_linear_forward(
            ExecutionBackend::Cpu,
            {backend::tensor_storage(input),
             backend::quantized_weight_storage(weight),
             backend::tensor_storage(projected),
             backend::QuantizedLinearDimensions{rows, input_width,
                                                output_width, block_size}});
        Tensor base = projected;
        if (bias_or_null != nullptr) {
            const Tensor bias(
                {output_width},
                std::vector<float>(bias_or_null, bias_or_null + output_width),
                ExecutionBackend::Cpu);
            base = ops::add(projected,
                            ops::broadcast_to(bias, {rows, output_width}));
        }
        const Tensor a({rank, input_width},
                       std::vector<float>(lora_a, lora_a + rank * input_width),
                       ExecutionBackend::Cpu);
        const Tensor b({output_width, rank},
                       std::vector<float>(lora_b,
                                          lora_b + output_width * rank),
                       ExecutionBackend::Cpu);
        const Tensor reduced = ops::matmul(input, ops::transpose_2d(a));
        const Tensor expanded = ops::matmul(reduced, ops::transpose_2d(b));
        const Tensor result =
            ops::add(base, ops::scale(expanded, lora_scale));
        const auto data = result.data();
        std::copy(data.begin(), data.end(), y);
    });
}

// The dispatcher's verdict on a scale storage held against an expected scale
// count (require_scale_storage, dispatch.cpp:108-154).  The storage is built
// by the CPU adapter itself, which checks nothing, with any combination of
// arrays the caller asks for; the dispatcher then sees it through a forward
// request whose dimensions (one row of 32 x expected_scale_count weights,
// block size 32) make `expected_scale_count` the count it demands.  Packed
// codes and tensors are sized to pass every check that runs before the scale
// check (dispatch.cpp:317-333,203-230), so the first verdict that can differ
// from "ok" is the scale storage's.
int nf4ref_validate_scale_storage(
    int encoding, const float* fp32_scales, std::size_t fp32_count,
    const std::uint8_t* scale_codes, std::size_t scale_code_count,
    const float* second_level, std::size_t second_level_count,
    std::size_t second_level_block, float offset,
    std::size_t expected_scale_count
) {
    return guarded([&] {
        backend::Nf4ScaleStorageData data;
        data.encoding = static_cast<backend::Nf4ScaleEncoding>(encoding);
        if (fp32_count != 0) {
            data.fp32_scales.assign(fp32_scales, fp32_scales + fp32_count);
        }
        if (scale_code_count != 0) {
            data.quantized_scales.assign(scale_codes,
                                         scale_codes + scale_code_count);
        }
        if (second_level_count != 0) {
            data.second_level_scales.assign(
                second_level, second_level + second_level_count);
        }
        data.second_level_block_size = second_level_block;
        data.offset = offset;
        const std::size_t input_width = 32 * expected_scale_count;
        const auto* adapter =
            backend::find_backend_adapter(ExecutionBackend::Cpu);
        const auto weight = adapter->make_nf4_weight_storage(
            std::vector<std::uint8_t>(input_width / 2, 0x77),
            std::move(data));
        const Tensor source({1, input_width}, ExecutionBackend::Cpu);
        Tensor target({1, 1}, ExecutionBackend::Cpu);
        backend::dispatch_quantized_linear_forward(
            ExecutionBackend::Cpu,
            {backend::tensor_storage(source), *weight,
             backend::tensor_storage(target),
             backend::QuantizedLinearDimensions{1, input_width, 1, 32}});
    });
}

// One training step's gradients through a real Linear of the reference: the
// dense weight is packed by the Linear itself (quantize_weight_nf4 or its
// double-quantised form), an adapter is attached and given the caller's A and
// B, forward(x) builds the autograd graph and backward(dy) runs it.  What
// comes back is what the reference leaves on x and on the adapter's two
// parameters, plus the forward value.  scale_block_size == 0: fp32 scales.
int nf4ref_lora_linear_backward(
    const float* dense_weight, std::size_t block_size,
    std::size_t scale_block_size, const float* bias_or_null, const float* x,
    const float* dy, const float* lora_a, const float* lora_b,
    std::size_t rank, float alpha, std::size_t rows, std::size_t input_width,
    std::size_t output_width, float* y, float* dx, float* d_lora_a,
    float* d_lora_b
) {
    using riftco_transformer::Linear;
    using riftco_transformer::Variable;
    return guarded([&] {
        Tensor weight({output_width, input_width},
                      std::vector<float>(
                          dense_weight,
                          dense_weight + output_width * input_width),
                      ExecutionBackend::Cpu);
        std::optional<Linear> linear;
        if (bias_or_null != nullptr) {
            linear.emplace(std::move(weight),
                           Tensor({output_width},
                                  std::vector<float>(
                                      bias_or_null,
                                      bias_or_null + output_width),
                                  ExecutionBackend::Cpu));
        } else {
            linear.emplace(std::move(weight));
        }
        if (scale_block_size == 0) {
            linear->quantize_weight_nf4(block_size);
        } else {
            linear->quantize_weight_nf4_double_quantized(block_size,
                                                         scale_block_size);
        }
        std::mt19937 random(0);
        linear->attach_lora(rank, alpha, random);
        riftco_transformer::Parameter* a = nullptr;
        riftco_transformer::Parameter* b = nullptr;
        const auto adapter_parameters = linear->lora_parameters();
        for (const auto& named : adapter_parameters) {
            if (named.name == "lora_a.weight") {
                a = named.parameter;
            } else if (named.name == "lora_b.weight") {
                b = named.parameter;
            }
        }
        if (a == nullptr || b == nullptr) {
            throw std::runtime_error("adapter parameters not found");
        }
        a->set_value(Tensor({rank, input_width},
                            std::vector<float>(lora_a,
                                               lora_a + rank * input_width),
                            ExecutionBackend::Cpu));
        b->set_value(Tensor({output_width, rank},
                            std::vector<float>(lora_b,
                                               lora_b + output_width * rank),
                            ExecutionBackend::Cpu));
        const Variable input(
            Tensor({rows, input_width},
                   std::vector<float>(x, x + rows * input_width),
                   ExecutionBackend::Cpu),
            true);
        const Variable output = linear->forward(input);
        output.backward(
            Tensor({rows, output_width},
                   std::vector<float>(dy, dy + rows * output_width),
                   ExecutionBackend::Cpu));
        const auto copy = [](const Tensor& tensor, float* target) {
            const auto data = tensor.data();
            std::copy(data.begin(), data.end(), target);
        };
        copy(output.value(), y);
        copy(input.gradient(), dx);
        copy(a->gradient(), d_lora_a);
        copy(b->gradient(), d_lora_b);
    });
}

}  // extern "C"
