// Compiled ONLY where the reference tree is present (the build container):
// hip_adapter.cpp is built with RIFTCO_TRANSFORMER_IN_TREE against the
// reference's own headers and linked with the reference's own objects, which
// proves that the adapter implements every pure virtual of the real
// BackendAdapter (src/core/backend/adapter.hpp:57-80) and accepts the real
// request types.  The hip adapter (on the host-only test runtime) is then
// compared with the reference's CPU adapter on the same packed payload, and a
// capability without a native kernel is checked to run the reference host
// loop on hip storage.

#include "core/backend/adapter.hpp"

#include <cmath>
#include <cstring>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

namespace riftco_transformer::backend_detail {
const BackendAdapter& hip_backend_adapter() noexcept;
}

namespace {

namespace backend = riftco_transformer::backend_detail;

void require(bool condition, const std::string& message) {
    if (!condition) {
        throw std::runtime_error(message);
    }
}

}  // namespace

int main() {
    try {
        const backend::BackendAdapter& hip = backend::hip_backend_adapter();
        const backend::BackendAdapter& cpu = backend::cpu_backend_adapter();
        require(hip.name() == "hip", "adapter name");
        require(hip.is_available(), std::string("hip must be available on the "
                                                "test runtime: ") +
                                        std::string(
                                            hip.unavailability_reason()));

        // A [4 x 64] weight, block 32, hand-made canonical payload.
        constexpr std::size_t out_w = 4, in_w = 64, block = 32, rows = 3;
        std::vector<std::uint8_t> codes(out_w * in_w / 2);
        for (std::size_t i = 0; i < codes.size(); ++i) {
            codes[i] = static_cast<std::uint8_t>((i * 37 + 11) & 0xFF);
        }
        for (const bool nested : {false, true}) {
            backend::Nf4ScaleStorageData scales;
            const std::size_t blocks = out_w * in_w / block;
            if (!nested) {
                for (std::size_t b = 0; b < blocks; ++b) {
                    scales.fp32_scales.push_back(0.25F + 0.125F * b);
                }
            } else {
                scales.encoding =
                    backend::Nf4ScaleEncoding::DoubleQuantizedUInt8;
                for (std::size_t b = 0; b < blocks; ++b) {
                    scales.quantized_scales.push_back(
                        static_cast<std::uint8_t>(40 + 25 * b));
                }
                scales.second_level_scales = {0.5F};
                scales.second_level_block_size = 32;
                scales.offset = 0.75F;
            }
            auto hip_weight = hip.make_nf4_weight_storage(codes, scales);
            auto cpu_weight = cpu.make_nf4_weight_storage(codes, scales);
            require(static_cast<int>(hip_weight->backend()) == 4,
                    "hip storage reports backend id 4");
            require(hip_weight->resident_payload_bytes() ==
                        cpu_weight->resident_payload_bytes(),
                    "resident bytes equal the CPU storage's logical payload");

            std::vector<float> x(rows * in_w), dy(rows * out_w);
            for (std::size_t i = 0; i < x.size(); ++i) {
                x[i] = 0.01F * static_cast<float>(static_cast<int>(i % 23) - 11);
            }
            for (std::size_t i = 0; i < dy.size(); ++i) {
                dy[i] = 0.125F * static_cast<float>(static_cast<int>(i % 7) - 3);
            }
            const backend::QuantizedLinearDimensions dims{rows, in_w, out_w,
                                                          block};
            auto hip_x = hip.make_storage(x);
            auto hip_y = hip.make_storage(rows * out_w, 0.0F);
            auto cpu_x = cpu.make_storage(x);
            auto cpu_y = cpu.make_storage(rows * out_w, 0.0F);
            hip.quantized_linear_forward({*hip_x, *hip_weight, *hip_y, dims});
            cpu.quantized_linear_forward({*cpu_x, *cpu_weight, *cpu_y, dims});
            const auto hy = std::as_const(*hip_y).data();
            const auto cy = std::as_const(*cpu_y).data();
            for (std::size_t i = 0; i < cy.size(); ++i) {
                require(std::fabs(hy[i] - cy[i]) <=
                            3e-5F * std::max(1.0F, std::fabs(cy[i])),
                        "forward differs from the reference CPU adapter");
            }
            auto hip_dy = hip.make_storage(dy);
            auto hip_dx = hip.make_storage(rows * in_w, 0.0F);
            auto cpu_dy = cpu.make_storage(dy);
            auto cpu_dx = cpu.make_storage(rows * in_w, 0.0F);
            hip.quantized_linear_input_backward(
                {*hip_dy, *hip_weight, *hip_dx, dims});
            cpu.quantized_linear_input_backward(
                {*cpu_dy, *cpu_weight, *cpu_dx, dims});
            const auto hd = std::as_const(*hip_dx).data();
            const auto cd = std::as_const(*cpu_dx).data();
            for (std::size_t i = 0; i < cd.size(); ++i) {
                require(std::fabs(hd[i] - cd[i]) <=
                            3e-5F * std::max(1.0F, std::fabs(cd[i])),
                        "input backward differs from the reference CPU "
                        "adapter");
            }

            // a delegated capability: y *= 2 through the reference host loop
            auto scaled = hip.make_storage(rows * out_w, 0.0F);
            hip.scale({*hip_y, *scaled, rows * out_w, 2.0F});
            const auto sy = std::as_const(*scaled).data();
            for (std::size_t i = 0; i < sy.size(); ++i) {
                require(sy[i] == 2.0F * hy[i],
                        "delegated scale must run on hip storage");
            }
        }
        // Dense matmul through the runtime: [2 x 3] x [3 x 2], batch of 2,
        // against the reference CPU adapter on the same values.
        {
            const std::vector<float> left = {1, 2, 3, 4, 5, 6,
                                             -1, 0, 2, 0.5F, 1.5F, -2};
            const std::vector<float> right = {1, 0, 0, 1, 2, -1,
                                              3, 1, -1, 2, 0, 0.25F};
            const backend::MatmulDimensions dimensions{2, 2, 3, 2};
            auto hip_left = hip.make_storage(left);
            auto hip_right = hip.make_storage(right);
            auto hip_out = hip.make_storage(8, 0.0F);
            hip.matmul({*hip_left, *hip_right, *hip_out, dimensions});
            auto cpu_left = cpu.make_storage(left);
            auto cpu_right = cpu.make_storage(right);
            auto cpu_out = cpu.make_storage(8, 0.0F);
            cpu.matmul({*cpu_left, *cpu_right, *cpu_out, dimensions});
            const auto ho = std::as_const(*hip_out).data();
            const auto co = std::as_const(*cpu_out).data();
            for (std::size_t i = 0; i < co.size(); ++i) {
                require(ho[i] == co[i], "matmul differs from the reference "
                                        "CPU adapter");
            }
            require(co[0] == 7.0F && co[1] == -1.0F, "matmul known answer");
        }
        std::cout << "in-tree conformance tests passed\n";
        return 0;
    } catch (const std::exception& error) {
        std::cerr << "in-tree conformance failure: " << error.what() << '\n';
        return 1;
    }
}
