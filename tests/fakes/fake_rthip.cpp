// TEST INFRASTRUCTURE ONLY: a host-only implementation of the kernel C ABI
// (include/rthip.h) so that the `hip` adapter, the dispatcher's validation,
// storage accounting and error mapping can be exercised on a machine without a
// GPU.  "Device memory" is host memory and the two products are computed by the
// CPU oracle.  It plays the role tests/fakes/fake_pjrt_tpu.cpp plays for the
// reference's TPU adapter.  The product never loads this library by itself: a
// test selects it with RIFTCO_TRANSFORMER_HIP_LIBRARY, and
// RIFTCO_TRANSFORMER_HIP_REJECT_TEST_PLUGIN=1 makes the adapter refuse it (it
// is recognised by the marker symbol below).

#include "../../include/rthip.h"
#include "../../oracle/nf4_oracle.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

extern "C" void nf4o_linear_forward_rowcached(
    const float*, const uint8_t*, const nf4o_scales*, float*, size_t, size_t,
    size_t, size_t);
extern "C" void nf4o_linear_input_backward_rowcached(
    const float*, const uint8_t*, const nf4o_scales*, float*, size_t, size_t,
    size_t, size_t);

namespace {

thread_local char g_error[256] = "";

rthip_status fail(rthip_status status, const char* message) {
    std::snprintf(g_error, sizeof(g_error), "%s", message);
    return status;
}

bool supported_block(uint64_t block) {
    for (uint64_t candidate = 32; candidate <= 4096; candidate *= 2) {
        if (block == candidate) {
            return true;
        }
    }
    return false;
}

// Rebuilds the oracle's scale view from the six ABI values.
rthip_status make_scales(const void* primary, const float* secondary,
                         int32_t encoding, uint64_t second_level_block,
                         float offset, size_t block_count,
                         nf4o_scales* scales) {
    std::memset(scales, 0, sizeof(*scales));
    scales->encoding = encoding;
    if (primary == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "primary scales must not be null");
    }
    if (encoding == RTHIP_NF4_SCALE_FLOAT32) {
        scales->fp32_scales = static_cast<const float*>(primary);
        scales->fp32_count = block_count;
        return RTHIP_OK;
    }
    if (encoding != RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8) {
        return fail(RTHIP_INVALID_ARGUMENT, "unknown NF4 scale encoding");
    }
    if (!supported_block(second_level_block) || secondary == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "invalid double-quantized scale description");
    }
    scales->quantized_scales = static_cast<const uint8_t*>(primary);
    scales->quantized_count = block_count;
    scales->second_level = secondary;
    scales->second_level_count =
        (block_count + second_level_block - 1) / second_level_block;
    scales->second_level_block = second_level_block;
    scales->offset = offset;
    return RTHIP_OK;
}

rthip_status check_dimensions(uint64_t rows, uint64_t input_width,
                              uint64_t output_width, uint64_t block_size) {
    if (rows == 0 || input_width == 0 || output_width == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear dimensions must be positive");
    }
    if (!supported_block(block_size)) {
        return fail(RTHIP_INVALID_ARGUMENT, "unsupported NF4 block size");
    }
    return RTHIP_OK;
}

}  // namespace

extern "C" {

// Recognised by the adapter's test-plugin gate.
int rthip_test_plugin_marker = 1;

uint32_t rthip_abi_version(void) {
    return (RTHIP_ABI_VERSION_MAJOR << 16) | RTHIP_ABI_VERSION_MINOR;
}
const char* rthip_last_error(void) { return g_error; }

rthip_status rthip_device_count(int32_t* count) {
    if (std::getenv("FAKE_RTHIP_NO_DEVICE") != nullptr) {
        *count = 0;
        return fail(RTHIP_UNAVAILABLE, "no HIP device is visible (fake)");
    }
    *count = 1;
    return RTHIP_OK;
}
rthip_status rthip_device_description(char* buffer, size_t capacity) {
    std::snprintf(buffer, capacity, "host-only test runtime");
    return RTHIP_OK;
}
rthip_status rthip_device_memory_host_visible(int32_t* visible) {
    *visible = std::getenv("FAKE_RTHIP_NO_BAR") != nullptr ? 0 : 1;
    return RTHIP_OK;
}

rthip_status rthip_malloc(void** pointer, size_t bytes) {
    *pointer = nullptr;
    if (bytes == 0) {
        return RTHIP_OK;
    }
    if (std::getenv("FAKE_RTHIP_OUT_OF_MEMORY") != nullptr) {
        return fail(RTHIP_OUT_OF_MEMORY, "device allocation: out of memory");
    }
    *pointer = std::aligned_alloc(256, (bytes + 255) / 256 * 256);
    return *pointer != nullptr ? RTHIP_OK
                               : fail(RTHIP_OUT_OF_MEMORY, "out of memory");
}
rthip_status rthip_free(void* pointer) {
    std::free(pointer);
    return RTHIP_OK;
}
rthip_status rthip_copy_to_device(void* device, const void* host,
                                  size_t bytes) {
    std::memcpy(device, host, bytes);
    return RTHIP_OK;
}
rthip_status rthip_copy_to_host(void* host, const void* device, size_t bytes) {
    std::memcpy(host, device, bytes);
    return RTHIP_OK;
}
rthip_status rthip_fill_f32(float* device, float value, uint64_t count,
                            void*) {
    for (uint64_t index = 0; index < count; ++index) {
        device[index] = value;
    }
    return RTHIP_OK;
}
rthip_status rthip_stream_synchronize(void*) { return RTHIP_OK; }

rthip_status rthip_nf4_select_algorithm(int32_t, uint64_t rows,
                                        uint64_t input_width,
                                        uint64_t output_width,
                                        uint64_t block_size,
                                        int32_t* algorithm) {
    if (const rthip_status status =
            check_dimensions(rows, input_width, output_width, block_size);
        status != RTHIP_OK) {
        return status;
    }
    *algorithm = RTHIP_NF4_ALGORITHM_GENERIC;
    return RTHIP_OK;
}

rthip_status rthip_nf4_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    float* y, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void*) {
    if (x == nullptr || y == nullptr || codes == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "null tensor pointer");
    }
    if (const rthip_status status =
            check_dimensions(rows, input_width, output_width, block_size);
        status != RTHIP_OK) {
        return status;
    }
    const size_t blocks =
        (output_width * input_width + block_size - 1) / block_size;
    nf4o_scales scales;
    if (const rthip_status status =
            make_scales(primary_scales, secondary_scales, encoding,
                        second_level_block, offset, blocks, &scales);
        status != RTHIP_OK) {
        return status;
    }
    nf4o_linear_forward_rowcached(x, codes, &scales, y, rows, input_width,
                                  output_width, block_size);
    if (bias_or_null != nullptr) {
        nf4o_add_bias(y, bias_or_null, rows, output_width);
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_linear_forward_group(
    const float* x, const rthip_nf4_member* members, uint64_t member_count,
    int32_t encoding, uint64_t second_level_block, uint64_t rows,
    uint64_t input_width, uint64_t block_size, void* stream) {
    if (members == nullptr || member_count == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "a group needs members");
    }
    for (uint64_t m = 0; m < member_count; ++m) {
        const rthip_nf4_member& member = members[m];
        if (const rthip_status status = rthip_nf4_linear_forward(
                x, member.codes, member.primary_scales,
                member.secondary_scales, encoding, second_level_block,
                member.offset, member.bias_or_null, member.y, rows,
                input_width, member.output_width, block_size, stream);
            status != RTHIP_OK) {
            return status;
        }
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size, void*) {
    if (dy == nullptr || dx == nullptr || codes == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "null tensor pointer");
    }
    if (const rthip_status status =
            check_dimensions(rows, input_width, output_width, block_size);
        status != RTHIP_OK) {
        return status;
    }
    const size_t blocks =
        (output_width * input_width + block_size - 1) / block_size;
    nf4o_scales scales;
    if (const rthip_status status =
            make_scales(primary_scales, secondary_scales, encoding,
                        second_level_block, offset, blocks, &scales);
        status != RTHIP_OK) {
        return status;
    }
    nf4o_linear_input_backward_rowcached(dy, codes, &scales, dx, rows,
                                         input_width, output_width,
                                         block_size);
    return RTHIP_OK;
}

rthip_status rthip_nf4_linear_input_backward_no_alloc(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream) {
    if (rows > 64) {
        return fail(RTHIP_UNSUPPORTED, "more than 64 rows");
    }
    return rthip_nf4_linear_input_backward(
        dy, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, dx, rows, input_width, output_width,
        block_size, stream);
}

rthip_status rthip_release_workspaces(void*, int32_t) { return RTHIP_OK; }

rthip_status rthip_nf4_linear_forward_with(
    int32_t, const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    float* y, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream) {
    return rthip_nf4_linear_forward(x, codes, primary_scales, secondary_scales,
                                    encoding, second_level_block, offset,
                                    bias_or_null, y, rows, input_width,
                                    output_width, block_size, stream);
}

rthip_status rthip_nf4_linear_input_backward_with(
    int32_t, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset, float* dx,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream) {
    return rthip_nf4_linear_input_backward(
        dy, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, dx, rows, input_width, output_width,
        block_size, stream);
}

rthip_status rthip_nf4_dequantize(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* out,
    uint64_t element_count, uint64_t block_size, void*) {
    if (out == nullptr || codes == nullptr || element_count == 0 ||
        !supported_block(block_size)) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid dequantize arguments");
    }
    const size_t blocks = (element_count + block_size - 1) / block_size;
    nf4o_scales scales;
    if (const rthip_status status =
            make_scales(primary_scales, secondary_scales, encoding,
                        second_level_block, offset, blocks, &scales);
        status != RTHIP_OK) {
        return status;
    }
    nf4o_dequantize(codes, &scales, element_count, block_size, out);
    return RTHIP_OK;
}

rthip_status rthip_matmul(const float* left, const float* right, float* out,
                          uint64_t batch_count, uint64_t rows,
                          uint64_t shared, uint64_t columns, void*) {
    if (left == nullptr || right == nullptr || out == nullptr ||
        batch_count == 0 || rows == 0 || shared == 0 || columns == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid matmul arguments");
    }
    for (uint64_t batch = 0; batch < batch_count; ++batch) {
        nf4o_matmul(left + batch * rows * shared,
                    right + batch * shared * columns,
                    out + batch * rows * columns, rows, shared, columns);
    }
    return RTHIP_OK;
}

rthip_status rthip_lora_reduce(const float* x, const float* lora_a,
                               float* reduced, uint64_t rows,
                               uint64_t input_width, uint64_t lora_rank,
                               void*) {
    if (x == nullptr || lora_a == nullptr || reduced == nullptr ||
        rows == 0 || input_width == 0 || lora_rank == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid LoRA reduce arguments");
    }
    nf4o_matmul_nt(x, lora_a, reduced, rows, input_width, lora_rank);
    return RTHIP_OK;
}

rthip_status rthip_nf4_lora_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    const float* lora_a, const float* lora_b, uint64_t lora_rank,
    float lora_scale, float* reduced, float* y, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream) {
    if (lora_b == nullptr || reduced == nullptr || lora_rank == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid LoRA arguments");
    }
    if (const rthip_status status = rthip_nf4_linear_forward(
            x, codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, bias_or_null, y, rows, input_width,
            output_width, block_size, stream);
        status != RTHIP_OK) {
        return status;
    }
    if (lora_a != nullptr) {
        nf4o_matmul_nt(x, lora_a, reduced, rows, input_width, lora_rank);
    }
    std::vector<float> expanded(rows * output_width);
    nf4o_matmul_nt(reduced, lora_b, expanded.data(), rows, lora_rank,
                   output_width);
    for (size_t index = 0; index < expanded.size(); ++index) {
        y[index] = y[index] + expanded[index] * lora_scale;
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_lora_linear_forward_group(
    const float* x, const rthip_nf4_lora_member* members,
    uint64_t member_count, int32_t encoding, uint64_t second_level_block,
    uint64_t rows, uint64_t input_width, uint64_t block_size, void* stream) {
    if (members == nullptr || member_count == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "a group needs members");
    }
    for (uint64_t m = 0; m < member_count; ++m) {
        const rthip_nf4_lora_member& member = members[m];
        const rthip_nf4_member& base = member.base;
        const rthip_status status =
            member.reduced == nullptr && member.lora_b == nullptr
                ? rthip_nf4_linear_forward(
                      x, base.codes, base.primary_scales,
                      base.secondary_scales, encoding, second_level_block,
                      base.offset, base.bias_or_null, base.y, rows,
                      input_width, base.output_width, block_size, stream)
                : rthip_nf4_lora_linear_forward(
                      x, base.codes, base.primary_scales,
                      base.secondary_scales, encoding, second_level_block,
                      base.offset, base.bias_or_null, member.lora_a,
                      member.lora_b, member.lora_rank, member.lora_scale,
                      member.reduced, base.y, rows, input_width,
                      base.output_width, block_size, stream);
        if (status != RTHIP_OK) {
            return status;
        }
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_lora_linear_forward_with(
    int32_t, const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    const float* lora_a, const float* lora_b, uint64_t lora_rank,
    float lora_scale, float* reduced, float* y, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream) {
    return rthip_nf4_lora_linear_forward(
        x, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, bias_or_null, lora_a, lora_b, lora_rank,
        lora_scale, reduced, y, rows, input_width, output_width, block_size,
        stream);
}

rthip_status rthip_lora_backward(
    const float* dy, const float* x, const float* reduced,
    const float* lora_b, uint64_t lora_rank, float lora_scale,
    float* d_reduced, float* d_lora_a, float* d_lora_b, uint64_t rows,
    uint64_t input_width, uint64_t output_width, void*) {
    if (dy == nullptr || lora_b == nullptr || d_reduced == nullptr ||
        (d_lora_a != nullptr && x == nullptr) ||
        (d_lora_b != nullptr && reduced == nullptr) || rows == 0 ||
        input_width == 0 || output_width == 0 || lora_rank == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "invalid adapter backward arguments");
    }
    std::vector<float> scaled(rows * output_width);
    for (size_t index = 0; index < scaled.size(); ++index) {
        scaled[index] = dy[index] * lora_scale;
    }
    nf4o_matmul(scaled.data(), lora_b, d_reduced, rows, output_width,
                lora_rank);
    for (uint64_t o = 0; d_lora_b != nullptr && o < output_width; ++o) {
        for (uint64_t j = 0; j < lora_rank; ++j) {
            float total = 0.0F;
            for (uint64_t m = 0; m < rows; ++m) {
                total += reduced[m * lora_rank + j] *
                         scaled[m * output_width + o];
            }
            d_lora_b[o * lora_rank + j] = total;
        }
    }
    for (uint64_t j = 0; d_lora_a != nullptr && j < lora_rank; ++j) {
        for (uint64_t i = 0; i < input_width; ++i) {
            float total = 0.0F;
            for (uint64_t m = 0; m < rows; ++m) {
                total += x[m * input_width + i] * d_reduced[m * lora_rank + j];
            }
            d_lora_a[j * input_width + i] = total;
        }
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_lora_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* lora_a,
    const float* d_reduced, uint64_t lora_rank, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream) {
    if (lora_a == nullptr || d_reduced == nullptr || lora_rank == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "invalid adapter input backward arguments");
    }
    if (const rthip_status status = rthip_nf4_linear_input_backward(
            dy, codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, dx, rows, input_width, output_width,
            block_size, stream);
        status != RTHIP_OK) {
        return status;
    }
    std::vector<float> through_a(rows * input_width);
    nf4o_matmul(d_reduced, lora_a, through_a.data(), rows, lora_rank,
                input_width);
    for (size_t index = 0; index < through_a.size(); ++index) {
        dx[index] = dx[index] + through_a[index];
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_lora_linear_input_backward_with(
    int32_t, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* lora_a, const float* d_reduced, uint64_t lora_rank,
    float* dx, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream) {
    return rthip_nf4_lora_linear_input_backward(
        dy, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, lora_a, d_reduced, lora_rank, dx, rows,
        input_width, output_width, block_size, stream);
}

rthip_status rthip_nf4_quantize(
    const float* values, uint64_t element_count, uint64_t block_size,
    int32_t encoding, uint64_t second_level_block, uint8_t* codes,
    void* primary_scales, float* secondary_scales, float* fp32_scale_scratch,
    float* host_offset, void*) {
    if (values == nullptr || codes == nullptr || primary_scales == nullptr ||
        element_count == 0 || !supported_block(block_size)) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid quantize arguments");
    }
    const bool nested = encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8;
    float* scales =
        nested ? fp32_scale_scratch : static_cast<float*>(primary_scales);
    if (scales == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "missing scale buffer");
    }
    if (nf4o_quantize(values, element_count, block_size, codes, scales) !=
        NF4O_OK) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 source values must be finite");
    }
    if (nested) {
        if (secondary_scales == nullptr || host_offset == nullptr ||
            !supported_block(second_level_block)) {
            return fail(RTHIP_INVALID_ARGUMENT, "invalid nested arguments");
        }
        const size_t blocks = (element_count + block_size - 1) / block_size;
        if (nf4o_double_quantize_scales(
                scales, blocks, second_level_block,
                static_cast<uint8_t*>(primary_scales), secondary_scales,
                host_offset) != NF4O_OK) {
            return fail(RTHIP_OVERFLOW, "NF4 scale mean exceeds the FP32 "
                                        "double-quantization range");
        }
    }
    return RTHIP_OK;
}

rthip_status rthip_nf4_check_payload(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, uint64_t element_count,
    uint64_t block_size, void*) {
    if (codes == nullptr || element_count == 0 ||
        !supported_block(block_size)) {
        return fail(RTHIP_INVALID_ARGUMENT, "invalid payload description");
    }
    const size_t blocks = (element_count + block_size - 1) / block_size;
    nf4o_scales scales;
    if (const rthip_status status =
            make_scales(primary_scales, secondary_scales, encoding,
                        second_level_block, offset, blocks, &scales);
        status != RTHIP_OK) {
        return status;
    }
    const char* message = "";
    if (nf4o_validate_payload(element_count, block_size, codes,
                              (element_count + 1) / 2, &scales,
                              &message) != NF4O_OK) {
        return fail(RTHIP_INVALID_ARGUMENT, message);
    }
    return RTHIP_OK;
}

}  // extern "C"
