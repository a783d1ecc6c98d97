/*
 * TEST INFRASTRUCTURE ONLY -- see nf4_oracle.h.  Plain C restatement of the
 * reference CPU backend's packed NF4 linear path.  Build with
 * -ffp-contract=off: the reference's x86-64 build has no fused multiply-add,
 * and bit-for-bit agreement with it depends on that.
 */
#include "nf4_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* src/core/quantization/nf4.cpp:14-31 (identical literals:
 * src/core/backend/nn/quantized_linear/reference/operations.cpp:13-30). */
static const float k_codebook[16] = {
    -1.0F,
    -0.6961928009986877F,
    -0.5250730514526367F,
    -0.39491748809814453F,
    -0.28444138169288635F,
    -0.18477343022823334F,
    -0.09105003625154495F,
    0.0F,
    0.07958029955625534F,
    0.16093020141124725F,
    0.24611230194568634F,
    0.33791524171829224F,
    0.44070982933044434F,
    0.5626170039176941F,
    0.7229568362236023F,
    1.0F,
};

const float* nf4o_codebook(void) { return k_codebook; }

size_t nf4o_scale_count(const nf4o_scales* scales) {
    return scales->encoding == NF4O_SCALE_FLOAT32 ? scales->fp32_count
                                                  : scales->quantized_count;
}

int nf4o_block_size_supported(size_t block_size) {
    /* nf4.cpp:39-53: the closed set 32, 64, ..., 4096 */
    size_t candidate;
    for (candidate = 32; candidate <= 4096; candidate *= 2) {
        if (block_size == candidate) {
            return 1;
        }
    }
    return 0;
}

size_t nf4o_block_count(size_t element_count, size_t block_size) {
    return element_count / block_size + (element_count % block_size != 0);
}

size_t nf4o_packed_byte_count(size_t element_count) {
    return element_count / 2 + (element_count % 2 != 0);
}

uint8_t nf4o_nearest_code(float normalized_value) {
    uint8_t best_code = 0;
    float best_distance = fabsf(normalized_value - k_codebook[0]);
    uint8_t code;
    for (code = 1; code < 16; ++code) {
        const float distance = fabsf(normalized_value - k_codebook[code]);
        if (distance < best_distance) {
            best_distance = distance;
            best_code = code;
        }
    }
    return best_code;
}

uint8_t nf4o_unpack_code(const uint8_t* packed, size_t flat_index) {
    const uint8_t byte = packed[flat_index / 2];
    return (flat_index % 2 == 0) ? (uint8_t)(byte & 0x0FU)
                                 : (uint8_t)(byte >> 4U);
}

void nf4o_pack_code(uint8_t* packed, size_t flat_index, uint8_t code) {
    const size_t byte_index = flat_index / 2;
    const unsigned shift = (flat_index % 2 == 0) ? 0U : 4U;
    const uint8_t mask = (uint8_t)(0x0FU << shift);
    packed[byte_index] = (uint8_t)((packed[byte_index] & (uint8_t)~mask) |
                                   (uint8_t)((code & 0x0FU) << shift));
}

int nf4o_quantize(const float* values, size_t n, size_t block_size,
                  uint8_t* codes, float* scales) {
    const size_t blocks = nf4o_block_count(n, block_size);
    size_t block;
    memset(codes, 0, nf4o_packed_byte_count(n));
    for (block = 0; block < blocks; ++block) {
        const size_t begin = block * block_size;
        const size_t end = begin + block_size < n ? begin + block_size : n;
        float scale = 0.0F;
        size_t index;
        for (index = begin; index < end; ++index) {
            float magnitude;
            if (!isfinite(values[index])) {
                return NF4O_INVALID_ARGUMENT;
            }
            magnitude = fabsf(values[index]);
            /* std::max(scale, |w|): keeps scale unless scale < |w| */
            scale = scale < magnitude ? magnitude : scale;
        }
        scales[block] = scale;
        for (index = begin; index < end; ++index) {
            const uint8_t code =
                scale == 0.0F ? (uint8_t)7
                              : nf4o_nearest_code(values[index] / scale);
            nf4o_pack_code(codes, index, code);
        }
    }
    return NF4O_OK;
}

int nf4o_double_quantize_scales(const float* block_scales, size_t block_count,
                                size_t scale_block_size, uint8_t* scale_codes,
                                float* second_level, float* offset_out) {
    const size_t groups = nf4o_block_count(block_count, scale_block_size);
    double sum = 0.0;
    float offset;
    size_t index;
    size_t group;
    for (index = 0; index < block_count; ++index) {
        scale_codes[index] = 128;
        sum += (double)block_scales[index];
    }
    for (group = 0; group < groups; ++group) {
        second_level[group] = 0.0F;
    }
    offset = (float)(sum / (double)block_count);
    *offset_out = offset;
    if (!isfinite(offset)) {
        return NF4O_OVERFLOW;
    }
    for (group = 0; group < groups; ++group) {
        const size_t begin = group * scale_block_size;
        const size_t end = begin + scale_block_size < block_count
                               ? begin + scale_block_size
                               : block_count;
        float absmax = 0.0F;
        for (index = begin; index < end; ++index) {
            const float distance = fabsf(block_scales[index] - offset);
            absmax = absmax < distance ? distance : absmax;
        }
        second_level[group] = absmax;
        if (absmax == 0.0F) {
            continue;
        }
        for (index = begin; index < end; ++index) {
            const float normalized = (block_scales[index] - offset) / absmax;
            const float scaled = normalized * 127.0F;
            const float rounded =
                scaled >= 0.0F ? floorf(scaled + 0.5F) : ceilf(scaled - 0.5F);
            int centered = (int)rounded;
            centered = centered < -127 ? -127 : (centered > 127 ? 127 : centered);
            scale_codes[index] = (uint8_t)(centered + 128);
        }
    }
    return NF4O_OK;
}

float nf4o_decode_scale(const nf4o_scales* scales, size_t scale_index) {
    int centered_code;
    float factor;
    float delta;
    float reconstructed;
    if (scales->encoding == NF4O_SCALE_FLOAT32) {
        return scales->fp32_scales[scale_index];
    }
    centered_code = (int)scales->quantized_scales[scale_index] - 128;
    factor = (float)centered_code / 127.0F;
    delta = scales->second_level[scale_index / scales->second_level_block] *
            factor;
    if (delta > 0.0F && scales->offset > FLT_MAX - delta) {
        return FLT_MAX;
    }
    reconstructed = scales->offset + delta;
    return reconstructed > 0.0F ? reconstructed : 0.0F;
}

/* decode_nf4, reference/operations.cpp:32-45 */
static float decode_weight(const uint8_t* codes, const nf4o_scales* scales,
                           size_t block_size, size_t flat_index) {
    const uint8_t packed = codes[flat_index / 2];
    const uint8_t code = (flat_index & 1U) == 0U ? (uint8_t)(packed & 0x0FU)
                                                 : (uint8_t)(packed >> 4U);
    return k_codebook[code] *
           nf4o_decode_scale(scales, flat_index / block_size);
}

void nf4o_dequantize(const uint8_t* codes, const nf4o_scales* scales,
                     size_t element_count, size_t block_size, float* out) {
    size_t index;
    for (index = 0; index < element_count; ++index) {
        /* quantized_weight.cpp:465: scale * codebook[code]; the product of two
         * floats is commutative, so this equals decode_weight bit for bit. */
        out[index] = nf4o_decode_scale(scales, index / block_size) *
                     k_codebook[nf4o_unpack_code(codes, index)];
    }
}

void nf4o_linear_forward(const float* x, const uint8_t* codes,
                         const nf4o_scales* scales, float* y, size_t rows,
                         size_t input_width, size_t output_width,
                         size_t block_size) {
    size_t row;
    for (row = 0; row < rows; ++row) {
        const size_t input_offset = row * input_width;
        const size_t output_offset = row * output_width;
        size_t output_column;
        for (output_column = 0; output_column < output_width; ++output_column) {
            const size_t weight_offset = output_column * input_width;
            float total = 0.0F;
            size_t input_column;
            for (input_column = 0; input_column < input_width; ++input_column) {
                total += x[input_offset + input_column] *
                         decode_weight(codes, scales, block_size,
                                       weight_offset + input_column);
            }
            y[output_offset + output_column] = total;
        }
    }
}

void nf4o_linear_input_backward(const float* dy, const uint8_t* codes,
                                const nf4o_scales* scales, float* dx,
                                size_t rows, size_t input_width,
                                size_t output_width, size_t block_size) {
    size_t row;
    for (row = 0; row < rows; ++row) {
        const size_t upstream_offset = row * output_width;
        const size_t gradient_offset = row * input_width;
        size_t input_column;
        for (input_column = 0; input_column < input_width; ++input_column) {
            float total = 0.0F;
            size_t output_column;
            for (output_column = 0; output_column < output_width;
                 ++output_column) {
                const size_t weight_index =
                    output_column * input_width + input_column;
                total += dy[upstream_offset + output_column] *
                         decode_weight(codes, scales, block_size, weight_index);
            }
            dx[gradient_offset + input_column] = total;
        }
    }
}

/*
 * Same results bit for bit as the two functions above, with the weight row
 * decoded once instead of once per multiply.  Each output still accumulates
 * the identical sequence of rounded products in the identical order, so only
 * the run time differs.  Used where a parity test needs more rows than the
 * faithful loops finish in seconds; never as the timed CPU baseline.
 */
void nf4o_linear_forward_rowcached(const float* x, const uint8_t* codes,
                                   const nf4o_scales* scales, float* y,
                                   size_t rows, size_t input_width,
                                   size_t output_width, size_t block_size) {
    float* weight_row = (float*)malloc(input_width * sizeof(float));
    size_t output_column;
    if (weight_row == NULL) {
        abort();
    }
    for (output_column = 0; output_column < output_width; ++output_column) {
        const size_t weight_offset = output_column * input_width;
        size_t input_column;
        size_t row;
        for (input_column = 0; input_column < input_width; ++input_column) {
            weight_row[input_column] = decode_weight(
                codes, scales, block_size, weight_offset + input_column);
        }
        for (row = 0; row < rows; ++row) {
            const float* input = x + row * input_width;
            float total = 0.0F;
            for (input_column = 0; input_column < input_width; ++input_column) {
                total += input[input_column] * weight_row[input_column];
            }
            y[row * output_width + output_column] = total;
        }
    }
    free(weight_row);
}

void nf4o_linear_input_backward_rowcached(const float* dy,
                                          const uint8_t* codes,
                                          const nf4o_scales* scales, float* dx,
                                          size_t rows, size_t input_width,
                                          size_t output_width,
                                          size_t block_size) {
    float* weight_row = (float*)malloc(input_width * sizeof(float));
    size_t output_column;
    size_t index;
    if (weight_row == NULL) {
        abort();
    }
    for (index = 0; index < rows * input_width; ++index) {
        dx[index] = 0.0F;
    }
    for (output_column = 0; output_column < output_width; ++output_column) {
        const size_t weight_offset = output_column * input_width;
        size_t input_column;
        size_t row;
        for (input_column = 0; input_column < input_width; ++input_column) {
            weight_row[input_column] = decode_weight(
                codes, scales, block_size, weight_offset + input_column);
        }
        for (row = 0; row < rows; ++row) {
            const float upstream = dy[row * output_width + output_column];
            float* gradient = dx + row * input_width;
            for (input_column = 0; input_column < input_width; ++input_column) {
                gradient[input_column] += upstream * weight_row[input_column];
            }
        }
    }
    free(weight_row);
}

void nf4o_add_bias(float* y, const float* bias, size_t rows,
                   size_t output_width) {
    size_t row;
    size_t column;
    for (row = 0; row < rows; ++row) {
        for (column = 0; column < output_width; ++column) {
            y[row * output_width + column] += bias[column];
        }
    }
}

void nf4o_matmul(const float* left, const float* right, float* out,
                 size_t rows, size_t shared, size_t columns) {
    size_t row;
    size_t column;
    size_t inner;
    for (row = 0; row < rows; ++row) {
        for (column = 0; column < columns; ++column) {
            float total = 0.0F;
            for (inner = 0; inner < shared; ++inner) {
                total += left[row * shared + inner] *
                         right[inner * columns + column];
            }
            out[row * columns + column] = total;
        }
    }
}

void nf4o_matmul_nt(const float* left, const float* right_t, float* out,
                    size_t rows, size_t shared, size_t columns) {
    size_t row;
    size_t column;
    size_t inner;
    for (row = 0; row < rows; ++row) {
        for (column = 0; column < columns; ++column) {
            float total = 0.0F;
            for (inner = 0; inner < shared; ++inner) {
                total += left[row * shared + inner] *
                         right_t[column * shared + inner];
            }
            out[row * columns + column] = total;
        }
    }
}

void nf4o_lora_linear_forward(const float* x, const uint8_t* codes,
                              const nf4o_scales* scales, const float* bias,
                              const float* lora_a, const float* lora_b,
                              size_t rank, float lora_scale, float* y,
                              size_t rows, size_t input_width,
                              size_t output_width, size_t block_size) {
    float* reduced = (float*)malloc(sizeof(float) * rows * rank);
    float* expanded = (float*)malloc(sizeof(float) * rows * output_width);
    size_t index;
    nf4o_linear_forward_rowcached(x, codes, scales, y, rows, input_width,
                                  output_width, block_size);
    if (bias != NULL) {
        nf4o_add_bias(y, bias, rows, output_width);
    }
    nf4o_matmul_nt(x, lora_a, reduced, rows, input_width, rank);
    nf4o_matmul_nt(reduced, lora_b, expanded, rows, rank, output_width);
    for (index = 0; index < rows * output_width; ++index) {
        const float scaled = expanded[index] * lora_scale;
        y[index] = y[index] + scaled;
    }
    free(reduced);
    free(expanded);
}

void nf4o_lora_linear_backward(const float* dy, const float* x,
                               const uint8_t* codes, const nf4o_scales* scales,
                               const float* lora_a, const float* lora_b,
                               size_t rank, float lora_scale, float* dx,
                               float* d_lora_a, float* d_lora_b, size_t rows,
                               size_t input_width, size_t output_width,
                               size_t block_size) {
    float* reduced = (float*)malloc(sizeof(float) * rows * rank);
    float* scaled = (float*)malloc(sizeof(float) * rows * output_width);
    float* d_reduced = (float*)malloc(sizeof(float) * rows * rank);
    float* adapter_dx = (float*)malloc(sizeof(float) * rows * input_width);
    size_t index;
    size_t row;
    size_t column;
    size_t slot;
    /* forward value the second matmul's closure keeps: x . A^T */
    nf4o_matmul_nt(x, lora_a, reduced, rows, input_width, rank);
    /* operator*(value, scalar): upstream times the constant, elementwise */
    for (index = 0; index < rows * output_width; ++index) {
        scaled[index] = dy[index] * lora_scale;
    }
    /* matmul(reduced, B^T): left gets upstream . (B^T)^T = scaled . B */
    nf4o_matmul(scaled, lora_b, d_reduced, rows, output_width, rank);
    /* ... right gets reduced^T . upstream, [rank, output]; transpose_2d
     * hands its transpose to B */
    for (column = 0; column < output_width; ++column) {
        for (slot = 0; slot < rank; ++slot) {
            float total = 0.0F;
            for (row = 0; row < rows; ++row) {
                total += reduced[row * rank + slot] *
                         scaled[row * output_width + column];
            }
            d_lora_b[column * rank + slot] = 0.0F + total;
        }
    }
    /* matmul(x, A^T): left gets d_reduced . A, right x^T . d_reduced,
     * [input, rank], whose transpose goes to A */
    nf4o_matmul(d_reduced, lora_a, adapter_dx, rows, rank, input_width);
    for (slot = 0; slot < rank; ++slot) {
        for (column = 0; column < input_width; ++column) {
            float total = 0.0F;
            for (row = 0; row < rows; ++row) {
                total += x[row * input_width + column] *
                         d_reduced[row * rank + slot];
            }
            d_lora_a[slot * input_width + column] = 0.0F + total;
        }
    }
    /* quantized_linear's closure, then one rounded addition per element as
     * the two contributions meet at x */
    nf4o_linear_input_backward(dy, codes, scales, dx, rows, input_width,
                               output_width, block_size);
    for (index = 0; index < rows * input_width; ++index) {
        dx[index] = (0.0F + dx[index]) + adapter_dx[index];
    }
    free(reduced);
    free(scaled);
    free(d_reduced);
    free(adapter_dx);
}

size_t nf4o_scale_payload_bytes(const nf4o_scales* scales) {
    if (scales->encoding == NF4O_SCALE_FLOAT32) {
        return scales->fp32_count * sizeof(float);
    }
    return scales->quantized_count +
           scales->second_level_count * sizeof(float) + sizeof(float);
}

static int fail(const char** message, const char* text, int status) {
    if (message != NULL) {
        *message = text;
    }
    return status;
}

int nf4o_validate_payload(size_t element_count, size_t block_size,
                          const uint8_t* codes, size_t code_bytes,
                          const nf4o_scales* scales, const char** message) {
    const size_t expected_bytes = nf4o_packed_byte_count(element_count);
    const size_t expected_blocks = nf4o_block_count(element_count, block_size);
    const int double_quantized =
        scales->encoding == NF4O_SCALE_DOUBLE_QUANTIZED_UINT8;
    size_t block;
    if (message != NULL) {
        *message = "";
    }
    if (code_bytes != expected_bytes) {
        return fail(message,
                    "NF4 packed byte count does not match the weight shape",
                    NF4O_INVALID_ARGUMENT);
    }
    if (element_count % 2 != 0 && (codes[code_bytes - 1] & 0xF0U) != 0) {
        return fail(message, "NF4 unused high nibble must be zero",
                    NF4O_INVALID_ARGUMENT);
    }
    if (!double_quantized) {
        if (scales->fp32_count != expected_blocks) {
            return fail(message,
                        "NF4 scale count does not match the weight shape and "
                        "block size",
                        NF4O_INVALID_ARGUMENT);
        }
    } else {
        size_t group;
        if (scales->fp32_count != 0) {
            return fail(message,
                        "double-quantized NF4 payload must not retain FP32 "
                        "block scales",
                        NF4O_INVALID_ARGUMENT);
        }
        if (!nf4o_block_size_supported(scales->second_level_block)) {
            return fail(message,
                        "NF4 block size must be one of 32, 64, 128, 256, 512, "
                        "1024, 2048, or 4096",
                        NF4O_INVALID_ARGUMENT);
        }
        if (scales->quantized_count != expected_blocks) {
            return fail(message,
                        "double-quantized NF4 scale-code count does not match "
                        "the weight",
                        NF4O_INVALID_ARGUMENT);
        }
        if (scales->second_level_count !=
            nf4o_block_count(expected_blocks, scales->second_level_block)) {
            return fail(message,
                        "double-quantized NF4 second-level scale count is "
                        "invalid",
                        NF4O_INVALID_ARGUMENT);
        }
        if (!isfinite(scales->offset) || scales->offset < 0.0F) {
            return fail(message,
                        "double-quantized NF4 scale offset must be finite and "
                        "nonnegative",
                        NF4O_INVALID_ARGUMENT);
        }
        for (group = 0; group < scales->second_level_count; ++group) {
            const float scale = scales->second_level[group];
            if (!isfinite(scale) || scale < 0.0F) {
                return fail(message,
                            "NF4 second-level scales must be finite and "
                            "nonnegative",
                            NF4O_INVALID_ARGUMENT);
            }
        }
    }
    for (block = 0; block < expected_blocks; ++block) {
        const float scale = nf4o_decode_scale(scales, block);
        size_t begin;
        size_t end;
        size_t index;
        if (!isfinite(scale) || scale < 0.0F) {
            return fail(message,
                        "NF4 block scales must be finite and nonnegative",
                        NF4O_INVALID_ARGUMENT);
        }
        if (scale != 0.0F || double_quantized) {
            continue;
        }
        begin = block * block_size;
        end = begin + block_size < element_count ? begin + block_size
                                                 : element_count;
        for (index = begin; index < end; ++index) {
            if (nf4o_unpack_code(codes, index) != 7) {
                return fail(message,
                            "zero-scale NF4 blocks must use canonical zero "
                            "code 7",
                            NF4O_INVALID_ARGUMENT);
            }
        }
    }
    return NF4O_OK;
}

static int finite_nonnegative(const float* values, size_t count) {
    size_t index;
    for (index = 0; index < count; ++index) {
        if (!isfinite(values[index]) || values[index] < 0.0F) {
            return 0;
        }
    }
    return 1;
}

int nf4o_validate_scale_storage(const nf4o_scales* scales,
                                size_t expected_scale_count,
                                const char** message) {
    size_t index;
    if (message != NULL) {
        *message = "";
    }
    if (scales->encoding == NF4O_SCALE_FLOAT32) {
        if (scales->fp32_count != expected_scale_count ||
            scales->quantized_count != 0 || scales->second_level_count != 0 ||
            scales->second_level_block != 0 || scales->offset != 0.0F) {
            return fail(message,
                        "legacy NF4 scale storage has an invalid "
                        "representation",
                        NF4O_INVALID_ARGUMENT);
        }
        if (!finite_nonnegative(scales->fp32_scales, scales->fp32_count)) {
            return fail(message,
                        "NF4 block scales must be finite and non-negative",
                        NF4O_INVALID_ARGUMENT);
        }
        return NF4O_OK;
    }
    if (scales->encoding == NF4O_SCALE_DOUBLE_QUANTIZED_UINT8) {
        if (scales->fp32_count != 0 ||
            scales->quantized_count != expected_scale_count ||
            scales->second_level_block == 0 ||
            !nf4o_block_size_supported(scales->second_level_block) ||
            !isfinite(scales->offset) || scales->offset < 0.0F) {
            return fail(message,
                        "double-quantized NF4 scale storage has an invalid "
                        "representation",
                        NF4O_INVALID_ARGUMENT);
        }
        if (scales->second_level_count !=
            1 + (expected_scale_count - 1) / scales->second_level_block) {
            return fail(message,
                        "double-quantized NF4 second-level scale count is "
                        "invalid",
                        NF4O_INVALID_ARGUMENT);
        }
        if (!finite_nonnegative(scales->second_level,
                                scales->second_level_count)) {
            return fail(message,
                        "NF4 block scales must be finite and non-negative",
                        NF4O_INVALID_ARGUMENT);
        }
        for (index = 0; index < expected_scale_count; ++index) {
            if (!isfinite(nf4o_decode_scale(scales, index))) {
                return fail(message,
                            "double-quantized NF4 scale reconstruction is "
                            "nonfinite",
                            NF4O_INVALID_ARGUMENT);
            }
        }
        return NF4O_OK;
    }
    return fail(message, "unknown NF4 scale encoding", NF4O_INVALID_ARGUMENT);
}
