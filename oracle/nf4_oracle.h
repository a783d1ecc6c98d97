/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement of the reference's packed NF4
 * linear path in plain C.  Nothing the product ships may link, load or call
 * this file: it exists to check the HIP kernels (tests/, the smoke check and
 * the CPU-baseline leg of the benchmark).
 *
 * Every function cites the reference file:line (under /root/reference) whose
 * behaviour it restates.  All arithmetic is IEEE binary32 with no FMA
 * contraction (build with -ffp-contract=off), matching a plain x86-64 build
 * of the reference.
 *
 * Parity pins (what each function is checked against, see tests/):
 *   codebook, pack/unpack, nearest code, quantize   - known-answer vectors of
 *       tests/core/test_quantization.cpp:62-152 and the compiled reference
 *   double_quantize_scales, decode_scale            - known answers of
 *       tests/core/test_quantization.cpp:155-205 and the compiled reference
 *   dequantize, forward, input_backward             - closed-form fixtures of
 *       tests/core/backend/test_quantized_linear_backend.cpp:89-169, an fp64
 *       brute force, and bit-for-bit agreement with the compiled reference
 *       (committed golden hashes/slices)
 *   validate_payload                                - the payload rules the
 *       reference's own tests exercise (tests/core/test_quantization.cpp:207-376)
 *       and outcome + message of the compiled reference on damaged payloads
 *   validate_scale_storage                          - outcome, exception type
 *       and message of the compiled reference's dispatcher on forty sound and
 *       damaged scale storages (committed as golden verdicts)
 *   matmul, matmul_nt, add_bias, lora_linear_forward - bit-for-bit agreement
 *       with the compiled reference's tensor operations
 *   lora_linear_backward                            - bit-for-bit agreement
 *       with the gradients the compiled reference's autograd leaves on x and
 *       on the adapter's parameters of a real Linear (packed weight, adapter
 *       attached), committed as golden vectors
 * No function here is "parity unpinned".
 */
#ifndef NF4_ORACLE_H
#define NF4_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* src/core/backend/nn/quantized_linear/storage.hpp:13-16 */
enum {
    NF4O_SCALE_FLOAT32 = 0,
    NF4O_SCALE_DOUBLE_QUANTIZED_UINT8 = 1,
};

/* Status codes of the validators (which exception the reference throws). */
enum {
    NF4O_OK = 0,
    NF4O_INVALID_ARGUMENT = 1, /* std::invalid_argument */
    NF4O_LOGIC_ERROR = 2,      /* std::logic_error      */
    NF4O_OVERFLOW = 3,         /* std::overflow_error   */
};

/* Non-owning view, the C mirror of Nf4ScaleStorageView
 * (src/core/backend/nn/quantized_linear/storage.hpp:31-45). */
typedef struct nf4o_scales {
    int32_t encoding;
    const float* fp32_scales;        /* Float32: one per block           */
    size_t fp32_count;
    const uint8_t* quantized_scales; /* DQ: one centred code per block   */
    size_t quantized_count;
    const float* second_level;       /* DQ: one per second_level_block   */
    size_t second_level_count;
    size_t second_level_block;
    float offset;
} nf4o_scales;

/* Nf4ScaleStorageView::scale_count, storage.hpp:39-44 */
size_t nf4o_scale_count(const nf4o_scales* scales);

/* src/core/quantization/nf4.cpp:14-35 */
const float* nf4o_codebook(void);

/* src/core/quantization/nf4.cpp:39-53 */
int nf4o_block_size_supported(size_t block_size);

/* src/core/quantization/quantized_weight.cpp:37-46 */
size_t nf4o_block_count(size_t element_count, size_t block_size);
size_t nf4o_packed_byte_count(size_t element_count);

/* src/core/quantization/nf4.cpp:55-68 (strict '<': ties pick the lower code) */
uint8_t nf4o_nearest_code(float normalized_value);

/* src/core/quantization/nf4.cpp:70-88 */
uint8_t nf4o_unpack_code(const uint8_t* packed, size_t flat_index);
void nf4o_pack_code(uint8_t* packed, size_t flat_index, uint8_t code);

/* pack_nf4, src/core/quantization/quantized_weight.cpp:176-206.
 * codes must hold nf4o_packed_byte_count(n) bytes, scales nf4o_block_count().
 * Returns NF4O_INVALID_ARGUMENT on a non-finite source value. */
int nf4o_quantize(const float* values, size_t n, size_t block_size,
                  uint8_t* codes, float* scales);

/* double_quantize_scales, src/core/quantization/quantized_weight.cpp:208-254.
 * scale_codes: block_count bytes; second_level: ceil(block_count/C) floats.
 * Returns NF4O_OVERFLOW when the mean is not finite. */
int nf4o_double_quantize_scales(const float* block_scales, size_t block_count,
                                size_t scale_block_size, uint8_t* scale_codes,
                                float* second_level, float* offset);

/* decode_nf4_block_scale, src/core/backend/nn/quantized_linear/storage.hpp:46-65
 * (same arithmetic: src/core/quantization/quantized_weight.cpp:82-100). */
float nf4o_decode_scale(const nf4o_scales* scales, size_t scale_index);

/* QuantizedWeight::dequantize, src/core/quantization/quantized_weight.cpp:453-467:
 * out[j] = scale(j / B) * codebook[code(j)], one rounded multiply. */
void nf4o_dequantize(const uint8_t* codes, const nf4o_scales* scales,
                     size_t element_count, size_t block_size, float* out);

/* reference_quantized_linear_forward,
 * src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81.
 * y[r,o] = sum_i x[r,i] * deq(W[o*I+i]); fp32 accumulator, ascending i. */
void nf4o_linear_forward(const float* x, const uint8_t* codes,
                         const nf4o_scales* scales, float* y, size_t rows,
                         size_t input_width, size_t output_width,
                         size_t block_size);

/* reference_quantized_linear_input_backward,
 * src/core/backend/nn/quantized_linear/reference/operations.cpp:83-115.
 * dx[r,i] = sum_o dy[r,o] * deq(W[o*I+i]); fp32 accumulator, ascending o. */
void nf4o_linear_input_backward(const float* dy, const uint8_t* codes,
                                const nf4o_scales* scales, float* dx,
                                size_t rows, size_t input_width,
                                size_t output_width, size_t block_size);

/* Bit-identical to the two functions above (same rounded products, same
 * order per output) with each weight row decoded once; for parity checks that
 * need more rows than the faithful loops finish in seconds. */
void nf4o_linear_forward_rowcached(const float* x, const uint8_t* codes,
                                   const nf4o_scales* scales, float* y,
                                   size_t rows, size_t input_width,
                                   size_t output_width, size_t block_size);
void nf4o_linear_input_backward_rowcached(const float* dy,
                                          const uint8_t* codes,
                                          const nf4o_scales* scales, float* dx,
                                          size_t rows, size_t input_width,
                                          size_t output_width,
                                          size_t block_size);

/* Bias as the reference applies it: a separate broadcast add after the
 * packed product, src/nn/linear.cpp:165-168. */
void nf4o_add_bias(float* y, const float* bias, size_t rows,
                   size_t output_width);

/* CpuBackendAdapter::matmul, src/core/backend/adapters/cpu/adapter.cpp:158-203,
 * one batch: out[r,c] = sum_k left[r,k] * right[k,c]; fp32 accumulator,
 * ascending k; left is [rows, shared], right [shared, columns], row-major. */
void nf4o_matmul(const float* left, const float* right, float* out,
                 size_t rows, size_t shared, size_t columns);

/* The same sums with the right operand given transposed ([columns, shared]
 * row-major): out[r,c] = sum_k left[r,k] * right_t[c,k].  This is what
 * matmul(x, transpose_2d(W)) computes once the transpose is materialised
 * (src/nn/linear.cpp:158-163, src/nn/low_rank_adapter.cpp:140-147). */
void nf4o_matmul_nt(const float* left, const float* right_t, float* out,
                    size_t rows, size_t shared, size_t columns);

/* Linear::forward with a packed weight, optional bias and an attached
 * low-rank adapter, src/nn/linear.cpp:147-172 and
 * src/nn/low_rank_adapter.cpp:126-151:
 *   base = x.deq(W)^T (+ bias, a separate broadcast add)
 *   reduced  = matmul(x, transpose(A))        A: [rank, input_width]
 *   expanded = matmul(reduced, transpose(B))  B: [output_width, rank]
 *   y = base + expanded * lora_scale
 * every step rounded to fp32 on its own.  bias may be NULL. */
void nf4o_lora_linear_forward(const float* x, const uint8_t* codes,
                              const nf4o_scales* scales, const float* bias,
                              const float* lora_a, const float* lora_b,
                              size_t rank, float lora_scale, float* y,
                              size_t rows, size_t input_width,
                              size_t output_width, size_t block_size);

/* The backward pass the reference's autograd runs through that Linear when
 * the base weight is packed (frozen) and the adapter trains: the closures of
 * src/core/autograd/operations.cpp recorded by LowRankAdapter::forward
 * (src/nn/low_rank_adapter.cpp:126-151) and quantized_linear
 * (src/nn/quantized_linear.cpp:60-80), met by Variable::accumulate_gradient
 * (src/core/autograd/graph.cpp:218-242):
 *   scaled    = dy * lora_scale                     operator* (:176-194)
 *   d_reduced = matmul(scaled, B)                   matmul    (:252-277)
 *   dB        = transpose(matmul(reduced^T, scaled))  with reduced = x.A^T
 *   dA        = transpose(matmul(x^T, d_reduced))   transpose_2d (:480-492)
 *   dx        = dy.deq(W) + matmul(d_reduced, A)
 * every product summed in ascending order of the contracted index in fp32,
 * every step rounded on its own.  x and dy are the values of one call
 * (gradients start from zero, as after zero_gradient). */
void nf4o_lora_linear_backward(const float* dy, const float* x,
                               const uint8_t* codes, const nf4o_scales* scales,
                               const float* lora_a, const float* lora_b,
                               size_t rank, float lora_scale, float* dx,
                               float* d_lora_a, float* d_lora_b, size_t rows,
                               size_t input_width, size_t output_width,
                               size_t block_size);

/* require_canonical_payload, src/core/quantization/quantized_weight.cpp:102-174.
 * Returns NF4O_OK or the status of the exception the reference throws;
 * *message (may be NULL) receives a static description. */
int nf4o_validate_payload(size_t element_count, size_t block_size,
                          const uint8_t* codes, size_t code_bytes,
                          const nf4o_scales* scales, const char** message);

/* require_scale_storage, src/core/backend/nn/quantized_linear/dispatch.cpp:108-154. */
int nf4o_validate_scale_storage(const nf4o_scales* scales,
                                size_t expected_scale_count,
                                const char** message);

/* nf4_scale_payload_bytes, src/core/backend/nn/quantized_linear/storage.hpp:67-75. */
size_t nf4o_scale_payload_bytes(const nf4o_scales* scales);

#ifdef __cplusplus
}
#endif

#endif /* NF4_ORACLE_H */
