/*
 * rthip.h -- kernel-level C ABI of the MI355X (gfx950) backend for the packed
 * NF4 QLoRA linear path of riftco-transformer.
 *
 * This is the whole boundary between host code and the GPU: plain pointers and
 * sizes, int status codes, no C++ types, no exceptions, no framework types.
 * The C++ `hip` backend adapter (the counterpart of the reference's CPU, Metal,
 * CUDA and TPU adapters) is the intended caller; Python reaches the same
 * symbols through ctypes for tests and measurement.
 *
 * Conventions
 *   - Every function returns an rthip_status; on failure a thread-local,
 *     NUL-terminated message is available from rthip_last_error().
 *   - All tensor pointers are DEVICE pointers unless named host_*.
 *   - Tensors are contiguous row-major fp32; packed codes are bytes with the
 *     even flat index in the low nibble (src/core/quantization/nf4.cpp:70-75).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *     Compute entry points only enqueue work; the caller synchronises.  The
 *     reference contract "an adapter finishes writing its output before
 *     returning" (docs/BACKENDS_AND_PYTHON.md:168) is met by the adapter, which
 *     calls rthip_stream_synchronize() after each launch.
 *   - A packed weight is described by the same six values the reference's CUDA
 *     launch passes to its kernels
 *     (src/core/backend/nn/quantized_linear/cuda/operations.cu:76-81,196-211):
 *       codes              uint8  [ceil(O*I/2)]
 *       primary_scales     float  [blocks]   when encoding == RTHIP_NF4_SCALE_FLOAT32
 *                          uint8  [blocks]   when encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8
 *       secondary_scales   float  [ceil(blocks / second_level_block)] (DQ only, else NULL)
 *       encoding, second_level_block, offset
 *     with blocks = ceil(O*I / block_size) counted over the FLATTENED weight
 *     (src/core/backend/nn/quantized_linear/reference/operations.cpp:44).
 */
#ifndef RTHIP_H
#define RTHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RTHIP_ABI_VERSION_MAJOR 1u
#define RTHIP_ABI_VERSION_MINOR 10u

typedef int32_t rthip_status;

enum {
    RTHIP_OK = 0,
    /* bad pointer/size/enum: the adapter maps it to std::invalid_argument */
    RTHIP_INVALID_ARGUMENT = 1,
    /* no usable gfx950 device: maps to "hip execution backend is unavailable" */
    RTHIP_UNAVAILABLE = 2,
    /* device allocation failed: maps to std::bad_alloc, as
     * src/core/backend/adapters/cuda/adapter.cu:25-32 does for CUDA */
    RTHIP_OUT_OF_MEMORY = 3,
    /* any other HIP runtime failure: maps to std::runtime_error */
    RTHIP_RUNTIME_ERROR = 4,
    /* a forced algorithm cannot handle the given shape */
    RTHIP_UNSUPPORTED = 5,
    /* a value left the fp32 range: maps to std::overflow_error */
    RTHIP_OVERFLOW = 6
};

/* Nf4ScaleEncoding, src/core/backend/nn/quantized_linear/storage.hpp:13-16 */
enum {
    RTHIP_NF4_SCALE_FLOAT32 = 0,
    RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8 = 1
};

/* Kernel families.  AUTO picks by shape; the others exist so that tests can
 * pin one family and compare it with another on the same inputs. */
enum {
    RTHIP_NF4_ALGORITHM_AUTO = 0,
    /* one thread per output, per-element decode, any shape or block size */
    RTHIP_NF4_ALGORITHM_GENERIC = 1,
    /* streaming kernels for decode-sized row counts (up to 4; HBM-bound):
     * forward, a wavefront-reduced GEMV; input backward, the packed weight
     * walked row by row as it lies in memory, a lane owning sixteen of its
     * columns, products on the 4x4x1 matrix instruction */
    RTHIP_NF4_ALGORITHM_GEMV = 2,
    /* LDS-tiled fp32 MFMA GEMM with dequantisation fused into the tile load */
    RTHIP_NF4_ALGORITHM_MFMA = 3,
    /* small batches (up to 64 rows): weights decoded straight into MFMA
     * operands, no LDS tile.  Forward: a slab kernel over the contraction;
     * input backward: the packed weight is walked row by row as it lies in
     * memory, a lane owning eight of its columns */
    RTHIP_NF4_ALGORITHM_SKINNY = 4,
    /* up to 128 rows (forward) with a row width of 1024..4096: like SKINNY,
     * but x stays in registers, 16 rows per workgroup, and the wavefronts
     * split the contraction axis */
    RTHIP_NF4_ALGORITHM_RESIDENT = 5
};

/* ---- library / device ------------------------------------------------- */

/* (major << 16) | minor of this ABI. */
uint32_t rthip_abi_version(void);

/* Thread-local message of the last failing call on this thread ("" if none). */
const char* rthip_last_error(void);

/* Number of usable gfx950 devices.  Returns RTHIP_UNAVAILABLE (and *count = 0)
 * when there is no driver or no device -- the adapter's is_available().
 * Replaces the role of cudaGetDeviceCount in
 * src/core/backend/adapters/cuda/adapter.cu:40-51. */
rthip_status rthip_device_count(int32_t* count);

/* Human-readable device description, e.g. "AMD Instinct MI355X (gfx950), 256 CUs". */
rthip_status rthip_device_description(char* buffer, size_t capacity);

/* *visible = 1 when pointers returned by rthip_malloc can be dereferenced by
 * the host (the whole HBM is mapped through a large PCIe BAR, the normal
 * configuration of MI300/MI350-class servers), 0 otherwise.  The adapter uses
 * it to decide whether packed-weight storage can serve the host-readable spans
 * of QuantizedWeightStorage
 * (src/core/backend/nn/quantized_linear/storage.hpp:85-88) straight from HBM,
 * with no mirror -- what the CUDA backend obtains from managed memory
 * (src/core/backend/nn/quantized_linear/cuda/storage.cu:22-43). */
rthip_status rthip_device_memory_host_visible(int32_t* visible);

/* ---- memory ----------------------------------------------------------- */

/* Device (HBM) allocation; *pointer is 256-byte aligned.  bytes == 0 yields
 * NULL.  Counterpart of the allocations in
 * src/core/backend/nn/quantized_linear/cuda/storage.cu:26-43. */
rthip_status rthip_malloc(void** pointer, size_t bytes);
rthip_status rthip_free(void* pointer);

/* Synchronous copies between host and device memory. */
rthip_status rthip_copy_to_device(void* device, const void* host, size_t bytes);
rthip_status rthip_copy_to_host(void* host, const void* device, size_t bytes);

/* Fills count floats (make_storage(element_count, fill_value),
 * src/core/backend/adapter.hpp:37-40).  Enqueued on `stream`. */
rthip_status rthip_fill_f32(float* device, float value, uint64_t count,
                            void* stream);

rthip_status rthip_stream_synchronize(void* stream);

/* ---- the hot path ----------------------------------------------------- */

/*
 * y[r,o] = sum_i x[r,i] * deq(W)[o,i]  (+ bias[o] when bias_or_null != NULL)
 *
 * Replaces BackendAdapter::quantized_linear_forward
 * (src/core/backend/nn/quantized_linear/capability.hpp:36-42), whose CPU form
 * is reference_quantized_linear_forward
 * (src/core/backend/nn/quantized_linear/reference/operations.cpp:49-81).
 * x is [rows, input_width], y is [rows, output_width] and is overwritten.
 * The optional bias fuses the broadcast add the reference performs afterwards
 * (src/nn/linear.cpp:165-168).  x/y must not overlap each other or the weight.
 */
rthip_status rthip_nf4_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    float* y, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream);

/*
 * dx[r,i] = sum_o dy[r,o] * deq(W)[o,i]
 *
 * Replaces BackendAdapter::quantized_linear_input_backward
 * (src/core/backend/nn/quantized_linear/capability.hpp:44-50; CPU form
 * src/core/backend/nn/quantized_linear/reference/operations.cpp:83-115).
 * dy is [rows, output_width], dx is [rows, input_width] and is overwritten.
 */
rthip_status rthip_nf4_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream);

/*
 * y_m = x.deq(W_m)^T (+ bias_m) for m < member_count: several packed weights
 * applied to the SAME x, as the query, key and value projections of an
 * attention block are (src/model/decoder_only_transformer.cpp:406-419 calls
 * query_, key_ and value_.forward on one normalised input; a gated feed-forward
 * does the same with its gate and up projections).  The result is, bit for
 * bit, that of member_count calls of rthip_nf4_linear_forward; the point is
 * the launch count: for rows <= 4 up to four members run as ONE streaming
 * launch, which removes the fixed cost between decode-sized kernels, and for
 * rows <= 128 with a row width of 1024, 2048, 3072 or 4096 up to four members
 * run as ONE launch of the kernel that keeps x in registers, which loads x
 * once for all of them.  Other shapes are launched one by one.  The members
 * share input_width, block_size, encoding and
 * second_level_block; each has its own output_width, offset, bias and y.
 * `members` is a HOST array, read before the call returns.
 */
typedef struct rthip_nf4_member {
    const uint8_t* codes;
    const void* primary_scales;
    const float* secondary_scales; /* NULL for fp32 scales */
    float offset;
    const float* bias_or_null;
    float* y;                      /* [rows, output_width] */
    uint64_t output_width;
} rthip_nf4_member;

rthip_status rthip_nf4_linear_forward_group(
    const float* x, const rthip_nf4_member* members, uint64_t member_count,
    int32_t encoding, uint64_t second_level_block, uint64_t rows,
    uint64_t input_width, uint64_t block_size, void* stream);

/*
 * The same grouped forward for layers that carry low-rank adapters: member m
 * gets y_m = x.deq(W_m)^T + bias_m + lora_scale_m * (reduced_m . B_m^T), as
 * rthip_nf4_lora_linear_forward below computes it.  With lora_a given,
 * `reduced` [rows, lora_rank] receives x.A_m^T first (the products of up to
 * four members in one launch while they are small); with lora_a NULL it already
 * holds it (one rthip_lora_reduce over the stacked A matrices of the members
 * serves them all when rows is 1).  A member whose lora_b and reduced are both
 * NULL has no adapter.  The reference reaches this
 * through Linear::forward (src/nn/linear.cpp:147-172) once per projection;
 * q, k and v of a layer with adapters on q and v are one launch here.
 * Every member's output equals its own rthip_nf4_lora_linear_forward (or
 * rthip_nf4_linear_forward) bit for bit.  One launch for up to four rows of x
 * (members the decode kernel takes) and for 5...128 rows of a row width of
 * 1024...4096; other members are launched one by one.
 */
typedef struct rthip_nf4_lora_member {
    rthip_nf4_member base;
    const float* lora_a;   /* [lora_rank, input_width]; NULL: `reduced` is given */
    const float* lora_b;   /* [output_width, lora_rank] */
    float* reduced;        /* [rows, lora_rank]; NULL (with lora_b): no adapter */
    uint64_t lora_rank;
    float lora_scale;
} rthip_nf4_lora_member;

rthip_status rthip_nf4_lora_linear_forward_group(
    const float* x, const rthip_nf4_lora_member* members,
    uint64_t member_count, int32_t encoding, uint64_t second_level_block,
    uint64_t rows, uint64_t input_width, uint64_t block_size, void* stream);

/*
 * y = x.deq(W)^T + bias + lora_scale * ((x.A^T).B^T)
 *
 * Linear::forward of a layer that holds a packed weight, an optional bias and
 * an attached low-rank adapter (src/nn/linear.cpp:147-172 with
 * LowRankAdapter::forward, src/nn/low_rank_adapter.cpp:126-151), which the
 * reference evaluates as six separate operations (packed product, broadcast,
 * add, two dense matmuls over materialised transposes, scale, add).  Here it
 * is two launches: reduced = x.A^T, then the packed product with bias and the
 * rank-sized sum in its epilogue.
 *   lora_a   [lora_rank, input_width]    (LowRankAdapter::a, "lora_a.weight")
 *   lora_b   [output_width, lora_rank]   (LowRankAdapter::b, "lora_b.weight")
 *   lora_scale = alpha / rank            (LowRankAdapter::scale)
 *   reduced  [rows, lora_rank]  caller-provided device buffer that receives
 *            x.A^T (the saved activation the adapter's backward needs)
 * lora_a may be NULL: `reduced` then already holds x.A^T (from
 * rthip_lora_reduce, for example one launch over the stacked A matrices of
 * several projections that share x) and only the second launch is made.
 * Rounding follows the reference: the rank sum in fp32 in ascending order,
 * times lora_scale, added to (product + bias).
 */
rthip_status rthip_nf4_lora_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    const float* lora_a, const float* lora_b, uint64_t lora_rank,
    float lora_scale, float* reduced, float* y, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream);

/*
 * out[b][r,c] = sum_k left[b][r,k] * right[b][k,c]
 *
 * Replaces BackendAdapter::matmul (src/core/backend/adapter.hpp:46-52; CPU form
 * src/core/backend/adapters/cpu/adapter.cpp:158-203) with MatmulDimensions
 * {batch_count, rows, shared, columns}: contiguous row-major operands, no
 * batch broadcasting, output overwritten.
 */
rthip_status rthip_matmul(const float* left, const float* right, float* out,
                          uint64_t batch_count, uint64_t rows,
                          uint64_t shared, uint64_t columns, void* stream);

/*
 * reduced[r,j] = sum_k x[r,k] * A[j,k]: matmul(x, transpose(A)), the first
 * product of LowRankAdapter::forward (src/nn/low_rank_adapter.cpp:140-143).
 * x is [rows, input_width], lora_a [lora_rank, input_width], reduced
 * [rows, lora_rank].
 */
rthip_status rthip_lora_reduce(const float* x, const float* lora_a,
                               float* reduced, uint64_t rows,
                               uint64_t input_width, uint64_t lora_rank,
                               void* stream);

/*
 * The adapter's gradients for one upstream gradient dy [rows, output_width]:
 *
 *   d_reduced = (dy * lora_scale) . B                 [rows, lora_rank]
 *   d_lora_b  = (dy * lora_scale)^T . reduced         [output_width, lora_rank]
 *   d_lora_a  = d_reduced^T . x                       [lora_rank, input_width]
 *
 * What the reference's autograd computes for LowRankAdapter::forward
 * (src/nn/low_rank_adapter.cpp:126-151) through the closures of operator*,
 * matmul and transpose_2d (src/core/autograd/operations.cpp:176-194,252-277,
 * 480-492): five dense matmuls over materialised transposes plus an
 * elementwise multiply there, three launches here (d_reduced, then the two
 * outer products; dy and x are each read once per product, dy * lora_scale is
 * rounded per element and never stored).  `reduced` is x.A^T as the forward
 * left it in its caller-provided buffer.  The gradients are written, not
 * added to what the buffers hold (the reference starts every backward pass
 * from zeroed gradients, src/core/autograd/graph.cpp:218-242).  d_lora_a
 * and/or d_lora_b may be NULL: that product is skipped (x and reduced may
 * then be NULL as well).  d_reduced is always written; the fused input
 * backward below consumes it.
 */
rthip_status rthip_lora_backward(
    const float* dy, const float* x, const float* reduced,
    const float* lora_b, uint64_t lora_rank, float lora_scale,
    float* d_reduced, float* d_lora_a, float* d_lora_b, uint64_t rows,
    uint64_t input_width, uint64_t output_width, void* stream);

/*
 * dx = dy.deq(W) + d_reduced.A
 *
 * The gradient that reaches the input of a Linear with a packed weight and an
 * adapter: quantized_linear's closure (src/nn/quantized_linear.cpp:60-80)
 * and the left-operand closure of the adapter's first matmul
 * (src/core/autograd/operations.cpp:252-277), which the reference adds with
 * one rounded addition per element where both arrive at x
 * (Variable::accumulate_gradient, src/core/autograd/graph.cpp:218-242).
 * Here the rank-sized sum is the epilogue of the packed-weight input
 * backward: one pass over dx instead of a dense matmul, a temporary and an
 * add.  lora_a is [lora_rank, input_width], d_reduced [rows, lora_rank] from
 * rthip_lora_backward on the same stream.
 */
rthip_status rthip_nf4_lora_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* lora_a,
    const float* d_reduced, uint64_t lora_rank, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream);

/* The same two operations with the kernel family pinned (tests, measurement).
 * RTHIP_UNSUPPORTED when `algorithm` cannot handle the shape. */
rthip_status rthip_nf4_linear_forward_with(
    int32_t algorithm, const float* x, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* bias_or_null, float* y, uint64_t rows, uint64_t input_width,
    uint64_t output_width, uint64_t block_size, void* stream);

rthip_status rthip_nf4_lora_linear_forward_with(
    int32_t algorithm, const float* x, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* bias_or_null, const float* lora_a, const float* lora_b,
    uint64_t lora_rank, float lora_scale, float* reduced, float* y,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream);
rthip_status rthip_nf4_linear_input_backward_with(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset, float* dx,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream);

rthip_status rthip_nf4_lora_linear_input_backward_with(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* lora_a, const float* d_reduced, uint64_t lora_rank,
    float* dx, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream);

/* Which family AUTO selects for a shape: direction 0 = forward, 1 = input
 * backward.  Pure host computation; needs no device.  Row counts just above
 * the small-batch families' 64 run as two launches of those families, the
 * first 64 rows and the rest (forward: up to 112 rows; backward: up to 96,
 * and up to 192 in three parts where output_width >= 2 * input_width).
 * Where the register-resident kernel takes the rows, 81...128 are one launch
 * of it and 129...224 two, 128 rows and the rest.  Larger row counts that end
 * 1...64 rows past a multiple of 128 run as a tiled launch for the whole
 * 128-row tiles and a small-batch launch for the rest, in both directions.
 * The family of the first part is reported. */
rthip_status rthip_nf4_select_algorithm(
    int32_t direction, uint64_t rows, uint64_t input_width,
    uint64_t output_width, uint64_t block_size, int32_t* algorithm);

/* The kernel instance that rthip_nf4_linear_forward (member_count == 1) or
 * rthip_nf4_linear_forward_group launches for weights of these output widths
 * when the one-row decode kernel serves the call, as a profiler prints it
 * without its namespace ("gemv1_forward_kernel<1, 8, 2, 4, false, false,
 * 4>"); an empty string where another family serves it.  For tools that have
 * to tell whether a stored profile still describes the kernels a build
 * launches.  Pure host computation; needs no device.  No counterpart in the
 * reference. */
rthip_status rthip_nf4_forward_kernel_name(
    uint64_t rows, uint64_t input_width, const uint64_t* output_widths,
    uint64_t member_count, uint64_t block_size, int32_t encoding,
    uint64_t second_level_block, char* name, uint64_t capacity);

/*
 * out[j] = scale(j / block_size) * codebook[code(j)] for j < element_count.
 *
 * Device form of QuantizedWeight::dequantize
 * (src/core/quantization/quantized_weight.cpp:453-467).  The linear kernels
 * never call it (they never materialise an fp32 weight); it exists so that the
 * bit-exactness of nibble unpack, codebook lookup and scale decode on the GPU
 * can be checked directly, and for the explicit dequantize() API.
 */
rthip_status rthip_nf4_dequantize(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* out,
    uint64_t element_count, uint64_t block_size, void* stream);

/*
 * The NF4 quantizer on the device: QuantizedWeight::quantize_nf4 /
 * quantize_nf4_double_quantized, i.e. pack_nf4 and double_quantize_scales
 * (src/core/quantization/quantized_weight.cpp:176-206, 208-254), bit for bit.
 *   values              fp32 [element_count], the weight flattened row-major
 *   codes               uint8 [ceil(element_count / 2)], overwritten
 * encoding == RTHIP_NF4_SCALE_FLOAT32:
 *   primary_scales      float [blocks], overwritten; the other outputs unused
 * encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8:
 *   primary_scales      uint8 [blocks] scale codes
 *   secondary_scales    float [ceil(blocks / second_level_block)]
 *   fp32_scale_scratch  float [blocks]: receives the plain block scales
 *   host_offset         HOST pointer that receives the offset
 * Unlike the compute entry points this one returns after the work is done
 * (it waits for `stream`, so it cannot be recorded into a graph):
 * a non-finite source value is reported as RTHIP_INVALID_ARGUMENT ("NF4 source
 * values must be finite") and a non-finite scale mean as RTHIP_OVERFLOW, the
 * two exceptions the reference throws (:189-191, :224-227).
 */
rthip_status rthip_nf4_quantize(
    const float* values, uint64_t element_count, uint64_t block_size,
    int32_t encoding, uint64_t second_level_block, uint8_t* codes,
    void* primary_scales, float* secondary_scales, float* fp32_scale_scratch,
    float* host_offset, void* stream);

/*
 * The content rules of QuantizedWeight::from_packed_nf4's
 * require_canonical_payload (src/core/quantization/quantized_weight.cpp:
 * 102-174) applied to a payload that is already in device memory -- what a
 * loader runs after copying a checkpoint's packed state
 * (src/c_api/model_state.cpp:166-300) straight into HBM, instead of a pass
 * over host vectors before the upload.  The array lengths are the caller's to
 * check; this call reads
 *   codes [ceil(element_count / 2)], primary_scales [blocks] (float or uint8),
 *   secondary_scales [ceil(blocks / second_level_block)] (nested only)
 * and returns, after the work is done (it waits for `stream`, so it cannot
 * be recorded into a graph), RTHIP_OK or RTHIP_INVALID_ARGUMENT
 * with the message of the exception the reference would throw first:
 * a non-zero unused high nibble, a negative or non-finite offset,
 * second-level scale or decoded block scale, or a block with an fp32 scale of
 * zero that holds a code other than 7.
 */
rthip_status rthip_nf4_check_payload(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, uint64_t element_count,
    uint64_t block_size, void* stream);

/*
 * Frees the scratch buffers the library keeps per (device, stream) for
 * kernels that pass partial results between workgroups (64 MiB each,
 * allocated by the first call on a stream that needs one): the buffer of
 * `stream` on the current device, or of every stream when every_stream != 0.
 * Waits for the device to finish with them; a later call allocates afresh.
 * A graph that was captured on such a stream keeps the address of the buffer
 * it was recorded with: do not release while such a graph may still be
 * replayed.  With every_stream != 0 the call also unbinds the static array of
 * rthip_nf4_linear_input_backward_no_alloc from its stream (after that stream
 * has finished).  No counterpart in the reference (its backends allocate per
 * call).
 */
rthip_status rthip_release_workspaces(void* stream, int32_t every_stream);

/*
 * rthip_nf4_linear_input_backward for callers that cannot allocate: code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  Same arguments and
 * the same result, bit for bit, but it covers the small-batch family only
 * (rows <= 64, input_width % 8 == 0, output_width % 4 == 0, aligned
 * pointers; RTHIP_UNSUPPORTED otherwise) and keeps the partial sums of the
 * weight-row chunks in a device array that is part of the library image
 * (RTHIP_NO_ALLOC_SCRATCH_BYTES on every GPU the library runs on, held until
 * the process ends) instead of the per-stream workspace.  A problem whose
 * partial sums -- chunks x rows x input_width x 4 bytes, chunks <= 16 --
 * exceed that size is refused with RTHIP_UNSUPPORTED and a message that
 * names both sizes.  It calls no hipMalloc, hipFree or allocating library
 * routine.  Every call on a GPU shares that GPU's array, and calls that
 * overlap on the GPU would race on it, so the array is bound to the stream of
 * the first call on that GPU: calls on that stream, from any number of host
 * threads, are ordered and safe (a thread holds the array until both of its
 * launches are enqueued); a call on ANOTHER stream is refused with
 * RTHIP_UNSUPPORTED until rthip_release_workspaces(stream, 1) has unbound the
 * array.  What the library cannot see stays the caller's to avoid: two graphs
 * that were captured on the bound stream and are replayed at the same time on
 * different streams.
 */
#define RTHIP_NO_ALLOC_SCRATCH_BYTES (24u << 20)
rthip_status rthip_nf4_linear_input_backward_no_alloc(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream);

#ifdef __cplusplus
}
#endif

#endif /* RTHIP_H */
