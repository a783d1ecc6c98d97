// The C ABI of include/rthip.h: argument validation, kernel-family selection
// and launch.  No C++ type crosses this boundary and no exception leaves it.

#include "../../include/rthip.h"

#include "kernels.hpp"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <limits>
#include <mutex>

namespace {

thread_local char g_last_error[512] = "";

rthip_status fail(rthip_status status, const char* format, ...) {
    va_list arguments;
    va_start(arguments, format);
    std::vsnprintf(g_last_error, sizeof(g_last_error), format, arguments);
    va_end(arguments);
    return status;
}

rthip_status ok() {
    g_last_error[0] = '\0';
    return RTHIP_OK;
}

rthip_status from_hip(hipError_t error, const char* what) {
    if (error == hipSuccess) {
        return ok();
    }
    const rthip_status status = error == hipErrorOutOfMemory
        ? RTHIP_OUT_OF_MEMORY
        : RTHIP_RUNTIME_ERROR;
    return fail(status, "%s: %s", what, hipGetErrorString(error));
}

// Device discovery runs once per process; the result (including the reason
// for unavailability) is immutable afterwards.
struct DeviceState {
    rthip_status status = RTHIP_UNAVAILABLE;
    int count = 0;
    bool large_bar = false;
    char description[256] = "";
    char reason[256] = "";
};

const DeviceState& device_state() {
    static DeviceState state;
    static std::once_flag once;
    std::call_once(once, [] {
        int count = 0;
        const hipError_t error = hipGetDeviceCount(&count);
        if (error != hipSuccess || count <= 0) {
            // Clear the sticky error so later calls report their own.
            static_cast<void>(hipGetLastError());
            std::snprintf(state.reason, sizeof(state.reason),
                          "no HIP device is visible (%s)",
                          error == hipSuccess ? "device count is zero"
                                              : hipGetErrorString(error));
            return;
        }
        hipDeviceProp_t properties;
        if (hipGetDeviceProperties(&properties, 0) != hipSuccess) {
            static_cast<void>(hipGetLastError());
            std::snprintf(state.reason, sizeof(state.reason),
                          "device 0 properties are unreadable");
            return;
        }
        if (std::strncmp(properties.gcnArchName, "gfx950", 6) != 0) {
            std::snprintf(state.reason, sizeof(state.reason),
                          "device 0 is %s; this library carries gfx950 code "
                          "only",
                          properties.gcnArchName);
            return;
        }
        state.status = RTHIP_OK;
        state.count = count;
        state.large_bar = properties.isLargeBar != 0;
        std::snprintf(state.description, sizeof(state.description),
                      "%s (%s), %d CUs, %.0f GiB", properties.name,
                      properties.gcnArchName, properties.multiProcessorCount,
                      static_cast<double>(properties.totalGlobalMem) /
                          (1024.0 * 1024.0 * 1024.0));
    });
    return state;
}

rthip_status require_device() {
    const DeviceState& state = device_state();
    if (state.status != RTHIP_OK) {
        return fail(RTHIP_UNAVAILABLE, "%s", state.reason);
    }
    return RTHIP_OK;
}

// The block sizes the format allows (src/core/quantization/nf4.cpp:39-53).
bool block_shift_for(uint64_t block_size, unsigned* shift) {
    for (unsigned candidate = 5; candidate <= 12; ++candidate) {
        if (block_size == (1ULL << candidate)) {
            *shift = candidate;
            return true;
        }
    }
    return false;
}

rthip_status make_weight_view(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, rthip::Nf4WeightView* view
) {
    if (codes == nullptr || primary_scales == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "packed codes and primary scales must not be null");
    }
    view->codes = codes;
    view->primary_scales = primary_scales;
    view->secondary_scales = nullptr;
    view->encoding = encoding;
    view->second_level_shift = 0;
    view->offset = 0.0F;
    if (encoding == RTHIP_NF4_SCALE_FLOAT32) {
        return RTHIP_OK;
    }
    if (encoding != RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8) {
        return fail(RTHIP_INVALID_ARGUMENT, "unknown NF4 scale encoding %d",
                    static_cast<int>(encoding));
    }
    unsigned shift = 0;
    if (!block_shift_for(second_level_block, &shift)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "second-level scale block %llu is not one of 32..4096",
                    static_cast<unsigned long long>(second_level_block));
    }
    if (secondary_scales == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "double-quantized scales need second-level scales");
    }
    view->secondary_scales = secondary_scales;
    view->second_level_shift = shift;
    view->offset = offset;
    return RTHIP_OK;
}

rthip_status check_dimensions(uint64_t rows, uint64_t input_width,
                              uint64_t output_width, uint64_t block_size,
                              unsigned* block_shift) {
    if (rows == 0 || input_width == 0 || output_width == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear dimensions must be positive");
    }
    if (!block_shift_for(block_size, block_shift)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 block size %llu is not one of 32..4096",
                    static_cast<unsigned long long>(block_size));
    }
    constexpr uint64_t kMax = std::numeric_limits<uint64_t>::max() / 4;
    if (input_width > kMax / output_width || rows > kMax / input_width ||
        rows > kMax / output_width) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear size exceeds addressable storage");
    }
    return RTHIP_OK;
}

rthip_status finish_launch(const char* what) {
    return from_hip(hipGetLastError(), what);
}

int32_t select_forward(const rthip::LinearProblem& problem) {
    if (problem.rows <= rthip::kGemvMaxRows &&
        rthip::gemv_forward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_GEMV;
    }
    if (problem.rows <= rthip::kResidentMaxRows &&
        rthip::resident_forward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_RESIDENT;
    }
    if (problem.rows <= rthip::kSkinnyMaxRows &&
        rthip::skinny_forward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_SKINNY;
    }
    if (rthip::mfma_forward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_MFMA;
    }
    return RTHIP_NF4_ALGORITHM_GENERIC;
}

// Row counts just above the small-batch kernels' limit run as two launches
// of those kernels (AUTO only; see linear_forward_common).
constexpr std::size_t kSplitHeadRows = 64;
constexpr std::size_t kForwardSplitMaxRows = 112;
// ... further up where the register-resident kernel takes the parts, in
// parts of its 128 rows: the tiled kernel pads 129...192 rows to two 128-row
// tiles, and a weight of few tiles is cut along the contraction there, which
// costs partial tiles.
constexpr std::size_t kResidentSplitMaxRows = 224;
// Up to here the resident kernel's parts are 64 rows and the rest: a fifth
// row group that is nearly empty costs a whole round of matrix instructions.
constexpr std::size_t kResidentSmallPartMaxRows = 80;
constexpr std::size_t kBackwardSplitMaxRows = 96;
bool split_rows(std::size_t rows, std::size_t limit) {
    return rows > kSplitHeadRows && rows <= limit;
}
bool small_batch_family(int32_t algorithm) {
    return algorithm == RTHIP_NF4_ALGORITHM_RESIDENT ||
           algorithm == RTHIP_NF4_ALGORITHM_SKINNY;
}

int32_t select_input_backward(const rthip::LinearProblem& problem) {
    // Streaming wins for one and two rows of dy, and for three and four where
    // the weight is large (measured: 4096 x 4096 at four rows 12.9 us against
    // 11.3 us through the small-batch kernel, 11008 x 4096 16.3 against 19.6):
    // every further row costs it a megabyte of partial sums.
    if (problem.rows <= rthip::kStreamBackwardMaxRows &&
        rthip::stream_input_backward_supports(problem) &&
        (problem.rows <= 2 ||
         problem.output_width * problem.input_width >= (std::size_t{1} << 25) ||
         !rthip::small_input_backward_supports(problem))) {
        return RTHIP_NF4_ALGORITHM_GEMV;
    }
    if (problem.rows <= rthip::kSmallBackwardMaxRows &&
        rthip::small_input_backward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_SKINNY;
    }
    if (rthip::mfma_input_backward_supports(problem)) {
        return RTHIP_NF4_ALGORITHM_MFMA;
    }
    return RTHIP_NF4_ALGORITHM_GENERIC;
}

// Just past the small-batch kernels' 64 rows the tiled kernel would run a
// 128-row tile that is mostly padding (65 rows of 11008 x 4096: 117 us against
// 57 us at 64 rows).  AUTO then sends the first 64 rows and the rest through
// the small-batch families, one launch after the other (65 rows: 74 us; equal
// to the tiled kernel from about 112 rows on).  Where the register-resident
// kernel takes the rows this goes on to 224: it runs 81...128 rows as ONE
// launch of up to eight row groups (65...80 as 64 and the rest), and 129...224
// as 128 and the rest.  Measured against the tiled kernel: 4096 x 4096 at 128
// rows 42 against 59 us, at 192 rows 67 against 92 us; 11008 x 4096 107
// against 115 us and 164 against 208 us; at 256 rows the tiled kernel is as
// fast or faster (88 against 89 us, 215 against 212 us; nested scales 95
// against 93 and 234 against 222).
// True if `problem` is such a case; `part` are then the problems and `family`
// their kernels.
constexpr std::size_t kMaxRowParts = 3;
struct RowSplit {
    rthip::LinearProblem part[kMaxRowParts];
    int32_t family[kMaxRowParts];
    std::size_t count;
};
static_assert(2 * rthip::kResidentMaxRows >= kResidentSplitMaxRows &&
              2 * kSplitHeadRows >= kForwardSplitMaxRows);
// Rows [first, first + rows) of `problem` as a problem of their own.
rthip::LinearProblem row_part(const rthip::LinearProblem& problem,
                              std::size_t first, std::size_t rows,
                              bool forward) {
    rthip::LinearProblem part = problem;
    part.rows = rows;
    if (problem.activations != nullptr) {  // null: a shape query
        part.activations +=
            first * (forward ? problem.input_width : problem.output_width);
        part.result +=
            first * (forward ? problem.output_width : problem.input_width);
    }
    if (part.lora.reduced != nullptr) {
        part.lora.reduced += first * problem.lora.rank;
    }
    return part;
}
bool forward_small_split(const rthip::LinearProblem& problem,
                         RowSplit* split) {
    if (problem.rows <= kSplitHeadRows) {
        return false;
    }
    rthip::LinearProblem head = problem;
    head.rows = kSplitHeadRows;
    const bool resident =
        select_forward(head) == RTHIP_NF4_ALGORITHM_RESIDENT;
    std::size_t part_rows = kSplitHeadRows;
    if (resident) {
        if (problem.rows > kResidentSplitMaxRows ||
            (problem.rows > kResidentSmallPartMaxRows &&
             problem.rows <= rthip::kResidentMaxRows)) {
            return false;  // (the second: one launch takes them all)
        }
        if (problem.rows > rthip::kResidentMaxRows) {
            part_rows = rthip::kResidentMaxRows;
        }
    } else if (problem.rows > kForwardSplitMaxRows) {
        return false;
    }
    split->count = (problem.rows + part_rows - 1) / part_rows;
    for (std::size_t index = 0; index < split->count; ++index) {
        const std::size_t first = index * part_rows;
        split->part[index] =
            row_part(problem, first,
                     std::min(part_rows, problem.rows - first), true);
        split->family[index] = select_forward(split->part[index]);
        // (a last part of up to four rows goes to the GEMV)
        if (!small_batch_family(split->family[index]) &&
            !(index > 0 &&
              split->family[index] == RTHIP_NF4_ALGORITHM_GEMV)) {
            return false;
        }
    }
    return true;
}
// The input backward likewise up to 96 rows (11008 x 4096: 117 -> 86...100
// us), unless dx is much wider than dy, where the tiled kernel is as fast
// (4096 x 11008: 117 against 113...132 us).  Where dy is at least twice as
// wide as dx (11008 x 4096) parts of 64 rows win up to 192 rows: the tiled
// kernel pads 129...192 rows to two row tiles of a long contraction (97 rows
// 110 -> 98 us, 192 rows 202 -> 168 us; a tie at 128; 4096 x 4096 gains
// nothing there).
constexpr std::size_t kLongBackwardSplitMaxRows = 192;
static_assert(kMaxRowParts * kSplitHeadRows >= kLongBackwardSplitMaxRows);
bool backward_small_split(const rthip::LinearProblem& problem,
                          RowSplit* split) {
    // (dx much wider than dy: only while the rows past 64 fit the streaming
    // kernel -- 4096 x 11008 at 65 rows 114 -> 97 us, at 72 rows a tie)
    const std::size_t limit =
        problem.output_width >= 2 * problem.input_width
            ? kLongBackwardSplitMaxRows
            : (problem.input_width > 2 * problem.output_width
                   ? kSplitHeadRows + rthip::kStreamBackwardMaxRows
                   : kBackwardSplitMaxRows);
    if (!split_rows(problem.rows, limit)) {
        return false;
    }
    split->count = (problem.rows + kSplitHeadRows - 1) / kSplitHeadRows;
    for (std::size_t index = 0; index < split->count; ++index) {
        const std::size_t first = index * kSplitHeadRows;
        split->part[index] =
            row_part(problem, first,
                     std::min(kSplitHeadRows, problem.rows - first), false);
        split->family[index] = select_input_backward(split->part[index]);
        // (a last part of up to four rows goes to the streaming family)
        if (split->family[index] != RTHIP_NF4_ALGORITHM_SKINNY &&
            !(index > 0 &&
              split->family[index] == RTHIP_NF4_ALGORITHM_GEMV)) {
            return false;
        }
    }
    return true;
}

// The tiled kernel works in row tiles of 128.  A row count that ends up to 64
// rows past a multiple of 128 would pay a whole tile row for them (11008 x
// 4096: ~93 us, whatever the count); AUTO gives those last rows to the
// small-batch families instead, after the tiled launch for the rows before
// them.  Measured, forward / input backward, nested scales: 272 rows of
// 11008 x 4096 320 -> 243 / 315 -> 237 us, 320 rows 319 -> 283 / 318 -> 273
// us, 2080 rows 1682 -> 1618 / 1649 -> 1594 us; 4096 x 4096 at 272 rows
// 144 -> 116 / 138 -> 112 us; with 94 rows left over both ways are even, so
// from 65 on the tile row stays.
constexpr std::size_t kTileRows = 128;
constexpr std::size_t kTailSplitMaxRows = 64;
bool tail_split(const rthip::LinearProblem& problem, bool forward,
                RowSplit* split) {
    const auto select = forward ? select_forward : select_input_backward;
    const std::size_t tail = problem.rows % kTileRows;
    if (problem.rows <= kTileRows || tail == 0 || tail > kTailSplitMaxRows ||
        select(problem) != RTHIP_NF4_ALGORITHM_MFMA) {
        return false;
    }
    split->count = 2;
    split->part[0] = row_part(problem, 0, problem.rows - tail, forward);
    split->part[1] = row_part(problem, problem.rows - tail, tail, forward);
    split->family[0] = select(split->part[0]);
    split->family[1] = select(split->part[1]);
    return split->family[0] == RTHIP_NF4_ALGORITHM_MFMA &&
           (small_batch_family(split->family[1]) ||
            split->family[1] == RTHIP_NF4_ALGORITHM_GEMV);
}
// Two to four rows of x against weight rows too wide for the GEMV to hold
// that many rows of x in registers (from 16384 weights on) run as two GEMV
// launches of fewer rows where that covers them: the small-batch kernel, the
// only other taker, needs 80 us for 8192 x 28672 where one row through the
// GEMV takes 27.
bool wide_row_split(const rthip::LinearProblem& problem, RowSplit* split) {
    if (problem.rows < 2 || problem.rows > rthip::kGemvMaxRows ||
        select_forward(problem) == RTHIP_NF4_ALGORITHM_GEMV) {
        return false;
    }
    for (std::size_t head = 2; head >= 1; --head) {
        if (head >= problem.rows || problem.rows > 2 * head) {
            continue;
        }
        split->count = 2;
        split->part[0] = row_part(problem, 0, head, true);
        split->part[1] = row_part(problem, head, problem.rows - head, true);
        split->family[0] = select_forward(split->part[0]);
        split->family[1] = select_forward(split->part[1]);
        if (split->family[0] == RTHIP_NF4_ALGORITHM_GEMV &&
            split->family[1] == RTHIP_NF4_ALGORITHM_GEMV) {
            return true;
        }
    }
    return false;
}
bool forward_row_split(const rthip::LinearProblem& problem, RowSplit* split) {
    return forward_small_split(problem, split) ||
           tail_split(problem, true, split) ||
           wide_row_split(problem, split);
}
bool backward_row_split(const rthip::LinearProblem& problem, RowSplit* split) {
    return backward_small_split(problem, split) ||
           tail_split(problem, false, split);
}

// ---- the entry point that allocates nothing ------------------------------
//
// Partial sums of the small-batch input backward, for callers that cannot
// call hipMalloc.  Every GPU holds its own copy of this array at its own
// address; host code never passes the array's name to a kernel or a copy
// (that name is a host-side stand-in), only the address that
// hipGetSymbolAddress gave for the current device.
constexpr std::size_t kStaticScratchBytes = RTHIP_NO_ALLOC_SCRATCH_BYTES;
static __device__ __align__(256) float
    scratch[kStaticScratchBytes / sizeof(float)];

constexpr int kMaxScratchDevices = 64;

// The array of one device: its address there (looked up once, with that
// device current), the stream its users are bound to, and the exclusive right
// to enqueue launches that use it.
struct StaticScratch {
    std::mutex busy;
    float* address = nullptr;
    bool bound = false;
    hipStream_t stream = nullptr;
};
StaticScratch* static_scratch_of_device(int device) {
    static StaticScratch all[kMaxScratchDevices];
    return device >= 0 && device < kMaxScratchDevices ? &all[device] : nullptr;
}

// Leases the current device's array for launches on `stream`; the caller
// holds `lock` until its last launch is enqueued, so that two threads cannot
// interleave their partial-sum and sum launches.  The array is bound to the
// first stream that uses it: launches on one stream are ordered, launches on
// two are not, and nothing here could wait for the other stream without a
// call that may not be made under graph capture.  A call on another stream
// is refused until rthip_release_workspaces has unbound the array.
rthip_status lease_static_scratch(hipStream_t stream, float** out,
                                  std::unique_lock<std::mutex>* lock) {
    int device = 0;
    if (const hipError_t error = hipGetDevice(&device); error != hipSuccess) {
        return from_hip(error, "current device query");
    }
    StaticScratch* const entry = static_scratch_of_device(device);
    if (entry == nullptr) {
        return fail(RTHIP_UNSUPPORTED, "device ordinal %d is out of range",
                    device);
    }
    std::unique_lock<std::mutex> held(entry->busy);
    if (entry->address == nullptr) {
        float* found = nullptr;
        if (const hipError_t error = hipGetSymbolAddress(
                reinterpret_cast<void**>(&found), HIP_SYMBOL(scratch));
            error != hipSuccess) {
            return from_hip(error, "static scratch address lookup");
        }
        if (found == nullptr) {
            return fail(RTHIP_RUNTIME_ERROR,
                        "static scratch address lookup returned null");
        }
        entry->address = found;
    }
    if (entry->bound && entry->stream != stream) {
        return fail(RTHIP_UNSUPPORTED,
                    "the device's static scratch array is in use by another "
                    "stream: calls that share it must be on one stream "
                    "(rthip_release_workspaces unbinds it)");
    }
    entry->bound = true;
    entry->stream = stream;
    *out = entry->address;
    *lock = std::move(held);
    return RTHIP_OK;
}

// After the device has finished with the current device's array, lets the
// next caller bind it to a stream of its choice.
rthip_status unbind_static_scratch() {
    int device = 0;
    if (const hipError_t error = hipGetDevice(&device); error != hipSuccess) {
        return from_hip(error, "current device query");
    }
    StaticScratch* const entry = static_scratch_of_device(device);
    if (entry == nullptr) {
        return RTHIP_OK;
    }
    const std::lock_guard<std::mutex> held(entry->busy);
    if (entry->bound) {
        if (const hipError_t error = hipStreamSynchronize(entry->stream);
            error != hipSuccess) {
            return from_hip(error, "static scratch release");
        }
        entry->bound = false;
    }
    return RTHIP_OK;
}

}  // namespace

extern "C" {

static rthip_status input_backward_common(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset, float* dx,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream, float* partial_sums,
    std::size_t partial_sum_bytes, const rthip::LoraEpilogue& adapter);


uint32_t rthip_abi_version(void) {
    return (RTHIP_ABI_VERSION_MAJOR << 16) | RTHIP_ABI_VERSION_MINOR;
}

const char* rthip_last_error(void) { return g_last_error; }

rthip_status rthip_device_count(int32_t* count) {
    if (count == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "count must not be null");
    }
    *count = 0;
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    *count = device_state().count;
    return ok();
}

rthip_status rthip_device_description(char* buffer, size_t capacity) {
    if (buffer == nullptr || capacity == 0) {
        return fail(RTHIP_INVALID_ARGUMENT, "buffer must not be empty");
    }
    buffer[0] = '\0';
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    std::snprintf(buffer, capacity, "%s", device_state().description);
    return ok();
}

rthip_status rthip_device_memory_host_visible(int32_t* visible) {
    if (visible == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "visible must not be null");
    }
    *visible = 0;
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    *visible = device_state().large_bar ? 1 : 0;
    return ok();
}

rthip_status rthip_malloc(void** pointer, size_t bytes) {
    if (pointer == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "pointer must not be null");
    }
    *pointer = nullptr;
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    if (bytes == 0) {
        return ok();
    }
    return from_hip(hipMalloc(pointer, bytes), "device allocation");
}

rthip_status rthip_free(void* pointer) {
    if (pointer == nullptr) {
        return ok();
    }
    return from_hip(hipFree(pointer), "device free");
}

rthip_status rthip_copy_to_device(void* device, const void* host,
                                  size_t bytes) {
    if (bytes == 0) {
        return ok();
    }
    if (device == nullptr || host == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "copy pointers must not be null");
    }
    return from_hip(hipMemcpy(device, host, bytes, hipMemcpyHostToDevice),
                    "host-to-device copy");
}

rthip_status rthip_copy_to_host(void* host, const void* device, size_t bytes) {
    if (bytes == 0) {
        return ok();
    }
    if (device == nullptr || host == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "copy pointers must not be null");
    }
    return from_hip(hipMemcpy(host, device, bytes, hipMemcpyDeviceToHost),
                    "device-to-host copy");
}

rthip_status rthip_fill_f32(float* device, float value, uint64_t count,
                            void* stream) {
    if (count == 0) {
        return ok();
    }
    if (device == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "fill target must not be null");
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    rthip::launch_fill(device, value, count,
                       static_cast<hipStream_t>(stream));
    return finish_launch("fill kernel launch");
}

rthip_status rthip_stream_synchronize(void* stream) {
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    return from_hip(hipStreamSynchronize(static_cast<hipStream_t>(stream)),
                    "stream synchronisation");
}

rthip_status rthip_nf4_select_algorithm(
    int32_t direction, uint64_t rows, uint64_t input_width,
    uint64_t output_width, uint64_t block_size, int32_t* algorithm
) {
    if (algorithm == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "algorithm must not be null");
    }
    unsigned block_shift = 0;
    if (const rthip_status status = check_dimensions(
            rows, input_width, output_width, block_size, &block_shift);
        status != RTHIP_OK) {
        return status;
    }
    rthip::LinearProblem problem{};
    problem.rows = rows;
    problem.input_width = input_width;
    problem.output_width = output_width;
    problem.block_shift = block_shift;
    RowSplit split;
    if (direction == 0) {
        *algorithm = forward_row_split(problem, &split)
                         ? split.family[0]
                         : select_forward(problem);
    } else if (direction == 1) {
        *algorithm = backward_row_split(problem, &split)
                         ? split.family[0]
                         : select_input_backward(problem);
    } else {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "direction must be 0 (forward) or 1 (input backward)");
    }
    return ok();
}

namespace {

// The adapter arguments of the *_lora_* entry points; a == nullptr: none.
constexpr uint64_t kMaxGroupMembers = 64;

struct LoraArguments {
    const float* a;
    const float* b;
    uint64_t rank;
    float scale;
    float* reduced;
};

rthip_status linear_forward_common(
    int32_t algorithm, const float* x, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* bias_or_null, const LoraArguments& lora, float* y,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream
) {
    if (x == nullptr || y == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "input and output must not be null");
    }
    if (static_cast<const void*>(x) == static_cast<const void*>(y)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear input and output must not alias");
    }
    rthip::LinearProblem problem{};
    if (const rthip_status status = check_dimensions(
            rows, input_width, output_width, block_size,
            &problem.block_shift);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = make_weight_view(
            codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, &problem.weight);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    problem.activations = x;
    problem.bias = bias_or_null;
    problem.result = y;
    problem.rows = rows;
    problem.input_width = input_width;
    problem.output_width = output_width;
    const hipStream_t hip_stream = static_cast<hipStream_t>(stream);

    if (lora.reduced != nullptr) {
        if (lora.a != nullptr) {
            // reduced = x A^T first; the main kernel's epilogue consumes it.
            rthip::launch_lora_reduce(x, lora.a, lora.reduced, rows,
                                      input_width, lora.rank, hip_stream);
        }
        problem.lora.reduced = lora.reduced;
        problem.lora.b = lora.b;
        problem.lora.rank = static_cast<unsigned>(lora.rank);
        problem.lora.scale = lora.scale;
        problem.lora.row_stride = static_cast<unsigned>(lora.rank);
        problem.lora.rank_stride = 1;
    }

    // One family on one problem; RTHIP_OK means "launched".
    const auto launch = [hip_stream](int32_t algorithm,
                                     const rthip::LinearProblem& problem)
        -> rthip_status {
    switch (algorithm) {
    case RTHIP_NF4_ALGORITHM_GENERIC:
        rthip::launch_generic_forward(problem, hip_stream);
        break;
    case RTHIP_NF4_ALGORITHM_GEMV:
        if (!rthip::gemv_forward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the GEMV family needs rows <= %zu, a row width that "
                        "is a multiple of 16 and of the block size and at "
                        "most 32768 (one row of x), 24576 (two) or 16384 "
                        "(three and four), and aligned pointers",
                        rthip::kGemvMaxRows);
        }
        rthip::launch_gemv_forward(problem, hip_stream);
        break;
    case RTHIP_NF4_ALGORITHM_MFMA:
        if (!rthip::mfma_forward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the MFMA family needs a row width that is a "
                        "multiple of 32 and aligned pointers");
        }
        if (const hipError_t status =
                rthip::launch_mfma_forward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "GEMM workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_SKINNY:
        if (!rthip::skinny_forward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the small-batch family needs rows <= %zu, a row "
                        "width that is a multiple of 64 and aligned pointers",
                        rthip::kSkinnyMaxRows);
        }
        if (const hipError_t status =
                rthip::launch_skinny_forward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "small-batch workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_RESIDENT:
        if (!rthip::resident_forward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the resident family needs rows <= %zu, a row width "
                        "of 1024, 2048, 3072 or 4096 and aligned pointers",
                        rthip::kResidentMaxRows);
        }
        if (const hipError_t status =
                rthip::launch_resident_forward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "resident kernel configuration");
        }
        break;
    default:
        return fail(RTHIP_INVALID_ARGUMENT, "unknown algorithm %d",
                    static_cast<int>(algorithm));
    }
    return RTHIP_OK;
    };

    if (algorithm == RTHIP_NF4_ALGORITHM_AUTO) {
        RowSplit split;
        if (forward_row_split(problem, &split)) {
            for (std::size_t index = 0; index < split.count; ++index) {
                if (const rthip_status status =
                        launch(split.family[index], split.part[index]);
                    status != RTHIP_OK) {
                    return status;
                }
            }
            return finish_launch("NF4 linear forward launch");
        }
        algorithm = select_forward(problem);
    }
    if (const rthip_status status = launch(algorithm, problem);
        status != RTHIP_OK) {
        return status;
    }
    return finish_launch("NF4 linear forward launch");
}

rthip_status check_lora_arguments(const LoraArguments& lora, const float* x,
                                  const float* y, uint64_t rows,
                                  uint64_t input_width,
                                  uint64_t output_width) {
    if (lora.b == nullptr || lora.reduced == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the adapter's B matrix and the reduced buffer must not "
                    "be null");
    }
    if (lora.rank == 0 || lora.rank > (1ULL << 20)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "LoRA rank must be greater than zero (and at most 2^20)");
    }
    if (!std::isfinite(lora.scale)) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA scale must be finite");
    }
    if (lora.rank > UINT64_MAX / sizeof(float) / rows ||
        lora.rank > UINT64_MAX / sizeof(float) / input_width ||
        lora.rank > UINT64_MAX / sizeof(float) / output_width) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA dimensions overflow");
    }
    const void* const reduced = lora.reduced;
    if (reduced == static_cast<const void*>(x) ||
        reduced == static_cast<const void*>(y) ||
        reduced == static_cast<const void*>(lora.a) ||
        reduced == static_cast<const void*>(lora.b)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the reduced buffer must not alias another operand");
    }
    return RTHIP_OK;
}

}  // namespace

rthip_status rthip_nf4_linear_forward_with(
    int32_t algorithm, const float* x, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* bias_or_null, float* y, uint64_t rows, uint64_t input_width,
    uint64_t output_width, uint64_t block_size, void* stream
) {
    return linear_forward_common(
        algorithm, x, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, bias_or_null,
        LoraArguments{nullptr, nullptr, 0, 0.0F, nullptr}, y, rows,
        input_width, output_width, block_size, stream);
}

rthip_status rthip_nf4_lora_linear_forward_with(
    int32_t algorithm, const float* x, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* bias_or_null, const float* lora_a, const float* lora_b,
    uint64_t lora_rank, float lora_scale, float* reduced, float* y,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream
) {
    const LoraArguments lora{lora_a, lora_b, lora_rank, lora_scale, reduced};
    if (rows == 0 || input_width == 0 || output_width == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear dimensions must be greater than zero");
    }
    if (const rthip_status status = check_lora_arguments(
            lora, x, y, rows, input_width, output_width);
        status != RTHIP_OK) {
        return status;
    }
    return linear_forward_common(
        algorithm, x, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, bias_or_null, lora, y, rows, input_width,
        output_width, block_size, stream);
}

rthip_status rthip_matmul(const float* left, const float* right, float* out,
                          uint64_t batch_count, uint64_t rows,
                          uint64_t shared, uint64_t columns, void* stream) {
    if (left == nullptr || right == nullptr || out == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "matmul operands must not be null");
    }
    if (batch_count == 0 || rows == 0 || shared == 0 || columns == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "matmul dimensions must be greater than zero");
    }
    constexpr uint64_t kMaxElements = UINT64_MAX / sizeof(float);
    if (rows > kMaxElements / shared || shared > kMaxElements / columns ||
        rows > kMaxElements / columns ||
        batch_count > kMaxElements / (rows * shared) ||
        batch_count > kMaxElements / (shared * columns) ||
        batch_count > kMaxElements / (rows * columns)) {
        return fail(RTHIP_INVALID_ARGUMENT, "matmul dimensions overflow");
    }
    if (static_cast<const void*>(out) == static_cast<const void*>(left) ||
        static_cast<const void*>(out) == static_cast<const void*>(right)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "matmul output must not alias an input");
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    if (const hipError_t status = rthip::launch_dense_matmul(
            left, right, out, batch_count, rows, shared, columns,
            static_cast<hipStream_t>(stream));
        status != hipSuccess) {
        return from_hip(status, "matmul workspace allocation");
    }
    return finish_launch("matmul launch");
}

rthip_status rthip_lora_reduce(const float* x, const float* lora_a,
                               float* reduced, uint64_t rows,
                               uint64_t input_width, uint64_t lora_rank,
                               void* stream) {
    if (x == nullptr || lora_a == nullptr || reduced == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "x, the adapter's A matrix and the reduced buffer must "
                    "not be null");
    }
    if (rows == 0 || input_width == 0 || lora_rank == 0 ||
        lora_rank > (1ULL << 20)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "rows, input width and LoRA rank must be greater than "
                    "zero (rank at most 2^20)");
    }
    if (input_width > UINT64_MAX / sizeof(float) / rows ||
        input_width > UINT64_MAX / sizeof(float) / lora_rank) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA dimensions overflow");
    }
    if (static_cast<const void*>(reduced) == static_cast<const void*>(x) ||
        static_cast<const void*>(reduced) ==
            static_cast<const void*>(lora_a)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the reduced buffer must not alias another operand");
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    rthip::launch_lora_reduce(x, lora_a, reduced, rows, input_width,
                              lora_rank, static_cast<hipStream_t>(stream));
    return finish_launch("LoRA reduce launch");
}

rthip_status rthip_nf4_lora_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    const float* lora_a, const float* lora_b, uint64_t lora_rank,
    float lora_scale, float* reduced, float* y, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream
) {
    return rthip_nf4_lora_linear_forward_with(
        RTHIP_NF4_ALGORITHM_AUTO, x, codes, primary_scales, secondary_scales,
        encoding, second_level_block, offset, bias_or_null, lora_a, lora_b,
        lora_rank, lora_scale, reduced, y, rows, input_width, output_width,
        block_size, stream);
}

rthip_status rthip_nf4_linear_forward(
    const float* x, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* bias_or_null,
    float* y, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream
) {
    return rthip_nf4_linear_forward_with(
        RTHIP_NF4_ALGORITHM_AUTO, x, codes, primary_scales, secondary_scales,
        encoding, second_level_block, offset, bias_or_null, y, rows,
        input_width, output_width, block_size, stream);
}

namespace {

// A member of a grouped forward: the weight, bias and output of
// rthip_nf4_member and, when `lora.reduced` is set, the adapter term of
// rthip_nf4_lora_member.
struct GroupMember {
    rthip_nf4_member base;
    LoraArguments lora;
};

static rthip_status forward_group(
    const float* x, const GroupMember* members, uint64_t member_count,
    int32_t encoding, uint64_t second_level_block, uint64_t rows,
    uint64_t input_width, uint64_t block_size, void* stream
) {
    if (member_count == 0 || member_count > kMaxGroupMembers) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "a group holds between 1 and %llu weights",
                    static_cast<unsigned long long>(kMaxGroupMembers));
    }
    rthip::LinearProblem problems[kMaxGroupMembers];
    for (uint64_t m = 0; m < member_count; ++m) {
        const rthip_nf4_member& member = members[m].base;
        const LoraArguments& lora = members[m].lora;
        rthip::LinearProblem& problem = problems[m];
        problem = rthip::LinearProblem{};
        if (member.y == nullptr) {
            return fail(RTHIP_INVALID_ARGUMENT,
                        "input and output must not be null");
        }
        if (static_cast<const void*>(x) == static_cast<const void*>(member.y)) {
            return fail(RTHIP_INVALID_ARGUMENT,
                        "quantized linear input and output must not alias");
        }
        for (uint64_t other = 0; other < m; ++other) {
            if (members[other].base.y == member.y) {
                return fail(RTHIP_INVALID_ARGUMENT,
                            "two members of a group write the same output");
            }
            if (lora.reduced != nullptr && lora.a != nullptr &&
                members[other].lora.reduced == lora.reduced) {
                return fail(RTHIP_INVALID_ARGUMENT,
                            "two members of a group write the same reduced "
                            "buffer");
            }
        }
        if (const rthip_status status = check_dimensions(
                rows, input_width, member.output_width, block_size,
                &problem.block_shift);
            status != RTHIP_OK) {
            return status;
        }
        if (const rthip_status status = make_weight_view(
                member.codes, member.primary_scales, member.secondary_scales,
                encoding, second_level_block, member.offset, &problem.weight);
            status != RTHIP_OK) {
            return status;
        }
        problem.activations = x;
        problem.bias = member.bias_or_null;
        problem.result = member.y;
        problem.rows = rows;
        problem.input_width = input_width;
        problem.output_width = member.output_width;
        if (lora.reduced != nullptr) {
            if (const rthip_status status = check_lora_arguments(
                    lora, x, member.y, rows, input_width, member.output_width);
                status != RTHIP_OK) {
                return status;
            }
            problem.lora.reduced = lora.reduced;
            problem.lora.b = lora.b;
            problem.lora.rank = static_cast<unsigned>(lora.rank);
            problem.lora.scale = lora.scale;
            problem.lora.row_stride = static_cast<unsigned>(lora.rank);
            problem.lora.rank_stride = 1;
        }
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    const hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    // x.A^T of the members that bring their A along: together where the
    // kernel takes several adapters, before any of the main launches
    {
        rthip::LoraReduceItem items[kMaxGroupMembers];
        std::size_t count = 0;
        for (uint64_t m = 0; m < member_count; ++m) {
            const LoraArguments& lora = members[m].lora;
            if (lora.reduced != nullptr && lora.a != nullptr) {
                items[count++] =
                    rthip::LoraReduceItem{lora.a, lora.reduced, lora.rank};
            }
        }
        if (count != 0) {
            rthip::launch_lora_reduce_group(x, items, count, rows,
                                            input_width, hip_stream);
            if (const rthip_status status =
                    finish_launch("LoRA reduce launch");
                status != RTHIP_OK) {
                return status;
            }
        }
    }
    const auto with_adapter = [&](uint64_t first, uint64_t length) {
        for (uint64_t m = first; m < first + length; ++m) {
            if (problems[m].lora.reduced != nullptr) {
                return true;
            }
        }
        return false;
    };
    uint64_t next = 0;
    while (next < member_count) {
        // the longest run of members from here that one streaming launch takes
        // (members with an adapter term: the one-row kernel only, and only
        // two or more -- one alone goes the way of a call of its own)
        uint64_t run = 0;
        if (rows <= rthip::kGemvMaxRows) {
            run = member_count - next < rthip::kGemvGroupMax
                      ? member_count - next
                      : rthip::kGemvGroupMax;
            while (run > 0 &&
                   !(with_adapter(next, run)
                         ? run > 1 && rthip::gemv1_group_supports(
                                          problems + next, run)
                         : rthip::gemv_group_supports(problems + next, run))) {
                --run;
            }
        }
        if (run > 0) {
            if (with_adapter(next, run)) {
                rthip::launch_gemv1_forward(problems + next, run, hip_stream);
            } else {
                rthip::launch_gemv_group(problems + next, run, hip_stream);
            }
            if (const rthip_status status =
                    finish_launch("NF4 linear forward launch");
                status != RTHIP_OK) {
                return status;
            }
            next += run;
            continue;
        }
        // ... or that the kernel which keeps x in registers takes (two or
        // more members for each of which that kernel is the automatic choice)
        run = member_count - next < rthip::kResidentGroupMax
                  ? member_count - next
                  : rthip::kResidentGroupMax;
        const auto resident_run = [&](uint64_t length) {
            for (uint64_t m = 0; m < length; ++m) {
                // ... as ONE launch: a row count that a call of its own
                // serves in two parts (65...80 rows: 64 and the rest) is
                // launched member by member, or a member's rows past the
                // first part would come from another kernel than in a call
                // of its own
                RowSplit split;
                if (forward_row_split(problems[next + m], &split) ||
                    select_forward(problems[next + m]) !=
                        RTHIP_NF4_ALGORITHM_RESIDENT) {
                    return false;
                }
            }
            return rthip::resident_group_supports(problems + next, length);
        };
        while (run > 1 && !resident_run(run)) {
            --run;
        }
        if (run > 1) {
            if (const hipError_t status = rthip::launch_resident_group(
                    problems + next, run, hip_stream);
                status != hipSuccess) {
                return from_hip(status, "NF4 linear forward launch");
            }
            if (const rthip_status status =
                    finish_launch("NF4 linear forward launch");
                status != RTHIP_OK) {
                return status;
            }
            next += run;
            continue;
        }
        const rthip_nf4_member& member = members[next].base;
        if (const rthip_status status = linear_forward_common(
                RTHIP_NF4_ALGORITHM_AUTO, x, member.codes,
                member.primary_scales, member.secondary_scales, encoding,
                second_level_block, member.offset, member.bias_or_null,
                LoraArguments{nullptr, members[next].lora.b,
                              members[next].lora.rank,
                              members[next].lora.scale,
                              members[next].lora.reduced},
                member.y, rows, input_width, member.output_width, block_size,
                stream);
            status != RTHIP_OK) {
            return status;
        }
        ++next;
    }
    return ok();
}

}  // namespace

rthip_status rthip_nf4_linear_forward_group(
    const float* x, const rthip_nf4_member* members, uint64_t member_count,
    int32_t encoding, uint64_t second_level_block, uint64_t rows,
    uint64_t input_width, uint64_t block_size, void* stream
) {
    if (x == nullptr || members == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "input and members must not be null");
    }
    GroupMember group[kMaxGroupMembers];
    for (uint64_t m = 0; m < member_count && m < kMaxGroupMembers; ++m) {
        group[m].base = members[m];
        group[m].lora = LoraArguments{nullptr, nullptr, 0, 0.0F, nullptr};
    }
    return forward_group(x, group, member_count, encoding, second_level_block,
                         rows, input_width, block_size, stream);
}

rthip_status rthip_nf4_lora_linear_forward_group(
    const float* x, const rthip_nf4_lora_member* members,
    uint64_t member_count, int32_t encoding, uint64_t second_level_block,
    uint64_t rows, uint64_t input_width, uint64_t block_size, void* stream
) {
    if (x == nullptr || members == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "input and members must not be null");
    }
    GroupMember group[kMaxGroupMembers];
    for (uint64_t m = 0; m < member_count && m < kMaxGroupMembers; ++m) {
        const rthip_nf4_lora_member& member = members[m];
        group[m].base = member.base;
        group[m].lora = LoraArguments{nullptr, nullptr, 0, 0.0F, nullptr};
        if (member.lora_b != nullptr || member.reduced != nullptr) {
            group[m].lora = LoraArguments{
                member.lora_a, member.lora_b, member.lora_rank,
                member.lora_scale, member.reduced};
            if (member.reduced == nullptr) {
                return fail(RTHIP_INVALID_ARGUMENT,
                            "the adapter's B matrix and the reduced buffer "
                            "must not be null");
            }
        }
    }
    return forward_group(x, group, member_count, encoding, second_level_block,
                         rows, input_width, block_size, stream);
}

rthip_status rthip_nf4_linear_input_backward_with(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset, float* dx,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream
) {
    return input_backward_common(
        algorithm, dy, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, dx, rows, input_width, output_width,
        block_size, stream, nullptr, 0, rthip::LoraEpilogue{});
}

rthip_status rthip_nf4_lora_linear_input_backward_with(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset,
    const float* lora_a, const float* d_reduced, uint64_t lora_rank,
    float* dx, uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream
) {
    if (lora_a == nullptr || d_reduced == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the adapter's A matrix and the reduced gradient must "
                    "not be null");
    }
    if (lora_rank == 0 || lora_rank > (1ULL << 20)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "LoRA rank must be greater than zero (and at most 2^20)");
    }
    if (rows == 0 || input_width == 0 || output_width == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear dimensions must be greater than zero");
    }
    if (input_width > UINT32_MAX || rows > UINT32_MAX ||
        lora_rank > UINT64_MAX / sizeof(float) / rows ||
        lora_rank > UINT64_MAX / sizeof(float) / input_width) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA dimensions overflow");
    }
    if (static_cast<const void*>(dx) == static_cast<const void*>(lora_a) ||
        static_cast<const void*>(dx) == static_cast<const void*>(d_reduced)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the input gradient must not alias an adapter operand");
    }
    rthip::LoraEpilogue adapter{};
    adapter.reduced = d_reduced;
    adapter.b = lora_a;
    adapter.rank = static_cast<unsigned>(lora_rank);
    adapter.scale = 1.0F;
    adapter.row_stride = 1;
    adapter.rank_stride = static_cast<unsigned>(input_width);
    return input_backward_common(
        algorithm, dy, codes, primary_scales, secondary_scales, encoding,
        second_level_block, offset, dx, rows, input_width, output_width,
        block_size, stream, nullptr, 0, adapter);
}

rthip_status rthip_nf4_lora_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, const float* lora_a,
    const float* d_reduced, uint64_t lora_rank, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream
) {
    return rthip_nf4_lora_linear_input_backward_with(
        RTHIP_NF4_ALGORITHM_AUTO, dy, codes, primary_scales, secondary_scales,
        encoding, second_level_block, offset, lora_a, d_reduced, lora_rank,
        dx, rows, input_width, output_width, block_size, stream);
}

rthip_status rthip_lora_backward(
    const float* dy, const float* x, const float* reduced,
    const float* lora_b, uint64_t lora_rank, float lora_scale,
    float* d_reduced, float* d_lora_a, float* d_lora_b, uint64_t rows,
    uint64_t input_width, uint64_t output_width, void* stream
) {
    if (dy == nullptr || lora_b == nullptr || d_reduced == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "upstream, the adapter's B matrix and the reduced "
                    "gradient must not be null");
    }
    if (d_lora_a != nullptr && x == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the gradient of A needs the layer's input");
    }
    if (d_lora_b != nullptr && reduced == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "the gradient of B needs the reduced activations");
    }
    if (rows == 0 || input_width == 0 || output_width == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear dimensions must be greater than zero");
    }
    if (lora_rank == 0 || lora_rank > (1ULL << 20)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "LoRA rank must be greater than zero (and at most 2^20)");
    }
    if (!std::isfinite(lora_scale)) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA scale must be finite");
    }
    constexpr uint64_t kMaxElements = UINT64_MAX / sizeof(float);
    if (rows > kMaxElements / output_width ||
        rows > kMaxElements / input_width ||
        lora_rank > kMaxElements / rows ||
        lora_rank > kMaxElements / input_width ||
        lora_rank > kMaxElements / output_width) {
        return fail(RTHIP_INVALID_ARGUMENT, "LoRA dimensions overflow");
    }
    const void* const outputs[3] = {d_reduced, d_lora_a, d_lora_b};
    const void* const inputs[4] = {dy, x, reduced, lora_b};
    for (int out = 0; out < 3; ++out) {
        if (outputs[out] == nullptr) {
            continue;
        }
        for (const void* input : inputs) {
            if (outputs[out] == input) {
                return fail(RTHIP_INVALID_ARGUMENT,
                            "an adapter gradient must not alias an input");
            }
        }
        for (int other = 0; other < out; ++other) {
            if (outputs[out] == outputs[other]) {
                return fail(RTHIP_INVALID_ARGUMENT,
                            "two adapter gradients share one buffer");
            }
        }
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    rthip::LoraBackwardProblem problem{};
    problem.upstream = dy;
    problem.activations = x;
    problem.reduced = reduced;
    problem.b = lora_b;
    problem.d_reduced = d_reduced;
    problem.d_a = d_lora_a;
    problem.d_b = d_lora_b;
    problem.rows = rows;
    problem.input_width = input_width;
    problem.output_width = output_width;
    problem.rank = lora_rank;
    problem.scale = lora_scale;
    if (const hipError_t status = rthip::launch_lora_backward(
            problem, static_cast<hipStream_t>(stream));
        status != hipSuccess) {
        return from_hip(status, "adapter-backward workspace allocation");
    }
    return finish_launch("adapter backward launch");
}

// One input backward.  partial_sums == nullptr: any family, partial results
// in the stream workspace.  Otherwise: the small-batch family only, partial
// results in that memory, nothing allocated.
static rthip_status input_backward_common(
    int32_t algorithm, const float* dy, const uint8_t* codes,
    const void* primary_scales, const float* secondary_scales,
    int32_t encoding, uint64_t second_level_block, float offset, float* dx,
    uint64_t rows, uint64_t input_width, uint64_t output_width,
    uint64_t block_size, void* stream, float* partial_sums,
    std::size_t partial_sum_bytes, const rthip::LoraEpilogue& adapter
) {
    if (dy == nullptr || dx == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "upstream and input gradient must not be null");
    }
    if (static_cast<const void*>(dy) == static_cast<const void*>(dx)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "quantized linear upstream and input gradient must not "
                    "alias");
    }
    rthip::LinearProblem problem{};
    if (const rthip_status status = check_dimensions(
            rows, input_width, output_width, block_size,
            &problem.block_shift);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = make_weight_view(
            codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, &problem.weight);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    problem.activations = dy;
    problem.bias = nullptr;
    problem.result = dx;
    problem.rows = rows;
    problem.input_width = input_width;
    problem.output_width = output_width;
    problem.scratch = partial_sums;
    problem.scratch_bytes = partial_sum_bytes;
    problem.lora = adapter;
    const hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    if (partial_sums != nullptr) {
        if (rows > rthip::kSmallBackwardMaxRows ||
            !rthip::small_input_backward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the entry point that allocates nothing covers the "
                        "small-batch input backward only: rows <= %zu, a row "
                        "width that is a multiple of 8, an output width that "
                        "is a multiple of 4 and aligned pointers",
                        rthip::kSmallBackwardMaxRows);
        }
        const std::size_t needed =
            rthip::small_input_backward_scratch_bytes(problem);
        if (needed > partial_sum_bytes) {
            return fail(RTHIP_UNSUPPORTED,
                        "this input backward needs %zu bytes for partial "
                        "sums; the entry point that allocates nothing has "
                        "%zu",
                        needed, partial_sum_bytes);
        }
        algorithm = RTHIP_NF4_ALGORITHM_SKINNY;
    }

    const auto launch = [hip_stream](int32_t algorithm,
                                     const rthip::LinearProblem& problem)
        -> rthip_status {
    switch (algorithm) {
    case RTHIP_NF4_ALGORITHM_GENERIC:
        if (const hipError_t status =
                rthip::launch_generic_input_backward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "input-backward workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_MFMA:
        if (!rthip::mfma_input_backward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the MFMA family needs an output width that is a "
                        "multiple of 32, a row width that is a multiple of "
                        "16 and aligned pointers");
        }
        if (const hipError_t status =
                rthip::launch_mfma_input_backward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "GEMM workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_SKINNY:
        if (!rthip::small_input_backward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the small-batch family needs rows <= %zu, a row "
                        "width that is a multiple of 8, an output width that "
                        "is a multiple of 4 and aligned pointers",
                        rthip::kSmallBackwardMaxRows);
        }
        if (const hipError_t status =
                rthip::launch_small_input_backward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "small-batch workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_GEMV:
        if (!rthip::stream_input_backward_supports(problem)) {
            return fail(RTHIP_UNSUPPORTED,
                        "the streaming family needs rows <= %zu, a block "
                        "size of at least 64 that divides the row width, a "
                        "row width that is a multiple of 16, an output width "
                        "that is a multiple of 4 and aligned pointers",
                        rthip::kStreamBackwardMaxRows);
        }
        if (const hipError_t status =
                rthip::launch_stream_input_backward(problem, hip_stream);
            status != hipSuccess) {
            return from_hip(status, "streaming-backward workspace allocation");
        }
        break;
    case RTHIP_NF4_ALGORITHM_RESIDENT:
        return fail(RTHIP_UNSUPPORTED,
                    "this family implements the forward product only");
    default:
        return fail(RTHIP_INVALID_ARGUMENT, "unknown algorithm %d",
                    static_cast<int>(algorithm));
    }
    return RTHIP_OK;
    };

    if (algorithm == RTHIP_NF4_ALGORITHM_AUTO) {
        RowSplit split;
        if (backward_row_split(problem, &split)) {
            for (std::size_t index = 0; index < split.count; ++index) {
                if (const rthip_status status =
                        launch(split.family[index], split.part[index]);
                    status != RTHIP_OK) {
                    return status;
                }
            }
            return finish_launch("NF4 linear input-backward launch");
        }
        algorithm = select_input_backward(problem);
    }
    if (const rthip_status status = launch(algorithm, problem);
        status != RTHIP_OK) {
        return status;
    }
    return finish_launch("NF4 linear input-backward launch");
}

rthip_status rthip_nf4_linear_input_backward(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream
) {
    return rthip_nf4_linear_input_backward_with(
        RTHIP_NF4_ALGORITHM_AUTO, dy, codes, primary_scales, secondary_scales,
        encoding, second_level_block, offset, dx, rows, input_width,
        output_width, block_size, stream);
}

rthip_status rthip_nf4_linear_input_backward_no_alloc(
    const float* dy, const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* dx, uint64_t rows,
    uint64_t input_width, uint64_t output_width, uint64_t block_size,
    void* stream
) {
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    float* partial_sums = nullptr;
    std::unique_lock<std::mutex> lease;  // until both launches are enqueued
    if (const rthip_status status = lease_static_scratch(
            static_cast<hipStream_t>(stream), &partial_sums, &lease);
        status != RTHIP_OK) {
        return status;
    }
    return input_backward_common(
        RTHIP_NF4_ALGORITHM_SKINNY, dy, codes, primary_scales,
        secondary_scales, encoding, second_level_block, offset, dx, rows,
        input_width, output_width, block_size, stream, partial_sums,
        kStaticScratchBytes, rthip::LoraEpilogue{});
}

rthip_status rthip_nf4_forward_kernel_name(
    uint64_t rows, uint64_t input_width, const uint64_t* output_widths,
    uint64_t member_count, uint64_t block_size, int32_t encoding,
    uint64_t second_level_block, char* name, uint64_t capacity
) {
    if (output_widths == nullptr || name == nullptr || capacity == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "output widths and the name buffer must not be null");
    }
    if (member_count == 0 || member_count > rthip::kGemvGroupMax) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "between 1 and %zu weights share a launch",
                    rthip::kGemvGroupMax);
    }
    name[0] = '\0';
    // stand-ins for device memory: only their alignment is looked at
    alignas(256) static const float activations[4] = {};
    alignas(256) static const std::uint8_t payload[16] = {};
    alignas(256) static float results[rthip::kGemvGroupMax][4];
    rthip::LinearProblem problems[rthip::kGemvGroupMax];
    for (uint64_t m = 0; m < member_count; ++m) {
        rthip::LinearProblem& problem = problems[m];
        problem = rthip::LinearProblem{};
        if (const rthip_status status = check_dimensions(
                rows, input_width, output_widths[m], block_size,
                &problem.block_shift);
            status != RTHIP_OK) {
            return status;
        }
        if (const rthip_status status = make_weight_view(
                payload, payload,
                encoding == RTHIP_NF4_SCALE_FLOAT32 ? nullptr : activations,
                encoding, second_level_block, 0.0F, &problem.weight);
            status != RTHIP_OK) {
            return status;
        }
        problem.activations = activations;
        problem.result = results[m];
        problem.rows = rows;
        problem.input_width = input_width;
        problem.output_width = output_widths[m];
        if (!rthip::gemv1_forward_supports(problem)) {
            return RTHIP_OK;  // another family: no name
        }
    }
    if (member_count > 1 &&
        !rthip::gemv_group_supports(problems, member_count)) {
        return RTHIP_OK;
    }
    rthip::gemv1_kernel_name(problems, member_count, name, capacity);
    return RTHIP_OK;
}

rthip_status rthip_release_workspaces(void* stream, int32_t every_stream) {
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    if (every_stream != 0) {
        if (const rthip_status status = unbind_static_scratch();
            status != RTHIP_OK) {
            return status;
        }
    }
    return from_hip(
        rthip::release_stream_workspaces(static_cast<hipStream_t>(stream),
                                         every_stream != 0),
        "workspace release");
}

rthip_status rthip_nf4_dequantize(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, float* out,
    uint64_t element_count, uint64_t block_size, void* stream
) {
    if (out == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT, "output must not be null");
    }
    if (element_count == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "element count must be positive");
    }
    unsigned block_shift = 0;
    if (!block_shift_for(block_size, &block_shift)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 block size %llu is not one of 32..4096",
                    static_cast<unsigned long long>(block_size));
    }
    rthip::Nf4WeightView weight{};
    if (const rthip_status status = make_weight_view(
            codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, &weight);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    rthip::launch_dequantize(weight, out, element_count, block_shift,
                             static_cast<hipStream_t>(stream));
    return finish_launch("NF4 dequantize launch");
}

rthip_status rthip_nf4_quantize(
    const float* values, uint64_t element_count, uint64_t block_size,
    int32_t encoding, uint64_t second_level_block, uint8_t* codes,
    void* primary_scales, float* secondary_scales, float* fp32_scale_scratch,
    float* host_offset, void* stream
) {
    if (values == nullptr || codes == nullptr || primary_scales == nullptr) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "source values, codes and scales must not be null");
    }
    if (element_count == 0 ||
        element_count > std::numeric_limits<uint64_t>::max() / 8) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "element count must be positive (and addressable)");
    }
    rthip::QuantizeProblem problem{};
    if (!block_shift_for(block_size, &problem.block_shift)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 block size %llu is not one of 32..4096",
                    static_cast<unsigned long long>(block_size));
    }
    problem.values = values;
    problem.element_count = element_count;
    problem.codes = codes;
    if (encoding == RTHIP_NF4_SCALE_FLOAT32) {
        problem.fp32_scales = static_cast<float*>(primary_scales);
    } else if (encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8) {
        if (secondary_scales == nullptr || fp32_scale_scratch == nullptr ||
            host_offset == nullptr) {
            return fail(RTHIP_INVALID_ARGUMENT,
                        "double-quantised scales need the second-level "
                        "buffer, the fp32 scratch and the offset pointer");
        }
        if (!block_shift_for(second_level_block,
                             &problem.second_level_shift)) {
            return fail(RTHIP_INVALID_ARGUMENT,
                        "second-level block size %llu is not one of 32..4096",
                        static_cast<unsigned long long>(second_level_block));
        }
        problem.fp32_scales = fp32_scale_scratch;
        problem.scale_codes = static_cast<uint8_t*>(primary_scales);
        problem.second_level = secondary_scales;
    } else {
        return fail(RTHIP_INVALID_ARGUMENT, "unknown NF4 scale encoding %d",
                    static_cast<int>(encoding));
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    const hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    // [0]: status bits, [1]: the offset (a float): the first status word of
    // the stream workspace, cleared by a kernel (no allocation per call).
    // The call waits for the stream below, so it cannot be captured.
    rthip::WorkspaceLease lease;
    if (const hipError_t error =
            rthip::lease_stream_workspace(hip_stream, &lease);
        error != hipSuccess) {
        return from_hip(error, "quantizer workspace allocation");
    }
    unsigned* const words = reinterpret_cast<unsigned*>(lease.status_words());
    unsigned host_words[2] = {0U, 0U};
    rthip::launch_fill(reinterpret_cast<float*>(words), 0.0F, 2, hip_stream);
    problem.status = words;
    problem.offset = reinterpret_cast<float*>(words + 1);
    rthip::launch_quantize(problem, hip_stream);
    hipError_t error = hipGetLastError();
    if (error == hipSuccess) {
        error = hipMemcpyAsync(host_words, words, sizeof(host_words),
                               hipMemcpyDeviceToHost, hip_stream);
    }
    if (error == hipSuccess) {
        error = hipStreamSynchronize(hip_stream);
    }
    if (error != hipSuccess) {
        return from_hip(error, "NF4 quantize");
    }
    if ((host_words[0] & 1U) != 0U) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 source values must be finite");
    }
    if ((host_words[0] & 2U) != 0U) {
        return fail(RTHIP_OVERFLOW,
                    "NF4 scale mean exceeds the FP32 double-quantization "
                    "range");
    }
    if (host_offset != nullptr) {
        std::memcpy(host_offset, &host_words[1], sizeof(float));
    }
    return ok();
}

rthip_status rthip_nf4_check_payload(
    const uint8_t* codes, const void* primary_scales,
    const float* secondary_scales, int32_t encoding,
    uint64_t second_level_block, float offset, uint64_t element_count,
    uint64_t block_size, void* stream
) {
    if (element_count == 0) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "element count must be positive");
    }
    unsigned block_shift = 0;
    if (!block_shift_for(block_size, &block_shift)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 block size %llu is not one of 32..4096",
                    static_cast<unsigned long long>(block_size));
    }
    rthip::Nf4WeightView weight{};
    if (const rthip_status status = make_weight_view(
            codes, primary_scales, secondary_scales, encoding,
            second_level_block, offset, &weight);
        status != RTHIP_OK) {
        return status;
    }
    if (const rthip_status status = require_device(); status != RTHIP_OK) {
        return status;
    }
    std::size_t second_level_count = 0;
    if (encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8) {
        const uint64_t blocks =
            (element_count + block_size - 1) >> block_shift;
        second_level_count = (blocks + second_level_block - 1) >>
                             weight.second_level_shift;
    }
    const hipStream_t hip_stream = static_cast<hipStream_t>(stream);
    // three status words of the stream workspace (initialised by the launch)
    rthip::WorkspaceLease lease;
    if (const hipError_t error =
            rthip::lease_stream_workspace(hip_stream, &lease);
        error != hipSuccess) {
        return from_hip(error, "payload check workspace allocation");
    }
    static_assert(sizeof(unsigned long long) == sizeof(std::uint64_t));
    unsigned long long* const words =
        reinterpret_cast<unsigned long long*>(lease.status_words());
    unsigned long long host_words[3] = {0, 0, 0};
    rthip::launch_check_payload(weight, element_count, block_shift,
                                second_level_count, words, hip_stream);
    hipError_t error = hipGetLastError();
    if (error == hipSuccess) {
        error = hipMemcpyAsync(host_words, words, sizeof(host_words),
                               hipMemcpyDeviceToHost, hip_stream);
    }
    if (error == hipSuccess) {
        error = hipStreamSynchronize(hip_stream);
    }
    if (error != hipSuccess) {
        return from_hip(error, "NF4 payload check");
    }
    // The reference's order: unused nibble, offset, second-level scales,
    // then the blocks.
    const rthip::PayloadViolation violation =
        rthip::classify_payload(host_words);
    if (violation == rthip::PayloadViolation::UnusedNibble) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 unused high nibble must be zero");
    }
    if (encoding == RTHIP_NF4_SCALE_DOUBLE_QUANTIZED_UINT8 &&
        (!std::isfinite(offset) || offset < 0.0F)) {
        return fail(RTHIP_INVALID_ARGUMENT,
                    "double-quantized NF4 scale offset must be finite and "
                    "nonnegative");
    }
    switch (violation) {
    case rthip::PayloadViolation::SecondLevelScale:
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 second-level scales must be finite and nonnegative");
    case rthip::PayloadViolation::BlockScale:
        return fail(RTHIP_INVALID_ARGUMENT,
                    "NF4 block scales must be finite and nonnegative");
    case rthip::PayloadViolation::ZeroBlockCode:
        return fail(RTHIP_INVALID_ARGUMENT,
                    "zero-scale NF4 blocks must use canonical zero code 7");
    default:
        return ok();
    }
}

}  // extern "C"
