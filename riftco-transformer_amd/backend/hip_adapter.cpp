// Implementation of the `hip` backend adapter.
//
// Device work goes through the kernel C ABI only (hip_runtime.hpp); nothing in
// this file includes a HIP header, so it builds with any C++20 host compiler.
//
// Storage model
//   HipTensorStorage     fp32 tensor in HBM plus a lazily synchronised host
//                        mirror, because TensorStorage::data() must hand out
//                        host spans (src/core/backend/storage.hpp:21-24) that
//                        callers may also write through.  A tensor that is
//                        only ever produced and consumed by kernels never
//                        allocates or touches the mirror.
//   HipNf4WeightStorage  immutable packed codes and scales in HBM.  On servers
//                        that map all of HBM through a large PCIe BAR the host
//                        spans of QuantizedWeightStorage point straight at that
//                        memory: one allocation, resident bytes == logical
//                        bytes, as the reference's accelerator test demands
//                        (tests/core/backend/test_quantized_linear_backend.cpp:424-430).
//                        Otherwise a host copy is kept and counted.
//
// Both operations are synchronous: they return after the stream has drained
// (docs/BACKENDS_AND_PYTHON.md:168).

#include "hip_adapter.hpp"

#include "hip_runtime.hpp"
#include "packed_state.hpp"

#if defined(RIFTCO_TRANSFORMER_IN_TREE)
#include "core/backend/attention/reference/flash_causal.hpp"
#include "core/backend/attention/reference/materialized_causal.hpp"
#include "core/backend/attention/reference/paged_decode.hpp"
#include "core/backend/nn/reference/operations.hpp"
#include "core/backend/optim/adam/reference/update.hpp"
#endif

#include <algorithm>
#include <array>
#include <atomic>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace riftco_transformer::backend_detail {
namespace {

[[noreturn]] void throw_unavailable(const HipRuntime& runtime) {
    std::string message = "hip execution backend is unavailable";
    if (!runtime.reason.empty()) {
        message += ": ";
        message += runtime.reason;
    }
    throw std::runtime_error(message);
}

const HipRuntime& require_runtime() {
    const HipRuntime& runtime = hip_runtime();
    if (!runtime.available) {
        throw_unavailable(runtime);
    }
    return runtime;
}

// Maps an rthip_status to the exception type the reference uses for the same
// condition (src/core/backend/adapters/cuda/adapter.cu:25-32 for bad_alloc).
void check(const HipRuntime& runtime, rthip_status status,
           std::string_view operation) {
    if (status == RTHIP_OK) {
        return;
    }
    std::string message = "hip " + std::string(operation) + ": " +
                          runtime.last_error();
    switch (status) {
    case RTHIP_INVALID_ARGUMENT:
        throw std::invalid_argument(message);
    case RTHIP_OUT_OF_MEMORY:
        throw std::bad_alloc();
    case RTHIP_UNAVAILABLE:
        throw_unavailable(runtime);
    default:
        throw std::runtime_error(message);
    }
}

bool environment_flag(const char* name) noexcept {
    const char* value = std::getenv(name);
    return value != nullptr && std::strcmp(value, "1") == 0;
}

// Decode-sized forwards that are held back to be merged (see
// PendingForwards below) name device memory by address, so they have to be
// launched before any of that memory changes hands or is looked at.
void launch_pending_forwards();
void launch_pending_forwards_or_abort() noexcept;

// Activation buffers come and go with every operation
// (src/nn/quantized_linear.cpp:41 allocates the output of each forward), and
// a device allocation costs far more than the decode kernels do.  Released
// buffers are therefore kept, by power-of-two size class, and handed out
// again.  Every launch and copy of the adapter goes to the default stream, so
// a buffer that is reused is only touched after the work that last used it.
// RIFTCO_TRANSFORMER_HIP_POOL=0 turns the pool off; it holds at most
// kPoolLimitBytes and never buffers above kLargestPooledBytes.
class BufferPool final {
public:
    static BufferPool& instance() {
        static BufferPool* pool = new BufferPool();  // outlives every tensor
        return *pool;
    }

    // Capacity actually allocated for a request (the size class).
    [[nodiscard]] static std::size_t capacity_for(std::size_t bytes) noexcept {
        if (bytes > kLargestPooledBytes) {
            return bytes;
        }
        std::size_t capacity = kSmallestClassBytes;
        while (capacity < bytes) {
            capacity *= 2;
        }
        return capacity;
    }

    [[nodiscard]] void* acquire(std::size_t capacity) {
        if (enabled_ && capacity <= kLargestPooledBytes) {
            const std::lock_guard<std::mutex> lock(guard_);
            auto& free_list = free_[capacity];
            if (!free_list.empty()) {
                void* pointer = free_list.back();
                free_list.pop_back();
                held_bytes_ -= capacity;
                return pointer;
            }
        }
        const HipRuntime& runtime = require_runtime();
        void* pointer = nullptr;
        rthip_status status = runtime.malloc(&pointer, capacity);
        if (status == RTHIP_OUT_OF_MEMORY && trim()) {
            status = runtime.malloc(&pointer, capacity);
        }
        check(runtime, status, "device allocation");
        return pointer;
    }

    void release(void* pointer, std::size_t capacity) noexcept {
        if (enabled_ && capacity <= kLargestPooledBytes) {
            const std::lock_guard<std::mutex> lock(guard_);
            if (held_bytes_ + capacity <= kPoolLimitBytes) {
                try {
                    free_[capacity].push_back(pointer);
                    held_bytes_ += capacity;
                    return;
                } catch (...) {
                    // fall through to a plain free
                }
            }
        }
        static_cast<void>(hip_runtime().free(pointer));
    }

private:
    static constexpr std::size_t kSmallestClassBytes = 256;
    static constexpr std::size_t kLargestPooledBytes = std::size_t{1} << 28;
    static constexpr std::size_t kPoolLimitBytes = std::size_t{1} << 31;

    BufferPool() {
        const char* value = std::getenv("RIFTCO_TRANSFORMER_HIP_POOL");
        enabled_ = value == nullptr || std::strcmp(value, "0") != 0;
    }

    // Gives everything back to the driver; true if that freed anything.
    bool trim() noexcept {
        const std::lock_guard<std::mutex> lock(guard_);
        bool freed = false;
        for (auto& [capacity, free_list] : free_) {
            for (void* pointer : free_list) {
                static_cast<void>(hip_runtime().free(pointer));
                freed = true;
            }
            free_list.clear();
        }
        held_bytes_ = 0;
        return freed;
    }

    bool enabled_ = true;
    std::mutex guard_;
    std::map<std::size_t, std::vector<void*>> free_;
    std::size_t held_bytes_ = 0;
};

// Owning handle of one HBM allocation.  Pooled buffers (activations) come
// from BufferPool; exact ones (weight payloads, which live as long as the
// model) are allocated and freed directly.
class DeviceBuffer final {
public:
    enum class Kind { Exact, Pooled };

    DeviceBuffer() = default;
    explicit DeviceBuffer(std::size_t bytes, Kind kind = Kind::Exact)
        : bytes_(bytes), kind_(kind) {
        if (bytes_ == 0) {
            return;
        }
        if (kind_ == Kind::Pooled) {
            capacity_ = BufferPool::capacity_for(bytes_);
            pointer_ = BufferPool::instance().acquire(capacity_);
        } else {
            capacity_ = bytes_;
            const HipRuntime& runtime = require_runtime();
            check(runtime, runtime.malloc(&pointer_, bytes_),
                  "device allocation");
        }
    }
    DeviceBuffer(const void* host, std::size_t bytes, Kind kind = Kind::Exact)
        : DeviceBuffer(bytes, kind) {
        if (bytes_ != 0) {
            const HipRuntime& runtime = require_runtime();
            const rthip_status status =
                runtime.copy_to_device(pointer_, host, bytes_);
            if (status != RTHIP_OK) {
                release();
                check(runtime, status, "host-to-device copy");
            }
        }
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    DeviceBuffer(DeviceBuffer&& other) noexcept
        : pointer_(std::exchange(other.pointer_, nullptr)),
          bytes_(std::exchange(other.bytes_, 0)),
          capacity_(std::exchange(other.capacity_, 0)),
          kind_(other.kind_) {}
    DeviceBuffer& operator=(DeviceBuffer&& other) noexcept {
        if (this != &other) {
            release();
            pointer_ = std::exchange(other.pointer_, nullptr);
            bytes_ = std::exchange(other.bytes_, 0);
            capacity_ = std::exchange(other.capacity_, 0);
            kind_ = other.kind_;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    [[nodiscard]] void* get() const noexcept { return pointer_; }
    [[nodiscard]] std::size_t bytes() const noexcept { return bytes_; }

private:
    void release() noexcept {
        if (pointer_ == nullptr) {
            return;
        }
        launch_pending_forwards_or_abort();
        if (kind_ == Kind::Pooled) {
            BufferPool::instance().release(pointer_, capacity_);
        } else {
            static_cast<void>(hip_runtime().free(pointer_));
        }
        pointer_ = nullptr;
    }

    void* pointer_ = nullptr;
    std::size_t bytes_ = 0;
    std::size_t capacity_ = 0;
    Kind kind_ = Kind::Exact;
};

// The reference contract is that an adapter has finished writing its output
// when it returns (docs/BACKENDS_AND_PYTHON.md:168).  Host code can only see
// a hip tensor through data(), which copies from the device with a call that
// itself waits for the default stream, so a synchronisation per operation is
// not needed for correctness, and by default there is none: operations queue
// behind each other on the device, and decode-sized forwards that share their
// input are merged (below).  RIFTCO_TRANSFORMER_HIP_MERGE=0 restores one
// launch per call, each followed by a synchronisation (unless
// RIFTCO_TRANSFORMER_HIP_ASYNC=1 keeps the queued execution).  Errors of a
// queued kernel surface at the next synchronising call.
bool merge_requested() noexcept {
    // on unless RIFTCO_TRANSFORMER_HIP_MERGE=0
    static const bool merge = [] {
        const char* value = std::getenv("RIFTCO_TRANSFORMER_HIP_MERGE");
        return value == nullptr || std::strcmp(value, "0") != 0;
    }();
    return merge;
}

void finish_operation(const HipRuntime& runtime, std::string_view operation) {
    static const bool deferred =
        environment_flag("RIFTCO_TRANSFORMER_HIP_ASYNC") || merge_requested();
    if (!deferred) {
        check(runtime, runtime.stream_synchronize(nullptr), operation);
    }
}

// Merged forwards (the default; RIFTCO_TRANSFORMER_HIP_MERGE=0 turns them
// off), which imply the queued execution of RIFTCO_TRANSFORMER_HIP_ASYNC=1.
// A decoder calls the query, key and value
// projections -- and gate and up -- one after the other on the same input
// (src/model/decoder_only_transformer.cpp:406-419), each through
// quantized_linear_forward.  At up to 128 rows a launch costs about as much
// as the bytes it reads, so consecutive forwards that share their input are
// held back here and go out together through rthip_nf4_linear_forward_group,
// whose outputs are bit for bit those of separate launches.
//
// What is held back is a list of device addresses, so it is launched
//   - when a forward arrives that does not fit the list (other input, shape,
//     encoding; an output already in the list) or the list is full,
//   - before any other operation of the adapter,
//   - before host code sees a tensor (data()), and
//   - before any device buffer is released.
// An error of a held-back launch is reported by the call that launches it.
class PendingForwards final {
public:
    // the range of the kernels that take several weights per launch
    static constexpr std::size_t kMaximumRows = 128;
    static constexpr std::size_t kCapacity = 4;     // weights per launch

    struct Shape {
        const float* input = nullptr;
        std::int32_t encoding = 0;
        std::size_t second_level_block = 0;
        std::size_t rows = 0;
        std::size_t input_width = 0;
        std::size_t block_size = 0;
        [[nodiscard]] bool operator==(const Shape&) const noexcept = default;
    };

    static PendingForwards& instance() {
        static PendingForwards pending;
        return pending;
    }

    void add(const Shape& shape, const rthip_nf4_lora_member& member) {
        const std::lock_guard<std::mutex> lock(mutex_);
        ++statistics_.requests;
        bool fits = count_ != 0 && count_ < kCapacity && shape == shape_;
        for (std::size_t m = 0; fits && m < count_; ++m) {
            fits = members_[m].base.y != member.base.y &&
                   (member.reduced == nullptr ||
                    members_[m].reduced != member.reduced);
        }
        if (!fits) {
            launch_locked();
        }
        shape_ = shape;
        members_[count_++] = member;
        if (count_ == kCapacity) {
            launch_locked();
        }
    }
    void add(const Shape& shape, const rthip_nf4_member& member) {
        rthip_nf4_lora_member plain{};
        plain.base = member;
        add(shape, plain);
    }

    void launch() {
        const std::lock_guard<std::mutex> lock(mutex_);
        launch_locked();
    }

    [[nodiscard]] HipForwardMergeStatistics statistics() noexcept {
        const std::lock_guard<std::mutex> lock(mutex_);
        return statistics_;
    }

private:
    void launch_locked() {
        if (count_ == 0) {
            return;
        }
        const std::size_t count = std::exchange(count_, 0);
        ++statistics_.launches;
        const HipRuntime& runtime = require_runtime();
        bool adapters = false;
        std::array<rthip_nf4_member, kCapacity> plain{};
        for (std::size_t m = 0; m < count; ++m) {
            adapters = adapters || members_[m].reduced != nullptr;
            plain[m] = members_[m].base;
        }
        check(runtime,
              adapters ? runtime.nf4_lora_linear_forward_group(
                             shape_.input, members_.data(), count,
                             shape_.encoding, shape_.second_level_block,
                             shape_.rows, shape_.input_width,
                             shape_.block_size, nullptr)
                       : runtime.nf4_linear_forward_group(
                             shape_.input, plain.data(), count,
                             shape_.encoding, shape_.second_level_block,
                             shape_.rows, shape_.input_width,
                             shape_.block_size, nullptr),
              "quantized-linear forward (merged launch)");
    }

    std::mutex mutex_;
    Shape shape_;
    std::array<rthip_nf4_lora_member, kCapacity> members_{};
    std::size_t count_ = 0;
    HipForwardMergeStatistics statistics_{};
};

void launch_pending_forwards() {
    if (merge_requested()) {
        PendingForwards::instance().launch();
    }
}

// For destructors and the noexcept accessors: a launch that fails there ends
// the process, as a failing read-back does (refresh_host).
void launch_pending_forwards_or_abort() noexcept {
    try {
        launch_pending_forwards();
    } catch (...) {
        std::abort();
    }
}

class HipTensorStorage final : public TensorStorage {
public:
    // A tensor of one value.  The value is written where it is first needed:
    // the outputs the reference allocates before every operation
    // (src/nn/quantized_linear.cpp:41) are overwritten by the kernel that
    // follows and never filled.
    HipTensorStorage(std::size_t element_count, float fill_value)
        : count_(element_count),
          device_(checked_bytes(element_count), DeviceBuffer::Kind::Pooled),
          fill_value_(fill_value),
          freshest_(Freshest::Neither) {
        static_cast<void>(require_runtime());
    }

    // A tensor of host values (the result of an operation that ran on the
    // host, an input a caller built): they go to HBM when a kernel first
    // reads the tensor -- never, if only host code does.
    explicit HipTensorStorage(std::vector<float> values)
        : count_(values.size()),
          device_(checked_bytes(values.size()), DeviceBuffer::Kind::Pooled),
          host_(std::move(values)),
          freshest_(Freshest::Host) {
        static_cast<void>(require_runtime());
    }

    [[nodiscard]] ExecutionBackend backend() const noexcept override {
        return kHipBackend;
    }
    [[nodiscard]] std::size_t size() const noexcept override {
        return count_;
    }

    // A writable span: from here on the host copy may be newer than HBM.
    [[nodiscard]] std::span<float> data() noexcept override {
        launch_pending_forwards_or_abort();
        const std::lock_guard<std::mutex> lock(sync_);
        refresh_host_locked();
        freshest_ = Freshest::Host;
        return host_;
    }
    // Readers may come from several threads at once (two forwards that share
    // an input, a forward and a host read): the lazily synchronised state is
    // guarded, and the span stays valid because the host copy is sized once.
    [[nodiscard]] std::span<const float> data() const noexcept override {
        launch_pending_forwards_or_abort();
        const std::lock_guard<std::mutex> lock(sync_);
        refresh_host_locked();
        return host_;
    }

    // The persistent HBM allocation; identifies the tensor for the
    // dispatcher's aliasing checks and triggers no transfer.
    [[nodiscard]] void* native_handle() noexcept override {
        return device_.get();
    }
    [[nodiscard]] const void* native_handle() const noexcept override {
        return device_.get();
    }

    [[nodiscard]] std::unique_ptr<TensorStorage> clone() const override {
        const auto values = data();
        return std::make_unique<HipTensorStorage>(
            std::vector<float>(values.begin(), values.end()));
    }

    // HBM pointer with the tensor's current contents.
    [[nodiscard]] const float* device_for_read() const {
        const std::lock_guard<std::mutex> lock(sync_);
        if (freshest_ == Freshest::Neither) {
            const HipRuntime& runtime = require_runtime();
            check(runtime,
                  runtime.fill_f32(static_cast<float*>(device_.get()),
                                   fill_value_, count_, nullptr),
                  "tensor fill");
            freshest_ = Freshest::Device;
            finish_operation(runtime, "tensor fill synchronisation");
        }
        if (freshest_ == Freshest::Host) {
            const HipRuntime& runtime = require_runtime();
            check(runtime,
                  runtime.copy_to_device(device_.get(), host_.data(),
                                         count_ * sizeof(float)),
                  "tensor upload");
            freshest_ = Freshest::Both;
        }
        return static_cast<const float*>(device_.get());
    }

    // HBM pointer that a kernel is about to overwrite completely.
    [[nodiscard]] float* device_for_overwrite() noexcept {
        const std::lock_guard<std::mutex> lock(sync_);
        freshest_ = Freshest::Device;
        return static_cast<float*>(device_.get());
    }

private:
    // Neither: no copy has been written yet, every element is fill_value_.
    enum class Freshest { Host, Device, Both, Neither };

    static std::size_t checked_bytes(std::size_t element_count) {
        if (element_count >
            std::numeric_limits<std::size_t>::max() / sizeof(float)) {
            throw std::overflow_error(
                "hip tensor allocation size overflow");
        }
        return element_count * sizeof(float);
    }

    // noexcept by contract: a failing device read-back ends the process, as a
    // failing access to a managed CUDA allocation would.
    // (sync_ held; queued forwards have been launched by the caller, outside
    // the lock: launching them reads and writes other tensors' state)
    void refresh_host_locked() const noexcept {
        if (freshest_ == Freshest::Neither) {
            host_.assign(count_, fill_value_);
            freshest_ = Freshest::Host;  // HBM gets it when a kernel reads it
            return;
        }
        if (freshest_ != Freshest::Device) {
            return;
        }
        host_.resize(count_);
        const HipRuntime& runtime = hip_runtime();
        if (count_ != 0 &&
            runtime.copy_to_host(host_.data(), device_.get(),
                                 count_ * sizeof(float)) != RTHIP_OK) {
            std::abort();
        }
        freshest_ = Freshest::Both;
    }

    std::size_t count_;
    DeviceBuffer device_;
    float fill_value_ = 0.0F;
    mutable std::mutex sync_;  // guards host_ and freshest_
    mutable std::vector<float> host_;
    mutable Freshest freshest_;
};

// One payload array of a packed weight: HBM allocation plus, only where HBM
// is not host-visible (or a mirror was asked for), a host copy.
template <typename Element>
class WeightArray final {
public:
    WeightArray() = default;
    WeightArray(std::vector<Element> values, bool keep_host_copy)
        : count_(values.size()),
          device_(values.data(), values.size() * sizeof(Element)) {
        if (keep_host_copy) {
            host_ = std::move(values);
        }
    }

    // From `count` elements stored as bytes that need not be aligned (a
    // checkpoint's packed state): copied to HBM from where they lie.
    WeightArray(std::span<const std::uint8_t> bytes, bool keep_host_copy)
        : count_(bytes.size() / sizeof(Element)),
          device_(bytes.data(), bytes.size()) {
        if (keep_host_copy && count_ != 0) {
            host_.resize(count_);
            std::memcpy(host_.data(), bytes.data(), bytes.size());
        }
    }

    [[nodiscard]] std::size_t size() const noexcept { return count_; }

    [[nodiscard]] std::span<const Element> values() const noexcept {
        if (!host_.empty()) {
            return host_;
        }
        return {static_cast<const Element*>(device_.get()), count_};
    }
    [[nodiscard]] const Element* device() const noexcept {
        return static_cast<const Element*>(device_.get());
    }
    [[nodiscard]] std::size_t resident_bytes() const noexcept {
        return count_ * sizeof(Element) + host_.size() * sizeof(Element);
    }

private:
    std::size_t count_ = 0;
    DeviceBuffer device_;
    std::vector<Element> host_;
};

bool scale_mirror_requested() noexcept {
    return environment_flag("RIFTCO_TRANSFORMER_HIP_SCALE_MIRROR");
}

class HipNf4WeightStorage final : public QuantizedWeightStorage,
                                  public ScaleValidationMemo {
public:
    HipNf4WeightStorage(std::vector<std::uint8_t> packed_codes,
                        Nf4ScaleStorageData scales, bool host_visible)
        : encoding_(scales.encoding),
          packed_codes_(std::move(packed_codes), !host_visible),
          fp32_scales_(std::move(scales.fp32_scales),
                       !host_visible || scale_mirror_requested()),
          quantized_scales_(std::move(scales.quantized_scales),
                            !host_visible || scale_mirror_requested()),
          second_level_scales_(std::move(scales.second_level_scales),
                               !host_visible || scale_mirror_requested()),
          second_level_block_size_(scales.second_level_block_size),
          offset_(scales.offset) {}

    // From one entry of a packed model state: every array goes from the
    // caller's bytes to HBM without an intermediate vector.
    HipNf4WeightStorage(const PackedWeightView& weight, bool host_visible)
        : encoding_(weight.double_quantized
                        ? Nf4ScaleEncoding::DoubleQuantizedUInt8
                        : Nf4ScaleEncoding::Float32),
          packed_codes_(weight.packed_codes, !host_visible),
          fp32_scales_(weight.block_scale_bytes,
                       !host_visible || scale_mirror_requested()),
          quantized_scales_(weight.scale_codes,
                            !host_visible || scale_mirror_requested()),
          second_level_scales_(weight.second_level_scale_bytes,
                               !host_visible || scale_mirror_requested()),
          second_level_block_size_(weight.scale_block_size),
          offset_(weight.offset) {}

    [[nodiscard]] ExecutionBackend backend() const noexcept override {
        return kHipBackend;
    }
    [[nodiscard]] std::span<const std::uint8_t> packed_codes()
        const noexcept override {
        return packed_codes_.values();
    }
    [[nodiscard]] Nf4ScaleStorageView scale_storage() const noexcept override {
        return {encoding_,
                fp32_scales_.values(),
                quantized_scales_.values(),
                second_level_scales_.values(),
                second_level_block_size_,
                offset_};
    }
    [[nodiscard]] const void* packed_codes_native_handle()
        const noexcept override {
        return packed_codes_.device();
    }
    [[nodiscard]] const void* primary_scales_native_handle()
        const noexcept override {
        return encoding_ == Nf4ScaleEncoding::Float32
            ? static_cast<const void*>(fp32_scales_.device())
            : static_cast<const void*>(quantized_scales_.device());
    }
    [[nodiscard]] const void* secondary_scales_native_handle()
        const noexcept override {
        return encoding_ == Nf4ScaleEncoding::DoubleQuantizedUInt8
            ? static_cast<const void*>(second_level_scales_.device())
            : nullptr;
    }
    // Every persistent byte: HBM plus any host copy; the 4-byte offset of the
    // double-quantised encoding lives in this object and counts once.
    [[nodiscard]] std::size_t resident_payload_bytes()
        const noexcept override {
        return packed_codes_.resident_bytes() + fp32_scales_.resident_bytes() +
               quantized_scales_.resident_bytes() +
               second_level_scales_.resident_bytes() +
               (encoding_ == Nf4ScaleEncoding::DoubleQuantizedUInt8
                    ? sizeof(float)
                    : 0);
    }

    [[nodiscard]] bool scales_validated() const noexcept override {
        return scales_validated_.load(std::memory_order_acquire);
    }
    void mark_scales_validated() const noexcept override {
        scales_validated_.store(true, std::memory_order_release);
    }

    [[nodiscard]] Nf4ScaleEncoding encoding() const noexcept {
        return encoding_;
    }
    [[nodiscard]] std::size_t second_level_block_size() const noexcept {
        return second_level_block_size_;
    }
    [[nodiscard]] float offset() const noexcept { return offset_; }

    [[nodiscard]] std::size_t packed_code_count() const noexcept {
        return packed_codes_.size();
    }
    [[nodiscard]] std::size_t fp32_scale_count() const noexcept {
        return fp32_scales_.size();
    }
    [[nodiscard]] std::size_t scale_code_count() const noexcept {
        return quantized_scales_.size();
    }
    [[nodiscard]] std::size_t second_level_scale_count() const noexcept {
        return second_level_scales_.size();
    }
    [[nodiscard]] const float* fp32_scales_device() const noexcept {
        return fp32_scales_.device();
    }
    [[nodiscard]] const std::uint8_t* scale_codes_device() const noexcept {
        return quantized_scales_.device();
    }
    [[nodiscard]] const float* second_level_scales_device() const noexcept {
        return second_level_scales_.device();
    }

private:
    Nf4ScaleEncoding encoding_;
    WeightArray<std::uint8_t> packed_codes_;
    WeightArray<float> fp32_scales_;
    WeightArray<std::uint8_t> quantized_scales_;
    WeightArray<float> second_level_scales_;
    std::size_t second_level_block_size_;
    float offset_;
    mutable std::atomic<bool> scales_validated_{false};
};

const HipTensorStorage& require_hip_tensor(const TensorStorage& storage,
                                           std::string_view operation) {
    const auto* tensor = dynamic_cast<const HipTensorStorage*>(&storage);
    if (tensor == nullptr) {
        throw std::invalid_argument("hip " + std::string(operation) +
                                    " requires hip tensor storage");
    }
    return *tensor;
}

HipTensorStorage& require_hip_tensor(TensorStorage& storage,
                                     std::string_view operation) {
    auto* tensor = dynamic_cast<HipTensorStorage*>(&storage);
    if (tensor == nullptr) {
        throw std::invalid_argument("hip " + std::string(operation) +
                                    " requires hip tensor storage");
    }
    return *tensor;
}

const HipNf4WeightStorage& require_hip_weight(
    const QuantizedWeightStorage& storage, std::string_view operation
) {
    const auto* weight = dynamic_cast<const HipNf4WeightStorage*>(&storage);
    if (weight == nullptr) {
        throw std::invalid_argument("hip " + std::string(operation) +
                                    " requires hip quantized-weight storage");
    }
    if (weight->packed_codes_native_handle() == nullptr ||
        weight->primary_scales_native_handle() == nullptr) {
        throw std::logic_error("hip " + std::string(operation) +
                               " received packed storage without a native "
                               "allocation");
    }
    return *weight;
}

class HipBackendAdapter final : public BackendAdapter {
public:
    [[nodiscard]] std::string_view name() const noexcept override {
        return "hip";
    }
    [[nodiscard]] bool is_available() const noexcept override {
        return hip_runtime().available;
    }
    [[nodiscard]] std::string_view unavailability_reason()
        const noexcept override {
        return hip_runtime().reason;
    }

    [[nodiscard]] std::unique_ptr<TensorStorage> make_storage(
        std::size_t element_count, float fill_value
    ) const override {
        return std::make_unique<HipTensorStorage>(element_count, fill_value);
    }
    [[nodiscard]] std::unique_ptr<TensorStorage> make_storage(
        std::vector<float> values
    ) const override {
        return std::make_unique<HipTensorStorage>(std::move(values));
    }

    [[nodiscard]] std::unique_ptr<QuantizedWeightStorage>
    make_nf4_weight_storage(std::vector<std::uint8_t> packed_codes,
                            Nf4ScaleStorageData scales) const override {
        const HipRuntime& runtime = require_runtime();
        return std::make_unique<HipNf4WeightStorage>(
            std::move(packed_codes), std::move(scales),
            runtime.host_visible_memory);
    }

    void quantized_linear_forward(
        const QuantizedLinearForwardRequest& request
    ) const override {
        constexpr std::string_view operation = "quantized-linear forward";
        const HipRuntime& runtime = require_runtime();
        const auto& input = require_hip_tensor(request.input, operation);
        const auto& weight = require_hip_weight(request.weight, operation);
        auto& output = require_hip_tensor(request.output, operation);
        const float* source = input.device_for_read();
        if (merge_requested() &&
            request.dimensions.rows <= PendingForwards::kMaximumRows) {
            rthip_nf4_member member{};
            member.codes = static_cast<const std::uint8_t*>(
                weight.packed_codes_native_handle());
            member.primary_scales = weight.primary_scales_native_handle();
            member.secondary_scales = static_cast<const float*>(
                weight.secondary_scales_native_handle());
            member.offset = weight.offset();
            member.bias_or_null = nullptr;
            member.y = output.device_for_overwrite();
            member.output_width = request.dimensions.output_width;
            PendingForwards::instance().add(
                {source, static_cast<std::int32_t>(weight.encoding()),
                 weight.second_level_block_size(), request.dimensions.rows,
                 request.dimensions.input_width,
                 request.dimensions.block_size},
                member);
            return;
        }
        launch_pending_forwards();
        check(runtime,
              runtime.nf4_linear_forward(
                  source,
                  static_cast<const std::uint8_t*>(
                      weight.packed_codes_native_handle()),
                  weight.primary_scales_native_handle(),
                  static_cast<const float*>(
                      weight.secondary_scales_native_handle()),
                  static_cast<int32_t>(weight.encoding()),
                  weight.second_level_block_size(), weight.offset(), nullptr,
                  output.device_for_overwrite(), request.dimensions.rows,
                  request.dimensions.input_width,
                  request.dimensions.output_width,
                  request.dimensions.block_size, nullptr),
              operation);
        finish_operation(runtime,
                         "quantized-linear forward synchronisation");
    }

    void quantized_linear_input_backward(
        const QuantizedLinearInputBackwardRequest& request
    ) const override {
        constexpr std::string_view operation =
            "quantized-linear input backward";
        const HipRuntime& runtime = require_runtime();
        const auto& upstream = require_hip_tensor(request.upstream, operation);
        const auto& weight = require_hip_weight(request.weight, operation);
        auto& gradient = require_hip_tensor(request.input_gradient, operation);
        launch_pending_forwards();
        const float* source = upstream.device_for_read();
        check(runtime,
              runtime.nf4_linear_input_backward(
                  source,
                  static_cast<const std::uint8_t*>(
                      weight.packed_codes_native_handle()),
                  weight.primary_scales_native_handle(),
                  static_cast<const float*>(
                      weight.secondary_scales_native_handle()),
                  static_cast<int32_t>(weight.encoding()),
                  weight.second_level_block_size(), weight.offset(),
                  gradient.device_for_overwrite(), request.dimensions.rows,
                  request.dimensions.input_width,
                  request.dimensions.output_width,
                  request.dimensions.block_size, nullptr),
              operation);
        finish_operation(runtime,
                         "quantized-linear input-backward synchronisation");
    }

#if defined(RIFTCO_TRANSFORMER_IN_TREE)
    // Inside the reference tree BackendAdapter has 27 more pure virtuals.  As
    // the TPU adapter does (src/core/backend/adapters/tpu/adapter.cpp:114-200),
    // capabilities without a native kernel run the reference host loops on
    // the storage's host spans; the mirror of HipTensorStorage keeps those
    // coherent with HBM.
    // Dense matmul runs on the device (BackendAdapter::matmul,
    // src/core/backend/adapter.hpp:46-52).
    void matmul(const MatmulRequest& request) const override {
        constexpr std::string_view operation = "matmul";
        const HipRuntime& runtime = require_runtime();
        launch_pending_forwards();
        const auto& left = require_hip_tensor(request.left, operation);
        const auto& right = require_hip_tensor(request.right, operation);
        auto& output = require_hip_tensor(request.output, operation);
        const float* left_device = left.device_for_read();
        const float* right_device = right.device_for_read();
        check(runtime,
              runtime.matmul(left_device, right_device,
                             output.device_for_overwrite(),
                             request.dimensions.batch_count,
                             request.dimensions.rows,
                             request.dimensions.shared,
                             request.dimensions.columns, nullptr),
              operation);
        finish_operation(runtime, "matmul synchronisation");
    }
    void unary_elementwise(
        const UnaryElementwiseRequest& request) const override {
        nn_reference_unary_elementwise(request);
    }
    void binary_elementwise(
        const BinaryElementwiseRequest& request) const override {
        nn_reference_binary_elementwise(request);
    }
    void scale(const ScaleRequest& request) const override {
        nn_reference_scale(request);
    }
    void gelu_forward(const GeluForwardRequest& request) const override {
        nn_reference_gelu_forward(request);
    }
    void gelu_backward(const GeluBackwardRequest& request) const override {
        nn_reference_gelu_backward(request);
    }
    void reduce(const ReductionRequest& request) const override {
        nn_reference_reduce(request);
    }
    void copy(const CopyRequest& request) const override {
        nn_reference_copy(request);
    }
    void permute(const PermuteRequest& request) const override {
        nn_reference_permute(request);
    }
    void broadcast(const BroadcastRequest& request) const override {
        nn_reference_broadcast(request);
    }
    void sum_to_shape(const SumToShapeRequest& request) const override {
        nn_reference_sum_to_shape(request);
    }
    void softmax_forward(
        const SoftmaxForwardRequest& request) const override {
        nn_reference_softmax_forward(request);
    }
    void softmax_backward(
        const SoftmaxBackwardRequest& request) const override {
        nn_reference_softmax_backward(request);
    }
    void causal_softmax_forward(
        const CausalSoftmaxForwardRequest& request) const override {
        nn_reference_causal_softmax_forward(request);
    }
    void causal_softmax_backward(
        const CausalSoftmaxBackwardRequest& request) const override {
        nn_reference_causal_softmax_backward(request);
    }
    void gather_rows(const GatherRowsRequest& request) const override {
        nn_reference_gather_rows(request);
    }
    void scatter_add_rows(
        const ScatterAddRowsRequest& request) const override {
        nn_reference_scatter_add_rows(request);
    }
    void layer_norm_forward(
        const LayerNormForwardRequest& request) const override {
        nn_reference_layer_norm_forward(request);
    }
    void layer_norm_backward(
        const LayerNormBackwardRequest& request) const override {
        nn_reference_layer_norm_backward(request);
    }
    void cross_entropy_forward(
        const CrossEntropyForwardRequest& request) const override {
        nn_reference_cross_entropy_forward(request);
    }
    void materialized_causal_attention_forward(
        const MaterializedCausalAttentionForwardRequest& request)
        const override {
        reference_materialized_causal_attention_forward(request);
    }
    void materialized_causal_attention_context_backward(
        const MaterializedCausalAttentionContextBackwardRequest& request)
        const override {
        reference_materialized_causal_attention_context_backward(request);
    }
    void materialized_causal_attention_probabilities_backward(
        const MaterializedCausalAttentionProbabilitiesBackwardRequest&
            request) const override {
        reference_materialized_causal_attention_probabilities_backward(
            request);
    }
    void flash_causal_attention_forward(
        const FlashCausalAttentionForwardRequest& request) const override {
        reference_flash_causal_attention_forward(request);
    }
    void flash_causal_attention_backward(
        const FlashCausalAttentionBackwardRequest& request) const override {
        reference_flash_causal_attention_backward(request);
    }
    void paged_decode_attention_forward(
        const PagedDecodeAttentionForwardRequest& request) const override {
        reference_paged_decode_attention_forward(request);
    }
    void adam_update(const AdamUpdateRequest& request) const override {
        adam_reference_update(request);
    }
#endif
};

}  // namespace

const BackendAdapter& hip_backend_adapter() noexcept {
    static const HipBackendAdapter adapter;
    return adapter;
}

HipForwardMergeStatistics hip_forward_merge_statistics() noexcept {
    return PendingForwards::instance().statistics();
}

void hip_quantized_linear_forward_group(
    std::span<const QuantizedLinearForwardRequest> requests
) {
    constexpr std::string_view operation = "quantized-linear forward group";
    if (requests.empty()) {
        throw std::invalid_argument(
            "a quantized-linear group needs at least one request");
    }
    const HipRuntime& runtime = require_runtime();
    launch_pending_forwards();
    const QuantizedLinearForwardRequest& first = requests.front();
    const auto& input = require_hip_tensor(first.input, operation);
    const auto& first_weight = require_hip_weight(first.weight, operation);
    std::vector<rthip_nf4_member> members;
    members.reserve(requests.size());
    for (const QuantizedLinearForwardRequest& request : requests) {
        const auto& weight = require_hip_weight(request.weight, operation);
        if (&request.input != &first.input ||
            request.dimensions.rows != first.dimensions.rows ||
            request.dimensions.input_width != first.dimensions.input_width ||
            request.dimensions.block_size != first.dimensions.block_size ||
            weight.encoding() != first_weight.encoding() ||
            weight.second_level_block_size() !=
                first_weight.second_level_block_size()) {
            throw std::invalid_argument(
                "the requests of a quantized-linear group must share their "
                "input, row count, input width, block size and scale "
                "encoding");
        }
    }
    const float* source = input.device_for_read();
    for (const QuantizedLinearForwardRequest& request : requests) {
        const auto& weight = require_hip_weight(request.weight, operation);
        auto& output = require_hip_tensor(request.output, operation);
        rthip_nf4_member member{};
        member.codes = static_cast<const std::uint8_t*>(
            weight.packed_codes_native_handle());
        member.primary_scales = weight.primary_scales_native_handle();
        member.secondary_scales = static_cast<const float*>(
            weight.secondary_scales_native_handle());
        member.offset = weight.offset();
        member.bias_or_null = nullptr;
        member.y = output.device_for_overwrite();
        member.output_width = request.dimensions.output_width;
        members.push_back(member);
    }
    check(runtime,
          runtime.nf4_linear_forward_group(
              source, members.data(), members.size(),
              static_cast<int32_t>(first_weight.encoding()),
              first_weight.second_level_block_size(), first.dimensions.rows,
              first.dimensions.input_width, first.dimensions.block_size,
              nullptr),
          operation);
    finish_operation(runtime,
                     "quantized-linear forward group synchronisation");
}

namespace {

void require_elements(const TensorStorage& storage, std::size_t rows,
                      std::size_t columns, std::string_view what) {
    if (columns != 0 && rows > SIZE_MAX / columns) {
        throw std::overflow_error("quantized-linear adapter dimensions "
                                  "overflow");
    }
    if (storage.size() != rows * columns) {
        throw std::invalid_argument(
            "quantized-linear adapter " + std::string(what) +
            " does not match the dimensions");
    }
}

// The adapter's own rules (LowRankAdapter's constructor,
// src/nn/low_rank_adapter.cpp:27-62) on what a request carries.
void require_adapter(std::size_t rank, float scale,
                     const QuantizedLinearDimensions& dimensions) {
    if (dimensions.rows == 0 || dimensions.input_width == 0 ||
        dimensions.output_width == 0) {
        throw std::invalid_argument(
            "quantized linear dimensions must be greater than zero");
    }
    if (rank == 0 ||
        rank > std::min(dimensions.input_width, dimensions.output_width)) {
        throw std::invalid_argument(
            "LoRA rank must be in [1, min(input_width, output_width)]");
    }
    if (!std::isfinite(scale) || scale <= 0.0F) {
        throw std::invalid_argument(
            "LoRA alpha divided by rank must be finite and positive");
    }
}

}  // namespace

void hip_quantized_linear_adapter_forward(
    const QuantizedLinearAdapterForwardRequest& request
) {
    constexpr std::string_view operation = "quantized-linear adapter forward";
    const QuantizedLinearDimensions& d = request.dimensions;
    require_adapter(request.rank, request.scale, d);
    require_elements(request.input, d.rows, d.input_width, "input");
    require_elements(request.output, d.rows, d.output_width, "output");
    require_elements(request.lora_a, request.rank, d.input_width, "A matrix");
    require_elements(request.lora_b, d.output_width, request.rank,
                     "B matrix");
    require_elements(request.reduced, d.rows, request.rank, "reduced buffer");
    if (request.bias != nullptr) {
        require_elements(*request.bias, 1, d.output_width, "bias");
    }
    const HipRuntime& runtime = require_runtime();
    const auto& input = require_hip_tensor(request.input, operation);
    const auto& weight = require_hip_weight(request.weight, operation);
    const auto& lora_a = require_hip_tensor(request.lora_a, operation);
    const auto& lora_b = require_hip_tensor(request.lora_b, operation);
    auto& reduced = require_hip_tensor(request.reduced, operation);
    auto& output = require_hip_tensor(request.output, operation);
    const float* bias = nullptr;
    if (request.bias != nullptr) {
        bias = require_hip_tensor(*request.bias, operation).device_for_read();
    }
    if (merge_requested() && d.rows <= PendingForwards::kMaximumRows) {
        // The layer joins the forwards that are held back for its input (the
        // query and value projections of a decoder carry adapters, the key
        // projection between them does not): the launch of the list takes
        // the members' x.A^T together, then the packed products with bias
        // and adapter terms.
        const float* source = input.device_for_read();
        rthip_nf4_lora_member member{};
        member.base.codes = static_cast<const std::uint8_t*>(
            weight.packed_codes_native_handle());
        member.base.primary_scales = weight.primary_scales_native_handle();
        member.base.secondary_scales = static_cast<const float*>(
            weight.secondary_scales_native_handle());
        member.base.offset = weight.offset();
        member.base.bias_or_null = bias;
        member.base.y = output.device_for_overwrite();
        member.base.output_width = d.output_width;
        member.lora_a = lora_a.device_for_read();
        member.lora_b = lora_b.device_for_read();
        member.reduced = reduced.device_for_overwrite();
        member.lora_rank = request.rank;
        member.lora_scale = request.scale;
        PendingForwards::instance().add(
            {source, static_cast<std::int32_t>(weight.encoding()),
             weight.second_level_block_size(), d.rows, d.input_width,
             d.block_size},
            member);
        return;
    }
    launch_pending_forwards();
    check(runtime,
          runtime.nf4_lora_linear_forward(
              input.device_for_read(),
              static_cast<const std::uint8_t*>(
                  weight.packed_codes_native_handle()),
              weight.primary_scales_native_handle(),
              static_cast<const float*>(
                  weight.secondary_scales_native_handle()),
              static_cast<int32_t>(weight.encoding()),
              weight.second_level_block_size(), weight.offset(), bias,
              lora_a.device_for_read(), lora_b.device_for_read(),
              request.rank, request.scale, reduced.device_for_overwrite(),
              output.device_for_overwrite(), d.rows, d.input_width,
              d.output_width, d.block_size, nullptr),
          operation);
    finish_operation(runtime,
                     "quantized-linear adapter forward synchronisation");
}

void hip_quantized_linear_adapter_backward(
    const QuantizedLinearAdapterBackwardRequest& request
) {
    constexpr std::string_view operation =
        "quantized-linear adapter backward";
    const QuantizedLinearDimensions& d = request.dimensions;
    require_adapter(request.rank, request.scale, d);
    require_elements(request.upstream, d.rows, d.output_width, "upstream");
    require_elements(request.input, d.rows, d.input_width, "input");
    require_elements(request.reduced, d.rows, request.rank, "reduced buffer");
    require_elements(request.lora_a, request.rank, d.input_width, "A matrix");
    require_elements(request.lora_b, d.output_width, request.rank,
                     "B matrix");
    require_elements(request.input_gradient, d.rows, d.input_width,
                     "input gradient");
    require_elements(request.lora_a_gradient, request.rank, d.input_width,
                     "A gradient");
    require_elements(request.lora_b_gradient, d.output_width, request.rank,
                     "B gradient");
    const HipRuntime& runtime = require_runtime();
    launch_pending_forwards();
    const auto& upstream = require_hip_tensor(request.upstream, operation);
    const auto& input = require_hip_tensor(request.input, operation);
    const auto& reduced = require_hip_tensor(request.reduced, operation);
    const auto& weight = require_hip_weight(request.weight, operation);
    const auto& lora_a = require_hip_tensor(request.lora_a, operation);
    const auto& lora_b = require_hip_tensor(request.lora_b, operation);
    auto& input_gradient =
        require_hip_tensor(request.input_gradient, operation);
    auto& a_gradient = require_hip_tensor(request.lora_a_gradient, operation);
    auto& b_gradient = require_hip_tensor(request.lora_b_gradient, operation);
    // (upstream * scale) . B, [rows, rank]: lives for this call only
    const DeviceBuffer reduced_gradient(
        d.rows * request.rank * sizeof(float), DeviceBuffer::Kind::Pooled);
    const float* dy = upstream.device_for_read();
    check(runtime,
          runtime.lora_backward(
              dy, input.device_for_read(), reduced.device_for_read(),
              lora_b.device_for_read(), request.rank, request.scale,
              static_cast<float*>(reduced_gradient.get()),
              a_gradient.device_for_overwrite(),
              b_gradient.device_for_overwrite(), d.rows, d.input_width,
              d.output_width, nullptr),
          operation);
    check(runtime,
          runtime.nf4_lora_linear_input_backward(
              dy,
              static_cast<const std::uint8_t*>(
                  weight.packed_codes_native_handle()),
              weight.primary_scales_native_handle(),
              static_cast<const float*>(
                  weight.secondary_scales_native_handle()),
              static_cast<int32_t>(weight.encoding()),
              weight.second_level_block_size(), weight.offset(),
              lora_a.device_for_read(),
              static_cast<const float*>(reduced_gradient.get()), request.rank,
              input_gradient.device_for_overwrite(), d.rows, d.input_width,
              d.output_width, d.block_size, nullptr),
          operation);
    // The temporary goes back to the pool when this function returns; the
    // kernels that read it are queued on the same (null) stream as whatever
    // uses the memory next, so that is ordered on the device.
    finish_operation(runtime,
                     "quantized-linear adapter backward synchronisation");
}

std::vector<HipPackedWeight> hip_load_packed_model_state(
    std::span<const std::uint8_t> state
) {
    const std::vector<PackedWeightView> entries =
        parse_packed_model_state(state);
    const HipRuntime& runtime = require_runtime();
    std::vector<HipPackedWeight> result;
    result.reserve(entries.size());
    for (const PackedWeightView& entry : entries) {
        const std::size_t element_count = require_payload_lengths(entry);
        auto storage = std::make_unique<HipNf4WeightStorage>(
            entry, runtime.host_visible_memory);
        const rthip_status status = runtime.nf4_check_payload(
            static_cast<const std::uint8_t*>(
                storage->packed_codes_native_handle()),
            storage->primary_scales_native_handle(),
            static_cast<const float*>(
                storage->secondary_scales_native_handle()),
            static_cast<std::int32_t>(storage->encoding()),
            storage->second_level_block_size(), storage->offset(),
            element_count, entry.block_size, nullptr);
        if (status == RTHIP_INVALID_ARGUMENT) {
            // the reference's own message, as from_packed_nf4 throws it
            throw std::invalid_argument(runtime.last_error());
        }
        check(runtime, status, "packed payload check");
        // The content rules include every rule the dispatcher re-checks
        // before each launch.
        storage->mark_scales_validated();
        result.push_back({entry.shape, entry.block_size, std::move(storage)});
    }
    return result;
}

std::vector<std::uint8_t> hip_packed_model_state_bytes(
    std::span<const HipPackedWeightSource> weights
) {
    const HipRuntime& runtime = require_runtime();
    // One allocation of the final size: the headers are appended in place
    // and nothing written so far is ever moved.
    std::size_t total = 16;
    for (const HipPackedWeightSource& source : weights) {
        if (source.storage != nullptr) {
            total += 64 + 8 * source.shape.size() +
                     source.storage->packed_codes().size() +
                     nf4_scale_payload_bytes(source.storage->scale_storage());
        }
    }
    std::vector<std::uint8_t> output;
    output.reserve(total);
    append_packed_state_prologue(output, weights.size());
    struct Pending {
        const HipNf4WeightStorage* storage;
        PackedWeightLayout layout;
    };
    std::vector<Pending> pending;
    pending.reserve(weights.size());
    for (const HipPackedWeightSource& source : weights) {
        if (source.storage == nullptr) {
            throw std::invalid_argument(
                "packed model state needs hip quantized-weight storage");
        }
        const HipNf4WeightStorage& storage =
            require_hip_weight(*source.storage, "packed model state");
        const bool nested =
            storage.encoding() == Nf4ScaleEncoding::DoubleQuantizedUInt8;
        pending.push_back(
            {&storage,
             append_packed_weight_header(
                 output, source.shape, source.block_size,
                 storage.packed_code_count(), storage.fp32_scale_count(),
                 nested, storage.scale_code_count(),
                 storage.second_level_scale_count(),
                 storage.second_level_block_size(), storage.offset())});
    }
    // The vector no longer grows: copy every array from HBM to its place.
    const auto fetch = [&](std::size_t offset, const void* device,
                           std::size_t bytes) {
        if (bytes != 0) {
            check(runtime,
                  runtime.copy_to_host(output.data() + offset, device, bytes),
                  "packed payload read-back");
        }
    };
    for (const Pending& item : pending) {
        const HipNf4WeightStorage& storage = *item.storage;
        fetch(item.layout.packed_codes, storage.packed_codes_native_handle(),
              storage.packed_code_count());
        fetch(item.layout.block_scales, storage.fp32_scales_device(),
              storage.fp32_scale_count() * sizeof(float));
        fetch(item.layout.scale_codes, storage.scale_codes_device(),
              storage.scale_code_count());
        fetch(item.layout.second_level_scales,
              storage.second_level_scales_device(),
              storage.second_level_scale_count() * sizeof(float));
    }
    return output;
}

}  // namespace riftco_transformer::backend_detail
