// tatara::backend::hip — C++ host view of the gfx950 backend, shaped like the
// reference's tatara::backend::metal (include/tatara/backend/metal/
// {resources,pipeline,commands}.h): move-only RAII handles, free functions,
// `{error enum, optional<Handle>}` results with explicit operator bool, no
// exceptions.  Everything is a thin inline layer over the C ABI of
// include/tatara_hip.h; a default-constructed handle is the invalid ("null")
// object the contract tests pass to check that validation precedes any device
// call.
//
// Differences from the Metal interface, all forced by discrete HBM:
//   * create_shared_buffer allocates HBM; HipBuffer::contents() is a pinned host
//     staging view.  did_modify_range() publishes host writes, and
//     synchronize_buffer() fetches results (Metal's managed-storage idiom).
//   * kernels come from the library linked into the backend, so
//     create_kernel_library(device) replaces create_library_with_source, and
//     create_compute_pipeline(library, name) folds create_function into it.
#pragma once

#include <array>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <optional>
#include <string>
#include <string_view>
#include <utility>

#include "tatara_hip.h"

namespace tatara::backend::hip {

inline constexpr std::uint32_t kMaxBufferArgumentIndex = TT_MAX_BUFFER_ARGUMENT_INDEX;
inline constexpr std::uint32_t kMaxInlineConstantBytes = TT_MAX_INLINE_CONSTANT_BYTES;
inline constexpr std::size_t kExecutionDiagnosticStorageBytes = TT_DIAGNOSTIC_STORAGE_BYTES;

// MetalCommandError (commands.h:232-262); values are the C ABI's status codes.
enum class HipCommandError : std::uint8_t {
    None = TT_OK,
    InvalidCommandQueue = TT_CMD_INVALID_COMMAND_QUEUE,
    InvalidCommandBuffer = TT_CMD_INVALID_COMMAND_BUFFER,
    InvalidEvent = TT_CMD_INVALID_EVENT,
    InvalidEventValue = TT_CMD_INVALID_EVENT_VALUE,
    InvalidComputePass = TT_CMD_INVALID_COMPUTE_PASS,
    InvalidBlitPass = TT_CMD_INVALID_BLIT_PASS,
    InvalidPipeline = TT_CMD_INVALID_PIPELINE,
    InvalidBuffer = TT_CMD_INVALID_BUFFER,
    InvalidBufferIndex = TT_CMD_INVALID_BUFFER_INDEX,
    InvalidBufferOffset = TT_CMD_INVALID_BUFFER_OFFSET,
    InvalidSourceRange = TT_CMD_INVALID_SOURCE_RANGE,
    InvalidDestinationRange = TT_CMD_INVALID_DESTINATION_RANGE,
    InvalidCopyExtent = TT_CMD_INVALID_COPY_EXTENT,
    InvalidFillExtent = TT_CMD_INVALID_FILL_EXTENT,
    InvalidDispatchExtent = TT_CMD_INVALID_DISPATCH_EXTENT,
    ContextOutOfRange = TT_CMD_CONTEXT_OUT_OF_RANGE,
    StateSlotMismatch = TT_CMD_STATE_SLOT_MISMATCH,
    InvalidPendingExecution = TT_CMD_INVALID_PENDING_EXECUTION,
    CommandBufferCreationFailed = TT_CMD_COMMAND_BUFFER_CREATION_FAILED,
    EncoderCreationFailed = TT_CMD_ENCODER_CREATION_FAILED,
    InvalidDevice = TT_CMD_INVALID_DEVICE,
    InvalidStreamGroup = TT_CMD_INVALID_STREAM_GROUP,
};

// MetalResourceError (resources.h:174-184).
enum class HipResourceError : std::uint8_t {
    None = 0,
    InvalidDevice = TT_RES_INVALID_DEVICE,
    SystemDeviceUnavailable = TT_RES_SYSTEM_DEVICE_UNAVAILABLE,
    CommandQueueCreationFailed = TT_RES_COMMAND_QUEUE_CREATION_FAILED,
    EventCreationFailed = TT_RES_EVENT_CREATION_FAILED,
    InvalidBufferSize = TT_RES_INVALID_BUFFER_SIZE,
    BufferCreationFailed = TT_RES_BUFFER_CREATION_FAILED,
    OwnershipFailure = TT_RES_OWNERSHIP_FAILURE,
    BufferWindowUnsupported = TT_RES_BUFFER_WINDOW_UNSUPPORTED,
};

// MetalPipelineError (pipeline.h:99-110).
enum class HipPipelineError : std::uint8_t {
    None = 0,
    InvalidDevice = TT_PIPE_INVALID_DEVICE,
    InvalidLibrary = TT_PIPE_INVALID_LIBRARY,
    InvalidFunctionName = TT_PIPE_INVALID_FUNCTION_NAME,
    LibraryCompilationFailed = TT_PIPE_LIBRARY_COMPILATION_FAILED,
    FunctionLookupFailed = TT_PIPE_FUNCTION_LOOKUP_FAILED,
    PipelineCreationFailed = TT_PIPE_PIPELINE_CREATION_FAILED,
};

// MetalExecutionFailure (commands.h:281-295).
enum class HipExecutionFailure : std::uint8_t {
    None = TT_FAILURE_NONE,
    Internal = TT_FAILURE_INTERNAL,
    Timeout = TT_FAILURE_TIMEOUT,
    PageFault = TT_FAILURE_PAGE_FAULT,
    OutOfMemory = TT_FAILURE_OUT_OF_MEMORY,
    InvalidResource = TT_FAILURE_INVALID_RESOURCE,
    DeviceRemoved = TT_FAILURE_DEVICE_REMOVED,
    UnknownError = TT_FAILURE_UNKNOWN_ERROR,
};

struct HipSize {
    std::uint64_t width;
    std::uint64_t height;
    std::uint64_t depth;
};

namespace detail {
// Owns one C-ABI handle; Destroy releases it.
template <typename T, void (*Destroy)(T*)> class Handle {
  public:
    Handle() noexcept = default;
    explicit Handle(T* raw) noexcept : raw_(raw) {}
    ~Handle() { reset(); }
    Handle(const Handle&) = delete;
    Handle& operator=(const Handle&) = delete;
    Handle(Handle&& other) noexcept : raw_(std::exchange(other.raw_, nullptr)) {}
    Handle& operator=(Handle&& other) noexcept {
        if (this != &other) {
            reset();
            raw_ = std::exchange(other.raw_, nullptr);
        }
        return *this;
    }
    T* get() const noexcept { return raw_; }
    T* release() noexcept { return std::exchange(raw_, nullptr); }
    void reset() noexcept {
        if (raw_ != nullptr) Destroy(raw_);
        raw_ = nullptr;
    }
    explicit operator bool() const noexcept { return raw_ != nullptr; }

  private:
    T* raw_ = nullptr;
};
}  // namespace detail

class HipDevice {
  public:
    HipDevice() noexcept = default;
    const std::string& name() const noexcept { return name_; }
    std::uint32_t compute_units() const noexcept { return tt_device_compute_units(h_.get()); }
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_device* native() const noexcept { return h_.get(); }

  private:
    friend struct HipDeviceResult create_system_device();
    detail::Handle<tt_device, tt_device_destroy> h_;
    std::string name_;
};

class HipCommandQueue {
  public:
    HipCommandQueue() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_queue* native() const noexcept { return h_.get(); }

  private:
    friend struct HipCommandQueueResult create_command_queue(const HipDevice&);
    detail::Handle<tt_queue, tt_queue_destroy> h_;
};

// create_event (resources.h:95-118, 240): a counter that command buffers of any queue of
// the device signal and wait for.
class HipEvent {
  public:
    HipEvent() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_event* native() const noexcept { return h_.get(); }

  private:
    friend struct HipEventResult create_event(const HipDevice&);
    detail::Handle<tt_event, tt_event_destroy> h_;
};

class HipBuffer {
  public:
    HipBuffer() noexcept = default;
    std::uint64_t size_bytes() const noexcept { return tt_buffer_size(h_.get()); }
    // Pinned host staging view (see the header comment); nullptr for a null buffer.
    void* contents() const noexcept { return tt_buffer_contents(h_.get()); }
    void* device_pointer() const noexcept { return tt_buffer_device_pointer(h_.get()); }
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_buffer* native() const noexcept { return h_.get(); }

  private:
    friend struct HipBufferResult create_shared_buffer(const HipDevice&, std::uint64_t);
    friend struct HipPooledBufferResult create_striped_pool_buffer(const HipDevice&, std::uint64_t,
                                                                   std::uint32_t);
    friend struct HipBufferResult create_buffer_window(const HipBuffer&, std::uint64_t,
                                                       std::uint64_t);
    friend struct HipBufferResult wrap_device_memory(const HipDevice&, void*, std::uint64_t);
    detail::Handle<tt_buffer, tt_buffer_destroy> h_;
};

class HipLibrary {
  public:
    HipLibrary() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_library* native() const noexcept { return h_.get(); }

  private:
    friend struct HipLibraryResult create_kernel_library(const HipDevice&);
    detail::Handle<tt_library, tt_library_destroy> h_;
};

class HipComputePipeline {
  public:
    HipComputePipeline() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_pipeline* native() const noexcept { return h_.get(); }

  private:
    friend struct HipComputePipelineResult create_compute_pipeline(const HipLibrary&,
                                                                   std::string_view);
    detail::Handle<tt_pipeline, tt_pipeline_destroy> h_;
};

// One native command buffer travels through these four states; each state is a
// distinct move-only type so the encode order of the reference is enforced by
// the type system (create -> begin pass -> end pass -> commit -> wait).
class HipCommandBuffer {
  public:
    HipCommandBuffer() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_command_buffer* native() const noexcept { return h_.get(); }

  private:
    friend struct HipCommandBufferResult create_command_buffer(const HipCommandQueue&);
    friend struct HipComputePassResult begin_compute_pass(HipCommandBuffer&&);
    friend struct HipBlitPassResult begin_blit_pass(HipCommandBuffer&&);
    friend struct HipCommandBufferResult end_compute_pass(class HipComputePass&&);
    friend struct HipCommandBufferResult end_blit_pass(class HipBlitPass&&);
    friend struct HipPendingExecutionResult commit(HipCommandBuffer&&);
    detail::Handle<tt_command_buffer, tt_command_buffer_destroy> h_;
};

class HipComputePass {
  public:
    HipComputePass() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_command_buffer* native() const noexcept { return h_.get(); }

  private:
    friend struct HipComputePassResult begin_compute_pass(HipCommandBuffer&&);
    friend struct HipCommandBufferResult end_compute_pass(HipComputePass&&);
    detail::Handle<tt_command_buffer, tt_command_buffer_destroy> h_;
};

class HipBlitPass {
  public:
    HipBlitPass() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }
    tt_command_buffer* native() const noexcept { return h_.get(); }

  private:
    friend struct HipBlitPassResult begin_blit_pass(HipCommandBuffer&&);
    friend struct HipCommandBufferResult end_blit_pass(HipBlitPass&&);
    detail::Handle<tt_command_buffer, tt_command_buffer_destroy> h_;
};

class HipPendingExecution {
  public:
    HipPendingExecution() noexcept = default;
    explicit operator bool() const noexcept { return static_cast<bool>(h_); }

  private:
    friend struct HipPendingExecutionResult commit(HipCommandBuffer&&);
    friend struct HipExecutionResult wait_until_completed(HipPendingExecution&&);
    detail::Handle<tt_command_buffer, tt_command_buffer_destroy> h_;
};

struct HipDeviceResult {
    HipResourceError error;
    std::optional<HipDevice> device;
    explicit operator bool() const noexcept {
        return error == HipResourceError::None && device.has_value();
    }
};
struct HipCommandQueueResult {
    HipResourceError error;
    std::optional<HipCommandQueue> command_queue;
    explicit operator bool() const noexcept {
        return error == HipResourceError::None && command_queue.has_value();
    }
};
struct HipEventResult {
    HipResourceError error;
    std::optional<HipEvent> event;
    explicit operator bool() const noexcept {
        return error == HipResourceError::None && event.has_value();
    }
};
struct HipBufferResult {
    HipResourceError error;
    std::optional<HipBuffer> buffer;
    explicit operator bool() const noexcept {
        return error == HipResourceError::None && buffer.has_value();
    }
};
struct HipPooledBufferResult {
    HipResourceError error;
    std::optional<HipBuffer> buffer;
    std::uint64_t stripe_stride_bytes;
    explicit operator bool() const noexcept {
        return error == HipResourceError::None && buffer.has_value();
    }
};
struct HipLibraryResult {
    HipPipelineError error;
    std::optional<HipLibrary> library;
    explicit operator bool() const noexcept {
        return error == HipPipelineError::None && library.has_value();
    }
};
struct HipComputePipelineResult {
    HipPipelineError error;
    std::optional<HipComputePipeline> pipeline;
    explicit operator bool() const noexcept {
        return error == HipPipelineError::None && pipeline.has_value();
    }
};
struct HipCommandBufferResult {
    HipCommandError error;
    std::optional<HipCommandBuffer> command_buffer;
    explicit operator bool() const noexcept {
        return error == HipCommandError::None && command_buffer.has_value();
    }
};
struct HipComputePassResult {
    HipCommandError error;
    std::optional<HipComputePass> compute_pass;
    explicit operator bool() const noexcept {
        return error == HipCommandError::None && compute_pass.has_value();
    }
};
struct HipBlitPassResult {
    HipCommandError error;
    std::optional<HipBlitPass> blit_pass;
    explicit operator bool() const noexcept {
        return error == HipCommandError::None && blit_pass.has_value();
    }
};
struct HipPendingExecutionResult {
    HipCommandError error;
    std::optional<HipPendingExecution> pending_execution;
    explicit operator bool() const noexcept {
        return error == HipCommandError::None && pending_execution.has_value();
    }
};

// MetalExecutionResult + MetalExecutionTiming (commands.h:374-416).
struct HipExecutionResult {
    HipCommandError error;
    bool completed;
    HipExecutionFailure failure;
    std::int64_t native_error_code;
    bool has_native_error_code;
    double gpu_milliseconds;
    std::array<char, kExecutionDiagnosticStorageBytes> failure_description{};
    explicit operator bool() const noexcept {
        return error == HipCommandError::None && completed &&
               failure == HipExecutionFailure::None;
    }
};

// ---- resources ----
inline HipDeviceResult create_system_device() {
    tt_device* raw = nullptr;
    const std::int32_t status = tt_device_create(&raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipDevice device;
    device.h_ = detail::Handle<tt_device, tt_device_destroy>(raw);
    device.name_ = tt_device_name(raw);
    return {HipResourceError::None, std::move(device)};
}

inline HipCommandQueueResult create_command_queue(const HipDevice& device) {
    if (!device) return {HipResourceError::InvalidDevice, std::nullopt};
    tt_queue* raw = nullptr;
    const std::int32_t status = tt_queue_create(device.native(), &raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipCommandQueue queue;
    queue.h_ = detail::Handle<tt_queue, tt_queue_destroy>(raw);
    return {HipResourceError::None, std::move(queue)};
}

inline HipBufferResult create_shared_buffer(const HipDevice& device, std::uint64_t size_bytes) {
    if (!device) return {HipResourceError::InvalidDevice, std::nullopt};
    tt_buffer* raw = nullptr;
    const std::int32_t status = tt_buffer_create(device.native(), size_bytes, &raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipBuffer buffer;
    buffer.h_ = detail::Handle<tt_buffer, tt_buffer_destroy>(raw);
    return {HipResourceError::None, std::move(buffer)};
}

inline HipPooledBufferResult create_striped_pool_buffer(const HipDevice& device,
                                                        std::uint64_t stripe_bytes,
                                                        std::uint32_t stripe_count) {
    if (!device) return {HipResourceError::InvalidDevice, std::nullopt, 0};
    tt_buffer* raw = nullptr;
    std::uint64_t stride = 0;
    const std::int32_t status =
        tt_pool_create(device.native(), stripe_bytes, stripe_count, &raw, &stride);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt, 0};
    HipBuffer buffer;
    buffer.h_ = detail::Handle<tt_buffer, tt_buffer_destroy>(raw);
    return {HipResourceError::None, std::move(buffer), stride};
}

inline HipBufferResult create_buffer_window(const HipBuffer& buffer, std::uint64_t offset,
                                            std::uint64_t length) {
    if (!buffer) return {HipResourceError::BufferWindowUnsupported, std::nullopt};
    tt_buffer* raw = nullptr;
    const std::int32_t status = tt_buffer_window(buffer.native(), offset, length, &raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipBuffer window;
    window.h_ = detail::Handle<tt_buffer, tt_buffer_destroy>(raw);
    return {HipResourceError::None, std::move(window)};
}

// Adopts device memory owned elsewhere (no reference counterpart).
inline HipBufferResult wrap_device_memory(const HipDevice& device, void* pointer,
                                          std::uint64_t size_bytes) {
    if (!device) return {HipResourceError::InvalidDevice, std::nullopt};
    tt_buffer* raw = nullptr;
    const std::int32_t status = tt_buffer_wrap(device.native(), pointer, size_bytes, &raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipBuffer buffer;
    buffer.h_ = detail::Handle<tt_buffer, tt_buffer_destroy>(raw);
    return {HipResourceError::None, std::move(buffer)};
}

inline HipCommandError did_modify_range(const HipBuffer& buffer, std::uint64_t offset,
                                        std::uint64_t length) {
    if (!buffer) return HipCommandError::InvalidBuffer;
    return static_cast<HipCommandError>(tt_buffer_did_modify(buffer.native(), offset, length));
}
inline HipCommandError synchronize_buffer(const HipBuffer& buffer, std::uint64_t offset,
                                          std::uint64_t length) {
    if (!buffer) return HipCommandError::InvalidBuffer;
    return static_cast<HipCommandError>(tt_buffer_synchronize(buffer.native(), offset, length));
}

// ---- pipelines ----
inline HipLibraryResult create_kernel_library(const HipDevice& device) {
    if (!device) return {HipPipelineError::InvalidDevice, std::nullopt};
    tt_library* raw = nullptr;
    const std::int32_t status = tt_library_create(device.native(), &raw);
    if (status != TT_OK) return {static_cast<HipPipelineError>(status), std::nullopt};
    HipLibrary library;
    library.h_ = detail::Handle<tt_library, tt_library_destroy>(raw);
    return {HipPipelineError::None, std::move(library)};
}

inline HipComputePipelineResult create_compute_pipeline(const HipLibrary& library,
                                                        std::string_view name) {
    if (!library) return {HipPipelineError::InvalidLibrary, std::nullopt};
    if (name.empty()) return {HipPipelineError::InvalidFunctionName, std::nullopt};
    const std::string owned(name);
    tt_pipeline* raw = nullptr;
    const std::int32_t status = tt_pipeline_create(library.native(), owned.c_str(), &raw);
    if (status != TT_OK) return {static_cast<HipPipelineError>(status), std::nullopt};
    HipComputePipeline pipeline;
    pipeline.h_ = detail::Handle<tt_pipeline, tt_pipeline_destroy>(raw);
    return {HipPipelineError::None, std::move(pipeline)};
}

// ---- commands ----
inline HipCommandBufferResult create_command_buffer(const HipCommandQueue& queue) {
    if (!queue) return {HipCommandError::InvalidCommandQueue, std::nullopt};
    tt_command_buffer* raw = nullptr;
    const std::int32_t status = tt_command_buffer_create(queue.native(), &raw);
    if (status != TT_OK) return {static_cast<HipCommandError>(status), std::nullopt};
    HipCommandBuffer cb;
    cb.h_ = detail::Handle<tt_command_buffer, tt_command_buffer_destroy>(raw);
    return {HipCommandError::None, std::move(cb)};
}

inline HipComputePassResult begin_compute_pass(HipCommandBuffer&& command_buffer) {
    if (!command_buffer) return {HipCommandError::InvalidCommandBuffer, std::nullopt};
    const std::int32_t status = tt_pass_begin(command_buffer.native());
    if (status != TT_OK) return {static_cast<HipCommandError>(status), std::nullopt};
    HipComputePass pass;
    pass.h_ = std::move(command_buffer.h_);
    return {HipCommandError::None, std::move(pass)};
}

inline HipCommandError set_compute_pipeline(HipComputePass& pass,
                                            const HipComputePipeline& pipeline) {
    if (!pass) return HipCommandError::InvalidComputePass;
    if (!pipeline) return HipCommandError::InvalidPipeline;
    return static_cast<HipCommandError>(tt_pass_set_pipeline(pass.native(), pipeline.native()));
}

inline HipCommandError set_buffer(HipComputePass& pass, const HipBuffer& buffer,
                                  std::uint64_t offset_bytes, std::uint32_t index) {
    if (!pass) return HipCommandError::InvalidComputePass;
    if (!buffer) return HipCommandError::InvalidBuffer;
    return static_cast<HipCommandError>(
        tt_pass_set_buffer(pass.native(), buffer.native(), offset_bytes, index));
}

inline HipCommandError set_bytes(HipComputePass& pass, const void* bytes,
                                 std::uint32_t length_bytes, std::uint32_t index) {
    if (!pass) return HipCommandError::InvalidComputePass;
    return static_cast<HipCommandError>(tt_pass_set_bytes(pass.native(), bytes, length_bytes, index));
}

inline HipCommandError dispatch_threadgroups(HipComputePass& pass, HipSize groups,
                                             HipSize threads) {
    if (!pass) return HipCommandError::InvalidComputePass;
    return static_cast<HipCommandError>(tt_pass_dispatch(pass.native(), groups.width, groups.height,
                                                         groups.depth, threads.width,
                                                         threads.height, threads.depth));
}

inline HipCommandError memory_barrier(HipComputePass& pass) {
    if (!pass) return HipCommandError::InvalidComputePass;
    return static_cast<HipCommandError>(tt_pass_barrier(pass.native()));
}

inline HipCommandBufferResult end_compute_pass(HipComputePass&& pass) {
    if (!pass) return {HipCommandError::InvalidComputePass, std::nullopt};
    const std::int32_t status = tt_pass_end(pass.native());
    if (status != TT_OK) return {static_cast<HipCommandError>(status), std::nullopt};
    HipCommandBuffer cb;
    cb.h_ = std::move(pass.h_);
    return {HipCommandError::None, std::move(cb)};
}

inline HipEventResult create_event(const HipDevice& device) {
    if (!device) return {HipResourceError::InvalidDevice, std::nullopt};
    tt_event* raw = nullptr;
    const std::int32_t status = tt_event_create(device.native(), &raw);
    if (status != TT_OK) return {static_cast<HipResourceError>(status), std::nullopt};
    HipEvent event;
    event.h_ = detail::Handle<tt_event, tt_event_destroy>(raw);
    return {HipResourceError::None, std::move(event)};
}

// encode_wait_for_event / encode_signal_event (commands.h:421-426): between passes.  The
// command buffer that signals must be committed before the one that waits for it.
inline HipCommandError encode_wait_for_event(HipCommandBuffer& command_buffer, const HipEvent& event,
                                             std::uint64_t value) {
    if (!command_buffer) return HipCommandError::InvalidCommandBuffer;
    return static_cast<HipCommandError>(
        tt_encode_wait_for_event(command_buffer.native(), event.native(), value));
}
inline HipCommandError encode_signal_event(HipCommandBuffer& command_buffer, const HipEvent& event,
                                           std::uint64_t value) {
    if (!command_buffer) return HipCommandError::InvalidCommandBuffer;
    return static_cast<HipCommandError>(
        tt_encode_signal_event(command_buffer.native(), event.native(), value));
}

inline HipBlitPassResult begin_blit_pass(HipCommandBuffer&& command_buffer) {
    if (!command_buffer) return {HipCommandError::InvalidCommandBuffer, std::nullopt};
    HipBlitPass pass;
    pass.h_ = std::move(command_buffer.h_);
    return {HipCommandError::None, std::move(pass)};
}

inline HipCommandError copy_buffer(HipBlitPass& pass, const HipBuffer& source,
                                   std::uint64_t source_offset, HipBuffer& destination,
                                   std::uint64_t destination_offset, std::uint64_t length) {
    if (!pass) return HipCommandError::InvalidBlitPass;
    if (!source || !destination) return HipCommandError::InvalidBuffer;
    return static_cast<HipCommandError>(tt_blit_copy(pass.native(), source.native(), source_offset,
                                                     destination.native(), destination_offset,
                                                     length));
}

inline HipCommandError fill_buffer(HipBlitPass& pass, HipBuffer& destination,
                                   std::uint64_t destination_offset, std::uint64_t length,
                                   std::byte value) {
    if (!pass) return HipCommandError::InvalidBlitPass;
    if (!destination) return HipCommandError::InvalidBuffer;
    return static_cast<HipCommandError>(tt_blit_fill(pass.native(), destination.native(),
                                                     destination_offset, length,
                                                     static_cast<std::uint8_t>(value)));
}

inline HipCommandBufferResult end_blit_pass(HipBlitPass&& pass) {
    if (!pass) return {HipCommandError::InvalidBlitPass, std::nullopt};
    HipCommandBuffer cb;
    cb.h_ = std::move(pass.h_);
    return {HipCommandError::None, std::move(cb)};
}

inline HipPendingExecutionResult commit(HipCommandBuffer&& command_buffer) {
    if (!command_buffer) return {HipCommandError::InvalidCommandBuffer, std::nullopt};
    const std::int32_t status = tt_commit(command_buffer.native());
    if (status != TT_OK) return {static_cast<HipCommandError>(status), std::nullopt};
    HipPendingExecution pending;
    pending.h_ = std::move(command_buffer.h_);
    return {HipCommandError::None, std::move(pending)};
}

inline HipExecutionResult wait_until_completed(HipPendingExecution&& pending) {
    HipExecutionResult result{};
    if (!pending) {
        result.error = HipCommandError::InvalidPendingExecution;
        return result;
    }
    tt_execution_result raw;
    const std::int32_t status = tt_wait(pending.h_.get(), &raw);
    result.error = static_cast<HipCommandError>(status);
    result.completed = raw.completed != 0;
    result.failure = static_cast<HipExecutionFailure>(raw.failure);
    result.native_error_code = raw.native_error_code;
    result.has_native_error_code = raw.has_native_error_code != 0;
    result.gpu_milliseconds = raw.gpu_ms;
    std::memcpy(result.failure_description.data(), raw.diagnostic, sizeof(raw.diagnostic));
    pending.h_.reset();
    return result;
}

}  // namespace tatara::backend::hip
