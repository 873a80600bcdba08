// C-ABI core: devices, HBM buffers with a pinned staging view, the kernel
// library (reference kernel names -> launchers), command recording, submission
// on an in-order HIP stream and completion reporting.  Mirrors the contract of
// the reference's backend (src/backend/metal/{resources,pipeline,commands}.mm):
// typed status codes, validation before any native call, no exceptions.
#include <atomic>
#include <cstdio>
#include <cstring>
#include <algorithm>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "tt_internal.h"

using tt::Bindings;
using tt::Grid;
using tt::KernelDesc;

struct tt_device {
    int ordinal = 0;
    std::string name;
    uint32_t compute_units = 0;
};

struct tt_queue {
    tt_device* device = nullptr;
    hipStream_t stream = nullptr;
    uint8_t* workspace = nullptr;   // see tt::StreamWorkspace
    uint64_t workspace_bytes = 0;
};

struct tt_buffer {
    tt_device* device = nullptr;
    uint8_t* dptr = nullptr;
    uint64_t size = 0;
    uint8_t* host = nullptr;  // pinned staging view, allocated on first contents()
    bool owns_device = false;
    tt_buffer* parent = nullptr;  // windows keep their parent alive
    uint64_t parent_offset = 0;
    std::atomic<int> refs{1};
};

// A counter command buffers signal and wait for: every signalled value owns a HIP event
// recorded where the signal was committed; a wait takes the smallest value that reaches it.
constexpr size_t kEventValuesKept = 64;

struct tt_event {
    std::mutex mutex;
    std::map<uint64_t, hipEvent_t> reached;
    std::atomic<int> refs{1};
};

struct tt_library {
    tt_device* device = nullptr;
    std::vector<KernelDesc> kernels;
};

struct tt_pipeline {
    KernelDesc desc{};
};

namespace tt {
uint32_t queue_compute_units(const tt_queue* queue) {
    return queue != nullptr && queue->device != nullptr ? queue->device->compute_units : 0;
}

hipStream_t queue_stream(const tt_queue* queue) {
    return queue != nullptr ? queue->stream : nullptr;
}

namespace {
std::mutex g_workspace_mutex;
std::map<hipStream_t, StreamWorkspace> g_workspaces;
}  // namespace

StreamWorkspace stream_workspace(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    const auto found = g_workspaces.find(stream);
    return found == g_workspaces.end() ? StreamWorkspace{} : found->second;
}
}  // namespace tt

namespace {

enum class CommandKind : uint8_t { Dispatch, Copy, Fill, Signal, Wait };

struct Command {
    CommandKind kind;
    const char* name;
    tt::LaunchFn launch;
    Bindings bindings;
    Grid grid;
    uint8_t* a;
    uint8_t* b;
    uint64_t length;
    uint8_t value;
    tt_event* event;        // Signal / Wait
    uint64_t event_value;
};

__global__ void tt_fill_bytes(uint8_t* dst, uint64_t length, uint8_t value) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < length;
         i += stride) {
        dst[i] = value;
    }
}

// Plain device-to-device copy: 16 bytes per thread where both ends allow it.
// Overlapping ranges are the caller's business, as with the reference's blit.
__global__ void tt_copy_bytes(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                              uint64_t length, uint32_t wide) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
    const uint64_t first = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    uint64_t done = 0;
    if (wide != 0u) {
        const uint64_t vectors = length / 16;
        const uint4* s = reinterpret_cast<const uint4*>(src);
        uint4* d = reinterpret_cast<uint4*>(dst);
        for (uint64_t i = first; i < vectors; i += stride) d[i] = s[i];
        done = vectors * 16;
    }
    for (uint64_t i = done + first; i < length; i += stride) dst[i] = src[i];
}

void release_buffer(tt_buffer* buffer) {
    if (buffer == nullptr) return;
    if (buffer->refs.fetch_sub(1) != 1) return;
    if (buffer->parent != nullptr) {
        release_buffer(buffer->parent);
    } else {
        if (buffer->host != nullptr) (void)hipHostFree(buffer->host);
        if (buffer->owns_device && buffer->dptr != nullptr) (void)hipFree(buffer->dptr);
    }
    delete buffer;
}

void release_event(tt_event* event) {
    if (event == nullptr) return;
    if (event->refs.fetch_sub(1) != 1) return;
    for (auto& reached : event->reached) (void)hipEventDestroy(reached.second);
    delete event;
}

int32_t classify(hipError_t error) {
    switch (error) {
    case hipSuccess:
        return TT_FAILURE_NONE;
    case hipErrorOutOfMemory:
        return TT_FAILURE_OUT_OF_MEMORY;
    case hipErrorIllegalAddress:
        return TT_FAILURE_PAGE_FAULT;
    case hipErrorLaunchTimeOut:
        return TT_FAILURE_TIMEOUT;
    case hipErrorInvalidValue:
    case hipErrorInvalidDevicePointer:
    case hipErrorInvalidHandle:
        return TT_FAILURE_INVALID_RESOURCE;
    case hipErrorNoDevice:
    case hipErrorInvalidDevice:
        return TT_FAILURE_DEVICE_REMOVED;
    case hipErrorLaunchFailure:
        return TT_FAILURE_INTERNAL;
    default:
        return TT_FAILURE_UNKNOWN_ERROR;
    }
}

}  // namespace

struct tt_command_buffer {
    tt_queue* queue = nullptr;
    std::vector<Command> commands;
    bool pass_open = false;
    const tt_pipeline* pipeline = nullptr;
    Bindings table{};
    const tt_buffer* bound[tt::kArgSlots] = {};   // the buffer behind each bound slot
    // Every buffer a recorded command names is kept alive until the recording is reset or
    // the command buffer destroyed (after its last submission has completed), as the
    // reference's command buffers retain their resources: a caller may destroy its handle
    // between encode and commit, or before a later replay.
    std::vector<tt_buffer*> retained;
    std::vector<tt_event*> retained_events;
    hipEvent_t begin = nullptr;
    hipEvent_t end = nullptr;
    bool committed = false;
    hipError_t submit_error = hipSuccess;
    hipGraph_t graph = nullptr;          // compiled form of the recording
    hipGraphExec_t graph_exec = nullptr;
    bool profiling = false;              // eager commits bracket every command with events
    std::vector<hipEvent_t> marks;       // marks[i], marks[i+1] bracket command i
    bool marks_valid = false;
};

static void drop_graph(tt_command_buffer* cb);

static void retain(tt_command_buffer* cb, const tt_buffer* buffer) {
    if (buffer == nullptr) return;
    if (!cb->retained.empty() && cb->retained.back() == buffer) return;   // same as the last one
    tt_buffer* held = const_cast<tt_buffer*>(buffer);
    held->refs.fetch_add(1);
    cb->retained.push_back(held);
}
static void release_retained(tt_command_buffer* cb) {
    for (tt_buffer* buffer : cb->retained) release_buffer(buffer);
    cb->retained.clear();
    for (tt_event* event : cb->retained_events) release_event(event);
    cb->retained_events.clear();
}

extern "C" {

uint32_t tt_abi_version(void) { return TT_ABI_VERSION; }

uint32_t tt_split_workgroups(const uint32_t* visible_keys, uint32_t rows, uint32_t split_keys) {
    if (visible_keys == nullptr || split_keys == 0) return 0;
    uint64_t groups = 0;
    for (uint32_t r = 0; r < rows; ++r) {
        groups += 2 * ((static_cast<uint64_t>(visible_keys[r]) + split_keys - 1) / split_keys);
    }
    return static_cast<uint32_t>(groups < UINT32_MAX ? groups : UINT32_MAX);
}

uint32_t tt_choose_split_keys(const uint32_t* visible_keys, uint32_t rows, uint32_t compute_units) {
    const uint64_t units = compute_units == 0 ? 1 : compute_units;
    uint64_t total = 0;
    for (uint32_t r = 0; visible_keys != nullptr && r < rows; ++r) total += visible_keys[r];
    // an even share of all keys, then coarser until the last, partly filled split of every
    // row fits too: one workgroup more than compute units costs a third of the walk
    uint64_t split = ((2 * total + units - 1) / units + 31) / 32 * 32;
    if (split < 128) split = 128;
    while (split < UINT32_MAX - 31 && 2 * static_cast<uint64_t>(rows) <= units &&
           tt_split_workgroups(visible_keys, rows, static_cast<uint32_t>(split)) > units) {
        split += 32;
    }
    return static_cast<uint32_t>(split);
}

uint32_t tt_flash_prefill_splits(uint32_t rows, uint32_t visible_keys, uint32_t compute_units) {
    return tt::flash_prefill_splits(rows, visible_keys, compute_units);
}

uint64_t tt_flash_prefill_scratch_bytes(uint32_t rows, uint32_t splits) {
    return tt::flash_prefill_scratch_bytes(rows, splits);
}

const char* tt_status_name(int32_t status) {
    switch (status) {
    case TT_OK: return "None";
    case TT_CMD_INVALID_COMMAND_QUEUE: return "InvalidCommandQueue";
    case TT_CMD_INVALID_COMMAND_BUFFER: return "InvalidCommandBuffer";
    case TT_CMD_INVALID_EVENT: return "InvalidEvent";
    case TT_CMD_INVALID_EVENT_VALUE: return "InvalidEventValue";
    case TT_CMD_INVALID_COMPUTE_PASS: return "InvalidComputePass";
    case TT_CMD_INVALID_BLIT_PASS: return "InvalidBlitPass";
    case TT_CMD_INVALID_PIPELINE: return "InvalidPipeline";
    case TT_CMD_INVALID_BUFFER: return "InvalidBuffer";
    case TT_CMD_INVALID_BUFFER_INDEX: return "InvalidBufferIndex";
    case TT_CMD_INVALID_BUFFER_OFFSET: return "InvalidBufferOffset";
    case TT_CMD_INVALID_SOURCE_RANGE: return "InvalidSourceRange";
    case TT_CMD_INVALID_DESTINATION_RANGE: return "InvalidDestinationRange";
    case TT_CMD_INVALID_COPY_EXTENT: return "InvalidCopyExtent";
    case TT_CMD_INVALID_FILL_EXTENT: return "InvalidFillExtent";
    case TT_CMD_INVALID_DISPATCH_EXTENT: return "InvalidDispatchExtent";
    case TT_CMD_CONTEXT_OUT_OF_RANGE: return "ContextOutOfRange";
    case TT_CMD_STATE_SLOT_MISMATCH: return "StateSlotMismatch";
    case TT_CMD_INVALID_PENDING_EXECUTION: return "InvalidPendingExecution";
    case TT_CMD_COMMAND_BUFFER_CREATION_FAILED: return "CommandBufferCreationFailed";
    case TT_CMD_ENCODER_CREATION_FAILED: return "EncoderCreationFailed";
    case TT_CMD_INVALID_DEVICE: return "InvalidDevice";
    case TT_CMD_INVALID_STREAM_GROUP: return "InvalidStreamGroup";
    case TT_CMD_STATIC_SCRATCH_EXCEEDED: return "StaticScratchExceeded";
    case TT_RES_INVALID_DEVICE: return "Resource.InvalidDevice";
    case TT_RES_SYSTEM_DEVICE_UNAVAILABLE: return "Resource.SystemDeviceUnavailable";
    case TT_RES_COMMAND_QUEUE_CREATION_FAILED: return "Resource.CommandQueueCreationFailed";
    case TT_RES_EVENT_CREATION_FAILED: return "Resource.EventCreationFailed";
    case TT_RES_INVALID_BUFFER_SIZE: return "Resource.InvalidBufferSize";
    case TT_RES_BUFFER_CREATION_FAILED: return "Resource.BufferCreationFailed";
    case TT_RES_OWNERSHIP_FAILURE: return "Resource.OwnershipFailure";
    case TT_RES_BUFFER_WINDOW_UNSUPPORTED: return "Resource.BufferWindowUnsupported";
    case TT_PIPE_INVALID_DEVICE: return "Pipeline.InvalidDevice";
    case TT_PIPE_INVALID_LIBRARY: return "Pipeline.InvalidLibrary";
    case TT_PIPE_INVALID_FUNCTION_NAME: return "Pipeline.InvalidFunctionName";
    case TT_PIPE_LIBRARY_COMPILATION_FAILED: return "Pipeline.LibraryCompilationFailed";
    case TT_PIPE_FUNCTION_LOOKUP_FAILED: return "Pipeline.FunctionLookupFailed";
    case TT_PIPE_PIPELINE_CREATION_FAILED: return "Pipeline.PipelineCreationFailed";
    default: return "Unknown";
    }
}

/* ---------------------------------------------------------------- resources */

int32_t tt_device_create(tt_device** out) {
    if (out == nullptr) return TT_RES_INVALID_DEVICE;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return TT_RES_SYSTEM_DEVICE_UNAVAILABLE;
    }
    hipDeviceProp_t properties;
    if (hipSetDevice(0) != hipSuccess || hipGetDeviceProperties(&properties, 0) != hipSuccess) {
        (void)hipGetLastError();
        return TT_RES_SYSTEM_DEVICE_UNAVAILABLE;
    }
    tt_device* device = new (std::nothrow) tt_device;
    if (device == nullptr) return TT_RES_OWNERSHIP_FAILURE;
    device->ordinal = 0;
    device->name = std::string(properties.name) + " (" + properties.gcnArchName + ")";
    device->compute_units = static_cast<uint32_t>(properties.multiProcessorCount);
    *out = device;
    return TT_OK;
}

void tt_device_destroy(tt_device* device) { delete device; }

const char* tt_device_name(const tt_device* device) {
    return device != nullptr ? device->name.c_str() : "";
}

uint32_t tt_device_compute_units(const tt_device* device) {
    return device != nullptr ? device->compute_units : 0;
}

int32_t tt_queue_create(tt_device* device, tt_queue** out) {
    if (out == nullptr) return TT_RES_INVALID_DEVICE;
    *out = nullptr;
    if (device == nullptr) return TT_RES_INVALID_DEVICE;
    hipStream_t stream = nullptr;
    if (hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) != hipSuccess) {
        (void)hipGetLastError();
        return TT_RES_COMMAND_QUEUE_CREATION_FAILED;
    }
    tt_queue* queue = new (std::nothrow) tt_queue;
    if (queue == nullptr) {
        (void)hipStreamDestroy(stream);
        return TT_RES_OWNERSHIP_FAILURE;
    }
    queue->device = device;
    queue->stream = stream;
    // The decode kernels' one-time set-up for this device (kernel attributes, the address
    // of the static scratch): done here so that an entry point that launches directly on
    // the queue never has to do it inside a stream capture.  A failure shows at that call.
    (void)tt::prepare_decode_kernels();
    // The queue's workspace.  Doing without it is not an error: the operators that would
    // use it run as they do on a foreign stream.
    const uint64_t bytes = tt::stream_workspace_bytes(device->compute_units);
    void* workspace = nullptr;
    if (bytes != 0 && hipMalloc(&workspace, bytes) == hipSuccess) {
        queue->workspace = static_cast<uint8_t*>(workspace);
        queue->workspace_bytes = bytes;
        std::lock_guard<std::mutex> lock(tt::g_workspace_mutex);
        tt::g_workspaces[stream] = tt::StreamWorkspace{queue->workspace, bytes, device->compute_units};
    } else {
        (void)hipGetLastError();
    }
    *out = queue;
    return TT_OK;
}

void tt_queue_destroy(tt_queue* queue) {
    if (queue == nullptr) return;
    if (queue->stream != nullptr) {
        (void)hipStreamSynchronize(queue->stream);
        {
            std::lock_guard<std::mutex> lock(tt::g_workspace_mutex);
            tt::g_workspaces.erase(queue->stream);
        }
        (void)hipStreamDestroy(queue->stream);
    }
    if (queue->workspace != nullptr) (void)hipFree(queue->workspace);
    delete queue;
}

void* tt_queue_native_stream(tt_queue* queue) {
    return queue != nullptr ? static_cast<void*>(queue->stream) : nullptr;
}

int32_t tt_buffer_create(tt_device* device, uint64_t size_bytes, tt_buffer** out) {
    if (out == nullptr) return TT_RES_INVALID_BUFFER_SIZE;
    *out = nullptr;
    if (device == nullptr) return TT_RES_INVALID_DEVICE;
    if (size_bytes == 0) return TT_RES_INVALID_BUFFER_SIZE;
    void* dptr = nullptr;
    if (hipMalloc(&dptr, size_bytes) != hipSuccess) {
        (void)hipGetLastError();
        return TT_RES_BUFFER_CREATION_FAILED;
    }
    if (hipMemset(dptr, 0, size_bytes) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(dptr);
        return TT_RES_BUFFER_CREATION_FAILED;
    }
    tt_buffer* buffer = new (std::nothrow) tt_buffer;
    if (buffer == nullptr) {
        (void)hipFree(dptr);
        return TT_RES_OWNERSHIP_FAILURE;
    }
    buffer->device = device;
    buffer->dptr = static_cast<uint8_t*>(dptr);
    buffer->size = size_bytes;
    buffer->owns_device = true;
    *out = buffer;
    return TT_OK;
}

int32_t tt_pool_create(tt_device* device, uint64_t stripe_bytes, uint32_t stripe_count,
                       tt_buffer** out, uint64_t* stride_out) {
    if (out == nullptr || stride_out == nullptr) return TT_RES_INVALID_BUFFER_SIZE;
    *out = nullptr;
    *stride_out = 0;
    if (device == nullptr) return TT_RES_INVALID_DEVICE;
    if (stripe_bytes == 0 || stripe_count == 0) return TT_RES_INVALID_BUFFER_SIZE;
    const uint64_t stride = (stripe_bytes + 255u) & ~uint64_t{255};
    if (stride > UINT64_MAX / stripe_count) return TT_RES_INVALID_BUFFER_SIZE;
    const int32_t status = tt_buffer_create(device, stride * stripe_count, out);
    if (status == TT_OK) *stride_out = stride;
    return status;
}

int32_t tt_buffer_window(tt_buffer* parent, uint64_t offset, uint64_t length, tt_buffer** out) {
    if (out == nullptr) return TT_RES_INVALID_BUFFER_SIZE;
    *out = nullptr;
    if (parent == nullptr) return TT_RES_BUFFER_WINDOW_UNSUPPORTED;
    if (length == 0 || offset > parent->size || parent->size - offset < length) {
        return TT_RES_INVALID_BUFFER_SIZE;
    }
    tt_buffer* root = parent->parent != nullptr ? parent->parent : parent;
    tt_buffer* window = new (std::nothrow) tt_buffer;
    if (window == nullptr) return TT_RES_OWNERSHIP_FAILURE;
    window->device = parent->device;
    window->dptr = parent->dptr + offset;
    window->size = length;
    window->parent = root;
    window->parent_offset = parent->parent_offset + offset;
    root->refs.fetch_add(1);
    *out = window;
    return TT_OK;
}

int32_t tt_buffer_wrap(tt_device* device, void* device_pointer, uint64_t size_bytes,
                       tt_buffer** out) {
    if (out == nullptr) return TT_RES_INVALID_BUFFER_SIZE;
    *out = nullptr;
    if (device == nullptr) return TT_RES_INVALID_DEVICE;
    if (device_pointer == nullptr || size_bytes == 0) return TT_RES_INVALID_BUFFER_SIZE;
    tt_buffer* buffer = new (std::nothrow) tt_buffer;
    if (buffer == nullptr) return TT_RES_OWNERSHIP_FAILURE;
    buffer->device = device;
    buffer->dptr = static_cast<uint8_t*>(device_pointer);
    buffer->size = size_bytes;
    buffer->owns_device = false;
    *out = buffer;
    return TT_OK;
}

void tt_buffer_destroy(tt_buffer* buffer) { release_buffer(buffer); }

uint64_t tt_buffer_size(const tt_buffer* buffer) { return buffer != nullptr ? buffer->size : 0; }

void* tt_buffer_contents(tt_buffer* buffer) {
    if (buffer == nullptr) return nullptr;
    tt_buffer* root = buffer->parent != nullptr ? buffer->parent : buffer;
    if (root->host == nullptr) {
        void* host = nullptr;
        if (hipHostMalloc(&host, root->size, hipHostMallocDefault) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        std::memset(host, 0, root->size);
        root->host = static_cast<uint8_t*>(host);
    }
    return root->host + buffer->parent_offset;
}

void* tt_buffer_device_pointer(tt_buffer* buffer) {
    return buffer != nullptr ? buffer->dptr : nullptr;
}

static int32_t range_ok(const tt_buffer* buffer, uint64_t offset, uint64_t length) {
    if (buffer == nullptr) return TT_CMD_INVALID_BUFFER;
    if (offset > buffer->size || buffer->size - offset < length) return TT_CMD_INVALID_BUFFER_OFFSET;
    return TT_OK;
}

int32_t tt_buffer_did_modify(tt_buffer* buffer, uint64_t offset, uint64_t length) {
    const int32_t status = range_ok(buffer, offset, length);
    if (status != TT_OK) return status;
    if (length == 0) return TT_OK;
    uint8_t* host = static_cast<uint8_t*>(tt_buffer_contents(buffer));
    if (host == nullptr) return TT_CMD_INVALID_BUFFER;
    if (hipMemcpy(buffer->dptr + offset, host + offset, length, hipMemcpyHostToDevice) !=
        hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_INVALID_DESTINATION_RANGE;
    }
    return TT_OK;
}

int32_t tt_buffer_synchronize(tt_buffer* buffer, uint64_t offset, uint64_t length) {
    const int32_t status = range_ok(buffer, offset, length);
    if (status != TT_OK) return status;
    if (length == 0) return TT_OK;
    uint8_t* host = static_cast<uint8_t*>(tt_buffer_contents(buffer));
    if (host == nullptr) return TT_CMD_INVALID_BUFFER;
    if (hipMemcpy(host + offset, buffer->dptr + offset, length, hipMemcpyDeviceToHost) !=
        hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_INVALID_SOURCE_RANGE;
    }
    return TT_OK;
}

int32_t tt_buffer_write(tt_buffer* buffer, uint64_t offset, const void* source, uint64_t length) {
    const int32_t status = range_ok(buffer, offset, length);
    if (status != TT_OK) return status;
    if (length == 0) return TT_OK;
    if (source == nullptr) return TT_CMD_INVALID_SOURCE_RANGE;
    if (hipMemcpy(buffer->dptr + offset, source, length, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_INVALID_DESTINATION_RANGE;
    }
    return TT_OK;
}

int32_t tt_buffer_read(tt_buffer* buffer, uint64_t offset, void* destination, uint64_t length) {
    const int32_t status = range_ok(buffer, offset, length);
    if (status != TT_OK) return status;
    if (length == 0) return TT_OK;
    if (destination == nullptr) return TT_CMD_INVALID_DESTINATION_RANGE;
    if (hipMemcpy(destination, buffer->dptr + offset, length, hipMemcpyDeviceToHost) !=
        hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_INVALID_SOURCE_RANGE;
    }
    return TT_OK;
}

/* ---------------------------------------------------------------- pipelines */

int32_t tt_library_create(tt_device* device, tt_library** out) {
    if (out == nullptr) return TT_PIPE_INVALID_LIBRARY;
    *out = nullptr;
    if (device == nullptr) return TT_PIPE_INVALID_DEVICE;
    tt_library* library = new (std::nothrow) tt_library;
    if (library == nullptr) return TT_PIPE_LIBRARY_COMPILATION_FAILED;
    library->device = device;
    if (!tt::prepare_decode_kernels() || !tt::prepare_prefill_kernels() ||
        !tt::prepare_q4_kernels() || !tt::prepare_stack_kernels()) {
        delete library;
        return TT_PIPE_LIBRARY_COMPILATION_FAILED;
    }
    const struct {
        const KernelDesc* table;
        uint32_t count;
    } families[] = {
        {tt::kAttentionDecodeKernels, tt::kAttentionDecodeKernelCount},
        {tt::kAttentionPrefillKernels, tt::kAttentionPrefillKernelCount},
        {tt::kAttentionFamilyKernels, tt::kAttentionFamilyKernelCount},
        {tt::kStackStepKernels, tt::kStackStepKernelCount},
        {tt::kQ4ProjectKernels, tt::kQ4ProjectKernelCount},
        {tt::kGdnDecodeKernels, tt::kGdnDecodeKernelCount},
        {tt::kGdnPrefillKernels, tt::kGdnPrefillKernelCount},
    };
    for (const auto& family : families) {
        for (uint32_t i = 0; i < family.count; ++i) library->kernels.push_back(family.table[i]);
    }
    *out = library;
    return TT_OK;
}

void tt_library_destroy(tt_library* library) { delete library; }

uint32_t tt_library_function_count(const tt_library* library) {
    return library != nullptr ? static_cast<uint32_t>(library->kernels.size()) : 0;
}

const char* tt_library_function_name(const tt_library* library, uint32_t index) {
    if (library == nullptr || index >= library->kernels.size()) return nullptr;
    return library->kernels[index].name;
}

int32_t tt_pipeline_create(tt_library* library, const char* function_name, tt_pipeline** out) {
    if (out == nullptr) return TT_PIPE_PIPELINE_CREATION_FAILED;
    *out = nullptr;
    if (library == nullptr) return TT_PIPE_INVALID_LIBRARY;
    if (function_name == nullptr || function_name[0] == '\0') return TT_PIPE_INVALID_FUNCTION_NAME;
    for (const KernelDesc& desc : library->kernels) {
        if (std::strcmp(desc.name, function_name) == 0) {
            tt_pipeline* pipeline = new (std::nothrow) tt_pipeline;
            if (pipeline == nullptr) return TT_PIPE_PIPELINE_CREATION_FAILED;
            pipeline->desc = desc;
            *out = pipeline;
            return TT_OK;
        }
    }
    return TT_PIPE_FUNCTION_LOOKUP_FAILED;
}

void tt_pipeline_destroy(tt_pipeline* pipeline) { delete pipeline; }

const char* tt_pipeline_name(const tt_pipeline* pipeline) {
    return pipeline != nullptr ? pipeline->desc.name : "";
}

/* ----------------------------------------------------------------- commands */

int32_t tt_command_buffer_create(tt_queue* queue, tt_command_buffer** out) {
    if (out == nullptr) return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
    *out = nullptr;
    if (queue == nullptr || queue->stream == nullptr) return TT_CMD_INVALID_COMMAND_QUEUE;
    tt_command_buffer* cb = new (std::nothrow) tt_command_buffer;
    if (cb == nullptr) return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
    if (hipEventCreate(&cb->begin) != hipSuccess || hipEventCreate(&cb->end) != hipSuccess) {
        (void)hipGetLastError();
        if (cb->begin != nullptr) (void)hipEventDestroy(cb->begin);
        delete cb;
        return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
    }
    cb->queue = queue;
    *out = cb;
    return TT_OK;
}

void tt_command_buffer_destroy(tt_command_buffer* cb) {
    if (cb == nullptr) return;
    if (cb->committed) (void)hipEventSynchronize(cb->end);
    if (cb->begin != nullptr) (void)hipEventDestroy(cb->begin);
    if (cb->end != nullptr) (void)hipEventDestroy(cb->end);
    for (hipEvent_t event : cb->marks) (void)hipEventDestroy(event);
    drop_graph(cb);
    release_retained(cb);
    delete cb;
}

int32_t tt_pass_begin(tt_command_buffer* cb) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_ENCODER_CREATION_FAILED;
    cb->pass_open = true;
    cb->pipeline = nullptr;
    std::memset(&cb->table, 0, sizeof(cb->table));
    std::memset(cb->bound, 0, sizeof(cb->bound));
    return TT_OK;
}

int32_t tt_pass_end(tt_command_buffer* cb) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    cb->pass_open = false;
    cb->pipeline = nullptr;
    return TT_OK;
}

int32_t tt_pass_set_pipeline(tt_command_buffer* cb, const tt_pipeline* pipeline) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    if (pipeline == nullptr || pipeline->desc.launch == nullptr) return TT_CMD_INVALID_PIPELINE;
    cb->pipeline = pipeline;
    return TT_OK;
}

int32_t tt_pass_set_buffer(tt_command_buffer* cb, const tt_buffer* buffer, uint64_t offset_bytes,
                           uint32_t index) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    if (buffer == nullptr || buffer->dptr == nullptr) return TT_CMD_INVALID_BUFFER;
    if (index > TT_MAX_BUFFER_ARGUMENT_INDEX) return TT_CMD_INVALID_BUFFER_INDEX;
    if (offset_bytes >= buffer->size) return TT_CMD_INVALID_BUFFER_OFFSET;
    cb->table.ptr[index] = buffer->dptr + offset_bytes;
    cb->table.bytes[index] = buffer->size - offset_bytes;
    cb->table.has_buffer |= 1u << index;
    cb->table.clen[index] = 0;
    cb->bound[index] = buffer;
    return TT_OK;
}

int32_t tt_pass_set_bytes(tt_command_buffer* cb, const void* bytes, uint32_t length_bytes,
                          uint32_t index) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    if (bytes == nullptr || length_bytes == 0 || length_bytes > TT_MAX_INLINE_CONSTANT_BYTES) {
        return TT_CMD_INVALID_BUFFER;
    }
    if (index > TT_MAX_BUFFER_ARGUMENT_INDEX) return TT_CMD_INVALID_BUFFER_INDEX;
    uint32_t word = 0;
    std::memcpy(&word, bytes, length_bytes < 4 ? length_bytes : 4);
    cb->table.cval[index] = word;
    cb->table.clen[index] = length_bytes;
    cb->table.has_buffer &= ~(1u << index);
    cb->bound[index] = nullptr;
    return TT_OK;
}

int32_t tt_pass_dispatch(tt_command_buffer* cb, uint64_t gx, uint64_t gy, uint64_t gz, uint64_t tx,
                         uint64_t ty, uint64_t tz) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    if (cb->pipeline == nullptr) return TT_CMD_INVALID_PIPELINE;
    constexpr uint64_t kLimit = 0x7fffffffull;
    if (gx == 0 || gy == 0 || gz == 0 || tx == 0 || ty == 0 || tz == 0 || gx > kLimit ||
        gy > kLimit || gz > kLimit || tx * ty * tz > 1024) {
        return TT_CMD_INVALID_DISPATCH_EXTENT;
    }
    Command command{};
    command.kind = CommandKind::Dispatch;
    command.name = cb->pipeline->desc.name;
    command.launch = cb->pipeline->desc.launch;
    command.bindings = cb->table;
    command.grid = Grid{gx, gy, gz, tx, ty, tz};
    const int32_t status = command.launch(command.bindings, command.grid, nullptr, true);
    if (status != TT_OK) return status;
    cb->commands.push_back(command);
    for (uint32_t index = 0; index < tt::kArgSlots; ++index) {
        if (cb->table.has_buffer & (1u << index)) retain(cb, cb->bound[index]);
    }
    return TT_OK;
}

int32_t tt_pass_barrier(tt_command_buffer* cb) {
    if (cb == nullptr || !cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    return TT_OK;
}

int32_t tt_blit_copy(tt_command_buffer* cb, const tt_buffer* source, uint64_t source_offset,
                     tt_buffer* destination, uint64_t destination_offset, uint64_t length) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_INVALID_BLIT_PASS;
    if (source == nullptr || destination == nullptr) return TT_CMD_INVALID_BUFFER;
    if (length == 0) return TT_CMD_INVALID_COPY_EXTENT;
    if (source_offset > source->size || source->size - source_offset < length) {
        return TT_CMD_INVALID_SOURCE_RANGE;
    }
    if (destination_offset > destination->size || destination->size - destination_offset < length) {
        return TT_CMD_INVALID_DESTINATION_RANGE;
    }
    Command command{};
    command.kind = CommandKind::Copy;
    command.name = "copy_buffer";
    command.a = source->dptr + source_offset;
    command.b = destination->dptr + destination_offset;
    command.length = length;
    cb->commands.push_back(command);
    retain(cb, source);
    retain(cb, destination);
    return TT_OK;
}

int32_t tt_blit_fill(tt_command_buffer* cb, tt_buffer* destination, uint64_t destination_offset,
                     uint64_t length, uint8_t value) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_INVALID_BLIT_PASS;
    if (destination == nullptr) return TT_CMD_INVALID_BUFFER;
    if (length == 0) return TT_CMD_INVALID_FILL_EXTENT;
    if (destination_offset > destination->size || destination->size - destination_offset < length) {
        return TT_CMD_INVALID_DESTINATION_RANGE;
    }
    Command command{};
    command.kind = CommandKind::Fill;
    command.name = "fill_buffer";
    command.b = destination->dptr + destination_offset;
    command.length = length;
    command.value = value;
    cb->commands.push_back(command);
    retain(cb, destination);
    return TT_OK;
}

uint32_t tt_command_count(const tt_command_buffer* cb) {
    return cb != nullptr ? static_cast<uint32_t>(cb->commands.size()) : 0;
}

static void drop_graph(tt_command_buffer* cb) {
    if (cb->graph_exec != nullptr) (void)hipGraphExecDestroy(cb->graph_exec);
    if (cb->graph != nullptr) (void)hipGraphDestroy(cb->graph);
    cb->graph_exec = nullptr;
    cb->graph = nullptr;
}

// Launches every recorded command on the stream in order; with marks, an event
// is recorded before the first and after each command.
static hipError_t issue_commands(tt_command_buffer* cb, hipStream_t stream, bool with_marks) {
    if (with_marks) {
        while (cb->marks.size() < cb->commands.size() + 1) {
            hipEvent_t event = nullptr;
            if (hipEventCreate(&event) != hipSuccess) return hipGetLastError();
            cb->marks.push_back(event);
        }
        (void)hipEventRecord(cb->marks[0], stream);
    }
    // A wait whose signal has not been committed fails the whole commit before anything is
    // launched: found at its own position, it would leave the command buffer half executed.
    // (A signal earlier in this same command buffer reaches a later wait of it.)
    {
        std::map<const tt_event*, uint64_t> signalled_here;
        for (const Command& command : cb->commands) {
            if (command.kind == CommandKind::Signal) {
                uint64_t& highest = signalled_here[command.event];
                highest = std::max(highest, command.event_value);
            } else if (command.kind == CommandKind::Wait) {
                const auto here = signalled_here.find(command.event);
                if (here != signalled_here.end() && here->second >= command.event_value) continue;
                std::lock_guard<std::mutex> lock(command.event->mutex);
                if (command.event->reached.lower_bound(command.event_value) ==
                    command.event->reached.end()) {
                    return hipErrorNotReady;
                }
            }
        }
    }
    size_t index = 0;
    for (const Command& command : cb->commands) {
        hipError_t error = hipSuccess;
        if (command.kind == CommandKind::Dispatch) {
            const int32_t status = command.launch(command.bindings, command.grid, stream, false);
            error = hipGetLastError();
            if (status != TT_OK && error == hipSuccess) error = hipErrorInvalidValue;
        } else if (command.kind == CommandKind::Signal) {
            // a fresh HIP event per signalled value, recorded behind everything issued so far
            std::lock_guard<std::mutex> lock(command.event->mutex);
            hipEvent_t& reached = command.event->reached[command.event_value];
            const bool fresh = reached == nullptr;
            if (fresh) error = hipEventCreateWithFlags(&reached, hipEventDisableTiming);
            if (error == hipSuccess) error = hipEventRecord(reached, stream);
            if (error != hipSuccess && fresh) {
                // no entry without a recorded event behind it: a later wait must not find one
                if (reached != nullptr) (void)hipEventDestroy(reached);
                command.event->reached.erase(command.event_value);
            }
            // A wait takes the smallest committed value that reaches the one it asks for, so
            // the oldest values can go once there are many: a late wait for one of them is
            // served by a newer signal, which the counter has passed as well.
            while (error == hipSuccess && command.event->reached.size() > kEventValuesKept &&
                   command.event->reached.begin()->first != command.event_value) {
                (void)hipEventDestroy(command.event->reached.begin()->second);
                command.event->reached.erase(command.event->reached.begin());
            }
        } else if (command.kind == CommandKind::Wait) {
            // the smallest committed signal that reaches the value
            std::lock_guard<std::mutex> lock(command.event->mutex);
            const auto reached = command.event->reached.lower_bound(command.event_value);
            error = reached == command.event->reached.end()
                        ? hipErrorNotReady
                        : hipStreamWaitEvent(stream, reached->second, 0);
        } else if (command.kind == CommandKind::Copy) {
            const bool wide = ((reinterpret_cast<uintptr_t>(command.a) |
                                reinterpret_cast<uintptr_t>(command.b)) & 15u) == 0;
            const uint64_t units = wide ? command.length / 16 + 15 : command.length;
            const uint64_t blocks = (units + 255) / 256;
            const unsigned grid = static_cast<unsigned>(blocks < 8192 ? (blocks ? blocks : 1) : 8192);
            hipLaunchKernelGGL(tt_copy_bytes, dim3(grid), dim3(256), 0, stream, command.a,
                               command.b, command.length, wide ? 1u : 0u);
            error = hipGetLastError();
        } else {
            const uint64_t blocks = (command.length + 255) / 256;
            const unsigned grid = static_cast<unsigned>(blocks < 4096 ? blocks : 4096);
            hipLaunchKernelGGL(tt_fill_bytes, dim3(grid), dim3(256), 0, stream, command.b,
                               command.length, command.value);
            error = hipGetLastError();
        }
        if (error != hipSuccess) return error;
        ++index;
        if (with_marks) (void)hipEventRecord(cb->marks[index], stream);
    }
    return hipSuccess;
}

int32_t tt_commit(tt_command_buffer* cb) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    hipStream_t stream = cb->queue->stream;
    cb->submit_error = hipSuccess;
    cb->marks_valid = false;
    (void)hipEventRecord(cb->begin, stream);
    if (cb->graph_exec != nullptr) {
        cb->submit_error = hipGraphLaunch(cb->graph_exec, stream);
    } else {
        cb->submit_error = issue_commands(cb, stream, cb->profiling);
        cb->marks_valid = cb->profiling && cb->submit_error == hipSuccess;
    }
    (void)hipEventRecord(cb->end, stream);
    cb->committed = true;
    return TT_OK;
}

int32_t tt_command_buffer_compile(tt_command_buffer* cb) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_INVALID_COMPUTE_PASS;
    if (cb->commands.empty()) return TT_CMD_INVALID_COMMAND_BUFFER;
    for (const Command& command : cb->commands) {
        if (command.kind == CommandKind::Signal || command.kind == CommandKind::Wait) {
            return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
        }
    }
    if (cb->committed) (void)hipEventSynchronize(cb->end);
    drop_graph(cb);
    hipStream_t stream = cb->queue->stream;
    if (hipStreamBeginCapture(stream, hipStreamCaptureModeRelaxed) != hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
    }
    const hipError_t issued = issue_commands(cb, stream, false);
    const hipError_t ended = hipStreamEndCapture(stream, &cb->graph);
    if (issued != hipSuccess || ended != hipSuccess || cb->graph == nullptr ||
        hipGraphInstantiate(&cb->graph_exec, cb->graph, nullptr, nullptr, 0) != hipSuccess) {
        (void)hipGetLastError();
        drop_graph(cb);
        return TT_CMD_COMMAND_BUFFER_CREATION_FAILED;
    }
    return TT_OK;
}

int32_t tt_command_buffer_set_profiling(tt_command_buffer* cb, int32_t enabled) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    cb->profiling = enabled != 0;
    return TT_OK;
}

const char* tt_command_name(const tt_command_buffer* cb, uint32_t index) {
    if (cb == nullptr || index >= cb->commands.size()) return nullptr;
    return cb->commands[index].name;
}

int32_t tt_command_gpu_ms(tt_command_buffer* cb, uint32_t index, double* ms_out) {
    if (cb == nullptr || ms_out == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    *ms_out = 0.0;
    if (!cb->marks_valid || cb->committed || index >= cb->commands.size()) {
        return TT_CMD_INVALID_PENDING_EXECUTION;
    }
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, cb->marks[index], cb->marks[index + 1]) != hipSuccess) {
        (void)hipGetLastError();
        return TT_CMD_INVALID_PENDING_EXECUTION;
    }
    *ms_out = ms;
    return TT_OK;
}

int32_t tt_wait(tt_command_buffer* cb, tt_execution_result* result) {
    if (result != nullptr) std::memset(result, 0, sizeof(*result));
    if (cb == nullptr || !cb->committed) {
        if (result != nullptr) result->status = TT_CMD_INVALID_PENDING_EXECUTION;
        return TT_CMD_INVALID_PENDING_EXECUTION;
    }
    hipError_t error = hipEventSynchronize(cb->end);
    if (error == hipSuccess) error = cb->submit_error;
    float ms = 0.0f;
    if (error == hipSuccess && hipEventElapsedTime(&ms, cb->begin, cb->end) != hipSuccess) {
        (void)hipGetLastError();
        ms = 0.0f;
    }
    cb->committed = false;
    if (result != nullptr) {
        result->status = TT_OK;
        result->completed = error == hipSuccess ? 1 : 0;
        result->failure = classify(error);
        result->gpu_ms = ms;
        if (error != hipSuccess) {
            result->has_native_error_code = 1;
            result->native_error_code = static_cast<int64_t>(error);
            const char* text = hipGetErrorString(error);
            std::snprintf(result->diagnostic, sizeof(result->diagnostic), "%s",
                          text != nullptr ? text : "unknown HIP error");
            result->diagnostic_length = std::strlen(result->diagnostic);
        }
    }
    return TT_OK;
}

static int32_t encode_event(tt_command_buffer* cb, tt_event* event, uint64_t value,
                            CommandKind kind) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->pass_open) return TT_CMD_INVALID_COMMAND_BUFFER;   // between passes only
    if (event == nullptr) return TT_CMD_INVALID_EVENT;
    if (value == 0) return TT_CMD_INVALID_EVENT_VALUE;
    Command command{};
    command.kind = kind;
    command.name = kind == CommandKind::Signal ? "signal_event" : "wait_for_event";
    command.event = event;
    command.event_value = value;
    event->refs.fetch_add(1);
    cb->retained_events.push_back(event);
    cb->commands.push_back(command);
    drop_graph(cb);
    return TT_OK;
}

int32_t tt_encode_signal_event(tt_command_buffer* cb, tt_event* event, uint64_t value) {
    return encode_event(cb, event, value, CommandKind::Signal);
}

int32_t tt_encode_wait_for_event(tt_command_buffer* cb, tt_event* event, uint64_t value) {
    return encode_event(cb, event, value, CommandKind::Wait);
}

int32_t tt_event_create(tt_device* device, tt_event** out) {
    if (out == nullptr) return TT_RES_EVENT_CREATION_FAILED;
    *out = nullptr;
    if (device == nullptr) return TT_RES_INVALID_DEVICE;
    tt_event* event = new (std::nothrow) tt_event;
    if (event == nullptr) return TT_RES_EVENT_CREATION_FAILED;
    *out = event;
    return TT_OK;
}

void tt_event_destroy(tt_event* event) { release_event(event); }

int32_t tt_command_buffer_reset(tt_command_buffer* cb) {
    if (cb == nullptr) return TT_CMD_INVALID_COMMAND_BUFFER;
    if (cb->committed) (void)hipEventSynchronize(cb->end);
    cb->committed = false;
    cb->commands.clear();
    cb->marks_valid = false;
    drop_graph(cb);
    release_retained(cb);
    cb->pass_open = false;
    cb->pipeline = nullptr;
    return TT_OK;
}

}  // extern "C"
