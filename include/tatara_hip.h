/*
 * tatara_hip.h — C ABI of the MI355X (gfx950) backend for Tatara's
 * attention-family hot path.
 *
 * This is the drop-in boundary: the entry points below are what a binding of
 * the reference's backend operator interface
 * (include/tatara/backend/metal/{resources,pipeline,commands}.h) would bind on
 * an AMD host.  Plain pointers, sizes and integer status codes only.  Each
 * declaration cites the reference interface it replaces.
 *
 * Model: a device owns HBM buffers; a kernel library resolves the reference's
 * kernel names ("attn_qk_rope", "attention_decode", "gdn_recurrence", ...) to
 * pipelines whose buffer-index argument tables are the reference's; a command
 * buffer records a compute pass (set_pipeline / set_buffer / set_bytes /
 * dispatch / barrier) and blit commands, `tt_commit` submits the recording to
 * the queue's HIP stream and `tt_wait` blocks until it has completed.
 * Validation (null handles, index > 30, offset >= size, zero extents, operand
 * shapes a kernel assumes) happens on the host before anything is launched and
 * is reported through the status codes; nothing throws.
 *
 * Memory model: buffers live in HBM.  `tt_buffer_contents` exposes a pinned
 * host staging view of the same size (allocated on first use);
 * `tt_buffer_did_modify` publishes host writes to HBM and
 * `tt_buffer_synchronize` fetches device results, the managed-storage idiom
 * (didModifyRange / synchronizeResource) standing in for the reference's
 * unified-memory `contents()`.  `tt_buffer_write/read` move bytes without a
 * staging view; `tt_buffer_wrap` adopts device memory owned by someone else
 * (a torch tensor, another allocator) without copying.
 */
#ifndef TATARA_HIP_H
#define TATARA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TT_ABI_VERSION 1u
/* commands.h:29,32 */
#define TT_MAX_BUFFER_ARGUMENT_INDEX 30u
#define TT_MAX_INLINE_CONSTANT_BYTES 4096u
/* commands.h:299 */
#define TT_DIAGNOSTIC_STORAGE_BYTES 512u

typedef struct tt_device tt_device;
typedef struct tt_queue tt_queue;
typedef struct tt_buffer tt_buffer;
typedef struct tt_library tt_library;
typedef struct tt_pipeline tt_pipeline;
typedef struct tt_command_buffer tt_command_buffer;
typedef struct tt_event tt_event;

/* Status codes.  0 is success in every family.  Command errors keep the
 * numbering of MetalCommandError (commands.h:232-262); resource errors are
 * MetalResourceError (resources.h:174-184) + 100; pipeline errors are
 * MetalPipelineError (pipeline.h:99-110) + 200. */
typedef enum tt_status {
    TT_OK = 0,
    TT_CMD_INVALID_COMMAND_QUEUE = 1,
    TT_CMD_INVALID_COMMAND_BUFFER = 2,
    TT_CMD_INVALID_EVENT = 3,
    TT_CMD_INVALID_EVENT_VALUE = 4,
    TT_CMD_INVALID_COMPUTE_PASS = 5,
    TT_CMD_INVALID_BLIT_PASS = 6,
    TT_CMD_INVALID_PIPELINE = 7,
    TT_CMD_INVALID_BUFFER = 8,
    TT_CMD_INVALID_BUFFER_INDEX = 9,
    TT_CMD_INVALID_BUFFER_OFFSET = 10,
    TT_CMD_INVALID_SOURCE_RANGE = 11,
    TT_CMD_INVALID_DESTINATION_RANGE = 12,
    TT_CMD_INVALID_COPY_EXTENT = 13,
    TT_CMD_INVALID_FILL_EXTENT = 14,
    TT_CMD_INVALID_DISPATCH_EXTENT = 15,
    TT_CMD_CONTEXT_OUT_OF_RANGE = 16,
    TT_CMD_STATE_SLOT_MISMATCH = 17,
    TT_CMD_INVALID_PENDING_EXECUTION = 18,
    TT_CMD_COMMAND_BUFFER_CREATION_FAILED = 19,
    TT_CMD_ENCODER_CREATION_FAILED = 20,
    TT_CMD_INVALID_DEVICE = 27,
    TT_CMD_INVALID_STREAM_GROUP = 28,
    /* no counterpart in MetalCommandError: a request needs more of the library's fixed
     * device scratch than TT_STATIC_SCRATCH_BYTES (tt_attention_decode_lanes_static) */
    TT_CMD_STATIC_SCRATCH_EXCEEDED = 40,
    TT_RES_INVALID_DEVICE = 101,
    TT_RES_SYSTEM_DEVICE_UNAVAILABLE = 102,
    TT_RES_COMMAND_QUEUE_CREATION_FAILED = 103,
    TT_RES_EVENT_CREATION_FAILED = 104,
    TT_RES_INVALID_BUFFER_SIZE = 105,
    TT_RES_BUFFER_CREATION_FAILED = 106,
    TT_RES_OWNERSHIP_FAILURE = 107,
    TT_RES_BUFFER_WINDOW_UNSUPPORTED = 108,
    TT_PIPE_INVALID_DEVICE = 201,
    TT_PIPE_INVALID_LIBRARY = 202,
    TT_PIPE_INVALID_FUNCTION_NAME = 205,
    TT_PIPE_LIBRARY_COMPILATION_FAILED = 206,
    TT_PIPE_FUNCTION_LOOKUP_FAILED = 207,
    TT_PIPE_PIPELINE_CREATION_FAILED = 208
} tt_status;

/* MetalExecutionFailure (commands.h:281-295). */
typedef enum tt_failure {
    TT_FAILURE_NONE = 0,
    TT_FAILURE_INTERNAL = 1,
    TT_FAILURE_TIMEOUT = 2,
    TT_FAILURE_PAGE_FAULT = 3,
    TT_FAILURE_OUT_OF_MEMORY = 6,
    TT_FAILURE_INVALID_RESOURCE = 7,
    TT_FAILURE_DEVICE_REMOVED = 9,
    TT_FAILURE_UNKNOWN_ERROR = 11
} tt_failure;

/* MetalExecutionResult + MetalExecutionTiming (commands.h:374-416).  gpu_ms is
 * the device time between the first and the last recorded command, measured
 * with HIP events on the queue's stream. */
typedef struct tt_execution_result {
    int32_t status;
    int32_t completed;
    int32_t failure;
    int32_t has_native_error_code;
    int64_t native_error_code;
    double gpu_ms;
    uint64_t diagnostic_length;
    char diagnostic[TT_DIAGNOSTIC_STORAGE_BYTES];
} tt_execution_result;

uint32_t tt_abi_version(void);
/* Human-readable name of a status code; never NULL. */
const char* tt_status_name(int32_t status);

/* ---- resources (resources.h:237-252) ---- */
/* create_system_device (resources.h:237): HIP device 0 of the process. */
int32_t tt_device_create(tt_device** out);
void tt_device_destroy(tt_device* device);
/* MetalDevice::name (resources.h:41). */
const char* tt_device_name(const tt_device* device);
/* Number of compute units of the device (no reference counterpart; used to size
 * split-K grids). */
uint32_t tt_device_compute_units(const tt_device* device);
/* create_command_queue (resources.h:239): one in-order HIP stream.  A queue also owns a
 * workspace in device memory (270,336 bytes per compute unit: 69 MB on 256) for operators
 * whose reference bindings carry no scratch - attention_flash_v2_blk / attention_streaming_blk
 * share the key walks of a block of few rows through it, attn_project_blk / gdn_project_blk /
 * outproj_blk the tiles of their last, partly filled round; a queue whose workspace could not
 * be allocated works without. */
int32_t tt_queue_create(tt_device* device, tt_queue** out);
void tt_queue_destroy(tt_queue* queue);
/* The HIP stream (hipStream_t) behind a queue, for event timing by the caller. */
void* tt_queue_native_stream(tt_queue* queue);
/* create_event (resources.h:240): a counter that command buffers of any queue of the
 * device signal and wait for (tt_encode_signal_event / tt_encode_wait_for_event). */
int32_t tt_event_create(tt_device* device, tt_event** out);
void tt_event_destroy(tt_event* event);

/* create_shared_buffer (resources.h:241) with the zeroed-allocation rule of
 * decode_step.cpp:49-57 built in: the HBM allocation is zero-filled. */
int32_t tt_buffer_create(tt_device* device, uint64_t size_bytes, tt_buffer** out);
/* create_striped_pool_buffer (resources.h:247): count equal stripes,
 * *stride_out bytes apart (stripe_bytes rounded up to 256). */
int32_t tt_pool_create(tt_device* device, uint64_t stripe_bytes, uint32_t stripe_count,
                       tt_buffer** out, uint64_t* stride_out);
/* create_buffer_window (resources.h:250): aliasing view; keeps the parent alive. */
int32_t tt_buffer_window(tt_buffer* parent, uint64_t offset, uint64_t length, tt_buffer** out);
/* Adopt caller-owned device memory (no reference counterpart). */
int32_t tt_buffer_wrap(tt_device* device, void* device_pointer, uint64_t size_bytes,
                       tt_buffer** out);
void tt_buffer_destroy(tt_buffer* buffer);
/* MetalBuffer::size_bytes / contents (resources.h:133-134). */
uint64_t tt_buffer_size(const tt_buffer* buffer);
void* tt_buffer_contents(tt_buffer* buffer);
void* tt_buffer_device_pointer(tt_buffer* buffer);
int32_t tt_buffer_did_modify(tt_buffer* buffer, uint64_t offset, uint64_t length);
int32_t tt_buffer_synchronize(tt_buffer* buffer, uint64_t offset, uint64_t length);
int32_t tt_buffer_write(tt_buffer* buffer, uint64_t offset, const void* source, uint64_t length);
int32_t tt_buffer_read(tt_buffer* buffer, uint64_t offset, void* destination, uint64_t length);

/* ---- pipelines (pipeline.h:141-144) ---- */
/* create_library_with_source (pipeline.h:141): the library is the gfx950 code
 * object linked into this shared object, so there is no source argument. */
int32_t tt_library_create(tt_device* device, tt_library** out);
void tt_library_destroy(tt_library* library);
/* Number of kernel names the library resolves and the i-th name. */
uint32_t tt_library_function_count(const tt_library* library);
const char* tt_library_function_name(const tt_library* library, uint32_t index);
/* create_function + create_compute_pipeline (pipeline.h:142-143) in one step. */
int32_t tt_pipeline_create(tt_library* library, const char* function_name, tt_pipeline** out);
void tt_pipeline_destroy(tt_pipeline* pipeline);
const char* tt_pipeline_name(const tt_pipeline* pipeline);

/* ---- command encoding (commands.h:418-507) ---- */
/* create_command_buffer (commands.h:418). */
int32_t tt_command_buffer_create(tt_queue* queue, tt_command_buffer** out);
void tt_command_buffer_destroy(tt_command_buffer* command_buffer);
/* begin_compute_pass / end_compute_pass (commands.h:420, 492).  At most one
 * pass is open at a time; pass commands outside one return
 * TT_CMD_INVALID_COMPUTE_PASS. */
int32_t tt_pass_begin(tt_command_buffer* command_buffer);
int32_t tt_pass_end(tt_command_buffer* command_buffer);
/* set_compute_pipeline (commands.h:440). */
int32_t tt_pass_set_pipeline(tt_command_buffer* command_buffer, const tt_pipeline* pipeline);
/* set_buffer (commands.h:442): index <= 30, offset < size. */
int32_t tt_pass_set_buffer(tt_command_buffer* command_buffer, const tt_buffer* buffer,
                           uint64_t offset_bytes, uint32_t index);
/* set_bytes (commands.h:456): 1..4096 bytes copied into the recording. */
int32_t tt_pass_set_bytes(tt_command_buffer* command_buffer, const void* bytes,
                          uint32_t length_bytes, uint32_t index);
/* dispatch_threadgroups (commands.h:444).  The grid is the reference call
 * site's; a pipeline validates it against the shape its operator is
 * dispatched with and derives its own HIP launch geometry from it. */
int32_t tt_pass_dispatch(tt_command_buffer* command_buffer, uint64_t groups_x, uint64_t groups_y,
                         uint64_t groups_z, uint64_t threads_x, uint64_t threads_y,
                         uint64_t threads_z);
/* memory_barrier (commands.h:461): the stream is in-order, so this only
 * validates the pass. */
int32_t tt_pass_barrier(tt_command_buffer* command_buffer);
/* copy_buffer / fill_buffer of a blit pass (commands.h:493-498), recorded
 * directly on the command buffer (outside a compute pass). */
int32_t tt_blit_copy(tt_command_buffer* command_buffer, const tt_buffer* source,
                     uint64_t source_offset, tt_buffer* destination, uint64_t destination_offset,
                     uint64_t length);
int32_t tt_blit_fill(tt_command_buffer* command_buffer, tt_buffer* destination,
                     uint64_t destination_offset, uint64_t length, uint8_t value);
/* encode_signal_event / encode_wait_for_event (commands.h:421-426), recorded on the command
 * buffer outside a pass.  A signal marks `value` reached once everything recorded before
 * it has completed; a wait holds everything recorded after it until the event has reached
 * `value` (a signal of `value` or more).  value 0 is TT_CMD_INVALID_EVENT_VALUE.  The
 * signal that a wait depends on must have been committed before the waiting command
 * buffer is committed (commits in dependency order, as the reference's lane queues do);
 * otherwise the commit fails and tt_wait reports it.  A command buffer with event
 * commands cannot be compiled into a graph. */
int32_t tt_encode_signal_event(tt_command_buffer* command_buffer, tt_event* event, uint64_t value);
int32_t tt_encode_wait_for_event(tt_command_buffer* command_buffer, tt_event* event,
                                 uint64_t value);
/* Number of commands recorded so far. */
uint32_t tt_command_count(const tt_command_buffer* command_buffer);
/* commit (commands.h:500): launches every recorded command on the queue's
 * stream, bracketed by HIP events.  The recording is kept, so the same command
 * buffer may be committed again after tt_wait (the per-token walk re-submits
 * an identical recording). */
int32_t tt_commit(tt_command_buffer* command_buffer);
/* wait_until_completed(_timed) (commands.h:501, 506). */
int32_t tt_wait(tt_command_buffer* command_buffer, tt_execution_result* result);
/* Compiles the recording into a HIP graph (stream capture); later commits
 * replay the graph in one launch instead of one launch per command.  Counterpart
 * of the reference's indirect-command-buffer command graph
 * (src/runtime/prefill_step.cpp:4165-5415) for launch-bound walks.  Row-batched
 * (_ms) recordings read contexts and state offsets from the state table in
 * device memory, so one compiled walk serves every token of a lane group. */
int32_t tt_command_buffer_compile(tt_command_buffer* command_buffer);
/* Per-command device timing, the dispatch-boundary counter sampling of
 * include/tatara/backend/metal/counter_sampling.h: when enabled, an eager
 * (uncompiled) commit brackets every command with HIP events; after tt_wait,
 * tt_command_gpu_ms reports command `index`'s device time. */
int32_t tt_command_buffer_set_profiling(tt_command_buffer* command_buffer, int32_t enabled);
const char* tt_command_name(const tt_command_buffer* command_buffer, uint32_t index);
int32_t tt_command_gpu_ms(tt_command_buffer* command_buffer, uint32_t index, double* ms_out);
/* Discards the recording so the command buffer can be encoded afresh. */
int32_t tt_command_buffer_reset(tt_command_buffer* command_buffer);

/* ---- entry point that allocates nothing ---- */
/* Has no counterpart in the reference.  It is for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It is the lane-batched split-K decode attention that a recording of
 * `attention_decode_split_ms` followed by `attention_decode_combine_ms` runs (same
 * kernels, same operands, same results bit for bit), launched directly on the queue's
 * stream, with the split records - the scratch those two dispatches otherwise take as a
 * caller-bound buffer - in a fixed array of TT_STATIC_SCRATCH_BYTES that the library's
 * code object holds on every GPU it is loaded on until the process ends.  It calls no
 * hipMalloc / hipFree and no allocating library routine.
 *
 *   q, gate, out     [rows][query_stride] bf16 slabs, 16 x 256 values used per row
 *   keys_pool, values_pool   bf16 caches, row r's at element offset table[4r]
 *   state_table      rows x {kv element offset, context, 0, 0} u32 in device memory
 *   *_bytes          bytes readable / writable behind each pointer (validated like bound
 *                    buffers: TT_CMD_INVALID_BUFFER for a null pointer,
 *                    TT_CMD_INVALID_BUFFER_OFFSET for an extent too small)
 *   rows 1..16, query_stride >= 4096, split_keys a positive multiple of 32
 *
 * Every row is processed (short contexts take one split).  The records need
 * rows * 16 * ceil(capacity / split_keys) * 1032 bytes; a request beyond
 * TT_STATIC_SCRATCH_BYTES returns TT_CMD_STATIC_SCRATCH_EXCEEDED and launches nothing
 * (raise split_keys or lower rows).  All calls on one GPU share that GPU's array, which
 * keeps the last call's records: every record a call reads was written by that call, so
 * nothing needs clearing, but two calls that overlap in time on one GPU (different
 * queues, or a replayed capture next to a direct call) race on it.  The call only
 * enqueues; completion is the stream's (hipStreamSynchronize on
 * tt_queue_native_stream, or a later tt_commit / tt_wait on the same queue). */
#define TT_STATIC_SCRATCH_BYTES (8u << 20)
int32_t tt_attention_decode_lanes_static(tt_queue* queue, const void* q, uint64_t q_bytes,
                                         const void* gate, uint64_t gate_bytes,
                                         const void* keys_pool, uint64_t keys_bytes,
                                         const void* values_pool, uint64_t values_bytes,
                                         const void* state_table, uint64_t table_bytes, void* out,
                                         uint64_t out_bytes, uint32_t rows, uint32_t capacity,
                                         uint32_t query_stride, uint32_t split_keys);

/* ---- planning of the split-K walk of a token wave ----------------------------------
 * The reference plans its split path per lane on the host (a fixed 256-key partition,
 * src/runtime/decode_step.cpp:1249-1259; include/tatara/runtime/decode_geometry.h:133-146
 * attention_partitions).  Here one grid serves every lane of a wave, and how many keys a
 * workgroup takes decides how well that grid fills the chip; the rule lives in the library
 * so that every caller (the C++ runtime, the Python mirror, a serving loop) plans alike.
 *
 * tt_split_workgroups: workgroups of one attention layer's split-K grid that hold keys
 * when lane r sees visible_keys[r] keys and a workgroup takes split_keys of them
 * (two kv heads x sum of ceil(keys / split_keys)); 0 for split_keys == 0.
 * tt_choose_split_keys: the finest multiple of 32, at least 128, with which those
 * workgroups fit compute_units one each (a lane count above compute_units / 2 cannot
 * fit and gets the even share). */
uint32_t tt_split_workgroups(const uint32_t* visible_keys, uint32_t rows, uint32_t split_keys);
uint32_t tt_choose_split_keys(const uint32_t* visible_keys, uint32_t rows, uint32_t compute_units);

/* Planning of attention_flash_split_blk (no counterpart in the reference, whose prefill walks
 * 256-row query tiles of blocks of at most 2048 rows, prefill_step.cpp:1469-1475): a block of
 * few rows is few workgroups - 2048 rows are 128 on 256 compute units - while each of them
 * walks the whole prefix, so the operator lets several workgroups share a position tile's
 * key walk, with the count and the scratch in the caller's hands.  (attention_flash_v2_blk
 * plans the same by itself and uses its queue's workspace.)
 *
 * tt_flash_prefill_splits: the sharers per tile (1..8) with which a block of `rows` rows, the
 * last of which sees visible_keys keys, fills compute_units (1 where the longest walk is
 * under 16 tiles of 32 keys); tt_flash_prefill_scratch_bytes: what the operator's scratch binding must
 * hold for that many (0 for one). */
uint32_t tt_flash_prefill_splits(uint32_t rows, uint32_t visible_keys, uint32_t compute_units);
uint64_t tt_flash_prefill_scratch_bytes(uint32_t rows, uint32_t splits);

#ifdef __cplusplus
}
#endif

#endif /* TATARA_HIP_H */
