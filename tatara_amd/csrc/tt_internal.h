// Internal contract between the C-ABI core (tt_abi.hip) and the kernel
// translation units: a kernel registers under the reference's kernel name with
// a launcher that reads the bound argument table (buffer pointers with their
// offsets already applied, 4-byte constants) and the call site's grid,
// validates them against what its HIP kernels assume, and launches.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tatara_hip.h"
#include "tt_constants.h"

namespace tt {

constexpr uint32_t kArgSlots = TT_MAX_BUFFER_ARGUMENT_INDEX + 1;

struct Bindings {
    void* ptr[kArgSlots];        // device address = buffer base + bound offset
    uint64_t bytes[kArgSlots];   // bytes available from ptr to the end of the buffer
    uint32_t cval[kArgSlots];    // first four bytes of a set_bytes constant
    uint32_t clen[kArgSlots];    // its length (0 = not bound)
    uint32_t has_buffer;         // bit i set when slot i holds a buffer
};

struct Grid {
    uint64_t gx, gy, gz;  // threadgroups
    uint64_t tx, ty, tz;  // threads per threadgroup
};

// validate_only: check bindings and shapes, launch nothing.
typedef int32_t (*LaunchFn)(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only);

struct KernelDesc {
    const char* name;
    LaunchFn launch;
};

// Accessors that fail the launch instead of dereferencing an unbound slot.
struct Args {
    const Bindings& b;
    int32_t status = TT_OK;
    explicit Args(const Bindings& bindings) : b(bindings) {}
    template <typename T>
    T* buffer(uint32_t index, uint64_t min_bytes) {
        if (index >= kArgSlots || !(b.has_buffer & (1u << index))) {
            fail(TT_CMD_INVALID_BUFFER);
            return nullptr;
        }
        if (b.bytes[index] < min_bytes) {
            fail(TT_CMD_INVALID_BUFFER_OFFSET);
            return nullptr;
        }
        return static_cast<T*>(b.ptr[index]);
    }
    uint64_t buffer_bytes(uint32_t index) const {
        return (index < kArgSlots && (b.has_buffer & (1u << index))) ? b.bytes[index] : 0;
    }
    uint32_t constant(uint32_t index) {
        if (index >= kArgSlots || b.clen[index] < 4) {
            fail(TT_CMD_INVALID_BUFFER);
            return 0;
        }
        return b.cval[index];
    }
    void require(bool ok, int32_t code) {
        if (!ok) fail(code);
    }
    void fail(int32_t code) {
        if (status == TT_OK) status = code;
    }
};

// A context is a cache position: equality with capacity is one past the
// allocation (reference include/tatara/runtime/decode_geometry.h:133-135).
inline bool context_ok(uint32_t context, uint32_t capacity) {
    return capacity != 0 && context < capacity;
}

inline bool grid_is(const Grid& g, uint64_t gx, uint64_t gy, uint64_t gz, uint64_t tx, uint64_t ty,
                    uint64_t tz) {
    return g.gx == gx && g.gy == gy && g.gz == gz && g.tx == tx && g.ty == ty && g.tz == tz;
}

// defined beside the decode rope kernel it shares, registered with the prefill family
int32_t op_attn_qk_rope_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only);

// The HIP stream of a queue (tt_queue is defined by the C-ABI core), for entry points
// that launch directly instead of recording.
hipStream_t queue_stream(const tt_queue* queue);
// Compute units of the device the queue was made on (0 for a null queue).
uint32_t queue_compute_units(const tt_queue* queue);

// Device memory a queue owns for operators whose reference bindings carry no scratch (the
// shared key walk of attention_flash_v2_blk on blocks of few rows).  Allocated when the queue
// is created, so never under a stream capture; commands of one queue run in order, so one
// operator at a time uses it.  base is null for a stream no queue of this library made, or
// where the allocation failed.
struct StreamWorkspace {
    uint8_t* base = nullptr;
    uint64_t bytes = 0;
    uint32_t compute_units = 0;
};
StreamWorkspace stream_workspace(hipStream_t stream);
// the bytes a queue's workspace holds on a device of that many compute units
uint64_t stream_workspace_bytes(uint32_t compute_units);

// attention_flash_split_blk: the workgroups that share a position tile's key walk so that a
// block of `rows` rows whose last row sees `visible` keys fills `compute_units`, and the
// scratch bytes that many need.
uint32_t flash_prefill_splits(uint32_t rows, uint32_t visible, uint32_t compute_units);
uint64_t flash_prefill_scratch_bytes(uint32_t rows, uint32_t splits);

// One-time kernel attribute set-up (large dynamic LDS opt-in); called when a
// library is created, so it never runs inside a stream capture.
bool prepare_decode_kernels();
bool prepare_prefill_kernels();
bool prepare_q4_kernels();
bool prepare_stack_kernels();

extern const KernelDesc kAttentionDecodeKernels[];
extern const uint32_t kAttentionDecodeKernelCount;
extern const KernelDesc kAttentionPrefillKernels[];
extern const uint32_t kAttentionPrefillKernelCount;
extern const KernelDesc kAttentionFamilyKernels[];
extern const uint32_t kAttentionFamilyKernelCount;
extern const KernelDesc kQ4ProjectKernels[];
extern const uint32_t kQ4ProjectKernelCount;
extern const KernelDesc kStackStepKernels[];
extern const uint32_t kStackStepKernelCount;
extern const KernelDesc kGdnDecodeKernels[];
extern const uint32_t kGdnDecodeKernelCount;
extern const KernelDesc kGdnPrefillKernels[];
extern const uint32_t kGdnPrefillKernelCount;

}  // namespace tt
