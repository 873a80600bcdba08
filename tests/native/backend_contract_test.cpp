// Null handles give the reference's typed errors before any device call
// (pattern of tests/native/metal_resources_contract_test.cpp and
// metal_lifecycle_contract_test.cpp).  Runs without a GPU.
#include "backend_hip.h"

using namespace tatara::backend::hip;

int main() {
    HipDevice device;
    if (device) return 1;
    if (create_command_queue(device).error != HipResourceError::InvalidDevice) return 2;
    if (create_shared_buffer(device, 64).error != HipResourceError::InvalidDevice) return 3;
    if (create_striped_pool_buffer(device, 64, 2).error != HipResourceError::InvalidDevice) return 4;
    if (create_kernel_library(device).error != HipPipelineError::InvalidDevice) return 5;
    HipLibrary library;
    if (create_compute_pipeline(library, "attention_decode").error !=
        HipPipelineError::InvalidLibrary) {
        return 6;
    }
    HipBuffer buffer;
    if (buffer.size_bytes() != 0 || buffer.contents() != nullptr) return 7;
    if (create_buffer_window(buffer, 0, 16).error != HipResourceError::BufferWindowUnsupported) {
        return 8;
    }
    HipCommandQueue queue;
    if (create_command_buffer(queue).error != HipCommandError::InvalidCommandQueue) return 9;
    HipCommandBuffer cb;
    if (begin_compute_pass(std::move(cb)).error != HipCommandError::InvalidCommandBuffer) return 10;
    HipComputePass pass;
    HipComputePipeline pipeline;
    if (set_compute_pipeline(pass, pipeline) != HipCommandError::InvalidComputePass) return 11;
    if (set_buffer(pass, buffer, 0, 0) != HipCommandError::InvalidComputePass) return 12;
    const std::uint32_t word = 1;
    if (set_bytes(pass, &word, 4, 0) != HipCommandError::InvalidComputePass) return 13;
    if (dispatch_threadgroups(pass, {1, 1, 1}, {1, 1, 1}) != HipCommandError::InvalidComputePass) {
        return 14;
    }
    if (memory_barrier(pass) != HipCommandError::InvalidComputePass) return 15;
    if (end_compute_pass(std::move(pass)).error != HipCommandError::InvalidComputePass) return 16;
    HipBlitPass blit;
    if (fill_buffer(blit, buffer, 0, 1, std::byte{0}) != HipCommandError::InvalidBlitPass) return 17;
    if (copy_buffer(blit, buffer, 0, buffer, 0, 1) != HipCommandError::InvalidBlitPass) return 18;
    HipCommandBuffer cb2;
    if (commit(std::move(cb2)).error != HipCommandError::InvalidCommandBuffer) return 19;
    HipPendingExecution pending;
    const HipExecutionResult waited = wait_until_completed(std::move(pending));
    if (waited.error != HipCommandError::InvalidPendingExecution || waited) return 20;
    if (did_modify_range(buffer, 0, 1) != HipCommandError::InvalidBuffer) return 21;
    if (create_event(device).error != HipResourceError::InvalidDevice) return 23;
    HipEvent event;
    HipCommandBuffer cb3;
    if (encode_signal_event(cb3, event, 1) != HipCommandError::InvalidCommandBuffer) return 24;
    if (encode_wait_for_event(cb3, event, 1) != HipCommandError::InvalidCommandBuffer) return 25;
    // system device: either a device or the typed "unavailable" error, never a crash
    const HipDeviceResult made = create_system_device();
    if (!made && made.error != HipResourceError::SystemDeviceUnavailable) return 22;
    return 0;
}
