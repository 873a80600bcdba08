// Lane bookkeeping without a device: slot compatibility, admission errors that
// precede any encoding, ping-pong flags, the state-offset table formula and the
// reset state machine (reference tests/native/decode_state_slot_contract_test.cpp,
// state table src/runtime/decode_step.cpp:1037-1071).
#include "runtime.h"

#include <utility>

using namespace tatara::runtime;
using tatara::backend::hip::HipBlitPass;
using tatara::backend::hip::HipCommandError;
using tatara::backend::hip::HipComputePass;

namespace {
DecodeStateSlot slot_for(DecodeStep& step) {
    DecodeStateSlot slot;
    slot.capacity = step.capacity;
    slot.schedule_identity = step.schedule.data();
    slot.layers.resize(step.schedule.size());
    return slot;
}
}  // namespace

int main() {
    DecodeStep step;
    step.capacity = 128;
    step.schedule = {LayerKind::GatedDelta, LayerKind::FullAttention, LayerKind::GatedDelta};
    step.state = slot_for(step);
    DecodeStateSlot external = slot_for(step);
    if (!decode_state_slot_compatible(step, step.state) ||
        !decode_state_slot_compatible(step, external)) {
        return 1;
    }
    // available (flags clean) but not ready (no buffers)
    if (!decode_state_slot_available(step, external) || decode_state_slot_ready(step, external)) {
        return 2;
    }
    DecodeStateSlot wrong_capacity = slot_for(step);
    wrong_capacity.capacity = 127;
    if (decode_state_slot_compatible(step, wrong_capacity)) return 3;
    DecodeStateSlot wrong_count = slot_for(step);
    wrong_count.layers.pop_back();
    if (decode_state_slot_compatible(step, wrong_count)) return 4;
    DecodeStep other;
    other.capacity = step.capacity;
    other.schedule = step.schedule;
    DecodeStateSlot wrong_owner = slot_for(other);
    if (decode_state_slot_compatible(step, wrong_owner)) return 5;

    // a moved step keeps its schedule storage, so slots stay compatible
    DecodeStep moved = std::move(step);
    if (!decode_state_slot_compatible(moved, moved.state) ||
        !decode_state_slot_compatible(moved, external)) {
        return 6;
    }

    HipComputePass invalid_pass;
    DecodeBatchScratch scratch;
    scratch.rows = 1;
    std::vector<LayerWeights> weights(3);
    const LayerStageHooks hooks{};
    if (encode_token(moved, wrong_owner, scratch, weights, hooks, invalid_pass, 0) !=
        HipCommandError::StateSlotMismatch) {
        return 7;
    }
    if (encode_token(moved, external, scratch, weights, hooks, invalid_pass, moved.capacity) !=
        HipCommandError::ContextOutOfRange) {
        return 8;
    }
    // in range, but the slot has no buffers: not ready
    if (encode_token(moved, external, scratch, weights, hooks, invalid_pass, 0) !=
        HipCommandError::StateSlotMismatch) {
        return 9;
    }

    advance_decode_state(moved, external);
    if (!external.layers[0].swapped || external.layers[1].swapped || !external.layers[2].swapped) {
        return 10;
    }
    external.status = DecodeStateSlotStatus::SnapshotPending;
    external.active_transfer_generation = 1;
    if (decode_state_slot_available(moved, external)) return 11;
    advance_decode_state(moved, external);  // refused: flags unchanged
    if (!external.layers[0].swapped || external.layers[1].swapped || !external.layers[2].swapped) {
        return 12;
    }
    advance_decode_state(moved, wrong_owner);
    if (wrong_owner.layers[0].swapped || wrong_owner.layers[2].swapped) return 13;
    external.status = DecodeStateSlotStatus::Ready;
    external.active_transfer_generation = 0;
    advance_prefill_state(moved, external, 2);  // even chunk count: no flip
    if (!external.layers[0].swapped) return 14;
    advance_prefill_state(moved, external, 3);  // odd: flip GDN layers only
    if (external.layers[0].swapped || external.layers[1].swapped || external.layers[2].swapped) {
        return 15;
    }

    // state-offset table: only strides and flags matter
    DecodeStatePool pool;
    pool.stripes = 4;
    pool.layers.resize(3);
    pool.layers[0].first_stride = 49152;     // conv stripe bytes
    pool.layers[0].second_stride = 2097152;  // recurrent stripe bytes
    pool.layers[1].first_stride = 2ull * 128 * 256 * 2;
    pool.layers[1].second_stride = 2ull * 128 * 256 * 2;
    pool.layers[2].first_stride = 49152;
    pool.layers[2].second_stride = 2097152;
    DecodeStateSlot a = slot_for(moved), b = slot_for(moved);
    b.layers[0].swapped = true;  // lane b is one token ahead in layer 0 only
    const DecodeStream streams[2] = {{&a, 100, 3}, {&b, 7, 1}};
    StateOffsetTable table;
    if (build_state_offset_table(moved, streams, pool, table) != HipCommandError::None) return 20;
    if (table.words.size() != 3 * 64 + 16) return 21;
    const std::uint32_t conv = 49152 / 2, rec = 2097152 / 4;
    const std::uint32_t* l0 = table.words.data();
    // row 0: stripe 3, parity 0 -> in = 2*3, out = 2*3+1
    if (l0[0] != 6 * conv || l0[1] != 7 * conv || l0[2] != 6 * rec || l0[3] != 7 * rec) return 22;
    // row 1: stripe 1, parity 1 -> in = 2*1+1, out = 2*1
    if (l0[4] != 3 * conv || l0[5] != 2 * conv || l0[6] != 3 * rec || l0[7] != 2 * rec) return 23;
    const std::uint32_t* l1 = table.words.data() + 64;
    const std::uint32_t kv = 2 * 128 * 256;  // elements per attention stripe
    if (l1[0] != 3 * kv || l1[1] != 100 || l1[2] != 0 || l1[3] != 0) return 24;
    if (l1[4] != 1 * kv || l1[5] != 7) return 25;
    const std::uint32_t* l2 = table.words.data() + 128;
    if (l2[4] != 2 * conv || l2[5] != 3 * conv) return 26;  // layer 2 of lane b is not swapped
    // both contexts fit one 256-key partition -> both rows are bucket rows, in order
    if (table.bucket_rows != 2 || table.words[192] != 0 || table.words[193] != 1) return 27;
    const DecodeStream mixed[2] = {{&a, 100, 0}, {&b, 100, 0}};
    (void)mixed;
    moved.capacity = 100000;
    a.capacity = b.capacity = 100000;
    const DecodeStream long_rows[2] = {{&a, 300, 0}, {&b, 255, 1}};
    if (build_state_offset_table(moved, long_rows, pool, table) != HipCommandError::None) return 28;
    if (table.bucket_rows != 1 || table.words[192] != 1) return 29;
    const DecodeStream bad_stripe[1] = {{&a, 1, 4}};
    if (build_state_offset_table(moved, bad_stripe, pool, table) !=
        HipCommandError::InvalidStreamGroup) {
        return 30;
    }
    if (build_state_offset_table(moved, {}, pool, table) != HipCommandError::InvalidStreamGroup) {
        return 31;
    }

    // batched walk: admission errors come before anything touches the pass
    DecodeBatchScratch batch;
    batch.rows = 2;
    if (encode_token_batch(moved, long_rows, pool, batch, weights, hooks, invalid_pass) !=
        HipCommandError::InvalidStreamGroup) {  // no state_offsets buffer
        return 32;
    }

    // reset state machine without a device
    HipBlitPass invalid_blit;
    external.status = DecodeStateSlotStatus::Poisoned;
    if (encode_state_slot_reset(moved, external, invalid_blit).error !=
        StateSlotResetError::PoisonedStateSlot) {
        return 40;
    }
    external.status = DecodeStateSlotStatus::Ready;
    external.capacity = moved.capacity;
    if (encode_state_slot_reset(moved, external, invalid_blit).error !=
        StateSlotResetError::InvalidStateSlot) {  // no buffers: not complete
        return 41;
    }
    StateSlotResetTicket stale{&moved, &external, 4, 100, 9, true};
    if (complete_state_slot_reset(stale, moved, external) != StateSlotResetError::StaleTicket) {
        return 42;
    }
    StateSlotResetTicket done = stale;
    done.pending = false;
    if (complete_state_slot_reset(done, moved, external) != StateSlotResetError::AlreadyCompleted) {
        return 43;
    }
    return 0;
}
