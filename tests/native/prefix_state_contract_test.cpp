// The canonical prefix-state payload without a device: frozen byte totals of the
// 40-layer plan, a gap-free segment walk that allocates nothing, the live-plane
// routes, a family-major synthetic schedule carried through host byte planes,
// typed layout errors and the ticket state machine
// (reference tests/native/prefix_state_transfer_test.cpp:199-534).
#include "runtime.h"

#include <array>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <new>
#include <utility>
#include <vector>

namespace {
std::size_t allocations = 0;
bool counting = false;
}  // namespace

void* operator new(std::size_t size) {
    if (counting) ++allocations;
    if (void* memory = std::malloc(size ? size : 1)) return memory;
    throw std::bad_alloc();
}
void* operator new[](std::size_t size) { return ::operator new(size); }
void operator delete(void* memory) noexcept { std::free(memory); }
void operator delete[](void* memory) noexcept { std::free(memory); }
void operator delete(void* memory, std::size_t) noexcept { std::free(memory); }
void operator delete[](void* memory, std::size_t) noexcept { std::free(memory); }

using namespace tatara::runtime;
using tatara::backend::hip::HipBuffer;

namespace {

struct HostLayer {
    std::array<std::vector<std::byte>, 4> planes;  // first, first_out, second, second_out
    bool swapped{false};
};

std::vector<std::byte>& plane(HostLayer& layer, PrefixStateBufferPlane which) {
    switch (which) {
    case PrefixStateBufferPlane::First: return layer.planes[0];
    case PrefixStateBufferPlane::FirstOutput: return layer.planes[1];
    case PrefixStateBufferPlane::Second: return layer.planes[2];
    case PrefixStateBufferPlane::SecondOutput: return layer.planes[3];
    case PrefixStateBufferPlane::Arena: break;
    }
    std::abort();
}

std::vector<std::byte> gather(const PrefixStateLayout& layout, std::vector<HostLayer>& lane) {
    std::vector<std::byte> payload(layout.total_bytes);
    for (std::uint32_t i = 0; i < layout.segment_count; ++i) {
        const PrefixStateSegment s = prefix_state_segment(layout, i).segment;
        const PrefixStateCopyRoute route = prefix_state_copy_route(
            s, PrefixStateTransferDirection::Snapshot, lane[s.layer_index].swapped);
        std::memcpy(payload.data() + s.snapshot_offset_bytes,
                    plane(lane[s.layer_index], route.source).data() + s.slot_offset_bytes,
                    s.length_bytes);
    }
    return payload;
}

// snapshot -> restore into a lane full of other bytes -> snapshot again: same payload
bool payload_survives(const PrefixStateLayout& layout, bool source_swapped) {
    const std::size_t layers = layout.specification.schedule.size();
    constexpr std::size_t kPlane = 1216;  // 4 heads x 19 rows x 16 bytes
    std::vector<HostLayer> source(layers), target(layers);
    for (std::size_t l = 0; l < layers; ++l) {
        const bool gated = layout.specification.schedule[l] == LayerKind::GatedDelta;
        for (std::size_t p = 0; p < 4; ++p) {
            source[l].planes[p].resize(kPlane);
            target[l].planes[p].assign(kPlane, std::byte{0xcd});
            for (std::size_t b = 0; b < kPlane; ++b) {
                source[l].planes[p][b] = static_cast<std::byte>((29 * l + 53 * p + b) % 241);
            }
        }
        source[l].swapped = gated && source_swapped;
        target[l].swapped = gated;  // whatever phase the recipient was in
    }
    const std::vector<std::byte> taken = gather(layout, source);
    for (std::uint32_t i = 0; i < layout.segment_count; ++i) {
        const PrefixStateSegment s = prefix_state_segment(layout, i).segment;
        const PrefixStateCopyRoute route = prefix_state_copy_route(
            s, PrefixStateTransferDirection::Restore, target[s.layer_index].swapped);
        std::memcpy(plane(target[s.layer_index], route.destination).data() + s.slot_offset_bytes,
                    taken.data() + s.snapshot_offset_bytes, s.length_bytes);
    }
    for (std::size_t l = 0; l < layers; ++l) target[l].swapped = false;  // what completion does
    return gather(layout, target) == taken;
}

PrefixStateTransferTicket pending_ticket(PrefixStateTransferDirection direction, DecodeStep& decode,
                                         DecodeStateSlot& state, const HipBuffer& arena,
                                         std::uint64_t generation) {
    state.active_transfer_generation = generation;
    state.active_transfer_arena = &arena;
    state.active_transfer_positions = 4;
    state.active_transfer_offset_bytes = 16;
    state.active_transfer_state_bytes = 32;
    return {direction, &decode, &state, &arena, 4, 16, 32, generation, true};
}

}  // namespace

int main() {
    const auto plan = tatara::model::qwen36::qwen36_35b_a3b_plan();
    DecodeStep decode;
    decode.capacity = 16384;
    decode.geometry = make_decode_geometry(plan, decode.capacity);
    decode.schedule.assign(plan.layers.begin(), plan.layers.end());
    PrefillPolicy policy;
    policy.schedule = PrefillSchedule::LayerMajor;
    policy.context_capacity = decode.capacity;
    policy.maximum_block_rows = 2048;
    policy.first_chunk_rows = 256;
    policy.query_tile_rows = 256;
    policy.gdn_gate_hoist = true;
    const PrefillGeometryResult prefill = make_prefill_geometry(plan, policy);
    if (!prefill) return 1;

    const PrefixStateLayoutResult planned = make_prefix_state_layout(decode, prefill.geometry, 4096);
    if (!planned) return 2;
    const PrefixStateLayout& layout = planned.layout;
    if (layout.gated_delta_layers != 30 || layout.attention_layers != 10) return 3;
    if (layout.segment_count != 100) return 4;
    if (prefix_state_phase_evidence_bytes(decode.schedule) != 5) return 5;
    // frozen figures of the reference's own test (prefix_state_transfer_test.cpp:229-233)
    if (layout.total_bytes != 148'275'200ull) return 6;
    if (layout.attention_segment_bytes != 2'097'152ull) return 7;
    if (layout.attention_slot_head_stride_bytes != 8'388'608ull) return 8;

    {   // prefix_state_transfer_test.cpp:248-265
        DecodeStep wide;
        wide.capacity = 65536;
        wide.geometry = make_decode_geometry(plan, wide.capacity);
        wide.schedule.assign(plan.layers.begin(), plan.layers.end());
        PrefillPolicy wide_policy = policy;
        wide_policy.context_capacity = wide.capacity;
        const PrefillGeometryResult wide_prefill = make_prefill_geometry(plan, wide_policy);
        if (!wide_prefill) return 9;
        const std::pair<std::uint32_t, std::uint64_t> frozen[] = {
            {4096, 148'275'200ull},
            {49408, 1'076'264'960ull},
            {50000, 1'088'389'120ull},
            {65536, 1'406'566'400ull},
        };
        for (const auto& [positions, bytes] : frozen) {
            const auto made = make_prefix_state_layout(wide, wide_prefill.geometry, positions);
            if (!made || made.layout.segment_count != 100 || made.layout.total_bytes != bytes) {
                return 10;
            }
        }
        if (make_prefix_state_layout(wide, wide_prefill.geometry, 65537).error !=
            PrefixStateLayoutError::PositionOutOfRange) {
            return 11;
        }
        // a prefill geometry of another capacity does not describe this step's buffers
        if (make_prefix_state_layout(wide, prefill.geometry, 4096).error !=
            PrefixStateLayoutError::InvalidGeometry) {
            return 12;
        }
    }

    // gap-free walk in payload order; no allocation
    std::uint64_t cursor = 0;
    std::uint32_t gated_segments = 0, attention_segments = 0;
    counting = true;
    const std::size_t before = allocations;
    for (std::uint32_t i = 0; i < layout.segment_count; ++i) {
        const PrefixStateSegmentResult found = prefix_state_segment(layout, i);
        if (!found || found.segment.snapshot_offset_bytes != cursor) return 20;
        cursor += found.segment.length_bytes;
        const PrefixStateSegment& s = found.segment;
        const bool gated = s.kind == PrefixStateSegmentKind::GatedDeltaConvolution ||
                           s.kind == PrefixStateSegmentKind::GatedDeltaRecurrent;
        if ((decode.schedule[s.layer_index] == LayerKind::GatedDelta) != gated) return 21;
        if (gated) {
            ++gated_segments;
            const bool conv = s.kind == PrefixStateSegmentKind::GatedDeltaConvolution;
            const auto in_phase = prefix_state_copy_route(s, PrefixStateTransferDirection::Snapshot, false);
            const auto out_phase = prefix_state_copy_route(s, PrefixStateTransferDirection::Snapshot, true);
            const auto back = prefix_state_copy_route(s, PrefixStateTransferDirection::Restore, true);
            if (in_phase.source != (conv ? PrefixStateBufferPlane::First : PrefixStateBufferPlane::Second) ||
                out_phase.source != (conv ? PrefixStateBufferPlane::FirstOutput
                                          : PrefixStateBufferPlane::SecondOutput) ||
                in_phase.destination != PrefixStateBufferPlane::Arena ||
                back.source != PrefixStateBufferPlane::Arena ||
                back.destination != (conv ? PrefixStateBufferPlane::First : PrefixStateBufferPlane::Second)) {
                return 22;
            }
            if (s.slot_offset_bytes != 0 || s.length_bytes != (conv ? 49152u : 2097152u)) return 23;
        } else {
            ++attention_segments;
            const bool value = s.kind == PrefixStateSegmentKind::AttentionValue;
            const auto out = prefix_state_copy_route(s, PrefixStateTransferDirection::Snapshot, true);
            const auto back = prefix_state_copy_route(s, PrefixStateTransferDirection::Restore, true);
            const auto want = value ? PrefixStateBufferPlane::Second : PrefixStateBufferPlane::First;
            if (out.source != want || back.destination != want) return 24;  // no ping-pong for KV
        }
    }
    counting = false;
    if (allocations != before) return 25;
    if (cursor != layout.total_bytes || gated_segments != 60 || attention_segments != 40) return 26;

    const PrefixStateSegment key0 = prefix_state_segment(layout, 60).segment;
    const PrefixStateSegment key1 = prefix_state_segment(layout, 61).segment;
    const PrefixStateSegment value0 = prefix_state_segment(layout, 62).segment;
    if (key0.layer_index != 3 || key0.kind != PrefixStateSegmentKind::AttentionKey ||
        key0.head_index != 0 || key0.slot_offset_bytes != 0) {
        return 27;
    }
    if (key1.kind != PrefixStateSegmentKind::AttentionKey || key1.head_index != 1 ||
        key1.slot_offset_bytes != layout.attention_slot_head_stride_bytes) {
        return 28;
    }
    if (value0.kind != PrefixStateSegmentKind::AttentionValue || value0.head_index != 0 ||
        value0.layer_index != 3) {
        return 29;
    }
    if (prefix_state_segment(layout, 64).segment.layer_index != 7) return 30;

    if (validate_prefix_state_arena_extent(layout, 64, layout.total_bytes + 64) !=
            PrefixStateTransferError::None ||
        validate_prefix_state_arena_extent(layout, 64, layout.total_bytes + 63) !=
            PrefixStateTransferError::ArenaOutOfRange ||
        validate_prefix_state_arena_extent(layout, std::numeric_limits<std::uint64_t>::max(),
                                           std::numeric_limits<std::uint64_t>::max()) !=
            PrefixStateTransferError::ArenaOutOfRange ||
        validate_prefix_state_arena_extent(PrefixStateLayout{}, 0, 1024) !=
            PrefixStateTransferError::InvalidLayout) {
        return 31;
    }

    // a schedule that starts with attention: the payload is still family-major
    constexpr std::array<LayerKind, 4> kMixed{LayerKind::FullAttention, LayerKind::GatedDelta,
                                              LayerKind::FullAttention, LayerKind::GatedDelta};
    PrefixStateLayoutSpec spec;
    spec.schedule = kMixed;
    spec.capacity = 19;
    spec.positions = 7;
    spec.key_value_heads = 4;
    spec.head_dimension = 8;
    spec.expected_gated_delta_layers = 2;
    spec.expected_attention_layers = 2;
    spec.gated_delta_convolution_bytes = 24;
    spec.gated_delta_recurrent_bytes = 40;
    spec.expected_total_bytes = 1920;  // 2 x 64 + 2 x 8 x 7 x 16
    const PrefixStateLayoutResult mixed = make_prefix_state_layout(spec);
    if (!mixed || mixed.layout.segment_count != 20 || mixed.layout.total_bytes != 1920) return 40;
    if (prefix_state_segment(mixed.layout, 0).segment.layer_index != 1 ||
        prefix_state_segment(mixed.layout, 2).segment.layer_index != 3 ||
        prefix_state_segment(mixed.layout, 4).segment.layer_index != 0 ||
        prefix_state_segment(mixed.layout, 12).segment.layer_index != 2) {
        return 41;
    }
    if (!payload_survives(mixed.layout, false) || !payload_survives(mixed.layout, true)) return 42;

    PrefixStateLayoutSpec bad = spec;
    bad.positions = 0;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::PositionOutOfRange) return 43;
    bad = spec;
    bad.positions = 20;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::PositionOutOfRange) return 44;
    bad = spec;
    bad.expected_attention_layers = 3;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::FamilyCountMismatch) return 45;
    bad = spec;
    ++bad.expected_total_bytes;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::TotalMismatch) return 46;
    bad = spec;
    bad.gated_delta_convolution_bytes = std::numeric_limits<std::uint64_t>::max();
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::Overflow) return 47;
    constexpr std::array<LayerKind, 2> kUnknown{LayerKind::GatedDelta, static_cast<LayerKind>(255)};
    bad = spec;
    bad.schedule = kUnknown;
    bad.expected_gated_delta_layers = 1;
    bad.expected_attention_layers = 1;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::InvalidSchedule) return 48;
    bad = spec;
    bad.schedule = {};
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::InvalidSchedule) return 49;
    bad = spec;
    bad.head_dimension = 0;
    if (make_prefix_state_layout(bad).error != PrefixStateLayoutError::InvalidGeometry) return 50;
    if (prefix_state_segment(mixed.layout, mixed.layout.segment_count).error !=
        PrefixStateLayoutError::SegmentOutOfRange) {
        return 51;
    }

    // ---- phase evidence and tickets ------------------------------------------------
    DecodeStep small;
    small.capacity = 8;
    small.schedule = {LayerKind::GatedDelta, LayerKind::FullAttention};
    DecodeStateSlot lane;
    lane.capacity = small.capacity;
    lane.schedule_identity = small.schedule.data();
    lane.layers.resize(small.schedule.size());
    HipBuffer arena;  // never dereferenced by the state machine

    lane.layers[0].swapped = true;
    lane.layers[1].swapped = true;  // meaningless for attention: must not show
    std::array<std::byte, 1> evidence{std::byte{0xff}};
    if (capture_prefix_state_phase_evidence(small, lane, evidence) != PrefixStateTransferError::None ||
        evidence[0] != std::byte{1}) {
        return 60;
    }
    lane.layers[0].swapped = false;
    if (capture_prefix_state_phase_evidence(small, lane, evidence) != PrefixStateTransferError::None ||
        evidence[0] != std::byte{0}) {
        return 61;
    }
    if (capture_prefix_state_phase_evidence(small, lane, {}) !=
        PrefixStateTransferError::PhaseEvidenceTooSmall) {
        return 62;
    }
    lane.layers[1].swapped = false;

    // the slot has no buffers: every encode is refused before any command
    {
        tatara::backend::hip::HipBlitPass no_pass;
        PrefillGeometry none;
        const auto refused = encode_prefix_state_restore(small, lane, none, no_pass, arena, 0, 4);
        if (refused.error != PrefixStateTransferError::InvalidStateSlot || refused.ticket) return 63;
        lane.status = DecodeStateSlotStatus::Poisoned;
        if (encode_prefix_state_snapshot(small, lane, none, no_pass, arena, 0, 4, evidence).error !=
            PrefixStateTransferError::PoisonedStateSlot) {
            return 64;
        }
        lane.status = DecodeStateSlotStatus::Ready;
    }

    lane.layers[0].swapped = true;
    lane.status = DecodeStateSlotStatus::RestorePending;
    PrefixStateTransferTicket restore =
        pending_ticket(PrefixStateTransferDirection::Restore, small, lane, arena, 7);
    counting = true;
    const std::size_t before_complete = allocations;
    if (complete_prefix_state_transfer(restore, small, lane, arena) != PrefixStateTransferError::None) {
        return 70;
    }
    counting = false;
    if (allocations != before_complete) return 71;
    if (lane.status != DecodeStateSlotStatus::Ready || lane.active_transfer_generation != 0 ||
        lane.active_transfer_arena != nullptr || lane.active_transfer_positions != 0 ||
        lane.active_transfer_offset_bytes != 0 || lane.active_transfer_state_bytes != 0 ||
        lane.layers[0].swapped || restore.pending) {
        return 72;
    }
    if (complete_prefix_state_transfer(restore, small, lane, arena) !=
        PrefixStateTransferError::AlreadyCompleted) {
        return 73;
    }

    lane.layers[0].swapped = true;
    lane.status = DecodeStateSlotStatus::SnapshotPending;
    PrefixStateTransferTicket snapshot =
        pending_ticket(PrefixStateTransferDirection::Snapshot, small, lane, arena, 8);
    PrefixStateTransferTicket copy = snapshot;
    PrefixStateTransferTicket shifted = snapshot;
    ++shifted.arena_offset_bytes;
    HipBuffer other_arena;
    if (complete_prefix_state_transfer(shifted, small, lane, arena) !=
            PrefixStateTransferError::StaleTicket ||
        complete_prefix_state_transfer(snapshot, small, lane, other_arena) !=
            PrefixStateTransferError::StaleTicket) {
        return 74;
    }
    if (complete_prefix_state_transfer(snapshot, small, lane, arena) != PrefixStateTransferError::None ||
        !lane.layers[0].swapped) {  // a snapshot never changes the phase
        return 75;
    }
    if (complete_prefix_state_transfer(copy, small, lane, arena) !=
        PrefixStateTransferError::StaleTicket) {
        return 76;
    }

    lane.status = DecodeStateSlotStatus::SnapshotPending;
    PrefixStateTransferTicket dropped =
        pending_ticket(PrefixStateTransferDirection::Snapshot, small, lane, arena, 9);
    if (abort_prefix_state_transfer(dropped, small, lane, arena) != PrefixStateTransferError::None) {
        return 77;
    }
    if (lane.status != DecodeStateSlotStatus::Poisoned || lane.active_transfer_generation != 0) {
        return 78;
    }
    if (abort_prefix_state_transfer(dropped, small, lane, arena) !=
        PrefixStateTransferError::AlreadyCompleted) {
        return 79;
    }
    PrefixStateTransferTicket late =
        pending_ticket(PrefixStateTransferDirection::Restore, small, lane, arena, 10);
    if (complete_prefix_state_transfer(late, small, lane, arena) !=
        PrefixStateTransferError::PoisonedStateSlot) {
        return 80;
    }
    if (abort_prefix_state_transfer(late, small, lane, arena) !=
            PrefixStateTransferError::PoisonedStateSlot ||
        late.pending) {
        return 81;
    }
    return 0;
}
