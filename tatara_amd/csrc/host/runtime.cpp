#include "runtime.h"

#include <algorithm>
#include <cstring>
#include <limits>

namespace tatara::model::qwen36 {

std::vector<LayerKind> make_hybrid_layer_schedule(std::size_t layer_count, std::size_t period,
                                                  std::size_t first) {
    std::vector<LayerKind> layers(layer_count, LayerKind::GatedDelta);
    if (period == 0) return layers;
    for (std::size_t index = first; index < layer_count; index += period) {
        layers[index] = LayerKind::FullAttention;
    }
    return layers;
}

ModelPlan qwen36_35b_a3b_plan() {
    return ModelPlan{
        .hidden = 2048,
        .vocabulary = 248320,
        .query_heads = 16,
        .key_value_heads = 2,
        .head_dimension = 256,
        .recurrent_heads = 32,
        .state_dimension = 128,
        .initial_serving_capacity = 16384,
        .layers = make_hybrid_layer_schedule(40, 4, 3),
    };
}

}  // namespace tatara::model::qwen36

namespace tatara::runtime {

using namespace backend::hip;

namespace {

bool is_gated(LayerKind kind) { return kind == LayerKind::GatedDelta; }

// Row counts shared by byte sizes and dispatch shapes (decode_geometry.h:188-203).
struct FamilyRows {
    std::uint32_t gdn_qk, gdn_values, gdn_conv, gdn_prepare, gdn_projection, attn_projection,
        attn_query;
};
FamilyRows family_rows(const model::qwen36::ModelPlan& plan) {
    FamilyRows r{};
    r.gdn_qk = 2u * (plan.recurrent_heads / 2u) * plan.state_dimension;
    r.gdn_values = plan.recurrent_heads * plan.state_dimension;
    r.gdn_conv = r.gdn_qk + r.gdn_values;
    r.gdn_prepare = r.gdn_conv + r.gdn_values;
    r.gdn_projection = r.gdn_prepare + 2u * plan.recurrent_heads;
    r.attn_projection = plan.query_heads * 2u * plan.head_dimension +
                        2u * plan.key_value_heads * plan.head_dimension;
    r.attn_query = plan.query_heads * plan.head_dimension;
    return r;
}

bool allocate_zeroed(const HipDevice& device, std::uint64_t bytes, HipBuffer& out) {
    // create_shared_buffer zero-fills the HBM allocation (zeroed-allocation rule,
    // decode_step.h:252-255), so no host memset is needed here.
    auto made = create_shared_buffer(device, bytes);
    if (!made) return false;
    out = std::move(*made.buffer);
    return true;
}

// Issues calls in order and latches the first error: once one is held every
// later call is skipped, so a rejected bind can never be followed by a recorded
// dispatch (decode_step.cpp:95-184).
struct Walk {
    HipComputePass& pass;
    HipCommandError error = HipCommandError::None;

    bool failed() const { return error != HipCommandError::None; }
    void check(HipCommandError result) {
        if (error == HipCommandError::None && result != HipCommandError::None) error = result;
    }
    void pipeline(const HipComputePipeline& p) {
        if (!failed()) check(set_compute_pipeline(pass, p));
    }
    void buffer(const HipBuffer& b, std::uint64_t offset, std::uint32_t index) {
        if (!failed()) check(set_buffer(pass, b, offset, index));
    }
    void weight(const HipBuffer* b, std::uint32_t index) {
        if (failed()) return;
        if (b == nullptr) {
            check(HipCommandError::InvalidBuffer);
            return;
        }
        check(set_buffer(pass, *b, 0, index));
    }
    void constant(std::uint32_t value, std::uint32_t index) {
        if (!failed()) check(set_bytes(pass, &value, sizeof(value), index));
    }
    void dispatch(HipSize groups, HipSize threads) {
        if (!failed()) check(dispatch_threadgroups(pass, groups, threads));
    }
    void dispatch(std::uint64_t gx, std::uint64_t tx, std::uint64_t gy = 1, std::uint64_t ty = 1,
                  std::uint64_t tz = 1) {
        dispatch(HipSize{gx, gy, 1}, HipSize{tx, ty, tz});
    }
    void barrier() {
        if (!failed()) check(memory_barrier(pass));
    }
    void hook(HipCommandError (*fn)(void*, HipComputePass&, std::size_t, LayerKind, std::uint32_t),
              void* user, std::size_t layer, LayerKind kind, std::uint32_t rows) {
        if (failed() || fn == nullptr) return;
        check(fn(user, pass, layer, kind, rows));
    }
};

HipCommandError stream_admissible(const DecodeStep& step, const DecodeStateSlot& state,
                                  std::uint32_t context) {
    if (!decode_state_slot_compatible(step, state)) return HipCommandError::StateSlotMismatch;
    if (!context_in_capacity(context, step.capacity)) return HipCommandError::ContextOutOfRange;
    if (!decode_state_slot_ready(step, state)) return HipCommandError::StateSlotMismatch;
    return HipCommandError::None;
}

template <typename Pipelines, typename Member>
bool resolve(const HipLibrary& library, Pipelines& out, Member member, const char* name,
             HipPipelineError& error) {
    auto made = create_compute_pipeline(library, name);
    if (!made) {
        error = made.error;
        return false;
    }
    out.*member = std::move(*made.pipeline);
    return true;
}

}  // namespace

DecodeGeometry make_decode_geometry(const model::qwen36::ModelPlan& plan, std::uint32_t capacity) {
    const FamilyRows rows = family_rows(plan);
    std::uint32_t gated = 0;
    std::uint32_t attention = 0;
    for (const LayerKind kind : plan.layers) (is_gated(kind) ? gated : attention) += 1;
    const std::uint32_t partitions = (capacity + kAttentionPartition - 1u) / kAttentionPartition;
    DecodeGeometry g{};
    g.gated_delta_layers = gated;
    g.attention_layers = attention;
    g.hidden_bytes = std::uint64_t{plan.hidden} * kBf16Bytes;
    g.layer_stream_bytes = plan.layers.size() * std::uint64_t{plan.hidden} * kBf16Bytes;
    g.gdn_projection_bytes = std::uint64_t{rows.gdn_projection} * kBf16Bytes;
    g.gdn_qk_bytes = std::uint64_t{rows.gdn_qk} * kBf16Bytes;
    g.gdn_value_bytes = std::uint64_t{rows.gdn_values} * kBf16Bytes;
    g.gdn_gate_bytes = g.gdn_value_bytes;
    g.gdn_conv_state_bytes = std::uint64_t{kConvShiftSteps} * rows.gdn_conv * kBf16Bytes;
    g.gdn_recurrent_state_bytes = std::uint64_t{plan.recurrent_heads} * plan.state_dimension *
                                  plan.state_dimension * kF32Bytes;
    g.attn_projection_bytes = std::uint64_t{rows.attn_projection} * kBf16Bytes;
    g.attn_query_bytes = std::uint64_t{rows.attn_query} * kBf16Bytes;
    g.attn_record_scratch_bytes =
        std::uint64_t{plan.query_heads} * partitions * kAttentionRecordFloats * kF32Bytes;
    g.attn_cache_bytes =
        std::uint64_t{plan.key_value_heads} * capacity * plan.head_dimension * kBf16Bytes;
    g.gdn_prepare = {rows.gdn_prepare / plan.state_dimension, plan.state_dimension};
    g.gdn_recurrence = {plan.state_dimension / 4u, plan.recurrent_heads, 32u, 4u};
    g.gdn_gate_norm = {plan.recurrent_heads, plan.state_dimension};
    g.attn_qk_rope = {plan.query_heads + plan.key_value_heads, plan.head_dimension};
    g.attention_head = {plan.query_heads, plan.head_dimension};
    g.attention_split = {plan.query_heads / 4u,
                         kAttentionPartition,
                         4u,
                         plan.key_value_heads,
                         32u,
                         plan.head_dimension / 64u,
                         plan.query_heads / plan.key_value_heads};
    g.rms = {1u, plan.hidden / 4u};
    return g;
}

std::uint32_t attention_partitions(std::uint32_t context) {
    const std::uint32_t count = context + 1;
    return count <= kAttentionPartition ? 1u
                                        : (count + kAttentionPartition - 1) / kAttentionPartition;
}

std::uint32_t split_workgroups(std::span<const std::uint32_t> visible_keys,
                               std::uint32_t split_keys) noexcept {
    // the rule lives in the backend library, one implementation for every caller
    return tt_split_workgroups(visible_keys.data(), static_cast<std::uint32_t>(visible_keys.size()),
                               split_keys);
}

std::uint32_t choose_split_keys(std::span<const std::uint32_t> visible_keys,
                                std::uint32_t compute_units) noexcept {
    return tt_choose_split_keys(visible_keys.data(), static_cast<std::uint32_t>(visible_keys.size()),
                                compute_units);
}

std::uint32_t choose_split_keys(std::uint32_t rows, std::uint32_t keys,
                                std::uint32_t compute_units) noexcept {
    const std::array<std::uint32_t, kMaximumBatchRows> same = [&] {
        std::array<std::uint32_t, kMaximumBatchRows> v{};
        v.fill(keys);
        return v;
    }();
    const std::size_t count = std::clamp<std::size_t>(rows, 1, same.size());
    return choose_split_keys(std::span<const std::uint32_t>(same.data(), count), compute_units);
}

DecodePipelinesResult resolve_decode_pipelines(const HipLibrary& library) {
    DecodePipelines p;
    HipPipelineError error = HipPipelineError::None;
    using P = DecodePipelines;
    const bool ok =
        resolve(library, p, &P::gdn_prepare, "gdn_prepare", error) &&
        resolve(library, p, &P::gdn_recurrence, "gdn_recurrence", error) &&
        resolve(library, p, &P::gdn_gate_norm, "gdn_gate_norm", error) &&
        resolve(library, p, &P::attn_qk_rope, "attn_qk_rope", error) &&
        resolve(library, p, &P::attention_decode, "attention_decode", error) &&
        resolve(library, p, &P::attention_scores_values_fused,
                "attention_decode_scores_values_gqa8", error) &&
        resolve(library, p, &P::attention_combine, "attention_decode_combine", error) &&
        resolve(library, p, &P::gdn_prepare_ms, "gdn_prepare_ms", error) &&
        resolve(library, p, &P::gdn_recurrence_ms, "gdn_recurrence_ms", error) &&
        resolve(library, p, &P::gate_norm_ms, "gdn_gate_norm_ms", error) &&
        resolve(library, p, &P::gdn_decode_fused_ms, "gdn_decode_fused_ms", error) &&
        resolve(library, p, &P::attn_qk_rope_ms, "attn_qk_rope_ms", error) &&
        resolve(library, p, &P::attention_decode_ms, "attention_decode_ms", error) &&
        resolve(library, p, &P::attention_split_ms, "attention_decode_split_ms", error) &&
        resolve(library, p, &P::attention_combine_ms, "attention_decode_combine_ms", error) &&
        resolve(library, p, &P::attention_token_ms, "attention_decode_token_ms", error) &&
        resolve(library, p, &P::attention_token_finish_ms, "attention_decode_token_finish_ms",
                error);
    if (!ok) return {error, std::nullopt};
    return {HipPipelineError::None, std::move(p)};
}

namespace {

DecodeStateSlotResult allocate_state_slot(const HipDevice& device, const DecodeGeometry& geometry,
                                          std::uint32_t capacity,
                                          std::span<const LayerKind> schedule,
                                          const LayerKind* schedule_identity) {
    if (!device) return {DecodeStepError::InvalidDevice, std::nullopt};
    if (capacity == 0 || schedule.empty() || schedule_identity == nullptr) {
        return {DecodeStepError::OffsetCountMismatch, std::nullopt};
    }
    DecodeStateSlot slot;
    slot.capacity = capacity;
    slot.schedule_identity = schedule_identity;
    slot.layers.reserve(schedule.size());
    for (const LayerKind kind : schedule) {
        DecodeLayerState state;
        const bool gated = is_gated(kind);
        const std::uint64_t first = gated ? geometry.gdn_conv_state_bytes : geometry.attn_cache_bytes;
        const std::uint64_t second =
            gated ? geometry.gdn_recurrent_state_bytes : geometry.attn_cache_bytes;
        if (!allocate_zeroed(device, first, state.first) ||
            !allocate_zeroed(device, second, state.second) ||
            (gated && (!allocate_zeroed(device, first, state.first_out) ||
                       !allocate_zeroed(device, second, state.second_out)))) {
            return {DecodeStepError::BufferAllocationFailed, std::nullopt};
        }
        slot.layers.push_back(std::move(state));
    }
    return {DecodeStepError::None, std::move(slot)};
}

}  // namespace

DecodeStepResult create_decode_step(const HipDevice& device, const DecodeGeometry& geometry,
                                    std::uint32_t capacity, std::span<const LayerKind> schedule,
                                    DecodePipelines pipelines) {
    if (!device) return {DecodeStepError::InvalidDevice, std::nullopt};
    if (schedule.empty() || capacity == 0) return {DecodeStepError::OffsetCountMismatch, std::nullopt};
    DecodeStep step;
    step.geometry = geometry;
    step.capacity = capacity;
    step.schedule.assign(schedule.begin(), schedule.end());
    step.pipelines = std::move(pipelines);
    auto state = allocate_state_slot(device, geometry, capacity, step.schedule, step.schedule.data());
    if (!state) return {state.error, std::nullopt};
    step.state = std::move(*state.slot);
    return {DecodeStepError::None, std::move(step)};
}

DecodeStateSlotResult create_decode_state_slot(const HipDevice& device, const DecodeStep& step) {
    return allocate_state_slot(device, step.geometry, step.capacity, step.schedule,
                               step.schedule.data());
}

namespace {

// What one layer of one lane keeps on the device.  Both layer kinds hold two buffers: `first`
// (conv history | keys) and `second` (recurrent state | values); a Gated DeltaNet layer holds
// each as a ping-pong pair of planes, an attention layer as a single plane.  Everything that
// walks a slot's buffers (pool carving, completeness) goes through this table.
struct LayerFootprint {
    std::uint64_t bytes[2];   // [0] first, [1] second
    std::uint32_t planes;     // 1 or 2 planes of each
};

LayerFootprint footprint_of(const DecodeGeometry& g, LayerKind kind) noexcept {
    if (is_gated(kind)) return {{g.gdn_conv_state_bytes, g.gdn_recurrent_state_bytes}, 2};
    return {{g.attn_cache_bytes, g.attn_cache_bytes}, 1};
}

// plane p of buffer b of a layer's state: [b][p]
HipBuffer DecodeLayerState::*const kPlaneOf[2][2] = {
    {&DecodeLayerState::first, &DecodeLayerState::first_out},
    {&DecodeLayerState::second, &DecodeLayerState::second_out},
};

}  // namespace

// One striped pool per layer and buffer (decode_step.cpp:460-540): slot s owns stripes
// planes * s .. planes * s + planes - 1, so a state table addresses a lane's planes as
// (planes * stripe + plane) * stride.  The slots' buffers are windows into the pools.
DecodeStateSlotPoolResult create_decode_state_slot_pool(const HipDevice& device,
                                                        const DecodeStep& step,
                                                        std::uint32_t count) {
    DecodeStateSlotPoolResult result{DecodeStepError::None, std::nullopt, {}};
    if (!device) {
        result.error = DecodeStepError::InvalidDevice;
        return result;
    }
    if (count == 0 || step.capacity == 0 || step.schedule.empty()) {
        result.error = DecodeStepError::OffsetCountMismatch;
        return result;
    }
    // state-table offsets are u32 element counts of at least two bytes (decode_step.cpp:476)
    constexpr std::uint64_t kAddressableBytes = 0xffffffffull * 2;
    DecodeStatePool pool;
    pool.stripes = count;
    std::vector<DecodeStateSlot> slots(count);
    for (DecodeStateSlot& slot : slots) {
        slot.capacity = step.capacity;
        slot.schedule_identity = step.schedule.data();
        slot.layers.resize(step.schedule.size());
    }
    bool ok = true;
    for (std::size_t index = 0; ok && index < step.schedule.size(); ++index) {
        const LayerFootprint shape = footprint_of(step.geometry, step.schedule[index]);
        DecodeStatePoolLayer layer;
        HipBuffer DecodeStatePoolLayer::*const pools[2] = {&DecodeStatePoolLayer::first,
                                                           &DecodeStatePoolLayer::second};
        std::uint64_t DecodeStatePoolLayer::*const strides[2] = {
            &DecodeStatePoolLayer::first_stride, &DecodeStatePoolLayer::second_stride};
        for (std::uint32_t b = 0; ok && b < 2; ++b) {
            auto striped = create_striped_pool_buffer(device, shape.bytes[b], shape.planes * count);
            ok = striped && striped.buffer->size_bytes() <= kAddressableBytes;
            if (!ok) break;
            layer.*pools[b] = std::move(*striped.buffer);
            layer.*strides[b] = striped.stripe_stride_bytes;
            for (std::uint32_t slot = 0; ok && slot < count; ++slot) {
                for (std::uint32_t plane = 0; ok && plane < shape.planes; ++plane) {
                    const std::uint64_t stripe = std::uint64_t{slot} * shape.planes + plane;
                    auto window = create_buffer_window(layer.*pools[b], stripe * (layer.*strides[b]),
                                                       shape.bytes[b]);
                    ok = static_cast<bool>(window);
                    if (ok) slots[slot].layers[index].*kPlaneOf[b][plane] = std::move(*window.buffer);
                }
            }
        }
        pool.layers.push_back(std::move(layer));
    }
    if (!ok) {
        result.error = DecodeStepError::BufferAllocationFailed;
        return result;
    }
    result.pool = std::move(pool);
    result.slots = std::move(slots);
    return result;
}

DecodeBatchScratchResult create_decode_batch_scratch(const HipDevice& device,
                                                     const DecodeStep& step, std::uint32_t rows) {
    if (rows == 0 || rows > kMaximumBatchRows) {
        return {DecodeStepError::OffsetCountMismatch, std::nullopt};
    }
    const DecodeGeometry& g = step.geometry;
    DecodeBatchScratch b;
    b.rows = rows;
    const std::uint64_t table_bytes = step.schedule.size() * 16 * 4 * 4 + 64;
    // split records down to the finest split choose_split_keys picks (128 keys); the
    // geometry's own figure is for the reference's 256-key partitions
    const std::uint64_t finest_splits = (std::uint64_t{step.capacity} + 127) / 128;
    const std::uint64_t record_bytes =
        std::max<std::uint64_t>(g.attn_record_scratch_bytes,
                                16 * finest_splits * kAttentionRecordFloats * kF32Bytes) * rows;
    if (!allocate_zeroed(device, rows * g.gdn_projection_bytes, b.gdn_projection) ||
        !allocate_zeroed(device, rows * g.gdn_qk_bytes, b.gdn_qk) ||
        !allocate_zeroed(device, rows * g.gdn_value_bytes, b.gdn_value) ||
        !allocate_zeroed(device, rows * g.gdn_gate_bytes, b.gdn_z) ||
        !allocate_zeroed(device, rows * g.gdn_value_bytes, b.gdn_y) ||
        !allocate_zeroed(device, rows * g.gdn_value_bytes, b.gdn_gated) ||
        !allocate_zeroed(device, rows * g.attn_projection_bytes, b.attn_projection) ||
        !allocate_zeroed(device, rows * g.attn_query_bytes, b.attn_query) ||
        !allocate_zeroed(device, rows * g.attn_query_bytes, b.attn_gate) ||
        !allocate_zeroed(device, rows * g.attn_query_bytes, b.attn_attended) ||
        !allocate_zeroed(device, record_bytes, b.attn_partials) ||
        !allocate_zeroed(device, table_bytes, b.state_offsets)) {
        return {DecodeStepError::BufferAllocationFailed, std::nullopt};
    }
    b.compute_units = std::max<std::uint32_t>(device.compute_units(), 1);
    return {DecodeStepError::None, std::move(b)};
}

// Slot predicates (decode_step.cpp:577-618), each the conjunction of the one before and one
// more condition: compatible (same step, same shape) -> available (idle and Ready) -> ready
// (every plane the schedule needs is there and large enough).
bool decode_state_slot_compatible(const DecodeStep& step, const DecodeStateSlot& state) noexcept {
    const bool same_step = state.schedule_identity == step.schedule.data();
    const bool same_shape =
        state.capacity == step.capacity && state.layers.size() == step.schedule.size();
    return step.capacity != 0 && same_step && same_shape;
}

bool decode_state_slot_complete(const DecodeStep& step, const DecodeStateSlot& state) noexcept {
    if (!decode_state_slot_compatible(step, state)) return false;
    for (std::size_t index = 0; index < step.schedule.size(); ++index) {
        const LayerFootprint shape = footprint_of(step.geometry, step.schedule[index]);
        for (std::uint32_t b = 0; b < 2; ++b) {
            for (std::uint32_t plane = 0; plane < shape.planes; ++plane) {
                const HipBuffer& buffer = state.layers[index].*kPlaneOf[b][plane];
                if (!buffer || buffer.size_bytes() < shape.bytes[b]) return false;
            }
        }
    }
    return true;
}

bool decode_state_slot_available(const DecodeStep& step, const DecodeStateSlot& state) noexcept {
    const bool idle = state.active_transfer_generation == 0 && state.active_reset_generation == 0 &&
                      state.active_reset_segments == 0 && state.active_reset_bytes == 0;
    return decode_state_slot_compatible(step, state) &&
           state.status == DecodeStateSlotStatus::Ready && idle;
}

bool decode_state_slot_ready(const DecodeStep& step, const DecodeStateSlot& state) noexcept {
    return decode_state_slot_available(step, state) && decode_state_slot_complete(step, state);
}

HipCommandError build_state_offset_table(const DecodeStep& step,
                                         std::span<const DecodeStream> streams,
                                         const DecodeStatePool& pool, StateOffsetTable& out) {
    const std::size_t layers = step.schedule.size();
    const std::uint32_t rows = static_cast<std::uint32_t>(streams.size());
    if (rows == 0 || rows > kMaximumBatchRows || pool.layers.size() != layers ||
        pool.stripes == 0) {
        return HipCommandError::InvalidStreamGroup;
    }
    out.words.assign(layers * 64 + 16, 0u);
    for (std::size_t layer = 0; layer < layers; ++layer) {
        const DecodeStatePoolLayer& pool_layer = pool.layers[layer];
        const bool gated = is_gated(step.schedule[layer]);
        for (std::uint32_t r = 0; r < rows; ++r) {
            if (streams[r].state == nullptr || streams[r].stripe >= pool.stripes ||
                streams[r].state->layers.size() != layers) {
                return HipCommandError::InvalidStreamGroup;
            }
            const std::uint32_t stripe = streams[r].stripe;
            std::uint32_t* entry = out.words.data() + layer * 64 + std::size_t{r} * 4;
            if (gated) {
                const auto conv_elems = static_cast<std::uint32_t>(pool_layer.first_stride / 2);
                const auto rec_elems = static_cast<std::uint32_t>(pool_layer.second_stride / 4);
                const std::uint32_t parity = streams[r].state->layers[layer].swapped ? 1u : 0u;
                entry[0] = (2u * stripe + parity) * conv_elems;
                entry[1] = (2u * stripe + 1u - parity) * conv_elems;
                entry[2] = (2u * stripe + parity) * rec_elems;
                entry[3] = (2u * stripe + 1u - parity) * rec_elems;
            } else {
                entry[0] = stripe * static_cast<std::uint32_t>(pool_layer.first_stride / 2);
                entry[1] = streams[r].context;
            }
        }
    }
    out.bucket_rows = 0;
    for (std::uint32_t r = 0; r < rows; ++r) {
        if (attention_partitions(streams[r].context) == 1) {
            out.words[layers * 64 + out.bucket_rows] = r;
            ++out.bucket_rows;
        }
    }
    return HipCommandError::None;
}

HipCommandError encode_token_batch(DecodeStep& step, std::span<const DecodeStream> streams,
                                   const DecodeStatePool& pool, DecodeBatchScratch& batch,
                                   std::span<const LayerWeights> weights,
                                   const LayerStageHooks& hooks, HipComputePass& pass) {
    const std::uint32_t rows = static_cast<std::uint32_t>(streams.size());
    if (rows == 0 || rows > batch.rows || rows > kMaximumBatchRows ||
        pool.layers.size() != step.schedule.size() || pool.stripes == 0 || !batch.state_offsets ||
        weights.size() != step.schedule.size() || batch.split_keys % 32u != 0) {
        return HipCommandError::InvalidStreamGroup;
    }
    for (std::size_t index = 0; index < streams.size(); ++index) {
        if (streams[index].state == nullptr || streams[index].stripe >= pool.stripes) {
            return HipCommandError::InvalidStreamGroup;
        }
        const HipCommandError admissible =
            stream_admissible(step, *streams[index].state, streams[index].context);
        if (admissible != HipCommandError::None) return admissible;
        for (std::size_t other = 0; other < index; ++other) {
            if (streams[other].state == streams[index].state) {
                return HipCommandError::InvalidStreamGroup;
            }
        }
    }
    StateOffsetTable table;
    const HipCommandError built = build_state_offset_table(step, streams, pool, table);
    if (built != HipCommandError::None) return built;
    void* host = batch.state_offsets.contents();
    const std::uint64_t table_bytes = table.words.size() * sizeof(std::uint32_t);
    if (host == nullptr || batch.state_offsets.size_bytes() < table_bytes) {
        return HipCommandError::InvalidBuffer;
    }
    std::memcpy(host, table.words.data(), table_bytes);
    const HipCommandError published = did_modify_range(batch.state_offsets, 0, table_bytes);
    if (published != HipCommandError::None) return published;

    const DecodeGeometry& g = step.geometry;
    const std::uint64_t bucket_offset = step.schedule.size() * 256;
    // Which rows take the split path: those with more than one 256-key partition - or, in the
    // token form, every row (its walk covers the cached keys only, the token itself is folded
    // in by the finishing dispatch).
    const bool token_form = batch.attention_token_form;
    bool any_long = false;
    for (const DecodeStream& s : streams) any_long |= attention_partitions(s.context) != 1;
    // Keys per split-K workgroup: chosen from the depths of the rows that take the split
    // path, but no finer than 4096 workgroups over the capacity.  The grid always covers the
    // capacity (the operator reads the contexts on the device and refuses a grid that could
    // miss keys); where that leaves workgroups without keys in a grid larger than the chip,
    // the ones with keys are placed first in the dispatch order (bit 2 of the flags).
    std::array<std::uint32_t, kMaximumBatchRows> visible{};
    std::size_t long_rows = 0;
    std::uint32_t deepest = 0;
    for (const DecodeStream& s : streams) {
        const bool splits = token_form ? s.context != 0 : attention_partitions(s.context) != 1;
        if (splits && long_rows < visible.size()) {
            visible[long_rows++] = token_form ? s.context : s.context + 1;
            deepest = std::max(deepest, visible[long_rows - 1]);
        }
    }
    const std::span<const std::uint32_t> long_keys(visible.data(), long_rows);
    const std::uint32_t units = std::max<std::uint32_t>(batch.compute_units, 1);
    std::uint32_t split_keys = batch.split_keys;
    if (split_keys == 0) {
        const std::uint64_t coarsest =
            ((std::uint64_t{step.capacity} * 2 * rows + 4095) / 4096 + 31) / 32 * 32;
        split_keys = std::max(choose_split_keys(long_keys, units),
                              static_cast<std::uint32_t>(std::min<std::uint64_t>(coarsest, 1u << 30)));
    }
    const std::uint32_t max_splits = (step.capacity + split_keys - 1) / split_keys;
    if ((any_long || token_form) &&
        batch.attn_partials.size_bytes() <
            std::uint64_t{rows} * 16 * max_splits * kAttentionRecordFloats * kF32Bytes) {
        return HipCommandError::InvalidBuffer;
    }
    // Flags of the split-K walk.  Bit 1: waves of one or two lanes deal a lane's 32-key
    // blocks to its workgroups in turn (measured 1-3 % faster there, 3 % slower at four
    // lanes).  Bit 2: the grid is larger than the chip and part of it holds no keys, so the
    // workgroups that do go first (0.4 us dearer than the order by grid position where that
    // is not so).  Bits 3..7: workgroups that take consecutive ranges start a rotated number
    // of blocks into them, so that the stride between ranges - the cache capacity - does
    // not decide how their requests of the moment fall on the memory channels (the same
    // 4 x 32768 keys took 46-77 us over capacities 32768 ... 131136 without, 46-48 us with).
    const std::uint64_t grid_groups = std::uint64_t{max_splits} * 2 * rows;
    const bool keyless_between =
        grid_groups > units && grid_groups > split_workgroups(long_keys, split_keys);
    const bool in_turn = rows <= 2;
    const std::uint32_t walk_flags = (in_turn ? 2u : 8u) | (keyless_between ? 4u : 0u);
    Walk walk{pass};
    const DecodePipelines& k = step.pipelines;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        const LayerKind kind = step.schedule[layer];
        const LayerWeights& w = weights[layer];
        walk.barrier();
        walk.hook(hooks.project, hooks.user, layer, kind, rows);
        walk.barrier();
        if (is_gated(kind) && batch.gdn_fused) {
            walk.pipeline(k.gdn_decode_fused_ms);
            walk.buffer(batch.gdn_projection, 0, 0);
            walk.buffer(pool.layers[layer].first, 0, 1);
            walk.weight(w.conv_weight, 2);
            walk.weight(w.a_log, 3);
            walk.weight(w.dt_bias, 4);
            walk.buffer(pool.layers[layer].second, 0, 5);
            walk.weight(w.norm_weight, 6);
            walk.buffer(batch.gdn_gated, 0, 7);
            walk.buffer(batch.state_offsets, layer * 256, 8);
            walk.constant(static_cast<std::uint32_t>(g.gdn_projection_bytes / 2), 9);
            walk.constant(static_cast<std::uint32_t>(g.gdn_value_bytes / 2), 10);
            walk.dispatch(HipSize{g.gdn_recurrence.head_groups, rows, 1}, HipSize{512, 1, 1});
        } else if (is_gated(kind)) {
            walk.pipeline(k.gdn_prepare_ms);
            walk.buffer(batch.gdn_projection, 0, 0);
            walk.buffer(pool.layers[layer].first, 0, 1);
            walk.weight(w.conv_weight, 2);
            walk.buffer(batch.gdn_qk, 0, 3);
            walk.buffer(batch.gdn_value, 0, 4);
            walk.buffer(batch.gdn_z, 0, 5);
            walk.buffer(batch.state_offsets, layer * 256, 6);
            walk.constant(static_cast<std::uint32_t>(g.gdn_projection_bytes / 2), 7);
            walk.constant(static_cast<std::uint32_t>(g.gdn_qk_bytes / 2), 8);
            walk.constant(static_cast<std::uint32_t>(g.gdn_value_bytes / 2), 9);
            walk.constant(static_cast<std::uint32_t>(g.gdn_gate_bytes / 2), 10);
            walk.dispatch(g.gdn_prepare.groups, g.gdn_prepare.threads, rows);
            walk.barrier();
            walk.pipeline(k.gdn_recurrence_ms);
            walk.buffer(batch.gdn_qk, 0, 0);
            walk.buffer(batch.gdn_value, 0, 1);
            walk.buffer(batch.gdn_projection, 0, 2);
            walk.weight(w.a_log, 3);
            walk.weight(w.dt_bias, 4);
            walk.buffer(pool.layers[layer].second, 0, 5);
            walk.buffer(batch.gdn_y, 0, 6);
            walk.buffer(batch.state_offsets, layer * 256, 7);
            walk.constant(static_cast<std::uint32_t>(g.gdn_qk_bytes / 2), 8);
            walk.constant(static_cast<std::uint32_t>(g.gdn_value_bytes / 2), 9);
            walk.constant(static_cast<std::uint32_t>(g.gdn_projection_bytes / 2), 10);
            walk.constant(static_cast<std::uint32_t>(g.gdn_value_bytes / 2), 11);
            walk.constant(g.gdn_recurrence.head_groups, 12);
            walk.dispatch(HipSize{1, g.gdn_recurrence.dimension_groups,
                                  std::uint64_t{g.gdn_recurrence.head_groups} * rows},
                          HipSize{g.gdn_recurrence.lane_threads,
                                  g.gdn_recurrence.dimension_threads, 1});
            walk.barrier();
            walk.pipeline(k.gate_norm_ms);
            walk.buffer(batch.gdn_y, 0, 0);
            walk.buffer(batch.gdn_z, 0, 1);
            walk.weight(w.norm_weight, 2);
            walk.buffer(batch.gdn_gated, 0, 3);
            walk.constant(static_cast<std::uint32_t>(g.gdn_value_bytes / 2), 4);
            walk.dispatch(g.gdn_gate_norm.groups, g.gdn_gate_norm.threads, rows);
        } else if (token_form) {
            for (const bool finishing : {false, true}) {
                if (finishing) walk.barrier();
                walk.pipeline(finishing ? k.attention_token_finish_ms : k.attention_token_ms);
                walk.buffer(batch.attn_projection, 0, 0);
                walk.weight(w.query_norm, 1);
                walk.weight(w.key_norm, 2);
                walk.buffer(pool.layers[layer].first, 0, 3);
                walk.buffer(pool.layers[layer].second, 0, 4);
                walk.buffer(batch.state_offsets, layer * 256, 5);
                walk.buffer(batch.attn_partials, 0, 6);
                walk.buffer(batch.attn_attended, 0, 7);
                walk.constant(step.capacity, 8);
                walk.constant(static_cast<std::uint32_t>(g.attn_projection_bytes / 2), 9);
                walk.constant(static_cast<std::uint32_t>(g.attn_query_bytes / 2), 10);
                walk.constant(split_keys, 11);
                walk.constant(max_splits, 12);
                walk.constant(walk_flags, 13);
                walk.constant((deepest + split_keys - 1) / split_keys, 14);
                if (finishing) {
                    walk.dispatch(g.attention_head.groups, g.attention_head.threads, rows);
                } else {
                    walk.dispatch(HipSize{max_splits, 2, rows}, HipSize{256, 1, 1});
                }
            }
        } else {
            walk.pipeline(k.attn_qk_rope_ms);
            walk.buffer(batch.attn_projection, 0, 0);
            walk.weight(w.query_norm, 1);
            walk.weight(w.key_norm, 2);
            walk.buffer(batch.attn_query, 0, 3);
            walk.buffer(batch.attn_gate, 0, 4);
            walk.buffer(pool.layers[layer].first, 0, 5);
            walk.buffer(pool.layers[layer].second, 0, 6);
            walk.constant(step.capacity, 7);
            walk.buffer(batch.state_offsets, layer * 256, 8);
            walk.constant(static_cast<std::uint32_t>(g.attn_projection_bytes / 2), 9);
            walk.constant(static_cast<std::uint32_t>(g.attn_query_bytes / 2), 10);
            walk.dispatch(g.attn_qk_rope.groups, g.attn_qk_rope.threads, rows);
            walk.barrier();
            if (any_long) {
                // every long row of the batch in one split-K grid + one combine
                walk.pipeline(k.attention_split_ms);
                walk.buffer(batch.attn_query, 0, 0);
                walk.buffer(pool.layers[layer].first, 0, 1);
                walk.buffer(pool.layers[layer].second, 0, 2);
                walk.buffer(batch.state_offsets, layer * 256, 3);
                walk.buffer(batch.attn_partials, 0, 4);
                walk.constant(step.capacity, 5);
                walk.constant(static_cast<std::uint32_t>(g.attn_query_bytes / 2), 6);
                walk.constant(split_keys, 7);
                walk.constant(max_splits, 8);
                // bit 0: short rows are left to the single-partition operator
                walk.constant(1u | walk_flags, 9);
                walk.dispatch(HipSize{max_splits, 2, rows}, HipSize{256, 1, 1});
                walk.barrier();
                walk.pipeline(k.attention_combine_ms);
                walk.buffer(batch.attn_partials, 0, 0);
                walk.buffer(batch.attn_gate, 0, 1);
                walk.buffer(batch.state_offsets, layer * 256, 2);
                walk.buffer(batch.attn_attended, 0, 3);
                walk.constant(split_keys, 4);
                walk.constant(max_splits, 5);
                walk.constant(static_cast<std::uint32_t>(g.attn_query_bytes / 2), 6);
                walk.constant(1u, 7);
                walk.constant(step.capacity, 8);
                walk.dispatch(g.attention_head.groups, g.attention_head.threads, rows);
            }
            if (table.bucket_rows != 0) {
                walk.pipeline(k.attention_decode_ms);
                walk.buffer(batch.attn_query, 0, 0);
                walk.buffer(batch.attn_gate, 0, 1);
                walk.buffer(pool.layers[layer].first, 0, 2);
                walk.buffer(pool.layers[layer].second, 0, 3);
                walk.buffer(batch.state_offsets, layer * 256, 4);
                walk.buffer(batch.attn_attended, 0, 5);
                walk.constant(step.capacity, 6);
                walk.buffer(batch.state_offsets, bucket_offset, 7);
                walk.constant(static_cast<std::uint32_t>(g.attn_query_bytes / 2), 8);
                walk.dispatch(g.attention_head.groups, g.attention_head.threads, table.bucket_rows);
            }
        }
        walk.barrier();
        walk.hook(hooks.finish, hooks.user, layer, kind, rows);
    }
    return walk.error;
}

HipCommandError encode_token(DecodeStep& step, DecodeStateSlot& state, DecodeBatchScratch& scratch,
                             std::span<const LayerWeights> weights, const LayerStageHooks& hooks,
                             HipComputePass& pass, std::uint32_t context) {
    const HipCommandError admissible = stream_admissible(step, state, context);
    if (admissible != HipCommandError::None) return admissible;
    if (weights.size() != step.schedule.size() || scratch.rows == 0) {
        return HipCommandError::InvalidStreamGroup;
    }
    const DecodeGeometry& g = step.geometry;
    const DecodePipelines& k = step.pipelines;
    Walk walk{pass};
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        const LayerKind kind = step.schedule[layer];
        const LayerWeights& w = weights[layer];
        DecodeLayerState& s = state.layers[layer];
        walk.barrier();
        walk.hook(hooks.project, hooks.user, layer, kind, 1);
        walk.barrier();
        if (is_gated(kind)) {
            const HipBuffer& conv_in = s.swapped ? s.first_out : s.first;
            const HipBuffer& conv_out = s.swapped ? s.first : s.first_out;
            const HipBuffer& rec_in = s.swapped ? s.second_out : s.second;
            const HipBuffer& rec_out = s.swapped ? s.second : s.second_out;
            walk.pipeline(k.gdn_prepare);
            walk.buffer(scratch.gdn_projection, 0, 0);
            walk.buffer(conv_in, 0, 1);
            walk.weight(w.conv_weight, 2);
            walk.buffer(scratch.gdn_qk, 0, 3);
            walk.buffer(scratch.gdn_value, 0, 4);
            walk.buffer(scratch.gdn_z, 0, 5);
            walk.buffer(conv_out, 0, 6);
            walk.dispatch(g.gdn_prepare.groups, g.gdn_prepare.threads);
            walk.barrier();
            walk.pipeline(k.gdn_recurrence);
            walk.buffer(scratch.gdn_qk, 0, 0);
            walk.buffer(scratch.gdn_value, 0, 1);
            walk.buffer(scratch.gdn_projection, 0, 2);
            walk.weight(w.a_log, 3);
            walk.weight(w.dt_bias, 4);
            walk.buffer(rec_in, 0, 5);
            walk.buffer(scratch.gdn_y, 0, 6);
            walk.buffer(rec_out, 0, 7);
            walk.dispatch(HipSize{1, g.gdn_recurrence.dimension_groups, g.gdn_recurrence.head_groups},
                          HipSize{g.gdn_recurrence.lane_threads, g.gdn_recurrence.dimension_threads,
                                  1});
            walk.barrier();
            walk.pipeline(k.gdn_gate_norm);
            walk.buffer(scratch.gdn_y, 0, 0);
            walk.buffer(scratch.gdn_z, 0, 1);
            walk.weight(w.norm_weight, 2);
            walk.buffer(scratch.gdn_gated, 0, 3);
            walk.dispatch(g.gdn_gate_norm.groups, g.gdn_gate_norm.threads);
        } else {
            walk.pipeline(k.attn_qk_rope);
            walk.buffer(scratch.attn_projection, 0, 0);
            walk.weight(w.query_norm, 1);
            walk.weight(w.key_norm, 2);
            walk.buffer(scratch.attn_query, 0, 3);
            walk.buffer(scratch.attn_gate, 0, 4);
            walk.buffer(s.first, 0, 5);
            walk.buffer(s.second, 0, 6);
            walk.constant(context, 7);
            walk.constant(step.capacity, 8);
            walk.dispatch(g.attn_qk_rope.groups, g.attn_qk_rope.threads);
            walk.barrier();
            const std::uint32_t partitions = attention_partitions(context);
            if (partitions == 1) {
                walk.pipeline(k.attention_decode);
                walk.buffer(scratch.attn_query, 0, 0);
                walk.buffer(scratch.attn_gate, 0, 1);
                walk.buffer(s.first, 0, 2);
                walk.buffer(s.second, 0, 3);
                walk.constant(context, 4);
                walk.buffer(scratch.attn_attended, 0, 5);
                walk.constant(step.capacity, 6);
                walk.dispatch(g.attention_head.groups, g.attention_head.threads);
            } else {
                walk.pipeline(k.attention_scores_values_fused);
                walk.buffer(scratch.attn_query, 0, 0);
                walk.buffer(s.first, 0, 1);
                walk.buffer(s.second, 0, 2);
                walk.constant(context, 3);
                walk.constant(step.capacity, 4);
                walk.constant(kAttentionPartition, 5);
                walk.buffer(scratch.attn_partials, 0, 6);
                walk.constant(partitions, 7);
                walk.dispatch(g.attention_split.value_groups, g.attention_split.score_threads,
                              partitions, g.attention_split.score_cohort_threads);
                walk.barrier();
                walk.pipeline(k.attention_combine);
                walk.buffer(scratch.attn_partials, 0, 0);
                walk.buffer(scratch.attn_gate, 0, 1);
                walk.constant(partitions, 2);
                walk.buffer(scratch.attn_attended, 0, 3);
                walk.dispatch(g.attention_head.groups, g.attention_head.threads);
            }
        }
        walk.barrier();
        walk.hook(hooks.finish, hooks.user, layer, kind, 1);
    }
    return walk.error;
}

// ---- the stages either side of the family, from the model's 4-bit weights ----
StagePipelinesResult resolve_stage_pipelines(const HipLibrary& library) {
    StagePipelines p;
    HipPipelineError error = HipPipelineError::None;
    using P = StagePipelines;
    const bool ok =
        resolve(library, p, &P::rms_ms, "rms_only_ms", error) &&
        resolve(library, p, &P::residual_rms_ms, "residual_rms_ms", error) &&
        resolve(library, p, &P::gdn_project_ms, "gdn_project_ms", error) &&
        resolve(library, p, &P::attn_project_ms, "attn_project_ms", error) &&
        resolve(library, p, &P::gdn_outproj_ms, "gdn_outproj_ms", error) &&
        resolve(library, p, &P::gdn_project_mfma_ms, "gdn_project_mfma_ms", error) &&
        resolve(library, p, &P::attn_project_mfma_ms, "attn_project_mfma_ms", error) &&
        resolve(library, p, &P::gdn_outproj_mfma_ms, "gdn_outproj_mfma_ms", error);
    if (!ok) return {error, std::nullopt};
    return {HipPipelineError::None, std::move(p)};
}

HiddenStreamsResult create_hidden_streams(const HipDevice& device, const DecodeGeometry& geometry,
                                          std::uint32_t rows) {
    if (rows == 0 || rows > kMaximumBatchRows) {
        return {DecodeStepError::OffsetCountMismatch, std::nullopt};
    }
    HiddenStreams h;
    h.rows = rows;
    const std::uint64_t bytes = rows * geometry.hidden_bytes;
    if (!allocate_zeroed(device, bytes, h.input) || !allocate_zeroed(device, bytes, h.normed) ||
        !allocate_zeroed(device, bytes, h.branch) || !allocate_zeroed(device, bytes, h.residual)) {
        return {DecodeStepError::BufferAllocationFailed, std::nullopt};
    }
    return {DecodeStepError::None, std::move(h)};
}

namespace {

// decode_geometry.h:147-148: one 32-lane group per output row, four (two) groups
// to a workgroup of the input (output) projections.
constexpr std::uint32_t kProjectionThreads = 128;
constexpr std::uint32_t kOutProjectionThreads = 64;

void bind_quantized(Walk& walk, const QuantizedBinding& q, std::uint32_t first) {
    walk.weight(q.weight, first);
    walk.weight(q.scales, first + 1);
    walk.weight(q.biases, first + 2);
}

bool stages_usable(const QuantizedLayerStages& s, std::size_t layer, LayerKind kind,
                   std::uint32_t rows) {
    return s.pipelines != nullptr && s.geometry != nullptr && s.scratch != nullptr &&
           s.streams != nullptr && layer < s.layers.size() && layer < s.schedule.size() &&
           s.schedule[layer] == kind && rows >= 1 && rows <= s.scratch->rows &&
           rows <= s.streams->rows && s.row_tile >= 1 && s.row_tile <= kMaximumBatchRows;
}

const HipBuffer& layer_input(const QuantizedLayerStages& s, std::size_t layer) {
    return layer != 0 && s.residual_feeds_next ? s.streams->residual : s.streams->input;
}

HipCommandError project_hook(void* user, HipComputePass& pass, std::size_t layer, LayerKind kind,
                             std::uint32_t rows) {
    return static_cast<const QuantizedLayerStages*>(user)->encode_project(pass, layer, kind, rows);
}
HipCommandError finish_hook(void* user, HipComputePass& pass, std::size_t layer, LayerKind kind,
                            std::uint32_t rows) {
    return static_cast<const QuantizedLayerStages*>(user)->encode_finish(pass, layer, kind, rows);
}

}  // namespace

LayerStageHooks QuantizedLayerStages::hooks() { return {this, &project_hook, &finish_hook}; }

HipCommandError QuantizedLayerStages::encode_project(HipComputePass& pass, std::size_t layer,
                                                     LayerKind kind, std::uint32_t rows) const {
    if (!stages_usable(*this, layer, kind, rows)) return HipCommandError::InvalidStreamGroup;
    const DecodeGeometry& g = *geometry;
    const StagePipelines& k = *pipelines;
    const LayerBindings& bound = layers[layer];
    const std::uint32_t hidden = static_cast<std::uint32_t>(g.hidden_bytes / 2);
    const std::uint32_t tiles = (rows + row_tile - 1) / row_tile;
    const bool wide = matrix_unit && rows >= 2;
    Walk walk{pass};
    walk.pipeline(k.rms_ms);
    walk.buffer(layer_input(*this, layer), 0, 0);
    walk.weight(bound.input_norm, 1);
    walk.buffer(streams->normed, 0, 2);
    walk.constant(hidden, 3);
    walk.constant(hidden, 4);
    walk.dispatch(HipSize{g.rms.groups, rows, 1}, HipSize{g.rms.threads, 1, 1});
    walk.barrier();
    if (is_gated(kind)) {
        const std::uint32_t out_rows = static_cast<std::uint32_t>(g.gdn_projection_bytes / 2);
        walk.pipeline(wide ? k.gdn_project_mfma_ms : k.gdn_project_ms);
        walk.buffer(streams->normed, 0, 0);
        bind_quantized(walk, bound.gated_delta.qkv, 1);
        bind_quantized(walk, bound.gated_delta.z, 4);
        bind_quantized(walk, bound.gated_delta.b, 7);
        bind_quantized(walk, bound.gated_delta.a, 10);
        walk.buffer(scratch->gdn_projection, 0, 13);
        walk.constant(rows, 14);
        walk.constant(row_tile, 15);
        walk.dispatch(HipSize{(out_rows + 3) / 4, tiles, 1}, HipSize{kProjectionThreads, 1, 1});
    } else {
        const std::uint32_t out_rows = static_cast<std::uint32_t>(g.attn_projection_bytes / 2);
        walk.pipeline(wide ? k.attn_project_mfma_ms : k.attn_project_ms);
        walk.buffer(streams->normed, 0, 0);
        bind_quantized(walk, bound.attention.query, 1);
        bind_quantized(walk, bound.attention.key, 4);
        bind_quantized(walk, bound.attention.value, 7);
        walk.buffer(scratch->attn_projection, 0, 10);
        walk.constant(rows, 11);
        walk.constant(row_tile, 12);
        walk.dispatch(HipSize{(out_rows + 3) / 4, tiles, 1}, HipSize{kProjectionThreads, 1, 1});
    }
    return walk.error;
}

HipCommandError QuantizedLayerStages::encode_finish(HipComputePass& pass, std::size_t layer,
                                                    LayerKind kind, std::uint32_t rows) const {
    if (!stages_usable(*this, layer, kind, rows)) return HipCommandError::InvalidStreamGroup;
    const DecodeGeometry& g = *geometry;
    const StagePipelines& k = *pipelines;
    const LayerBindings& bound = layers[layer];
    const std::uint32_t hidden = static_cast<std::uint32_t>(g.hidden_bytes / 2);
    const std::uint32_t tiles = (rows + row_tile - 1) / row_tile;
    const bool wide = matrix_unit && rows >= 2;
    Walk walk{pass};
    walk.barrier();
    walk.pipeline(wide ? k.gdn_outproj_mfma_ms : k.gdn_outproj_ms);
    walk.buffer(is_gated(kind) ? scratch->gdn_gated : scratch->attn_attended, 0, 0);
    bind_quantized(walk, is_gated(kind) ? bound.gated_delta.out : bound.attention.out, 1);
    walk.buffer(streams->branch, 0, 4);
    walk.constant(rows, 5);
    walk.constant(hidden, 6);
    walk.constant(row_tile, 7);
    walk.dispatch(HipSize{hidden / 2, tiles, 1}, HipSize{kOutProjectionThreads, 1, 1});
    walk.barrier();
    walk.pipeline(k.residual_rms_ms);
    walk.buffer(layer_input(*this, layer), 0, 0);
    walk.buffer(streams->branch, 0, 1);
    walk.buffer(streams->residual, 0, 2);
    walk.weight(bound.post_norm, 3);
    walk.buffer(streams->normed, 0, 4);
    walk.constant(hidden, 5);
    walk.constant(hidden, 6);
    walk.constant(hidden, 7);
    walk.dispatch(HipSize{g.rms.groups, rows, 1}, HipSize{g.rms.threads, 1, 1});
    return walk.error;
}

BlockStagePipelinesResult resolve_block_stage_pipelines(const HipLibrary& library) {
    BlockStagePipelines p;
    HipPipelineError error = HipPipelineError::None;
    using P = BlockStagePipelines;
    const bool ok = resolve(library, p, &P::rms, "rms_only_ms", error) &&
                    resolve(library, p, &P::residual_rms, "residual_rms_ms", error) &&
                    resolve(library, p, &P::gdn_project, "gdn_project_blk", error) &&
                    resolve(library, p, &P::attn_project, "attn_project_blk", error) &&
                    resolve(library, p, &P::out_projection, "outproj_blk", error);
    if (!ok) return {error, std::nullopt};
    return {HipPipelineError::None, std::move(p)};
}

BlockStreamsResult create_block_streams(const HipDevice& device, const PrefillGeometry& geometry,
                                        std::uint32_t hidden) {
    const std::uint32_t rows = geometry.policy.maximum_block_rows;
    // the norm kernels hold four values per thread of one workgroup
    if (rows == 0 || hidden == 0 || hidden % 128 != 0 || hidden > 4096) {
        return {DecodeStepError::OffsetCountMismatch, std::nullopt};
    }
    BlockStreams b;
    b.block_rows = rows;
    b.hidden = hidden;
    const std::uint64_t bytes = std::uint64_t{rows} * hidden * kBf16Bytes;
    if (!allocate_zeroed(device, bytes, b.normalized) || !allocate_zeroed(device, bytes, b.branch) ||
        !allocate_zeroed(device, bytes, b.block_hidden)) {
        return {DecodeStepError::BufferAllocationFailed, std::nullopt};
    }
    return {DecodeStepError::None, std::move(b)};
}

namespace {

bool block_stage_usable(const PrefillScratch& scratch, const BlockStreams& streams,
                        const PrefillChunk& chunk) {
    return chunk.rows >= 1 && chunk.rows <= scratch.block_rows && chunk.rows <= streams.block_rows &&
           streams.hidden != 0;
}

}  // namespace

HipCommandError encode_prefill_layer_input(const BlockStagePipelines& pipelines,
                                           const PrefillGeometry& geometry, PrefillScratch& scratch,
                                           BlockStreams& streams, const LayerBindings& bindings,
                                           LayerKind kind, const PrefillChunk& chunk,
                                           const HipBuffer& input, std::uint64_t input_offset,
                                           HipComputePass& pass) {
    if (!block_stage_usable(scratch, streams, chunk)) return HipCommandError::InvalidDispatchExtent;
    Walk walk{pass};
    walk.barrier();
    walk.pipeline(pipelines.rms);
    walk.buffer(input, input_offset, 0);
    walk.weight(bindings.input_norm, 1);
    walk.buffer(streams.normalized, 0, 2);
    walk.constant(streams.hidden, 3);
    walk.constant(streams.hidden, 4);
    walk.dispatch(HipSize{1, chunk.rows, 1}, HipSize{streams.hidden / 4, 1, 1});
    walk.barrier();
    if (is_gated(kind)) {
        walk.pipeline(pipelines.gdn_project);
        walk.buffer(streams.normalized, 0, 0);
        bind_quantized(walk, bindings.gated_delta.qkv, 1);
        bind_quantized(walk, bindings.gated_delta.z, 4);
        bind_quantized(walk, bindings.gated_delta.b, 7);
        bind_quantized(walk, bindings.gated_delta.a, 10);
        walk.buffer(scratch.gdn_projection, 0, 13);
        walk.constant(chunk.rows, 14);
        walk.dispatch(HipSize{(geometry.gdn_projection_rows + 3) / 4, 1, 1},
                      HipSize{kProjectionThreads, 1, 1});
    } else {
        walk.pipeline(pipelines.attn_project);
        walk.buffer(streams.normalized, 0, 0);
        bind_quantized(walk, bindings.attention.query, 1);
        bind_quantized(walk, bindings.attention.key, 4);
        bind_quantized(walk, bindings.attention.value, 7);
        walk.buffer(scratch.attn_projection, 0, 10);
        walk.constant(chunk.rows, 11);
        walk.dispatch(HipSize{(geometry.attention_projection_rows + 3) / 4, 1, 1},
                      HipSize{kProjectionThreads, 1, 1});
    }
    walk.barrier();
    return walk.error;
}

HipCommandError encode_prefill_layer_output(const BlockStagePipelines& pipelines,
                                            const PrefillGeometry& geometry, PrefillScratch& scratch,
                                            BlockStreams& streams, const LayerBindings& bindings,
                                            LayerKind kind, const PrefillChunk& chunk,
                                            const HipBuffer& input, std::uint64_t input_offset,
                                            HipComputePass& pass) {
    if (!block_stage_usable(scratch, streams, chunk)) return HipCommandError::InvalidDispatchExtent;
    Walk walk{pass};
    walk.barrier();
    walk.pipeline(pipelines.out_projection);
    walk.buffer(is_gated(kind) ? scratch.gdn_gated : scratch.attn_attended, 0, 0);
    bind_quantized(walk, is_gated(kind) ? bindings.gated_delta.out : bindings.attention.out, 1);
    walk.buffer(streams.branch, 0, 4);
    walk.constant(chunk.rows, 5);
    walk.constant(is_gated(kind) ? geometry.gdn_value_values : geometry.attention_vector_values, 6);
    walk.dispatch(HipSize{streams.hidden / 2, 1, 1}, HipSize{kOutProjectionThreads, 1, 1});
    walk.barrier();
    walk.pipeline(pipelines.residual_rms);
    walk.buffer(input, input_offset, 0);
    walk.buffer(streams.branch, 0, 1);
    walk.buffer(streams.block_hidden, 0, 2);
    walk.weight(bindings.post_norm, 3);
    walk.buffer(streams.normalized, 0, 4);
    walk.constant(streams.hidden, 5);
    walk.constant(streams.hidden, 6);
    walk.constant(streams.hidden, 7);
    walk.dispatch(HipSize{1, chunk.rows, 1}, HipSize{streams.hidden / 4, 1, 1});
    walk.barrier();
    return walk.error;
}

void advance_decode_state(const DecodeStep& step, DecodeStateSlot& state) {
    if (!decode_state_slot_available(step, state)) return;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (is_gated(step.schedule[layer])) {
            state.layers[layer].swapped = !state.layers[layer].swapped;
        }
    }
}

void advance_decode_state(DecodeStep& step) { advance_decode_state(step, step.state); }

void advance_prefill_state(const DecodeStep& step, DecodeStateSlot& state, std::uint32_t chunks) {
    if (!decode_state_slot_available(step, state)) return;
    if ((chunks & 1u) == 0u) return;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (is_gated(step.schedule[layer])) {
            state.layers[layer].swapped = !state.layers[layer].swapped;
        }
    }
}

StateSlotResetResult encode_state_slot_reset(const DecodeStep& step, DecodeStateSlot& state,
                                             HipBlitPass& blit_pass) noexcept {
    const auto failure = [](StateSlotResetError error,
                            HipCommandError command = HipCommandError::None) {
        return StateSlotResetResult{error, command, 0, 0, std::nullopt};
    };
    if (state.status == DecodeStateSlotStatus::Poisoned) {
        return failure(StateSlotResetError::PoisonedStateSlot);
    }
    if (!decode_state_slot_compatible(step, state) || !decode_state_slot_complete(step, state)) {
        return failure(StateSlotResetError::InvalidStateSlot);
    }
    if (!decode_state_slot_ready(step, state)) return failure(StateSlotResetError::StateSlotNotReady);
    if (state.next_reset_generation == 0) return failure(StateSlotResetError::GenerationExhausted);
    if (!blit_pass) {
        return failure(StateSlotResetError::CommandEncodingFailed, HipCommandError::InvalidBlitPass);
    }
    std::uint32_t segments = 0;
    std::uint64_t bytes = 0;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (!is_gated(step.schedule[layer])) continue;
        DecodeLayerState& s = state.layers[layer];
        // only the two live-capable planes that hold carried state need zeroing
        // at the canonical phase: first/second (state_slot_reset.cpp:265-286)
        HipBuffer* planes[2] = {&s.first, &s.second};
        const std::uint64_t lengths[2] = {step.geometry.gdn_conv_state_bytes,
                                          step.geometry.gdn_recurrent_state_bytes};
        for (int p = 0; p < 2; ++p) {
            const HipCommandError command =
                fill_buffer(blit_pass, *planes[p], 0, lengths[p], std::byte{0});
            if (command != HipCommandError::None) {
                state.status = DecodeStateSlotStatus::Poisoned;
                state.active_reset_generation = 0;
                state.active_reset_segments = 0;
                state.active_reset_bytes = 0;
                return failure(StateSlotResetError::CommandEncodingFailed, command);
            }
            ++segments;
            bytes += lengths[p];
        }
    }
    const std::uint64_t generation = state.next_reset_generation;
    state.next_reset_generation =
        generation == std::numeric_limits<std::uint64_t>::max() ? 0 : generation + 1u;
    state.active_reset_generation = generation;
    state.active_reset_segments = segments;
    state.active_reset_bytes = bytes;
    state.status = DecodeStateSlotStatus::ResetPending;
    return StateSlotResetResult{
        StateSlotResetError::None, HipCommandError::None, segments, bytes,
        StateSlotResetTicket{&step, &state, segments, bytes, generation, true}};
}

StateSlotResetError complete_state_slot_reset(StateSlotResetTicket& ticket, const DecodeStep& step,
                                              DecodeStateSlot& state) noexcept {
    if (!ticket.pending) return StateSlotResetError::AlreadyCompleted;
    if (state.status == DecodeStateSlotStatus::Poisoned) return StateSlotResetError::PoisonedStateSlot;
    if (ticket.owner != &step || ticket.state_owner != &state ||
        state.status != DecodeStateSlotStatus::ResetPending ||
        ticket.generation != state.active_reset_generation ||
        ticket.segment_count != state.active_reset_segments ||
        ticket.state_bytes != state.active_reset_bytes) {
        return StateSlotResetError::StaleTicket;
    }
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (is_gated(step.schedule[layer])) state.layers[layer].swapped = false;
    }
    state.active_reset_generation = 0;
    state.active_reset_segments = 0;
    state.active_reset_bytes = 0;
    state.status = DecodeStateSlotStatus::Ready;
    ticket.pending = false;
    return StateSlotResetError::None;
}

// ------------------------------------------------------------ block prefill --

namespace {
PrefillRequestValidation validate_common(const PrefillPolicy& policy, std::uint32_t live_context,
                                         std::uint32_t context_base,
                                         std::span<const std::uint32_t> tokens,
                                         std::uint32_t vocabulary, bool bounded_block) noexcept {
    if (tokens.empty()) return {PrefillRequestError::EmptyPrefix, 0};
    if (bounded_block && tokens.size() > policy.maximum_block_rows) {
        return {PrefillRequestError::BlockOutOfRange, 0};
    }
    if (context_base != live_context || context_base > policy.context_capacity) {
        return {PrefillRequestError::ContextOutOfRange, 0};
    }
    if (tokens.size() > policy.context_capacity - context_base) {
        return {PrefillRequestError::ContextOverflow, 0};
    }
    for (const std::uint32_t token : tokens) {
        if (token >= vocabulary) return {PrefillRequestError::TokenOutOfRange, 0};
    }
    return {PrefillRequestError::None, context_base + static_cast<std::uint32_t>(tokens.size())};
}

bool mul(std::uint64_t a, std::uint64_t b, std::uint64_t& out) {
    if (a != 0 && b > std::numeric_limits<std::uint64_t>::max() / a) return false;
    out = a * b;
    return true;
}
}  // namespace

PrefillRequestValidation validate_prefill_request(const PrefillPolicy& policy,
                                                  std::uint32_t live_context,
                                                  std::uint32_t context_base,
                                                  std::span<const std::uint32_t> tokens,
                                                  std::uint32_t vocabulary) noexcept {
    return validate_common(policy, live_context, context_base, tokens, vocabulary, true);
}

PrefillRequestValidation validate_prefill_prefix(const PrefillPolicy& policy,
                                                 std::uint32_t live_context,
                                                 std::uint32_t context_base,
                                                 std::span<const std::uint32_t> tokens,
                                                 std::uint32_t vocabulary) noexcept {
    return validate_common(policy, live_context, context_base, tokens, vocabulary, false);
}

PrefillGeometryResult make_prefill_geometry(const model::qwen36::ModelPlan& plan,
                                            const PrefillPolicy& policy) {
    if (plan.layers.empty() || plan.hidden == 0 || plan.vocabulary == 0 || plan.query_heads == 0 ||
        plan.key_value_heads == 0 || plan.query_heads % plan.key_value_heads != 0 ||
        plan.query_heads / plan.key_value_heads != 8 || plan.head_dimension != kAttentionPartition ||
        plan.recurrent_heads == 0 || plan.recurrent_heads % 2 != 0 || plan.state_dimension != 128) {
        return {PrefillGeometryError::InvalidPlan, {}};
    }
    if ((policy.schedule != PrefillSchedule::ChunkMajor &&
         policy.schedule != PrefillSchedule::LayerMajor) ||
        policy.context_capacity == 0 || policy.context_capacity > kPrefillMaximumContext ||
        policy.maximum_block_rows == 0 || policy.maximum_block_rows > kPrefillMaximumBlockRows ||
        policy.first_chunk_rows == 0 || policy.first_chunk_rows > policy.maximum_block_rows ||
        policy.query_tile_rows == 0 || policy.query_tile_rows > policy.maximum_block_rows ||
        policy.query_tile_rows % kPrefillQueryTileMultiple != 0 ||
        policy.attention_partition != kAttentionPartition ||
        (policy.gdn_tape && (!policy.gdn_gate_hoist || policy.gdn_chunked ||
                             plan.layers.size() > kGdnTapeLayers))) {
        return {PrefillGeometryError::InvalidPolicy, {}};
    }
    PrefillGeometry g;
    g.policy = policy;
    for (const LayerKind kind : plan.layers) {
        (is_gated(kind) ? g.gated_delta_layers : g.attention_layers) += 1;
    }
    if (g.gated_delta_layers == 0 || g.attention_layers == 0) {
        return {PrefillGeometryError::InvalidPlan, {}};
    }
    const FamilyRows rows = family_rows(plan);
    const std::uint64_t block = policy.maximum_block_rows;
    const std::uint64_t capacity = policy.context_capacity;
    g.attention_partitions =
        (policy.context_capacity + policy.attention_partition - 1u) / policy.attention_partition;
    g.key_value_heads = plan.key_value_heads;
    g.attention_head_dimension = plan.head_dimension;
    g.gdn_projection_rows = rows.gdn_projection;
    g.gdn_qk_values = rows.gdn_qk;
    g.gdn_value_values = rows.gdn_values;
    g.attention_projection_rows = rows.attn_projection;
    g.attention_vector_values = rows.attn_query;
    g.gdn_projection_bytes = block * rows.gdn_projection * kBf16Bytes;
    g.gdn_qk_bytes = block * rows.gdn_qk * kBf16Bytes;
    g.gdn_value_bytes = block * rows.gdn_values * kBf16Bytes;
    g.gdn_parameter_bytes = (policy.gdn_gate_hoist || policy.gdn_chunked)
                                ? block * plan.recurrent_heads * kF32Bytes
                                : 0;
    g.gdn_chunk_bytes = policy.gdn_chunked ? ((std::min<std::uint64_t>(block, kGdnChunkGroupRows) +
                                               kGdnChunkRows - 1u) / kGdnChunkRows) *
                                                 plan.recurrent_heads * kGdnChunkRecordBytes
                                           : 0;
    g.gdn_tape_bytes = policy.gdn_tape ? kGdnTapeBytes : 0;
    g.gdn_conv_tape_bytes = policy.gdn_tape ? kGdnConvTapeBytes : 0;
    g.attention_projection_bytes = block * rows.attn_projection * kBf16Bytes;
    g.attention_vector_bytes = block * rows.attn_query * kBf16Bytes;
    std::uint64_t records = 0;
    if (!mul(std::uint64_t{plan.query_heads} * policy.query_tile_rows, g.attention_partitions,
             records) ||
        !mul(records, (plan.head_dimension + 2u) * std::uint64_t{kF32Bytes},
             g.attention_partial_bytes)) {
        return {PrefillGeometryError::Overflow, {}};
    }
    const std::uint64_t conv = std::uint64_t{kConvShiftSteps} * rows.gdn_conv * kBf16Bytes;
    const std::uint64_t recurrent = std::uint64_t{plan.recurrent_heads} * plan.state_dimension *
                                    plan.state_dimension * kF32Bytes;
    const std::uint64_t cache_plane =
        std::uint64_t{plan.key_value_heads} * capacity * plan.head_dimension * kBf16Bytes;
    g.gdn_live_state_bytes_per_layer = conv + recurrent;
    g.gdn_slot_state_bytes_per_layer = 2u * g.gdn_live_state_bytes_per_layer;
    g.attention_state_bytes_per_position_per_layer =
        2ull * plan.key_value_heads * plan.head_dimension * kBf16Bytes;
    g.attention_slot_state_bytes_per_layer = 2u * cache_plane;
    g.slot_state_bytes = g.gated_delta_layers * g.gdn_slot_state_bytes_per_layer +
                         g.attention_layers * g.attention_slot_state_bytes_per_layer;
    return {PrefillGeometryError::None, g};
}

PrefixStateSnapshotGeometry make_prefix_state_snapshot_geometry(const PrefillGeometry& geometry,
                                                                std::uint32_t positions) noexcept {
    PrefixStateSnapshotGeometry s;
    if (geometry.policy.context_capacity == 0 || geometry.gated_delta_layers == 0 ||
        geometry.attention_layers == 0 || positions == 0 ||
        positions > geometry.policy.context_capacity) {
        return s;
    }
    s.valid = true;
    s.positions = positions;
    s.gated_delta_bytes = geometry.gated_delta_layers * geometry.gdn_live_state_bytes_per_layer;
    s.attention_bytes = std::uint64_t{geometry.attention_layers} * positions *
                        geometry.attention_state_bytes_per_position_per_layer;
    s.total_bytes = s.gated_delta_bytes + s.attention_bytes;
    return s;
}

namespace {
std::uint32_t first_rows(const PrefillPolicy& policy, std::uint32_t context_base) {
    return policy.schedule == PrefillSchedule::LayerMajor && context_base == 0
               ? policy.first_chunk_rows
               : policy.maximum_block_rows;
}
}  // namespace

std::uint32_t prefill_chunk_count(const PrefillPolicy& policy, std::uint32_t context_base,
                                  std::uint32_t rows) {
    const std::uint32_t first = first_rows(policy, context_base);
    if (rows <= first) return 1;
    return 1u + (rows - first + policy.maximum_block_rows - 1u) / policy.maximum_block_rows;
}

PrefillChunk prefill_chunk_at(const PrefillPolicy& policy, std::uint32_t context_base,
                              std::uint32_t total_rows, std::uint32_t ordinal) {
    const std::uint32_t first = first_rows(policy, context_base);
    if (ordinal == 0) return {0, std::min(total_rows, first), 0};
    const std::uint32_t offset = first + (ordinal - 1u) * policy.maximum_block_rows;
    return {offset, std::min(total_rows - offset, policy.maximum_block_rows), ordinal};
}

PrefillPipelinesResult resolve_prefill_pipelines(const HipLibrary& library) {
    PrefillPipelines p;
    HipPipelineError error = HipPipelineError::None;
    using P = PrefillPipelines;
    const bool ok =
        resolve(library, p, &P::attn_qk_rope_blk, "attn_qk_rope_blk", error) &&
        resolve(library, p, &P::attention_flash_blk, "attention_flash_v2_blk", error) &&
        resolve(library, p, &P::attention_flash_split_blk, "attention_flash_split_blk", error) &&
        resolve(library, p, &P::gdn_conv_blk, "gdn_conv_blk", error) &&
        resolve(library, p, &P::gdn_gates_blk, "gdn_gates_blk", error) &&
        resolve(library, p, &P::gdn_recurrence_gates_blk, "gdn_recurrence_gates_blk", error) &&
        resolve(library, p, &P::gdn_recurrence_blk, "gdn_recurrence_blk", error) &&
        resolve(library, p, &P::gdn_gate_norm_blk, "gdn_gate_norm_blk", error) &&
        resolve(library, p, &P::gdn_chunk_recurrence_blk, "gdn_chunk_recurrence_blk", error) &&
        resolve(library, p, &P::gdn_conv_tape_blk, "gdn_conv_tape_blk", error) &&
        resolve(library, p, &P::gdn_recurrence_gates_tape_blk, "gdn_recurrence_gates_tape_blk",
                error) &&
        resolve(library, p, &P::gdn_tape_replay_blk, "gdn_tape_replay_blk", error);
    if (!ok) return {error, std::nullopt};
    return {HipPipelineError::None, std::move(p)};
}

PrefillScratchResult create_prefill_scratch(const HipDevice& device,
                                            const PrefillGeometry& geometry) {
    if (!device) return {DecodeStepError::InvalidDevice, std::nullopt};
    PrefillScratch s;
    s.block_rows = geometry.policy.maximum_block_rows;
    s.compute_units = std::max<std::uint32_t>(device.compute_units(), 1);
    // the most any block of up to block_rows rows needs when its key walks are shared
    std::uint64_t shared_walk_bytes = 0;
    for (std::uint32_t rows = 32; rows <= std::max<std::uint32_t>(s.block_rows, 32); rows += 32) {
        shared_walk_bytes = std::max<std::uint64_t>(
            shared_walk_bytes,
            tt_flash_prefill_scratch_bytes(
                rows, tt_flash_prefill_splits(rows, geometry.policy.context_capacity, s.compute_units)));
    }
    const std::uint64_t parameter_bytes =
        std::uint64_t{s.block_rows} * 32u * kF32Bytes;  // [rows][32] decay / beta
    if (!allocate_zeroed(device, geometry.gdn_projection_bytes, s.gdn_projection) ||
        !allocate_zeroed(device, geometry.gdn_qk_bytes, s.gdn_qk) ||
        !allocate_zeroed(device, geometry.gdn_value_bytes, s.gdn_value) ||
        !allocate_zeroed(device, geometry.gdn_value_bytes, s.gdn_gate) ||
        !allocate_zeroed(device, geometry.gdn_value_bytes, s.gdn_recurrence) ||
        !allocate_zeroed(device, geometry.gdn_value_bytes, s.gdn_gated) ||
        !allocate_zeroed(device, parameter_bytes, s.gdn_decay) ||
        !allocate_zeroed(device, parameter_bytes, s.gdn_beta) ||
        (geometry.gdn_chunk_bytes != 0 &&
         !allocate_zeroed(device, geometry.gdn_chunk_bytes, s.gdn_chunk)) ||
        (geometry.gdn_tape_bytes != 0 &&
         (!allocate_zeroed(device, geometry.gdn_tape_bytes, s.gdn_tape) ||
          !allocate_zeroed(device, geometry.gdn_conv_tape_bytes, s.gdn_conv_tape))) ||
        !allocate_zeroed(device, geometry.attention_projection_bytes, s.attn_projection) ||
        !allocate_zeroed(device, geometry.attention_vector_bytes, s.attn_query) ||
        !allocate_zeroed(device, geometry.attention_vector_bytes, s.attn_gate) ||
        !allocate_zeroed(device, geometry.attention_vector_bytes, s.attn_attended) ||
        (shared_walk_bytes != 0 && !allocate_zeroed(device, shared_walk_bytes, s.attn_shared_walk))) {
        return {DecodeStepError::BufferAllocationFailed, std::nullopt};
    }
    return {DecodeStepError::None, std::move(s)};
}

HipCommandError encode_prefill_attention(const PrefillPipelines& pipelines,
                                         const PrefillGeometry& geometry, PrefillScratch& scratch,
                                         const DecodeLayerState& state, const LayerWeights& weights,
                                         const PrefillChunk& chunk, std::uint32_t context_base,
                                         HipComputePass& pass) {
    const std::uint32_t rows = chunk.rows;
    const std::uint32_t capacity = geometry.policy.context_capacity;
    if (rows == 0 || rows > scratch.block_rows) return HipCommandError::InvalidDispatchExtent;
    const std::uint64_t position = std::uint64_t{context_base} + chunk.offset;
    if (position + rows > capacity) return HipCommandError::ContextOutOfRange;
    Walk walk{pass};
    walk.pipeline(pipelines.attn_qk_rope_blk);
    walk.buffer(scratch.attn_projection, 0, 0);
    walk.weight(weights.query_norm, 1);
    walk.weight(weights.key_norm, 2);
    walk.buffer(scratch.attn_query, 0, 3);
    walk.buffer(scratch.attn_gate, 0, 4);
    walk.buffer(state.first, 0, 5);
    walk.buffer(state.second, 0, 6);
    walk.constant(static_cast<std::uint32_t>(position), 7);
    walk.constant(capacity, 8);
    walk.dispatch(18, 256, rows);
    walk.barrier();
    const std::uint32_t visible = static_cast<std::uint32_t>(position) + rows;
    const std::uint32_t sharers =
        scratch.attn_shared_walk ? tt_flash_prefill_splits(rows, visible, scratch.compute_units) : 1;
    walk.pipeline(sharers > 1 ? pipelines.attention_flash_split_blk : pipelines.attention_flash_blk);
    walk.buffer(scratch.attn_query, 0, 0);
    walk.buffer(state.first, 0, 1);
    walk.buffer(state.second, 0, 2);
    walk.buffer(scratch.attn_gate, 0, 3);
    walk.buffer(scratch.attn_attended, 0, 4);
    walk.constant(visible, 5);
    walk.constant(capacity, 6);
    walk.constant(rows, 7);
    walk.constant(static_cast<std::uint32_t>(position), 8);
    if (sharers > 1) {
        walk.buffer(scratch.attn_shared_walk, 0, 9);
        walk.constant(sharers, 10);
    }
    walk.dispatch(16, 256, (rows + 15u) / 16u);
    return walk.error;
}

HipCommandError encode_prefill_gated_delta(const PrefillPipelines& pipelines,
                                           const PrefillGeometry& geometry, PrefillScratch& scratch,
                                           const DecodeLayerState& state,
                                           const LayerWeights& weights, const PrefillChunk& chunk,
                                           std::uint32_t recurrence_ordinal, HipComputePass& pass,
                                           std::uint32_t layer_index) {
    const std::uint32_t rows = chunk.rows;
    if (rows == 0 || rows > scratch.block_rows) return HipCommandError::InvalidDispatchExtent;
    const bool taped = geometry.policy.gdn_tape;
    if (taped && (!scratch.gdn_tape || !scratch.gdn_conv_tape || layer_index >= kGdnTapeLayers)) {
        return HipCommandError::InvalidBuffer;
    }
    const bool phase = state.swapped ^ ((recurrence_ordinal & 1u) != 0u);
    const HipBuffer& conv_in = phase ? state.first_out : state.first;
    const HipBuffer& conv_out = phase ? state.first : state.first_out;
    const HipBuffer& recurrent_in = phase ? state.second_out : state.second;
    const HipBuffer& recurrent_out = phase ? state.second : state.second_out;
    Walk walk{pass};
    walk.pipeline(taped ? pipelines.gdn_conv_tape_blk : pipelines.gdn_conv_blk);
    walk.buffer(scratch.gdn_projection, 0, 0);
    walk.buffer(conv_in, 0, 1);
    walk.weight(weights.conv_weight, 2);
    walk.buffer(scratch.gdn_qk, 0, 3);
    walk.buffer(scratch.gdn_value, 0, 4);
    walk.buffer(scratch.gdn_gate, 0, 5);
    walk.buffer(conv_out, 0, 6);
    walk.constant(rows, 7);
    if (taped) {
        walk.buffer(scratch.gdn_conv_tape, 0, 8);
        walk.constant(layer_index, 9);
    }
    walk.dispatch(96, 128, rows);
    walk.barrier();
    if (geometry.policy.gdn_chunked) {
        if (!scratch.gdn_chunk) return HipCommandError::InvalidBuffer;
        walk.pipeline(pipelines.gdn_gates_blk);
        walk.buffer(scratch.gdn_projection, 0, 0);
        walk.weight(weights.a_log, 1);
        walk.weight(weights.dt_bias, 2);
        walk.buffer(scratch.gdn_decay, 0, 3);
        walk.buffer(scratch.gdn_beta, 0, 4);
        walk.constant(rows, 5);
        walk.dispatch(HipSize{1, (rows + 3u) / 4u, 1}, HipSize{32, 4, 1});
        walk.barrier();
        walk.pipeline(pipelines.gdn_chunk_recurrence_blk);
        walk.buffer(scratch.gdn_qk, 0, 0);
        walk.buffer(scratch.gdn_value, 0, 1);
        walk.buffer(scratch.gdn_decay, 0, 2);
        walk.buffer(scratch.gdn_beta, 0, 3);
        walk.buffer(scratch.gdn_chunk, 0, 4);
        walk.buffer(recurrent_in, 0, 5);
        walk.buffer(scratch.gdn_recurrence, 0, 6);
        walk.buffer(recurrent_out, 0, 7);
        walk.constant(rows, 8);
        walk.dispatch(HipSize{8, 32, 1}, HipSize{256, 1, 1});
        walk.barrier();
        walk.pipeline(pipelines.gdn_gate_norm_blk);
        walk.buffer(scratch.gdn_recurrence, 0, 0);
        walk.buffer(scratch.gdn_gate, 0, 1);
        walk.weight(weights.norm_weight, 2);
        walk.buffer(scratch.gdn_gated, 0, 3);
        walk.dispatch(32, 128, rows);
        return walk.error;
    }
    if (geometry.policy.gdn_gate_hoist) {
        walk.pipeline(pipelines.gdn_gates_blk);
        walk.buffer(scratch.gdn_projection, 0, 0);
        walk.weight(weights.a_log, 1);
        walk.weight(weights.dt_bias, 2);
        walk.buffer(scratch.gdn_decay, 0, 3);
        walk.buffer(scratch.gdn_beta, 0, 4);
        walk.constant(rows, 5);
        walk.dispatch(HipSize{1, (rows + 3u) / 4u, 1}, HipSize{32, 4, 1});
        walk.barrier();
        walk.pipeline(taped ? pipelines.gdn_recurrence_gates_tape_blk
                            : pipelines.gdn_recurrence_gates_blk);
        walk.buffer(scratch.gdn_qk, 0, 0);
        walk.buffer(scratch.gdn_value, 0, 1);
        walk.buffer(scratch.gdn_decay, 0, 2);
        walk.weight(weights.a_log, 3);
        walk.buffer(scratch.gdn_beta, 0, 4);
        if (taped) {
            walk.buffer(scratch.gdn_tape, 0, 9);
            walk.constant(layer_index, 10);
        }
    } else {
        walk.pipeline(pipelines.gdn_recurrence_blk);
        walk.buffer(scratch.gdn_qk, 0, 0);
        walk.buffer(scratch.gdn_value, 0, 1);
        walk.buffer(scratch.gdn_projection, 0, 2);
        walk.weight(weights.a_log, 3);
        walk.weight(weights.dt_bias, 4);
    }
    walk.buffer(recurrent_in, 0, 5);
    walk.buffer(scratch.gdn_recurrence, 0, 6);
    walk.buffer(recurrent_out, 0, 7);
    walk.constant(rows, 8);
    walk.dispatch(HipSize{1, 32, 32}, HipSize{32, 4, 1});
    walk.barrier();
    walk.pipeline(pipelines.gdn_gate_norm_blk);
    walk.buffer(scratch.gdn_recurrence, 0, 0);
    walk.buffer(scratch.gdn_gate, 0, 1);
    walk.weight(weights.norm_weight, 2);
    walk.buffer(scratch.gdn_gated, 0, 3);
    walk.dispatch(32, 128, rows);
    return walk.error;
}

HipCommandError encode_gdn_tape_replay(const PrefillPipelines& pipelines, const DecodeStep& step,
                                       const DecodeStateSlot& state, const PrefillScratch& scratch,
                                       std::uint32_t committed, HipComputePass& pass) {
    if (!decode_state_slot_compatible(step, state) || !decode_state_slot_ready(step, state)) {
        return HipCommandError::StateSlotMismatch;
    }
    if (!scratch.gdn_tape || step.schedule.size() > kGdnTapeLayers) {
        return HipCommandError::InvalidBuffer;
    }
    if (committed == 0 || committed > kGdnTapeRows) return HipCommandError::InvalidDispatchExtent;
    Walk walk{pass};
    for (std::uint32_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (!is_gated(step.schedule[layer])) continue;
        const DecodeLayerState& s = state.layers[layer];
        walk.pipeline(pipelines.gdn_tape_replay_blk);
        walk.buffer(scratch.gdn_tape, 0, 0);
        walk.buffer(s.swapped ? s.second_out : s.second, 0, 1);
        walk.buffer(s.swapped ? s.second : s.second_out, 0, 2);
        walk.constant(committed, 3);
        walk.constant(layer, 4);
        walk.dispatch(HipSize{1, 32, 32}, HipSize{32, 4, 1});
    }
    return walk.error;
}

HipCommandError encode_gdn_tape_windows(const DecodeStep& step, DecodeStateSlot& state,
                                        const PrefillScratch& scratch, std::uint32_t committed,
                                        HipBlitPass& blit_pass) {
    if (!decode_state_slot_compatible(step, state) || !decode_state_slot_ready(step, state)) {
        return HipCommandError::StateSlotMismatch;
    }
    if (!scratch.gdn_conv_tape || step.schedule.size() > kGdnTapeLayers) {
        return HipCommandError::InvalidBuffer;
    }
    if (committed == 0 || committed > kGdnTapeRows) return HipCommandError::InvalidCopyExtent;
    const std::uint64_t window = step.geometry.gdn_conv_state_bytes;
    for (std::uint32_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (!is_gated(step.schedule[layer])) continue;
        DecodeLayerState& s = state.layers[layer];
        const HipCommandError copied = copy_buffer(
            blit_pass, scratch.gdn_conv_tape,
            (std::uint64_t{layer} * kGdnTapeRows + (committed - 1u)) * window,
            s.swapped ? s.first : s.first_out, 0, window);
        if (copied != HipCommandError::None) return copied;
    }
    return HipCommandError::None;
}

void complete_gdn_tape_rollback(const DecodeStep& step, DecodeStateSlot& state) {
    advance_prefill_state(step, state, 1);
}

// ---- lane state record (Q36BRS01) ------------------------------------------

namespace {

constexpr std::uint64_t kRecordKvHeads = 2;                 // decode_harness.cpp:26
constexpr std::uint64_t kRecordHeadRowBytes = 256 * 2;      // decode_harness.cpp:27

bool fetch(const HipBuffer& buffer, std::uint64_t offset, std::byte* destination,
           std::uint64_t length) {
    return tt_buffer_read(buffer.native(), offset, destination, length) == TT_OK;
}
bool store(const HipBuffer& buffer, std::uint64_t offset, const std::byte* source,
           std::uint64_t length) {
    return tt_buffer_write(buffer.native(), offset, source, length) == TT_OK;
}

}  // namespace

namespace {

// The body of a record is a sequence of byte runs taken from (or installed into) a lane's
// buffers, in schedule order: a Gated DeltaNet layer contributes its conv window and its
// recurrent state whole, an attention layer the first `positions` rows of each kv head of the
// keys, then of the values - packed, although the caches are capacity-strided
// (decode_harness.cpp:339-460).  One walker produces the runs; sizing, writing and loading are
// three visitors of it.
struct RecordRun {
    std::size_t layer;
    std::uint32_t buffer;        // 0: first (conv | keys), 1: second (recurrent | values)
    std::uint64_t slot_offset;   // byte offset inside the lane's buffer
    std::uint64_t bytes;
};

template <typename Visit>   // bool visit(const RecordRun&): false stops the walk
bool walk_state_record(const DecodeStep& step, std::uint32_t positions, Visit&& visit) {
    const std::uint64_t packed_head = positions * kRecordHeadRowBytes;
    const std::uint64_t cache_head = std::uint64_t{step.capacity} * kRecordHeadRowBytes;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        const bool gated = is_gated(step.schedule[layer]);
        for (std::uint32_t buffer = 0; buffer < 2; ++buffer) {
            if (gated) {
                const std::uint64_t whole = buffer == 0 ? step.geometry.gdn_conv_state_bytes
                                                        : step.geometry.gdn_recurrent_state_bytes;
                if (!visit(RecordRun{layer, buffer, 0, whole})) return false;
                continue;
            }
            for (std::uint64_t head = 0; head < kRecordKvHeads; ++head) {
                if (!visit(RecordRun{layer, buffer, head * cache_head, packed_head})) return false;
            }
        }
    }
    return true;
}

}  // namespace

std::uint64_t state_record_bytes(const DecodeStep& step, std::uint32_t positions) noexcept {
    if (positions == 0 || positions > step.capacity) return 0;
    std::uint64_t bytes = kStateRecordHeaderBytes;
    walk_state_record(step, positions, [&bytes](const RecordRun& run) {
        bytes += run.bytes;
        return true;
    });
    return bytes;
}

StateRecordError write_state_record(const DecodeStep& step, const DecodeStateSlot& state,
                                    std::uint32_t positions, std::vector<std::byte>& record) {
    if (!decode_state_slot_ready(step, state)) return StateRecordError::InvalidState;
    const std::uint64_t total = state_record_bytes(step, positions);
    if (total == 0) return StateRecordError::InvalidPositions;
    record.assign(total, std::byte{0});
    std::memcpy(record.data(), kStateRecordMagic, 8);
    std::memcpy(record.data() + 8, &positions, 4);
    std::byte* cursor = record.data() + kStateRecordHeaderBytes;
    // a record carries the LIVE plane of each ping-pong pair
    const bool moved = walk_state_record(step, positions, [&](const RecordRun& run) {
        const DecodeLayerState& s = state.layers[run.layer];
        const bool out_plane = is_gated(step.schedule[run.layer]) && gated_delta_live_is_out(s.swapped);
        const HipBuffer& source = run.buffer == 0 ? (out_plane ? s.first_out : s.first)
                                                  : (out_plane ? s.second_out : s.second);
        if (!fetch(source, run.slot_offset, cursor, run.bytes)) return false;
        cursor += run.bytes;
        return true;
    });
    if (!moved || cursor != record.data() + total) return StateRecordError::TransferFailed;
    return StateRecordError::None;
}

StateRecordError load_state_record(std::span<const std::byte> record, const DecodeStep& step,
                                   DecodeStateSlot& state, std::uint32_t& positions) {
    if (!decode_state_slot_ready(step, state)) return StateRecordError::InvalidState;
    if (record.size() < kStateRecordHeaderBytes) return StateRecordError::Truncated;
    if (std::memcmp(record.data(), kStateRecordMagic, 8) != 0) return StateRecordError::MagicMismatch;
    std::uint32_t count = 0;
    std::memcpy(&count, record.data() + 8, 4);
    const std::uint64_t total = state_record_bytes(step, count);
    if (total == 0) return StateRecordError::InvalidPositions;
    if (record.size() < total) return StateRecordError::Truncated;
    if (record.size() > total) return StateRecordError::TrailingBytes;
    // the whole record has been checked against the step before the first byte moves; it is
    // installed into `first` / `second`, which the cleared phase below makes the live planes
    const std::byte* cursor = record.data() + kStateRecordHeaderBytes;
    const bool moved = walk_state_record(step, count, [&](const RecordRun& run) {
        DecodeLayerState& s = state.layers[run.layer];
        if (!store(run.buffer == 0 ? s.first : s.second, run.slot_offset, cursor, run.bytes)) {
            return false;
        }
        cursor += run.bytes;
        return true;
    });
    if (!moved) return StateRecordError::TransferFailed;
    for (std::size_t layer = 0; layer < step.schedule.size(); ++layer) {
        if (is_gated(step.schedule[layer])) state.layers[layer].swapped = false;
    }
    positions = count;
    return StateRecordError::None;
}

// ---- prefix state snapshot / restore ---------------------------------------
namespace {

// 64-bit products and sums that report wrap-around instead of hiding it
bool product(std::uint64_t a, std::uint64_t b, std::uint64_t& out) noexcept {
    return !__builtin_mul_overflow(a, b, &out);
}
bool total(std::uint64_t a, std::uint64_t b, std::uint64_t& out) noexcept {
    return !__builtin_add_overflow(a, b, &out);
}
bool extent_holds(std::uint64_t offset, std::uint64_t length, std::uint64_t extent) noexcept {
    return offset <= extent && length <= extent - offset;
}
bool known_kind(LayerKind kind) noexcept {
    return kind == LayerKind::GatedDelta || kind == LayerKind::FullAttention;
}

constexpr std::uint32_t kNoLayer = std::numeric_limits<std::uint32_t>::max();

// schedule index of the `ordinal`-th layer of one family
std::uint32_t nth_of_family(std::span<const LayerKind> schedule, bool gated,
                            std::uint32_t ordinal) noexcept {
    for (std::uint32_t layer = 0; layer < schedule.size(); ++layer) {
        if (is_gated(schedule[layer]) != gated) continue;
        if (ordinal == 0) return layer;
        --ordinal;
    }
    return kNoLayer;
}

const HipBuffer* plane_of(const DecodeLayerState& layer, PrefixStateBufferPlane plane) noexcept {
    switch (plane) {
    case PrefixStateBufferPlane::First: return &layer.first;
    case PrefixStateBufferPlane::FirstOutput: return &layer.first_out;
    case PrefixStateBufferPlane::Second: return &layer.second;
    case PrefixStateBufferPlane::SecondOutput: return &layer.second_out;
    case PrefixStateBufferPlane::Arena: break;
    }
    return nullptr;
}

void forget_transfer(DecodeStateSlot& state) noexcept {
    state.active_transfer_generation = 0;
    state.active_transfer_arena = nullptr;
    state.active_transfer_positions = 0;
    state.active_transfer_offset_bytes = 0;
    state.active_transfer_state_bytes = 0;
}

PrefixStateTransferResult refused(PrefixStateTransferError error,
                                  PrefixStateLayoutError layout = PrefixStateLayoutError::None,
                                  HipCommandError command = HipCommandError::None) noexcept {
    PrefixStateTransferResult r;
    r.error = error;
    r.layout_error = layout;
    r.command_error = command;
    return r;
}

bool ticket_current(const PrefixStateTransferTicket& ticket, const DecodeStep& decode,
                    const DecodeStateSlot& state, const HipBuffer& arena) noexcept {
    const DecodeStateSlotStatus pending =
        ticket.direction == PrefixStateTransferDirection::Snapshot
            ? DecodeStateSlotStatus::SnapshotPending
            : DecodeStateSlotStatus::RestorePending;
    return ticket.generation != 0 && ticket.owner == &decode && ticket.state_owner == &state &&
           ticket.arena_owner == &arena && state.status == pending &&
           decode_state_slot_compatible(decode, state) &&
           state.active_transfer_generation == ticket.generation &&
           state.active_transfer_arena == &arena &&
           state.active_transfer_positions == ticket.positions &&
           state.active_transfer_offset_bytes == ticket.arena_offset_bytes &&
           state.active_transfer_state_bytes == ticket.state_bytes;
}

// One copy of a transfer: the slot-side buffer and both offsets.
struct PlannedCopy {
    const HipBuffer* slot_buffer{nullptr};
    std::uint64_t slot_offset{0};
    std::uint64_t arena_offset{0};
    std::uint64_t length{0};
};

bool plan_copy(const PrefixStateLayout& layout, std::uint32_t index,
               PrefixStateTransferDirection direction, const DecodeStateSlot& state,
               const HipBuffer& arena, std::uint64_t arena_base, PlannedCopy& copy,
               PrefixStateLayoutError& layout_error) noexcept {
    const PrefixStateSegmentResult found = prefix_state_segment(layout, index);
    layout_error = found.error;
    if (!found || found.segment.layer_index >= state.layers.size()) return false;
    const DecodeLayerState& layer = state.layers[found.segment.layer_index];
    const PrefixStateCopyRoute route = prefix_state_copy_route(found.segment, direction, layer.swapped);
    copy.slot_buffer = plane_of(layer, direction == PrefixStateTransferDirection::Snapshot
                                           ? route.source
                                           : route.destination);
    copy.slot_offset = found.segment.slot_offset_bytes;
    copy.length = found.segment.length_bytes;
    return copy.slot_buffer != nullptr && copy.slot_buffer != &arena &&
           extent_holds(copy.slot_offset, copy.length, copy.slot_buffer->size_bytes()) &&
           total(arena_base, found.segment.snapshot_offset_bytes, copy.arena_offset) &&
           extent_holds(copy.arena_offset, copy.length, arena.size_bytes());
}

PrefixStateTransferResult encode_prefix_transfer(PrefixStateTransferDirection direction,
                                                 const DecodeStep& decode, DecodeStateSlot& state,
                                                 const PrefillGeometry& geometry,
                                                 HipBlitPass& blit_pass, HipBuffer& arena,
                                                 std::uint64_t arena_base, std::uint32_t positions,
                                                 std::span<std::byte> evidence) noexcept {
    const bool snapshot = direction == PrefixStateTransferDirection::Snapshot;
    if (state.status == DecodeStateSlotStatus::Poisoned) {
        return refused(PrefixStateTransferError::PoisonedStateSlot);
    }
    if (!decode_state_slot_compatible(decode, state) || !decode_state_slot_complete(decode, state)) {
        return refused(PrefixStateTransferError::InvalidStateSlot);
    }
    if (!decode_state_slot_ready(decode, state)) {
        return refused(PrefixStateTransferError::StateSlotNotReady);
    }
    if (!arena) return refused(PrefixStateTransferError::InvalidArena);
    const std::size_t evidence_bytes =
        snapshot ? prefix_state_phase_evidence_bytes(decode.schedule) : 0;
    if (evidence.size() < evidence_bytes) {
        return refused(PrefixStateTransferError::PhaseEvidenceTooSmall);
    }
    const PrefixStateLayoutResult made = make_prefix_state_layout(decode, geometry, positions);
    if (!made) return refused(PrefixStateTransferError::InvalidLayout, made.error);
    const PrefixStateLayout& layout = made.layout;
    if (validate_prefix_state_arena_extent(layout, arena_base, arena.size_bytes()) !=
        PrefixStateTransferError::None) {
        return refused(PrefixStateTransferError::ArenaOutOfRange);
    }
    if (state.next_transfer_generation == 0) {
        return refused(PrefixStateTransferError::GenerationExhausted);
    }
    if (!blit_pass) {
        return refused(PrefixStateTransferError::CommandEncodingFailed, PrefixStateLayoutError::None,
                       HipCommandError::InvalidBlitPass);
    }
    // every copy is checked before the first one is issued, so a refusal leaves
    // both the slot and the arena untouched
    for (std::uint32_t index = 0; index < layout.segment_count; ++index) {
        PlannedCopy copy;
        PrefixStateLayoutError layout_error = PrefixStateLayoutError::None;
        if (!plan_copy(layout, index, direction, state, arena, arena_base, copy, layout_error)) {
            return layout_error != PrefixStateLayoutError::None
                       ? refused(PrefixStateTransferError::InvalidLayout, layout_error)
                       : refused(PrefixStateTransferError::InvalidStateSlot);
        }
    }
    for (std::uint32_t index = 0; index < layout.segment_count; ++index) {
        PlannedCopy copy;
        PrefixStateLayoutError layout_error = PrefixStateLayoutError::None;
        (void)plan_copy(layout, index, direction, state, arena, arena_base, copy, layout_error);
        const HipCommandError command =
            snapshot ? copy_buffer(blit_pass, *copy.slot_buffer, copy.slot_offset, arena,
                                   copy.arena_offset, copy.length)
                     : copy_buffer(blit_pass, arena, copy.arena_offset,
                                   const_cast<HipBuffer&>(*copy.slot_buffer), copy.slot_offset,
                                   copy.length);
        if (command != HipCommandError::None) {
            state.status = DecodeStateSlotStatus::Poisoned;
            forget_transfer(state);
            return refused(PrefixStateTransferError::CommandEncodingFailed,
                           PrefixStateLayoutError::None, command);
        }
    }
    if (snapshot) {
        const PrefixStateTransferError captured =
            capture_prefix_state_phase_evidence(decode, state, evidence.first(evidence_bytes));
        if (captured != PrefixStateTransferError::None) return refused(captured);
    }
    const std::uint64_t generation = state.next_transfer_generation;
    state.next_transfer_generation =
        generation == std::numeric_limits<std::uint64_t>::max() ? 0 : generation + 1u;
    state.active_transfer_generation = generation;
    state.active_transfer_arena = &arena;
    state.active_transfer_positions = positions;
    state.active_transfer_offset_bytes = arena_base;
    state.active_transfer_state_bytes = layout.total_bytes;
    state.status = snapshot ? DecodeStateSlotStatus::SnapshotPending
                            : DecodeStateSlotStatus::RestorePending;
    PrefixStateTransferResult done;
    done.error = PrefixStateTransferError::None;
    done.segment_count = layout.segment_count;
    done.state_bytes = layout.total_bytes;
    done.source_phase_evidence_bytes = evidence_bytes;
    done.ticket = PrefixStateTransferTicket{direction,  &decode,          &state,
                                            &arena,     positions,        arena_base,
                                            layout.total_bytes, generation, true};
    return done;
}

}  // namespace

PrefixStateLayoutResult make_prefix_state_layout(const PrefixStateLayoutSpec& spec) noexcept {
    const auto fail = [](PrefixStateLayoutError error) {
        return PrefixStateLayoutResult{error, {}};
    };
    if (spec.schedule.empty() || spec.schedule.size() > std::numeric_limits<std::uint32_t>::max()) {
        return fail(PrefixStateLayoutError::InvalidSchedule);
    }
    if (spec.capacity == 0 || spec.key_value_heads == 0 || spec.head_dimension == 0 ||
        spec.expected_gated_delta_layers == 0 || spec.expected_attention_layers == 0 ||
        spec.gated_delta_convolution_bytes == 0 || spec.gated_delta_recurrent_bytes == 0 ||
        spec.expected_total_bytes == 0) {
        return fail(PrefixStateLayoutError::InvalidGeometry);
    }
    if (spec.positions == 0 || spec.positions > spec.capacity) {
        return fail(PrefixStateLayoutError::PositionOutOfRange);
    }
    PrefixStateLayout layout;
    layout.specification = spec;
    for (const LayerKind kind : spec.schedule) {
        if (!known_kind(kind)) return fail(PrefixStateLayoutError::InvalidSchedule);
        (is_gated(kind) ? layout.gated_delta_layers : layout.attention_layers) += 1;
    }
    if (layout.gated_delta_layers != spec.expected_gated_delta_layers ||
        layout.attention_layers != spec.expected_attention_layers) {
        return fail(PrefixStateLayoutError::FamilyCountMismatch);
    }
    // payload = G x (conv + recurrent) + A x 2 x kv_heads x positions x head_dimension bf16
    const std::uint64_t row_bytes = std::uint64_t{spec.head_dimension} * kBf16Bytes;
    std::uint64_t live_pair = 0, head_segments = 0, segments = 0;
    const bool fits =
        total(spec.gated_delta_convolution_bytes, spec.gated_delta_recurrent_bytes, live_pair) &&
        product(live_pair, layout.gated_delta_layers, layout.gated_delta_bytes) &&
        product(spec.positions, row_bytes, layout.attention_segment_bytes) &&
        product(spec.capacity, row_bytes, layout.attention_slot_head_stride_bytes) &&
        product(std::uint64_t{layout.attention_layers} * 2u, spec.key_value_heads, head_segments) &&
        product(head_segments, layout.attention_segment_bytes, layout.attention_bytes) &&
        total(layout.gated_delta_bytes, layout.attention_bytes, layout.total_bytes) &&
        total(std::uint64_t{layout.gated_delta_layers} * 2u, head_segments, segments) &&
        segments <= std::numeric_limits<std::uint32_t>::max();
    if (!fits) return fail(PrefixStateLayoutError::Overflow);
    if (layout.total_bytes != spec.expected_total_bytes) {
        return fail(PrefixStateLayoutError::TotalMismatch);
    }
    layout.segment_count = static_cast<std::uint32_t>(segments);
    return {PrefixStateLayoutError::None, layout};
}

PrefixStateLayoutResult make_prefix_state_layout(const DecodeStep& decode,
                                                 const PrefillGeometry& geometry,
                                                 std::uint32_t positions) noexcept {
    const auto fail = [](PrefixStateLayoutError error) {
        return PrefixStateLayoutResult{error, {}};
    };
    if (decode.capacity == 0 || geometry.policy.context_capacity != decode.capacity ||
        geometry.key_value_heads == 0 || geometry.attention_head_dimension == 0 ||
        geometry.gated_delta_layers == 0 || geometry.attention_layers == 0) {
        return fail(PrefixStateLayoutError::InvalidGeometry);
    }
    // the prefill extents must describe the very buffers this step allocated
    const std::uint64_t live_pair =
        decode.geometry.gdn_conv_state_bytes + decode.geometry.gdn_recurrent_state_bytes;
    const std::uint64_t per_position = 2ull * geometry.key_value_heads *
                                       geometry.attention_head_dimension * kBf16Bytes;
    if (live_pair != geometry.gdn_live_state_bytes_per_layer ||
        per_position != geometry.attention_state_bytes_per_position_per_layer ||
        2u * decode.geometry.attn_cache_bytes != geometry.attention_slot_state_bytes_per_layer) {
        return fail(PrefixStateLayoutError::InvalidGeometry);
    }
    if (positions == 0 || positions > decode.capacity) {
        return fail(PrefixStateLayoutError::PositionOutOfRange);
    }
    const PrefixStateSnapshotGeometry sized = make_prefix_state_snapshot_geometry(geometry, positions);
    if (!sized.valid) return fail(PrefixStateLayoutError::InvalidGeometry);
    PrefixStateLayoutSpec spec;
    spec.schedule = decode.schedule;
    spec.capacity = decode.capacity;
    spec.positions = positions;
    spec.key_value_heads = geometry.key_value_heads;
    spec.head_dimension = geometry.attention_head_dimension;
    spec.expected_gated_delta_layers = geometry.gated_delta_layers;
    spec.expected_attention_layers = geometry.attention_layers;
    spec.gated_delta_convolution_bytes = decode.geometry.gdn_conv_state_bytes;
    spec.gated_delta_recurrent_bytes = decode.geometry.gdn_recurrent_state_bytes;
    spec.expected_total_bytes = sized.total_bytes;
    return make_prefix_state_layout(spec);
}

PrefixStateSegmentResult prefix_state_segment(const PrefixStateLayout& layout,
                                              std::uint32_t index) noexcept {
    if (index >= layout.segment_count) return {PrefixStateLayoutError::SegmentOutOfRange, {}};
    const PrefixStateLayoutSpec& spec = layout.specification;
    PrefixStateSegment segment;
    const std::uint32_t gated_segments = 2u * layout.gated_delta_layers;
    if (index < gated_segments) {
        // (conv, recurrent) pairs, one pair per gated-delta layer
        const std::uint32_t ordinal = index >> 1;
        const bool recurrent = (index & 1u) != 0;
        segment.layer_index = nth_of_family(spec.schedule, true, ordinal);
        segment.kind = recurrent ? PrefixStateSegmentKind::GatedDeltaRecurrent
                                 : PrefixStateSegmentKind::GatedDeltaConvolution;
        segment.length_bytes =
            recurrent ? spec.gated_delta_recurrent_bytes : spec.gated_delta_convolution_bytes;
        segment.snapshot_offset_bytes =
            ordinal * (spec.gated_delta_convolution_bytes + spec.gated_delta_recurrent_bytes) +
            (recurrent ? spec.gated_delta_convolution_bytes : 0);
    } else {
        // per attention layer: keys of head 0..H-1, then values of head 0..H-1
        const std::uint32_t packed = index - gated_segments;
        const std::uint32_t per_layer = 2u * spec.key_value_heads;
        const std::uint32_t within = packed % per_layer;
        const bool value = within >= spec.key_value_heads;
        segment.layer_index = nth_of_family(spec.schedule, false, packed / per_layer);
        segment.kind =
            value ? PrefixStateSegmentKind::AttentionValue : PrefixStateSegmentKind::AttentionKey;
        segment.head_index = value ? within - spec.key_value_heads : within;
        segment.slot_offset_bytes = segment.head_index * layout.attention_slot_head_stride_bytes;
        segment.length_bytes = layout.attention_segment_bytes;
        segment.snapshot_offset_bytes =
            layout.gated_delta_bytes + packed * layout.attention_segment_bytes;
    }
    if (segment.layer_index == kNoLayer) return {PrefixStateLayoutError::FamilyCountMismatch, {}};
    return {PrefixStateLayoutError::None, segment};
}

PrefixStateCopyRoute prefix_state_copy_route(const PrefixStateSegment& segment,
                                             PrefixStateTransferDirection direction,
                                             bool gated_delta_swapped) noexcept {
    // the slot-side plane: a snapshot reads the live plane, a restore always
    // writes the in plane (completion then clears `swapped`)
    const bool out_plane =
        direction == PrefixStateTransferDirection::Snapshot && gated_delta_swapped;
    PrefixStateBufferPlane slot = PrefixStateBufferPlane::First;
    switch (segment.kind) {
    case PrefixStateSegmentKind::GatedDeltaConvolution:
        slot = out_plane ? PrefixStateBufferPlane::FirstOutput : PrefixStateBufferPlane::First;
        break;
    case PrefixStateSegmentKind::GatedDeltaRecurrent:
        slot = out_plane ? PrefixStateBufferPlane::SecondOutput : PrefixStateBufferPlane::Second;
        break;
    case PrefixStateSegmentKind::AttentionKey: slot = PrefixStateBufferPlane::First; break;
    case PrefixStateSegmentKind::AttentionValue: slot = PrefixStateBufferPlane::Second; break;
    }
    return direction == PrefixStateTransferDirection::Snapshot
               ? PrefixStateCopyRoute{slot, PrefixStateBufferPlane::Arena}
               : PrefixStateCopyRoute{PrefixStateBufferPlane::Arena, slot};
}

PrefixStateTransferError validate_prefix_state_arena_extent(const PrefixStateLayout& layout,
                                                            std::uint64_t arena_offset_bytes,
                                                            std::uint64_t arena_capacity_bytes) noexcept {
    if (layout.total_bytes == 0 || layout.segment_count == 0) {
        return PrefixStateTransferError::InvalidLayout;
    }
    return extent_holds(arena_offset_bytes, layout.total_bytes, arena_capacity_bytes)
               ? PrefixStateTransferError::None
               : PrefixStateTransferError::ArenaOutOfRange;
}

std::size_t prefix_state_phase_evidence_bytes(std::span<const LayerKind> schedule) noexcept {
    return (schedule.size() + 7u) / 8u;
}

PrefixStateTransferError capture_prefix_state_phase_evidence(const DecodeStep& decode,
                                                             const DecodeStateSlot& state,
                                                             std::span<std::byte> phase_evidence) noexcept {
    if (phase_evidence.size() < prefix_state_phase_evidence_bytes(decode.schedule)) {
        return PrefixStateTransferError::PhaseEvidenceTooSmall;
    }
    if (!decode_state_slot_compatible(decode, state)) {
        return PrefixStateTransferError::InvalidStateSlot;
    }
    for (std::byte& b : phase_evidence) b = std::byte{0};
    for (std::size_t layer = 0; layer < decode.schedule.size(); ++layer) {
        if (is_gated(decode.schedule[layer]) && state.layers[layer].swapped) {
            phase_evidence[layer >> 3] |= std::byte(1u << (layer & 7u));
        }
    }
    return PrefixStateTransferError::None;
}

PrefixStateTransferResult encode_prefix_state_snapshot(const DecodeStep& decode,
                                                       DecodeStateSlot& state,
                                                       const PrefillGeometry& geometry,
                                                       HipBlitPass& blit_pass, HipBuffer& state_arena,
                                                       std::uint64_t arena_offset_bytes,
                                                       std::uint32_t positions,
                                                       std::span<std::byte> source_phase_evidence) noexcept {
    return encode_prefix_transfer(PrefixStateTransferDirection::Snapshot, decode, state, geometry,
                                  blit_pass, state_arena, arena_offset_bytes, positions,
                                  source_phase_evidence);
}

PrefixStateTransferResult encode_prefix_state_restore(const DecodeStep& decode, DecodeStateSlot& state,
                                                      const PrefillGeometry& geometry,
                                                      HipBlitPass& blit_pass, HipBuffer& state_arena,
                                                      std::uint64_t arena_offset_bytes,
                                                      std::uint32_t positions) noexcept {
    return encode_prefix_transfer(PrefixStateTransferDirection::Restore, decode, state, geometry,
                                  blit_pass, state_arena, arena_offset_bytes, positions, {});
}

PrefixStateTransferError complete_prefix_state_transfer(PrefixStateTransferTicket& ticket,
                                                        const DecodeStep& decode,
                                                        DecodeStateSlot& state,
                                                        const HipBuffer& state_arena) noexcept {
    if (!ticket.pending) return PrefixStateTransferError::AlreadyCompleted;
    if (state.status == DecodeStateSlotStatus::Poisoned) {
        return PrefixStateTransferError::PoisonedStateSlot;
    }
    if (!ticket_current(ticket, decode, state, state_arena)) {
        return PrefixStateTransferError::StaleTicket;
    }
    if (ticket.direction == PrefixStateTransferDirection::Restore) {
        for (std::size_t layer = 0; layer < decode.schedule.size(); ++layer) {
            if (is_gated(decode.schedule[layer])) state.layers[layer].swapped = false;
        }
    }
    forget_transfer(state);
    state.status = DecodeStateSlotStatus::Ready;
    ticket.pending = false;
    return PrefixStateTransferError::None;
}

PrefixStateTransferError abort_prefix_state_transfer(PrefixStateTransferTicket& ticket,
                                                     const DecodeStep& decode, DecodeStateSlot& state,
                                                     const HipBuffer& state_arena) noexcept {
    if (!ticket.pending) return PrefixStateTransferError::AlreadyCompleted;
    if (state.status == DecodeStateSlotStatus::Poisoned) {
        forget_transfer(state);
        ticket.pending = false;
        return PrefixStateTransferError::PoisonedStateSlot;
    }
    if (!ticket_current(ticket, decode, state, state_arena)) {
        return PrefixStateTransferError::StaleTicket;
    }
    // the copies may have landed partly: the slot is kept but never trusted again
    forget_transfer(state);
    state.status = DecodeStateSlotStatus::Poisoned;
    ticket.pending = false;
    return PrefixStateTransferError::None;
}

}  // namespace tatara::runtime
