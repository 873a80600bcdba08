// Integer pins of the attention-family geometry: every value below is the one
// the reference pins for the same plan and capacity
// (tests/native/decode_geometry_test.cpp:34-88,
//  tests/native/prefill_geometry_test.cpp:22-94,
//  tests/native/prefill_step_contract_test.cpp:451-478).
#include "runtime.h"

using namespace tatara::runtime;
using tatara::model::qwen36::LayerKind;

int main() {
    const auto plan = tatara::model::qwen36::qwen36_35b_a3b_plan();
    if (plan.layers.size() != 40) return 1;
    for (std::size_t i = 0; i < 40; ++i) {
        const bool attention = i % 4 == 3;
        if ((plan.layers[i] == LayerKind::FullAttention) != attention) return 2;
    }
    const DecodeGeometry g = make_decode_geometry(plan, 16384);
    if (g.gated_delta_layers != 30 || g.attention_layers != 10) return 3;
    if (g.hidden_bytes != 4096 || g.layer_stream_bytes != 40ull * 4096) return 4;
    if (g.gdn_projection_bytes != 24704 || g.gdn_qk_bytes != 8192 || g.gdn_value_bytes != 8192) {
        return 5;
    }
    if (g.gdn_conv_state_bytes != 49152 || g.gdn_recurrent_state_bytes != 2097152) return 6;
    if (g.attn_projection_bytes != 18432 || g.attn_query_bytes != 8192) return 7;
    if (g.attn_record_scratch_bytes != 16ull * 64 * 258 * 4) return 8;
    if (g.attn_cache_bytes != 2ull * 16384 * 256 * 2) return 9;
    if (g.gdn_prepare.groups != 96 || g.gdn_prepare.threads != 128) return 10;
    if (g.gdn_recurrence.dimension_groups != 32 || g.gdn_recurrence.head_groups != 32 ||
        g.gdn_recurrence.lane_threads != 32 || g.gdn_recurrence.dimension_threads != 4) {
        return 11;
    }
    if (g.gdn_gate_norm.groups != 32 || g.gdn_gate_norm.threads != 128) return 12;
    if (g.attn_qk_rope.groups != 18 || g.attn_qk_rope.threads != 256) return 13;
    if (g.attention_head.groups != 16 || g.attention_head.threads != 256) return 14;
    if (g.attention_split.score_groups != 4 || g.attention_split.score_threads != 256 ||
        g.attention_split.score_cohort_threads != 4 || g.attention_split.value_groups != 2 ||
        g.attention_split.value_lane_threads != 32 ||
        g.attention_split.value_dimension_threads != 4 ||
        g.attention_split.value_head_threads != 8) {
        return 15;
    }
    if (g.rms.groups != 1 || g.rms.threads != 512) return 16;

    // a context is a cache position: equality with capacity is one past the end
    if (!context_in_capacity(0, 1) || context_in_capacity(1, 1) || context_in_capacity(0, 0) ||
        !context_in_capacity(16383, 16384) || context_in_capacity(16384, 16384)) {
        return 17;
    }
    if (attention_partitions(0) != 1 || attention_partitions(255) != 1 ||
        attention_partitions(256) != 2 || attention_partitions(511) != 2 ||
        attention_partitions(512) != 3 || attention_partitions(32767) != 128) {
        return 18;
    }
    // split choice: the workgroups that hold keys (2 kv heads x splits of every row) fit 256
    // compute units one each; at least 128 keys, a multiple of 32
    if (choose_split_keys(4, 32768) != 1024 || choose_split_keys(1, 32768) != 256 ||
        choose_split_keys(1, 100000) != 800 || choose_split_keys(4, 16384) != 512 ||
        choose_split_keys(1, 1) != 128 || choose_split_keys(16, 262144) != 32768 ||
        choose_split_keys(0, 0, 0) != 128 || choose_split_keys(1, 20000) % 32 != 0 ||
        choose_split_keys(4, 100000) != 3136 || choose_split_keys(3, 32768) != 800) {
        return 19;
    }
    {
        const std::array<std::uint32_t, 4> ragged{32768, 30000, 24576, 8192};
        const std::array<std::uint32_t, 8> wide{65536, 50001, 40001, 30001, 20001, 10001, 5001, 1001};
        if (choose_split_keys(ragged) != 768 || split_workgroups(ragged, 768) != 252 ||
            split_workgroups(ragged, 1024) != 188 || choose_split_keys(wide) != 1792 ||
            split_workgroups(wide, 1792) != 254 ||
            choose_split_keys(std::span<const std::uint32_t>{}) != 128) {
            return 19;
        }
    }

    const PrefillPolicy policy{.schedule = PrefillSchedule::LayerMajor,
                               .context_capacity = 16384,
                               .maximum_block_rows = 2048,
                               .first_chunk_rows = 256,
                               .query_tile_rows = 256,
                               .attention_partition = 256,
                               .gdn_gate_hoist = false};
    const auto made = make_prefill_geometry(plan, policy);
    if (!made) return 20;
    const PrefillGeometry& p = made.geometry;
    if (p.gated_delta_layers != 30 || p.attention_layers != 10 || p.attention_partitions != 64) {
        return 21;
    }
    if (p.gdn_live_state_bytes_per_layer != 2146304 || p.gdn_slot_state_bytes_per_layer != 4292608) {
        return 22;
    }
    if (p.attention_state_bytes_per_position_per_layer != 2048 ||
        p.attention_slot_state_bytes_per_layer != 33554432) {
        return 23;
    }
    if (p.slot_state_bytes != 464322560) return 24;
    if (p.gdn_projection_bytes != 50593792 || p.attention_projection_bytes != 37748736) return 25;
    if (p.attention_partial_bytes != 270532608) return 26;
    const auto s4 = make_prefix_state_snapshot_geometry(p, 4096);
    if (!s4.valid || s4.gated_delta_bytes != 64389120 || s4.attention_bytes != 83886080 ||
        s4.total_bytes != 148275200) {
        return 27;
    }
    const auto s16 = make_prefix_state_snapshot_geometry(p, 16384);
    if (!s16.valid || s16.attention_bytes != 335544320 || s16.total_bytes != 399933440) return 28;
    if (make_prefix_state_snapshot_geometry(p, 0).valid ||
        make_prefix_state_snapshot_geometry(p, 16385).valid) {
        return 29;
    }
    auto wide = policy;
    wide.context_capacity = 100000;
    const auto g100 = make_prefill_geometry(plan, wide);
    if (!g100) return 30;
    const auto s100 = make_prefix_state_snapshot_geometry(g100.geometry, 100000);
    if (!s100.valid || s100.attention_bytes != 10ull * 100000 * 2048) return 31;

    // policy bounds
    auto bad = policy;
    bad.query_tile_rows = 250;
    if (make_prefill_geometry(plan, bad).error != PrefillGeometryError::InvalidPolicy) return 32;
    bad = policy;
    bad.maximum_block_rows = 4096;
    if (make_prefill_geometry(plan, bad).error != PrefillGeometryError::InvalidPolicy) return 33;
    bad = policy;
    bad.context_capacity = 262145;
    if (make_prefill_geometry(plan, bad).error != PrefillGeometryError::InvalidPolicy) return 34;
    auto odd_plan = plan;
    odd_plan.head_dimension = 128;
    if (make_prefill_geometry(odd_plan, policy).error != PrefillGeometryError::InvalidPlan) return 35;

    // chunk planning: 3925 rows from an empty context, layer-major -> {256, 2048, 1621}
    if (prefill_chunk_count(policy, 0, 3925) != 3) return 40;
    const PrefillChunk c0 = prefill_chunk_at(policy, 0, 3925, 0);
    const PrefillChunk c1 = prefill_chunk_at(policy, 0, 3925, 1);
    const PrefillChunk c2 = prefill_chunk_at(policy, 0, 3925, 2);
    if (c0.offset != 0 || c0.rows != 256 || c1.offset != 256 || c1.rows != 2048 ||
        c2.offset != 2304 || c2.rows != 1621 || c2.ordinal != 2) {
        return 41;
    }
    // with live context the first chunk is a full block; chunk-major never shortens it
    if (prefill_chunk_count(policy, 256, 3925) != 2 ||
        prefill_chunk_at(policy, 256, 3925, 0).rows != 2048) {
        return 42;
    }
    auto chunk_major = policy;
    chunk_major.schedule = PrefillSchedule::ChunkMajor;
    if (prefill_chunk_at(chunk_major, 0, 3925, 0).rows != 2048) return 43;
    if (prefill_chunk_count(policy, 0, 100) != 1 || prefill_chunk_at(policy, 0, 100, 0).rows != 100) {
        return 44;
    }

    // request validation (prefill_geometry_test.cpp:228-252 cases)
    const std::uint32_t tokens[3] = {1, 2, 3};
    if (validate_prefill_request(policy, 0, 0, {}, 10).error != PrefillRequestError::EmptyPrefix) {
        return 50;
    }
    if (validate_prefill_request(policy, 5, 4, tokens, 10).error !=
        PrefillRequestError::ContextOutOfRange) {
        return 51;
    }
    if (validate_prefill_request(policy, 16383, 16383, tokens, 10).error !=
        PrefillRequestError::ContextOverflow) {
        return 52;
    }
    if (validate_prefill_request(policy, 0, 0, tokens, 3).error !=
        PrefillRequestError::TokenOutOfRange) {
        return 53;
    }
    const auto ok = validate_prefill_request(policy, 7, 7, tokens, 10);
    if (!ok || ok.next_context != 10) return 54;
    std::vector<std::uint32_t> many(2049, 0);
    if (validate_prefill_request(policy, 0, 0, many, 10).error !=
        PrefillRequestError::BlockOutOfRange) {
        return 55;
    }
    if (!validate_prefill_prefix(policy, 0, 0, many, 10)) return 56;
    return 0;
}
