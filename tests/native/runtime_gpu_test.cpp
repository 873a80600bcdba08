// The C++ host layer end to end on the GPU against the CPU checker: a 4-layer
// stack (G,G,G,A) over pooled lanes, two batched token steps with the ping-pong
// flip in between, a two-chunk block prefill on a private slot, and a lane
// reset.  Returns a distinct non-zero code per failed check and prints the
// error figures it accepts (max-abs <= 2e-2, mean-abs <= 2e-3 on bf16 outputs;
// cache/state slot placement exact).
#include <array>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "runtime.h"
#include "tatara_oracle.h"

using namespace tatara::runtime;
using namespace tatara::backend::hip;

namespace {

constexpr std::uint32_t kCapacity = 1024;
constexpr std::uint32_t kLanes = 3;

std::vector<std::uint16_t> gauss16(std::uint64_t seed, std::size_t n, double sigma = 1.0) {
    std::vector<std::uint16_t> v(n);
    tto_fill_gaussian_bf16(seed, 0.0, sigma, v.data(), n);
    return v;
}
std::vector<float> gauss32(std::uint64_t seed, std::size_t n, double sigma) {
    std::vector<float> v(n);
    tto_fill_gaussian_f32(seed, 0.0, sigma, v.data(), n);
    return v;
}

template <typename T> bool upload(const HipBuffer& b, const std::vector<T>& v, std::uint64_t off = 0) {
    return tt_buffer_write(b.native(), off, v.data(), v.size() * sizeof(T)) == TT_OK;
}
template <typename T> std::vector<T> download(const HipBuffer& b, std::size_t n, std::uint64_t off = 0) {
    std::vector<T> v(n);
    if (tt_buffer_read(b.native(), off, v.data(), n * sizeof(T)) != TT_OK) v.clear();
    return v;
}

// max-abs 2e-2 / mean-abs 2e-3; steps > 0 widens the max-abs bar to that many
// bf16 steps of the expected value where a step is larger than the bar.
bool close16(const std::vector<std::uint16_t>& got, const std::uint16_t* want, std::size_t n,
             const char* what, int steps = 0) {
    if (got.size() != n) return false;
    double max_abs = 0.0, sum = 0.0;
    bool inside = true;
    for (std::size_t i = 0; i < n; ++i) {
        const double w = tto_f32_from_bf16(want[i]);
        const double e = std::fabs(double(tto_f32_from_bf16(got[i])) - w);
        if (!(e == e)) return false;
        double bar = 2e-2;
        if (steps > 0 && w != 0.0) {
            bar = std::max(bar, steps * std::exp2(std::floor(std::log2(std::fabs(w))) - 7.0));
        }
        inside = inside && e <= bar;
        max_abs = std::max(max_abs, e);
        sum += e;
    }
    std::printf("[parity] %s: max-abs %.3e mean-abs %.3e\n", what, max_abs, sum / double(n));
    std::fflush(stdout);
    return inside && sum / double(n) <= 2e-3;
}
bool close32(const std::vector<float>& got, const std::vector<float>& want, const char* what) {
    if (got.size() != want.size()) return false;
    double max_abs = 0.0;
    for (std::size_t i = 0; i < got.size(); ++i) {
        max_abs = std::max(max_abs, std::fabs(double(got[i]) - want[i]));
    }
    std::printf("[parity] %s: max-abs %.3e\n", what, max_abs);
    std::fflush(stdout);
    return max_abs <= 2e-3;
}

struct Weights {
    std::vector<std::uint16_t> conv_w, a_log, dt_bias, norm_w, q_norm, k_norm;
    HipBuffer b_conv_w, b_a_log, b_dt_bias, b_norm_w, b_q_norm, b_k_norm;
};

struct Submit {
    const HipCommandQueue& queue;
    // encodes `body` into one compute pass, commits, waits; 0 on success
    template <typename Body> int run(Body body) const {
        auto cb = create_command_buffer(queue);
        if (!cb) return 1;
        auto pass = begin_compute_pass(std::move(*cb.command_buffer));
        if (!pass) return 2;
        const HipCommandError encoded = body(*pass.compute_pass);
        if (encoded != HipCommandError::None) {
            std::printf("encode error %d\n", int(encoded));
            return 3;
        }
        auto ended = end_compute_pass(std::move(*pass.compute_pass));
        if (!ended) return 4;
        auto pending = commit(std::move(*ended.command_buffer));
        if (!pending) return 5;
        const HipExecutionResult done = wait_until_completed(std::move(*pending.pending_execution));
        if (!done) {
            std::printf("execution failed: %s\n", done.failure_description.data());
            return 6;
        }
        return 0;
    }
};

}  // namespace

int main() {
    auto device = create_system_device();
    if (!device) return 1;
    auto queue = create_command_queue(*device.device);
    auto library = create_kernel_library(*device.device);
    if (!queue || !library) return 2;
    auto decode_pipes = resolve_decode_pipelines(*library.library);
    auto prefill_pipes = resolve_prefill_pipelines(*library.library);
    if (!decode_pipes || !prefill_pipes) return 3;
    const Submit submit{*queue.command_queue};

    auto plan = tatara::model::qwen36::qwen36_35b_a3b_plan();
    plan.layers = tatara::model::qwen36::make_hybrid_layer_schedule(4, 4, 3);
    const DecodeGeometry geometry = make_decode_geometry(plan, kCapacity);
    auto made = create_decode_step(*device.device, geometry, kCapacity, plan.layers,
                                   std::move(*decode_pipes.pipelines));
    if (!made) return 4;
    DecodeStep& step = *made.step;
    if (!decode_state_slot_ready(step, step.state)) return 5;

    // per-layer weights
    std::vector<Weights> weights(4);
    std::vector<LayerWeights> bound(4);
    for (std::size_t l = 0; l < 4; ++l) {
        Weights& w = weights[l];
        w.conv_w = gauss16(100 + l, 4 * 8192, 0.5);
        w.a_log.assign(32, 0xC040);  // -3.0
        w.dt_bias = gauss16(120 + l, 32, 0.3);
        w.norm_w.assign(128, 0x3F80);
        w.q_norm.assign(256, 0x3F80);
        w.k_norm.assign(256, 0x3F80);
        HipBuffer* dst[6] = {&w.b_conv_w, &w.b_a_log, &w.b_dt_bias, &w.b_norm_w, &w.b_q_norm,
                             &w.b_k_norm};
        const std::vector<std::uint16_t>* src[6] = {&w.conv_w, &w.a_log, &w.dt_bias, &w.norm_w,
                                                    &w.q_norm, &w.k_norm};
        for (int i = 0; i < 6; ++i) {
            auto b = create_shared_buffer(*device.device, src[i]->size() * 2);
            if (!b) return 6;
            *dst[i] = std::move(*b.buffer);
            if (!upload(*dst[i], *src[i])) return 7;
        }
        bound[l] = LayerWeights{&w.b_conv_w, &w.b_a_log, &w.b_dt_bias,
                                &w.b_norm_w, &w.b_q_norm, &w.b_k_norm};
    }

    // ---- pooled lanes, two batched token steps -------------------------------
    auto pooled = create_decode_state_slot_pool(*device.device, step, kLanes);
    if (!pooled) return 10;
    auto batch_made = create_decode_batch_scratch(*device.device, step, kLanes);
    if (!batch_made) return 11;
    DecodeBatchScratch& batch = *batch_made.scratch;
    batch.split_keys = 256;
    std::uint32_t contexts[kLanes] = {700, 100, 300};
    const std::uint32_t stripes[kLanes] = {2, 0, 1};  // lane r lives on stripe stripes[r]
    // host copies of every lane's state (the checker's side)
    struct LaneState {
        std::vector<std::uint16_t> conv[3];
        std::vector<float> rec[3];
        std::vector<std::uint16_t> keys, values;
    };
    std::vector<LaneState> lanes(kLanes);
    for (std::uint32_t r = 0; r < kLanes; ++r) {
        DecodeStateSlot& slot = pooled.slots[stripes[r]];
        for (int l = 0; l < 3; ++l) {
            lanes[r].conv[l] = gauss16(1000 + r * 10 + l, 3 * 8192, 0.5);
            lanes[r].rec[l] = gauss32(2000 + r * 10 + l, 32 * 128 * 128, 0.02);
            if (!upload(slot.layers[l].first, lanes[r].conv[l]) ||
                !upload(slot.layers[l].second, lanes[r].rec[l])) {
                return 12;
            }
        }
        lanes[r].keys.assign(2 * kCapacity * 256, 0);
        lanes[r].values.assign(2 * kCapacity * 256, 0);
        const auto k = gauss16(3000 + r, 2 * kCapacity * 256);
        const auto v = gauss16(4000 + r, 2 * kCapacity * 256);
        for (std::uint32_t h = 0; h < 2; ++h) {
            const std::size_t n = std::size_t{contexts[r]} * 256;
            std::memcpy(&lanes[r].keys[h * kCapacity * 256], &k[h * kCapacity * 256], n * 2);
            std::memcpy(&lanes[r].values[h * kCapacity * 256], &v[h * kCapacity * 256], n * 2);
        }
        if (!upload(slot.layers[3].first, lanes[r].keys) ||
            !upload(slot.layers[3].second, lanes[r].values)) {
            return 13;
        }
    }
    const LayerStageHooks no_hooks{};
    for (int token = 0; token < 2; ++token) {
        std::vector<std::uint16_t> gdn_proj, attn_proj;
        for (std::uint32_t r = 0; r < kLanes; ++r) {
            const auto g = gauss16(5000 + token * 10 + r, 12352, 0.5);
            const auto a = gauss16(6000 + token * 10 + r, 9216);
            gdn_proj.insert(gdn_proj.end(), g.begin(), g.end());
            attn_proj.insert(attn_proj.end(), a.begin(), a.end());
        }
        if (!upload(batch.gdn_projection, gdn_proj) || !upload(batch.attn_projection, attn_proj)) {
            return 14;
        }
        std::vector<DecodeStream> streams;
        for (std::uint32_t r = 0; r < kLanes; ++r) {
            streams.push_back({&pooled.slots[stripes[r]], contexts[r], stripes[r]});
        }
        const int rc = submit.run([&](HipComputePass& pass) {
            return encode_token_batch(step, streams, *pooled.pool, batch, bound, no_hooks, pass);
        });
        if (rc != 0) return 20 + rc;
        const auto gated = download<std::uint16_t>(batch.gdn_gated, kLanes * 4096);
        const auto attended = download<std::uint16_t>(batch.attn_attended, kLanes * 4096);
        for (std::uint32_t r = 0; r < kLanes; ++r) {
            DecodeStateSlot& slot = pooled.slots[stripes[r]];
            std::vector<std::uint16_t> want_gated(4096);
            for (int l = 0; l < 3; ++l) {
                std::vector<std::uint16_t> ncs(3 * 8192);
                std::vector<float> so(32 * 128 * 128);
                tto_gdn_decode_step(&gdn_proj[r * 12352], lanes[r].conv[l].data(),
                                    weights[l].conv_w.data(), weights[l].a_log.data(),
                                    weights[l].dt_bias.data(), weights[l].norm_w.data(),
                                    lanes[r].rec[l].data(), ncs.data(), so.data(),
                                    want_gated.data(), 4);
                const DecodeLayerState& s = slot.layers[l];
                const HipBuffer& conv_out = s.swapped ? s.first : s.first_out;
                const HipBuffer& rec_out = s.swapped ? s.second : s.second_out;
                if (download<std::uint16_t>(conv_out, 3 * 8192) != ncs) return 30 + l;
                if (!close32(download<float>(rec_out, so.size()), so, "pooled recurrent state")) {
                    return 33 + l;
                }
                lanes[r].conv[l] = ncs;
                lanes[r].rec[l] = so;
            }
            if (!close16(std::vector<std::uint16_t>(gated.begin() + r * 4096,
                                                    gated.begin() + (r + 1) * 4096),
                         want_gated.data(), 4096, "batched gdn gated (layer 2)")) {
                return 36;
            }
            std::vector<std::uint16_t> q(4096), gate(4096), want(4096);
            tto_attn_qk_rope(&attn_proj[r * 9216], weights[3].q_norm.data(),
                             weights[3].k_norm.data(), contexts[r], kCapacity, q.data(), gate.data(),
                             lanes[r].keys.data(), lanes[r].values.data());
            tto_attention_decode_split(q.data(), gate.data(), lanes[r].keys.data(),
                                       lanes[r].values.data(), contexts[r], kCapacity, 256, nullptr,
                                       want.data(), 4);
            if (!close16(std::vector<std::uint16_t>(attended.begin() + r * 4096,
                                                    attended.begin() + (r + 1) * 4096),
                         want.data(), 4096, "batched attention")) {
                return 37;
            }
            // the appended V row is a raw copy at exactly (head, context)
            const auto got_v = download<std::uint16_t>(slot.layers[3].second, 2 * kCapacity * 256);
            if (got_v != lanes[r].values) return 38;
            advance_decode_state(step, slot);
            contexts[r] += 1;
        }
        for (int l = 0; l < 3; ++l) {
            if (pooled.slots[0].layers[l].swapped != (token == 0)) return 39;
        }
    }

    // ---- block prefill on a private slot: 100 rows in chunks of 64, with the
    // register-loop recurrence and then with the chunked MFMA recurrence --------
    auto slot_made = create_decode_state_slot(*device.device, step);
    if (!slot_made) return 50;
    DecodeStateSlot& slot = *slot_made.slot;
    std::vector<std::uint16_t> final_values, conv0_final;
    for (const bool chunked : {false, true}) {
    if (chunked) {  // fresh planes for the second pass
        auto again = create_decode_state_slot(*device.device, step);
        if (!again) return 50;
        slot = std::move(*again.slot);
    }
    std::printf("[case] block prefill, gdn_chunked=%d\n", int(chunked));
    const PrefillPolicy policy{.schedule = PrefillSchedule::ChunkMajor,
                               .context_capacity = kCapacity,
                               .maximum_block_rows = 64,
                               .first_chunk_rows = 64,
                               .query_tile_rows = 64,
                               .attention_partition = 256,
                               .gdn_gate_hoist = true,
                               .gdn_chunked = chunked};
    const auto pg = make_prefill_geometry(plan, policy);
    if (!pg) return 51;
    auto scratch_made = create_prefill_scratch(*device.device, pg.geometry);
    if (!scratch_made) return 52;
    PrefillScratch& ps = *scratch_made.scratch;
    const std::uint32_t total_rows = 100;
    const std::uint32_t chunks = prefill_chunk_count(policy, 0, total_rows);
    if (chunks != 2) return 53;
    const auto gproj = gauss16(7000, total_rows * 12352, 0.5);
    const auto aproj = gauss16(7001, total_rows * 9216);
    std::vector<std::uint16_t> conv0(3 * 8192, 0), keys(2 * kCapacity * 256, 0),
        values(2 * kCapacity * 256, 0);
    std::vector<float> rec0(32 * 128 * 128, 0.0f);
    for (std::uint32_t c = 0; c < chunks; ++c) {
        const PrefillChunk chunk = prefill_chunk_at(policy, 0, total_rows, c);
        const std::vector<std::uint16_t> gp(gproj.begin() + chunk.offset * 12352,
                                            gproj.begin() + (chunk.offset + chunk.rows) * 12352);
        const std::vector<std::uint16_t> ap(aproj.begin() + chunk.offset * 9216,
                                            aproj.begin() + (chunk.offset + chunk.rows) * 9216);
        if (!upload(ps.gdn_projection, gp) || !upload(ps.attn_projection, ap)) return 54;
        const int rc = submit.run([&](HipComputePass& pass) {
            HipCommandError e = encode_prefill_gated_delta(*prefill_pipes.pipelines, pg.geometry, ps,
                                                           slot.layers[0], bound[0], chunk, c, pass);
            if (e != HipCommandError::None) return e;
            e = memory_barrier(pass);
            if (e != HipCommandError::None) return e;
            return encode_prefill_attention(*prefill_pipes.pipelines, pg.geometry, ps,
                                            slot.layers[3], bound[3], chunk, 0, pass);
        });
        if (rc != 0) return 60 + rc;
        std::vector<std::uint16_t> ncs(3 * 8192), want_gated(chunk.rows * 4096);
        std::vector<float> so(rec0.size());
        tto_gdn_prefill(gp.data(), chunk.rows, conv0.data(), weights[0].conv_w.data(),
                        weights[0].a_log.data(), weights[0].dt_bias.data(), weights[0].norm_w.data(),
                        rec0.data(), ncs.data(), so.data(), want_gated.data(), nullptr, nullptr,
                        nullptr, 4);
        if (!close16(download<std::uint16_t>(ps.gdn_gated, chunk.rows * 4096), want_gated.data(),
                     want_gated.size(), "prefill gdn gated", chunked ? 4 : 0)) {
            return 70;
        }
        // phase = swapped ^ (ordinal & 1): chunk 0 writes the out planes, chunk 1 the in planes
        const bool phase = (c & 1u) != 0u;
        const HipBuffer& conv_out = phase ? slot.layers[0].first : slot.layers[0].first_out;
        const HipBuffer& rec_out = phase ? slot.layers[0].second : slot.layers[0].second_out;
        if (download<std::uint16_t>(conv_out, 3 * 8192) != ncs) return 71;
        if (!close32(download<float>(rec_out, so.size()), so, "prefill recurrent state")) return 72;
        conv0 = ncs;
        rec0 = so;
        std::vector<std::uint16_t> query(chunk.rows * 4096), gate(chunk.rows * 4096),
            want(chunk.rows * 4096);
        tto_attention_prefill(ap.data(), weights[3].q_norm.data(), weights[3].k_norm.data(),
                              chunk.rows, chunk.offset, kCapacity, query.data(), gate.data(),
                              keys.data(), values.data(), nullptr, 0, want.data(), 4);
        if (!close16(download<std::uint16_t>(ps.attn_attended, chunk.rows * 4096), want.data(),
                     want.size(), "prefill attention")) {
            return 73;
        }
    }
    if (download<std::uint16_t>(slot.layers[3].second, values.size()) != values) return 74;
    advance_prefill_state(step, slot, chunks);  // even chunk count: live planes unchanged
    if (slot.layers[0].swapped) return 75;
    if (download<std::uint16_t>(slot.layers[0].first, 3 * 8192) != conv0) return 76;
    final_values = values;
    conv0_final = conv0;
    }

    // ---- lane state record (Q36BRS01): write, install into a fresh slot, round trip --
    {
        std::printf("[case] lane state record\n");
        const std::uint32_t positions = 100;
        // a second gated-delta layer whose live planes are the out planes
        const auto marker_conv = gauss16(9100, 3 * 8192, 0.5);
        std::vector<float> marker_rec(32 * 128 * 128);
        for (std::size_t i = 0; i < marker_rec.size(); ++i) marker_rec[i] = 1e-3f * float(i % 977);
        if (!upload(slot.layers[1].first_out, marker_conv)) return 100;
        if (tt_buffer_write(slot.layers[1].second_out.native(), 0, marker_rec.data(),
                            marker_rec.size() * 4) != TT_OK) {
            return 100;
        }
        slot.layers[1].swapped = true;
        std::vector<std::byte> record;
        if (write_state_record(step, slot, positions, record) != StateRecordError::None) return 101;
        const std::uint64_t gdn_bytes = 3 * 8192 * 2 + 32ull * 128 * 128 * 4;
        const std::uint64_t expect = 12 + 3 * gdn_bytes + 4ull * positions * 512;
        if (record.size() != expect || state_record_bytes(step, positions) != expect) return 102;
        if (state_record_bytes(step, 0) != 0 || state_record_bytes(step, kCapacity + 1) != 0) return 103;
        std::uint32_t stored = 0;
        std::memcpy(&stored, record.data() + 8, 4);
        if (std::memcmp(record.data(), "Q36BRS01", 8) != 0 || stored != positions) return 104;
        // layer 0: the in planes are live; layer 1: the out planes
        if (std::memcmp(record.data() + 12, conv0_final.data(), 3 * 8192 * 2) != 0) return 105;
        if (std::memcmp(record.data() + 12 + gdn_bytes, marker_conv.data(), 3 * 8192 * 2) != 0) return 106;
        if (std::memcmp(record.data() + 12 + gdn_bytes + 3 * 8192 * 2, marker_rec.data(),
                        marker_rec.size() * 4) != 0) {
            return 107;
        }
        // attention layer 3: keys head 0, keys head 1, values head 0, values head 1, packed
        const std::byte* values0 = record.data() + 12 + 3 * gdn_bytes + 2ull * positions * 512;
        if (std::memcmp(values0, final_values.data(), positions * 512) != 0) return 108;
        if (std::memcmp(values0 + positions * 512, final_values.data() + std::size_t{kCapacity} * 256,
                        positions * 512) != 0) {
            return 109;
        }

        auto fresh_made = create_decode_state_slot(*device.device, step);
        if (!fresh_made) return 110;
        DecodeStateSlot& fresh = *fresh_made.slot;
        std::uint32_t context = 0;
        if (load_state_record(record, step, fresh, context) != StateRecordError::None) return 111;
        if (context != positions) return 112;
        if (download<std::uint16_t>(fresh.layers[0].first, 3 * 8192) != conv0_final) return 113;
        if (download<std::uint16_t>(fresh.layers[1].first, 3 * 8192) != marker_conv) return 114;
        if (fresh.layers[1].swapped) return 115;
        if (download<float>(fresh.layers[1].second, marker_rec.size()) != marker_rec) return 116;
        const auto loaded_values = download<std::uint16_t>(fresh.layers[3].second, final_values.size());
        for (std::size_t head = 0; head < 2; ++head) {
            for (std::size_t i = 0; i < std::size_t{kCapacity} * 256; ++i) {
                const std::size_t at = head * kCapacity * 256 + i;
                const std::uint16_t want = i < positions * 256 ? final_values[at] : 0;
                if (loaded_values[at] != want) return 117;
            }
        }
        std::vector<std::byte> again;
        if (write_state_record(step, fresh, positions, again) != StateRecordError::None) return 118;
        if (again != record) return 119;

        // malformed records leave the slot untouched and name the defect
        auto other_made = create_decode_state_slot(*device.device, step);
        if (!other_made) return 120;
        DecodeStateSlot& other = *other_made.slot;
        std::vector<std::byte> bad = record;
        bad[0] = std::byte{'X'};
        if (load_state_record(bad, step, other, context) != StateRecordError::MagicMismatch) return 121;
        bad = record;
        bad.pop_back();
        if (load_state_record(bad, step, other, context) != StateRecordError::Truncated) return 122;
        bad = record;
        bad.push_back(std::byte{0});
        if (load_state_record(bad, step, other, context) != StateRecordError::TrailingBytes) return 123;
        bad = record;
        const std::uint32_t zero = 0, beyond = kCapacity + 1;
        std::memcpy(bad.data() + 8, &zero, 4);
        if (load_state_record(bad, step, other, context) != StateRecordError::InvalidPositions) return 124;
        std::memcpy(bad.data() + 8, &beyond, 4);
        if (load_state_record(bad, step, other, context) != StateRecordError::InvalidPositions) return 125;
        if (load_state_record(std::span<const std::byte>(record.data(), 5), step, other, context) !=
            StateRecordError::Truncated) {
            return 126;
        }
        if (write_state_record(step, slot, 0, again) != StateRecordError::InvalidPositions) return 127;
        for (const float v : download<float>(other.layers[0].second, 64)) {
            if (v != 0.0f) return 128;
        }

        // ---- the same state as a device-resident prefix payload --------------------
        std::printf("[case] prefix snapshot / restore\n");
        const PrefillPolicy policy{.schedule = PrefillSchedule::ChunkMajor,
                                   .context_capacity = kCapacity,
                                   .maximum_block_rows = 64,
                                   .first_chunk_rows = 64,
                                   .query_tile_rows = 64,
                                   .attention_partition = 256,
                                   .gdn_gate_hoist = true,
                                   .gdn_chunked = true};
        const auto pg = make_prefill_geometry(plan, policy);
        if (!pg) return 130;
        const auto made = make_prefix_state_layout(step, pg.geometry, positions);
        if (!made || made.layout.segment_count != 3 * 2 + 4 ||
            made.layout.total_bytes != expect - 12) {
            return 130;
        }
        const std::uint64_t arena_base = 256;
        auto arena_made = tatara::backend::hip::create_shared_buffer(
            *device.device, arena_base + made.layout.total_bytes + 64);
        if (!arena_made) return 131;
        HipBuffer& arena = *arena_made.buffer;
        std::vector<std::uint8_t> guard(arena.size_bytes(), 0xa5);
        if (tt_buffer_write(arena.native(), 0, guard.data(), guard.size()) != TT_OK) return 131;
        std::array<std::byte, 1> evidence{};
        {
            auto cb = create_command_buffer(*queue.command_queue);
            if (!cb) return 132;
            auto blit = begin_blit_pass(std::move(*cb.command_buffer));
            if (!blit) return 132;
            // one byte short of the payload is refused before any copy
            if (encode_prefix_state_snapshot(step, slot, pg.geometry, *blit.blit_pass, arena,
                                             arena_base + 65, positions, evidence)
                        .error != PrefixStateTransferError::ArenaOutOfRange ||
                slot.status != DecodeStateSlotStatus::Ready) {
                return 133;
            }
            PrefixStateTransferResult taken = encode_prefix_state_snapshot(
                step, slot, pg.geometry, *blit.blit_pass, arena, arena_base, positions, evidence);
            if (!taken || taken.segment_count != 10 || taken.state_bytes != made.layout.total_bytes ||
                taken.source_phase_evidence_bytes != 1 || evidence[0] != std::byte{0b010}) {
                return 134;
            }
            if (slot.status != DecodeStateSlotStatus::SnapshotPending ||
                decode_state_slot_ready(step, slot)) {
                return 135;
            }
            auto ended = end_blit_pass(std::move(*blit.blit_pass));
            auto pending = commit(std::move(*ended.command_buffer));
            if (!pending || !wait_until_completed(std::move(*pending.pending_execution))) return 136;
            if (complete_prefix_state_transfer(*taken.ticket, step, slot, arena) !=
                    PrefixStateTransferError::None ||
                slot.status != DecodeStateSlotStatus::Ready || !slot.layers[1].swapped) {
                return 137;
            }
        }
        // payload == the record's pieces, family-major; the guard bytes either side survive
        const auto image = download<std::uint8_t>(arena, arena.size_bytes());
        for (std::size_t i = 0; i < arena_base; ++i) {
            if (image[i] != 0xa5) return 138;
        }
        for (std::size_t i = arena_base + made.layout.total_bytes; i < image.size(); ++i) {
            if (image[i] != 0xa5) return 138;
        }
        // schedule is G G G A, so the record body and the payload coincide byte for byte
        if (std::memcmp(image.data() + arena_base, record.data() + 12, made.layout.total_bytes) != 0) {
            return 139;
        }
        {
            auto target_made = create_decode_state_slot(*device.device, step);
            if (!target_made) return 140;
            DecodeStateSlot& target = *target_made.slot;
            target.layers[0].swapped = true;  // the recipient's own phase does not matter
            auto cb = create_command_buffer(*queue.command_queue);
            if (!cb) return 141;
            auto blit = begin_blit_pass(std::move(*cb.command_buffer));
            if (!blit) return 141;
            PrefixStateTransferResult put = encode_prefix_state_restore(
                step, target, pg.geometry, *blit.blit_pass, arena, arena_base, positions);
            if (!put || target.status != DecodeStateSlotStatus::RestorePending) return 142;
            // a lane with a transfer in flight admits no second one
            if (encode_prefix_state_restore(step, target, pg.geometry, *blit.blit_pass, arena,
                                            arena_base, positions)
                    .error != PrefixStateTransferError::StateSlotNotReady) {
                return 143;
            }
            auto ended = end_blit_pass(std::move(*blit.blit_pass));
            auto pending = commit(std::move(*ended.command_buffer));
            if (!pending || !wait_until_completed(std::move(*pending.pending_execution))) return 144;
            if (complete_prefix_state_transfer(*put.ticket, step, target, arena) !=
                    PrefixStateTransferError::None ||
                target.layers[0].swapped || target.layers[1].swapped) {
                return 145;
            }
            std::vector<std::byte> from_target;
            if (write_state_record(step, target, positions, from_target) != StateRecordError::None ||
                from_target != record) {
                return 146;
            }
            // rows past the prefix were not touched
            const auto target_keys = download<std::uint16_t>(target.layers[3].first, 2 * kCapacity * 256);
            for (std::size_t i = positions * 256; i < std::size_t{kCapacity} * 256; ++i) {
                if (target_keys[i] != 0) return 147;
            }
        }

        // ---- a taped block of 12 rows rolled back to its first 5 -------------------
        std::printf("[case] taped block, rollback to a prefix\n");
        PrefillPolicy tape_policy = policy;
        tape_policy.maximum_block_rows = tape_policy.first_chunk_rows =
            tape_policy.query_tile_rows = 16;
        tape_policy.gdn_chunked = false;
        PrefillPolicy plain_policy = tape_policy;
        tape_policy.gdn_tape = true;
        {
            PrefillPolicy refused = tape_policy;
            refused.gdn_chunked = true;
            if (make_prefill_geometry(plan, refused).error != PrefillGeometryError::InvalidPolicy) {
                return 150;
            }
            refused = tape_policy;
            refused.gdn_gate_hoist = false;
            if (make_prefill_geometry(plan, refused).error != PrefillGeometryError::InvalidPolicy) {
                return 150;
            }
        }
        const auto taped_geometry = make_prefill_geometry(plan, tape_policy);
        const auto plain_geometry = make_prefill_geometry(plan, plain_policy);
        if (!taped_geometry || !plain_geometry) return 151;
        if (taped_geometry.geometry.gdn_tape_bytes != 15'892'480ull ||
            taped_geometry.geometry.gdn_conv_tape_bytes != 31'457'280ull ||
            plain_geometry.geometry.gdn_tape_bytes != 0) {
            return 152;
        }
        auto taped_scratch_made = create_prefill_scratch(*device.device, taped_geometry.geometry);
        auto plain_scratch_made = create_prefill_scratch(*device.device, plain_geometry.geometry);
        if (!taped_scratch_made || !plain_scratch_made) return 153;
        PrefillScratch& taped_scratch = *taped_scratch_made.scratch;
        PrefillScratch& plain_scratch = *plain_scratch_made.scratch;
        const std::uint32_t block_rows = 12, committed = 5;
        const auto block = gauss16(7100, block_rows * 12352, 0.5);
        const std::vector<std::uint16_t> prefix(block.begin(), block.begin() + committed * 12352);
        auto lane_a_made = create_decode_state_slot(*device.device, step);
        auto lane_b_made = create_decode_state_slot(*device.device, step);
        if (!lane_a_made || !lane_b_made) return 154;
        DecodeStateSlot& lane_a = *lane_a_made.slot;
        DecodeStateSlot& lane_b = *lane_b_made.slot;
        std::uint32_t base_a = 0, base_b = 0;
        if (load_state_record(record, step, lane_a, base_a) != StateRecordError::None ||
            load_state_record(record, step, lane_b, base_b) != StateRecordError::None) {
            return 155;
        }
        const auto run_block = [&](const PrefillGeometry& geometry, PrefillScratch& scratch,
                                   DecodeStateSlot& lane, std::uint32_t rows) {
            const PrefillChunk chunk{0, rows, 0};
            return submit.run([&](HipComputePass& pass) {
                for (std::uint32_t layer = 0; layer < 3; ++layer) {
                    HipCommandError e = encode_prefill_gated_delta(
                        *prefill_pipes.pipelines, geometry, scratch, lane.layers[layer],
                        bound[layer], chunk, 0, pass, layer);
                    if (e != HipCommandError::None) return e;
                    e = memory_barrier(pass);
                    if (e != HipCommandError::None) return e;
                }
                return HipCommandError::None;
            });
        };
        // lane A: the whole block with the tape on, then back to `committed` rows
        if (!upload(taped_scratch.gdn_projection, block)) return 156;
        if (run_block(taped_geometry.geometry, taped_scratch, lane_a, block_rows) != 0) return 157;
        {
            HipComputePass no_pass;
            if (encode_gdn_tape_replay(*prefill_pipes.pipelines, step, lane_a, taped_scratch, 0,
                                       no_pass) != HipCommandError::InvalidDispatchExtent ||
                encode_gdn_tape_replay(*prefill_pipes.pipelines, step, lane_a, taped_scratch, 17,
                                       no_pass) != HipCommandError::InvalidDispatchExtent ||
                encode_gdn_tape_replay(*prefill_pipes.pipelines, step, lane_a, plain_scratch,
                                       committed, no_pass) != HipCommandError::InvalidBuffer) {
                return 158;
            }
        }
        if (submit.run([&](HipComputePass& pass) {
                return encode_gdn_tape_replay(*prefill_pipes.pipelines, step, lane_a, taped_scratch,
                                              committed, pass);
            }) != 0) {
            return 159;
        }
        {
            auto cb = create_command_buffer(*queue.command_queue);
            if (!cb) return 160;
            auto blit = begin_blit_pass(std::move(*cb.command_buffer));
            if (!blit) return 160;
            if (encode_gdn_tape_windows(step, lane_a, taped_scratch, committed, *blit.blit_pass) !=
                HipCommandError::None) {
                return 161;
            }
            auto ended = end_blit_pass(std::move(*blit.blit_pass));
            auto pending = commit(std::move(*ended.command_buffer));
            if (!pending || !wait_until_completed(std::move(*pending.pending_execution))) return 162;
        }
        complete_gdn_tape_rollback(step, lane_a);
        // lane B: only the committed rows, no tape
        if (!upload(plain_scratch.gdn_projection, prefix)) return 163;
        if (run_block(plain_geometry.geometry, plain_scratch, lane_b, committed) != 0) return 164;
        advance_prefill_state(step, lane_b, 1);
        if (!lane_a.layers[0].swapped || !lane_b.layers[0].swapped) return 165;
        std::vector<std::byte> record_a, record_b;
        if (write_state_record(step, lane_a, positions, record_a) != StateRecordError::None ||
            write_state_record(step, lane_b, positions, record_b) != StateRecordError::None) {
            return 166;
        }
        if (record_a == record) return 167;  // the block did change the state
        if (record_a != record_b) return 168;
        slot.layers[1].swapped = false;
    }

    // ---- lane reset -----------------------------------------------------------
    {
        auto cb = create_command_buffer(*queue.command_queue);
        if (!cb) return 80;
        auto blit = begin_blit_pass(std::move(*cb.command_buffer));
        if (!blit) return 81;
        slot.layers[0].swapped = true;
        StateSlotResetResult reset = encode_state_slot_reset(step, slot, *blit.blit_pass);
        if (reset.error != StateSlotResetError::None || !reset.ticket ||
            reset.segment_count != 6 || reset.state_bytes != 3ull * (49152 + 2097152)) {
            return 82;
        }
        if (slot.status != DecodeStateSlotStatus::ResetPending) return 83;
        if (decode_state_slot_available(step, slot)) return 84;
        auto ended = end_blit_pass(std::move(*blit.blit_pass));
        auto pending = commit(std::move(*ended.command_buffer));
        if (!pending || !wait_until_completed(std::move(*pending.pending_execution))) return 85;
        if (complete_state_slot_reset(*reset.ticket, step, slot) != StateSlotResetError::None) {
            return 86;
        }
        if (slot.status != DecodeStateSlotStatus::Ready || slot.layers[0].swapped) return 87;
        for (const float v : download<float>(slot.layers[0].second, 32 * 128 * 128)) {
            if (v != 0.0f) return 88;
        }
        if (complete_state_slot_reset(*reset.ticket, step, slot) !=
            StateSlotResetError::AlreadyCompleted) {
            return 89;
        }
        // attention KV is never cleared by a reset
        if (download<std::uint16_t>(slot.layers[3].second, final_values.size()) != final_values) {
            return 90;
        }
    }
    std::printf("runtime gpu test ok\n");
    return 0;
}
