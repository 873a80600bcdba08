// tatara::runtime — host side of the attention-family path over the HIP
// backend: model plan, buffer geometry, per-lane state slots and striped pools,
// the state-offset table of a lane batch, the per-token layer walk and the
// block-prefill layer walk.  Types and functions keep the reference's names and
// meaning (include/tatara/runtime/{decode_geometry,decode_step,
// prefill_geometry}.h, src/runtime/{decode_step,prefill_step,
// state_slot_reset}.cpp) so call sites and contract tests read the same; only
// the attention and Gated DeltaNet branches of the walk are real.  The stages
// around them (input norm, Q4 projections, MoE, LM head) are a caller-supplied
// hook: this repository ships a bf16 dense stand-in for them (StackStages).
#pragma once

#include <cstddef>
#include <cstdint>
#include <optional>
#include <span>
#include <vector>

#include "backend_hip.h"

namespace tatara::model::qwen36 {

// include/tatara/model/qwen36_plan.h:12-15
enum class LayerKind : std::uint8_t { GatedDelta, FullAttention };

// The fields of StaticModelPlan (qwen36_plan.h:118-131) the path depends on.
struct ModelPlan {
    std::uint32_t hidden;
    std::uint32_t vocabulary;
    std::uint32_t query_heads;
    std::uint32_t key_value_heads;
    std::uint32_t head_dimension;
    std::uint32_t recurrent_heads;
    std::uint32_t state_dimension;
    std::uint32_t initial_serving_capacity;
    std::vector<LayerKind> layers;
};

// qwen36-35b-a3b (catalog/model_packages/qwen36-35b-a3b/model.toml:9-34):
// 40 layers, full attention at 3, 7, ..., 39 (make_hybrid_layer_schedule,
// qwen36_plan.h:101-113 with period 4, first 3).
ModelPlan qwen36_35b_a3b_plan();
std::vector<LayerKind> make_hybrid_layer_schedule(std::size_t layer_count, std::size_t period,
                                                  std::size_t first);

}  // namespace tatara::model::qwen36

namespace tatara::runtime {

using backend::hip::HipBuffer;
using backend::hip::HipCommandError;
using backend::hip::HipComputePass;
using backend::hip::HipBlitPass;
using backend::hip::HipComputePipeline;
using backend::hip::HipDevice;
using backend::hip::HipLibrary;
using model::qwen36::LayerKind;

inline constexpr std::uint32_t kAttentionRecordFloats = 258;   // decode_geometry.h:111
inline constexpr std::uint32_t kAttentionPartition = 256;      // decode_geometry.h:112
inline constexpr std::uint32_t kConvShiftSteps = 3;
inline constexpr std::uint32_t kGdnChunkRows = 64;             // tokens per chunk of the MFMA recurrence
inline constexpr std::uint32_t kGdnChunkRecordBytes = 115712;  // scratch per (chunk, value head)
inline constexpr std::uint32_t kGdnChunkGroupRows = 2048;      // rows whose records are live at once
inline constexpr std::uint32_t kGdnTapeRows = 16;              // rows a rollback tape holds
inline constexpr std::uint32_t kGdnTapeLayers = 40;            // layers the tape is laid out for
inline constexpr std::uint64_t kGdnTapeBytes =                 // prefill_step.cpp:3231-3233
    std::uint64_t{40} * 16u * (32u * 128u + 16u * 128u + 64u) * 4u;
inline constexpr std::uint64_t kGdnConvTapeBytes =             // prefill_step.cpp:3235-3237
    std::uint64_t{40} * 16u * 3u * 8192u * 2u;
inline constexpr std::uint32_t kBf16Bytes = 2;
inline constexpr std::uint32_t kF32Bytes = 4;
inline constexpr std::uint32_t kMaximumBatchRows = 16;         // decode_step.cpp:554, 1008
inline constexpr std::uint32_t kPrefillMaximumContext = 262144;   // prefill_geometry.h:14
inline constexpr std::uint32_t kPrefillMaximumBlockRows = 2048;   // prefill_geometry.h:15
inline constexpr std::uint32_t kPrefillQueryTileMultiple = 16;    // prefill_geometry.h:16

// decode_geometry.h:133-135
constexpr bool context_in_capacity(std::uint32_t context, std::uint32_t capacity) {
    return capacity != 0 && context < capacity;
}

struct DispatchShape {
    std::uint32_t groups;
    std::uint32_t threads;
};
struct RecurrenceDispatch {
    std::uint32_t dimension_groups, head_groups, lane_threads, dimension_threads;
};
struct AttentionSplitDispatch {
    std::uint32_t score_groups, score_threads, score_cohort_threads;
    std::uint32_t value_groups, value_lane_threads, value_dimension_threads, value_head_threads;
};

// Attention-family subset of DecodeGeometry / DecodeDispatch
// (decode_geometry.h:43-108); field names and values are the reference's.
struct DecodeGeometry {
    std::uint32_t gated_delta_layers;
    std::uint32_t attention_layers;
    std::uint64_t hidden_bytes;
    std::uint64_t layer_stream_bytes;
    std::uint64_t gdn_projection_bytes;
    std::uint64_t gdn_qk_bytes;
    std::uint64_t gdn_value_bytes;
    std::uint64_t gdn_gate_bytes;
    std::uint64_t gdn_conv_state_bytes;
    std::uint64_t gdn_recurrent_state_bytes;
    std::uint64_t attn_projection_bytes;
    std::uint64_t attn_query_bytes;
    std::uint64_t attn_record_scratch_bytes;
    std::uint64_t attn_cache_bytes;
    DispatchShape gdn_prepare;
    RecurrenceDispatch gdn_recurrence;
    DispatchShape gdn_gate_norm;
    DispatchShape attn_qk_rope;
    DispatchShape attention_head;
    AttentionSplitDispatch attention_split;
    DispatchShape rms;
};

DecodeGeometry make_decode_geometry(const model::qwen36::ModelPlan& plan, std::uint32_t capacity);

// decode_step.cpp:15-19
std::uint32_t attention_partitions(std::uint32_t context);

// decode_step.h:66-100
struct DecodeLayerState {
    HipBuffer first;
    HipBuffer first_out;
    HipBuffer second;
    HipBuffer second_out;
    bool swapped{false};
};

enum class DecodeStateSlotStatus : std::uint8_t {
    Ready,
    SnapshotPending,
    RestorePending,
    ResetPending,
    Poisoned,
};

struct DecodeStateSlot {
    std::uint32_t capacity{0};
    const LayerKind* schedule_identity{nullptr};
    std::vector<DecodeLayerState> layers;
    DecodeStateSlotStatus status{DecodeStateSlotStatus::Ready};
    std::uint64_t next_transfer_generation{1};
    std::uint64_t active_transfer_generation{0};
    const HipBuffer* active_transfer_arena{nullptr};
    std::uint32_t active_transfer_positions{0};
    std::uint64_t active_transfer_offset_bytes{0};
    std::uint64_t active_transfer_state_bytes{0};
    std::uint64_t next_reset_generation{1};
    std::uint64_t active_reset_generation{0};
    std::uint32_t active_reset_segments{0};
    std::uint64_t active_reset_bytes{0};
};

enum class DecodeStepError : std::uint8_t {
    None,
    InvalidDevice,
    InvalidImage,
    OffsetCountMismatch,
    BufferAllocationFailed,
};

// Pipelines of the attention-family walk, resolved by name from the kernel
// library (decode_step.h:26-61, 322-345).  attention_split_ms/combine_ms fold
// every long row of a batch into one split-K grid; the reference re-dispatches
// the one-lane split path per long row (decode_step.cpp:1249-1259).
struct DecodePipelines {
    HipComputePipeline gdn_prepare, gdn_recurrence, gdn_gate_norm;
    HipComputePipeline attn_qk_rope, attention_decode, attention_scores_values_fused,
        attention_combine;
    HipComputePipeline gdn_prepare_ms, gdn_recurrence_ms, gate_norm_ms, gdn_decode_fused_ms;
    HipComputePipeline attn_qk_rope_ms, attention_decode_ms, attention_split_ms,
        attention_combine_ms;
    HipComputePipeline attention_token_ms, attention_token_finish_ms;
};
struct DecodePipelinesResult {
    backend::hip::HipPipelineError error;
    std::optional<DecodePipelines> pipelines;
    explicit operator bool() const noexcept {
        return error == backend::hip::HipPipelineError::None && pipelines.has_value();
    }
};
DecodePipelinesResult resolve_decode_pipelines(const HipLibrary& library);

// Every per-token buffer as a [rows x stride] slab (decode_step.h:202-231,
// 281-305); strides are the single-stream byte sizes of DecodeGeometry.
struct DecodeBatchScratch {
    std::uint32_t rows{0};
    HipBuffer gdn_projection, gdn_qk, gdn_value, gdn_z, gdn_y, gdn_gated;
    HipBuffer attn_projection, attn_query, attn_gate, attn_attended, attn_partials;
    HipBuffer state_offsets;
    // keys per split-K workgroup of the batched path (a multiple of 32); 0: chosen for
    // every wave from the depths of its rows by choose_split_keys
    std::uint32_t split_keys{0};
    // compute units of the device the scratch was made on: what the automatic split fills
    std::uint32_t compute_units{256};
    // One dispatch per Gated DeltaNet layer (gdn_decode_fused_ms) instead of the
    // reference's prepare / recurrence / gate-norm triple; same results bit for bit.
    bool gdn_fused{true};
    // The attention layer of a wave as attention_decode_token_ms +
    // attention_decode_token_finish_ms (norm and rotation inside the split-K walk over the
    // cached keys; the token's own key and value folded in, and appended, by the finishing
    // dispatch) instead of rope, split path, combine and the short-row bucket: every row
    // through the same two dispatches, records in `attn_partials`.  The default: a 40-layer
    // wave is 2 to 7 % shorter with it (one dispatch less per attention layer), at any depth.
    bool attention_token_form{true};
};

// Keys per split-K workgroup for one attention layer of a wave whose rows see
// `visible_keys[r]` keys each: the finest multiple of 32, at least 128, with which the
// workgroups that hold keys (two kv heads x the rows' ceil(keys / split)) fit the compute
// units one each.  The second form: `rows` rows at the same depth.
std::uint32_t choose_split_keys(std::span<const std::uint32_t> visible_keys,
                                std::uint32_t compute_units = 256) noexcept;
std::uint32_t choose_split_keys(std::uint32_t rows, std::uint32_t keys,
                                std::uint32_t compute_units = 256) noexcept;
// Workgroups of that layer's split-K grid that hold keys.
std::uint32_t split_workgroups(std::span<const std::uint32_t> visible_keys,
                               std::uint32_t split_keys) noexcept;

// The step: geometry, schedule and pipelines; its own primary slot (decode_step.h:115-153).
struct DecodeStep {
    DecodeGeometry geometry{};
    std::uint32_t capacity{0};
    std::vector<LayerKind> schedule;
    DecodePipelines pipelines;
    DecodeStateSlot state;
};
struct DecodeStepResult {
    DecodeStepError error;
    std::optional<DecodeStep> step;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && step.has_value();
    }
};
struct DecodeStateSlotResult {
    DecodeStepError error;
    std::optional<DecodeStateSlot> slot;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && slot.has_value();
    }
};

// decode_step.h:177-197
struct DecodeStatePoolLayer {
    HipBuffer first;
    HipBuffer second;
    std::uint64_t first_stride{0};
    std::uint64_t second_stride{0};
};
struct DecodeStatePool {
    std::uint32_t stripes{0};
    std::vector<DecodeStatePoolLayer> layers;
};
struct DecodeStateSlotPoolResult {
    DecodeStepError error;
    std::optional<DecodeStatePool> pool;
    std::vector<DecodeStateSlot> slots;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && pool.has_value();
    }
};
struct DecodeBatchScratchResult {
    DecodeStepError error;
    std::optional<DecodeBatchScratch> scratch;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && scratch.has_value();
    }
};

// decode_step.h:245-250
struct DecodeStream {
    DecodeStateSlot* state{nullptr};
    std::uint32_t context{0};
    std::uint32_t stripe{0};
};

DecodeStepResult create_decode_step(const HipDevice& device, const DecodeGeometry& geometry,
                                    std::uint32_t capacity, std::span<const LayerKind> schedule,
                                    DecodePipelines pipelines);
DecodeStateSlotResult create_decode_state_slot(const HipDevice& device, const DecodeStep& step);
DecodeStateSlotPoolResult create_decode_state_slot_pool(const HipDevice& device,
                                                        const DecodeStep& step,
                                                        std::uint32_t count);
DecodeBatchScratchResult create_decode_batch_scratch(const HipDevice& device,
                                                     const DecodeStep& step, std::uint32_t rows);

bool decode_state_slot_compatible(const DecodeStep& step, const DecodeStateSlot& state) noexcept;
bool decode_state_slot_complete(const DecodeStep& step, const DecodeStateSlot& state) noexcept;
bool decode_state_slot_available(const DecodeStep& step, const DecodeStateSlot& state) noexcept;
bool decode_state_slot_ready(const DecodeStep& step, const DecodeStateSlot& state) noexcept;

// Host image of the per-layer state-offset table of a lane batch: 64 u32 per
// layer (16 rows x 4), then the bucket list of short-context rows
// (decode_step.cpp:1037-1071).  Pure integers; exact by construction.
struct StateOffsetTable {
    std::vector<std::uint32_t> words;   // layers*64 entries + 16 bucket rows
    std::uint32_t bucket_rows{0};
};
HipCommandError build_state_offset_table(const DecodeStep& step,
                                         std::span<const DecodeStream> streams,
                                         const DecodeStatePool& pool, StateOffsetTable& out);

// Stages of the walk outside the attention family.  project() must fill
// scratch.gdn_projection / attn_projection ([rows][stride] bf16) for `layer`
// from the caller's hidden stream; finish() consumes scratch.gdn_gated /
// attn_attended.  Both encode into the same pass; returning an error aborts
// the walk.  A null hook leaves the projection slabs as the caller filled them.
struct LayerStageHooks {
    void* user{nullptr};
    HipCommandError (*project)(void* user, HipComputePass& pass, std::size_t layer, LayerKind kind,
                               std::uint32_t rows){nullptr};
    HipCommandError (*finish)(void* user, HipComputePass& pass, std::size_t layer, LayerKind kind,
                              std::uint32_t rows){nullptr};
};

struct LayerWeights {
    // GatedDelta: conv_weight [8192][4], a_log [32], dt_bias [32], norm_weight [128];
    // FullAttention: query_norm [256], key_norm [256] (all bf16).
    const HipBuffer* conv_weight{nullptr};
    const HipBuffer* a_log{nullptr};
    const HipBuffer* dt_bias{nullptr};
    const HipBuffer* norm_weight{nullptr};
    const HipBuffer* query_norm{nullptr};
    const HipBuffer* key_norm{nullptr};
};

// One batched token step for up to 16 streams over pool-striped slots
// (encode_token_batch, decode_step.cpp:1002-1426, attention-family branches).
// Admission errors (StateSlotMismatch, ContextOutOfRange, InvalidStreamGroup)
// are returned before anything is encoded.  The host writes the state-offset
// table first, so the previous step must have completed.
HipCommandError encode_token_batch(DecodeStep& step, std::span<const DecodeStream> streams,
                                   const DecodeStatePool& pool, DecodeBatchScratch& batch,
                                   std::span<const LayerWeights> weights,
                                   const LayerStageHooks& hooks, HipComputePass& pass);

// One token, one lane, un-batched operators (encode_token, decode_step.cpp:828-842).
HipCommandError encode_token(DecodeStep& step, DecodeStateSlot& state, DecodeBatchScratch& scratch,
                             std::span<const LayerWeights> weights, const LayerStageHooks& hooks,
                             HipComputePass& pass, std::uint32_t context);

// ---- the stages either side of the family, from the model's 4-bit weights ----
// An affine 4-bit matrix, group 64 (decode_bindings.h:17-24): weight [rows][k/8]
// u32, scales and biases [rows][k/64] bf16.
struct QuantizedBinding {
    const HipBuffer* weight{nullptr};
    const HipBuffer* scales{nullptr};
    const HipBuffer* biases{nullptr};
};
// decode_bindings.h:27-48
struct GatedDeltaBindings {
    QuantizedBinding qkv, z, b, a, out;
};
struct AttentionBindings {
    QuantizedBinding query, key, value, out;
};
// The attention-family members of LayerBindings (decode_bindings.h:50-64);
// input_norm and post_norm are [hidden] bf16.
struct LayerBindings {
    const HipBuffer* input_norm{nullptr};
    const HipBuffer* post_norm{nullptr};
    GatedDeltaBindings gated_delta;
    AttentionBindings attention;
};
struct StagePipelines {
    HipComputePipeline rms_ms, residual_rms_ms;
    HipComputePipeline gdn_project_ms, attn_project_ms, gdn_outproj_ms;
    // the same bindings evaluated on the matrix unit (another summation order)
    HipComputePipeline gdn_project_mfma_ms, attn_project_mfma_ms, gdn_outproj_mfma_ms;
};
struct StagePipelinesResult {
    backend::hip::HipPipelineError error;
    std::optional<StagePipelines> pipelines;
    explicit operator bool() const noexcept {
        return error == backend::hip::HipPipelineError::None && pipelines.has_value();
    }
};
StagePipelinesResult resolve_stage_pipelines(const HipLibrary& library);

// The hidden-width rows of one wave (decode_step.h:202-231: input, normed,
// branch_stream, residual_stream), each [rows][hidden] bf16.
struct HiddenStreams {
    std::uint32_t rows{0};
    HipBuffer input, normed, branch, residual;
};
struct HiddenStreamsResult {
    DecodeStepError error;
    std::optional<HiddenStreams> streams;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && streams.has_value();
    }
};
HiddenStreamsResult create_hidden_streams(const HipDevice& device, const DecodeGeometry& geometry,
                                          std::uint32_t rows);

// LayerStageHooks that run the reference's own stages around the family
// (decode_step.cpp:1102-1135, 1196-1211, 1280-1310):
//   project: normed = rms(layer input, input_norm); projection slab = Q4(normed)
//   finish:  branch = Q4 out-projection(gated / attended);
//            residual = bf16(layer input + branch); normed = rms(residual, post_norm)
// The layer input is streams.input for layer 0.  For later layers it is what
// the expert stage (outside this path) left in streams.input, or, with
// residual_feeds_next, the previous layer's residual.  The object must outlive
// the encoding; scratch and streams must hold at least the wave's rows.
struct QuantizedLayerStages {
    const StagePipelines* pipelines{nullptr};
    const DecodeGeometry* geometry{nullptr};
    std::span<const LayerKind> schedule;
    std::span<const LayerBindings> layers;
    DecodeBatchScratch* scratch{nullptr};
    HiddenStreams* streams{nullptr};
    bool residual_feeds_next{true};
    // waves of two or more rows on the matrix unit; one row always runs the
    // reference's summation order
    bool matrix_unit{true};
    std::uint32_t row_tile{16};          // rows per tile of the _ms operators (decode_step.cpp:1080-1093)

    LayerStageHooks hooks();
    HipCommandError encode_project(HipComputePass& pass, std::size_t layer, LayerKind kind,
                                   std::uint32_t rows) const;
    HipCommandError encode_finish(HipComputePass& pass, std::size_t layer, LayerKind kind,
                                  std::uint32_t rows) const;
};

// decode_step.cpp:1432-1441: toggles `swapped` on Gated DeltaNet layers of an
// available, compatible slot; anything else is left untouched.
void advance_decode_state(const DecodeStep& step, DecodeStateSlot& state);
void advance_decode_state(DecodeStep& step);
// prefill_step.cpp:3526-3538: toggles iff the chunk count is odd.
void advance_prefill_state(const DecodeStep& step, DecodeStateSlot& state, std::uint32_t chunks);

// Lane recycle (state_slot_reset.cpp:176-286): zero-fill both planes of every
// Gated DeltaNet layer through a blit pass, then complete -> swapped=false,
// Ready.  Attention KV is never cleared: validity is `context`.
enum class StateSlotResetError : std::uint8_t {
    None,
    InvalidStateSlot,
    StateSlotNotReady,
    PoisonedStateSlot,
    GenerationExhausted,
    CommandEncodingFailed,
    StaleTicket,
    AlreadyCompleted,
};
struct StateSlotResetTicket {
    const DecodeStep* owner{nullptr};
    DecodeStateSlot* state_owner{nullptr};
    std::uint32_t segment_count{0};
    std::uint64_t state_bytes{0};
    std::uint64_t generation{0};
    bool pending{false};
};
struct StateSlotResetResult {
    StateSlotResetError error;
    HipCommandError command_error;
    std::uint32_t segment_count;
    std::uint64_t state_bytes;
    std::optional<StateSlotResetTicket> ticket;
};
StateSlotResetResult encode_state_slot_reset(const DecodeStep& step, DecodeStateSlot& state,
                                             HipBlitPass& blit_pass) noexcept;
StateSlotResetError complete_state_slot_reset(StateSlotResetTicket& ticket, const DecodeStep& step,
                                              DecodeStateSlot& state) noexcept;

// ---- block prefill ----
enum class PrefillSchedule : std::uint8_t { ChunkMajor, LayerMajor };

// prefill_geometry.h:25-34 (attention-family fields)
struct PrefillPolicy {
    PrefillSchedule schedule{PrefillSchedule::ChunkMajor};
    std::uint32_t context_capacity{0};
    std::uint32_t maximum_block_rows{0};
    std::uint32_t first_chunk_rows{0};
    std::uint32_t query_tile_rows{0};
    std::uint32_t attention_partition{kAttentionPartition};
    bool gdn_gate_hoist{false};
    // Evaluate the block recurrence 64 tokens at a time on MFMA (gdn_chunk_recurrence_blk)
    // instead of the reference's token-by-token register loop.
    // Implies hoisted gates.  The reference has no such switch.
    bool gdn_chunked{false};
    // Record the rollback tape while a block of at most kGdnTapeRows rows runs through
    // the register loop (PrefillGdnRecurrence::RegisterLoopTape, prefill_step.cpp:1931-1933).
    // Needs hoisted gates, excludes gdn_chunked, and at most kGdnTapeLayers layers.
    bool gdn_tape{false};
};

enum class PrefillRequestError : std::uint8_t {
    None,
    EmptyPrefix,
    BlockOutOfRange,
    ContextOutOfRange,
    ContextOverflow,
    TokenOutOfRange,
};
struct PrefillRequestValidation {
    PrefillRequestError error{PrefillRequestError::EmptyPrefix};
    std::uint32_t next_context{0};
    explicit constexpr operator bool() const noexcept {
        return error == PrefillRequestError::None;
    }
};
// prefill_geometry.h:248-299
PrefillRequestValidation validate_prefill_request(const PrefillPolicy& policy,
                                                  std::uint32_t live_context,
                                                  std::uint32_t context_base,
                                                  std::span<const std::uint32_t> tokens,
                                                  std::uint32_t vocabulary) noexcept;
PrefillRequestValidation validate_prefill_prefix(const PrefillPolicy& policy,
                                                 std::uint32_t live_context,
                                                 std::uint32_t context_base,
                                                 std::span<const std::uint32_t> tokens,
                                                 std::uint32_t vocabulary) noexcept;

enum class PrefillGeometryError : std::uint8_t { None, InvalidPlan, InvalidPolicy, Overflow };

// Persistent-state and attention-family extents of PrefillGeometry
// (prefill_geometry.h:65-131, 301-496).
struct PrefillGeometry {
    PrefillPolicy policy;
    std::uint32_t gated_delta_layers{0};
    std::uint32_t attention_layers{0};
    std::uint32_t attention_partitions{0};
    std::uint32_t key_value_heads{0};
    std::uint32_t attention_head_dimension{0};
    std::uint32_t gdn_projection_rows{0};
    std::uint32_t gdn_qk_values{0};
    std::uint32_t gdn_value_values{0};
    std::uint32_t attention_projection_rows{0};
    std::uint32_t attention_vector_values{0};
    std::uint64_t gdn_live_state_bytes_per_layer{0};
    std::uint64_t gdn_slot_state_bytes_per_layer{0};
    std::uint64_t attention_state_bytes_per_position_per_layer{0};
    std::uint64_t attention_slot_state_bytes_per_layer{0};
    std::uint64_t slot_state_bytes{0};
    std::uint64_t gdn_projection_bytes{0};
    std::uint64_t gdn_qk_bytes{0};
    std::uint64_t gdn_value_bytes{0};
    std::uint64_t gdn_parameter_bytes{0};
    std::uint64_t gdn_chunk_bytes{0};  // chunk records of the MFMA recurrence; 0 when unused
    std::uint64_t gdn_tape_bytes{0};       // rollback tape (fp32 regions); 0 when unused
    std::uint64_t gdn_conv_tape_bytes{0};  // conv windows after each taped row; 0 when unused
    std::uint64_t attention_projection_bytes{0};
    std::uint64_t attention_vector_bytes{0};
    std::uint64_t attention_partial_bytes{0};
};
struct PrefillGeometryResult {
    PrefillGeometryError error;
    PrefillGeometry geometry;
    explicit operator bool() const noexcept { return error == PrefillGeometryError::None; }
};
PrefillGeometryResult make_prefill_geometry(const model::qwen36::ModelPlan& plan,
                                            const PrefillPolicy& policy);

// Canonical snapshot payload sizes (prefill_geometry.h:215-246).
struct PrefixStateSnapshotGeometry {
    bool valid{false};
    std::uint32_t positions{0};
    std::uint64_t gated_delta_bytes{0};
    std::uint64_t attention_bytes{0};
    std::uint64_t total_bytes{0};
};
PrefixStateSnapshotGeometry make_prefix_state_snapshot_geometry(const PrefillGeometry& geometry,
                                                                std::uint32_t positions) noexcept;

// prefill_step.cpp:511-550
struct PrefillChunk {
    std::uint32_t offset;
    std::uint32_t rows;
    std::uint32_t ordinal;
};
std::uint32_t prefill_chunk_count(const PrefillPolicy& policy, std::uint32_t context_base,
                                  std::uint32_t rows);
PrefillChunk prefill_chunk_at(const PrefillPolicy& policy, std::uint32_t context_base,
                              std::uint32_t total_rows, std::uint32_t ordinal);

struct PrefillPipelines {
    HipComputePipeline attn_qk_rope_blk, attention_flash_blk, attention_flash_split_blk;
    HipComputePipeline gdn_conv_blk, gdn_gates_blk, gdn_recurrence_gates_blk, gdn_recurrence_blk,
        gdn_gate_norm_blk, gdn_chunk_recurrence_blk;
    HipComputePipeline gdn_conv_tape_blk, gdn_recurrence_gates_tape_blk, gdn_tape_replay_blk;
};
struct PrefillPipelinesResult {
    backend::hip::HipPipelineError error;
    std::optional<PrefillPipelines> pipelines;
    explicit operator bool() const noexcept {
        return error == backend::hip::HipPipelineError::None && pipelines.has_value();
    }
};
PrefillPipelinesResult resolve_prefill_pipelines(const HipLibrary& library);

// Block scratch: [maximum_block_rows x width] slabs of the family's stages.
struct PrefillScratch {
    std::uint32_t block_rows{0};
    HipBuffer gdn_projection, gdn_qk, gdn_value, gdn_gate, gdn_recurrence, gdn_gated;
    HipBuffer gdn_decay, gdn_beta, gdn_chunk;
    HipBuffer gdn_tape, gdn_conv_tape;
    HipBuffer attn_projection, attn_query, attn_gate, attn_attended;
    // attention_flash_split_blk: a block of few rows is few workgroups, so several share each
    // position tile's key walk (tt_flash_prefill_splits) and exchange their results here
    HipBuffer attn_shared_walk;
    std::uint32_t compute_units{256};
};
struct PrefillScratchResult {
    DecodeStepError error;
    std::optional<PrefillScratch> scratch;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && scratch.has_value();
    }
};
PrefillScratchResult create_prefill_scratch(const HipDevice& device,
                                            const PrefillGeometry& geometry);

// encode_attention (prefill_step.cpp:1386-1851): rope + append the chunk's rows
// at context_base + chunk.offset, then causal attention of the chunk (one flash
// dispatch for the whole chunk; the reference walks 256-row query tiles).  Chunks of too
// few rows to fill the device take attention_flash_split_blk.
HipCommandError encode_prefill_attention(const PrefillPipelines& pipelines,
                                         const PrefillGeometry& geometry, PrefillScratch& scratch,
                                         const DecodeLayerState& state, const LayerWeights& weights,
                                         const PrefillChunk& chunk, std::uint32_t context_base,
                                         HipComputePass& pass);
// encode_gated_delta (prefill_step.cpp:1854-2081): phase = swapped ^ (ordinal & 1)
// selects the ping-pong planes; conv over the block, gates (hoisted or inline),
// register-loop scan or, with policy.gdn_chunked, the chunked MFMA recurrence,
// gate-norm.  With policy.gdn_tape the conv and the scan also record the rollback
// tape of `layer_index` (rows beyond kGdnTapeRows record nothing).
HipCommandError encode_prefill_gated_delta(const PrefillPipelines& pipelines,
                                           const PrefillGeometry& geometry, PrefillScratch& scratch,
                                           const DecodeLayerState& state,
                                           const LayerWeights& weights, const PrefillChunk& chunk,
                                           std::uint32_t recurrence_ordinal, HipComputePass& pass,
                                           std::uint32_t layer_index = 0);

// Rollback of a taped block to its first `committed` rows (tape_rollback,
// speculative_decode.cpp:517-600).  Call while the slot's flags still name the planes
// the block READ (that is, instead of advance_prefill_state for the block): every
// gated-delta layer's recurrent state is replayed from that plane into the opposite
// one, the conv window after row committed-1 is copied from the conv tape into the
// opposite conv plane, and completion toggles `swapped` exactly as a block of
// `committed` rows would have.  Attention caches need nothing: rows past the
// committed context are never read.
HipCommandError encode_gdn_tape_replay(const PrefillPipelines& pipelines, const DecodeStep& step,
                                       const DecodeStateSlot& state, const PrefillScratch& scratch,
                                       std::uint32_t committed, HipComputePass& pass);
HipCommandError encode_gdn_tape_windows(const DecodeStep& step, DecodeStateSlot& state,
                                        const PrefillScratch& scratch, std::uint32_t committed,
                                        HipBlitPass& blit_pass);
void complete_gdn_tape_rollback(const DecodeStep& step, DecodeStateSlot& state);

// ---- the block's stages either side of the family, from 4-bit weights ---------
// encode_layer / encode_moe's head (prefill_step.cpp:2535-2567, 2236-2267) with
// the projections of encode_gated_delta / encode_attention (1428-1446, 1909-1926,
// 2063-2078):
//   input:  normalized = rms(input rows, input_norm); projection slab = Q4(normalized)
//   output: branch = Q4 out-projection(gated / attended);
//           block_hidden = bf16(input + branch); normalized = rms(block_hidden, post_norm)
// Blocks of more than 16 rows run on the matrix unit (another summation order
// than the reference's), shorter ones in the reference's order.
struct BlockStagePipelines {
    HipComputePipeline rms, residual_rms, gdn_project, attn_project, out_projection;
};
struct BlockStagePipelinesResult {
    backend::hip::HipPipelineError error;
    std::optional<BlockStagePipelines> pipelines;
    explicit operator bool() const noexcept {
        return error == backend::hip::HipPipelineError::None && pipelines.has_value();
    }
};
BlockStagePipelinesResult resolve_block_stage_pipelines(const HipLibrary& library);

// [maximum_block_rows][hidden] bf16 each (prefill_step.h: normalized, branch, block_hidden).
struct BlockStreams {
    std::uint32_t block_rows{0};
    std::uint32_t hidden{0};
    HipBuffer normalized, branch, block_hidden;
};
struct BlockStreamsResult {
    DecodeStepError error;
    std::optional<BlockStreams> streams;
    explicit operator bool() const noexcept {
        return error == DecodeStepError::None && streams.has_value();
    }
};
BlockStreamsResult create_block_streams(const HipDevice& device, const PrefillGeometry& geometry,
                                        std::uint32_t hidden);

// `input` holds the chunk's rows ([rows][hidden] bf16) from input_offset bytes on.
HipCommandError encode_prefill_layer_input(const BlockStagePipelines& pipelines,
                                           const PrefillGeometry& geometry, PrefillScratch& scratch,
                                           BlockStreams& streams, const LayerBindings& bindings,
                                           LayerKind kind, const PrefillChunk& chunk,
                                           const HipBuffer& input, std::uint64_t input_offset,
                                           HipComputePass& pass);
HipCommandError encode_prefill_layer_output(const BlockStagePipelines& pipelines,
                                            const PrefillGeometry& geometry, PrefillScratch& scratch,
                                            BlockStreams& streams, const LayerBindings& bindings,
                                            LayerKind kind, const PrefillChunk& chunk,
                                            const HipBuffer& input, std::uint64_t input_offset,
                                            HipComputePass& pass);

// ---- lane state record (Q36BRS01) ------------------------------------------
// The file / wire form of exactly the buffers a lane owns on this path
// (tools/native/decode_harness.cpp:25-27, 339-460; decode_harness.h:112-125):
//   8 bytes magic "Q36BRS01", u32 positions, then per layer in schedule order
//   gated delta: conv window [3][8192] bf16, recurrent state [32][128][128] f32 of
//                the LIVE plane of each ping-pong pair;
//   attention:   keys of kv head 0, keys of kv head 1, values of head 0, values of
//                head 1, each `positions` rows of 256 bf16, packed (the caches are
//                capacity-strided, the record is not).
// The live plane is the one the last step wrote: advance_decode_state toggles
// `swapped` after the write, so live is first_out / second_out exactly when
// `swapped` is set (decode_harness.h:100-114).
inline constexpr char kStateRecordMagic[8] = {'Q', '3', '6', 'B', 'R', 'S', '0', '1'};
inline constexpr std::uint64_t kStateRecordHeaderBytes = 12;
constexpr bool gated_delta_live_is_out(bool swapped) { return swapped; }

enum class StateRecordError : std::uint8_t {
    None,
    InvalidState,       // slot not compatible with the step, or not Ready
    InvalidPositions,   // zero, or more than the capacity
    MagicMismatch,
    Truncated,
    TrailingBytes,
    TransferFailed,
};
// Size of the record of `positions` cached tokens; 0 when positions is out of range.
std::uint64_t state_record_bytes(const DecodeStep& step, std::uint32_t positions) noexcept;
// Reads the lane's live planes and the first `positions` cache rows back from the
// device into `record` (resized).  The slot is not modified.
StateRecordError write_state_record(const DecodeStep& step, const DecodeStateSlot& state,
                                    std::uint32_t positions, std::vector<std::byte>& record);
// Installs a record into a Ready slot: gated-delta planes go to first / second and
// `swapped` is cleared (the next step reads exactly those), attention rows go to
// cache rows [0, positions).  On success `positions` is the context the lane
// continues from.  Nothing is written unless the whole record parses.
StateRecordError load_state_record(std::span<const std::byte> record, const DecodeStep& step,
                                   DecodeStateSlot& state, std::uint32_t& positions);

// ---- prefix state snapshot / restore ---------------------------------------
// The device-resident form of the same state: one lane's live planes and its
// first `positions` cache rows packed into a byte range of an arena buffer, and
// back (prefix_state_transfer.h:13-186, prefix_state_transfer.cpp:311-575).
// Unlike the record above the payload is family-major: every gated-delta layer
// in schedule order (conv window, then recurrent state), then every attention
// layer in schedule order (keys of each kv head, then values of each kv head,
// `positions` rows each).  Restore always installs gated-delta bytes into
// first / second and completion clears `swapped`.
inline constexpr std::uint32_t kPrefixStateLayoutSchemaVersion = 1;
inline constexpr std::uint32_t kPrefixStateTransferSchemaVersion = 1;

enum class PrefixStateLayoutError : std::uint8_t {
    None,
    InvalidSchedule,
    InvalidGeometry,
    PositionOutOfRange,
    FamilyCountMismatch,
    TotalMismatch,
    Overflow,
    SegmentOutOfRange,
};
enum class PrefixStateSegmentKind : std::uint8_t {
    GatedDeltaConvolution,
    GatedDeltaRecurrent,
    AttentionKey,
    AttentionValue,
};
enum class PrefixStateBufferPlane : std::uint8_t { First, FirstOutput, Second, SecondOutput, Arena };
enum class PrefixStateTransferDirection : std::uint8_t { Snapshot, Restore };

struct PrefixStateLayoutSpec {
    std::span<const LayerKind> schedule;
    std::uint32_t capacity{0};
    std::uint32_t positions{0};
    std::uint32_t key_value_heads{0};
    std::uint32_t head_dimension{0};
    std::uint32_t expected_gated_delta_layers{0};
    std::uint32_t expected_attention_layers{0};
    std::uint64_t gated_delta_convolution_bytes{0};
    std::uint64_t gated_delta_recurrent_bytes{0};
    std::uint64_t expected_total_bytes{0};
};
struct PrefixStateLayout {
    PrefixStateLayoutSpec specification;
    std::uint32_t gated_delta_layers{0};
    std::uint32_t attention_layers{0};
    std::uint32_t segment_count{0};
    std::uint64_t attention_segment_bytes{0};           // positions x head_dimension bf16
    std::uint64_t attention_slot_head_stride_bytes{0};  // capacity x head_dimension bf16
    std::uint64_t gated_delta_bytes{0};
    std::uint64_t attention_bytes{0};
    std::uint64_t total_bytes{0};
};
struct PrefixStateLayoutResult {
    PrefixStateLayoutError error{PrefixStateLayoutError::InvalidGeometry};
    PrefixStateLayout layout;
    explicit constexpr operator bool() const noexcept {
        return error == PrefixStateLayoutError::None;
    }
};
struct PrefixStateSegment {
    PrefixStateSegmentKind kind{PrefixStateSegmentKind::GatedDeltaConvolution};
    std::uint32_t layer_index{0};
    std::uint32_t head_index{0};
    std::uint64_t slot_offset_bytes{0};
    std::uint64_t snapshot_offset_bytes{0};
    std::uint64_t length_bytes{0};
};
struct PrefixStateSegmentResult {
    PrefixStateLayoutError error{PrefixStateLayoutError::SegmentOutOfRange};
    PrefixStateSegment segment;
    explicit constexpr operator bool() const noexcept {
        return error == PrefixStateLayoutError::None;
    }
};
struct PrefixStateCopyRoute {
    PrefixStateBufferPlane source{PrefixStateBufferPlane::First};
    PrefixStateBufferPlane destination{PrefixStateBufferPlane::Arena};
};

PrefixStateLayoutResult make_prefix_state_layout(const PrefixStateLayoutSpec& specification) noexcept;
PrefixStateLayoutResult make_prefix_state_layout(const DecodeStep& decode,
                                                 const PrefillGeometry& geometry,
                                                 std::uint32_t positions) noexcept;
// Segment `segment_index` of the payload, in payload order; allocates nothing.
PrefixStateSegmentResult prefix_state_segment(const PrefixStateLayout& layout,
                                              std::uint32_t segment_index) noexcept;
PrefixStateCopyRoute prefix_state_copy_route(const PrefixStateSegment& segment,
                                             PrefixStateTransferDirection direction,
                                             bool gated_delta_swapped) noexcept;

enum class PrefixStateTransferError : std::uint8_t {
    None,
    InvalidLayout,
    InvalidStateSlot,
    StateSlotNotReady,
    InvalidArena,
    ArenaOutOfRange,
    GenerationExhausted,
    PhaseEvidenceTooSmall,
    CommandEncodingFailed,
    StaleTicket,
    AlreadyCompleted,
    PoisonedStateSlot,
};

PrefixStateTransferError validate_prefix_state_arena_extent(const PrefixStateLayout& layout,
                                                            std::uint64_t arena_offset_bytes,
                                                            std::uint64_t arena_capacity_bytes) noexcept;
// One bit per schedule entry, set for a gated-delta layer whose live planes were
// the out planes when the snapshot was taken.
std::size_t prefix_state_phase_evidence_bytes(std::span<const LayerKind> schedule) noexcept;
PrefixStateTransferError capture_prefix_state_phase_evidence(const DecodeStep& decode,
                                                             const DecodeStateSlot& state,
                                                             std::span<std::byte> phase_evidence) noexcept;

struct PrefixStateTransferTicket {
    PrefixStateTransferDirection direction{PrefixStateTransferDirection::Snapshot};
    const DecodeStep* owner{nullptr};
    DecodeStateSlot* state_owner{nullptr};
    const HipBuffer* arena_owner{nullptr};
    std::uint32_t positions{0};
    std::uint64_t arena_offset_bytes{0};
    std::uint64_t state_bytes{0};
    std::uint64_t generation{0};
    bool pending{false};
};
struct PrefixStateTransferResult {
    PrefixStateTransferError error{PrefixStateTransferError::InvalidLayout};
    PrefixStateLayoutError layout_error{PrefixStateLayoutError::None};
    HipCommandError command_error{HipCommandError::None};
    std::uint32_t segment_count{0};
    std::uint64_t state_bytes{0};
    std::size_t source_phase_evidence_bytes{0};
    std::optional<PrefixStateTransferTicket> ticket;
    explicit operator bool() const noexcept {
        return error == PrefixStateTransferError::None && ticket.has_value();
    }
};

// Both encode device-to-device copies on the blit pass's queue and leave the slot
// SnapshotPending / RestorePending until the ticket is completed after the
// command buffer finished.  A copy that fails to encode poisons the slot.
PrefixStateTransferResult encode_prefix_state_snapshot(const DecodeStep& decode,
                                                       DecodeStateSlot& state,
                                                       const PrefillGeometry& geometry,
                                                       HipBlitPass& blit_pass, HipBuffer& state_arena,
                                                       std::uint64_t arena_offset_bytes,
                                                       std::uint32_t positions,
                                                       std::span<std::byte> source_phase_evidence) noexcept;
PrefixStateTransferResult encode_prefix_state_restore(const DecodeStep& decode, DecodeStateSlot& state,
                                                      const PrefillGeometry& geometry,
                                                      HipBlitPass& blit_pass, HipBuffer& state_arena,
                                                      std::uint64_t arena_offset_bytes,
                                                      std::uint32_t positions) noexcept;
PrefixStateTransferError complete_prefix_state_transfer(PrefixStateTransferTicket& ticket,
                                                        const DecodeStep& decode,
                                                        DecodeStateSlot& state,
                                                        const HipBuffer& state_arena) noexcept;
PrefixStateTransferError abort_prefix_state_transfer(PrefixStateTransferTicket& ticket,
                                                     const DecodeStep& decode, DecodeStateSlot& state,
                                                     const HipBuffer& state_arena) noexcept;

}  // namespace tatara::runtime
