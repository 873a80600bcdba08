/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * CPU restatement of the arithmetic of Tatara's attention-family layers
 * (full-attention decode / block prefill and Gated DeltaNet decode / block
 * prefill for Qwen3.6-35B-A3B).  It is the checker the HIP kernels are judged
 * against.  Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
 * bench.py may load this library; nothing the product ships may call it.
 *
 * Every function follows a function of the reference's scalar model
 * (reference: tests/native/kernel_reference.cpp) or, where that file has no
 * model, the Metal kernel that defines the semantics; the citation is on each
 * declaration.  Values the reference harness point-queried from the Apple GPU
 * (rsqrt, exp, log, cos, sin) come from libm in single precision here, the
 * multiply-add chains use the fused order, simdgroup sums use the
 * adjacent-pairs tree and 256-slot sums the halving tree.
 *
 * Pinning status (what each entry point is checked against, see
 * tests/test_oracle_*.py):
 *   - bf16 conversion / flush-to-zero: the reference's known answers
 *     (kernel_reference_test.cpp:15-35, 37-54).
 *   - every tto_attn_* and tto_gdn_* single-step function: bit-equality with
 *     the unmodified reference file compiled into oracle/_ref (where it
 *     builds), the committed golden fixtures under tests/golden/, and the
 *     closed forms of kernel_reference_test.cpp:95-109, 198-229, 257-275.
 *   - tto_attention_prefill / tto_gdn_prefill: defined as repeated decode
 *     steps (prefill_attention.metal:117-119, prefill_gdn.metal:198-203), so
 *     they inherit the pins of the step functions; additionally checked
 *     against an fp64 textbook evaluation.
 *   - tto_gdn_chunked_f64: brute-force equality with the sequential fp64
 *     recurrence on small shapes.
 *   - tto_q4_dot / tto_q4_project: bit-equality with the reference's
 *     q4_dot_reference (oracle/_ref), the packed-nibble addressing and affine
 *     known answers of kernel_reference_test.cpp:327-345 restated for this
 *     layout, and an fp64 dequantised dot product.
 *   - tto_gdn_conv_tape / tto_gdn_scan_tape / tto_gdn_tape_replay: the
 *     reference holds no test or fixture for the tape; pinned by what the
 *     definition fixes: replaying c rows equals, bit for bit, the state the
 *     pinned tto_gdn_scan stores after exactly c rows (every c in 0..16), the
 *     taped scan equals the plain scan, tape rows equal the scan's operands,
 *     one step from a zero state tapes delta = v * beta, and conv tape row c-1
 *     equals the conv state tto_gdn_prefill commits after c rows.
 */
#pragma once

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- model constants (catalog/model_packages/qwen36-35b-a3b/model.toml:9-34,
 *      tools/generate_kernel_library.py:173-182, 1981-2015) ---- */
enum {
    TTO_ATTN_QUERY_HEADS = 16,
    TTO_ATTN_KV_HEADS = 2,
    TTO_ATTN_HEAD_DIM = 256,
    TTO_ATTN_ROPE_PAIRS = 32,
    TTO_ATTN_PROJECTION_ROWS = 9216,
    TTO_ATTN_QGATE_ROWS = 8192,
    TTO_ATTN_V_OFFSET = 8704,
    TTO_ATTN_PARTITION = 256,
    TTO_ATTN_RECORD_FLOATS = 258,
    TTO_GDN_VALUE_HEADS = 32,
    TTO_GDN_KEY_HEADS = 16,
    TTO_GDN_HEAD_DIM = 128,
    TTO_GDN_CONV_CHANNELS = 8192,
    TTO_GDN_QK_VALUES = 4096,
    TTO_GDN_VALUE_VALUES = 4096,
    TTO_GDN_K_OFFSET = 2048,
    TTO_GDN_B_OFFSET = 12288,
    TTO_GDN_A_OFFSET = 12320,
    TTO_GDN_PROJECTION_ROWS = 12352,
    TTO_GDN_CONV_WIDTH = 4,
    /* rollback tape (tools/generate_kernel_library.py:2045-2049) */
    TTO_GDN_TAPE_ROWS = 16,
    TTO_GDN_TAPE_LAYERS = 40,
    TTO_GDN_TAPE_KEY_OFFSET = 40 * 16 * 32 * 128,
    TTO_GDN_TAPE_GATE_OFFSET = 40 * 16 * 32 * 128 + 40 * 16 * 16 * 128,
    TTO_GDN_TAPE_FLOATS = 40 * 16 * (32 * 128 + 16 * 128 + 64),
    TTO_GDN_CONV_TAPE_VALUES = 40 * 16 * 3 * 8192
};

/* ---- numeric primitives (kernel_reference.cpp:77-103) ---- */
uint16_t tto_bf16_from_f32(float value);
float tto_f32_from_bf16(uint16_t bits);
uint16_t tto_flush_bf16(uint16_t bits);
float tto_flush_f32(float value);
/* bf16 x bf16 rounded to bf16 with flushes (kernel_reference.cpp:148-152). */
uint16_t tto_bf16_mul(uint16_t a, uint16_t b);
/* 32-lane adjacent-pairs tree and 256-slot halving tree
 * (kernel_reference.cpp:24-35, 601-610). */
float tto_tree_adjacent32(const float* lanes);
float tto_tree_halving256(const float* slots);

/* ---- deterministic inputs ---- */
/* xorshift64* stream (kernel_reference.cpp:105-113). */
uint64_t tto_xorshift_next(uint64_t* state);
/* The reference's exponent-banded bf16 fixture values
 * (kernel_reference.cpp:123-129); state is seeded like its constructor. */
void tto_fill_banded_bf16(uint64_t seed, uint16_t* out, uint64_t count);
/* Same stream widened to fp32 (gdn_fixture_probe.cpp:298-300). */
void tto_fill_banded_f32(uint64_t seed, float* out, uint64_t count);
/* Gaussian N(mean, sigma) by Box-Muller in fp64 over the xorshift64* stream,
 * rounded to bf16 (RNE) or fp32; the synthetic inputs of the benchmark
 * configurations. */
void tto_fill_gaussian_bf16(uint64_t seed, double mean, double sigma, uint16_t* out,
                            uint64_t count);
void tto_fill_gaussian_f32(uint64_t seed, double mean, double sigma, float* out, uint64_t count);
void tto_fill_uniform_f32(uint64_t seed, double low, double high, float* out, uint64_t count);

/* ---- full attention ---- */
/* One token through qk-RMSNorm + partial rotary + cache append
 * (attention.metal:43-113; attn_rms_argument kernel_reference.cpp:616-634,
 * attn_qk_rope_reference :636-689).  projection[9216]; q_out, gate_out[4096];
 * keys/values are [2][capacity][256]. */
void tto_attn_qk_rope(const uint16_t* projection, const uint16_t* q_weight,
                      const uint16_t* k_weight, uint32_t position, uint32_t capacity,
                      uint16_t* q_out, uint16_t* gate_out, uint16_t* keys, uint16_t* values);

/* Tiled online-softmax decode over keys [0, context], all 16 heads
 * (attention.metal:200-276; attention_decode_reference
 * kernel_reference.cpp:725-784).  threads > 1 spreads heads over std::threads. */
void tto_attention_decode(const uint16_t* q, const uint16_t* gate, const uint16_t* keys,
                          const uint16_t* values, uint32_t context, uint32_t capacity,
                          uint16_t* out, uint32_t threads);

/* Split path: per-partition score record (attention.metal:373-448;
 * kernel_reference.cpp:813-845), value stage (attention.metal:995-1036;
 * :847-873) and combine (attention.metal:1086-1108; :886-918). */
void tto_attention_scores_record(const uint16_t* q, const uint16_t* keys, uint32_t head,
                                 uint32_t context, uint32_t capacity, uint32_t part,
                                 uint32_t partition, float* record258);
void tto_attention_values_record(const float* weight_record258, const uint16_t* values,
                                 uint32_t kv_head, uint32_t context, uint32_t capacity,
                                 uint32_t part, uint32_t partition, float* partial258);
/* guard_empty != 0 gives the block-prefill combine, which weights an
 * all-masked partition by zero (prefill_attention.metal:231-236). */
void tto_attention_combine(const float* partial_records, const uint16_t* gate_head,
                           uint32_t nparts, int guard_empty, uint16_t* out_head);
/* scores -> values -> combine for all heads; partials (may be NULL) receives
 * [16][nparts][258] floats. */
void tto_attention_decode_split(const uint16_t* q, const uint16_t* gate, const uint16_t* keys,
                                const uint16_t* values, uint32_t context, uint32_t capacity,
                                uint32_t part, float* partials, uint16_t* out, uint32_t threads);

/* Block prefill (exact control path): rope + append for every row, then causal
 * attention of the selected rows; row r sees keys [0, context_base + r]
 * (prefill_attention.metal:1-92, 97-254).  projection[rows][9216];
 * query/gate/attended are [rows][16][256].  row_select == NULL computes all
 * rows, otherwise only the n_select listed rows (others left untouched). */
void tto_attention_prefill(const uint16_t* projection, const uint16_t* q_weight,
                           const uint16_t* k_weight, uint32_t rows, uint32_t context_base,
                           uint32_t capacity, uint16_t* query, uint16_t* gate, uint16_t* keys,
                           uint16_t* values, const uint32_t* row_select, uint32_t n_select,
                           uint16_t* attended, uint32_t threads);
/* Attention of already-roped rows only (no rope, no append). */
void tto_attention_prefill_rows(const uint16_t* query, const uint16_t* gate,
                                const uint16_t* keys, const uint16_t* values,
                                uint32_t context_base, uint32_t capacity,
                                const uint32_t* row_select, uint32_t n_select,
                                uint16_t* attended, uint32_t threads);

/* ---- Gated DeltaNet ---- */
/* conv4 + bf16 SiLU chain + q/k RMS-norm*scale, z copy, conv state shift
 * (gdn.metal:48-112; conv4_reference kernel_reference.cpp:377-386,
 * gdn_conv_forward :445-464, bf16_sigmoid_candidate :335-346,
 * gdn_head_rsqrt_argument :466-480, gdn_qk_normalize :482-496). */
void tto_gdn_prepare(const uint16_t* projection, const uint16_t* conv_state,
                     const uint16_t* conv_weights, uint16_t* qk, uint16_t* value, uint16_t* z,
                     uint16_t* new_conv_state);
/* Per-head decay and beta from the a/b projection rows (gdn.metal:133-150;
 * gdn_decay_candidate kernel_reference.cpp:355-375, bf16_sigmoid_candidate). */
void tto_gdn_gates(const uint16_t* projection, const uint16_t* a_log, const uint16_t* dt_bias,
                   float* decay32, float* beta32);
/* Delta-rule update of the [32][128][128] fp32 state (gdn.metal:151-171;
 * gdn_recurrence_reference kernel_reference.cpp:498-563).  heads limits the
 * value heads processed (32 for the model; the reference's closed-form test
 * uses 4 with 2 key heads -> pass key_heads accordingly). */
void tto_gdn_recurrence(const uint16_t* qk, const uint16_t* value, const float* decay,
                        const float* beta, const float* state_in, uint32_t key_heads,
                        uint32_t value_heads, uint16_t* y, float* state_out, uint32_t threads);
/* Head RMS-norm * weight, fp32 SiLU gate (gdn.metal:174-207;
 * gdn_gate_norm_reference kernel_reference.cpp:565-583, f32_sigmoid_candidate
 * :348-353). */
void tto_gdn_gate_norm(const uint16_t* y, const uint16_t* z, const uint16_t* norm_weight,
                       uint32_t heads, uint16_t* out);
/* One whole decode step of a GDN layer: prepare -> gates -> recurrence ->
 * gate-norm (decode_step.cpp:666-697). */
void tto_gdn_decode_step(const uint16_t* projection, const uint16_t* conv_state,
                         const uint16_t* conv_weights, const uint16_t* a_log,
                         const uint16_t* dt_bias, const uint16_t* norm_weight,
                         const float* state_in, uint16_t* new_conv_state, float* state_out,
                         uint16_t* gated, uint32_t threads);
/* Block prefill = rows sequential decode steps; only the last row's conv state
 * is committed (prefill_gdn.metal:4-88, 204-320).  projection[rows][12352],
 * gated[rows][4096]; qk/value/y (each may be NULL) receive the per-row
 * intermediates [rows][4096]. */
void tto_gdn_prefill(const uint16_t* projection, uint32_t rows, const uint16_t* conv_state,
                     const uint16_t* conv_weights, const uint16_t* a_log,
                     const uint16_t* dt_bias, const uint16_t* norm_weight, const float* state_in,
                     uint16_t* new_conv_state, float* state_out, uint16_t* gated, uint16_t* qk,
                     uint16_t* value, uint16_t* y, uint32_t threads);
/* Sequential scan with caller-supplied gates, the prefill register loop
 * (prefill_gdn.metal:137-196).  qk/value are [steps][4096], decay/beta
 * [steps][32]. */
void tto_gdn_scan(const uint16_t* qk, const uint16_t* value, const float* decay,
                  const float* beta, uint32_t steps, const float* state_in, uint16_t* y,
                  float* state_out, uint32_t threads);

/* Rollback tape of a block of at most 16 rows and its replay
 * (prefill_gdn.metal:322-400, 432-511, 520-569).
 * tto_gdn_conv_tape: conv_tape[layer][row][tap][8192] = the conv window as it
 * stands after `row` (taps 1..3 of that row); rows > 16 writes nothing.
 * tto_gdn_scan_tape: tto_gdn_scan that also records, per step, delta[32][128],
 * the keys widened to fp32 [16][128] and {decay, beta}[32] into the three
 * regions of `tape` (TTO_GDN_TAPE_* offsets, in floats); steps > 16 records
 * nothing.
 * tto_gdn_tape_replay: state_out = state_in advanced by the first `steps` taped
 * rows with the scan's own two update statements (state *= decay;
 * state = fma(key, delta, state)).
 * Parity pins (no reference test covers the tape): replay(steps = c) equals the
 * state tto_gdn_scan stores after exactly c rows, bit for bit, for every c; the
 * conv tape row c-1 equals the new_conv_state of tto_gdn_prefill over c rows;
 * from a zero state one step tapes delta = v * beta exactly. */
void tto_gdn_conv_tape(const uint16_t* projection, uint32_t rows, const uint16_t* conv_state,
                       uint16_t* conv_tape, uint32_t tape_layer);
void tto_gdn_scan_tape(const uint16_t* qk, const uint16_t* value, const float* decay,
                       const float* beta, uint32_t steps, const float* state_in, uint16_t* y,
                       float* state_out, float* tape, uint32_t tape_layer, uint32_t threads);
void tto_gdn_tape_replay(const float* tape, const float* state_in, float* state_out,
                         uint32_t steps, uint32_t tape_layer, uint32_t threads);

/* Affine 4-bit projections (group 64): w[n][k] = scale[n][k/64] * nibble + bias[n][k/64],
 * eight nibbles to a 32-bit word, low nibble first (q4_dot.metal:9-41;
 * q4_dot_reference kernel_reference.cpp:388-443 in the fused order with the
 * adjacent-pairs tree).  One lane of 32 owns 16 consecutive inputs of every 512
 * block; the place value of a masked nibble is undone by exact power-of-two
 * pre-scaling of the input.  k_size is a multiple of 512.
 * tto_q4_project: out[r][n] = bf16(q4_dot(x[r], row n)) for n < out_rows, the
 * arithmetic of attn_project / gdn_project / gdn_outproj and their _ms / _blk
 * forms (attention.metal:1-41, gdn.metal:1-47, 209-230; prefill_dense.metal:120-260),
 * whose batching never changes a row's sequence of operations. */
float tto_q4_dot(const uint16_t* x, const uint32_t* words, const uint16_t* scales,
                 const uint16_t* biases, uint32_t k_size);
void tto_q4_project(const uint16_t* x, uint64_t x_stride, uint32_t rows, const uint32_t* words,
                    const uint16_t* scales, const uint16_t* biases, uint32_t k_size,
                    uint32_t out_rows, uint16_t* out, uint64_t out_stride, uint32_t threads);

/* The steps either side of the path in a stacked run.
 * tto_rms_only: row RMS norm with the double rounding bf16(w * bf16(x * inv))
 * (rms_only.metal:5-42; rms_total_of_squares / rms_only_reference
 * kernel_reference.cpp:174-222), hidden a multiple of 128 up to 4096.
 * tto_dense_bf16: out[r][n] = bf16(sum_k x[r][k] w[n][k]), fp32 accumulation; a
 * stand-in for the reference's Q4 projections (no reference counterpart: any
 * fixed summation order serves, results are compared at tolerance).
 * tto_add_bf16: bf16(a + b), the residual sum (residual_rms_rounded_sums
 * kernel_reference.cpp:1160-1165). */
void tto_rms_only(const uint16_t* input, const uint16_t* weight, uint32_t rows, uint32_t hidden,
                  uint16_t* output);
void tto_dense_bf16(const uint16_t* input, const uint16_t* weights, uint32_t rows, uint32_t in_dim,
                    uint32_t out_dim, uint16_t* output, uint32_t threads);
void tto_add_bf16(const uint16_t* a, const uint16_t* b, uint64_t count, uint16_t* out);

/* fp64 evaluations used only to pin the algorithms (not reference
 * restatements): sequential delta rule and its chunked WY form for one head.
 * q,k [steps][dk], v [steps][dv], state [dv][dk] (key index contiguous). */
void tto_gdn_sequential_f64(const double* q, const double* k, const double* v,
                            const double* decay, const double* beta, uint32_t steps, uint32_t dk,
                            uint32_t dv, double* state, double* y);
void tto_gdn_chunked_f64(const double* q, const double* k, const double* v, const double* decay,
                         const double* beta, uint32_t steps, uint32_t dk, uint32_t dv,
                         uint32_t chunk, double* state, double* y);

#ifdef __cplusplus
}
#endif
