// TEST INFRASTRUCTURE — NOT PRODUCT CODE.
//
// C entry points over the UNMODIFIED reference scalar model
// (tests/native/kernel_reference.{h,cpp} of the reference tree), compiled from
// where those sources lie by oracle/Makefile into oracle/_ref/.  The reference
// model takes the transcendental values its Apple harness point-queried from
// the GPU as input arrays; this shim supplies them from single-precision libm,
// exactly where the restatement in tatara_oracle.cpp evaluates them itself, so
// the two can be compared bit for bit.
#include "kernel_reference.h"

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

using namespace tatara::testing;

namespace {
constexpr AttnGeometry kAttn{.query_heads = 16, .kv_heads = 2, .head_dimension = 256};
constexpr std::uint32_t kD = 256;
constexpr float kEps = 1e-6f;

std::vector<float> exps_of(const std::vector<float>& args) {
    std::vector<float> out(args.size());
    for (std::size_t i = 0; i < args.size(); ++i) out[i] = std::exp(args[i]);
    return out;
}
}  // namespace

extern "C" {

std::uint16_t ref_bf16_from_f32(float v) { return bf16_from_f32(v); }
float ref_f32_from_bf16(std::uint16_t b) { return f32_from_bf16(b); }
std::uint16_t ref_flush_bf16(std::uint16_t b) { return flush_subnormal_bf16(b); }
std::uint16_t ref_bf16_mul(std::uint16_t a, std::uint16_t b) {
    return bfloat_multiply_candidate(a, b);
}
void ref_fill_banded_bf16(std::uint64_t seed, std::uint16_t* out, std::uint64_t count) {
    Xorshift64Star g(seed);
    for (std::uint64_t i = 0; i < count; ++i) out[i] = g.next_banded_bf16();
}
float ref_tree_sum(const float* lanes, std::uint32_t count, std::uint32_t shape) {
    return simd_tree_sum(std::span<const float>(lanes, count), static_cast<SimdTreeShape>(shape));
}
void ref_rms_only(const std::uint16_t* in, const std::uint16_t* w, std::uint32_t hidden,
                  std::uint32_t shape, std::uint32_t rsqrt_order, std::uint16_t* out) {
    rms_only_reference(std::span<const std::uint16_t>(in, hidden),
                       std::span<const std::uint16_t>(w, hidden), hidden, kEps,
                       static_cast<SimdTreeShape>(shape), static_cast<RsqrtOrder>(rsqrt_order),
                       std::span<std::uint16_t>(out, hidden));
}

float ref_q4_dot(const std::uint16_t* x, const std::uint32_t* words, const std::uint16_t* scales,
                 const std::uint16_t* biases, std::uint32_t k_size) {
    return q4_dot_reference(std::span<const std::uint16_t>(x, k_size),
                            std::span<const std::uint32_t>(words, k_size / 8),
                            std::span<const std::uint16_t>(scales, k_size / 64),
                            std::span<const std::uint16_t>(biases, k_size / 64), k_size,
                            SimdTreeShape::AdjacentPairs, ChainOrder::Fused);
}

void ref_residual_sums(const std::uint16_t* a, const std::uint16_t* b, std::uint64_t count,
                       std::uint16_t* out) {
    residual_rms_rounded_sums(std::span<const std::uint16_t>(a, count),
                              std::span<const std::uint16_t>(b, count),
                              std::span<std::uint16_t>(out, count));
}

void ref_attn_qk_rope(const std::uint16_t* projection, const std::uint16_t* q_weight,
                      const std::uint16_t* k_weight, std::uint32_t position,
                      std::uint32_t capacity, std::uint16_t* q_out, std::uint16_t* gate_out,
                      std::uint16_t* keys, std::uint16_t* values) {
    std::span<const std::uint16_t> proj(projection, 9216);
    std::vector<float> inverses(18);
    for (std::uint32_t head = 0; head < 18; ++head) {
        const std::uint32_t base = head < 16 ? head * 512 : 8192 + (head - 16) * 256;
        inverses[head] = rsqrt_candidate(attn_rms_argument(proj, base, kD, kEps),
                                         RsqrtOrder::ReciprocalOfSqrt);
    }
    std::vector<float> cosines(32), sines(32);
    for (std::uint32_t pair = 0; pair < 32; ++pair) {
        const float theta = static_cast<float>(position) /
                            std::pow(1.0e7f, static_cast<float>(pair) / 32.0f);
        cosines[pair] = std::cos(theta);
        sines[pair] = std::sin(theta);
    }
    const std::size_t cache = std::size_t{2} * capacity * kD;
    attn_qk_rope_reference(proj, std::span<const std::uint16_t>(q_weight, kD),
                           std::span<const std::uint16_t>(k_weight, kD), position, capacity,
                           kAttn, inverses, cosines, sines, ChainOrder::Fused,
                           std::span<std::uint16_t>(q_out, 4096),
                           std::span<std::uint16_t>(gate_out, 4096),
                           std::span<std::uint16_t>(keys, cache),
                           std::span<std::uint16_t>(values, cache));
}

void ref_attention_decode(const std::uint16_t* q, const std::uint16_t* gate,
                          const std::uint16_t* keys, const std::uint16_t* values,
                          std::uint32_t context, std::uint32_t capacity, std::uint16_t* out) {
    const std::size_t cache = std::size_t{2} * capacity * kD;
    std::span<const std::uint16_t> qs(q, 4096), gs(gate, 4096), ks(keys, cache), vs(values, cache);
    for (std::uint32_t head = 0; head < 16; ++head) {
        std::vector<float> args;
        attention_decode_arguments(qs, ks, head, context, capacity, kAttn, args);
        const std::vector<float> exps = exps_of(args);
        attention_decode_reference(qs, gs, ks, vs, head, context, capacity, kAttn, exps,
                                   ChainOrder::Fused, std::span<std::uint16_t>(out, 4096));
    }
}

// scores -> values -> combine; partials (nullable) receives [16][nparts][258]
void ref_attention_decode_split(const std::uint16_t* q, const std::uint16_t* gate,
                                const std::uint16_t* keys, const std::uint16_t* values,
                                std::uint32_t context, std::uint32_t capacity, std::uint32_t part,
                                float* partials, std::uint16_t* out) {
    const std::size_t cache = std::size_t{2} * capacity * kD;
    std::span<const std::uint16_t> qs(q, 4096), gs(gate, 4096), ks(keys, cache), vs(values, cache);
    const std::uint32_t n = context + 1;
    const std::uint32_t nparts = n <= part ? 1u : (n + part - 1) / part;
    std::vector<float> records(std::size_t{nparts} * 258);
    for (std::uint32_t head = 0; head < 16; ++head) {
        for (std::uint32_t p = 0; p < nparts; ++p) {
            std::vector<float> args;
            attention_scores_gqa4_arguments(qs, ks, head, context, capacity, part, p, kAttn, args);
            const std::vector<float> exps = exps_of(args);
            std::vector<float> weights(258);
            attention_scores_gqa4_reference(qs, ks, head, context, capacity, part, p, kAttn, exps,
                                            weights);
            attention_values_gqa8_reference(weights, vs, head >> 3, context, capacity, part, p,
                                            kAttn, ChainOrder::Fused,
                                            std::span<float>(records.data() + p * 258, 258));
        }
        std::vector<float> cargs;
        attention_combine_arguments(records, nparts, cargs);
        const std::vector<float> cexps = exps_of(cargs);
        std::vector<float> gate_exps(kD);
        for (std::uint32_t d = 0; d < kD; ++d) {
            gate_exps[d] = std::exp(-f32_from_bf16(gate[head * kD + d]));
        }
        attention_combine_reference(records, gs, head, nparts, kAttn, cexps, gate_exps,
                                    ChainOrder::Fused,
                                    std::span<std::uint16_t>(out + head * kD, kD));
        if (partials) {
            std::memcpy(partials + std::size_t{head} * nparts * 258, records.data(),
                        records.size() * sizeof(float));
        }
    }
}

void ref_gdn_prepare(const std::uint16_t* projection, const std::uint16_t* conv_state,
                     const std::uint16_t* conv_weights, std::uint16_t* qk, std::uint16_t* value,
                     std::uint16_t* z, std::uint16_t* new_conv_state) {
    constexpr std::uint32_t C = 8192;
    constexpr GdnGeometry geo{.key_heads = 16, .value_heads = 32, .head_dimension = 128};
    std::vector<std::uint16_t> convolved(C), activated(C);
    gdn_conv_forward(std::span<const std::uint16_t>(projection, 12352),
                     std::span<const std::uint16_t>(conv_state, 3 * C),
                     std::span<const std::uint16_t>(conv_weights, 4 * C), C, convolved,
                     std::span<std::uint16_t>(new_conv_state, 3 * C));
    for (std::uint32_t c = 0; c < C; ++c) {
        activated[c] = bfloat_multiply_candidate(
            convolved[c], bf16_sigmoid_candidate(convolved[c], TranscendentalModel::FloatLibm));
    }
    std::vector<float> inverses(32);
    for (std::uint32_t head = 0; head < 32; ++head) {
        inverses[head] = rsqrt_candidate(
            gdn_head_rsqrt_argument(activated, head, 128, kEps, SimdTreeShape::AdjacentPairs),
            RsqrtOrder::ReciprocalOfSqrt);
    }
    gdn_qk_normalize(activated, inverses, geo, 0x3C00, 0x3DB5, std::span<std::uint16_t>(qk, 4096));
    std::memcpy(value, activated.data() + 4096, 4096 * 2);
    std::memcpy(z, projection + C, 4096 * 2);
}

void ref_gdn_gates(const std::uint16_t* projection, const std::uint16_t* a_log,
                   const std::uint16_t* dt_bias, float* decay32, float* beta32) {
    for (std::uint32_t h = 0; h < 32; ++h) {
        const std::uint16_t shifted = bfloat_add_candidate(projection[12320 + h], dt_bias[h]);
        decay32[h] = gdn_decay_candidate(shifted, a_log[h], TranscendentalModel::FloatLibm);
        beta32[h] = f32_from_bf16(
            bf16_sigmoid_candidate(projection[12288 + h], TranscendentalModel::FloatLibm));
    }
}

void ref_gdn_recurrence(const std::uint16_t* qk, const std::uint16_t* value, const float* decay,
                        const float* beta, const float* state_in, std::uint32_t key_heads,
                        std::uint32_t value_heads, std::uint16_t* y, float* state_out) {
    const GdnGeometry geo{.key_heads = key_heads, .value_heads = value_heads,
                          .head_dimension = 128};
    const std::size_t st = std::size_t{value_heads} * 128 * 128;
    gdn_recurrence_reference(std::span<const std::uint16_t>(qk, 2 * key_heads * 128),
                             std::span<const std::uint16_t>(value, value_heads * 128),
                             std::span<const float>(decay, value_heads),
                             std::span<const float>(beta, value_heads),
                             std::span<const float>(state_in, st), geo,
                             SimdTreeShape::AdjacentPairs, ChainOrder::Fused,
                             std::span<std::uint16_t>(y, value_heads * 128),
                             std::span<float>(state_out, st));
}

void ref_gdn_gate_norm(const std::uint16_t* y, const std::uint16_t* z,
                       const std::uint16_t* norm_weight, std::uint32_t heads, std::uint16_t* out) {
    const std::uint32_t n = heads * 128;
    std::span<const std::uint16_t> ys(y, n);
    std::vector<float> inverses(heads), sig(n);
    for (std::uint32_t h = 0; h < heads; ++h) {
        inverses[h] = rsqrt_candidate(
            gdn_head_rsqrt_argument(ys, h, 128, kEps, SimdTreeShape::AdjacentPairs),
            RsqrtOrder::ReciprocalOfSqrt);
    }
    for (std::uint32_t i = 0; i < n; ++i) {
        sig[i] = f32_sigmoid_candidate(f32_from_bf16(z[i]), TranscendentalModel::FloatLibm);
    }
    gdn_gate_norm_reference(ys, std::span<const std::uint16_t>(z, n),
                            std::span<const std::uint16_t>(norm_weight, 128), inverses, sig, heads,
                            128, std::span<std::uint16_t>(out, n));
}

}  // extern "C"
