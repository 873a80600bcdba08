// TEST INFRASTRUCTURE — NOT PRODUCT CODE.  See tatara_oracle.h for scope,
// citations and pinning status.  Build with -ffp-contract=off: every fused
// multiply-add below is written explicitly with std::fma.
#include "tatara_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <limits>
#include <thread>
#include <vector>

namespace {

constexpr uint32_t kQH = TTO_ATTN_QUERY_HEADS;
constexpr uint32_t kKVH = TTO_ATTN_KV_HEADS;
constexpr uint32_t kD = TTO_ATTN_HEAD_DIM;
constexpr uint32_t kGroup = kQH / kKVH;  // query heads per kv head
constexpr uint32_t kVH = TTO_GDN_VALUE_HEADS;
constexpr uint32_t kGD = TTO_GDN_HEAD_DIM;
constexpr uint32_t kCh = TTO_GDN_CONV_CHANNELS;
constexpr float kEps = 1e-6f;
constexpr float kScoreScale = 0.0625f;         // 1/sqrt(256)
constexpr float kRopeBase = 1.0e7f;
constexpr uint16_t kOneBf16 = 0x3F80;
constexpr uint16_t kGdnQueryScaleBf16 = 0x3C00;  // 1/128
constexpr uint16_t kGdnKeyScaleBf16 = 0x3DB5;    // bf16(1/sqrt(128)) = 0.08837890625
constexpr float kNegInf = -std::numeric_limits<float>::infinity();

inline uint32_t bits_of(float v) {
    uint32_t b;
    std::memcpy(&b, &v, 4);
    return b;
}
inline float float_of(uint32_t b) {
    float v;
    std::memcpy(&v, &b, 4);
    return v;
}

// round-to-nearest-even narrowing; infinities and NaNs truncate
inline uint16_t narrow(float v) {
    const uint32_t b = bits_of(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
inline float widen(uint16_t h) { return float_of(static_cast<uint32_t>(h) << 16); }
inline uint16_t fz16(uint16_t h) { return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u); }
inline float fz32(float v) {
    const uint32_t b = bits_of(v);
    return (b & 0x7F800000u) ? v : float_of(b & 0x80000000u);
}
// narrow with both flushes: the "store as bfloat" of an fp32 arithmetic result
inline uint16_t store16(float v) { return fz16(narrow(fz32(v))); }

inline uint16_t mul16(uint16_t a, uint16_t b) { return store16(widen(fz16(a)) * widen(fz16(b))); }
inline uint16_t add16(uint16_t a, uint16_t b) { return store16(widen(fz16(a)) + widen(fz16(b))); }
inline uint16_t sub16(uint16_t a, uint16_t b) { return store16(widen(fz16(a)) - widen(fz16(b))); }
inline uint16_t div16(uint16_t a, uint16_t b) { return store16(widen(fz16(a)) / widen(fz16(b))); }

// pairwise (0+1),(2+3),... repeated: the simdgroup sum shape
float adjacent32(const float* lanes) {
    float level[32];
    std::memcpy(level, lanes, sizeof(level));
    for (uint32_t width = 32; width > 1; width >>= 1) {
        for (uint32_t i = 0; i < width / 2; ++i) level[i] = level[2 * i] + level[2 * i + 1];
    }
    return level[0];
}
// i += i+off for off = 128..1: the threadgroup reduction shape
float halving256(const float* slots) {
    float red[256];
    std::memcpy(red, slots, sizeof(red));
    for (uint32_t off = 128; off; off >>= 1) {
        for (uint32_t i = 0; i < off; ++i) red[i] += red[i + off];
    }
    return red[0];
}

// sigmoid evaluated in bf16 steps with the |x| branch (bf16_sigmoid_candidate)
uint16_t sigmoid16(uint16_t in) {
    const float x = widen(fz16(in));
    const uint16_t e = store16(std::exp(std::fabs(x)));
    const uint16_t low = div16(kOneBf16, add16(kOneBf16, e));
    return x < 0.0f ? low : sub16(kOneBf16, low);
}
// fp32 sigmoid with the |x| branch (f32_sigmoid_candidate)
float sigmoid32(float x) {
    const float low = fz32(1.0f / (1.0f + fz32(std::exp(std::fabs(x)))));
    return x < 0.0f ? low : 1.0f - low;
}
// exp(-exp(A_log) * softplus_bf16(shifted)) (gdn_decay_candidate)
float decay_from(uint16_t shifted, uint16_t a_log) {
    const uint16_t s = fz16(shifted);
    const bool pos = widen(s) > 0.0f;
    const uint16_t hi = pos ? s : uint16_t{0};
    const uint16_t lo = pos ? uint16_t{0} : s;
    const uint16_t diff = sub16(lo, hi);
    const uint16_t e = store16(std::exp(widen(diff)));
    const float one_plus = 1.0f + widen(e);
    uint16_t l1p = e;
    if (one_plus != 1.0f) {
        l1p = store16(widen(e) * (std::log(one_plus) / (one_plus - 1.0f)));
    }
    const uint16_t softplus = add16(hi, l1p);
    return std::exp(-std::exp(widen(fz16(a_log))) * widen(softplus));
}

// sum of squares of 4 consecutive bf16 values, ascending
inline float squares4(const uint16_t* p) {
    float acc = 0.0f;
    for (int j = 0; j < 4; ++j) {
        const float v = widen(p[j]);
        acc += v * v;
    }
    return acc;
}

// 1/sqrt(mean-square + eps) over a 256-wide head: 64 threads x 4 values,
// two simdgroup trees then a tree over the 32-slot stage (attn_rms_argument)
float attn_head_inverse(const uint16_t* head) {
    float stage[32] = {0};
    float lanes[32];
    for (uint32_t sg = 0; sg < 2; ++sg) {
        for (uint32_t l = 0; l < 32; ++l) lanes[l] = squares4(head + (sg * 32 + l) * 4);
        stage[sg] = adjacent32(lanes);
    }
    const float arg = adjacent32(stage) / static_cast<float>(kD) + kEps;
    return 1.0f / std::sqrt(arg);
}
// 1/sqrt(mean-square + eps) over a 128-wide head: 32 lanes x 4 (gdn_head_rsqrt_argument)
float gdn_head_inverse(const uint16_t* head) {
    float lanes[32];
    for (uint32_t l = 0; l < 32; ++l) lanes[l] = squares4(head + l * 4);
    const float arg = adjacent32(lanes) / static_cast<float>(kGD) + kEps;
    return 1.0f / std::sqrt(arg);
}

// (q . k) * 1/16 with the lane-strided partial sums (lane_strided_dot)
inline float score_of(const uint16_t* q, const uint16_t* k) {
    float lanes[32];
    for (uint32_t l = 0; l < 32; ++l) lanes[l] = 0.0f;
    for (uint32_t d0 = 0; d0 < kD; d0 += 32) {
        for (uint32_t l = 0; l < 32; ++l) lanes[l] += widen(q[d0 + l]) * widen(k[d0 + l]);
    }
    return fz32(adjacent32(lanes) * kScoreScale);
}

inline float gate_sigmoid(uint16_t g) {
    return fz32(1.0f / (1.0f + fz32(std::exp(-widen(g)))));
}

// One 258-float score record for keys [start, start+count) of one head.
void scores_record(const uint16_t* q_head, const uint16_t* keys_kv, uint32_t start,
                   uint32_t count, float* record) {
    float s[256];
    float pmax = kNegInf;
    for (uint32_t t = 0; t < count; ++t) {
        s[t] = score_of(q_head, keys_kv + static_cast<size_t>(start + t) * kD);
        pmax = std::max(pmax, s[t]);
    }
    float probs[256];
    for (uint32_t t = 0; t < 256; ++t) probs[t] = t < count ? std::exp(s[t] - pmax) : 0.0f;
    const float psum = halving256(probs);
    std::memcpy(record, probs, sizeof(probs));
    record[256] = pmax;
    record[257] = psum;
}

void values_record(const float* weights, const uint16_t* values_kv, uint32_t start,
                   uint32_t count, float* partial) {
    float acc[kD];
    for (uint32_t d = 0; d < kD; ++d) acc[d] = 0.0f;
    for (uint32_t p = 0; p < count; ++p) {
        const float w = weights[p];
        const uint16_t* row = values_kv + static_cast<size_t>(start + p) * kD;
        for (uint32_t d = 0; d < kD; ++d) acc[d] = std::fma(w, widen(row[d]), acc[d]);
    }
    std::memcpy(partial, acc, sizeof(acc));
    partial[256] = weights[256];
    partial[257] = weights[257];
}

void combine_records(const float* records, const uint16_t* gate_head, uint32_t nparts,
                     bool guard_empty, uint16_t* out_head) {
    float gmax = kNegInf;
    for (uint32_t p = 0; p < nparts; ++p) gmax = std::max(gmax, records[p * 258 + 256]);
    float acc[kD];
    for (uint32_t d = 0; d < kD; ++d) acc[d] = 0.0f;
    float denom = 0.0f;
    for (uint32_t p = 0; p < nparts; ++p) {
        const float* rec = records + static_cast<size_t>(p) * 258;
        const float w = (guard_empty && rec[256] == kNegInf) ? 0.0f : std::exp(rec[256] - gmax);
        for (uint32_t d = 0; d < kD; ++d) acc[d] = std::fma(w, rec[d], acc[d]);
        denom = std::fma(w, rec[257], denom);
    }
    for (uint32_t d = 0; d < kD; ++d) {
        const float v = fz32(acc[d] / denom);
        out_head[d] = store16(v * gate_sigmoid(gate_head[d]));
    }
}

// split attention of one head over n visible keys; records may be null
void attend_head_split(const uint16_t* q_head, const uint16_t* gate_head,
                       const uint16_t* keys_kv, const uint16_t* values_kv, uint32_t n,
                       uint32_t part, bool guard_empty, float* records_out, uint16_t* out_head) {
    const uint32_t nparts = n <= part ? 1u : (n + part - 1) / part;
    std::vector<float> local;
    float* records = records_out;
    if (records == nullptr) {
        local.resize(static_cast<size_t>(nparts) * 258);
        records = local.data();
    }
    float weights[258];
    for (uint32_t p = 0; p < nparts; ++p) {
        const uint32_t start = p * part;
        const uint32_t count = start < n ? std::min(n - start, part) : 0u;
        scores_record(q_head, keys_kv, start, count, weights);
        values_record(weights, values_kv, start, count, records + static_cast<size_t>(p) * 258);
    }
    combine_records(records, gate_head, nparts, guard_empty, out_head);
}

// tiled online softmax of one head over n visible keys (attention_decode)
void attend_head_tiled(const uint16_t* q_head, const uint16_t* gate_head,
                       const uint16_t* keys_kv, const uint16_t* values_kv, uint32_t n,
                       uint16_t* out_head) {
    float running = kNegInf;
    float denom = 0.0f;
    float acc[kD];
    for (uint32_t d = 0; d < kD; ++d) acc[d] = 0.0f;
    float s[256];
    float probs[256];
    for (uint32_t tile = 0; tile < n; tile += 256) {
        const uint32_t count = std::min(n - tile, 256u);
        float tmax = kNegInf;
        for (uint32_t t = 0; t < count; ++t) {
            s[t] = score_of(q_head, keys_kv + static_cast<size_t>(tile + t) * kD);
            tmax = std::max(tmax, s[t]);
        }
        const float next = std::max(running, tmax);
        const float rescale = running == kNegInf ? 0.0f : std::exp(running - next);
        for (uint32_t t = 0; t < 256; ++t) probs[t] = t < count ? std::exp(s[t] - next) : 0.0f;
        const float tsum = halving256(probs);
        for (uint32_t d = 0; d < kD; ++d) acc[d] = fz32(acc[d] * rescale);
        for (uint32_t t = 0; t < count; ++t) {
            const uint16_t* row = values_kv + static_cast<size_t>(tile + t) * kD;
            const float p = probs[t];
            for (uint32_t d = 0; d < kD; ++d) acc[d] = std::fma(p, widen(row[d]), acc[d]);
        }
        denom = fz32(fz32(denom * rescale) + tsum);
        running = next;
    }
    for (uint32_t d = 0; d < kD; ++d) {
        const float v = fz32(acc[d] / denom);
        out_head[d] = store16(v * gate_sigmoid(gate_head[d]));
    }
}

template <typename Fn>
void parallel_for(uint32_t count, uint32_t threads, Fn fn) {
    if (threads <= 1 || count <= 1) {
        for (uint32_t i = 0; i < count; ++i) fn(i);
        return;
    }
    const uint32_t workers = std::min(threads, count);
    std::vector<std::thread> pool;
    pool.reserve(workers);
    for (uint32_t w = 0; w < workers; ++w) {
        pool.emplace_back([=]() {
            for (uint32_t i = w; i < count; i += workers) fn(i);
        });
    }
    for (auto& t : pool) t.join();
}

struct Xs64 {
    uint64_t s;
    explicit Xs64(uint64_t seed) : s(seed ? seed : 0x9E3779B97F4A7C15ull) {}
    uint64_t next() {
        s ^= s >> 12;
        s ^= s << 25;
        s ^= s >> 27;
        return s * 0x2545F4914F6CDD1Dull;
    }
    uint16_t banded() {
        const uint64_t draw = next();
        const uint16_t sign = static_cast<uint16_t>((draw >> 15) & 0x8000u);
        const uint16_t expo = static_cast<uint16_t>((0x70u + draw % 0x18u) << 7);
        const uint16_t mant = static_cast<uint16_t>((draw >> 32) & 0x7Fu);
        return static_cast<uint16_t>(sign | expo | mant);
    }
    double unit() { return (static_cast<double>(next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }
};

// Box-Muller over the xorshift stream; both variates of a pair are used
struct Gauss {
    Xs64 rng;
    bool have = false;
    double spare = 0.0;
    explicit Gauss(uint64_t seed) : rng(seed) {}
    double next() {
        if (have) {
            have = false;
            return spare;
        }
        const double u1 = rng.unit();
        const double u2 = rng.unit();
        const double r = std::sqrt(-2.0 * std::log(u1));
        const double a = 6.283185307179586476925286766559 * u2;
        spare = r * std::sin(a);
        have = true;
        return r * std::cos(a);
    }
};

// conv4 + SiLU for one channel from its four taps
inline uint16_t conv_silu(const uint16_t* w4, const float* taps, uint16_t* convolved_out) {
    float acc = 0.0f;
    for (int i = 0; i < 4; ++i) acc = fz32(acc + fz32(widen(fz16(w4[i])) * taps[i]));
    const uint16_t conv = fz16(narrow(acc));
    if (convolved_out) *convolved_out = conv;
    return mul16(conv, sigmoid16(conv));
}

void normalize_qk_heads(const uint16_t* activated, uint16_t* qk) {
    for (uint32_t head = 0; head < 2 * TTO_GDN_KEY_HEADS; ++head) {
        const float inv = gdn_head_inverse(activated + head * kGD);
        const uint16_t scale = head < TTO_GDN_KEY_HEADS ? kGdnQueryScaleBf16 : kGdnKeyScaleBf16;
        for (uint32_t i = 0; i < kGD; ++i) {
            const uint16_t normed = store16(widen(activated[head * kGD + i]) * inv);
            qk[head * kGD + i] = mul16(normed, scale);
        }
    }
}

// delta-rule update of one (value head, value dim) state row
inline uint16_t recurrence_row(const float* row_in, float* row_out, const uint16_t* q,
                               const uint16_t* k, float v, float decay, float beta,
                               float* delta_out = nullptr) {
    float st[kGD];
    float part[32];
    for (uint32_t l = 0; l < 32; ++l) {
        float kv = 0.0f;
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t e = l * 4 + i;
            st[e] = fz32(row_in[e] * decay);
            kv = std::fma(st[e], widen(k[e]), kv);
        }
        part[l] = kv;
    }
    const float key_value = adjacent32(part);
    const float delta = fz32(fz32(v - key_value) * beta);
    if (delta_out) *delta_out = delta;
    for (uint32_t l = 0; l < 32; ++l) {
        float o = 0.0f;
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t e = l * 4 + i;
            st[e] = std::fma(widen(k[e]), delta, st[e]);
            row_out[e] = st[e];
            o = std::fma(st[e], widen(q[e]), o);
        }
        part[l] = o;
    }
    return store16(adjacent32(part));
}

void recurrence_heads(const uint16_t* qk, const uint16_t* value, const float* decay,
                      const float* beta, const float* state_in, uint32_t key_heads,
                      uint32_t value_heads, uint16_t* y, float* state_out, uint32_t threads) {
    const uint32_t k_offset = key_heads * kGD;
    parallel_for(value_heads, threads, [=](uint32_t h) {
        const uint32_t kh = h >> 1;
        const uint16_t* q = qk + kh * kGD;
        const uint16_t* k = qk + k_offset + kh * kGD;
        for (uint32_t j = 0; j < kGD; ++j) {
            const size_t base = (static_cast<size_t>(h) * kGD + j) * kGD;
            y[h * kGD + j] = recurrence_row(state_in + base, state_out + base, q, k,
                                            widen(value[h * kGD + j]), decay[h], beta[h]);
        }
    });
}

}  // namespace

extern "C" {

uint16_t tto_bf16_from_f32(float value) { return narrow(value); }
float tto_f32_from_bf16(uint16_t bits) { return widen(bits); }
uint16_t tto_flush_bf16(uint16_t bits) { return fz16(bits); }
float tto_flush_f32(float value) { return fz32(value); }
uint16_t tto_bf16_mul(uint16_t a, uint16_t b) { return mul16(a, b); }
float tto_tree_adjacent32(const float* lanes) { return adjacent32(lanes); }
float tto_tree_halving256(const float* slots) { return halving256(slots); }

uint64_t tto_xorshift_next(uint64_t* state) {
    Xs64 g(*state);
    const uint64_t v = g.next();
    *state = g.s;
    return v;
}
void tto_fill_banded_bf16(uint64_t seed, uint16_t* out, uint64_t count) {
    Xs64 g(seed);
    for (uint64_t i = 0; i < count; ++i) out[i] = g.banded();
}
void tto_fill_banded_f32(uint64_t seed, float* out, uint64_t count) {
    Xs64 g(seed);
    for (uint64_t i = 0; i < count; ++i) out[i] = widen(g.banded());
}
void tto_fill_gaussian_bf16(uint64_t seed, double mean, double sigma, uint16_t* out,
                            uint64_t count) {
    Gauss g(seed);
    for (uint64_t i = 0; i < count; ++i) out[i] = narrow(static_cast<float>(mean + sigma * g.next()));
}
void tto_fill_gaussian_f32(uint64_t seed, double mean, double sigma, float* out, uint64_t count) {
    Gauss g(seed);
    for (uint64_t i = 0; i < count; ++i) out[i] = static_cast<float>(mean + sigma * g.next());
}
void tto_fill_uniform_f32(uint64_t seed, double low, double high, float* out, uint64_t count) {
    Xs64 g(seed);
    for (uint64_t i = 0; i < count; ++i) out[i] = static_cast<float>(low + (high - low) * g.unit());
}

void tto_attn_qk_rope(const uint16_t* projection, const uint16_t* q_weight,
                      const uint16_t* k_weight, uint32_t position, uint32_t capacity,
                      uint16_t* q_out, uint16_t* gate_out, uint16_t* keys, uint16_t* values) {
    float cosines[TTO_ATTN_ROPE_PAIRS];
    float sines[TTO_ATTN_ROPE_PAIRS];
    for (uint32_t pair = 0; pair < TTO_ATTN_ROPE_PAIRS; ++pair) {
        const float theta = static_cast<float>(position) /
                            std::pow(kRopeBase, static_cast<float>(pair) /
                                                    static_cast<float>(TTO_ATTN_ROPE_PAIRS));
        cosines[pair] = std::cos(theta);
        sines[pair] = std::sin(theta);
    }
    float normed[kD];
    for (uint32_t head = 0; head < kQH + kKVH; ++head) {
        const bool is_q = head < kQH;
        const uint32_t local = is_q ? head : head - kQH;
        const uint32_t base = is_q ? head * 2 * kD : TTO_ATTN_QGATE_ROWS + local * kD;
        const uint16_t* weight = is_q ? q_weight : k_weight;
        const float inv = attn_head_inverse(projection + base);
        for (uint32_t d = 0; d < kD; ++d) {
            const uint16_t scaled = store16(widen(projection[base + d]) * inv);
            normed[d] = widen(mul16(weight[d], scaled));
        }
        for (uint32_t d = 0; d < kD; ++d) {
            float r = normed[d];
            if (d < 2 * TTO_ATTN_ROPE_PAIRS) {
                const uint32_t pair = d & 31u;
                r = d < 32 ? std::fma(-normed[d + 32], sines[pair], normed[d] * cosines[pair])
                           : std::fma(normed[d - 32], sines[pair], normed[d] * cosines[pair]);
                r = fz32(r);
            }
            const uint16_t stored = fz16(narrow(r));
            if (is_q) {
                q_out[head * kD + d] = stored;
                gate_out[head * kD + d] = projection[head * 2 * kD + kD + d];
            } else {
                const size_t at = (static_cast<size_t>(local) * capacity + position) * kD + d;
                keys[at] = stored;
                values[at] = projection[TTO_ATTN_V_OFFSET + local * kD + d];
            }
        }
    }
}

void tto_attention_decode(const uint16_t* q, const uint16_t* gate, const uint16_t* keys,
                          const uint16_t* values, uint32_t context, uint32_t capacity,
                          uint16_t* out, uint32_t threads) {
    parallel_for(kQH, threads, [=](uint32_t head) {
        const size_t kv = static_cast<size_t>(head / kGroup) * capacity * kD;
        attend_head_tiled(q + head * kD, gate + head * kD, keys + kv, values + kv, context + 1,
                          out + head * kD);
    });
}

void tto_attention_scores_record(const uint16_t* q, const uint16_t* keys, uint32_t head,
                                 uint32_t context, uint32_t capacity, uint32_t part,
                                 uint32_t partition, float* record258) {
    const uint32_t n = context + 1;
    const uint32_t start = partition * part;
    const uint32_t count = start < n ? std::min(n - start, part) : 0u;
    scores_record(q + head * kD, keys + static_cast<size_t>(head / kGroup) * capacity * kD, start,
                  count, record258);
}

void tto_attention_values_record(const float* weight_record258, const uint16_t* values,
                                 uint32_t kv_head, uint32_t context, uint32_t capacity,
                                 uint32_t part, uint32_t partition, float* partial258) {
    const uint32_t n = context + 1;
    const uint32_t start = partition * part;
    const uint32_t count = start < n ? std::min(n - start, part) : 0u;
    values_record(weight_record258, values + static_cast<size_t>(kv_head) * capacity * kD, start,
                  count, partial258);
}

void tto_attention_combine(const float* partial_records, const uint16_t* gate_head,
                           uint32_t nparts, int guard_empty, uint16_t* out_head) {
    combine_records(partial_records, gate_head, nparts, guard_empty != 0, out_head);
}

void tto_attention_decode_split(const uint16_t* q, const uint16_t* gate, const uint16_t* keys,
                                const uint16_t* values, uint32_t context, uint32_t capacity,
                                uint32_t part, float* partials, uint16_t* out, uint32_t threads) {
    const uint32_t n = context + 1;
    const uint32_t nparts = n <= part ? 1u : (n + part - 1) / part;
    parallel_for(kQH, threads, [=](uint32_t head) {
        const size_t kv = static_cast<size_t>(head / kGroup) * capacity * kD;
        float* rec = partials ? partials + static_cast<size_t>(head) * nparts * 258 : nullptr;
        attend_head_split(q + head * kD, gate + head * kD, keys + kv, values + kv, n, part, false,
                          rec, out + head * kD);
    });
}

void tto_attention_prefill_rows(const uint16_t* query, const uint16_t* gate,
                                const uint16_t* keys, const uint16_t* values,
                                uint32_t context_base, uint32_t capacity,
                                const uint32_t* row_select, uint32_t n_select,
                                uint16_t* attended, uint32_t threads) {
    parallel_for(n_select * kQH, threads, [=](uint32_t item) {
        const uint32_t row = row_select[item / kQH];
        const uint32_t head = item % kQH;
        const size_t kv = static_cast<size_t>(head / kGroup) * capacity * kD;
        const size_t at = (static_cast<size_t>(row) * kQH + head) * kD;
        attend_head_split(query + at, gate + at, keys + kv, values + kv, context_base + row + 1,
                          TTO_ATTN_PARTITION, true, nullptr, attended + at);
    });
}

void tto_attention_prefill(const uint16_t* projection, const uint16_t* q_weight,
                           const uint16_t* k_weight, uint32_t rows, uint32_t context_base,
                           uint32_t capacity, uint16_t* query, uint16_t* gate, uint16_t* keys,
                           uint16_t* values, const uint32_t* row_select, uint32_t n_select,
                           uint16_t* attended, uint32_t threads) {
    parallel_for(rows, threads, [=](uint32_t row) {
        tto_attn_qk_rope(projection + static_cast<size_t>(row) * TTO_ATTN_PROJECTION_ROWS,
                         q_weight, k_weight, context_base + row, capacity,
                         query + static_cast<size_t>(row) * kQH * kD,
                         gate + static_cast<size_t>(row) * kQH * kD, keys, values);
    });
    std::vector<uint32_t> all;
    if (row_select == nullptr) {
        all.resize(rows);
        for (uint32_t r = 0; r < rows; ++r) all[r] = r;
        row_select = all.data();
        n_select = rows;
    }
    tto_attention_prefill_rows(query, gate, keys, values, context_base, capacity, row_select,
                               n_select, attended, threads);
}

void tto_gdn_prepare(const uint16_t* projection, const uint16_t* conv_state,
                     const uint16_t* conv_weights, uint16_t* qk, uint16_t* value, uint16_t* z,
                     uint16_t* new_conv_state) {
    std::vector<uint16_t> activated(kCh);
    for (uint32_t c = 0; c < kCh; ++c) {
        const float taps[4] = {widen(conv_state[c]), widen(conv_state[kCh + c]),
                               widen(conv_state[2 * kCh + c]), widen(projection[c])};
        activated[c] = conv_silu(conv_weights + static_cast<size_t>(c) * 4, taps, nullptr);
        const uint16_t t1 = conv_state[kCh + c];
        const uint16_t t2 = conv_state[2 * kCh + c];
        new_conv_state[c] = t1;
        new_conv_state[kCh + c] = t2;
        new_conv_state[2 * kCh + c] = projection[c];
    }
    normalize_qk_heads(activated.data(), qk);
    std::memcpy(value, activated.data() + TTO_GDN_QK_VALUES, TTO_GDN_VALUE_VALUES * 2);
    std::memcpy(z, projection + kCh, TTO_GDN_VALUE_VALUES * 2);
}

void tto_gdn_gates(const uint16_t* projection, const uint16_t* a_log, const uint16_t* dt_bias,
                   float* decay32, float* beta32) {
    for (uint32_t h = 0; h < kVH; ++h) {
        const uint16_t shifted = add16(projection[TTO_GDN_A_OFFSET + h], dt_bias[h]);
        decay32[h] = decay_from(shifted, a_log[h]);
        beta32[h] = widen(sigmoid16(projection[TTO_GDN_B_OFFSET + h]));
    }
}

void tto_gdn_recurrence(const uint16_t* qk, const uint16_t* value, const float* decay,
                        const float* beta, const float* state_in, uint32_t key_heads,
                        uint32_t value_heads, uint16_t* y, float* state_out, uint32_t threads) {
    recurrence_heads(qk, value, decay, beta, state_in, key_heads, value_heads, y, state_out,
                     threads);
}

void tto_gdn_gate_norm(const uint16_t* y, const uint16_t* z, const uint16_t* norm_weight,
                       uint32_t heads, uint16_t* out) {
    for (uint32_t h = 0; h < heads; ++h) {
        const float inv = gdn_head_inverse(y + h * kGD);
        for (uint32_t i = 0; i < kGD; ++i) {
            const uint32_t at = h * kGD + i;
            const uint16_t weighted = mul16(norm_weight[i], store16(widen(y[at]) * inv));
            const float g = widen(z[at]);
            out[at] = store16(fz32(g * sigmoid32(g)) * widen(weighted));
        }
    }
}

void tto_gdn_decode_step(const uint16_t* projection, const uint16_t* conv_state,
                         const uint16_t* conv_weights, const uint16_t* a_log,
                         const uint16_t* dt_bias, const uint16_t* norm_weight,
                         const float* state_in, uint16_t* new_conv_state, float* state_out,
                         uint16_t* gated, uint32_t threads) {
    std::vector<uint16_t> qk(TTO_GDN_QK_VALUES), v(TTO_GDN_VALUE_VALUES), z(TTO_GDN_VALUE_VALUES),
        y(TTO_GDN_VALUE_VALUES);
    float decay[kVH], beta[kVH];
    tto_gdn_prepare(projection, conv_state, conv_weights, qk.data(), v.data(), z.data(),
                    new_conv_state);
    tto_gdn_gates(projection, a_log, dt_bias, decay, beta);
    recurrence_heads(qk.data(), v.data(), decay, beta, state_in, TTO_GDN_KEY_HEADS, kVH, y.data(),
                     state_out, threads);
    tto_gdn_gate_norm(y.data(), z.data(), norm_weight, kVH, gated);
}

void tto_gdn_scan(const uint16_t* qk, const uint16_t* value, const float* decay,
                  const float* beta, uint32_t steps, const float* state_in, uint16_t* y,
                  float* state_out, uint32_t threads) {
    parallel_for(kVH, threads, [=](uint32_t h) {
        const uint32_t kh = h >> 1;
        std::vector<float> st(static_cast<size_t>(kGD) * kGD);
        std::memcpy(st.data(), state_in + static_cast<size_t>(h) * kGD * kGD,
                    st.size() * sizeof(float));
        for (uint32_t t = 0; t < steps; ++t) {
            const uint16_t* q = qk + static_cast<size_t>(t) * TTO_GDN_QK_VALUES + kh * kGD;
            const uint16_t* k = q + TTO_GDN_K_OFFSET;
            const uint16_t* v = value + static_cast<size_t>(t) * TTO_GDN_VALUE_VALUES + h * kGD;
            uint16_t* yo = y + static_cast<size_t>(t) * TTO_GDN_VALUE_VALUES + h * kGD;
            for (uint32_t j = 0; j < kGD; ++j) {
                float* row = st.data() + static_cast<size_t>(j) * kGD;
                yo[j] = recurrence_row(row, row, q, k, widen(v[j]), decay[t * kVH + h],
                                       beta[t * kVH + h]);
            }
        }
        std::memcpy(state_out + static_cast<size_t>(h) * kGD * kGD, st.data(),
                    st.size() * sizeof(float));
    });
}

void tto_gdn_conv_tape(const uint16_t* projection, uint32_t rows, const uint16_t* conv_state,
                       uint16_t* conv_tape, uint32_t tape_layer) {
    if (rows > TTO_GDN_TAPE_ROWS) return;
    const size_t P = TTO_GDN_PROJECTION_ROWS;
    for (uint32_t r = 0; r < rows; ++r) {
        uint16_t* window =
            conv_tape + (static_cast<size_t>(tape_layer) * TTO_GDN_TAPE_ROWS + r) * 3 * kCh;
        for (uint32_t tap = 0; tap < 3; ++tap) {
            const uint32_t logical = r + tap + 1;  // taps 1..3 of row r
            for (uint32_t c = 0; c < kCh; ++c) {
                window[tap * kCh + c] = logical < 3 ? conv_state[logical * kCh + c]
                                                    : projection[(logical - 3) * P + c];
            }
        }
    }
}

void tto_gdn_scan_tape(const uint16_t* qk, const uint16_t* value, const float* decay,
                       const float* beta, uint32_t steps, const float* state_in, uint16_t* y,
                       float* state_out, float* tape, uint32_t tape_layer, uint32_t threads) {
    const bool taped = steps <= TTO_GDN_TAPE_ROWS;
    parallel_for(kVH, threads, [=](uint32_t h) {
        const uint32_t kh = h >> 1;
        std::vector<float> st(static_cast<size_t>(kGD) * kGD);
        std::memcpy(st.data(), state_in + static_cast<size_t>(h) * kGD * kGD,
                    st.size() * sizeof(float));
        for (uint32_t t = 0; t < steps; ++t) {
            const uint16_t* q = qk + static_cast<size_t>(t) * TTO_GDN_QK_VALUES + kh * kGD;
            const uint16_t* k = q + TTO_GDN_K_OFFSET;
            const uint16_t* v = value + static_cast<size_t>(t) * TTO_GDN_VALUE_VALUES + h * kGD;
            uint16_t* yo = y + static_cast<size_t>(t) * TTO_GDN_VALUE_VALUES + h * kGD;
            const size_t tape_row = static_cast<size_t>(tape_layer) * TTO_GDN_TAPE_ROWS + t;
            for (uint32_t j = 0; j < kGD; ++j) {
                float* row = st.data() + static_cast<size_t>(j) * kGD;
                float delta = 0.0f;
                yo[j] = recurrence_row(row, row, q, k, widen(v[j]), decay[t * kVH + h],
                                       beta[t * kVH + h], &delta);
                if (taped) tape[(tape_row * kVH + h) * kGD + j] = delta;
            }
            if (!taped) continue;
            if ((h & 1) == 0) {
                float* keys = tape + TTO_GDN_TAPE_KEY_OFFSET +
                              (tape_row * TTO_GDN_KEY_HEADS + kh) * kGD;
                for (uint32_t e = 0; e < kGD; ++e) keys[e] = widen(k[e]);
            }
            float* gates = tape + TTO_GDN_TAPE_GATE_OFFSET + (tape_row * kVH + h) * 2;
            gates[0] = decay[t * kVH + h];
            gates[1] = beta[t * kVH + h];
        }
        std::memcpy(state_out + static_cast<size_t>(h) * kGD * kGD, st.data(),
                    st.size() * sizeof(float));
    });
}

void tto_gdn_tape_replay(const float* tape, const float* state_in, float* state_out,
                         uint32_t steps, uint32_t tape_layer, uint32_t threads) {
    parallel_for(kVH, threads, [=](uint32_t h) {
        const uint32_t kh = h >> 1;
        for (uint32_t j = 0; j < kGD; ++j) {
            const size_t base = (static_cast<size_t>(h) * kGD + j) * kGD;
            float st[kGD];
            std::memcpy(st, state_in + base, sizeof(st));
            for (uint32_t t = 0; t < steps; ++t) {
                const size_t tape_row = static_cast<size_t>(tape_layer) * TTO_GDN_TAPE_ROWS + t;
                const float step_decay = tape[TTO_GDN_TAPE_GATE_OFFSET + (tape_row * kVH + h) * 2];
                const float delta = tape[(tape_row * kVH + h) * kGD + j];
                const float* keys =
                    tape + TTO_GDN_TAPE_KEY_OFFSET + (tape_row * TTO_GDN_KEY_HEADS + kh) * kGD;
                for (uint32_t e = 0; e < kGD; ++e) {
                    st[e] = fz32(st[e] * step_decay);
                    st[e] = std::fma(keys[e], delta, st[e]);
                }
            }
            std::memcpy(state_out + base, st, sizeof(st));
        }
    });
}

void tto_gdn_prefill(const uint16_t* projection, uint32_t rows, const uint16_t* conv_state,
                     const uint16_t* conv_weights, const uint16_t* a_log,
                     const uint16_t* dt_bias, const uint16_t* norm_weight, const float* state_in,
                     uint16_t* new_conv_state, float* state_out, uint16_t* gated, uint16_t* qk_out,
                     uint16_t* value_out, uint16_t* y_out, uint32_t threads) {
    const size_t P = TTO_GDN_PROJECTION_ROWS;
    std::vector<uint16_t> qk(static_cast<size_t>(rows) * TTO_GDN_QK_VALUES);
    std::vector<uint16_t> v(static_cast<size_t>(rows) * TTO_GDN_VALUE_VALUES);
    std::vector<uint16_t> y(static_cast<size_t>(rows) * TTO_GDN_VALUE_VALUES);
    std::vector<float> decay(static_cast<size_t>(rows) * kVH), beta(static_cast<size_t>(rows) * kVH);
    // conv over the logical sequence {state rows 0..2, block rows}; every row
    // is independent once its four taps are gathered (gdn_conv_blk)
    parallel_for(rows, threads, [&](uint32_t r) {
        std::vector<uint16_t> activated(kCh);
        for (uint32_t c = 0; c < kCh; ++c) {
            float taps[4];
            for (uint32_t tap = 0; tap < 4; ++tap) {
                const uint32_t logical = r + tap;
                taps[tap] = logical < 3 ? widen(conv_state[logical * kCh + c])
                                        : widen(projection[(logical - 3) * P + c]);
            }
            activated[c] = conv_silu(conv_weights + static_cast<size_t>(c) * 4, taps, nullptr);
        }
        normalize_qk_heads(activated.data(), qk.data() + static_cast<size_t>(r) * TTO_GDN_QK_VALUES);
        std::memcpy(v.data() + static_cast<size_t>(r) * TTO_GDN_VALUE_VALUES,
                    activated.data() + TTO_GDN_QK_VALUES, TTO_GDN_VALUE_VALUES * 2);
        tto_gdn_gates(projection + r * P, a_log, dt_bias, decay.data() + static_cast<size_t>(r) * kVH,
                      beta.data() + static_cast<size_t>(r) * kVH);
    });
    for (uint32_t tap = 0; tap < 3; ++tap) {
        const uint32_t logical = rows + tap;  // taps[tap+1] of the last row
        for (uint32_t c = 0; c < kCh; ++c) {
            new_conv_state[tap * kCh + c] = logical < 3 ? conv_state[logical * kCh + c]
                                                        : projection[(logical - 3) * P + c];
        }
    }
    tto_gdn_scan(qk.data(), v.data(), decay.data(), beta.data(), rows, state_in, y.data(),
                 state_out, threads);
    parallel_for(rows, threads, [&](uint32_t r) {
        tto_gdn_gate_norm(y.data() + static_cast<size_t>(r) * TTO_GDN_VALUE_VALUES,
                          projection + r * P + kCh, norm_weight, kVH,
                          gated + static_cast<size_t>(r) * TTO_GDN_VALUE_VALUES);
    });
    if (qk_out) std::memcpy(qk_out, qk.data(), qk.size() * 2);
    if (value_out) std::memcpy(value_out, v.data(), v.size() * 2);
    if (y_out) std::memcpy(y_out, y.data(), y.size() * 2);
}

float tto_q4_dot(const uint16_t* x, const uint32_t* words, const uint16_t* scales,
                 const uint16_t* biases, uint32_t k_size) {
    const uint16_t* packed = reinterpret_cast<const uint16_t*>(words);
    float lanes[32];
    for (uint32_t lane = 0; lane < 32; ++lane) {
        float result = 0.0f;
        for (uint32_t k = 0; k < k_size; k += 512) {
            const uint16_t* xs = x + k + lane * 16;
            float scaled[16];
            float sum = 0.0f;
            for (uint32_t i = 0; i < 16; i += 4) {
                const float a0 = widen(xs[i]), a1 = widen(xs[i + 1]), a2 = widen(xs[i + 2]),
                            a3 = widen(xs[i + 3]);
                sum = fz32(sum + fz32((fz32(a0 + a1) + a2) + a3));
                scaled[i] = a0;
                scaled[i + 1] = a1 / 16.0f;
                scaled[i + 2] = a2 / 256.0f;
                scaled[i + 3] = a3 / 4096.0f;
            }
            float quant = 0.0f;
            const uint16_t* w = packed + (k >> 2) + lane * 4;
            for (uint32_t i = 0; i < 4; ++i) {
                // masked, unshifted nibbles: 0..15, 0..240, 0..3840, 0..61440
                quant = std::fma(scaled[i * 4], static_cast<float>(w[i] & 0x000Fu), quant);
                quant = std::fma(scaled[i * 4 + 1], static_cast<float>(w[i] & 0x00F0u), quant);
                quant = std::fma(scaled[i * 4 + 2], static_cast<float>(w[i] & 0x0F00u), quant);
                quant = std::fma(scaled[i * 4 + 3], static_cast<float>(w[i] & 0xF000u), quant);
            }
            const uint32_t group = (k >> 6) + (lane >> 2);
            result = std::fma(sum, widen(biases[group]), std::fma(widen(scales[group]), quant, result));
        }
        lanes[lane] = result;
    }
    return adjacent32(lanes);
}

void tto_q4_project(const uint16_t* x, uint64_t x_stride, uint32_t rows, const uint32_t* words,
                    const uint16_t* scales, const uint16_t* biases, uint32_t k_size,
                    uint32_t out_rows, uint16_t* out, uint64_t out_stride, uint32_t threads) {
    parallel_for(out_rows, threads, [=](uint32_t n) {
        const uint32_t* w = words + static_cast<size_t>(n) * (k_size / 8);
        const uint16_t* s = scales + static_cast<size_t>(n) * (k_size / 64);
        const uint16_t* b = biases + static_cast<size_t>(n) * (k_size / 64);
        for (uint32_t r = 0; r < rows; ++r) {
            out[r * out_stride + n] = store16(tto_q4_dot(x + r * x_stride, w, s, b, k_size));
        }
    });
}

void tto_rms_only(const uint16_t* input, const uint16_t* weight, uint32_t rows, uint32_t hidden,
                  uint16_t* output) {
    // hidden / 4 threads of 4 values, simdgroup trees over 32 lanes, then a tree over
    // the 32-slot stage (zero padded)
    const uint32_t simdgroups = hidden / 128;
    for (uint32_t r = 0; r < rows; ++r) {
        const uint16_t* in = input + static_cast<size_t>(r) * hidden;
        uint16_t* out = output + static_cast<size_t>(r) * hidden;
        float stage[32] = {0};
        float lanes[32];
        for (uint32_t sg = 0; sg < simdgroups; ++sg) {
            for (uint32_t l = 0; l < 32; ++l) lanes[l] = squares4(in + (sg * 32 + l) * 4);
            stage[sg] = adjacent32(lanes);
        }
        const float inverse =
            1.0f / std::sqrt(adjacent32(stage) / static_cast<float>(hidden) + kEps);
        for (uint32_t i = 0; i < hidden; ++i) {
            out[i] = mul16(weight[i], store16(widen(in[i]) * inverse));
        }
    }
}

void tto_dense_bf16(const uint16_t* input, const uint16_t* weights, uint32_t rows, uint32_t in_dim,
                    uint32_t out_dim, uint16_t* output, uint32_t threads) {
    parallel_for(out_dim, threads, [=](uint32_t n) {
        const uint16_t* w = weights + static_cast<size_t>(n) * in_dim;
        for (uint32_t r = 0; r < rows; ++r) {
            const uint16_t* x = input + static_cast<size_t>(r) * in_dim;
            // eight interleaved fp32 partial sums, folded pairwise: fixed order,
            // vectorisable, and close to what a blocked GPU sum does
            float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (uint32_t k = 0; k < in_dim; k += 8) {
                for (uint32_t e = 0; e < 8; ++e) acc[e] += widen(x[k + e]) * widen(w[k + e]);
            }
            const float total =
                ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
            output[static_cast<size_t>(r) * out_dim + n] = store16(total);
        }
    });
}

void tto_add_bf16(const uint16_t* a, const uint16_t* b, uint64_t count, uint16_t* out) {
    for (uint64_t i = 0; i < count; ++i) out[i] = add16(a[i], b[i]);
}

void tto_gdn_sequential_f64(const double* q, const double* k, const double* v,
                            const double* decay, const double* beta, uint32_t steps, uint32_t dk,
                            uint32_t dv, double* state, double* y) {
    for (uint32_t t = 0; t < steps; ++t) {
        const double* qt = q + static_cast<size_t>(t) * dk;
        const double* kt = k + static_cast<size_t>(t) * dk;
        for (uint32_t j = 0; j < dv; ++j) {
            double* row = state + static_cast<size_t>(j) * dk;
            double kv = 0.0;
            for (uint32_t i = 0; i < dk; ++i) {
                row[i] *= decay[t];
                kv += row[i] * kt[i];
            }
            const double delta = (v[static_cast<size_t>(t) * dv + j] - kv) * beta[t];
            double o = 0.0;
            for (uint32_t i = 0; i < dk; ++i) {
                row[i] += kt[i] * delta;
                o += row[i] * qt[i];
            }
            y[static_cast<size_t>(t) * dv + j] = o;
        }
    }
}

// Chunked (WY) evaluation.  Within a chunk starting from S0, with
// G_t = prod_{s<=t} decay_s:
//   u_t = beta_t (v_t - G_t S0 k_t - sum_{s<t} (G_t/G_s)(k_s.k_t) u_s)
//   y_t = G_t S0 q_t + sum_{s<=t} (G_t/G_s)(k_s.q_t) u_s
//   S_C = G_C S0 + sum_s (G_C/G_s) u_s k_s^T
void tto_gdn_chunked_f64(const double* q, const double* k, const double* v, const double* decay,
                         const double* beta, uint32_t steps, uint32_t dk, uint32_t dv,
                         uint32_t chunk, double* state, double* y) {
    std::vector<double> logG(chunk), u(static_cast<size_t>(chunk) * dv);
    for (uint32_t c0 = 0; c0 < steps; c0 += chunk) {
        const uint32_t len = std::min(chunk, steps - c0);
        double run = 0.0;
        for (uint32_t t = 0; t < len; ++t) {
            run += std::log(decay[c0 + t]);
            logG[t] = run;
        }
        for (uint32_t t = 0; t < len; ++t) {
            const double* kt = k + static_cast<size_t>(c0 + t) * dk;
            const double Gt = std::exp(logG[t]);
            for (uint32_t j = 0; j < dv; ++j) {
                const double* row = state + static_cast<size_t>(j) * dk;
                double s0k = 0.0;
                for (uint32_t i = 0; i < dk; ++i) s0k += row[i] * kt[i];
                u[static_cast<size_t>(t) * dv + j] = v[static_cast<size_t>(c0 + t) * dv + j] - Gt * s0k;
            }
            for (uint32_t s = 0; s < t; ++s) {
                const double* ks = k + static_cast<size_t>(c0 + s) * dk;
                double kk = 0.0;
                for (uint32_t i = 0; i < dk; ++i) kk += ks[i] * kt[i];
                const double w = std::exp(logG[t] - logG[s]) * kk;
                for (uint32_t j = 0; j < dv; ++j) {
                    u[static_cast<size_t>(t) * dv + j] -= w * u[static_cast<size_t>(s) * dv + j];
                }
            }
            for (uint32_t j = 0; j < dv; ++j) u[static_cast<size_t>(t) * dv + j] *= beta[c0 + t];
        }
        for (uint32_t t = 0; t < len; ++t) {
            const double* qt = q + static_cast<size_t>(c0 + t) * dk;
            const double Gt = std::exp(logG[t]);
            for (uint32_t j = 0; j < dv; ++j) {
                const double* row = state + static_cast<size_t>(j) * dk;
                double s0q = 0.0;
                for (uint32_t i = 0; i < dk; ++i) s0q += row[i] * qt[i];
                y[static_cast<size_t>(c0 + t) * dv + j] = Gt * s0q;
            }
            for (uint32_t s = 0; s <= t; ++s) {
                const double* ks = k + static_cast<size_t>(c0 + s) * dk;
                double kq = 0.0;
                for (uint32_t i = 0; i < dk; ++i) kq += ks[i] * qt[i];
                const double w = std::exp(logG[t] - logG[s]) * kq;
                for (uint32_t j = 0; j < dv; ++j) {
                    y[static_cast<size_t>(c0 + t) * dv + j] += w * u[static_cast<size_t>(s) * dv + j];
                }
            }
        }
        const double GC = std::exp(logG[len - 1]);
        for (uint32_t j = 0; j < dv; ++j) {
            double* row = state + static_cast<size_t>(j) * dk;
            for (uint32_t i = 0; i < dk; ++i) row[i] *= GC;
            for (uint32_t s = 0; s < len; ++s) {
                const double w = std::exp(logG[len - 1] - logG[s]) * u[static_cast<size_t>(s) * dv + j];
                const double* ks = k + static_cast<size_t>(c0 + s) * dk;
                for (uint32_t i = 0; i < dk; ++i) row[i] += w * ks[i];
            }
        }
    }
}

}  // extern "C"
