// The reference's alternative numerical families of full attention, behind their
// own kernel names and argument tables.  They give the same results as the
// primary operators within the reference's bands and exist so that a runtime
// policy selecting them keeps working; they are straightforward, not tuned.
//
//   src/backend/metal/kernels/attention.metal
//     attention_decode_vector_2pass_part (:854), _combine (:927): decode with keys
//     dealt round-robin to `blocks` sequence blocks, one online softmax per
//     (head, block), numerators kept in bf16.
//   src/backend/metal/kernels/prefill_attention.metal
//     attention_staged_scores_blk (:290), attention_staged_softmax_blk (:450),
//     attention_staged_softmax_bf16_blk (:543), attention_staged_values_blk (:638),
//     attention_gate_apply_blk (:1568): block prefill with the score matrix of a
//     query tile materialised in memory.
#include "../tt_internal.h"

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;

constexpr uint32_t kD = kAttnHeadDim;

__device__ __forceinline__ float widen(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t narrow(float v) {
    const uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float wave_sum(float v) {
    for (uint32_t off = 1; off < 64; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    for (uint32_t off = 1; off < 64; off <<= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ uint32_t pack_pair(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
// eight floats to bf16 hi and lo MFMA operands (x ~ hi + lo to 2^-17)
__device__ __forceinline__ void split8(const float* x, bf16x8& hi, bf16x8& lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (uint32_t e = 0; e < 4; ++e) {
        h[e] = pack_pair(x[2 * e], x[2 * e + 1]);
        l[e] = pack_pair(x[2 * e] - __uint_as_float(h[e] << 16),
                         x[2 * e + 1] - __uint_as_float(h[e] & 0xFFFF0000u));
    }
    hi = __builtin_bit_cast(bf16x8, u32x4{h[0], h[1], h[2], h[3]});
    lo = __builtin_bit_cast(bf16x8, u32x4{l[0], l[1], l[2], l[3]});
}

// ------------------------------------------------------ vector two-pass ------

// grid (2 kv heads, blocks) x 512: wave = one of the 8 query heads of the kv
// head, lane owns 4 dimensions.  Block b walks keys b, b + blocks, ...
__global__ __launch_bounds__(512) void vector_part_kernel(const uint16_t* q, const uint16_t* keys,
                                                          const uint16_t* values,
                                                          uint16_t* partials, float* sums,
                                                          float* maxs, uint32_t context,
                                                          uint32_t capacity, uint32_t blocks) {
    const uint32_t kv = blockIdx.x;
    const uint32_t block = blockIdx.y;
    const uint32_t head = kv * kAttnHeadsPerKv + (threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t d0 = lane * 4;
    float query[4], numerator[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    {
        const u32x2 raw = *reinterpret_cast<const u32x2*>(q + head * kD + d0);
        query[0] = kAttnScale * __uint_as_float(raw.x << 16);
        query[1] = kAttnScale * __uint_as_float(raw.x & 0xFFFF0000u);
        query[2] = kAttnScale * __uint_as_float(raw.y << 16);
        query[3] = kAttnScale * __uint_as_float(raw.y & 0xFFFF0000u);
    }
    float part_max = -INFINITY;
    float part_sum = 0.0f;
    const uint32_t n = context + 1;
    for (uint32_t position = block; position < n; position += blocks) {
        const uint64_t base = (static_cast<uint64_t>(kv) * capacity + position) * kD + d0;
        const u32x2 kr = *reinterpret_cast<const u32x2*>(keys + base);
        const u32x2 vr = *reinterpret_cast<const u32x2*>(values + base);
        float score = query[0] * __uint_as_float(kr.x << 16);
        score += query[1] * __uint_as_float(kr.x & 0xFFFF0000u);
        score += query[2] * __uint_as_float(kr.y << 16);
        score += query[3] * __uint_as_float(kr.y & 0xFFFF0000u);
        score = wave_sum(score);
        const float new_max = fmaxf(part_max, score);
        const float old_factor = __expf(part_max - new_max);
        const float score_factor = __expf(score - new_max);
        part_max = new_max;
        part_sum = part_sum * old_factor + score_factor;
        numerator[0] = numerator[0] * old_factor + score_factor * __uint_as_float(vr.x << 16);
        numerator[1] = numerator[1] * old_factor + score_factor * __uint_as_float(vr.x & 0xFFFF0000u);
        numerator[2] = numerator[2] * old_factor + score_factor * __uint_as_float(vr.y << 16);
        numerator[3] = numerator[3] * old_factor + score_factor * __uint_as_float(vr.y & 0xFFFF0000u);
    }
    const uint64_t record = (static_cast<uint64_t>(head) * blocks + block) * kD + d0;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) partials[record + i] = narrow(numerator[i]);
    if (lane == 0) {
        sums[static_cast<uint64_t>(head) * blocks + block] = part_sum;
        maxs[static_cast<uint64_t>(head) * blocks + block] = part_max;
    }
}

// grid 16 heads x 256: thread = output dimension.
__global__ __launch_bounds__(256) void vector_combine_kernel(const uint16_t* partials,
                                                             const float* sums, const float* maxs,
                                                             const uint16_t* gate, uint32_t blocks,
                                                             uint16_t* out) {
    __shared__ float shared[4];
    const uint32_t head = blockIdx.x;
    const uint32_t d = threadIdx.x;
    const float* head_sums = sums + static_cast<uint64_t>(head) * blocks;
    const float* head_maxs = maxs + static_cast<uint64_t>(head) * blocks;
    float global_max = -INFINITY;
    for (uint32_t block = d; block < blocks; block += 256) global_max = fmaxf(global_max, head_maxs[block]);
    global_max = wave_max(global_max);
    if ((d & 63) == 0) shared[d >> 6] = global_max;
    __syncthreads();
    global_max = fmaxf(fmaxf(shared[0], shared[1]), fmaxf(shared[2], shared[3]));
    __syncthreads();
    float denominator = 0.0f;
    for (uint32_t block = d; block < blocks; block += 256) {
        denominator += __expf(head_maxs[block] - global_max) * head_sums[block];
    }
    denominator = wave_sum(denominator);
    if ((d & 63) == 0) shared[d >> 6] = denominator;
    __syncthreads();
    denominator = (shared[0] + shared[1]) + (shared[2] + shared[3]);
    float numerator = 0.0f;
    for (uint32_t block = 0; block < blocks; ++block) {
        // a block with no key (max = -inf) carries factor exp(-inf) = 0
        const float factor = __expf(head_maxs[block] - global_max);
        numerator += factor * widen(partials[(static_cast<uint64_t>(head) * blocks + block) * kD + d]);
    }
    const float g = widen(gate[head * kD + d]);
    out[head * kD + d] = narrow((numerator / denominator) * (1.0f / (1.0f + __expf(-g))));
}

// attention_decode_vector_2pass_part: b0 q, b1 keys, b2 values, b3 partials bf16
// [16][blocks][256], b4 sums [16][blocks], b5 maxs, c6 context, c7 capacity,
// c8 blocks; grid (2, blocks) x (32, 8) (attention_fixture_probe.cpp:905-912).
int32_t op_vector_part(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t context = a.constant(6);
    const uint32_t capacity = a.constant(7);
    const uint32_t blocks = a.constant(8);
    a.require(blocks >= 1 && blocks <= 65535 && g.gx == kAttnKvHeads && g.gy == blocks &&
                  g.gz == 1 && g.tx == 32 && g.ty == 8 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(context_ok(context, capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    if (a.status != TT_OK) return a.status;
    const uint64_t cache = static_cast<uint64_t>(kAttnKvHeads) * capacity * kD * 2;
    const uint16_t* q = a.buffer<const uint16_t>(0, kAttnQueryValues * 2);
    const uint16_t* keys = a.buffer<const uint16_t>(1, cache);
    const uint16_t* values = a.buffer<const uint16_t>(2, cache);
    uint16_t* partials = a.buffer<uint16_t>(3, static_cast<uint64_t>(kAttnQueryHeads) * blocks * kD * 2);
    float* sums = a.buffer<float>(4, static_cast<uint64_t>(kAttnQueryHeads) * blocks * 4);
    float* maxs = a.buffer<float>(5, static_cast<uint64_t>(kAttnQueryHeads) * blocks * 4);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(vector_part_kernel, dim3(kAttnKvHeads, blocks), dim3(512), 0, stream, q, keys,
                       values, partials, sums, maxs, context, capacity, blocks);
    return TT_OK;
}

// attention_decode_vector_2pass_combine: b0 partials, b1 sums, b2 maxs, b3 gate,
// c4 blocks, b5 out; grid 16 x 1024 (attention_fixture_probe.cpp:913-919).
int32_t op_vector_combine(const Bindings& b, const Grid& g, hipStream_t stream,
                          bool validate_only) {
    Args a(b);
    const uint32_t blocks = a.constant(4);
    a.require(blocks >= 1 && blocks <= 65535 && g.gx == kAttnQueryHeads && g.gy == 1 && g.gz == 1 &&
                  g.tx == 1024 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint16_t* partials =
        a.buffer<const uint16_t>(0, static_cast<uint64_t>(kAttnQueryHeads) * blocks * kD * 2);
    const float* sums = a.buffer<const float>(1, static_cast<uint64_t>(kAttnQueryHeads) * blocks * 4);
    const float* maxs = a.buffer<const float>(2, static_cast<uint64_t>(kAttnQueryHeads) * blocks * 4);
    const uint16_t* gate = a.buffer<const uint16_t>(3, kAttnQueryValues * 2);
    uint16_t* out = a.buffer<uint16_t>(5, kAttnQueryValues * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(vector_combine_kernel, dim3(kAttnQueryHeads), dim3(256), 0, stream, partials,
                       sums, maxs, gate, blocks, out);
    return TT_OK;
}

// --------------------------------------------------------- staged family -----

// S[row][head][key] = scale * Q[row][head][:] . K[kv(head)][key][:] for every key
// below `visible`.  grid (ceil(visible/64), 16 heads, ceil(rows/16)) x 256: a wave
// owns a 16 x 16 tile on v_mfma_f32_16x16x32_bf16.
__global__ __launch_bounds__(256) void staged_scores_kernel(const uint16_t* query,
                                                            const uint16_t* keys, float* scores,
                                                            uint32_t visible, uint32_t capacity,
                                                            uint32_t rows) {
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t head = blockIdx.y;
    const uint32_t row0 = blockIdx.z * 16;
    const uint32_t key0 = blockIdx.x * 64 + wave * 16;
    if (key0 >= visible) return;
    const uint32_t qrow = min(row0 + m, rows - 1);
    const uint32_t krow = min(key0 + m, visible - 1);
    const uint16_t* qp = query + (static_cast<uint64_t>(qrow) * kAttnQueryHeads + head) * kD;
    const uint16_t* kp =
        keys + (static_cast<uint64_t>(head / kAttnHeadsPerKv) * capacity + krow) * kD;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t kk = 0; kk < 8; ++kk) {
        const bf16x8 qa = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(qp + kk * 32 + g * 8));
        const bf16x8 kb = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(kp + kk * 32 + g * 8));
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qa, kb, acc, 0, 0, 0);
    }
    // lane holds rows row0 + 4g + i of key column key0 + m
    const uint32_t key = key0 + m;
    if (key < visible) {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t row = row0 + g * 4 + i;
            if (row < rows) {
                scores[(static_cast<uint64_t>(row) * kAttnQueryHeads + head) * visible + key] =
                    acc[i] * kAttnScale;
            }
        }
    }
}

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* shared) {
    v = take_max ? wave_max(v) : wave_sum(v);
    __syncthreads();  // the previous use of `shared` is over
    if ((threadIdx.x & 63) == 0) shared[threadIdx.x >> 6] = v;
    __syncthreads();
    return take_max ? fmaxf(fmaxf(shared[0], shared[1]), fmaxf(shared[2], shared[3]))
                    : (shared[0] + shared[1]) + (shared[2] + shared[3]);
}

// In-place causal softmax of one (row, head) score row: keys [0, limit) with
// limit = query_context + row + 1, zeros from limit to visible.  BF16 = scores
// are unscaled bf16 dot products and the scale is applied here.
template <bool BF16>
__global__ __launch_bounds__(256) void staged_softmax_kernel(void* scores, uint32_t visible,
                                                             uint32_t query_context) {
    __shared__ float shared[4];
    const uint32_t row = blockIdx.x;
    const uint32_t head = blockIdx.y;
    const uint32_t limit = query_context + row + 1;
    if (limit > visible) return;
    const uint64_t base = (static_cast<uint64_t>(row) * kAttnQueryHeads + head) * visible;
    float* f = static_cast<float*>(scores) + base;
    uint16_t* h = static_cast<uint16_t*>(scores) + base;
    auto load = [&](uint32_t key) { return BF16 ? widen(h[key]) * kAttnScale : f[key]; };
    float maximum = -INFINITY;
    for (uint32_t key = threadIdx.x; key < limit; key += 256) maximum = fmaxf(maximum, load(key));
    maximum = block_reduce(maximum, true, shared);
    float denominator = 0.0f;
    for (uint32_t key = threadIdx.x; key < limit; key += 256) {
        const float value = __expf(load(key) - maximum);
        if (BF16) {
            h[key] = narrow(value);
        } else {
            f[key] = value;
        }
        denominator += value;
    }
    denominator = block_reduce(denominator, false, shared);
    const float inverse = 1.0f / denominator;
    for (uint32_t key = threadIdx.x; key < limit; key += 256) {
        if (BF16) {
            h[key] = narrow(widen(h[key]) * inverse);
        } else {
            f[key] *= inverse;
        }
    }
    for (uint32_t key = limit + threadIdx.x; key < visible; key += 256) {
        if (BF16) {
            h[key] = 0;
        } else {
            f[key] = 0.0f;
        }
    }
}

// Both forms are launched from a launcher template that only the host-side table
// instantiates; the device pass needs them named explicitly.
template __global__ void staged_softmax_kernel<false>(void*, uint32_t, uint32_t);
template __global__ void staged_softmax_kernel<true>(void*, uint32_t, uint32_t);

// out[row][head][dim] = bf16((P[row][head][:] . V[:, dim]) * sigmoid(gate)).
// grid (4, 16 heads, ceil(rows/16)) x 256: a wave owns 16 rows x 16 dims; the fp32
// probabilities enter the MFMA as bf16 hi/lo pairs, values are exact.
__global__ __launch_bounds__(256) void staged_values_kernel(const float* probabilities,
                                                            const uint16_t* values, uint16_t* out,
                                                            uint32_t visible, uint32_t capacity,
                                                            uint32_t rows, const uint16_t* gate) {
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t head = blockIdx.y;
    const uint32_t row0 = blockIdx.z * 16;
    const uint32_t dim = blockIdx.x * 64 + wave * 16 + m;  // this lane's B-operand column
    const uint32_t prow = min(row0 + m, rows - 1);
    const float* pp = probabilities + (static_cast<uint64_t>(prow) * kAttnQueryHeads + head) * visible;
    const uint16_t* vp = values + static_cast<uint64_t>(head / kAttnHeadsPerKv) * capacity * kD + dim;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t key0 = 0; key0 < visible; key0 += 32) {
        float p[8];
        uint32_t vbits[8];
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t key = key0 + g * 8 + e;
            const bool inside = key < visible;
            p[e] = inside ? pp[key] : 0.0f;
            vbits[e] = inside ? vp[static_cast<uint64_t>(key) * kD] : 0u;
        }
        bf16x8 p_hi, p_lo;
        split8(p, p_hi, p_lo);
        const bf16x8 vb = __builtin_bit_cast(
            bf16x8, u32x4{vbits[0] | (vbits[1] << 16), vbits[2] | (vbits[3] << 16),
                          vbits[4] | (vbits[5] << 16), vbits[6] | (vbits[7] << 16)});
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_lo, vb, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(p_hi, vb, acc, 0, 0, 0);
    }
    // lane holds rows row0 + 4g + i of dimension column `dim`
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint32_t row = row0 + g * 4 + i;
        if (row < rows) {
            const uint64_t at = (static_cast<uint64_t>(row) * kAttnQueryHeads + head) * kD + dim;
            out[at] = narrow(acc[i] / (1.0f + __expf(-widen(gate[at]))));
        }
    }
}

__global__ __launch_bounds__(256) void gate_apply_kernel(uint16_t* attended, const uint16_t* gate,
                                                         uint32_t count) {
    const uint32_t at = blockIdx.x * 256 + threadIdx.x;
    if (at >= count) return;
    attended[at] = narrow(widen(attended[at]) / (1.0f + __expf(-widen(gate[at]))));
}

uint64_t cache_bytes(uint32_t capacity) {
    return static_cast<uint64_t>(kAttnKvHeads) * capacity * kD * 2;
}

// attention_staged_scores_blk: b0 query(+tile), b1 keys, b2 scores f32
// [rows][16][visible], c3 visible, c4 capacity, c5 rows; grid (ceil(visible/32), 1,
// 16 * ceil(rows/16)) x 64 (prefill_step.cpp:1723-1741).
int32_t op_staged_scores(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t visible = a.constant(3);
    const uint32_t capacity = a.constant(4);
    const uint32_t rows = a.constant(5);
    a.require(rows >= 1 && rows <= 65535 && visible >= 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t row_tiles = (rows + 15) / 16;
    a.require(g.gx == (visible + 31) / 32 && g.gy == 1 && g.gz == kAttnQueryHeads * row_tiles &&
                  g.tx == 64 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(visible <= capacity, TT_CMD_CONTEXT_OUT_OF_RANGE);
    const uint16_t* query = a.buffer<const uint16_t>(0, static_cast<uint64_t>(rows) * kAttnQueryValues * 2);
    const uint16_t* keys = a.buffer<const uint16_t>(1, cache_bytes(capacity));
    float* scores = a.buffer<float>(2, static_cast<uint64_t>(rows) * kAttnQueryHeads * visible * 4);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(staged_scores_kernel, dim3((visible + 63) / 64, kAttnQueryHeads, row_tiles),
                       dim3(256), 0, stream, query, keys, scores, visible, capacity, rows);
    return TT_OK;
}

// attention_staged_softmax_blk / _bf16_blk: b0 scores (in place), c1 visible,
// c2 query_context; grid (rows, 16) x 256 (prefill_step.cpp:1743-1756, 1578-1589).
template <bool BF16>
int32_t op_staged_softmax(const Bindings& b, const Grid& g, hipStream_t stream,
                          bool validate_only) {
    Args a(b);
    const uint32_t visible = a.constant(1);
    const uint32_t query_context = a.constant(2);
    a.require(g.gx >= 1 && g.gx <= 65535 && g.gy == kAttnQueryHeads && g.gz == 1 && g.tx == 256 &&
                  g.ty == 1 && g.tz == 1 && visible >= 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t rows = static_cast<uint32_t>(g.gx);
    a.require(static_cast<uint64_t>(query_context) + rows <= visible, TT_CMD_CONTEXT_OUT_OF_RANGE);
    void* scores = a.buffer<void>(0, static_cast<uint64_t>(rows) * kAttnQueryHeads * visible *
                                         (BF16 ? 2 : 4));
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(staged_softmax_kernel<BF16>, dim3(rows, kAttnQueryHeads), dim3(256), 0, stream,
                       scores, visible, query_context);
    return TT_OK;
}

// attention_staged_values_blk: b0 probabilities f32, b1 values, b2 attended(+tile),
// c3 visible, c4 capacity, c5 rows, b6 gate(+tile); grid (8, 1, 16 * ceil(rows/16))
// x 64 (prefill_step.cpp:1758-1778).
int32_t op_staged_values(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t visible = a.constant(3);
    const uint32_t capacity = a.constant(4);
    const uint32_t rows = a.constant(5);
    a.require(rows >= 1 && rows <= 65535 && visible >= 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t row_tiles = (rows + 15) / 16;
    a.require(g.gx == kD / 32 && g.gy == 1 && g.gz == kAttnQueryHeads * row_tiles && g.tx == 64 &&
                  g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(visible <= capacity, TT_CMD_CONTEXT_OUT_OF_RANGE);
    const uint64_t row_bytes = static_cast<uint64_t>(rows) * kAttnQueryValues * 2;
    const float* probabilities =
        a.buffer<const float>(0, static_cast<uint64_t>(rows) * kAttnQueryHeads * visible * 4);
    const uint16_t* values = a.buffer<const uint16_t>(1, cache_bytes(capacity));
    uint16_t* out = a.buffer<uint16_t>(2, row_bytes);
    const uint16_t* gate = a.buffer<const uint16_t>(6, row_bytes);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(staged_values_kernel, dim3(kD / 64, kAttnQueryHeads, row_tiles), dim3(256), 0,
                       stream, probabilities, values, out, visible, capacity, rows, gate);
    return TT_OK;
}

// attention_gate_apply_blk: b0 attended (in place), b1 gate, c2 element count;
// grid ceil(count/256) x 256 (prefill_step.cpp:1644-1658).
int32_t op_gate_apply(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t count = a.constant(2);
    a.require(count >= 1 && g.gx == (static_cast<uint64_t>(count) + 255) / 256 && g.gy == 1 &&
                  g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    uint16_t* attended = a.buffer<uint16_t>(0, static_cast<uint64_t>(count) * 2);
    const uint16_t* gate = a.buffer<const uint16_t>(1, static_cast<uint64_t>(count) * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gate_apply_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, attended,
                       gate, count);
    return TT_OK;
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side table of launchers
const KernelDesc kAttentionFamilyKernels[] = {
    {"attention_decode_vector_2pass_part", op_vector_part},
    {"attention_decode_vector_2pass_combine", op_vector_combine},
    {"attention_staged_scores_blk", op_staged_scores},
    {"attention_staged_softmax_blk", op_staged_softmax<false>},
    {"attention_staged_softmax_bf16_blk", op_staged_softmax<true>},
    {"attention_staged_values_blk", op_staged_values},
    {"attention_gate_apply_blk", op_gate_apply},
};
const uint32_t kAttentionFamilyKernelCount =
    sizeof(kAttentionFamilyKernels) / sizeof(kAttentionFamilyKernels[0]);
#endif

}  // namespace tt
