// Gated DeltaNet layers for gfx950: causal conv1d(4) + bf16 SiLU + q/k
// RMS-norm, gate/decay evaluation, the gated delta-rule update of the
// [32][128][128] fp32 state, and the gated head norm; decode (one token per
// lane) and block prefill (a run of tokens of one lane).
//
// Operators registered here, with the reference kernels whose argument tables
// they accept (src/backend/metal/kernels/gdn.metal, prefill_gdn.metal):
//   gdn_prepare (gdn.metal:48), gdn_prepare_ms (:231), gdn_conv_blk (prefill_gdn.metal:4)
//   gdn_recurrence (:114), gdn_recurrence_ms (:309)
//   gdn_gate_norm (:174), gdn_gate_norm_ms (:552), gdn_gate_norm_blk (prefill_gdn.metal:283)
//   gdn_gates_blk (prefill_gdn.metal:94), gdn_recurrence_gates_blk (:137),
//   gdn_recurrence_blk (:204)
// plus the chunked evaluation of the block recurrence the reference lacks:
//   gdn_chunk_prepare_blk, gdn_chunk_scan_blk.
//
// State row layout: S[h][j][0..127] with the key index contiguous; one half
// wave (32 lanes x 4 floats = 512 B) owns one row, so a wave64 load
// instruction moves two rows = 1 KiB contiguous.  The 32-lane sums are xor
// butterflies (1,2,4,8,16), which is the adjacent-pairs tree of the reference
// bit for bit.
#include "../tt_internal.h"
#include "lane_sums.h"

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr uint32_t kGD = kGdnHeadDim;
constexpr uint32_t kCh = kGdnConvChannels;
constexpr uint32_t kMaxBatchRows = 16;

__device__ __forceinline__ float widen(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t narrow(float v) {
    const uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
// one bf16 arithmetic step: operate in fp32, round the result to bf16 (narrow, widened
// again: the carry of the rounding add runs into the exponent as it should, infinities stay,
// NaNs keep their upper bits)
__device__ __forceinline__ float rb(float v) {
    const uint32_t b = __float_as_uint(v);
    const uint32_t rounded = (b + 0x7FFFu + ((b >> 16) & 1u)) & 0xFFFF0000u;
    return __uint_as_float(v != v ? (b & 0xFFFF0000u) : rounded);
}

// bf16(1 / d) for a bf16 value d.  The reciprocal instruction is within one fp32 ulp of the
// quotient, and that is enough to round like the quotient itself: with d = D 2^a (D an
// 8-bit integer) and a midpoint between bf16 neighbours M = (2K + 1) 2^b, 1 - d M is a
// multiple of 2^-17 and not zero unless d is a power of two (where the instruction is
// exact), so 1 / d stays 2^-17 of its own size away from every midpoint.  Outside the range
// where the instruction keeps full precision the division is taken.
__device__ __forceinline__ float rb_reciprocal(float d) {
    const float size = fabsf(d);
    if (!(size >= 0x1p-100f && size <= 0x1p+100f)) return rb(1.0f / d);
    return rb(__builtin_amdgcn_rcpf(d));
}

// sigmoid in bf16 steps with the |x| branch (gdn.metal:76-79)
__device__ __forceinline__ float sigmoid_bf16(float x) {
    const float e = rb(expf(fabsf(x)));
    const float low = rb_reciprocal(rb(1.0f + e));
    return x < 0.0f ? low : rb(1.0f - low);
}

// The same bf16 steps for two values at once, rounded by the hardware's packed conversion
// (round to nearest even: the bits of rb for every finite value and for infinities; a NaN
// comes out quiet instead of with its upper bits kept) - one instruction and two to pull the
// halves apart again where rb takes five a value.  For the block kernels, whose time is these
// roundings.
typedef __attribute__((ext_vector_type(2))) float rb_f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 rb_bf16x2;
__device__ __forceinline__ uint32_t rb_pair_bits(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(rb_f32x2{a, b}, rb_bf16x2));
}
__device__ __forceinline__ void rb_pair(float& a, float& b) {
    const uint32_t pair = rb_pair_bits(a, b);
    a = __uint_as_float(pair << 16);
    b = __uint_as_float(pair & 0xFFFF0000u);
}
__device__ __forceinline__ float reciprocal_for_bf16(float d) {   // see rb_reciprocal
    const float size = fabsf(d);
    return (size >= 0x1p-100f && size <= 0x1p+100f) ? __builtin_amdgcn_rcpf(d) : 1.0f / d;
}
__device__ __forceinline__ void sigmoid_bf16_pair(float x0, float x1, float& s0, float& s1) {
    float e0 = expf(fabsf(x0)), e1 = expf(fabsf(x1));
    rb_pair(e0, e1);
    float d0 = 1.0f + e0, d1 = 1.0f + e1;
    rb_pair(d0, d1);
    float low0 = reciprocal_for_bf16(d0), low1 = reciprocal_for_bf16(d1);
    rb_pair(low0, low1);
    float high0 = 1.0f - low0, high1 = 1.0f - low1;
    rb_pair(high0, high1);
    s0 = x0 < 0.0f ? low0 : high0;
    s1 = x1 < 0.0f ? low1 : high1;
}

// decay and beta of one value head from the a / b projection rows
// (gdn.metal:133-150): softplus as bf16 LogAddExp, outer exponentials in fp32
__device__ __forceinline__ void head_gates(uint16_t a_bits, uint16_t b_bits, uint16_t a_log,
                                           uint16_t dt_bias, float& decay, float& beta) {
    const float shifted = rb(widen(a_bits) + widen(dt_bias));
    const float hi = shifted > 0.0f ? shifted : 0.0f;
    const float lo = shifted > 0.0f ? 0.0f : shifted;
    const float diff = rb(lo - hi);
    const float e = rb(expf(diff));
    const float one_plus = 1.0f + e;
    const float l1p = one_plus == 1.0f ? e : rb(e * (logf(one_plus) / (one_plus - 1.0f)));
    const float softplus = rb(hi + l1p);
    decay = expf(-expf(widen(a_log)) * softplus);
    beta = sigmoid_bf16(widen(b_bits));
}

// ------------------------------------------------------------ prepare/conv ---

struct PrepareArgs {
    const uint16_t* projection;   // [rows][projection_stride]
    const uint16_t* conv_in;      // [3][8192] (+ table offset per row)
    const uint16_t* conv_weights; // [8192][4]
    uint16_t* qk;                 // [rows][qk_stride]
    uint16_t* value;
    uint16_t* z;
    uint16_t* conv_out;
    const uint32_t* table;        // per row {conv_in, conv_out} element offsets, or null
    uint32_t projection_stride, qk_stride, value_stride, z_stride;
    uint32_t block_mode;          // 1: rows are consecutive tokens of one lane
    uint32_t rows;
    uint16_t* conv_tape;          // [40][16][3][8192] window after each row, or null
    uint32_t tape_layer;
};

constexpr uint32_t kBlockRowsPerGroup = 16;  // block mode: rows one workgroup walks

// grid (96, rows) x 128 (decode) or (96, ceil(rows/16)) (block mode, a workgroup
// walks 16 consecutive rows with a sliding tap window): groups 0..63 convolve one
// 128-channel head each (0..15 q, 16..31 k, 32..63 v), groups 64..95 copy the z gate.
__global__ __launch_bounds__(128) void gdn_prepare_kernel(PrepareArgs a) {
    __shared__ float partial[2];
    const uint32_t group = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint32_t row_begin = a.block_mode ? blockIdx.y * kBlockRowsPerGroup : blockIdx.y;
    const uint32_t row_end = a.block_mode ? min(a.rows, row_begin + kBlockRowsPerGroup) : row_begin + 1;
    if (group >= kCh / kGD) {
        const uint32_t index = (group - kCh / kGD) * kGD + lane;
        for (uint32_t row = row_begin; row < row_end; ++row) {
            a.z[static_cast<uint64_t>(row) * a.z_stride + index] =
                a.projection[static_cast<uint64_t>(row) * a.projection_stride + kCh + index];
        }
        return;
    }
    const uint16_t* conv_in = a.conv_in;
    uint16_t* conv_out = a.conv_out;
    if (a.table != nullptr) {
        conv_in += a.table[row_begin * 4];
        conv_out += a.table[row_begin * 4 + 1];
    }
    const uint32_t c = group * kGD + lane;
    // logical sequence = three state rows then the block's projection rows; a decode
    // row is a block of one
    const uint32_t first = a.block_mode ? row_begin : 0u;
    auto logical = [&](uint32_t index) -> uint16_t {
        if (index < 3) return conv_in[index * kCh + c];
        const uint32_t prow = a.block_mode ? index - 3 : row_begin;
        return a.projection[static_cast<uint64_t>(prow) * a.projection_stride + c];
    };
    uint16_t t0 = logical(first), t1 = logical(first + 1), t2 = logical(first + 2);
    const uint16_t* w = a.conv_weights + static_cast<uint64_t>(c) * 4;
    const float w0 = widen(w[0]), w1 = widen(w[1]), w2 = widen(w[2]), w3 = widen(w[3]);
    for (uint32_t row = row_begin; row < row_end; ++row) {
        const uint16_t t3 = a.projection[static_cast<uint64_t>(row) * a.projection_stride + c];
        // fixed four-term shape; bf16 x bf16 products are exact in fp32
        const float convolved = w0 * widen(t0) + w1 * widen(t1) + w2 * widen(t2) + w3 * widen(t3);
        const float conv_b = rb(convolved);
        const float act = rb(conv_b * sigmoid_bf16(conv_b));
        if (!a.block_mode || row == a.rows - 1) {
            conv_out[c] = t1;
            conv_out[kCh + c] = t2;
            conv_out[2 * kCh + c] = t3;
        }
        if (group < kGdnQkValues / kGD) {
            // RMS over the head: lane l (< 32) sums values 4l..4l+3, then the tree
            float sq = act * act;
            // gather 4 consecutive squares in ascending order onto lane 4k
            const float s1 = quad_lane<1>(sq);
            const float s2 = quad_lane<2>(sq);
            const float s3 = quad_lane<3>(sq);
            const float neighbour_sum = ((sq + s1) + s2) + s3;
            // lanes 4k hold thread-k partials; bring them to lanes 0..15 of each wave
            const uint32_t wave = lane >> 6;
            const uint32_t wl = lane & 63;
            float v = __shfl(neighbour_sum, (wl & 15) * 4, 64);  // 16 partials per wave
            // adjacent-pairs over 32 partials = pairs within each wave, then across
            v = row_sum(v);
            __syncthreads();  // the previous row's readers are done with `partial`
            if (wl == 0) partial[wave] = v;
            __syncthreads();
            const float total = partial[0] + partial[1];
            const float inverse = 1.0f / sqrtf(total / static_cast<float>(kGD) + kRmsNormEpsilon);
            const float scale = widen(group < kGdnKeyHeads ? kGdnQueryScaleBits : kGdnKeyScaleBits);
            a.qk[static_cast<uint64_t>(row) * a.qk_stride + c] = narrow(rb(act * inverse) * scale);
        } else {
            a.value[static_cast<uint64_t>(row) * a.value_stride + c - kGdnQkValues] = narrow(act);
        }
        t0 = t1;
        t1 = t2;
        t2 = t3;
    }
}

// Block form of the prepare step for rows that are consecutive tokens of one lane:
// a lane owns 8 adjacent channels (16-byte loads and stores), a workgroup of 256
// lanes 2048 channels, and walks kBlockRowsPerGroup rows with the three earlier taps
// in registers, so every projection element is read once.  grid.x: 0 q heads, 1 k
// heads, 2..3 value heads, 4..5 the z gate copy.  Same arithmetic, operation for
// operation, as gdn_prepare_kernel: a head's 128 squares are summed as 32 runs of
// four, then the adjacent-pairs tree - a lane holds two runs, 16 lanes a head.

__device__ __forceinline__ float widen_half(uint32_t word, uint32_t j) {
    return __uint_as_float((j & 1) ? (word & 0xFFFF0000u) : (word << 16));
}
__device__ __forceinline__ uint32_t narrow_pair(float a, float b) {
    return static_cast<uint32_t>(narrow(a)) | (static_cast<uint32_t>(narrow(b)) << 16);
}

__global__ __launch_bounds__(256) void gdn_prepare_block_kernel(PrepareArgs a) {
    const uint32_t unit = blockIdx.x * 256 + threadIdx.x;  // 8 channels each
    const uint32_t row_begin = blockIdx.y * kBlockRowsPerGroup;
    const uint32_t row_end = min(a.rows, row_begin + kBlockRowsPerGroup);
    if (unit >= kCh / 8) {
        const uint32_t index = (unit - kCh / 8) * 8;
        for (uint32_t row = row_begin; row < row_end; ++row) {
            *reinterpret_cast<u32x4*>(a.z + static_cast<uint64_t>(row) * a.z_stride + index) =
                *reinterpret_cast<const u32x4*>(
                    a.projection + static_cast<uint64_t>(row) * a.projection_stride + kCh + index);
        }
        return;
    }
    const uint32_t c = unit * 8;
    // logical sequence = three state rows, then the block's projection rows
    auto logical = [&](uint32_t index) -> u32x4 {
        if (index < 3) return *reinterpret_cast<const u32x4*>(a.conv_in + index * kCh + c);
        return *reinterpret_cast<const u32x4*>(
            a.projection + static_cast<uint64_t>(index - 3) * a.projection_stride + c);
    };
    u32x4 t0 = logical(row_begin), t1 = logical(row_begin + 1), t2 = logical(row_begin + 2);
    float w[8][4];
    {
        const u32x4* wp = reinterpret_cast<const u32x4*>(a.conv_weights + static_cast<uint64_t>(c) * 4);
#pragma unroll
        for (uint32_t q = 0; q < 4; ++q) {  // 16 bytes = two channels x four taps
            const u32x4 bits = wp[q];
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) w[q * 2 + (e >> 2)][e & 3] = widen_half(bits[e >> 1], e);
        }
    }
    const bool normalised = c < kGdnQkValues;
    const float scale = widen(c < kGdnQkValues / 2 ? kGdnQueryScaleBits : kGdnKeyScaleBits);
    for (uint32_t row = row_begin; row < row_end; ++row) {
        const u32x4 t3 = *reinterpret_cast<const u32x4*>(
            a.projection + static_cast<uint64_t>(row) * a.projection_stride + c);
        float act[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; j += 2) {
            // fixed four-term shape; bf16 x bf16 products are exact in fp32
            float conv[2];
#pragma unroll
            for (uint32_t e = 0; e < 2; ++e) {
                conv[e] = w[j + e][0] * widen_half(t0[j >> 1], e) + w[j + e][1] * widen_half(t1[j >> 1], e) +
                          w[j + e][2] * widen_half(t2[j >> 1], e) + w[j + e][3] * widen_half(t3[j >> 1], e);
            }
            rb_pair(conv[0], conv[1]);
            float gate0, gate1;
            sigmoid_bf16_pair(conv[0], conv[1], gate0, gate1);
            act[j] = conv[0] * gate0;
            act[j + 1] = conv[1] * gate1;
            rb_pair(act[j], act[j + 1]);
        }
        if (row == a.rows - 1) {
            *reinterpret_cast<u32x4*>(a.conv_out + c) = t1;
            *reinterpret_cast<u32x4*>(a.conv_out + kCh + c) = t2;
            *reinterpret_cast<u32x4*>(a.conv_out + 2 * kCh + c) = t3;
        }
        // what conv_out would hold had the block ended at this row
        // (prefill_gdn.metal:376-386): a block no longer than the tape records it
        if (a.conv_tape != nullptr && a.rows <= kGdnTapeRows) {
            uint16_t* tape =
                a.conv_tape + (static_cast<uint64_t>(a.tape_layer) * kGdnTapeRows + row) * 3 * kCh + c;
            *reinterpret_cast<u32x4*>(tape) = t1;
            *reinterpret_cast<u32x4*>(tape + kCh) = t2;
            *reinterpret_cast<u32x4*>(tape + 2 * kCh) = t3;
        }
        u32x4 packed;
        if (normalised) {
            const float run0 = ((act[0] * act[0] + act[1] * act[1]) + act[2] * act[2]) + act[3] * act[3];
            const float run1 = ((act[4] * act[4] + act[5] * act[5]) + act[6] * act[6]) + act[7] * act[7];
            float total = run0 + run1;
            total = row_sum(total);
            const float inverse = 1.0f / sqrtf(total / static_cast<float>(kGD) + kRmsNormEpsilon);
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                float n0 = act[2 * j] * inverse, n1 = act[2 * j + 1] * inverse;
                rb_pair(n0, n1);
                packed[j] = rb_pair_bits(n0 * scale, n1 * scale);
            }
            *reinterpret_cast<u32x4*>(a.qk + static_cast<uint64_t>(row) * a.qk_stride + c) = packed;
        } else {
            // already bf16 values: their upper halves are the bits
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                packed[j] = (__float_as_uint(act[2 * j]) >> 16) | (__float_as_uint(act[2 * j + 1]) & 0xFFFF0000u);
            }
            *reinterpret_cast<u32x4*>(a.value + static_cast<uint64_t>(row) * a.value_stride + c -
                                      kGdnQkValues) = packed;
        }
        t0 = t1;
        t1 = t2;
        t2 = t3;
    }
}

// ------------------------------------------------------------- recurrence ----

struct RecurrenceArgs {
    const uint16_t* qk;          // [rows or steps][qk_stride]
    const uint16_t* value;
    const uint16_t* projection;  // a/b rows (null when decay/beta are given)
    const uint16_t* a_log;
    const uint16_t* dt_bias;
    const float* decay;          // [steps][32] (scan with hoisted gates)
    const float* beta;
    const float* state_in;
    float* state_out;
    uint16_t* y;
    const uint32_t* table;       // per row {.., .., rec_in, rec_out} element offsets
    uint32_t qk_stride, value_stride, projection_stride, y_stride;
    uint32_t steps;              // tokens walked per state row (1 for decode)
    float* tape;                 // rollback tape (kTape instantiation only)
    uint32_t tape_layer;
};

// One half wave per state row; a 256-thread workgroup covers 8 rows of one
// (row-of-batch, value head).  grid (16, 32, rows).  The token loop serves the
// block-prefill register scan: state stays in registers across steps
// (prefill_gdn.metal:204-281).
//
// kTape (prefill_gdn.metal:432-511): a block of at most 16 steps also records, per
// step, what a later replay needs to rebuild the state up to any row: the delta of
// every state row, the keys as fp32, and {decay, beta} per value head.
template <bool kTape>
__global__ __launch_bounds__(256) void gdn_recurrence_kernel(RecurrenceArgs a) {
    const uint32_t half = threadIdx.x >> 5;              // 0..7
    const uint32_t lane = threadIdx.x & 31;
    const uint32_t j = blockIdx.x * 8 + half;            // value dimension
    const uint32_t h = blockIdx.y;                       // value head
    const uint32_t row = blockIdx.z;
    const uint32_t kh = h >> 1;
    const float* state_in = a.state_in;
    float* state_out = a.state_out;
    if (a.table != nullptr) {
        state_in += a.table[row * 4 + 2];
        state_out += a.table[row * 4 + 3];
    }
    const uint64_t base = (static_cast<uint64_t>(h) * kGD + j) * kGD + lane * 4;
    f32x4 st = *reinterpret_cast<const f32x4*>(state_in + base);
    const uint64_t row_qk = static_cast<uint64_t>(row) * a.qk_stride;
    const uint64_t row_v = static_cast<uint64_t>(row) * a.value_stride;
    const uint64_t row_p = static_cast<uint64_t>(row) * a.projection_stride;
    const uint64_t row_y = static_cast<uint64_t>(row) * a.y_stride;
    for (uint32_t step = 0; step < a.steps; ++step) {
        const uint16_t* qk = a.qk + row_qk + static_cast<uint64_t>(step) * a.qk_stride;
        float decay, beta;
        if (a.decay != nullptr) {
            decay = a.decay[step * kGdnValueHeads + h];
            beta = a.beta[step * kGdnValueHeads + h];
        } else {
            const uint16_t* proj =
                a.projection + row_p + static_cast<uint64_t>(step) * a.projection_stride;
            head_gates(proj[kGdnARowOffset + h], proj[kGdnBRowOffset + h], a.a_log[h],
                       a.dt_bias[h], decay, beta);
        }
        const u32x2 kq = *reinterpret_cast<const u32x2*>(qk + kGdnKOffset + kh * kGD + lane * 4);
        const u32x2 qq = *reinterpret_cast<const u32x2*>(qk + kh * kGD + lane * 4);
        const float k4[4] = {__uint_as_float(kq.x << 16), __uint_as_float(kq.x & 0xFFFF0000u),
                             __uint_as_float(kq.y << 16), __uint_as_float(kq.y & 0xFFFF0000u)};
        const float q4[4] = {__uint_as_float(qq.x << 16), __uint_as_float(qq.x & 0xFFFF0000u),
                             __uint_as_float(qq.y << 16), __uint_as_float(qq.y & 0xFFFF0000u)};
        float kv = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            st[i] *= decay;
            kv = fmaf(st[i], k4[i], kv);
        }
        kv = half_wave_sum(kv);
        const float v = widen(a.value[row_v + static_cast<uint64_t>(step) * a.value_stride +
                                      h * kGD + j]);
        const float delta = (v - kv) * beta;
        if constexpr (kTape) {
            if (a.steps <= kGdnTapeRows) {
                const uint64_t tape_row = static_cast<uint64_t>(a.tape_layer) * kGdnTapeRows + step;
                if (lane == 0) a.tape[(tape_row * kGdnValueHeads + h) * kGD + j] = delta;
                if (j == 0) {
                    if ((h & 1) == 0) {
                        *reinterpret_cast<f32x4*>(a.tape + kGdnTapeKeyOffset +
                                                  (tape_row * kGdnKeyHeads + kh) * kGD + lane * 4) =
                            f32x4{k4[0], k4[1], k4[2], k4[3]};
                    }
                    if (lane == 0) {
                        float* gates = a.tape + kGdnTapeGateOffset + (tape_row * kGdnValueHeads + h) * 2;
                        gates[0] = decay;
                        gates[1] = beta;
                    }
                }
            }
        }
        float out = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            st[i] = fmaf(k4[i], delta, st[i]);
            out = fmaf(st[i], q4[i], out);
        }
        out = half_wave_sum(out);
        if (lane == 0) {
            a.y[row_y + static_cast<uint64_t>(step) * a.y_stride + h * kGD + j] = narrow(out);
        }
    }
    __builtin_nontemporal_store(st, reinterpret_cast<f32x4*>(state_out + base));  // read next by a later dispatch
}

// gdn_tape_replay_blk (prefill_gdn.metal:520-569): the state after `steps` rows of
// a taped block, rebuilt from the state before the block.  The two update
// statements are the forward scan's own, so the result equals, bit for bit, what a
// forward scan of exactly `steps` rows would have stored.  Same state-row mapping as
// the forward kernel: grid (16, 32) x 256.
__global__ __launch_bounds__(256) void gdn_tape_replay_kernel(const float* tape,
                                                              const float* state_in,
                                                              float* state_out, uint32_t steps,
                                                              uint32_t tape_layer) {
    const uint32_t half = threadIdx.x >> 5;
    const uint32_t lane = threadIdx.x & 31;
    const uint32_t j = blockIdx.x * 8 + half;
    const uint32_t h = blockIdx.y;
    const uint32_t kh = h >> 1;
    const uint64_t base = (static_cast<uint64_t>(h) * kGD + j) * kGD + lane * 4;
    f32x4 st = *reinterpret_cast<const f32x4*>(state_in + base);
    for (uint32_t step = 0; step < steps; ++step) {
        const uint64_t tape_row = static_cast<uint64_t>(tape_layer) * kGdnTapeRows + step;
        const float decay = tape[kGdnTapeGateOffset + (tape_row * kGdnValueHeads + h) * 2];
        const float delta = tape[(tape_row * kGdnValueHeads + h) * kGD + j];
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(
            tape + kGdnTapeKeyOffset + (tape_row * kGdnKeyHeads + kh) * kGD + lane * 4);
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            st[i] *= decay;
            st[i] = fmaf(k4[i], delta, st[i]);
        }
    }
    *reinterpret_cast<f32x4*>(state_out + base) = st;
}

// gdn_gates_blk: decay/beta for every (step, head) (prefill_gdn.metal:94-135)
__global__ void gdn_gates_kernel(const uint16_t* projection, const uint16_t* a_log,
                                 const uint16_t* dt_bias, float* decay, float* beta,
                                 uint32_t steps) {
    const uint32_t h = threadIdx.x;
    const uint32_t step = blockIdx.x * blockDim.y + threadIdx.y;
    if (h >= kGdnValueHeads || step >= steps) return;
    const uint16_t* proj = projection + static_cast<uint64_t>(step) * kGdnProjectionRows;
    float d, b;
    head_gates(proj[kGdnARowOffset + h], proj[kGdnBRowOffset + h], a_log[h], dt_bias[h], d, b);
    decay[step * kGdnValueHeads + h] = d;
    beta[step * kGdnValueHeads + h] = b;
}

// --------------------------------------------------------------- gate norm ---

// grid (32, ceil(rows / rows_per_group)) x 128: y * rsqrt(mean y^2 + eps) rounded to
// bf16, times the weight rounded to bf16, times fp32 SiLU(z); one bf16 rounding at
// the end (gdn.metal:174-207).
__global__ __launch_bounds__(128) void gdn_gate_norm_kernel(const uint16_t* y, const uint16_t* z,
                                                            const uint16_t* weight, uint16_t* out,
                                                            uint32_t stride, uint32_t rows,
                                                            uint32_t rows_per_group) {
    __shared__ float partial[2];
    const uint32_t head = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const float w = widen(weight[lane]);
    const uint32_t row_end = min(rows, (blockIdx.y + 1) * rows_per_group);
    for (uint32_t row = blockIdx.y * rows_per_group; row < row_end; ++row) {
        const uint64_t at = static_cast<uint64_t>(row) * stride + head * kGD + lane;
        const float v = widen(y[at]);
        const float sq = v * v;
        const float s1 = quad_lane<1>(sq);
        const float s2 = quad_lane<2>(sq);
        const float s3 = quad_lane<3>(sq);
        const float four = ((sq + s1) + s2) + s3;
        const uint32_t wl = lane & 63;
        float t = __shfl(four, (wl & 15) * 4, 64);
        t = row_sum(t);
        __syncthreads();  // the previous row's readers are done with `partial`
        if (wl == 0) partial[lane >> 6] = t;
        __syncthreads();
        const float inverse =
            1.0f / sqrtf((partial[0] + partial[1]) / static_cast<float>(kGD) + kRmsNormEpsilon);
        const float normed = rb(w * rb(v * inverse));
        const float g = widen(z[at]);
        const float low = 1.0f / (1.0f + expf(fabsf(g)));
        const float sig = g < 0.0f ? low : 1.0f - low;
        out[at] = narrow((g * sig) * normed);
    }
}

// Block form: a lane owns 8 adjacent channels, 16 lanes a head, a workgroup of 256
// lanes half a row; grid (2, ceil(rows / rows_per_group)).  Same arithmetic as
// gdn_gate_norm_kernel (two runs of four squares per lane, then the pair tree).
__global__ __launch_bounds__(256) void gdn_gate_norm_block_kernel(
    const uint16_t* y, const uint16_t* z, const uint16_t* weight, uint16_t* out, uint32_t stride,
    uint32_t rows, uint32_t rows_per_group) {
    const uint32_t c = (blockIdx.x * 256 + threadIdx.x) * 8;
    float w[8];
    {
        const u32x4 bits = *reinterpret_cast<const u32x4*>(weight + (c & (kGD - 1)));
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) w[j] = widen_half(bits[j >> 1], j);
    }
    const uint32_t row_end = min(rows, (blockIdx.y + 1) * rows_per_group);
    for (uint32_t row = blockIdx.y * rows_per_group; row < row_end; ++row) {
        const uint64_t at = static_cast<uint64_t>(row) * stride + c;
        const u32x4 yb = *reinterpret_cast<const u32x4*>(y + at);
        const u32x4 zb = *reinterpret_cast<const u32x4*>(z + at);
        float v[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) v[j] = widen_half(yb[j >> 1], j);
        const float run0 = ((v[0] * v[0] + v[1] * v[1]) + v[2] * v[2]) + v[3] * v[3];
        const float run1 = ((v[4] * v[4] + v[5] * v[5]) + v[6] * v[6]) + v[7] * v[7];
        float total = run0 + run1;
        total = row_sum(total);
        const float inverse = 1.0f / sqrtf(total / static_cast<float>(kGD) + kRmsNormEpsilon);
        u32x4 packed;
#pragma unroll
        for (uint32_t j = 0; j < 8; j += 2) {
            float r[2];
            float n0 = v[j] * inverse, n1 = v[j + 1] * inverse;
            rb_pair(n0, n1);
            n0 *= w[j];
            n1 *= w[j + 1];
            rb_pair(n0, n1);
            const float normed[2] = {n0, n1};
#pragma unroll
            for (uint32_t e = 0; e < 2; ++e) {
                const float g = widen_half(zb[j >> 1], e);
                const float low = 1.0f / (1.0f + expf(fabsf(g)));
                const float sig = g < 0.0f ? low : 1.0f - low;
                r[e] = (g * sig) * normed[e];
            }
            packed[j >> 1] = rb_pair_bits(r[0], r[1]);
        }
        *reinterpret_cast<u32x4*>(out + at) = packed;
    }
}

// ------------------------------------------------- fused decode step ---------

struct FusedDecodeArgs {
    const uint16_t* projection;    // [rows][projection_stride]
    const uint16_t* conv_pool;     // planes addressed through the table
    uint16_t* conv_pool_out;
    const uint16_t* conv_weights;  // [8192][4]
    const uint16_t* a_log;
    const uint16_t* dt_bias;
    const float* rec_pool;
    float* rec_pool_out;
    const uint16_t* norm_weight;   // [128]
    uint16_t* out;                 // [rows][out_stride]
    const uint32_t* table;         // per row {conv_in, conv_out, rec_in, rec_out} element offsets
    uint32_t projection_stride, out_stride;
};

// One decode step of a whole value head in one workgroup: conv + SiLU of the
// head's q, k and v channels, q/k norms, gates, the delta-rule update of the
// head's 128 x 128 state and the gate-norm of its 128 outputs, with the
// arithmetic of gdn_prepare / gdn_recurrence / gdn_gate_norm operation for
// operation (so the results are theirs bit for bit) and none of their
// intermediates in memory.  grid (32 heads, rows) x kFusedThreads: sixteen half waves, each
// walking 8 state rows with 4 key columns per lane.  The two value heads that
// share a key head both evaluate its q/k channels; the even one writes their new
// conv history.
// 512 threads: sixteen half waves of eight state rows.  1024 (four rows each) measured 0.2 us
// slower - more waves to start and to meet at the barriers than the shorter row loop wins.
constexpr uint32_t kFusedThreads = 512;

template <uint32_t kThreads>
__global__ __launch_bounds__(kThreads) void gdn_decode_fused_kernel(FusedDecodeArgs a) {
    constexpr uint32_t kWavesHere = kThreads / 64;
    constexpr uint32_t kRowsEach = kGD / (kThreads / 32);   // state rows a half wave walks
    static_assert(kThreads >= 3 * kGD && (kRowsEach == 4 || kRowsEach == 8), "one thread per q, k, v channel; whole slices per half wave");
    __shared__ float act_v[kGD];        // activated v channels (bf16 values)
    __shared__ float qk_n[2 * kGD];     // normalised, scaled q | k (bf16 values)
    __shared__ float y_head[kGD];       // bf16 values of the head's outputs
    __shared__ float wave_squares[kWavesHere];   // per wave: sum of its 64 channels' squares
    __shared__ float wave_outputs[kWavesHere];   // per wave: sum of its outputs' squares
    const uint32_t h = blockIdx.x;
    const uint32_t row = blockIdx.y;
    const uint32_t kh = h >> 1;
    const uint32_t tid = threadIdx.x;
    const uint16_t* proj = a.projection + static_cast<uint64_t>(row) * a.projection_stride;
    const uint16_t* conv_in = a.conv_pool + a.table[row * 4];
    uint16_t* conv_out = a.conv_pool_out + a.table[row * 4 + 1];
    const float* state_in = a.rec_pool + a.table[row * 4 + 2];
    float* state_out = a.rec_pool_out + a.table[row * 4 + 3];
    const uint32_t half = tid >> 5;
    const uint32_t lane = tid & 31;
    // Loads come back in the order they were requested.  The few bytes the conv, norm and
    // gate stages need go out first, the head's 64 KiB of state right behind them: those
    // stages then run while the state is still arriving instead of after it.
    // Every thread issues every one of them (threads past the 384 channels repeat the value
    // channels): a load inside a branch would be waited for before the branch ends, one
    // round trip after the other.
    const uint16_t z_bits = proj[kCh + h * kGD + (tid & 127)];
    const uint16_t norm_bits = a.norm_weight[tid & 127];
    const uint32_t part = min(tid >> 7, 2u);  // 0 q, 1 k, 2 v
    const uint32_t c = (part == 0 ? kh * kGD : part == 1 ? kGdnKOffset + kh * kGD
                                                         : kGdnQkValues + h * kGD) + (tid & 127);
    const uint16_t t0 = conv_in[c];
    const uint16_t t1 = conv_in[kCh + c];
    const uint16_t t2 = conv_in[2 * kCh + c];
    const uint16_t t3 = proj[c];
    const uint16_t* w = a.conv_weights + static_cast<uint64_t>(c) * 4;
    const uint16_t w0 = w[0], w1 = w[1], w2 = w[2], w3 = w[3];
    const uint16_t gate_a = proj[kGdnARowOffset + h];
    const uint16_t gate_b = proj[kGdnBRowOffset + h];
    const uint16_t gate_log = a.a_log[h];
    const uint16_t gate_bias = a.dt_bias[h];
    f32x4 st[kRowsEach];
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) {
        const uint32_t j = half * kRowsEach + it;
        st[it] = *reinterpret_cast<const f32x4*>(
            state_in + (static_cast<uint64_t>(h) * kGD + j) * kGD + lane * 4);
    }

    // computed by every thread as well, so that the loads above cannot be moved into a
    // branch behind the state loads; only the stores are conditional
    const float convolved = widen(w0) * widen(t0) + widen(w1) * widen(t1) +
                            widen(w2) * widen(t2) + widen(w3) * widen(t3);
    const float conv_b = rb(convolved);
    const float activated = rb(conv_b * sigmoid_bf16(conv_b));
    float decay, beta;
    head_gates(gate_a, gate_b, gate_log, gate_bias, decay, beta);
    // the output gate needs nothing but z: done here, while the state is in flight
    const float gate_value = widen(z_bits);
    const float gate_low = 1.0f / (1.0f + expf(fabsf(gate_value)));
    const float gated = gate_value * (gate_value < 0.0f ? gate_low : 1.0f - gate_low);
    if (tid < 3 * kGD) {
        if (part == 2) act_v[tid - 2 * kGD] = activated;
        if (part == 2 || (h & 1) == 0) {
            conv_out[c] = t1;
            conv_out[kCh + c] = t2;
            conv_out[2 * kCh + c] = t3;
        }
    }
    // RMS over the q head (waves 0, 1) and the k head (waves 2, 3) without a trip through
    // LDS per stage: a quad sums its four squares in order (slice l of gdn_prepare's lane l),
    // then the adjacent-pairs tree over the 32 slices runs over quads (mirrors of a half row
    // and a row: a quad holds one value), rows, the halves of the wave, and the two waves.
    const float sq = activated * activated;
    float slices = ((quad_lane<0>(sq) + quad_lane<1>(sq)) + quad_lane<2>(sq)) + quad_lane<3>(sq);
    slices += lane_dpp<0x141>(slices);   // row_half_mirror: the neighbouring quad
    slices += lane_dpp<0x140>(slices);   // row_mirror: the neighbouring pair of quads
    slices += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(slices), 0x401F));  // lane ^ 16
    const float wave_slices = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(slices), 0)) +
                              __int_as_float(__builtin_amdgcn_readlane(__float_as_int(slices), 32));
    if ((tid & 63) == 0) wave_squares[tid >> 6] = wave_slices;
    __syncthreads();
    if (tid < 2 * kGD) {
        const float sum = wave_squares[(tid >> 7) * 2] + wave_squares[(tid >> 7) * 2 + 1];
        const float inverse = 1.0f / sqrtf(sum / static_cast<float>(kGD) + kRmsNormEpsilon);
        const float scale = widen(tid < kGD ? kGdnQueryScaleBits : kGdnKeyScaleBits);
        qk_n[tid] = rb(rb(activated * inverse) * scale);
    }
    __syncthreads();

    float q4[4], k4[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        q4[i] = qk_n[lane * 4 + i];
        k4[i] = qk_n[kGD + lane * 4 + i];
    }
    // The eight rows of a half wave go through each step side by side, not row after row:
    // a row's two cross-lane sums are chains of dependent lane exchanges (the last through the
    // LDS crossbar), and eight independent chains fill each other's waits.
    float kv[kRowsEach], out[kRowsEach];
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) {
        kv[it] = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            st[it][i] *= decay;
            kv[it] = fmaf(st[it][i], k4[i], kv[it]);
        }
    }
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) kv[it] = half_wave_sum(kv[it]);
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) {
        const float delta = (act_v[half * kRowsEach + it] - kv[it]) * beta;
        out[it] = 0.0f;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            st[it][i] = fmaf(k4[i], delta, st[it][i]);
            out[it] = fmaf(st[it][i], q4[i], out[it]);
        }
        // written once, read by the next token's dispatch at the earliest: stored past the
        // cache (nontemporal), so the dispatch does not end on a write-back of the whole state
        __builtin_nontemporal_store(st[it], reinterpret_cast<f32x4*>(
            state_out + (static_cast<uint64_t>(h) * kGD + half * kRowsEach + it) * kGD + lane * 4));
    }
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) out[it] = half_wave_sum(out[it]);
    // Gate-norm: every lane of a half wave holds its eight outputs, two slices of four of the
    // RMS tree (gdn_gate_norm's lane sums four squares in order, then adjacent pairs over the
    // 32 slices).  The first step of the tree is the half wave's own pair, the second the
    // wave's two halves, the rest the eight waves - one value per wave through LDS.
    float y8[kRowsEach], squares[kRowsEach / 4];
#pragma unroll
    for (uint32_t it = 0; it < kRowsEach; ++it) y8[it] = rb(out[it]);
#pragma unroll
    for (uint32_t sl = 0; sl < kRowsEach / 4; ++sl) {
        squares[sl] = ((y8[4 * sl] * y8[4 * sl] + y8[4 * sl + 1] * y8[4 * sl + 1]) +
                       y8[4 * sl + 2] * y8[4 * sl + 2]) + y8[4 * sl + 3] * y8[4 * sl + 3];
    }
    const float pair = kRowsEach == 8 ? squares[0] + squares[kRowsEach / 4 - 1] : squares[0];
    const float wave_pair = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pair), 0)) +
                            __int_as_float(__builtin_amdgcn_readlane(__float_as_int(pair), 32));
    if (lane == 0) {
#pragma unroll
        for (uint32_t it = 0; it < kRowsEach; ++it) y_head[half * kRowsEach + it] = y8[it];
    }
    if ((tid & 63) == 0) wave_outputs[tid >> 6] = wave_pair;
    __syncthreads();
    if (tid < kGD) {
        float level[kWavesHere];
#pragma unroll
        for (uint32_t w = 0; w < kWavesHere; ++w) level[w] = wave_outputs[w];
#pragma unroll
        for (uint32_t width = kWavesHere; width > 1; width >>= 1) {   // adjacent pairs, level by level
#pragma unroll
            for (uint32_t w = 0; w < width / 2; ++w) level[w] = level[2 * w] + level[2 * w + 1];
        }
        const float total = level[0];
        const float inv = 1.0f / sqrtf(total / static_cast<float>(kGD) + kRmsNormEpsilon);
        const float normed = rb(widen(norm_bits) * rb(y_head[tid] * inv));
        a.out[static_cast<uint64_t>(row) * a.out_stride + h * kGD + tid] = narrow(gated * normed);
    }
}

// ------------------------------------------- chunked (WY) block prefill ------
//
// The reference walks a block token by token (prefill_gdn.metal:204-281).  The
// same recurrence is evaluated here 64 tokens at a time so that its products run
// on MFMA.  With g_t the product of the decays up to token t inside a chunk,
// L[t][s] = beta_t (g_t/g_s)(k_t.k_s) for s < t and A[t][s] = (g_t/g_s)(q_t.k_s)
// for s <= t, the per-token deltas u_t of the delta rule satisfy
//     (I + L) U = beta o (V - (g o K) S0^T)
// so with Wk = (I+L)^-1 (beta o g o K) and Wv = (I+L)^-1 (beta o V):
//     U  = Wv - Wk S0^T
//     Y  = (g o Q) S0^T + A U
//     S' = g_C S0 + U^T ((g_C/g) o K)
// Stage 1 (parallel over chunks and heads) builds Wk, Wv, g o Q, (g_C/g) o K and
// A for every chunk: the k.k and q.k Gram tiles on MFMA, the unit-triangular
// solve by forward substitution in fp32 (one right-hand-side column per thread).
// Stage 2 walks the chunks in order, one workgroup per (value head, 32-wide
// slice of the value dimension), with the fp32 state slice held in MFMA
// accumulators and every product on v_mfma_f32_16x16x32_bf16.

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

constexpr uint32_t kChunk = 64;
// per (chunk, head) record, byte offsets.  Everything that feeds the recurrent
// state or the output keeps fp32-grade precision: bf16 MFMA operands that are
// not exact already are stored as hi/lo pairs, Wv in fp32 (it is only added).
// Operands are stored in the order stage 2 consumes them: one 1 KiB fragment per
// wave-level load (64 lanes x 16 B, lane = 16 g + m), so every load instruction
// of stage 2 reads whole cache lines.
//   token-by-key operands (Wk hi, Wk lo, Q): fragment (token tile w, key step kk),
//     lane (m, g) = token 16w+m, keys 32kk+8g..+7
//   K^T: fragment (key tile 2w+mt, token step k2), lane = key 16(2w+mt)+m, tokens 32k2+8g..+7
//   A hi/lo: fragment (token tile w, token step k2), lane = token 16w+m, tokens 32k2+8g..+7
//   Wv (fp32): fragment (value slice of 16, token tile w), lane = value 16 slice+m, tokens 16w+4g..+3
constexpr uint32_t kRecWkHi = 0;
constexpr uint32_t kRecWkLo = 16384;
constexpr uint32_t kRecQ = 32768;
constexpr uint32_t kRecKt = 49152;
constexpr uint32_t kRecAqkHi = 65536;
constexpr uint32_t kRecAqkLo = 73728;
constexpr uint32_t kRecWv = 81920;
constexpr uint32_t kRecRatio = 114688;                  // f32  [64]: g_C / g_t
constexpr uint32_t kRecGam = 114944;                    // f32  [64]: g_t
constexpr uint32_t kRecGamma = 115200;                  // f32: g_C
constexpr uint32_t kRecBytes = 115712;

struct ChunkPrepareArgs {
    const uint16_t* qk;      // [rows][4096]
    const uint16_t* value;   // [rows][4096]
    const float* decay;      // [rows][32]
    const float* beta;       // [rows][32]
    uint8_t* scratch;        // [chunks][32] records
    uint32_t rows;
};

__device__ __forceinline__ bf16x8 operand(const uint16_t* p) {
    return __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(p));
}

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

// Two floats to a packed bf16 pair with the hardware conversion (round to
// nearest even).  Used for MFMA operands only: operator outputs go through
// narrow().
__device__ __forceinline__ uint32_t pack_pair(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
// x ~ hi + lo to 2^-17: the pair's hi parts, then the remainders.
__device__ __forceinline__ void split_pair(float a, float b, uint32_t& hi, uint32_t& lo) {
    hi = pack_pair(a, b);
    lo = pack_pair(a - __uint_as_float(hi << 16), b - __uint_as_float(hi & 0xFFFF0000u));
}

// Four floats to packed hi and lo bf16 quads.
__device__ __forceinline__ void split4(const f32x4 v, u32x2& hi, u32x2& lo) {
    uint32_t h0, h1, l0, l1;
    split_pair(v[0], v[1], h0, l0);
    split_pair(v[2], v[3], h1, l1);
    hi = u32x2{h0, h1};
    lo = u32x2{l0, l1};
}

// Splits eight floats into bf16 hi and lo MFMA operands.
__device__ __forceinline__ void split8(const float* x, bf16x8& hi, bf16x8& lo) {
    uint32_t h[4], l[4];
#pragma unroll
    for (uint32_t e = 0; e < 4; ++e) split_pair(x[2 * e], x[2 * e + 1], h[e], l[e]);
    hi = __builtin_bit_cast(bf16x8, u32x4{h[0], h[1], h[2], h[3]});
    lo = __builtin_bit_cast(bf16x8, u32x4{l[0], l[1], l[2], l[3]});
}

// A wave's 16 x 16 MFMA result tile (this lane: rows 4g+i of column m) as bf16 hi/lo
// pairs into fragment order: through a per-wave LDS tile so that every lane ends
// up with eight consecutive columns of one row and stores 16 bytes; lanes 0..31
// write the hi fragment piece, lanes 32..63 the lo piece, 512 contiguous bytes each.
// `piece` is the byte offset of the tile's 512-byte run inside a fragment array.
__device__ __forceinline__ void store_tile_hi_lo(uint16_t (*tile)[16][24], const f32x4 acc,
                                                 uint32_t lane, uint8_t* hi_base, uint8_t* lo_base,
                                                 uint32_t piece) {
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        const uint16_t hi = narrow(acc[i]);
        tile[0][g * 4 + i][m] = hi;
        tile[1][g * 4 + i][m] = narrow(acc[i] - widen(hi));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const uint32_t half = lane >> 5;
    const uint32_t row = lane & 15;
    const uint32_t group = (lane >> 4) & 1;  // which run of eight columns
    const u32x4 v = *reinterpret_cast<const u32x4*>(&tile[half][row][group * 8]);
    *reinterpret_cast<u32x4*>((half ? lo_base : hi_base) + piece + (group * 16 + row) * 16) = v;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Stage 1, grid (chunks, 32) x 256: decay products, Gram tiles on MFMA, the
// inverse T of the unit lower-triangular I + L (diagonal 16x16 blocks by forward
// substitution in registers, the rest by block recursion, all fp32), then
// [Wk | Wv] = T (beta o [g o K | V]) on MFMA with hi/lo operands.
__global__ __launch_bounds__(256) void gdn_chunk_prepare_kernel(ChunkPrepareArgs a) {
    constexpr uint32_t kLd = 68;  // fp32 row stride: 16-byte aligned, bank-skewed
    constexpr uint32_t kTileLd = 136;  // bf16 row stride of the key and value tiles
    constexpr uint32_t kStripLd = 72;  // 64 rows + pad: 16-byte reads of 16 columns spread over the banks
    __shared__ __attribute__((aligned(16))) float lower[kChunk][kLd];
    // inverses of the four 16x16 diagonal blocks of I + L: tdiag[16 b + r][c]
    __shared__ __attribute__((aligned(16))) float tdiag[kChunk][20];
    // per wave: a 16-column strip of the solution as bf16 hi/lo, [half][column][row]
    // (rows 0..47 the finished block rows, 48..63 the right-hand side being solved),
    // rows contiguous so that a lane reads its 8 contraction slots with 16 bytes; the
    // same memory stages the 16x16 result tiles on their way to the record
    __shared__ __attribute__((aligned(16))) uint16_t strip[4][2][16][kStripLd];
    __shared__ __attribute__((aligned(16))) float log_g[kChunk];
    __shared__ __attribute__((aligned(16))) float scale_k[kChunk];  // beta_t g_t
    __shared__ __attribute__((aligned(16))) float scale_v[kChunk];  // beta_t
    // the head's keys and values of the chunk, row-major [token][128], rows padded to
    // 272 bytes so that 16-byte operand reads of 16 rows spread over the banks
    __shared__ __attribute__((aligned(16))) uint16_t ktile[kChunk][kTileLd];
    __shared__ __attribute__((aligned(16))) uint16_t vtile[kChunk][kTileLd];
    const uint32_t chunk = blockIdx.x;
    const uint32_t h = blockIdx.y;
    const uint32_t kh = h >> 1;
    const uint32_t tid = threadIdx.x;
    const uint32_t wave = tid >> 6;
    const uint32_t lane = tid & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t t0 = chunk * kChunk;
    const uint32_t valid = min(kChunk, a.rows - t0);
    uint8_t* rec = a.scratch + (static_cast<uint64_t>(chunk) * kGdnValueHeads + h) * kRecBytes;

    // Keys and values of the chunk into LDS with 16-byte loads: 16 lanes per row, 16
    // rows per pass; rows past the block repeat the last one (their scales are zero).
    // The wave's query rows (token rows 16w .. 16w+15) are requested with them.
    const bool is_k = wave < 2;
    bf16x8 aq[4];
    {
        const uint16_t* qrow = a.qk + static_cast<uint64_t>(t0 + min(wave * 16 + m, valid - 1)) * kGdnQkValues +
                               kh * kGD;
#pragma unroll
        for (uint32_t kk = 0; kk < 4; ++kk) aq[kk] = operand(qrow + kk * 32 + g * 8);
    }
    {
        const uint16_t* ksrc = a.qk + static_cast<uint64_t>(t0) * kGdnQkValues + kGdnKOffset + kh * kGD;
        const uint16_t* vsrc = a.value + static_cast<uint64_t>(t0) * kGdnValueValues + h * kGD;
        u32x4 kv[4], vv[4];
#pragma unroll
        for (uint32_t pass = 0; pass < 4; ++pass) {
            const uint32_t r = min(pass * 16 + (tid >> 4), valid - 1);
            kv[pass] = *reinterpret_cast<const u32x4*>(ksrc + static_cast<uint64_t>(r) * kGdnQkValues +
                                                       (tid & 15) * 8);
            vv[pass] = *reinterpret_cast<const u32x4*>(vsrc + static_cast<uint64_t>(r) * kGdnValueValues +
                                                       (tid & 15) * 8);
        }
#pragma unroll
        for (uint32_t pass = 0; pass < 4; ++pass) {
            *reinterpret_cast<u32x4*>(&ktile[pass * 16 + (tid >> 4)][(tid & 15) * 8]) = kv[pass];
            *reinterpret_cast<u32x4*>(&vtile[pass * 16 + (tid >> 4)][(tid & 15) * 8]) = vv[pass];
        }
    }

    if (tid < kChunk) {
        float dec = 1.0f;
        float b = 0.0f;
        if (tid < valid) {
            dec = a.decay[static_cast<uint64_t>(t0 + tid) * kGdnValueHeads + h];
            b = a.beta[static_cast<uint64_t>(t0 + tid) * kGdnValueHeads + h];
        }
        float lg = fmaxf(logf(dec), -87.0f);  // a zero decay acts as exp(-87)
        for (uint32_t off = 1; off < kChunk; off <<= 1) {
            const float up = __shfl_up(lg, off, 64);
            if (lane >= off) lg += up;
        }
        log_g[tid] = lg;
        scale_k[tid] = b * __expf(lg);
        scale_v[tid] = b;
        const float log_gc = __shfl(lg, kChunk - 1, 64);
        reinterpret_cast<float*>(rec + kRecRatio)[tid] = __expf(log_gc - lg);
        reinterpret_cast<float*>(rec + kRecGam)[tid] = __expf(lg);
        if (tid == kChunk - 1) *reinterpret_cast<float*>(rec + kRecGamma) = __expf(lg);
    }
    __syncthreads();

    {
        // wave w owns token rows 16w..16w+15 against all 64 columns
        bf16x8 ak[4];
#pragma unroll
        for (uint32_t kk = 0; kk < 4; ++kk) {
            ak[kk] = operand(&ktile[wave * 16 + m][kk * 32 + g * 8]);
            *reinterpret_cast<u32x4*>(rec + kRecQ + ((wave * 4 + kk) * 64 + lane) * 16) =
                __builtin_bit_cast(u32x4, aq[kk]);
        }
#pragma unroll
        for (uint32_t nt = 0; nt < 4; ++nt) {
            f32x4 kkacc = {0.0f, 0.0f, 0.0f, 0.0f};
            f32x4 qkacc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (uint32_t kk = 0; kk < 4; ++kk) {
                const bf16x8 bk = operand(&ktile[nt * 16 + m][kk * 32 + g * 8]);
                kkacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak[kk], bk, kkacc, 0, 0, 0);
                qkacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(aq[kk], bk, qkacc, 0, 0, 0);
            }
            const uint32_t s = nt * 16 + m;
            f32x4 aqk;
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                const uint32_t t = wave * 16 + g * 4 + i;
                const float ratio = s <= t ? __expf(log_g[t] - log_g[s]) : 0.0f;
                lower[t][s] = (s < t && t < valid) ? scale_v[t] * ratio * kkacc[i] : 0.0f;
                aqk[i] = (s <= t && t < valid) ? ratio * qkacc[i] : 0.0f;
            }
            // fragment (token tile `wave`, token step nt >> 1), column groups 2(nt&1), +1
            store_tile_hi_lo(reinterpret_cast<uint16_t (*)[16][24]>(&strip[wave][0][0][0]), aqk, lane, rec + kRecAqkHi, rec + kRecAqkLo,
                             ((wave * 2 + (nt >> 1)) * 64 + (nt & 1) * 32) * 16);
        }
    }
    __syncthreads();

    // diagonal blocks: thread (block b, column c) solves (I + L_bb) x = e_c
    if (tid < kChunk) {
        const uint32_t b = tid >> 4;
        const uint32_t c = tid & 15;
        float x[16];
#pragma unroll
        for (uint32_t r = 0; r < 16; ++r) {
            float acc = r == c ? 1.0f : 0.0f;
#pragma unroll
            for (uint32_t s = 0; s < r; ++s) acc = fmaf(-lower[b * 16 + r][b * 16 + s], x[s], acc);
            x[r] = acc;
        }
#pragma unroll
        for (uint32_t r = 0; r < 16; ++r) tdiag[b * 16 + r][c] = x[r];
    }
    __syncthreads();
    // [Wk | Wv] = (I + L)^-1 B with B = beta o [g o K | V], solved by block forward
    // substitution, every wave for its own 64 columns (waves 0,1 the keys, 2,3 the
    // values): W_i = T_ii (B_i - sum_{j<i} L_ij W_j) with the diagonal inverses T_ii.
    // All products on MFMA with hi/lo operand pairs; a finished block row goes, as
    // bf16 hi/lo, into the wave's strip in LDS, from where it is read back as the
    // right operand of the next products (rows contiguous: one 16-byte read per lane).
    uint16_t (*hi_strip)[kStripLd] = strip[wave][0];
    uint16_t (*lo_strip)[kStripLd] = strip[wave][1];
    // left operands, the same for every column: lane (row m, slot group g).  K = 16
    // products use slot groups 0 and 1 only; the other lanes hold zeros.
    const auto left = [&](const float* row8, bool live, bool negate, bf16x8& hi, bf16x8& lo) {
        float x[8];
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) x[e] = live ? (negate ? -row8[e] : row8[e]) : 0.0f;
        split8(x, hi, lo);
    };
    bf16x8 t_hi[4], t_lo[4];       // T_ii, K = 16
    bf16x8 l10_hi, l10_lo;         // -L_10, K = 16
    bf16x8 l2_hi, l2_lo;           // -L_2,[0 1], K = 32
    bf16x8 l3_hi, l3_lo;           // -L_3,[0 1], K = 32
    bf16x8 l32_hi, l32_lo;         // -L_32, K = 16
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) left(&tdiag[16 * i + m][(g & 1) * 8], g < 2, false, t_hi[i], t_lo[i]);
    left(&lower[16 + m][(g & 1) * 8], g < 2, true, l10_hi, l10_lo);
    left(&lower[32 + m][g * 8], true, true, l2_hi, l2_lo);
    left(&lower[48 + m][g * 8], true, true, l3_hi, l3_lo);
    left(&lower[48 + m][32 + (g & 1) * 8], g < 2, true, l32_hi, l32_lo);

    const auto product = [](const bf16x8 a_hi, const bf16x8 a_lo, const bf16x8 b_hi, const bf16x8 b_lo,
                            f32x4 acc) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, b_hi, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_lo, acc, 0, 0, 0);
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, b_hi, acc, 0, 0, 0);
    };
    // a 16x16 tile (this lane: rows 4g+i of column m) into strip rows row0 + 4g + i
    const auto put = [&](const f32x4 v, uint32_t row0) {
        u32x2 hi, lo;
        split4(v, hi, lo);
        *reinterpret_cast<u32x2*>(&hi_strip[m][row0 + g * 4]) = hi;
        *reinterpret_cast<u32x2*>(&lo_strip[m][row0 + g * 4]) = lo;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // right operand from strip rows row0 + 8g .. +7 of column m; with `narrow_k` only
    // slot groups 0 and 1 are live (K = 16)
    const auto get = [&](uint32_t row0, bool narrow_k, bf16x8& hi, bf16x8& lo) {
        const uint32_t row = row0 + (narrow_k ? (g & 1) : g) * 8;
        u32x4 h = *reinterpret_cast<const u32x4*>(&hi_strip[m][row]);
        u32x4 l = *reinterpret_cast<const u32x4*>(&lo_strip[m][row]);
        if (narrow_k && g >= 2) {
            h = u32x4{0u, 0u, 0u, 0u};
            l = u32x4{0u, 0u, 0u, 0u};
        }
        hi = __builtin_bit_cast(bf16x8, h);
        lo = __builtin_bit_cast(bf16x8, l);
    };
    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    // every wave holds its left operands: `lower` and `tdiag` are free from here on
    __syncthreads();

    // Block column `wave` of T = (I + L)^-1 by block forward substitution on the
    // identity: X_i = T_ii (E_i - sum_{j<i} L_ij X_j).  All products on MFMA with hi/lo
    // operand pairs; a finished block goes, as bf16 hi/lo, into the wave's strip in LDS,
    // from where it is read back as the right operand of the next products (rows
    // contiguous: one 16-byte read per lane).  The four waves run the four columns side
    // by side; the finished fp32 blocks overwrite `lower`.
    {
        f32x4 rhs[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) rhs[i][r] = (i == wave && g * 4 + r == m) ? 1.0f : 0.0f;
        }
        bf16x8 b_hi, b_lo;
        f32x4 w[4];
        put(rhs[0], 48);
        get(48, true, b_hi, b_lo);
        w[0] = product(t_hi[0], t_lo[0], b_hi, b_lo, zero);
        put(w[0], 0);
        get(0, true, b_hi, b_lo);
        f32x4 x = product(l10_hi, l10_lo, b_hi, b_lo, rhs[1]);
        put(x, 48);
        get(48, true, b_hi, b_lo);
        w[1] = product(t_hi[1], t_lo[1], b_hi, b_lo, zero);
        put(w[1], 16);
        bf16x8 w01_hi, w01_lo;
        get(0, false, w01_hi, w01_lo);
        x = product(l2_hi, l2_lo, w01_hi, w01_lo, rhs[2]);
        put(x, 48);
        get(48, true, b_hi, b_lo);
        w[2] = product(t_hi[2], t_lo[2], b_hi, b_lo, zero);
        put(w[2], 32);
        x = product(l3_hi, l3_lo, w01_hi, w01_lo, rhs[3]);
        get(32, true, b_hi, b_lo);
        x = product(l32_hi, l32_lo, b_hi, b_lo, x);
        put(x, 48);
        get(48, true, b_hi, b_lo);
        w[3] = product(t_hi[3], t_lo[3], b_hi, b_lo, zero);
#pragma unroll
        for (uint32_t mt = 0; mt < 4; ++mt) {
#pragma unroll
            for (uint32_t r = 0; r < 4; ++r) lower[16 * mt + 4 * g + r][16 * wave + m] = w[mt][r];
        }
    }
    __syncthreads();

    // [Wk | Wv] = T (beta o [g o K | V]) = (T o scale) [K | V]: the scales go into the
    // columns of T (fp32, then hi/lo), which leaves the exact bf16 keys and values as the
    // other operand - two products per step and no chain between them.  Every wave takes
    // its own 64 columns (waves 0,1 the keys, 2,3 the values).  Block (mt, ks) of T,
    // token rows 16 mt .., token columns 32 ks ..; T is lower triangular: ks <= mt / 2.
    const uint16_t (*source)[kTileLd] = is_k ? ktile : vtile;
    const float* scale = is_k ? scale_k : scale_v;
    bf16x8 ts_hi[4][2], ts_lo[4][2];
#pragma unroll
    for (uint32_t mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (uint32_t ks = 0; ks < 2; ++ks) {
            if (2 * ks > mt) continue;
            float x[8];
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) {
                x[e] = lower[16 * mt + m][32 * ks + 8 * g + e] * scale[32 * ks + 8 * g + e];
            }
            split8(x, ts_hi[mt][ks], ts_lo[mt][ks]);
        }
    }
    for (uint32_t ct = 0; ct < 4; ++ct) {
        const uint32_t col0 = (wave & 1) * 64 + ct * 16;
        // the exact rows, token-contiguous: lane = column col0 + m, tokens 32 ks + 8 g .. +7,
        // by transposing reads (16 lanes hand in 4 token rows x 16 columns, lane m
        // receives column m of the 4 rows)
        bf16x8 rows8[2];
#pragma unroll
        for (uint32_t ks = 0; ks < 2; ++ks) {
            const uint16_t* at = &source[ks * 32 + g * 8 + (m >> 2)][col0 + (m & 3) * 4];
            const s16x4 first = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(at));
            const s16x4 second = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(at + 4 * kTileLd));
            uint32_t bits[8];
#pragma unroll
            for (uint32_t e = 0; e < 4; ++e) {
                bits[e] = ks * 32 + g * 8 + e < valid ? static_cast<uint16_t>(first[e]) : 0u;
                bits[4 + e] = ks * 32 + g * 8 + 4 + e < valid ? static_cast<uint16_t>(second[e]) : 0u;
            }
            const u32x4 packed = u32x4{bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16),
                                       bits[4] | (bits[5] << 16), bits[6] | (bits[7] << 16)};
            rows8[ks] = __builtin_bit_cast(bf16x8, packed);
            if (is_k) {
                // fragment (key tile, token step ks) of the record
                *reinterpret_cast<u32x4*>(rec + kRecKt + (((col0 >> 4) * 2 + ks) * 64 + lane) * 16) = packed;
            }
        }
        f32x4 w[4];
#pragma unroll
        for (uint32_t mt = 0; mt < 4; ++mt) {
            f32x4 acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ts_lo[mt][0], rows8[0], zero, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ts_hi[mt][0], rows8[0], acc, 0, 0, 0);
            if (mt >= 2) {
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ts_lo[mt][1], rows8[1], acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ts_hi[mt][1], rows8[1], acc, 0, 0, 0);
            }
            w[mt] = acc;
        }
        // lane holds tokens 16mt+4g+i of column col0 + m
#pragma unroll
        for (uint32_t mt = 0; mt < 4; ++mt) {
            if (is_k) {
                // fragment (token tile mt, key step col0 >> 5), column groups (col0 & 31) >> 3, +1
                store_tile_hi_lo(reinterpret_cast<uint16_t (*)[16][24]>(&strip[wave][0][0][0]), w[mt],
                                 lane, rec + kRecWkHi, rec + kRecWkLo,
                                 ((mt * 4 + (col0 >> 5)) * 64 + ((col0 & 31) >> 3) * 16) * 16);
            } else {
                *reinterpret_cast<f32x4*>(rec + kRecWv +
                                          ((((col0 + m) >> 4) * 4 + mt) * 64 + g * 16 + m) * 16) = w[mt];
            }
        }
    }
}

struct ChunkScanArgs {
    const uint8_t* scratch;
    const float* state_in;
    float* state_out;
    uint16_t* y;             // [rows][4096]
    uint32_t rows;
};

// One chunk's operands of one wave, loaded a chunk ahead of their use.  The state
// waves carry the recurrence, the output waves everything that only leaves it.
template <uint32_t NT>
struct StateOperands {
    bf16x8 wk_hi[4], wk_lo[4], kt[2][2];
    f32x4 wv[NT];
    f32x4 ratio;
    float gamma_c;
};
struct OutputOperands {
    bf16x8 q[4], aq_hi[2], aq_lo[2];
    f32x4 gam;
};

__device__ __forceinline__ const uint8_t* chunk_record(const ChunkScanArgs& a, uint32_t chunk,
                                                       uint32_t h) {
    return a.scratch + (static_cast<uint64_t>(chunk) * kGdnValueHeads + h) * kRecBytes;
}
__device__ __forceinline__ u32x4 record_fragment(const uint8_t* rec, uint32_t base, uint32_t index,
                                                 uint32_t lane) {
    return *reinterpret_cast<const u32x4*>(rec + base + (index * 64 + lane) * 16);
}

template <uint32_t NT>
__device__ __forceinline__ StateOperands<NT> load_state_operands(const uint8_t* rec, uint32_t slice,
                                                                 uint32_t w, uint32_t lane) {
    StateOperands<NT> o;
    const uint32_t g = lane >> 4;
#pragma unroll
    for (uint32_t kk = 0; kk < 4; ++kk) {
        o.wk_hi[kk] = __builtin_bit_cast(bf16x8, record_fragment(rec, kRecWkHi, w * 4 + kk, lane));
        o.wk_lo[kk] = __builtin_bit_cast(bf16x8, record_fragment(rec, kRecWkLo, w * 4 + kk, lane));
    }
#pragma unroll
    for (uint32_t k2 = 0; k2 < 2; ++k2) {
#pragma unroll
        for (uint32_t mt = 0; mt < 2; ++mt) {
            o.kt[mt][k2] =
                __builtin_bit_cast(bf16x8, record_fragment(rec, kRecKt, (w * 2 + mt) * 2 + k2, lane));
        }
    }
#pragma unroll
    for (uint32_t nt = 0; nt < NT; ++nt) {
        o.wv[nt] = __builtin_bit_cast(f32x4, record_fragment(rec, kRecWv, (slice * NT + nt) * 4 + w, lane));
    }
    o.ratio = *reinterpret_cast<const f32x4*>(rec + kRecRatio + (w * 16 + g * 4) * 4);
    o.gamma_c = *reinterpret_cast<const float*>(rec + kRecGamma);
    return o;
}

__device__ __forceinline__ OutputOperands load_output_operands(const uint8_t* rec, uint32_t w,
                                                               uint32_t lane) {
    OutputOperands o;
    const uint32_t g = lane >> 4;
#pragma unroll
    for (uint32_t kk = 0; kk < 4; ++kk) {
        o.q[kk] = __builtin_bit_cast(bf16x8, record_fragment(rec, kRecQ, w * 4 + kk, lane));
    }
#pragma unroll
    for (uint32_t k2 = 0; k2 < 2; ++k2) {
        o.aq_hi[k2] = __builtin_bit_cast(bf16x8, record_fragment(rec, kRecAqkHi, w * 2 + k2, lane));
        o.aq_lo[k2] = __builtin_bit_cast(bf16x8, record_fragment(rec, kRecAqkLo, w * 2 + k2, lane));
    }
    o.gam = *reinterpret_cast<const f32x4*>(rec + kRecGam + (w * 16 + g * 4) * 4);
    return o;
}

// Stage 2.  grid (8, 32) x 512: a workgroup owns a 16-wide slice of the value
// dimension of one head and walks the chunks in order.  Waves 0..3 (state waves)
// carry the recurrence: wave w owns token rows 16w..16w+15 of U and key columns
// 32w..32w+31 of the state slice, whose fp32 master copy lives in its MFMA
// accumulators for the whole block.  Waves 4..7 (output waves) compute what only
// leaves the recurrence - Y = g o (Q S^T) + A U of token rows 16w..16w+15 - from the
// state and U copies in LDS, so that their loads, products and stores stay off the
// chain from one chunk's state to the next.  Two barriers per chunk order the two
// LDS copies between all eight waves.
template <uint32_t NT>
__global__ __launch_bounds__(512) void gdn_chunk_scan_kernel(ChunkScanArgs a) {
    constexpr uint32_t DV = 16 * NT;
    __shared__ __attribute__((aligned(16))) uint16_t s_hi[DV][136];  // bf16 S slice [dv][dk+pad]
    __shared__ __attribute__((aligned(16))) uint16_t s_lo[DV][136];  // S - s_hi
    __shared__ __attribute__((aligned(16))) uint16_t u_hi[DV][72];   // U^T [dv][token+pad]
    __shared__ __attribute__((aligned(16))) uint16_t u_lo[DV][72];
    __shared__ __attribute__((aligned(16))) uint16_t d_hi[DV][72];   // ((g_C/g) o U)^T
    __shared__ __attribute__((aligned(16))) uint16_t d_lo[DV][72];
    // Workgroups are dealt round-robin over the 8 XCDs, each with its own L2, in
    // linear order (x fastest): blockIdx.x names the XCD.  All slices of a head
    // read the same chunk records, so a head's slices stay on one XCD.
    constexpr uint32_t kSlicesPerHead = kGD / DV;
    const uint32_t local = blockIdx.y;
    const uint32_t slice = local % kSlicesPerHead;
    const uint32_t h = blockIdx.x * (kGdnValueHeads / 8) + local / kSlicesPerHead;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t w = wave & 3;
    const bool state_wave = wave < 4;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t chunks = (a.rows + kChunk - 1) / kChunk;
    const uint32_t at = w * 16 + g * 4;  // this lane's token rows of a chunk

    if (state_wave) {
        // State slice transposed, [dk tile][dv]: this lane holds key rows
        // 32w+16mt+4g+i of value column m, four consecutive keys of one state row.
        f32x4 sacc[2][NT];
#pragma unroll
        for (uint32_t mt = 0; mt < 2; ++mt) {
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
                const uint32_t j = nt * 16 + m;
                const uint32_t dk = w * 32 + mt * 16 + g * 4;
                const f32x4 v = *reinterpret_cast<const f32x4*>(
                    a.state_in + (static_cast<uint64_t>(h) * kGD + slice * DV + j) * kGD + dk);
                sacc[mt][nt] = v;
                u32x2 hi, lo;
                split4(v, hi, lo);
                *reinterpret_cast<u32x2*>(&s_hi[j][dk]) = hi;
                *reinterpret_cast<u32x2*>(&s_lo[j][dk]) = lo;
            }
        }
        const uint32_t last = chunks - 1;
        const auto fetch = [&](uint32_t chunk) {
            return load_state_operands<NT>(chunk_record(a, min(chunk, last), h), slice, w, lane);
        };
        // one chunk of the recurrence with the operands `cur`
        const auto step = [&](const StateOperands<NT>& cur) {
            // P1 = Wk S^T for token tile w: [16 x DV]
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
                f32x4 p1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (uint32_t kk = 0; kk < 4; ++kk) {
                    const bf16x8 sh = operand(&s_hi[nt * 16 + m][kk * 32 + g * 8]);
                    const bf16x8 sl = operand(&s_lo[nt * 16 + m][kk * 32 + g * 8]);
                    p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.wk_lo[kk], sh, p1, 0, 0, 0);
                    p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.wk_hi[kk], sl, p1, 0, 0, 0);
                    p1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.wk_hi[kk], sh, p1, 0, 0, 0);
                }
                // U = Wv - P1; this lane holds tokens 16w+4g+i of value column 16nt+m
                const f32x4 u = cur.wv[nt] - p1;
                const f32x4 d = u * cur.ratio;
                u32x2 uh, ul, dh, dl;
                split4(u, uh, ul);
                split4(d, dh, dl);
                *reinterpret_cast<u32x2*>(&u_hi[nt * 16 + m][at]) = uh;
                *reinterpret_cast<u32x2*>(&u_lo[nt * 16 + m][at]) = ul;
                *reinterpret_cast<u32x2*>(&d_hi[nt * 16 + m][at]) = dh;
                *reinterpret_cast<u32x2*>(&d_lo[nt * 16 + m][at]) = dl;
            }
            __syncthreads();  // U^T complete; every read of the old state copy is done
            // S^T = g_C S^T + K^T ((g_C/g) o U) for key rows 32w..32w+31
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
                bf16x8 dlo[2], dhi[2];
#pragma unroll
                for (uint32_t k2 = 0; k2 < 2; ++k2) {
                    dlo[k2] = operand(&d_lo[nt * 16 + m][k2 * 32 + g * 8]);
                    dhi[k2] = operand(&d_hi[nt * 16 + m][k2 * 32 + g * 8]);
                }
#pragma unroll
                for (uint32_t mt = 0; mt < 2; ++mt) {
                    sacc[mt][nt] *= cur.gamma_c;
#pragma unroll
                    for (uint32_t k2 = 0; k2 < 2; ++k2) {
                        sacc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.kt[mt][k2], dlo[k2],
                                                                               sacc[mt][nt], 0, 0, 0);
                        sacc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.kt[mt][k2], dhi[k2],
                                                                               sacc[mt][nt], 0, 0, 0);
                    }
                    u32x2 hi, lo;
                    split4(sacc[mt][nt], hi, lo);
                    const uint32_t dk = w * 32 + mt * 16 + g * 4;
                    *reinterpret_cast<u32x2*>(&s_hi[nt * 16 + m][dk]) = hi;
                    *reinterpret_cast<u32x2*>(&s_lo[nt * 16 + m][dk]) = lo;
                }
            }
            __syncthreads();  // new state copy visible; U^T free for the next chunk
        };
        // Operands are requested two chunks ahead of their use, in three register sets
        // that take turns (no copies: a copy would wait for the newest request).
        StateOperands<NT> set_a = fetch(0);
        StateOperands<NT> set_b = fetch(1);
        __syncthreads();
        for (uint32_t chunk = 0; chunk < chunks; chunk += 3) {
            const StateOperands<NT> set_c = fetch(chunk + 2);
            step(set_a);
            if (chunk + 1 < chunks) {
                set_a = fetch(chunk + 3);
                step(set_b);
            }
            if (chunk + 2 < chunks) {
                set_b = fetch(chunk + 4);
                step(set_c);
            }
        }
#pragma unroll
        for (uint32_t mt = 0; mt < 2; ++mt) {
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
                const uint32_t dk = w * 32 + mt * 16 + g * 4;
                *reinterpret_cast<f32x4*>(a.state_out + (static_cast<uint64_t>(h) * kGD + slice * DV +
                                                         nt * 16 + m) * kGD + dk) = sacc[mt][nt];
            }
        }
    } else {
        const uint32_t last = chunks - 1;
        const auto fetch = [&](uint32_t chunk) {
            return load_output_operands(chunk_record(a, min(chunk, last), h), w, lane);
        };
        const auto step = [&](const OutputOperands& cur, uint32_t chunk) {
            // P2 = Q S^T for token tile w against the state the chunk starts from
            f32x4 y[NT];
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
                f32x4 p2 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (uint32_t kk = 0; kk < 4; ++kk) {
                    const bf16x8 sh = operand(&s_hi[nt * 16 + m][kk * 32 + g * 8]);
                    const bf16x8 sl = operand(&s_lo[nt * 16 + m][kk * 32 + g * 8]);
                    p2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.q[kk], sl, p2, 0, 0, 0);
                    p2 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.q[kk], sh, p2, 0, 0, 0);
                }
                y[nt] = p2 * cur.gam;
            }
            __syncthreads();  // U^T complete; this wave is done with the old state copy
            // Y = g o (Q S^T) + A U
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (uint32_t k2 = 0; k2 < 2; ++k2) {
                    const bf16x8 bh = operand(&u_hi[nt * 16 + m][k2 * 32 + g * 8]);
                    const bf16x8 bl = operand(&u_lo[nt * 16 + m][k2 * 32 + g * 8]);
                    y[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.aq_lo[k2], bh, y[nt], 0, 0, 0);
                    y[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.aq_hi[k2], bl, y[nt], 0, 0, 0);
                    y[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.aq_hi[k2], bh, y[nt], 0, 0, 0);
                }
            }
            __syncthreads();  // this wave is done with U^T
#pragma unroll
            for (uint32_t nt = 0; nt < NT; ++nt) {
#pragma unroll
                for (uint32_t i = 0; i < 4; ++i) {
                    const uint32_t token = chunk * kChunk + at + i;
                    if (token < a.rows) {
                        a.y[static_cast<uint64_t>(token) * kGdnValueValues + h * kGD + slice * DV +
                            nt * 16 + m] = narrow(y[nt][i]);
                    }
                }
            }
        };
        OutputOperands set_a = fetch(0);
        OutputOperands set_b = fetch(1);
        __syncthreads();
        for (uint32_t chunk = 0; chunk < chunks; chunk += 3) {
            const OutputOperands set_c = fetch(chunk + 2);
            step(set_a, chunk);
            if (chunk + 1 < chunks) {
                set_a = fetch(chunk + 3);
                step(set_b, chunk + 1);
            }
            if (chunk + 2 < chunks) {
                set_b = fetch(chunk + 4);
                step(set_c, chunk + 2);
            }
        }
    }
}

// value tiles of 16 per scan workgroup: 1 -> 256 workgroups (0.47 ms for 16384 rows),
// 2 -> 128 workgroups with half the L2 traffic (0.57 ms: the chunk chain gets longer)
constexpr uint32_t kScanTiles = 1;

// ---------------------------------------------------------------- launchers --

int32_t launch_prepare(const PrepareArgs& p, hipStream_t stream) {
    if (p.block_mode) {
        hipLaunchKernelGGL(gdn_prepare_block_kernel,
                           dim3((kCh + kGdnValueValues) / 8 / 256,
                                (p.rows + kBlockRowsPerGroup - 1) / kBlockRowsPerGroup),
                           dim3(256), 0, stream, p);
        return TT_OK;
    }
    hipLaunchKernelGGL(gdn_prepare_kernel, dim3(96, p.rows), dim3(128), 0, stream, p);
    return TT_OK;
}

// gdn_prepare: b0 projection, b1 conv_in, b2 conv_w, b3 qk, b4 value, b5 z,
// b6 conv_out; grid 96 x 128 (decode_step.cpp:666-674).
int32_t op_gdn_prepare(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    PrepareArgs p{};
    p.projection = a.buffer<const uint16_t>(0, kGdnProjectionRows * 2);
    p.conv_in = a.buffer<const uint16_t>(1, 3 * kCh * 2);
    p.conv_weights = a.buffer<const uint16_t>(2, 4 * kCh * 2);
    p.qk = a.buffer<uint16_t>(3, kGdnQkValues * 2);
    p.value = a.buffer<uint16_t>(4, kGdnValueValues * 2);
    p.z = a.buffer<uint16_t>(5, kGdnValueValues * 2);
    p.conv_out = a.buffer<uint16_t>(6, 3 * kCh * 2);
    p.projection_stride = kGdnProjectionRows;
    p.qk_stride = kGdnQkValues;
    p.value_stride = p.z_stride = kGdnValueValues;
    p.rows = 1;
    a.require(grid_is(g, 96, 1, 1, 128, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_prepare(p, stream);
}

// gdn_prepare_ms: b0 projection slab, b1 conv_pool, b2 conv_w, b3 qk slab,
// b4 value slab, b5 z slab, b6 state_table, c7..c10 strides;
// grid (96, rows) x 128 (decode_step.cpp:1136-1148).
int32_t op_gdn_prepare_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                          bool validate_only) {
    Args a(b);
    PrepareArgs p{};
    p.projection_stride = a.constant(7);
    p.qk_stride = a.constant(8);
    p.value_stride = a.constant(9);
    p.z_stride = a.constant(10);
    p.rows = static_cast<uint32_t>(g.gy);
    a.require(g.gx == 96 && g.gz == 1 && g.tx == 128 && g.ty == 1 && g.tz == 1 && p.rows >= 1 &&
                  p.rows <= kMaxBatchRows,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(p.projection_stride >= kGdnProjectionRows && p.qk_stride >= kGdnQkValues &&
                  p.value_stride >= kGdnValueValues && p.z_stride >= kGdnValueValues,
              TT_CMD_INVALID_BUFFER);
    const uint64_t last = p.rows - 1;
    p.projection =
        a.buffer<const uint16_t>(0, (last * p.projection_stride + kGdnProjectionRows) * 2);
    uint16_t* pool = a.buffer<uint16_t>(1, 2 * 3 * kCh * 2);
    p.conv_in = pool;
    p.conv_out = pool;
    p.conv_weights = a.buffer<const uint16_t>(2, 4 * kCh * 2);
    p.qk = a.buffer<uint16_t>(3, (last * p.qk_stride + kGdnQkValues) * 2);
    p.value = a.buffer<uint16_t>(4, (last * p.value_stride + kGdnValueValues) * 2);
    p.z = a.buffer<uint16_t>(5, (last * p.z_stride + kGdnValueValues) * 2);
    p.table = a.buffer<const uint32_t>(6, p.rows * 16);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_prepare(p, stream);
}

// gdn_conv_blk: b0 projection[rows][12352], b1 conv_in, b2 conv_w, b3 qk[rows][4096],
// b4 value, b5 gate, b6 conv_out, c7 rows; grid (96, rows) x 128
// (prefill_step.cpp:1934-1955).
int32_t conv_blk_common(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                        bool taped) {
    Args a(b);
    PrepareArgs p{};
    p.rows = a.constant(7);
    if (taped) {
        p.conv_tape = a.buffer<uint16_t>(8, static_cast<uint64_t>(kGdnConvTapeElements) * 2);
        p.tape_layer = a.constant(9);
        a.require(p.tape_layer < kLayers, TT_CMD_INVALID_BUFFER);
    }
    a.require(p.rows >= 1 && g.gx == 96 && g.gy == p.rows && g.gz == 1 && g.tx == 128 &&
                  g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t rows = p.rows;
    p.projection = a.buffer<const uint16_t>(0, rows * kGdnProjectionRows * 2);
    p.conv_in = a.buffer<const uint16_t>(1, 3 * kCh * 2);
    p.conv_weights = a.buffer<const uint16_t>(2, 4 * kCh * 2);
    p.qk = a.buffer<uint16_t>(3, rows * kGdnQkValues * 2);
    p.value = a.buffer<uint16_t>(4, rows * kGdnValueValues * 2);
    p.z = a.buffer<uint16_t>(5, rows * kGdnValueValues * 2);
    p.conv_out = a.buffer<uint16_t>(6, 3 * kCh * 2);
    p.projection_stride = kGdnProjectionRows;
    p.qk_stride = kGdnQkValues;
    p.value_stride = p.z_stride = kGdnValueValues;
    p.block_mode = 1;
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_prepare(p, stream);
}
int32_t op_gdn_conv_blk(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    return conv_blk_common(b, g, stream, validate_only, false);
}
// gdn_conv_tape_blk: gdn_conv_blk + b8 conv tape [40][16][3][8192] bf16, c9 layer; a
// block of more than 16 rows leaves the tape untouched (prefill_step.cpp:1931-1947).
int32_t op_gdn_conv_tape_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                             bool validate_only) {
    return conv_blk_common(b, g, stream, validate_only, true);
}

int32_t launch_recurrence(const RecurrenceArgs& r, uint32_t rows, hipStream_t stream) {
    if (r.tape != nullptr) {
        hipLaunchKernelGGL(gdn_recurrence_kernel<true>, dim3(kGD / 8, kGdnValueHeads, rows),
                           dim3(256), 0, stream, r);
        return TT_OK;
    }
    hipLaunchKernelGGL(gdn_recurrence_kernel<false>, dim3(kGD / 8, kGdnValueHeads, rows), dim3(256),
                       0, stream, r);
    return TT_OK;
}

constexpr uint64_t kStateBytes = static_cast<uint64_t>(kGdnStateFloats) * 4;

// gdn_recurrence: b0 qk, b1 value, b2 projection, b3 a_log, b4 dt_bias,
// b5 state_in, b6 y, b7 state_out; grid (1,32,32) x (32,4,1)
// (decode_step.cpp:676-690).
int32_t op_gdn_recurrence(const Bindings& b, const Grid& g, hipStream_t stream,
                          bool validate_only) {
    Args a(b);
    RecurrenceArgs r{};
    r.qk = a.buffer<const uint16_t>(0, kGdnQkValues * 2);
    r.value = a.buffer<const uint16_t>(1, kGdnValueValues * 2);
    r.projection = a.buffer<const uint16_t>(2, kGdnProjectionRows * 2);
    r.a_log = a.buffer<const uint16_t>(3, kGdnValueHeads * 2);
    r.dt_bias = a.buffer<const uint16_t>(4, kGdnValueHeads * 2);
    r.state_in = a.buffer<const float>(5, kStateBytes);
    r.y = a.buffer<uint16_t>(6, kGdnValueValues * 2);
    r.state_out = a.buffer<float>(7, kStateBytes);
    r.qk_stride = kGdnQkValues;
    r.value_stride = r.y_stride = kGdnValueValues;
    r.projection_stride = kGdnProjectionRows;
    r.steps = 1;
    a.require(grid_is(g, 1, 32, 32, 32, 4, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_recurrence(r, 1, stream);
}

// gdn_recurrence_ms: b0 qk, b1 value, b2 projection, b3 a_log, b4 dt_bias,
// b5 rec_pool, b6 y slab, b7 state_table, c8 qk stride, c9 value stride,
// c10 projection stride, c11 output stride, c12 value_heads;
// grid (1,32,32*rows) x (32,4,1) (decode_step.cpp:1154-1173).
int32_t op_gdn_recurrence_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                             bool validate_only) {
    Args a(b);
    RecurrenceArgs r{};
    r.qk_stride = a.constant(8);
    r.value_stride = a.constant(9);
    r.projection_stride = a.constant(10);
    r.y_stride = a.constant(11);
    const uint32_t heads = a.constant(12);
    a.require(heads == kGdnValueHeads && g.gx == 1 && g.gy == 32 && g.gz % 32 == 0 &&
                  g.gz / 32 >= 1 && g.gz / 32 <= kMaxBatchRows && g.tx == 32 && g.ty == 4 &&
                  g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint32_t rows = static_cast<uint32_t>(g.gz / 32);
    a.require(r.qk_stride >= kGdnQkValues && r.value_stride >= kGdnValueValues &&
                  r.projection_stride >= kGdnProjectionRows && r.y_stride >= kGdnValueValues,
              TT_CMD_INVALID_BUFFER);
    const uint64_t last = rows ? rows - 1 : 0;
    r.qk = a.buffer<const uint16_t>(0, (last * r.qk_stride + kGdnQkValues) * 2);
    r.value = a.buffer<const uint16_t>(1, (last * r.value_stride + kGdnValueValues) * 2);
    r.projection =
        a.buffer<const uint16_t>(2, (last * r.projection_stride + kGdnProjectionRows) * 2);
    r.a_log = a.buffer<const uint16_t>(3, kGdnValueHeads * 2);
    r.dt_bias = a.buffer<const uint16_t>(4, kGdnValueHeads * 2);
    float* pool = a.buffer<float>(5, 2 * kStateBytes);
    r.state_in = pool;
    r.state_out = pool;
    r.y = a.buffer<uint16_t>(6, (last * r.y_stride + kGdnValueValues) * 2);
    r.table = a.buffer<const uint32_t>(7, rows * 16);
    r.steps = 1;
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_recurrence(r, rows, stream);
}

// gdn_decode_fused_ms (no reference counterpart: gdn_prepare_ms + gdn_recurrence_ms
// + gdn_gate_norm_ms of decode_step.cpp:1116-1211 in one dispatch): b0 projection
// slab, b1 conv pool, b2 conv weights, b3 a_log, b4 dt_bias, b5 recurrent pool,
// b6 norm weight, b7 gated output slab, b8 state table, c9 projection stride,
// c10 output stride; grid (32, rows) x 512.
int32_t op_gdn_decode_fused_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                               bool validate_only) {
    Args a(b);
    FusedDecodeArgs f{};
    f.projection_stride = a.constant(9);
    f.out_stride = a.constant(10);
    a.require(g.gx == kGdnValueHeads && g.gy >= 1 && g.gy <= kMaxBatchRows && g.gz == 1 &&
                  g.tx == 512 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(f.projection_stride >= kGdnProjectionRows && f.out_stride >= kGdnValueValues,
              TT_CMD_INVALID_BUFFER);
    if (a.status != TT_OK) return a.status;
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    const uint64_t last = rows - 1;
    f.projection =
        a.buffer<const uint16_t>(0, (last * f.projection_stride + kGdnProjectionRows) * 2);
    uint16_t* conv = a.buffer<uint16_t>(1, 2ull * 3 * kCh * 2);
    f.conv_pool = conv;
    f.conv_pool_out = conv;
    f.conv_weights = a.buffer<const uint16_t>(2, 4ull * kCh * 2);
    f.a_log = a.buffer<const uint16_t>(3, kGdnValueHeads * 2);
    f.dt_bias = a.buffer<const uint16_t>(4, kGdnValueHeads * 2);
    float* rec = a.buffer<float>(5, 2 * kStateBytes);
    f.rec_pool = rec;
    f.rec_pool_out = rec;
    f.norm_weight = a.buffer<const uint16_t>(6, kGD * 2);
    f.out = a.buffer<uint16_t>(7, (last * f.out_stride + kGdnValueValues) * 2);
    f.table = a.buffer<const uint32_t>(8, rows * 16);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gdn_decode_fused_kernel<kFusedThreads>, dim3(kGdnValueHeads, rows), dim3(kFusedThreads), 0, stream, f);
    return TT_OK;
}

// gdn_gates_blk: b0 projection, b1 a_log, b2 dt_bias, b3 decay[rows][32],
// b4 beta[rows][32], c5 rows; grid (1, ceil(rows/4)) x (32, 4)
// (prefill_step.cpp:1989-2001).
int32_t op_gdn_gates_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                         bool validate_only) {
    Args a(b);
    const uint32_t rows = a.constant(5);
    a.require(rows >= 1 && g.gx == 1 && g.gy == (rows + 3) / 4 && g.gz == 1 && g.tx == 32 &&
                  g.ty == 4 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint16_t* projection =
        a.buffer<const uint16_t>(0, static_cast<uint64_t>(rows) * kGdnProjectionRows * 2);
    const uint16_t* a_log = a.buffer<const uint16_t>(1, kGdnValueHeads * 2);
    const uint16_t* dt_bias = a.buffer<const uint16_t>(2, kGdnValueHeads * 2);
    float* decay = a.buffer<float>(3, static_cast<uint64_t>(rows) * kGdnValueHeads * 4);
    float* beta = a.buffer<float>(4, static_cast<uint64_t>(rows) * kGdnValueHeads * 4);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gdn_gates_kernel, dim3((rows + 3) / 4), dim3(32, 4), 0, stream, projection,
                       a_log, dt_bias, decay, beta, rows);
    return TT_OK;
}

// gdn_recurrence_gates_blk: b0 qk[rows][4096], b1 value, b2 decay, b3 a_log
// (unused), b4 beta, b5 state_in, b6 y[rows][4096], b7 state_out, c8 steps;
// gdn_recurrence_blk: b2 projection, b3 a_log, b4 dt_bias instead.
// grid (1,32,32) x (32,4,1) (prefill_step.cpp:2003-2036).
int32_t op_gdn_scan(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                    bool hoisted_gates, bool taped = false) {
    Args a(b);
    RecurrenceArgs r{};
    r.steps = a.constant(8);
    if (taped) {
        r.tape = a.buffer<float>(9, static_cast<uint64_t>(kGdnTapeFloats) * 4);
        r.tape_layer = a.constant(10);
        a.require(r.tape_layer < kLayers, TT_CMD_INVALID_BUFFER);
    }
    a.require(r.steps >= 1, TT_CMD_INVALID_BUFFER);
    const uint64_t steps = r.steps;
    r.qk = a.buffer<const uint16_t>(0, steps * kGdnQkValues * 2);
    r.value = a.buffer<const uint16_t>(1, steps * kGdnValueValues * 2);
    if (hoisted_gates) {
        r.decay = a.buffer<const float>(2, steps * kGdnValueHeads * 4);
        r.beta = a.buffer<const float>(4, steps * kGdnValueHeads * 4);
    } else {
        r.projection = a.buffer<const uint16_t>(2, steps * kGdnProjectionRows * 2);
        r.a_log = a.buffer<const uint16_t>(3, kGdnValueHeads * 2);
        r.dt_bias = a.buffer<const uint16_t>(4, kGdnValueHeads * 2);
    }
    r.state_in = a.buffer<const float>(5, kStateBytes);
    r.y = a.buffer<uint16_t>(6, steps * kGdnValueValues * 2);
    r.state_out = a.buffer<float>(7, kStateBytes);
    r.qk_stride = kGdnQkValues;
    r.value_stride = r.y_stride = kGdnValueValues;
    r.projection_stride = kGdnProjectionRows;
    a.require(grid_is(g, 1, 32, 32, 32, 4, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_recurrence(r, 1, stream);
}
int32_t op_gdn_recurrence_gates_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                                    bool validate_only) {
    return op_gdn_scan(b, g, stream, validate_only, true);
}
int32_t op_gdn_recurrence_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                              bool validate_only) {
    return op_gdn_scan(b, g, stream, validate_only, false);
}
// gdn_recurrence_gates_tape_blk: gdn_recurrence_gates_blk + b9 tape (fp32, three
// regions), c10 layer; more than 16 steps leave the tape untouched
// (prefill_step.cpp:2003-2028).
int32_t op_gdn_recurrence_gates_tape_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                                         bool validate_only) {
    return op_gdn_scan(b, g, stream, validate_only, true, true);
}
// gdn_tape_replay_blk: b0 tape, b1 state_in, b2 state_out, c3 steps (0..16), c4 layer;
// grid (1,32,32) x (32,4,1) (speculative_decode.cpp:546-556).
int32_t op_gdn_tape_replay_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                               bool validate_only) {
    Args a(b);
    const float* tape = a.buffer<const float>(0, static_cast<uint64_t>(kGdnTapeFloats) * 4);
    const float* state_in = a.buffer<const float>(1, kStateBytes);
    float* state_out = a.buffer<float>(2, kStateBytes);
    const uint32_t steps = a.constant(3);
    const uint32_t layer = a.constant(4);
    a.require(steps <= kGdnTapeRows && layer < kLayers, TT_CMD_INVALID_BUFFER);
    a.require(grid_is(g, 1, 32, 32, 32, 4, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gdn_tape_replay_kernel, dim3(kGD / 8, kGdnValueHeads), dim3(256), 0, stream,
                       tape, state_in, state_out, steps, layer);
    return TT_OK;
}

int32_t gate_norm_common(Args& a, const Grid& g, uint32_t rows, uint32_t stride,
                         hipStream_t stream, bool validate_only) {
    const uint64_t bytes = (static_cast<uint64_t>(rows - 1) * stride + kGdnValueValues) * 2;
    const uint16_t* y = a.buffer<const uint16_t>(0, bytes);
    const uint16_t* z = a.buffer<const uint16_t>(1, bytes);
    const uint16_t* w = a.buffer<const uint16_t>(2, kGD * 2);
    uint16_t* out = a.buffer<uint16_t>(3, bytes);
    a.require(g.gx == 32 && g.gy == rows && g.gz == 1 && g.tx == 128 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    if (rows > kMaxBatchRows && stride % 8 == 0) {  // blocks: 8 channels per lane, 8 rows per group
        hipLaunchKernelGGL(gdn_gate_norm_block_kernel, dim3(kGdnValueValues / 8 / 256, (rows + 7) / 8),
                           dim3(256), 0, stream, y, z, w, out, stride, rows, 8u);
        return TT_OK;
    }
    hipLaunchKernelGGL(gdn_gate_norm_kernel, dim3(32, rows), dim3(128), 0, stream, y, z, w, out,
                       stride, rows, 1u);
    return TT_OK;
}

// gdn_gate_norm: b0 y, b1 z, b2 norm_w, b3 gated; grid 32 x 128 (decode_step.cpp:692-697)
int32_t op_gdn_gate_norm(const Bindings& b, const Grid& g, hipStream_t stream,
                         bool validate_only) {
    Args a(b);
    return gate_norm_common(a, g, 1, kGdnValueValues, stream, validate_only);
}
// gdn_gate_norm_ms: + c4 value stride; grid (32, rows) x 128 (decode_step.cpp:1184-1190)
int32_t op_gdn_gate_norm_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only) {
    Args a(b);
    const uint32_t stride = a.constant(4);
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    a.require(stride >= kGdnValueValues && rows >= 1 && rows <= kMaxBatchRows,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    return gate_norm_common(a, g, rows, stride, stream, validate_only);
}
// gdn_gate_norm_blk: rows from the grid; grid (32, rows) x 128 (prefill_step.cpp:2040-2050)
int32_t op_gdn_gate_norm_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                             bool validate_only) {
    Args a(b);
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    a.require(rows >= 1 && g.gy <= 0x7fffffffull / kGdnValueValues,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    return gate_norm_common(a, g, rows, kGdnValueValues, stream, validate_only);
}


uint64_t chunk_scratch_bytes(uint32_t rows) {
    const uint64_t chunks = (static_cast<uint64_t>(rows) + kChunk - 1) / kChunk;
    return chunks * kGdnValueHeads * kRecBytes;
}

// gdn_chunk_prepare_blk (no reference counterpart: stage 1 of the chunked
// evaluation of gdn_recurrence_gates_blk): b0 qk[rows][4096], b1 value[rows][4096],
// b2 decay[rows][32], b3 beta[rows][32], b4 scratch (ceil(rows/64)*32 records of
// 115712 B), c5 rows; grid (ceil(rows/64), 32) x 256.
int32_t op_gdn_chunk_prepare(const Bindings& b, const Grid& g, hipStream_t stream,
                             bool validate_only) {
    Args a(b);
    ChunkPrepareArgs p{};
    p.rows = a.constant(5);
    a.require(p.rows >= 1 && p.rows <= (1u << 22), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t chunks = (p.rows + kChunk - 1) / kChunk;
    a.require(g.gx == chunks && g.gy == 32 && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t rows = p.rows;
    p.qk = a.buffer<const uint16_t>(0, rows * kGdnQkValues * 2);
    p.value = a.buffer<const uint16_t>(1, rows * kGdnValueValues * 2);
    p.decay = a.buffer<const float>(2, rows * kGdnValueHeads * 4);
    p.beta = a.buffer<const float>(3, rows * kGdnValueHeads * 4);
    p.scratch = a.buffer<uint8_t>(4, chunk_scratch_bytes(p.rows));
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gdn_chunk_prepare_kernel, dim3(chunks, kGdnValueHeads), dim3(256), 0, stream,
                       p);
    return TT_OK;
}

// gdn_chunk_scan_blk (stage 2): b0 scratch, b1 state_in, b2 y[rows][4096],
// b3 state_out, c4 rows; grid (8, 32) x 256.  state_in and state_out may be the
// same plane.
int32_t op_gdn_chunk_scan(const Bindings& b, const Grid& g, hipStream_t stream,
                          bool validate_only) {
    Args a(b);
    ChunkScanArgs p{};
    p.rows = a.constant(4);
    a.require(p.rows >= 1 && p.rows <= (1u << 22), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    a.require(grid_is(g, 8, 32, 1, 256, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    p.scratch = a.buffer<const uint8_t>(0, chunk_scratch_bytes(p.rows));
    p.state_in = a.buffer<const float>(1, kGdnStateFloats * 4ull);
    p.y = a.buffer<uint16_t>(2, static_cast<uint64_t>(p.rows) * kGdnValueValues * 2);
    p.state_out = a.buffer<float>(3, kGdnStateFloats * 4ull);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(gdn_chunk_scan_kernel<kScanTiles>, dim3(8, kGdnValueHeads / kScanTiles), dim3(512), 0, stream, p);
    return TT_OK;
}

// Rows one prepare + scan pair of gdn_chunk_recurrence_blk covers: the chunk records
// of a group (118 MB) stay in the 256 MB last-level cache between the two stages.
constexpr uint32_t kChunkGroupRows = 2048;

// gdn_chunk_recurrence_blk (no reference counterpart: the chunked evaluation of
// gdn_recurrence_gates_blk, prefill_step.cpp:1988-2040, in one dispatch): b0 qk
// [rows][4096], b1 value [rows][4096], b2 decay [rows][32], b3 beta [rows][32],
// b4 scratch (chunk records of min(rows, 2048) rows), b5 state_in, b6 y [rows][4096],
// b7 state_out, c8 rows; grid (8, 32) x 256.  Walks the block in groups of 2048
// rows, stage 1 then stage 2 per group; state_in and state_out may be the same plane.
int32_t op_gdn_chunk_recurrence(const Bindings& b, const Grid& g, hipStream_t stream,
                                bool validate_only) {
    Args a(b);
    const uint32_t rows = a.constant(8);
    a.require(rows >= 1 && rows <= (1u << 22), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    a.require(grid_is(g, 8, 32, 1, 256, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t row_bytes = static_cast<uint64_t>(rows) * kGdnValueValues * 2;
    const uint16_t* qk = a.buffer<const uint16_t>(0, row_bytes);
    const uint16_t* value = a.buffer<const uint16_t>(1, row_bytes);
    const float* decay = a.buffer<const float>(2, static_cast<uint64_t>(rows) * kGdnValueHeads * 4);
    const float* beta = a.buffer<const float>(3, static_cast<uint64_t>(rows) * kGdnValueHeads * 4);
    uint8_t* scratch = a.buffer<uint8_t>(4, chunk_scratch_bytes(min(rows, kChunkGroupRows)));
    const float* state_in = a.buffer<const float>(5, kGdnStateFloats * 4ull);
    uint16_t* y = a.buffer<uint16_t>(6, row_bytes);
    float* state_out = a.buffer<float>(7, kGdnStateFloats * 4ull);
    if (a.status != TT_OK || validate_only) return a.status;
    for (uint32_t start = 0; start < rows; start += kChunkGroupRows) {
        const uint32_t count = min(kChunkGroupRows, rows - start);
        ChunkPrepareArgs p{};
        p.qk = qk + static_cast<uint64_t>(start) * kGdnQkValues;
        p.value = value + static_cast<uint64_t>(start) * kGdnValueValues;
        p.decay = decay + static_cast<uint64_t>(start) * kGdnValueHeads;
        p.beta = beta + static_cast<uint64_t>(start) * kGdnValueHeads;
        p.scratch = scratch;
        p.rows = count;
        hipLaunchKernelGGL(gdn_chunk_prepare_kernel, dim3((count + kChunk - 1) / kChunk, kGdnValueHeads),
                           dim3(256), 0, stream, p);
        ChunkScanArgs c{};
        c.scratch = scratch;
        c.state_in = start == 0 ? state_in : state_out;
        c.state_out = state_out;
        c.y = y + static_cast<uint64_t>(start) * kGdnValueValues;
        c.rows = count;
        hipLaunchKernelGGL(gdn_chunk_scan_kernel<kScanTiles>, dim3(8, kGdnValueHeads / kScanTiles), dim3(512), 0, stream, c);
    }
    return TT_OK;
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side tables of launchers
const KernelDesc kGdnDecodeKernels[] = {
    {"gdn_prepare", op_gdn_prepare},
    {"gdn_prepare_ms", op_gdn_prepare_ms},
    {"gdn_recurrence", op_gdn_recurrence},
    {"gdn_recurrence_ms", op_gdn_recurrence_ms},
    {"gdn_gate_norm", op_gdn_gate_norm},
    {"gdn_gate_norm_ms", op_gdn_gate_norm_ms},
    {"gdn_decode_fused_ms", op_gdn_decode_fused_ms},
};
const uint32_t kGdnDecodeKernelCount = sizeof(kGdnDecodeKernels) / sizeof(kGdnDecodeKernels[0]);

const KernelDesc kGdnPrefillKernels[] = {
    {"gdn_conv_blk", op_gdn_conv_blk},
    {"gdn_gates_blk", op_gdn_gates_blk},
    {"gdn_recurrence_gates_blk", op_gdn_recurrence_gates_blk},
    {"gdn_recurrence_blk", op_gdn_recurrence_blk},
    {"gdn_gate_norm_blk", op_gdn_gate_norm_blk},
    {"gdn_conv_tape_blk", op_gdn_conv_tape_blk},
    {"gdn_recurrence_gates_tape_blk", op_gdn_recurrence_gates_tape_blk},
    {"gdn_tape_replay_blk", op_gdn_tape_replay_blk},
    {"gdn_chunk_prepare_blk", op_gdn_chunk_prepare},
    {"gdn_chunk_scan_blk", op_gdn_chunk_scan},
    {"gdn_chunk_recurrence_blk", op_gdn_chunk_recurrence},
};
const uint32_t kGdnPrefillKernelCount = sizeof(kGdnPrefillKernels) / sizeof(kGdnPrefillKernels[0]);

#endif

}  // namespace tt
