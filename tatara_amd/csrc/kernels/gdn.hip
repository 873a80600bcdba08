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
//
// State row layout: S[h][j][0..127] with the key index contiguous; one half
// wave (32 lanes x 4 floats = 512 B) owns one row, so a wave64 load
// instruction moves two rows = 1 KiB contiguous.  The 32-lane sums are xor
// butterflies (1,2,4,8,16), which is the adjacent-pairs tree of the reference
// bit for bit.
#include "../tt_internal.h"

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(4))) float f32x4;
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
// one bf16 arithmetic step: operate in fp32, round the result to bf16
__device__ __forceinline__ float rb(float v) { return widen(narrow(v)); }

// sigmoid in bf16 steps with the |x| branch (gdn.metal:76-79)
__device__ __forceinline__ float sigmoid_bf16(float x) {
    const float e = rb(expf(fabsf(x)));
    const float low = rb(1.0f / rb(1.0f + e));
    return x < 0.0f ? low : rb(1.0f - low);
}

__device__ __forceinline__ float half_wave_sum(float v) {
    for (uint32_t off = 1; off < 32; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
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
};

// grid (96, rows) x 128: groups 0..63 convolve one 128-channel head each
// (0..15 q, 16..31 k, 32..63 v), groups 64..95 copy the z gate.
__global__ __launch_bounds__(128) void gdn_prepare_kernel(PrepareArgs a) {
    __shared__ float partial[2];
    const uint32_t group = blockIdx.x;
    const uint32_t row = blockIdx.y;
    const uint32_t lane = threadIdx.x;
    const uint16_t* proj = a.projection + static_cast<uint64_t>(row) * a.projection_stride;
    if (group >= kCh / kGD) {
        const uint32_t index = (group - kCh / kGD) * kGD + lane;
        a.z[static_cast<uint64_t>(row) * a.z_stride + index] = proj[kCh + index];
        return;
    }
    const uint16_t* conv_in = a.conv_in;
    uint16_t* conv_out = a.conv_out;
    if (a.table != nullptr) {
        conv_in += a.table[row * 4];
        conv_out += a.table[row * 4 + 1];
    }
    const uint32_t c = group * kGD + lane;
    float taps[4];
    uint16_t tap_bits[4];
#pragma unroll
    for (uint32_t tap = 0; tap < 4; ++tap) {
        // logical sequence = three state rows then the block's projection rows
        const uint32_t logical = (a.block_mode ? row : 0u) + tap;
        tap_bits[tap] = logical < 3
                            ? conv_in[logical * kCh + c]
                            : (a.block_mode
                                   ? a.projection[static_cast<uint64_t>(logical - 3) *
                                                      a.projection_stride + c]
                                   : proj[c]);
        taps[tap] = widen(tap_bits[tap]);
    }
    const uint16_t* w = a.conv_weights + static_cast<uint64_t>(c) * 4;
    // fixed four-term shape; bf16 x bf16 products are exact in fp32
    const float convolved = widen(w[0]) * taps[0] + widen(w[1]) * taps[1] +
                            widen(w[2]) * taps[2] + widen(w[3]) * taps[3];
    const float conv_b = rb(convolved);
    const float act = rb(conv_b * sigmoid_bf16(conv_b));
    if (!a.block_mode || row == a.rows - 1) {
        conv_out[c] = tap_bits[1];
        conv_out[kCh + c] = tap_bits[2];
        conv_out[2 * kCh + c] = tap_bits[3];
    }
    if (group < kGdnQkValues / kGD) {
        // RMS over the head: lane l (< 32) sums values 4l..4l+3, then the tree
        const float neighbour_sum = [&]() {
            float sq = act * act;
            // gather 4 consecutive squares in ascending order onto lane 4k
            const float s1 = __shfl_down(sq, 1, 64);
            const float s2 = __shfl_down(sq, 2, 64);
            const float s3 = __shfl_down(sq, 3, 64);
            return ((sq + s1) + s2) + s3;
        }();
        // lanes 4k hold thread-k partials; bring them to lanes 0..15 of each wave
        const uint32_t wave = lane >> 6;
        const uint32_t wl = lane & 63;
        float v = __shfl(neighbour_sum, (wl & 15) * 4, 64);  // 16 partials per wave
        // adjacent-pairs over 32 partials = pairs within each wave, then across
        for (uint32_t off = 1; off < 16; off <<= 1) v += __shfl_xor(v, off, 64);
        if (wl == 0) partial[wave] = v;
        __syncthreads();
        const float total = partial[0] + partial[1];
        const float inverse = 1.0f / sqrtf(total / static_cast<float>(kGD) + kRmsNormEpsilon);
        const float scale = widen(group < kGdnKeyHeads ? kGdnQueryScaleBits : kGdnKeyScaleBits);
        a.qk[static_cast<uint64_t>(row) * a.qk_stride + c] = narrow(rb(act * inverse) * scale);
    } else {
        a.value[static_cast<uint64_t>(row) * a.value_stride + c - kGdnQkValues] = narrow(act);
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
};

// One half wave per state row; a 256-thread workgroup covers 8 rows of one
// (row-of-batch, value head).  grid (16, 32, rows).  The token loop serves the
// block-prefill register scan: state stays in registers across steps
// (prefill_gdn.metal:204-281).
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

// grid (32, rows) x 128: y * rsqrt(mean y^2 + eps) rounded to bf16, times the
// weight rounded to bf16, times fp32 SiLU(z); one bf16 rounding at the end
// (gdn.metal:174-207).
__global__ __launch_bounds__(128) void gdn_gate_norm_kernel(const uint16_t* y, const uint16_t* z,
                                                            const uint16_t* weight, uint16_t* out,
                                                            uint32_t stride) {
    __shared__ float partial[2];
    const uint32_t head = blockIdx.x;
    const uint32_t lane = threadIdx.x;
    const uint64_t at = static_cast<uint64_t>(blockIdx.y) * stride + head * kGD + lane;
    const float v = widen(y[at]);
    const float sq = v * v;
    const float s1 = __shfl_down(sq, 1, 64);
    const float s2 = __shfl_down(sq, 2, 64);
    const float s3 = __shfl_down(sq, 3, 64);
    const float four = ((sq + s1) + s2) + s3;
    const uint32_t wl = lane & 63;
    float t = __shfl(four, (wl & 15) * 4, 64);
    for (uint32_t off = 1; off < 16; off <<= 1) t += __shfl_xor(t, off, 64);
    if (wl == 0) partial[lane >> 6] = t;
    __syncthreads();
    const float inverse =
        1.0f / sqrtf((partial[0] + partial[1]) / static_cast<float>(kGD) + kRmsNormEpsilon);
    const float normed = rb(widen(weight[lane]) * rb(v * inverse));
    const float g = widen(z[at]);
    const float low = 1.0f / (1.0f + expf(fabsf(g)));
    const float sig = g < 0.0f ? low : 1.0f - low;
    out[at] = narrow((g * sig) * normed);
}

// ---------------------------------------------------------------- launchers --

int32_t launch_prepare(const PrepareArgs& p, hipStream_t stream) {
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
int32_t op_gdn_conv_blk(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    PrepareArgs p{};
    p.rows = a.constant(7);
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

int32_t launch_recurrence(const RecurrenceArgs& r, uint32_t rows, hipStream_t stream) {
    hipLaunchKernelGGL(gdn_recurrence_kernel, dim3(kGD / 8, kGdnValueHeads, rows), dim3(256), 0,
                       stream, r);
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
                    bool hoisted_gates) {
    Args a(b);
    RecurrenceArgs r{};
    r.steps = a.constant(8);
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
    hipLaunchKernelGGL(gdn_gate_norm_kernel, dim3(32, rows), dim3(128), 0, stream, y, z, w, out,
                       stride);
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

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side tables of launchers
const KernelDesc kGdnDecodeKernels[] = {
    {"gdn_prepare", op_gdn_prepare},
    {"gdn_prepare_ms", op_gdn_prepare_ms},
    {"gdn_recurrence", op_gdn_recurrence},
    {"gdn_recurrence_ms", op_gdn_recurrence_ms},
    {"gdn_gate_norm", op_gdn_gate_norm},
    {"gdn_gate_norm_ms", op_gdn_gate_norm_ms},
};
const uint32_t kGdnDecodeKernelCount = sizeof(kGdnDecodeKernels) / sizeof(kGdnDecodeKernels[0]);

const KernelDesc kGdnPrefillKernels[] = {
    {"gdn_conv_blk", op_gdn_conv_blk},
    {"gdn_gates_blk", op_gdn_gates_blk},
    {"gdn_recurrence_gates_blk", op_gdn_recurrence_gates_blk},
    {"gdn_recurrence_blk", op_gdn_recurrence_blk},
    {"gdn_gate_norm_blk", op_gdn_gate_norm_blk},
};
const uint32_t kGdnPrefillKernelCount = sizeof(kGdnPrefillKernels) / sizeof(kGdnPrefillKernels[0]);

#endif

}  // namespace tt
