// The steps either side of the attention family in a stacked run: the layer
// input norm, dense projections standing in for the reference's Q4 GEMV/GEMM,
// and the residual sum.  They let a hybrid 40-layer stack run end to end on the
// GPU so that the family's kernels are exercised (and timed) in place.
//
//   rms_only, rms_only_ms  src/backend/metal/kernels/rms_only.metal:5, :44
//       (dispatch: decode_step.cpp:641-645, 1103-1109; grid 1 x hidden/4 threads,
//       _ms adds the row in grid y with element strides in c3 / c4)
//   residual_rms, residual_rms_ms  src/backend/metal/kernels/moe.metal:1, :551
//       (dispatch: decode_step.cpp:735-742, 1298-1308): residual = bf16(a + b), then the
//       same row norm over the rounded sums, both written
//   dense_bf16, add_bf16   no reference counterpart: the reference projects with
//       4-bit weights (q4_dot.metal); here the weights are plain bf16.
#include "../tt_internal.h"
#include "lane_sums.h"
#include "rms_row.h"

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

__device__ __forceinline__ float widen(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
// round to nearest even with subnormal results flushed to signed zero
__device__ __forceinline__ uint16_t store16(float v) {
    uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0) b &= 0x80000000u;
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    const uint16_t h = static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
    return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u);
}
__device__ __forceinline__ uint16_t fz16(uint16_t h) {
    return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u);
}

// One row of `hidden` values (a multiple of 128, at most 4096) per workgroup of
// hidden/4 threads: thread t squares values 4t..4t+3 in order, 32-lane groups sum
// in the adjacent-pairs tree (= xor butterfly), the group sums land in a 32-slot
// stage that is summed by the same tree; out = bf16(w * bf16(x * inverse)).
// With `addend`, the row normalised is residual = bf16(input + addend), which is also
// written to `residual_out` (residual_rms): the norm consumes the rounded sums.
__global__ __launch_bounds__(1024) void rms_only_kernel(const uint16_t* input, const uint16_t* weight,
                                                        uint16_t* output, uint32_t hidden,
                                                        uint32_t in_stride, uint32_t out_stride,
                                                        const uint16_t* addend, uint16_t* residual_out,
                                                        uint32_t residual_stride) {
    __shared__ float stage[32];
    __shared__ float inverse_norm;
    const uint32_t t = threadIdx.x;
    const uint16_t* in = input + static_cast<uint64_t>(blockIdx.y) * in_stride;
    uint16_t* out = output + static_cast<uint64_t>(blockIdx.y) * out_stride;
    u32x2 raw = *reinterpret_cast<const u32x2*>(in + 4 * t);
    // requested with the row, not after the reduction
    const u32x2 wraw = *reinterpret_cast<const u32x2*>(weight + 4 * t);
    if (addend != nullptr) {
        const u32x2 other = *reinterpret_cast<const u32x2*>(
            addend + static_cast<uint64_t>(blockIdx.y) * residual_stride + 4 * t);
        uint16_t sum[4];
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint16_t xa = static_cast<uint16_t>(raw[i >> 1] >> ((i & 1) * 16));
            const uint16_t xb = static_cast<uint16_t>(other[i >> 1] >> ((i & 1) * 16));
            sum[i] = store16(widen(fz16(xa)) + widen(fz16(xb)));
        }
        raw = u32x2{sum[0] | (static_cast<uint32_t>(sum[1]) << 16),
                    sum[2] | (static_cast<uint32_t>(sum[3]) << 16)};
        *reinterpret_cast<u32x2*>(residual_out + static_cast<uint64_t>(blockIdx.y) * residual_stride +
                                  4 * t) = raw;
    }
    float sum = rms_slice_squares(raw.x, raw.y);
    sum = half_wave_sum(sum);
    if (t < 32) stage[t] = 0.0f;
    __syncthreads();
    if ((t & 31) == 0) stage[t >> 5] = sum;
    __syncthreads();
    if (t < 32) {
        float total = stage[t];
        total = half_wave_sum(total);
        if (t == 0) inverse_norm = rms_inverse(total, hidden);
    }
    __syncthreads();
    const float inverse = inverse_norm;
    *reinterpret_cast<u32x2*>(out + 4 * t) =
        u32x2{rms_scale_pair(raw.x, wraw.x, inverse), rms_scale_pair(raw.y, wraw.y, inverse)};
}

// out[r][n] = bf16(sum_k x[r][k] w[n][k]).  grid (ceil(N/64), ceil(rows/16)) x 256:
// a wave owns 16 outputs x 16 rows on v_mfma_f32_16x16x32_bf16, operands straight
// from memory.
__global__ __launch_bounds__(256) void dense_bf16_kernel(const uint16_t* input,
                                                         const uint16_t* weights, uint16_t* output,
                                                         uint32_t rows, uint32_t in_dim,
                                                         uint32_t out_dim) {
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t n0 = blockIdx.x * 64 + wave * 16;
    const uint32_t r0 = blockIdx.y * 16;
    if (n0 >= out_dim) return;
    const uint16_t* wp = weights + static_cast<uint64_t>(min(n0 + m, out_dim - 1)) * in_dim + g * 8;
    const uint16_t* xp = input + static_cast<uint64_t>(min(r0 + m, rows - 1)) * in_dim + g * 8;
    f32x4 acc0 = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4 acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t k = 0; k < in_dim; k += 64) {
        const bf16x8 wa0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(wp + k));
        const bf16x8 xb0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(xp + k));
        const bf16x8 wa1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(wp + k + 32));
        const bf16x8 xb1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(xp + k + 32));
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa0, xb0, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa1, xb1, acc1, 0, 0, 0);
    }
    // lane holds outputs n0 + 4g + i of row r0 + m
    const uint32_t row = r0 + m;
    if (row < rows) {
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t n = n0 + g * 4 + i;
            if (n < out_dim) output[static_cast<uint64_t>(row) * out_dim + n] = store16(acc0[i] + acc1[i]);
        }
    }
}

// The same for at most 16 rows (a decode wave), sized for latency: a workgroup owns 16
// outputs, its kWaves waves split K = 512 kWaves in slices of 512 columns, and a lane
// requests all 16 weight fragments and all 16 x fragments of its slice before the first
// product (the kernel above walks K with one dependent load pair after the other, which
// makes a 64 KB weight stream per wave a chain of 32 round trips).  The slices are summed
// through LDS in wave order.  grid ceil(N / 16) x 64 kWaves.
template <uint32_t kWaves>
__global__ __launch_bounds__(64 * kWaves) void dense_rows_kernel(const uint16_t* input,
                                                                 const uint16_t* weights,
                                                                 uint16_t* output, uint32_t rows,
                                                                 uint32_t out_dim) {
    constexpr uint32_t kInDim = 512 * kWaves;
    __shared__ float partial[kWaves][4][64];
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16;
    const uint16_t* wp =
        weights + static_cast<uint64_t>(min(n0 + m, out_dim - 1)) * kInDim + wave * 512 + g * 8;
    const uint16_t* xp = input + static_cast<uint64_t>(min(m, rows - 1)) * kInDim + wave * 512 + g * 8;
    u32x4 w[16], x[16];
#pragma unroll
    for (uint32_t s = 0; s < 16; ++s) w[s] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wp + s * 32));
#pragma unroll
    for (uint32_t s = 0; s < 16; ++s) x[s] = *reinterpret_cast<const u32x4*>(xp + s * 32);
    f32x4 acc0 = {0.0f, 0.0f, 0.0f, 0.0f};
    f32x4 acc1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (uint32_t s = 0; s < 16; s += 2) {
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[s]),
                                                       __builtin_bit_cast(bf16x8, x[s]), acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, w[s + 1]),
                                                       __builtin_bit_cast(bf16x8, x[s + 1]), acc1, 0, 0, 0);
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) partial[wave][i][lane] = acc0[i] + acc1[i];
    __syncthreads();
    if (wave != 0 || m >= rows) return;
    // lane holds outputs n0 + 4g + i of row m
    uint16_t result[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        float total = partial[0][i][lane];
#pragma unroll
        for (uint32_t v = 1; v < kWaves; ++v) total += partial[v][i][lane];
        result[i] = store16(total);
    }
    uint16_t* out = output + static_cast<uint64_t>(m) * out_dim + n0 + g * 4;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        if (n0 + g * 4 + i < out_dim) out[i] = result[i];
    }
}

__global__ __launch_bounds__(256) void add_bf16_kernel(const uint16_t* a, const uint16_t* b,
                                                       uint16_t* out, uint32_t count) {
    const uint32_t at = blockIdx.x * 256 + threadIdx.x;
    if (at >= count) return;
    out[at] = store16(widen(fz16(a[at])) + widen(fz16(b[at])));
}

int32_t launch_rms(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                   bool strided) {
    Args a(b);
    a.require(g.gx == 1 && g.gz == 1 && g.ty == 1 && g.tz == 1 && g.tx >= 32 && g.tx <= 1024 &&
                  g.tx % 32 == 0 && g.gy >= 1 && g.gy <= 65535 && (strided || g.gy == 1),
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t hidden = static_cast<uint32_t>(g.tx) * 4;
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    const uint32_t in_stride = strided ? a.constant(3) : hidden;
    const uint32_t out_stride = strided ? a.constant(4) : hidden;
    a.require(in_stride >= hidden && out_stride >= hidden, TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint16_t* input =
        a.buffer<const uint16_t>(0, (static_cast<uint64_t>(rows - 1) * in_stride + hidden) * 2);
    const uint16_t* weight = a.buffer<const uint16_t>(1, static_cast<uint64_t>(hidden) * 2);
    uint16_t* output =
        a.buffer<uint16_t>(2, (static_cast<uint64_t>(rows - 1) * out_stride + hidden) * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(rms_only_kernel, dim3(1, rows), dim3(hidden / 4), 0, stream, input, weight,
                       output, hidden, in_stride, out_stride, static_cast<const uint16_t*>(nullptr),
                       static_cast<uint16_t*>(nullptr), 0u);
    return TT_OK;
}

// residual_rms: b0 a, b1 b, b2 residual out (may alias b), b3 weight, b4 normed out;
// grid 1 x hidden/4 (decode_step.cpp:735-742).  residual_rms_ms: + c5 row stride of a,
// c6 row stride of b and of the residual, c7 row stride of the normed output
// (elements); grid (1, rows) x hidden/4 (decode_step.cpp:1298-1308).
int32_t launch_residual_rms(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only, bool strided) {
    Args a(b);
    a.require(g.gx == 1 && g.gz == 1 && g.ty == 1 && g.tz == 1 && g.tx >= 32 && g.tx <= 1024 &&
                  g.tx % 32 == 0 && g.gy >= 1 && g.gy <= 65535 && (strided || g.gy == 1),
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint32_t hidden = static_cast<uint32_t>(g.tx) * 4;
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    const uint32_t a_stride = strided ? a.constant(5) : hidden;
    const uint32_t lane_stride = strided ? a.constant(6) : hidden;
    const uint32_t normed_stride = strided ? a.constant(7) : hidden;
    a.require(a_stride >= hidden && lane_stride >= hidden && normed_stride >= hidden,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const auto extent = [&](uint32_t stride) {
        return (static_cast<uint64_t>(rows - 1) * stride + hidden) * 2;
    };
    const uint16_t* first = a.buffer<const uint16_t>(0, extent(a_stride));
    const uint16_t* second = a.buffer<const uint16_t>(1, extent(lane_stride));
    uint16_t* residual = a.buffer<uint16_t>(2, extent(lane_stride));
    const uint16_t* weight = a.buffer<const uint16_t>(3, static_cast<uint64_t>(hidden) * 2);
    uint16_t* normed = a.buffer<uint16_t>(4, extent(normed_stride));
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(rms_only_kernel, dim3(1, rows), dim3(hidden / 4), 0, stream, first, weight,
                       normed, hidden, a_stride, normed_stride, second, residual, lane_stride);
    return TT_OK;
}
int32_t op_residual_rms(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    return launch_residual_rms(b, g, stream, validate_only, false);
}
int32_t op_residual_rms_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                           bool validate_only) {
    return launch_residual_rms(b, g, stream, validate_only, true);
}

// rms_only: b0 input, b1 weight, b2 output; grid 1 x hidden/4.
int32_t op_rms_only(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    return launch_rms(b, g, stream, validate_only, false);
}
// rms_only_ms: + c3 input row stride, c4 output row stride (elements); grid (1, rows) x hidden/4.
int32_t op_rms_only_ms(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    return launch_rms(b, g, stream, validate_only, true);
}

// dense_bf16: b0 input [rows][in], b1 weights [out][in], b2 output [rows][out], c3 rows,
// c4 in (multiple of 64), c5 out; grid (ceil(out/64), ceil(rows/16)) x 256.
int32_t op_dense_bf16(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t rows = a.constant(3);
    const uint32_t in_dim = a.constant(4);
    const uint32_t out_dim = a.constant(5);
    a.require(rows >= 1 && rows <= (1u << 20) && in_dim >= 64 && in_dim % 64 == 0 && out_dim >= 1 &&
                  g.gx == (out_dim + 63) / 64 && g.gy == (rows + 15) / 16 && g.gz == 1 &&
                  g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint16_t* input = a.buffer<const uint16_t>(0, static_cast<uint64_t>(rows) * in_dim * 2);
    const uint16_t* weights = a.buffer<const uint16_t>(1, static_cast<uint64_t>(out_dim) * in_dim * 2);
    uint16_t* output = a.buffer<uint16_t>(2, static_cast<uint64_t>(rows) * out_dim * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    // a decode wave over one of the model's two widths: the latency-sized form
    if (rows <= 16 && in_dim == 2048) {
        hipLaunchKernelGGL(dense_rows_kernel<4>, dim3((out_dim + 15) / 16), dim3(256), 0, stream, input,
                           weights, output, rows, out_dim);
    } else if (rows <= 16 && in_dim == 4096) {
        hipLaunchKernelGGL(dense_rows_kernel<8>, dim3((out_dim + 15) / 16), dim3(512), 0, stream, input,
                           weights, output, rows, out_dim);
    } else {
        hipLaunchKernelGGL(dense_bf16_kernel, dim3((out_dim + 63) / 64, (rows + 15) / 16), dim3(256), 0,
                           stream, input, weights, output, rows, in_dim, out_dim);
    }
    return TT_OK;
}

// add_bf16: b0 a, b1 b, b2 out (may alias a or b), c3 count; grid ceil(count/256) x 256.
int32_t op_add_bf16(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    const uint32_t count = a.constant(3);
    a.require(count >= 1 && g.gx == (static_cast<uint64_t>(count) + 255) / 256 && g.gy == 1 &&
                  g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    const uint16_t* x = a.buffer<const uint16_t>(0, static_cast<uint64_t>(count) * 2);
    const uint16_t* y = a.buffer<const uint16_t>(1, static_cast<uint64_t>(count) * 2);
    uint16_t* out = a.buffer<uint16_t>(2, static_cast<uint64_t>(count) * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(add_bf16_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, x, y, out,
                       count);
    return TT_OK;
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side table of launchers
const KernelDesc kStackStepKernels[] = {
    {"rms_only", op_rms_only},
    {"rms_only_ms", op_rms_only_ms},
    {"residual_rms", op_residual_rms},
    {"residual_rms_ms", op_residual_rms_ms},
    {"dense_bf16", op_dense_bf16},
    {"add_bf16", op_add_bf16},
};
const uint32_t kStackStepKernelCount = sizeof(kStackStepKernels) / sizeof(kStackStepKernels[0]);
#endif

}  // namespace tt
