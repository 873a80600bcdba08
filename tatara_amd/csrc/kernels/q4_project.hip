// Affine 4-bit (group 64) projections either side of the attention family: the
// input projections of both layer kinds and the output projection back to the
// hidden width.  Weight format (MLX affine, bits 4): w[n][k] = scale[n][k/64] *
// nibble + bias[n][k/64], eight nibbles to a 32-bit word, low nibble first;
// scales and biases bf16.
//
//   attn_project, attn_project_ms{,_v2}   attention.metal:1-41, 1111-1222
//   gdn_project, gdn_project_ms{,_v2}     gdn.metal:1-47, 380-491
//   gdn_outproj, gdn_outproj_ms{,_v2}     gdn.metal:209-230, 492-551 (the out_projection
//                                         pipeline of both layer kinds, decode_step.cpp:697-733)
//   gdn_project_blk, attn_project_blk, outproj_blk   prefill_dense.metal:120-260
//
// Two evaluations:
//  * rows kernel (up to 16 input rows): the reference's own sequence of operations
//    (q4_dot.metal:9-41 - one lane of 32 per 16 consecutive inputs of a 512 block,
//    power-of-two pre-scaled inputs against masked nibbles, fused chains, the
//    adjacent-pairs tree), so every output is the reference's bit pattern.  A half
//    wave owns an output row; the weights are read once for all input rows.
//  * block kernel (more rows): the nibbles are exact bf16 integers, so
//    sum_k x q per 64-column group runs on MFMA with fp32 accumulation and the affine
//    terms (scale per group and output row, bias against the group sums of x) are
//    applied in fp32 - the same mathematics in another summation order.
#include "../tt_internal.h"

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr uint32_t kQ4Block = 512;        // columns one pass of a 32-lane row group covers
constexpr uint32_t kQ4Group = 64;         // columns per {scale, bias}
constexpr uint32_t kQ4BatchRowsMax = 16;  // q4_dot.metal:49
constexpr uint32_t kMaxSegments = 4;

__device__ __forceinline__ float widen(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ float widen_half(uint32_t word, uint32_t j) {
    return __uint_as_float((j & 1) ? (word & 0xFFFF0000u) : (word << 16));
}
// round to nearest even with subnormal results flushed to signed zero
__device__ __forceinline__ uint16_t store16(float v) {
    uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0) b &= 0x80000000u;
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    const uint16_t h = static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
    return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u);
}
__device__ __forceinline__ float half_wave_sum(float v) {
    for (uint32_t off = 1; off < 32; off <<= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// A projection = up to four weight matrices stacked along the output rows.
struct Q4Projection {
    const uint32_t* words[kMaxSegments];
    const uint16_t* scales[kMaxSegments];
    const uint16_t* biases[kMaxSegments];
    uint32_t first_row[kMaxSegments + 1];  // first output row of each matrix; [segments] = total
    uint32_t segments;
    uint32_t k_size;                       // input width, a multiple of 512
    const uint16_t* input;                 // [rows][input_stride]
    uint16_t* output;                      // [rows][output_stride]
    uint64_t input_stride, output_stride;
    uint32_t rows;                         // input rows in this dispatch
    uint32_t row_tile;                     // input rows one workgroup carries (<= 16)
};

// grid (ceil(out_rows / 8), ceil(rows / row_tile)) x 256: half wave h of a workgroup
// owns output row 8 * blockIdx.x + h for the tile's input rows.
__global__ __launch_bounds__(256) void q4_rows_kernel(Q4Projection p) {
    const uint32_t lane = threadIdx.x & 31;
    const uint32_t n = blockIdx.x * 8 + (threadIdx.x >> 5);
    if (n >= p.first_row[p.segments]) return;
    uint32_t segment = 0;
    while (segment + 1 < p.segments && n >= p.first_row[segment + 1]) ++segment;
    const uint32_t local = n - p.first_row[segment];
    const uint32_t* words = p.words[segment] + static_cast<uint64_t>(local) * (p.k_size / 8);
    const uint16_t* scales = p.scales[segment] + static_cast<uint64_t>(local) * (p.k_size / kQ4Group);
    const uint16_t* biases = p.biases[segment] + static_cast<uint64_t>(local) * (p.k_size / kQ4Group);
    const uint32_t row_base = blockIdx.y * p.row_tile;
    const uint32_t tile_rows = min(p.row_tile, p.rows - row_base);
    const uint16_t* x0 = p.input + static_cast<uint64_t>(row_base) * p.input_stride;

    float acc[kQ4BatchRowsMax];
#pragma unroll
    for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) acc[r] = 0.0f;
    for (uint32_t k = 0; k < p.k_size; k += kQ4Block) {
        // four 16-bit words = this lane's 16 nibbles; masked, never shifted
        const u32x2 packed = *reinterpret_cast<const u32x2*>(words + (k >> 3) + lane * 2);
        float wq[16];
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t word = (i & 1) ? (packed[i >> 1] >> 16) : (packed[i >> 1] & 0xFFFFu);
            wq[i * 4] = static_cast<float>(word & 0x000Fu);
            wq[i * 4 + 1] = static_cast<float>(word & 0x00F0u);
            wq[i * 4 + 2] = static_cast<float>(word & 0x0F00u);
            wq[i * 4 + 3] = static_cast<float>(word & 0xF000u);
        }
        const uint32_t group = (k >> 6) + (lane >> 2);
        const float scale = widen(scales[group]);
        const float bias = widen(biases[group]);
        const uint16_t* xk = x0 + k + lane * 16;
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < tile_rows) {
                const u32x4* xr = reinterpret_cast<const u32x4*>(xk + r * p.input_stride);
                const u32x4 lo = xr[0], hi = xr[1];
                float sum = 0.0f, quant = 0.0f;
#pragma unroll
                for (uint32_t i = 0; i < 4; ++i) {
                    const uint32_t w0 = i < 2 ? lo[2 * i] : hi[2 * i - 4];
                    const uint32_t w1 = i < 2 ? lo[2 * i + 1] : hi[2 * i - 3];
                    const float a0 = widen_half(w0, 0), a1 = widen_half(w0, 1);
                    const float a2 = widen_half(w1, 0), a3 = widen_half(w1, 1);
                    sum += ((a0 + a1) + a2) + a3;
                    quant = fmaf(a0, wq[i * 4], quant);
                    quant = fmaf(a1 * 0.0625f, wq[i * 4 + 1], quant);
                    quant = fmaf(a2 * 0.00390625f, wq[i * 4 + 2], quant);
                    quant = fmaf(a3 * 0.000244140625f, wq[i * 4 + 3], quant);
                }
                acc[r] = fmaf(sum, bias, fmaf(scale, quant, acc[r]));
            }
        }
    }
#pragma unroll
    for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
        if (r < tile_rows) {
            const float total = half_wave_sum(acc[r]);
            if (lane == 0) {
                p.output[static_cast<uint64_t>(row_base + r) * p.output_stride + n] = store16(total);
            }
        }
    }
}

int32_t launch_rows(const Q4Projection& p, hipStream_t stream) {
    const uint32_t out_rows = p.first_row[p.segments];
    hipLaunchKernelGGL(q4_rows_kernel, dim3((out_rows + 7) / 8, (p.rows + p.row_tile - 1) / p.row_tile),
                       dim3(256), 0, stream, p);
    return TT_OK;
}

// Binds `count` weight matrices from buffer slots first, first+3, ...: words, scales,
// biases of each, sized for its rows.
void bind_segments(Args& a, Q4Projection& p, uint32_t first_slot, const uint32_t* rows,
                   uint32_t count, uint32_t k_size) {
    p.segments = count;
    p.k_size = k_size;
    p.first_row[0] = 0;
    for (uint32_t s = 0; s < count; ++s) {
        const uint32_t slot = first_slot + 3 * s;
        p.words[s] = a.buffer<const uint32_t>(slot, static_cast<uint64_t>(rows[s]) * (k_size / 8) * 4);
        p.scales[s] =
            a.buffer<const uint16_t>(slot + 1, static_cast<uint64_t>(rows[s]) * (k_size / kQ4Group) * 2);
        p.biases[s] =
            a.buffer<const uint16_t>(slot + 2, static_cast<uint64_t>(rows[s]) * (k_size / kQ4Group) * 2);
        p.first_row[s + 1] = p.first_row[s] + rows[s];
    }
}

constexpr uint32_t kMaxBatchRows = 16;              // rows of a decode wave (decode_step.cpp:554)
constexpr uint32_t kProjectionRowThreads = 128;     // decode_geometry.h:147
constexpr uint32_t kOutProjectionRowThreads = 64;   // decode_geometry.h:148

// One projection operator family: its weight matrices (slots 1, 4, 7, ...), input
// width, the slot of the output and the threads per group of the reference's grid
// (one 32-lane group per output row).
struct Family {
    uint32_t segment_rows[kMaxSegments];
    uint32_t segments;
    uint32_t k_size;
    uint32_t out_slot;
    uint32_t threads;
    constexpr uint32_t out_rows() const {
        uint32_t total = 0;
        for (uint32_t s = 0; s < segments; ++s) total += segment_rows[s];
        return total;
    }
    constexpr uint64_t groups() const {
        const uint32_t per_group = threads / 32;
        return (out_rows() + per_group - 1) / per_group;
    }
};
constexpr Family kAttnProject{{kAttnQGateRows, kAttnVRowOffset - kAttnQGateRows,
                               kAttnProjectionRows - kAttnVRowOffset, 0},
                              3, kHidden, 10, kProjectionRowThreads};
constexpr Family kGdnProject{{kGdnConvChannels, kGdnValueValues, kGdnValueHeads, kGdnValueHeads},
                             4, kHidden, 13, kProjectionRowThreads};
constexpr Family kOutProject{{kHidden, 0, 0, 0}, 1, kGdnValueValues, 4, kOutProjectionRowThreads};
static_assert(kAttnProject.out_rows() == kAttnProjectionRows && kAttnProject.groups() == 2304);
static_assert(kGdnProject.out_rows() == kGdnProjectionRows && kGdnProject.groups() == 3088);
static_assert(kOutProject.out_rows() == kHidden && kOutProject.groups() == 1024);

// Binds input, weights and output once rows / strides / tiling are known, checks the
// reference's grid (groups, tiles) x threads, and launches.
int32_t finish(Args& a, const Grid& g, hipStream_t stream, bool validate_only, const Family& f,
               Q4Projection& p, uint32_t k_size, uint64_t tiles) {
    const uint32_t out_rows = f.out_rows();
    a.require(p.output_stride >= out_rows, TT_CMD_INVALID_BUFFER);
    a.require(grid_is(g, f.groups(), tiles, 1, f.threads, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    p.input_stride = k_size;
    p.input = a.buffer<const uint16_t>(0, static_cast<uint64_t>(p.rows) * k_size * 2);
    bind_segments(a, p, 1, f.segment_rows, f.segments, k_size);
    p.output = a.buffer<uint16_t>(
        f.out_slot, (static_cast<uint64_t>(p.rows - 1) * p.output_stride + out_rows) * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_rows(p, stream);
}

// one input row; grid (groups) x threads
int32_t project_single(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                       const Family& f) {
    Args a(b);
    Q4Projection p{};
    p.rows = p.row_tile = 1;
    p.output_stride = f.out_rows();
    return finish(a, g, stream, validate_only, f, p, f.k_size, 1);
}

// rows of a decode wave: c[out+1] rows (1..16), then the output row stride where the
// operator has one, then the row tile; grid (groups, ceil(rows / tile)) x threads
int32_t project_tiled(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                      const Family& f, bool strided_output) {
    Args a(b);
    Q4Projection p{};
    p.rows = a.constant(f.out_slot + 1);
    p.output_stride = strided_output ? a.constant(f.out_slot + 2) : f.out_rows();
    p.row_tile = a.constant(f.out_slot + (strided_output ? 3 : 2));
    a.require(p.rows >= 1 && p.rows <= kMaxBatchRows && p.row_tile >= 1 &&
                  p.row_tile <= kQ4BatchRowsMax,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    return finish(a, g, stream, validate_only, f, p, f.k_size,
                  (p.rows + p.row_tile - 1) / p.row_tile);
}

// a block of consecutive tokens: c[out+1] rows, then the input width where the
// operator takes one; grid (groups) x threads
int32_t project_block(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                      const Family& f, bool variable_width) {
    Args a(b);
    Q4Projection p{};
    p.rows = a.constant(f.out_slot + 1);
    const uint32_t k_size = variable_width ? a.constant(f.out_slot + 2) : f.k_size;
    a.require(p.rows >= 1 && k_size >= kQ4Block && k_size % kQ4Block == 0 && k_size <= 8192,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    p.row_tile = kQ4BatchRowsMax;
    p.output_stride = f.out_rows();
    return finish(a, g, stream, validate_only, f, p, k_size, 1);
}

// attn_project: b0 input[2048], b1-3 query+gate (8192 rows), b4-6 key (512), b7-9 value
// (512), b10 projection[9216]; grid 2304 x 128 (decode_step.cpp:705-711).
int32_t op_attn_project(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_single(b, g, s, v, kAttnProject);
}
// attn_project_ms{,_v2}: + c11 rows, c12 row tile; grid (2304, ceil(rows/tile)) x 128
// (decode_step.cpp:1213-1229).
int32_t op_attn_project_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kAttnProject, false);
}
// attn_project_blk: + c11 block rows; grid 2304 x 128 (prefill_step.cpp:1428-1446).
int32_t op_attn_project_blk(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_block(b, g, s, v, kAttnProject, false);
}
// gdn_project: b0 input[2048], b1-3 qkv (8192 rows), b4-6 z (4096), b7-9 b (32), b10-12 a
// (32), b13 projection[12352]; grid 3088 x 128 (decode_step.cpp:657-664).
int32_t op_gdn_project(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_single(b, g, s, v, kGdnProject);
}
// gdn_project_ms{,_v2}: + c14 rows, c15 row tile (decode_step.cpp:1117-1130).
int32_t op_gdn_project_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kGdnProject, false);
}
// gdn_project_blk: + c14 block rows (prefill_step.cpp:1909-1926).
int32_t op_gdn_project_blk(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_block(b, g, s, v, kGdnProject, false);
}
// gdn_outproj: b0 input[4096], b1-3 weights (2048 rows), b4 output[2048]; grid 1024 x 64
// (decode_step.cpp:697-701, 729-733: the out_projection pipeline of both layer kinds).
int32_t op_gdn_outproj(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_single(b, g, s, v, kOutProject);
}
// gdn_outproj_ms{,_v2}: + c5 rows, c6 output row stride, c7 row tile (decode_step.cpp:1196-1206).
int32_t op_gdn_outproj_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kOutProject, true);
}
// outproj_blk: + c5 block rows, c6 input width (prefill_step.cpp:2063-2078).
int32_t op_outproj_blk(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_block(b, g, s, v, kOutProject, true);
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side table of launchers
const KernelDesc kQ4ProjectKernels[] = {
    {"attn_project", op_attn_project},
    {"attn_project_ms", op_attn_project_ms},
    {"attn_project_ms_v2", op_attn_project_ms},
    {"attn_project_blk", op_attn_project_blk},
    {"gdn_project", op_gdn_project},
    {"gdn_project_ms", op_gdn_project_ms},
    {"gdn_project_ms_v2", op_gdn_project_ms},
    {"gdn_project_blk", op_gdn_project_blk},
    {"gdn_outproj", op_gdn_outproj},
    {"gdn_outproj_ms", op_gdn_outproj_ms},
    {"gdn_outproj_ms_v2", op_gdn_outproj_ms},
    {"outproj_blk", op_outproj_blk},
};
const uint32_t kQ4ProjectKernelCount = sizeof(kQ4ProjectKernels) / sizeof(kQ4ProjectKernels[0]);
#endif

}  // namespace tt
