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
#include "lane_sums.h"
#include "rms_row.h"

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
    // the decode-wave kernel only:
    const uint16_t* norm_weight;           // not null: the input rows go through the RMS norm first
    const uint16_t* residual;              // not null: output = bf16(residual + bf16(projection)),
    uint64_t residual_stride;              //   [rows][residual_stride]; may be the output itself
    // the block kernel only: how its tiles are dealt to workgroups (see launch_block)
    uint32_t tiles_n;                      // tiles along the output rows
    uint32_t whole_tiles;                  // tiles 0 .. whole_tiles - 1 have a workgroup each
    uint32_t sharers;                      // the others are shared by this many, a slice of K each
    uint8_t* exchange;                     // arrival counts, then the sharers' partial sums
};

// The weight matrix that holds output row `n`, with n the same for every lane (matrices have
// multiples of 16 rows, so a workgroup's 8 or 16 rows share one): the operands are picked with
// selects on scalar registers.  Indexing the argument arrays with a per-lane value instead
// turns into vector loads from the argument block - a round trip to memory before the
// first weight can be requested.
struct Q4Matrix {
    const uint32_t* words;
    const uint16_t* scales;
    const uint16_t* biases;
    uint32_t first_row;
};
__device__ __forceinline__ Q4Matrix matrix_of_row(const Q4Projection& p, uint32_t n) {
    Q4Matrix m{p.words[0], p.scales[0], p.biases[0], 0};
#pragma unroll
    for (uint32_t s = 1; s < kMaxSegments; ++s) {
        const bool here = s < p.segments && n >= p.first_row[s];
        m.words = here ? p.words[s] : m.words;
        m.scales = here ? p.scales[s] : m.scales;
        m.biases = here ? p.biases[s] : m.biases;
        m.first_row = here ? p.first_row[s] : m.first_row;
    }
    return m;
}

// grid (ceil(out_rows / 8), ceil(rows / row_tile)) x 256: half wave h of a workgroup
// owns output row 8 * blockIdx.x + h for the tile's input rows.  kBlocks = k_size / 512:
// all of the row's nibbles, scales and biases are requested before the first is used, so
// one row keeps kBlocks loads per lane in flight instead of one.  The tile's x rows are
// the same for all eight output rows: they come in once with coalesced 16-byte loads,
// requested first, and are read back from LDS (every half wave fetching its own copy from
// global memory cost as much as streaming the weights).  LDS layout of one 512-column
// block of a row: the even 16-byte pieces, then the odd ones, so that the 32 lanes of a
// half wave read 512 contiguous bytes twice.  Where the tiles of the workgroups that share
// a compute unit do not fit its LDS (kStaged = false) x is read from global memory: there
// the workgroups per compute unit matter more than the x traffic.
template <uint32_t kBlocks, bool kStaged>
__global__ __launch_bounds__(256) void q4_rows_kernel(Q4Projection p) {
    extern __shared__ __align__(16) uint8_t rows_lds[];   // [tile rows][kBlocks][1024]
    constexpr uint32_t kPiecesPerRow = kBlocks * 64;
    const uint32_t lane = threadIdx.x & 31;
    const uint32_t row_base = blockIdx.y * p.row_tile;
    const uint32_t tile_rows = min(p.row_tile, p.rows - row_base);
    for (uint32_t piece = threadIdx.x; kStaged && piece < tile_rows * kPiecesPerRow; piece += 256) {
        const uint32_t r = piece / kPiecesPerRow, c = piece % kPiecesPerRow;
        const u32x4 staged = *reinterpret_cast<const u32x4*>(
            p.input + static_cast<uint64_t>(row_base + r) * p.input_stride + c * 8);
        const uint32_t slot = (c & ~63u) + ((c & 63u) >> 1) + (c & 1u) * 32;
        *reinterpret_cast<u32x4*>(rows_lds + (r * kPiecesPerRow + slot) * 16) = staged;
    }
    // rows past the last one compute on the last row and store nothing
    const uint32_t n = min(blockIdx.x * 8 + (threadIdx.x >> 5), p.first_row[p.segments] - 1);
    const bool stores = blockIdx.x * 8 + (threadIdx.x >> 5) < p.first_row[p.segments];
    const Q4Matrix matrix = matrix_of_row(p, min(blockIdx.x * 8, p.first_row[p.segments] - 1));
    const uint32_t local = n - matrix.first_row;
    const uint32_t* words = matrix.words + static_cast<uint64_t>(local) * (kBlocks * 64);
    const uint16_t* scales = matrix.scales + static_cast<uint64_t>(local) * (kBlocks * 8);
    const uint16_t* biases = matrix.biases + static_cast<uint64_t>(local) * (kBlocks * 8);

    u32x2 packed[kBlocks];
    uint16_t scale_bits[kBlocks], bias_bits[kBlocks];
#pragma unroll
    for (uint32_t b = 0; b < kBlocks; ++b) {
        // four 16-bit words = this lane's 16 nibbles of block b
        packed[b] = *reinterpret_cast<const u32x2*>(words + b * 64 + lane * 2);
        scale_bits[b] = scales[b * 8 + (lane >> 2)];
        bias_bits[b] = biases[b * 8 + (lane >> 2)];
    }
    if (kStaged) __syncthreads();
    const uint16_t* x0 = p.input + static_cast<uint64_t>(row_base) * p.input_stride + lane * 16;
    float acc[kQ4BatchRowsMax];
#pragma unroll
    for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) acc[r] = 0.0f;
#pragma unroll
    for (uint32_t b = 0; b < kBlocks; ++b) {
        float wq[16];   // masked, never shifted
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            const uint32_t word = (i & 1) ? (packed[b][i >> 1] >> 16) : (packed[b][i >> 1] & 0xFFFFu);
            wq[i * 4] = static_cast<float>(word & 0x000Fu);
            wq[i * 4 + 1] = static_cast<float>(word & 0x00F0u);
            wq[i * 4 + 2] = static_cast<float>(word & 0x0F00u);
            wq[i * 4 + 3] = static_cast<float>(word & 0xF000u);
        }
        const float scale = widen(scale_bits[b]);
        const float bias = widen(bias_bits[b]);
        const uint8_t* xk = rows_lds + b * 1024 + lane * 16;
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < tile_rows) {
                u32x4 lo, hi;
                if (kStaged) {
                    lo = *reinterpret_cast<const u32x4*>(xk + r * (kPiecesPerRow * 16));
                    hi = *reinterpret_cast<const u32x4*>(xk + r * (kPiecesPerRow * 16) + 512);
                } else {
                    const u32x4* xr =
                        reinterpret_cast<const u32x4*>(x0 + b * kQ4Block + r * p.input_stride);
                    lo = xr[0];
                    hi = xr[1];
                }
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
            if (lane == 0 && stores) {
                p.output[static_cast<uint64_t>(row_base + r) * p.output_stride + n] = store16(total);
            }
        }
    }
}

constexpr uint32_t kRowsStagedBytes = 128 * 1024;   // of the 160 KB of a compute unit

// 0 when the width has no instantiation
int32_t launch_rows(const Q4Projection& p, hipStream_t stream) {
    const uint32_t out_rows = p.first_row[p.segments];
    const dim3 grid((out_rows + 7) / 8, (p.rows + p.row_tile - 1) / p.row_tile);
    const uint32_t tile_rows = min(p.rows, p.row_tile);
    // as many workgroups as the grid puts on a compute unit (up to eight) must still fit
    const uint32_t resident = min(8u, (grid.x * grid.y + 255) / 256);
    const auto staged = [&](uint32_t row_bytes) {
        return tile_rows * row_bytes * resident <= kRowsStagedBytes;
    };
    switch (p.k_size / kQ4Block) {
    // LDS: the tile's x rows where they fit kRowsStagedBytes
    case 4:
        if (staged(4096)) {
            hipLaunchKernelGGL((q4_rows_kernel<4, true>), grid, dim3(256), tile_rows * 4096, stream, p);
        } else {
            hipLaunchKernelGGL((q4_rows_kernel<4, false>), grid, dim3(256), 0, stream, p);
        }
        break;
    case 8:
        if (staged(8192)) {
            hipLaunchKernelGGL((q4_rows_kernel<8, true>), grid, dim3(256), tile_rows * 8192, stream, p);
        } else {
            hipLaunchKernelGGL((q4_rows_kernel<8, false>), grid, dim3(256), 0, stream, p);
        }
        break;
    default: return TT_CMD_INVALID_DISPATCH_EXTENT;
    }
    return TT_OK;
}

// ------------------------------------------------------------ block kernel ---
//
// out[m][n] = sum_g scale[n][g] * (sum_{k in g} x[m][k] q[n][k]) + bias[n][g] * xs[m][g],
// xs[m][g] = sum_{k in g} x[m][k].  A workgroup of eight waves owns 128 output rows (n) x
// 256 input rows (m) and walks K one group (64 columns) at a time:
//   * x (three stages), the nibble words (a pair of groups per transfer, two stages) and
//     the scales and biases (a window of eight groups per transfer, two stages) go from
//     global memory straight into LDS (no registers), x two groups ahead.  A nibble becomes
//     the bf16 number 16 + nibble (dropped into mantissa bits 3..6 of 0x4180, three
//     instructions a pair) and is written to one of two unpacked stages.  Rows are 128 B
//     without padding; 16-byte piece p of row r sits in slot p ^ (r & 7), which keeps the
//     16-byte fragment reads of sixteen consecutive rows free of bank conflicts.
//   * each wave multiplies a 64 x 64 part as 4 x 4 tiles of v_mfma_f32_16x16x32_bf16 with m
//     along the rows of the result, so a lane holds one n per tile and needs one scale per
//     tile and group: two MFMAs per tile and group from a zero accumulator, then
//     acc += scale[n] * partial in fp32.
//   * xs comes from the same MFMA unit (a ones operand against the x fragments), is split
//     into bf16 hi + lo and, once every four groups, multiplied by one
//     v_mfma_f32_16x16x16_bf16 per tile: slots {hi, lo, hi, lo} of four groups against
//     {bias, bias, -16 scale, -16 scale}, the latter taking the nibble offset back out.
//   * the eight waves work as two sets of four that alternate between the matrix unit and
//     everything else of a group, so that the two waves of a SIMD are never in the same
//     phase (see the schedule before the main loop).
//   * the result leaves through LDS, so that a row of 64 outputs is stored as 128
//     contiguous bytes.
constexpr uint32_t kBlockN = 128;                    // output rows of a workgroup tile
constexpr uint32_t kBlockM = 256;                    // input rows of a workgroup tile
constexpr uint32_t kBlockThreads = 512;
constexpr uint32_t kStages = 3;                      // of what arrives from global memory
constexpr uint32_t kRowBytes = 128;                  // one group of one row: 64 bf16
constexpr uint32_t kXStageBytes = kBlockM * kRowBytes;                   // 32768, three of them
// the nibble words of a pair of groups (an even one and the next): [n][16 words], two of them
constexpr uint32_t kWordBase = kStages * kXStageBytes;
constexpr uint32_t kWordPairBytes = kBlockN * 64;
constexpr uint32_t kQStageBytes = kBlockN * kRowBytes;                   // unpacked: 16384, two of them
constexpr uint32_t kQBase = kWordBase + 2 * kWordPairBytes;
constexpr uint32_t kGroupSumBase = kQBase + 2 * kQStageBytes;
constexpr uint32_t kGroupSumBytes = 2 * kBlockM * 8 * 2;                 // [window of 4 groups][m][4 hi, 4 lo] bf16
// scales and biases of a window of eight groups, two windows: [window][scales, biases][n]
// [8 bf16]
constexpr uint32_t kMetaBase = kGroupSumBase + kGroupSumBytes;
constexpr uint32_t kMetaKindBytes = kBlockN * 16;
constexpr uint32_t kMetaWindowBytes = 2 * kMetaKindBytes;
constexpr uint32_t kBlockLdsBytes = kMetaBase + 2 * kMetaWindowBytes;    // 163840
constexpr uint32_t kOutRowBytes = 144;               // a wave's 64 results of one m on the way out
constexpr uint32_t kExchangeCountBytes = 4096;       // arrival counts of the shared tiles (at most 1024)
constexpr uint64_t kExchangeShareBytes = 512 * 64 * 4;   // a sharer's partial sums: 64 floats a lane
static_assert(kBlockLdsBytes <= 160 * 1024, "one workgroup per compute unit");
static_assert(8 * 64 * kOutRowBytes <= kWordBase, "the results leave through the idle x stages");

typedef __attribute__((ext_vector_type(4))) short bf16x4_bits;
constexpr float kNibbleOffset = 16.0f;   // nibbles enter the matrix unit as 16 + nibble

// eight nibbles of `word` -> the eight bf16 numbers 16 + nibble, low nibble first
__device__ __forceinline__ u32x4 offset_nibbles(uint32_t word) {
    // byte i of `even` = 0x80 | nibble 2 i << 3, of `odd` the same for nibble 2 i + 1: the
    // low byte of the bf16 pattern 0x4180 | nibble << 3
    const uint32_t even = ((word << 3) & 0x78787878u) | 0x80808080u;
    const uint32_t odd = ((word >> 1) & 0x78787878u) | 0x80808080u;
    u32x4 out;
    out[0] = __builtin_amdgcn_perm(odd, even, 0x0C040C00u) | 0x41004100u;
    out[1] = __builtin_amdgcn_perm(odd, even, 0x0C050C01u) | 0x41004100u;
    out[2] = __builtin_amdgcn_perm(odd, even, 0x0C060C02u) | 0x41004100u;
    out[3] = __builtin_amdgcn_perm(odd, even, 0x0C070C03u) | 0x41004100u;
    return out;
}

__device__ __forceinline__ uint16_t truncate16(float v) {
    return static_cast<uint16_t>(__float_as_uint(v) >> 16);
}

// Global memory -> LDS without passing through registers: lane l's 16 bytes at base +
// offset land at lds_address + 16 l.  Issued as assembly so that the only waits are the
// ones written below; M0 is used for nothing else in this kernel.
__device__ __forceinline__ void transfer_to_lds(const uint8_t* base, uint32_t offset,
                                                uint32_t lds_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(offset), "s"(base)
                 : "memory");
}

// the same at an address of the lane's own
__device__ __forceinline__ void transfer_piece_to_lds(const void* address, uint32_t lds_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(address)
                 : "memory");
}

// the same for 4 bytes per lane at an address of the lane's own: lands at lds_address + 4 l
__device__ __forceinline__ void transfer_dword_to_lds(const void* address, uint32_t lds_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(address)
                 : "memory");
}

__global__ __launch_bounds__(kBlockThreads) void q4_block_kernel(Q4Projection p) {
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t t = threadIdx.x;
    const uint32_t lane = t & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t i16 = lane & 15, g = lane >> 4;
    const uint32_t out_rows = p.first_row[p.segments];
    // tiles in rounds of one per compute unit, n fastest; those of the last, partly filled
    // round are shared: `sharers` workgroups each take a slice of K (whole windows of eight
    // groups) and the last to finish adds the others' sums to its own
    const uint32_t shared = blockIdx.x >= p.whole_tiles;
    const uint32_t beyond = shared ? blockIdx.x - p.whole_tiles : 0;
    const uint32_t tile_index = shared ? p.whole_tiles + beyond / p.sharers : blockIdx.x;
    const uint32_t sharers = shared ? p.sharers : 1;
    const uint32_t share = shared ? beyond % p.sharers : 0;
    const uint32_t n0 = (tile_index % p.tiles_n) * kBlockN, m0 = (tile_index / p.tiles_n) * kBlockM;
    const uint32_t all_groups = p.k_size / kQ4Group;
    const uint32_t first_group = all_groups / sharers * share;   // a multiple of 8
    const uint32_t groups = first_group + all_groups / sharers;   // this workgroup's end
    const uint32_t lds_base = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)lds));
    // multiply role: the waves form two sets of four, the two waves that share a SIMD in
    // different sets (waves w and w + 4, as a workgroup's waves are dealt to the SIMDs in
    // turn); wave (mq, nh) owns m in [64 mq, +64), n in [64 nh, +64) of the tile
    const uint32_t second_set = wave >> 2;
    const uint32_t nh = wave & 1, mq = 2 * second_set + ((wave >> 1) & 1);

    // which weight matrix a global output row lives in
    auto locate = [&](uint32_t n, const uint32_t*& words, const uint16_t*& scales,
                      const uint16_t*& biases) {
        uint32_t segment = 0;
        while (segment + 1 < p.segments && n >= p.first_row[segment + 1]) ++segment;
        const uint64_t local = n - p.first_row[segment];
        words = p.words[segment] + local * (p.k_size / 8);
        scales = p.scales[segment] + local * all_groups;
        biases = p.biases[segment] + local * all_groups;
    };

    // ---- staging roles
    // x: transfer j of wave w fills rows 32 w + 8 j .. + 7; lane l lands in row + (l >> 3),
    // slot l & 7, so it fetches piece (l & 7) ^ (l >> 3) of that row
    const uint8_t* x_base = reinterpret_cast<const uint8_t*>(p.input);
    uint32_t x_offset[4];
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const uint32_t row = min(m0 + 32 * wave + 8 * j + (lane >> 3), p.rows - 1);
        x_offset[j] = static_cast<uint32_t>(row * p.input_stride * 2) + (((lane & 7) ^ (lane >> 3)) * 16);
    }
    // words: one transfer of wave w per pair of groups fills rows 16 w .. 16 w + 15 with the
    // sixteen words of the pair (lane l: piece l & 3 of row l >> 2); the same wave unpacks
    // them (lane l: words 2 (l & 3), 2 (l & 3) + 1 of a group of row l >> 2), so its own wait
    // covers them
    const uint32_t* word_source;
    {
        const uint16_t *unused_scales, *unused_bias;
        locate(min(n0 + 16 * wave + (lane >> 2), out_rows - 1), word_source, unused_scales, unused_bias);
        word_source += 4 * (lane & 3);
    }
    // scales and biases: one 4-byte transfer each per window of eight groups and wave, for a
    // quarter of the rows of the wave's n half (lane l: groups 2 (l & 3), 2 (l & 3) + 1 of
    // the window, row l >> 2 of the quarter); the other quarters come from the other three
    // waves of the half, and two barriers pass between a window's arrival and its first use
    const uint16_t *scale_source, *bias_source;
    {
        const uint32_t* unused_words;
        locate(min(n0 + 64 * nh + 16 * (wave >> 1) + (lane >> 2), out_rows - 1), unused_words,
               scale_source, bias_source);
        scale_source += 2 * (lane & 3);
        bias_source += 2 * (lane & 3);
    }
    const uint32_t q_row = t >> 2, q_quarter = t & 3;
    const uint32_t q_slot0 = q_row * kRowBytes + (((2 * q_quarter) ^ (q_row & 7)) * 16);
    const uint32_t q_slot1 = q_row * kRowBytes + (((2 * q_quarter + 1) ^ (q_row & 7)) * 16);

    auto request = [&](uint32_t group) {
        const uint32_t stage = lds_base + (group % kStages) * kXStageBytes;
        const uint8_t* x_group = x_base + group * kRowBytes;   // uniform: scalar arithmetic
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            transfer_to_lds(x_group, x_offset[j], stage + (32 * wave + 8 * j) * kRowBytes);
        }
        if ((group & 1) == 0) {
            transfer_piece_to_lds(word_source + group * 8,
                                  lds_base + kWordBase + ((group >> 1) & 1) * kWordPairBytes +
                                      16 * wave * 64);
        }
        if ((group & 7) == 0) {
            const uint32_t window = lds_base + kMetaBase + ((group >> 3) & 1) * kMetaWindowBytes +
                                    (64 * nh + 16 * (wave >> 1)) * 16;
            transfer_dword_to_lds(scale_source + group, window);
            transfer_dword_to_lds(bias_source + group, window + kMetaKindBytes);
        }
    };
    // the nibble words of `group` that this lane unpacks
    auto read_words = [&](uint32_t group) {
        return *reinterpret_cast<const u32x2*>(lds + kWordBase + ((group >> 1) & 1) * kWordPairBytes +
                                               q_row * 64 + (group & 1) * 32 + q_quarter * 8);
    };
    auto commit = [&](uint32_t group, u32x2 words) {
        uint8_t* stage = lds + kQBase + (group & 1) * kQStageBytes;
        *reinterpret_cast<u32x4*>(stage + q_slot0) = offset_nibbles(words[0]);
        *reinterpret_cast<u32x4*>(stage + q_slot1) = offset_nibbles(words[1]);
    };

    // ---- multiply role: in a 16 x 16 result the lane holds m = 4 g .. 4 g + 3 of column n = i16
    // fragment of (row, 32-column step): piece 4 step + g, stored at slot piece ^ (row & 7)
    const uint32_t piece_offset[2] = {((g ^ (i16 & 7)) * 16), (((4 + g) ^ (i16 & 7)) * 16)};
    const uint32_t x_frag = (64 * mq + i16) * kRowBytes;
    const uint32_t q_frag = (64 * nh + i16) * kRowBytes;
    uint16_t* group_sums = reinterpret_cast<uint16_t*>(lds + kGroupSumBase);
    f32x4 acc[4][4];
#pragma unroll
    for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
        for (uint32_t tm = 0; tm < 4; ++tm) acc[tn][tm] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    bf16x8 ones;
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) ones[e] = static_cast<__bf16>(1.0f);
    const f32x4 zero = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // sum_g (bias[n][g] - 16 scale[n][g]) xs[m][g] over the four groups that start at
    // `first_group`: one MFMA per tile with the sixteen slots {hi, lo, hi, lo} of the sums
    // against {bias, bias, -16 scale, -16 scale}
    bf16x4_bits affine_weights[4], affine_sums[4];
    auto read_affine_terms = [&](uint32_t first_group) __attribute__((always_inline)) {
        const uint8_t* meta = lds + kMetaBase + ((first_group >> 3) & 1) * kMetaWindowBytes +
                              (1 - (g >> 1)) * kMetaKindBytes + (first_group & 4) * 2;
        // lanes g = 0, 1 carry the biases (which sit after the scales), g = 2, 3 the scales
        const float factor = (g >> 1) ? -kNibbleOffset : 1.0f;
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
            const uint32_t row = 64 * nh + 16 * tn + i16;
            const u32x2 pairs = *reinterpret_cast<const u32x2*>(meta + row * 16);
            u32x2 bits;
#pragma unroll
            for (uint32_t j = 0; j < 2; ++j) {
                const uint32_t pair = pairs[j];
                // times 1 or times -16: exact in bf16
                const float low = factor * __uint_as_float(pair << 16);
                const float high = factor * __uint_as_float(pair & 0xFFFF0000u);
                bits[j] = (__float_as_uint(low) >> 16) | (__float_as_uint(high) & 0xFFFF0000u);
            }
            affine_weights[tn] = __builtin_bit_cast(bf16x4_bits, bits);
        }
        const uint16_t* sums_window = group_sums + ((first_group >> 2) & 1) * (kBlockM * 8);
#pragma unroll
        for (uint32_t tm = 0; tm < 4; ++tm) {
            affine_sums[tm] = *reinterpret_cast<const bf16x4_bits*>(
                sums_window + (64 * mq + 16 * tm + i16) * 8 + 4 * (g & 1));
        }
    };
    auto add_affine_terms = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t tm = 0; tm < 4; ++tm) {
#pragma unroll
            for (uint32_t tn = 0; tn < 4; ++tn) {
                acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
                    affine_sums[tm], affine_weights[tn], acc[tn][tm], 0, 0, 0);
            }
        }
    };

    // The two sets alternate: while one multiplies group g from registers (the matrix
    // unit), the other does everything else of its group - requests the transfers of two
    // groups ahead, reads its fragments from LDS, unpacks its share of the next group's
    // nibbles - and a barrier separates the slots.  The second set runs one slot behind the
    // first.  In the slot of its `fetch (g)` a wave
    //   * waits for the transfers it requested in its fetch (g - 1): group g + 1,
    //   * reads the fragments of group g: x (g) has landed and the nibbles of g are unpacked,
    //     because every wave waited for its transfers of g and unpacked its share in its
    //     fetch (g - 1), one or two slots ago,
    //   * requests group g + 2 into the x stage that both sets read in their fetch (g - 1),
    //   * unpacks its share of the nibbles of group g + 1 into the unpacked stage that both
    //     sets read in their fetch (g - 1).
    // The group sums are exchanged between the two waves of an m quarter, which belong to
    // the same set; a window of scales and biases arrives two barriers before its first use.
    bf16x8 xf[4][2], qf[4][2];
    float scale[4];
    auto fetch = [&](uint32_t group) __attribute__((always_inline)) {
        // the transfers this wave requested in its last fetch (group g + 1) have landed
        __builtin_amdgcn_s_waitcnt(0x0F70);
        u32x2 words;
        if (group + 1 < groups) words = read_words(group + 1);   // first, to have them first
        const uint8_t* stage = lds + (group % kStages) * kXStageBytes;
        const uint8_t* q_stage = lds + kQBase + (group & 1) * kQStageBytes;
#pragma unroll
        for (uint32_t tile = 0; tile < 4; ++tile) {
#pragma unroll
            for (uint32_t step = 0; step < 2; ++step) {
                xf[tile][step] = *reinterpret_cast<const bf16x8*>(
                    stage + x_frag + tile * 16 * kRowBytes + piece_offset[step]);
                qf[tile][step] = *reinterpret_cast<const bf16x8*>(
                    q_stage + q_frag + tile * 16 * kRowBytes + piece_offset[step]);
            }
        }
        // everything else the multiply reads from LDS, so that the multiply reads nothing:
        // the group's scales and, every fourth group, the affine terms of the four before
        const uint8_t* scale_pairs = lds + kMetaBase + ((group >> 3) & 1) * kMetaWindowBytes +
                                     ((group >> 1) & 3) * 4;
        // bytes {0, 1} (even group) or {2, 3} (odd group) of a pair into the upper half, zeros below
        const uint32_t pick = (group & 1) ? 0x03020C0Cu : 0x01000C0Cu;
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
            scale[tn] = __uint_as_float(__builtin_amdgcn_perm(
                0u, *reinterpret_cast<const uint32_t*>(scale_pairs + (64 * nh + 16 * tn + i16) * 16), pick));
        }
        if ((group & 3) == 0 && group != first_group) read_affine_terms(group - 4);
        // the transfers overlap the reads above; they go into the x stage that both sets read
        // in their fetch (g - 1)
        if (group + 2 < groups) request(group + 2);
        if (group + 1 < groups) commit(group + 1, words);
    };
    auto multiply = [&](uint32_t group) __attribute__((always_inline)) {
        __builtin_amdgcn_s_setprio(1);
        // the four groups before this one are complete since this set's last multiply
        if ((group & 3) == 0 && group != first_group) add_affine_terms();
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
            for (uint32_t tm = 0; tm < 4; ++tm) {
                f32x4 part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[tm][0], qf[tn][0], zero, 0, 0, 0);
                part = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xf[tm][1], qf[tn][1], part, 0, 0, 0);
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) acc[tn][tm][j] = fmaf(scale[tn], part[j], acc[tn][tm][j]);
            }
        }
        // issue order: the scale FMAs of a tile go into the shadow of the MFMAs two tiles on
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
#pragma unroll
        for (uint32_t tile = 0; tile < 14; ++tile) {
            __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);
        // the FMAs belong to this block: left to itself the compiler sinks all 64 behind the
        // group sums, where nothing overlaps them
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
            for (uint32_t tm = 0; tm < 4; ++tm) asm volatile("" : "+v"(acc[tn][tm]));
        }
        // group sums of two of this wave's four m tiles (the other n half takes the others):
        // every row of the result is the sum; lanes g = 0, 2 store hi, lanes g = 1, 3 lo (the
        // same value to the same place twice, so that no lane has to be switched off)
        uint16_t* sum_slot = group_sums + ((group >> 2) & 1) * (kBlockM * 8) + (64 * mq + i16) * 8 +
                             4 * (g & 1) + (group & 3);
#pragma unroll
        for (uint32_t tm = 0; tm < 4; ++tm) {
            if ((tm >> 1) != nh) continue;   // wave-uniform; keeps the fragment index static
            f32x4 sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xf[tm][0], zero, 0, 0, 0);
            sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, xf[tm][1], sum, 0, 0, 0);
            const float hi = __uint_as_float(__float_as_uint(sum[0]) & 0xFFFF0000u);
            sum_slot[16 * tm * 8] = truncate16((g & 1) ? sum[0] - hi : hi);
        }
        __builtin_amdgcn_s_setprio(0);
    };

    request(first_group);
    request(first_group + 1);   // the group count of a share is a multiple of 8
    __builtin_amdgcn_s_waitcnt(0x0F70);
    commit(first_group, read_words(first_group));
    __syncthreads();
    // every wave passes 2 * groups + 1 barriers: the second set one before its first slot,
    // the first set one after its last
    if (second_set) __syncthreads();
    for (uint32_t group = first_group; group < groups; ++group) {
        fetch(group);
        __syncthreads();
        multiply(group);
        __syncthreads();
    }
    if (!second_set) __syncthreads();
    read_affine_terms(groups - 4);
    add_affine_terms();

    __syncthreads();   // nobody reads the stages any more (nor the sums, which the tiles do not reach)
    if (sharers > 1) {
        // Every sharer but the last to finish leaves its sums - device-scope stores of single
        // words, which go through to memory whatever an L2 holds, [value][thread] so that a
        // store instruction writes 256 contiguous bytes - waits for their acknowledgement,
        // counts itself in and goes; the one whose count comes back sharers - 1 adds the
        // others' to its own and stores the tile.  The launcher clears the counts.
        uint32_t* const arrival = reinterpret_cast<uint32_t*>(lds + kBlockLdsBytes - 16);
        float* const sums = reinterpret_cast<float*>(p.exchange + kExchangeCountBytes) +
                            static_cast<uint64_t>(beyond / p.sharers) * p.sharers * (kBlockThreads * 64);
        float* const mine = sums + static_cast<uint64_t>(share) * (kBlockThreads * 64) + t;
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
            for (uint32_t tm = 0; tm < 4; ++tm) {
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) {
                    __hip_atomic_store(reinterpret_cast<uint32_t*>(mine + ((tn * 4 + tm) * 4 + j) * kBlockThreads),
                                       __float_as_uint(acc[tn][tm][j]), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        if (t == 0) {
            *arrival = __hip_atomic_fetch_add(reinterpret_cast<uint32_t*>(p.exchange) + beyond / p.sharers, 1u,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (*arrival != sharers - 1) return;
        for (uint32_t other = 0; other < sharers; ++other) {
            if (other == share) continue;
            const float* theirs = sums + static_cast<uint64_t>(other) * (kBlockThreads * 64) + t;
#pragma unroll
            for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
                for (uint32_t tm = 0; tm < 4; ++tm) {
#pragma unroll
                    for (uint32_t j = 0; j < 4; ++j) {
                        acc[tn][tm][j] += __uint_as_float(__hip_atomic_load(
                            reinterpret_cast<const uint32_t*>(theirs + ((tn * 4 + tm) * 4 + j) * kBlockThreads),
                            __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
                    }
                }
            }
        }
        __syncthreads();   // the count has been read by every wave before the tiles reach its place
    }
    // ---- store: through a tile of the wave's own in LDS ([m][n], rows 16 B apart from a
    // multiple of 128), read back as 16-byte pieces: 128 contiguous bytes per m
    uint8_t* tile = lds + wave * 64 * kOutRowBytes;
#pragma unroll
    for (uint32_t tm = 0; tm < 4; ++tm) {
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                *reinterpret_cast<uint16_t*>(tile + (16 * tm + 4 * g + j) * kOutRowBytes +
                                             (16 * tn + i16) * 2) = store16(acc[tn][tm][j]);
            }
        }
    }
    const bool wide = ((reinterpret_cast<uintptr_t>(p.output) | (p.output_stride * 2)) & 15) == 0;
#pragma unroll
    for (uint32_t piece = lane; piece < 64 * 8; piece += 64) {
        const uint32_t row = piece >> 3, m = m0 + 64 * mq + row;
        const uint32_t n = n0 + 64 * nh + 8 * (piece & 7);
        if (m >= p.rows || n >= out_rows) continue;
        const u32x4 eight = *reinterpret_cast<const u32x4*>(tile + row * kOutRowBytes + (piece & 7) * 16);
        uint16_t* out = p.output + static_cast<uint64_t>(m) * p.output_stride + n;
        if (wide && n + 8 <= out_rows) {
            *reinterpret_cast<u32x4*>(out) = eight;
        } else {
            for (uint32_t e = 0; e < 8 && n + e < out_rows; ++e) {
                out[e] = static_cast<uint16_t>(eight[e >> 1] >> (16 * (e & 1)));
            }
        }
    }
}

// What the block kernel assumes of its operands beyond their sizes: its transfers move
// 16-byte pieces of x and of the nibble words and 4-byte pairs of scales and biases, and it
// addresses x with 32-bit byte offsets.
int32_t check_block_operands(const Q4Projection& p) {
    uintptr_t wide = reinterpret_cast<uintptr_t>(p.input), narrow = 0;
    for (uint32_t s = 0; s < p.segments; ++s) {
        wide |= reinterpret_cast<uintptr_t>(p.words[s]);
        narrow |= reinterpret_cast<uintptr_t>(p.scales[s]) | reinterpret_cast<uintptr_t>(p.biases[s]);
    }
    if ((wide & 15) != 0 || (narrow & 3) != 0 || ((p.input_stride * 2) & 15) != 0) {
        return TT_CMD_INVALID_BUFFER_OFFSET;
    }
    if (static_cast<uint64_t>(p.rows) * p.input_stride * 2 >= (1ull << 32)) {
        return TT_CMD_INVALID_DISPATCH_EXTENT;
    }
    return TT_OK;
}

__global__ void clear_counts_kernel(uint32_t* words, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) words[i] = 0;
}

// Tiles go to workgroups in rounds of one per compute unit.  A block of the reference's size
// leaves the last round partly filled - 2048 rows of the attention in-projection are 576 tiles,
// two rounds and a quarter on 256 compute units, of the out-projection 128, half a round - and
// a partly filled round costs a whole one.  Where the queue has a workspace, the tiles of that
// round are shared: 2, 4 or 8 workgroups (as many as fit the idle compute units and divide
// the windows of eight groups) take a slice of K each and exchange their sums through it.
int32_t launch_block(const Q4Projection& projection, hipStream_t stream) {
    Q4Projection p = projection;
    const uint32_t out_rows = p.first_row[p.segments];
    p.tiles_n = (out_rows + kBlockN - 1) / kBlockN;
    const uint32_t tiles = p.tiles_n * ((p.rows + kBlockM - 1) / kBlockM);
    p.whole_tiles = tiles;
    p.sharers = 1;
    p.exchange = nullptr;
    const StreamWorkspace workspace = stream_workspace(stream);
    if (workspace.base != nullptr && workspace.compute_units != 0) {
        const uint32_t units = workspace.compute_units;
        const uint32_t last_round = tiles % units;
        const uint32_t windows = p.k_size / (8 * kQ4Group);
        uint32_t sharers = 1;
        for (uint32_t s = 8; s >= 2 && last_round != 0; s >>= 1) {
            if (last_round * s <= units && windows % s == 0) {
                sharers = s;
                break;
            }
        }
        if (sharers > 1 && last_round * 4 <= kExchangeCountBytes &&
            kExchangeCountBytes + last_round * sharers * kExchangeShareBytes <= workspace.bytes) {
            p.whole_tiles = tiles - last_round;
            p.sharers = sharers;
            p.exchange = workspace.base;
            hipLaunchKernelGGL(clear_counts_kernel, dim3((last_round + 255) / 256), dim3(256), 0, stream,
                               reinterpret_cast<uint32_t*>(p.exchange), last_round);
        }
    }
    const uint32_t workgroups = p.whole_tiles + (tiles - p.whole_tiles) * p.sharers;
    hipLaunchKernelGGL(q4_block_kernel, dim3(workgroups), dim3(kBlockThreads), kBlockLdsBytes, stream, p);
    return TT_OK;
}

// ------------------------------------------------------- decode-wave kernel ---
//
// The same mathematics as the block kernel for 2..16 input rows (a decode wave), sized for
// latency: a workgroup owns 16 output rows and all input rows, its waves split K in slices
// of 512 columns (eight groups each), every operand of a slice is requested before the
// first is used, and the slices are summed through LDS in a fixed order.  Per group four
// v_mfma_f32_16x16x16_bf16 multiply the x rows with the nibbles as bf16 16 + nibble (lane g
// of a row owns the group's columns 16 g .. 16 g + 15) and four more, against a ones operand, give
// the group sums of x; then acc += scale[n] * products + bias[n] * sums in fp32.  The
// result has n along its columns, so a lane needs one scale and one bias per group, and
// reads all eight of a slice with two 16-byte loads.

// nibbles 0..3 (upper = false) or 4..7 of `word` -> the four bf16 numbers 16 + nibble: a
// nibble dropped into mantissa bits 3..6 of bf16 16.0 (0x4180), where it counts units.  The
// offset leaves the products as 16 * (sum of x) too much, which the caller takes out of the
// bias term; 16 is the smallest offset that keeps all sixteen values in one binade, and
// keeps the fp32 partial sums about three times as large as the plain ones.
template <bool upper>
__device__ __forceinline__ bf16x4_bits offset_four(uint32_t word) {
    constexpr uint32_t kBase = 0x41804180u, kLow = 0x00000078u, kHigh = 0x00780000u;
    // nibble i sits at bits 4 i .. 4 i + 3; the even one of a pair goes to bits 3..6, the
    // odd one to bits 19..22
    u32x2 out;
    if (!upper) {
        out[0] = ((word << 15) & kHigh) | (((word << 3) & kLow) | kBase);   // nibbles 0, 1
        out[1] = ((word << 7) & kHigh) | (((word >> 5) & kLow) | kBase);    // nibbles 2, 3
    } else {
        out[0] = ((word >> 1) & kHigh) | (((word >> 13) & kLow) | kBase);   // nibbles 4, 5
        out[1] = ((word >> 9) & kHigh) | (((word >> 21) & kLow) | kBase);   // nibbles 6, 7
    }
    return __builtin_bit_cast(bf16x4_bits, out);
}

// bytes between the x rows staged in LDS: 16 more than a row, so that the sixteen lanes of
// a fragment read (one row each, the same columns) fall on different banks
template <uint32_t kWaves>
constexpr uint32_t kWaveRowBytes = kWaves * 1024 + 16;

template <uint32_t kWaves, bool kNorm = false, bool kResidual = false>   // kWaves = k_size / 512
__global__ __launch_bounds__(64 * kWaves) void q4_wave_kernel(Q4Projection p) {
    // [rows][kWaveRowBytes] of x, then the waves' partial results
    extern __shared__ __align__(16) uint8_t wave_lds[];
    constexpr uint32_t kThreads = 64 * kWaves;
    constexpr uint32_t kPiecesPerRow = kWaves * 64;          // 16-byte pieces of an x row
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i16 = lane & 15, g = lane >> 4;
    const uint32_t n = blockIdx.x * 16 + i16;   // every matrix has a multiple of 16 rows
    const Q4Matrix matrix = matrix_of_row(p, blockIdx.x * 16);
    const uint64_t local = n - matrix.first_row;
    const uint32_t first_group = wave * 8;
    const uint32_t* words = matrix.words + local * (kWaves * 64) + first_group * 8 + 2 * g;
    const uint16_t* scales = matrix.scales + local * (kWaves * 8) + first_group;
    const uint16_t* biases = matrix.biases + local * (kWaves * 8) + first_group;

    // The x rows are the same for every workgroup: they come in once with coalesced 16-byte
    // loads (requested first, so that storing them does not wait for the weights) and are
    // read back from LDS as fragments; each lane loading its own 32 bytes per group from
    // global memory cost as much as streaming the weights.
    float* partial = reinterpret_cast<float*>(wave_lds + p.rows * kWaveRowBytes<kWaves>);
    u32x2 q[8];
    u32x4 scale_bits, bias_bits;
    auto request_weights = [&]() {
#pragma unroll
        for (uint32_t group = 0; group < 8; ++group) {
            q[group] = *reinterpret_cast<const u32x2*>(words + group * 8);
        }
        scale_bits = *reinterpret_cast<const u32x4*>(scales);
        bias_bits = *reinterpret_cast<const u32x4*>(biases);
    };
    if constexpr (kNorm) {
        // The rows go through the RMS norm on their way into LDS, bit for bit as the norm
        // operator does it with one thread per four values: a thread here holds eight
        // values of a row, the slices of that operator's threads 2 t and 2 t + 1, whose
        // sum is the first step of its 32-lane tree; the other four steps run over the 16
        // lanes of a row of this wave, and the sixteen sums of a row of x meet in the same
        // zero-padded 32-slot tree.
        static_assert(kWaves == 4, "one 16-byte piece of a 2048-wide row per thread");
        float* stage = partial;   // [rows][16], before the partial results need the space
        u32x4 raw[kQ4BatchRowsMax];
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < p.rows) {
                raw[r] = *reinterpret_cast<const u32x4*>(
                    p.input + static_cast<uint64_t>(r) * p.input_stride + threadIdx.x * 8);
            }
        }
        const u32x4 weight = *reinterpret_cast<const u32x4*>(p.norm_weight + threadIdx.x * 8);
        request_weights();   // in flight while the rows are normed
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < p.rows) {
                const float slices = rms_slice_squares(raw[r][0], raw[r][1]) +
                                     rms_slice_squares(raw[r][2], raw[r][3]);
                const float sixteen = row_sum(slices);
                if ((threadIdx.x & 15) == 0) stage[r * 16 + (threadIdx.x >> 4)] = sixteen;
            }
        }
        __syncthreads();
        float inverse[kQ4BatchRowsMax];
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < p.rows) {
                const float slot = (lane & 31) < 16 ? stage[r * 16 + (lane & 15)] : 0.0f;
                inverse[r] = rms_inverse(half_wave_sum(slot), kWaves * kQ4Block);
            }
        }
        __syncthreads();   // the stage is read before the partial results overwrite it
#pragma unroll
        for (uint32_t r = 0; r < kQ4BatchRowsMax; ++r) {
            if (r < p.rows) {
                u32x4 normed;
#pragma unroll
                for (uint32_t j = 0; j < 4; ++j) normed[j] = rms_scale_pair(raw[r][j], weight[j], inverse[r]);
                *reinterpret_cast<u32x4*>(wave_lds + r * kWaveRowBytes<kWaves> + threadIdx.x * 16) = normed;
            }
        }
    } else {
        for (uint32_t piece = threadIdx.x; piece < p.rows * kPiecesPerRow; piece += 4 * kThreads) {
            u32x4 staged[4];
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                const uint32_t at = min(piece + j * kThreads, p.rows * kPiecesPerRow - 1);
                staged[j] = *reinterpret_cast<const u32x4*>(
                    p.input + static_cast<uint64_t>(at / kPiecesPerRow) * p.input_stride +
                    (at % kPiecesPerRow) * 8);
            }
#pragma unroll
            for (uint32_t j = 0; j < 4; ++j) {
                const uint32_t at = min(piece + j * kThreads, p.rows * kPiecesPerRow - 1);
                *reinterpret_cast<u32x4*>(wave_lds + (at / kPiecesPerRow) * kWaveRowBytes<kWaves> +
                                          (at % kPiecesPerRow) * 16) = staged[j];
            }
        }
        request_weights();
    }
    __syncthreads();

    const uint8_t* x_row = wave_lds + min(i16, p.rows - 1) * kWaveRowBytes<kWaves> +
                           first_group * (kQ4Group * 2) + 32 * g;
    const bf16x4_bits ones = {0x3F80, 0x3F80, 0x3F80, 0x3F80};
    const f32x4 zero = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    f32x4 acc = zero;
#pragma unroll
    for (uint32_t group = 0; group < 8; ++group) {
        const u32x4 x_low = *reinterpret_cast<const u32x4*>(x_row + group * (kQ4Group * 2));
        const u32x4 x_high = *reinterpret_cast<const u32x4*>(x_row + group * (kQ4Group * 2) + 16);
        f32x4 products = zero, sums = zero;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const u32x4 half = j < 2 ? x_low : x_high;
            const u32x2 x_bits = {half[2 * (j & 1)], half[2 * (j & 1) + 1]};
            const bf16x4_bits xf = __builtin_bit_cast(bf16x4_bits, x_bits);
            const uint32_t word = q[group][j >> 1];
            const bf16x4_bits qf = (j & 1) ? offset_four<true>(word) : offset_four<false>(word);
            products = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(xf, qf, products, 0, 0, 0);
            sums = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(xf, ones, sums, 0, 0, 0);
        }
        const float scale = widen_half(scale_bits[group >> 1], group & 1);
        // scale * (products - 16 sums) + bias * sums
        const float bias = fmaf(-kNibbleOffset, scale, widen_half(bias_bits[group >> 1], group & 1));
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) acc[i] = fmaf(bias, sums[i], fmaf(scale, products[i], acc[i]));
    }
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) partial[(wave * 4 + i) * 64 + lane] = acc[i];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
        float total = partial[i * 64 + lane];
#pragma unroll
        for (uint32_t w = 1; w < kWaves; ++w) total += partial[(w * 4 + i) * 64 + lane];
        const uint32_t m = 4 * g + i;   // the result has the input rows along its rows
        if (m < p.rows) {
            uint16_t result = store16(total);
            if constexpr (kResidual) {
                // the residual sum of the step that follows (moe.metal:1-46), on the rounded projection
                const uint16_t before = p.residual[static_cast<uint64_t>(m) * p.residual_stride + n];
                result = rms_store16(rms_widen(rms_fz16(before)) + rms_widen(rms_fz16(result)));
            }
            p.output[static_cast<uint64_t>(m) * p.output_stride + n] = result;
        }
    }
}

template <uint32_t kWaves>
constexpr uint32_t wave_lds_bytes(uint32_t rows) {
    return rows * kWaveRowBytes<kWaves> + kWaves * 4 * 64 * 4;
}

int32_t launch_wave(const Q4Projection& p, hipStream_t stream) {
    const uint32_t out_rows = p.first_row[p.segments];
    switch (p.k_size / kQ4Block) {
    case 4:
        if (p.residual != nullptr) return TT_CMD_INVALID_DISPATCH_EXTENT;
        if (p.norm_weight != nullptr) {
            hipLaunchKernelGGL((q4_wave_kernel<4, true, false>), dim3(out_rows / 16), dim3(256),
                               wave_lds_bytes<4>(p.rows), stream, p);
        } else {
            hipLaunchKernelGGL((q4_wave_kernel<4>), dim3(out_rows / 16), dim3(256),
                               wave_lds_bytes<4>(p.rows), stream, p);
        }
        break;
    case 8:
        if (p.norm_weight != nullptr) return TT_CMD_INVALID_DISPATCH_EXTENT;
        if (p.residual != nullptr) {
            hipLaunchKernelGGL((q4_wave_kernel<8, false, true>), dim3(out_rows / 16), dim3(512),
                               wave_lds_bytes<8>(p.rows), stream, p);
        } else {
            hipLaunchKernelGGL((q4_wave_kernel<8>), dim3(out_rows / 16), dim3(512),
                               wave_lds_bytes<8>(p.rows), stream, p);
        }
        break;
    default: return TT_CMD_INVALID_DISPATCH_EXTENT;
    }
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
               Q4Projection& p, uint32_t k_size, uint64_t tiles, bool wave_kernel = false) {
    const uint32_t out_rows = f.out_rows();
    a.require(p.output_stride >= out_rows, TT_CMD_INVALID_BUFFER);
    a.require(grid_is(g, f.groups(), tiles, 1, f.threads, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    p.input_stride = k_size;
    p.input = a.buffer<const uint16_t>(0, static_cast<uint64_t>(p.rows) * k_size * 2);
    bind_segments(a, p, 1, f.segment_rows, f.segments, k_size);
    p.output = a.buffer<uint16_t>(
        f.out_slot, (static_cast<uint64_t>(p.rows - 1) * p.output_stride + out_rows) * 2);
    if (a.status != TT_OK) return a.status;
    // a handful of rows is a weight-streaming problem: the exact rows kernel; a block
    // is a matrix product: MFMA
    const bool block = !wave_kernel && p.rows > kQ4BatchRowsMax;
    if (block) {
        const int32_t status = check_block_operands(p);
        if (status != TT_OK) return status;
    }
    if (validate_only) return TT_OK;
    if (wave_kernel) return launch_wave(p, stream);
    return block ? launch_block(p, stream) : launch_rows(p, stream);
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
enum class WaveExtra { None, NormedInput, ResidualOutput };

int32_t project_tiled(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                      const Family& f, bool strided_output, bool wave_kernel = false,
                      WaveExtra extra = WaveExtra::None) {
    Args a(b);
    Q4Projection p{};
    p.rows = a.constant(f.out_slot + 1);
    p.output_stride = strided_output ? a.constant(f.out_slot + 2) : f.out_rows();
    p.row_tile = a.constant(f.out_slot + (strided_output ? 3 : 2));
    a.require(p.rows >= 1 && p.rows <= kMaxBatchRows && p.row_tile >= 1 &&
                  p.row_tile <= kQ4BatchRowsMax,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    // the buffer after the operator's last constant: the norm weight of the input rows, or
    // the rows the projection is added to (same row stride as the output)
    const uint32_t extra_slot = f.out_slot + (strided_output ? 4 : 3);
    if (extra == WaveExtra::NormedInput) {
        p.norm_weight = a.buffer<const uint16_t>(extra_slot, static_cast<uint64_t>(f.k_size) * 2);
    } else if (extra == WaveExtra::ResidualOutput && a.status == TT_OK) {
        p.residual_stride = p.output_stride;
        p.residual = a.buffer<const uint16_t>(
            extra_slot, (static_cast<uint64_t>(p.rows - 1) * p.residual_stride + f.out_rows()) * 2);
    }
    if (a.status != TT_OK) return a.status;
    return finish(a, g, stream, validate_only, f, p, f.k_size,
                  (p.rows + p.row_tile - 1) / p.row_tile, wave_kernel);
}

// a block of consecutive tokens: c[out+1] rows, then the input width where the
// operator takes one; grid (groups) x threads
int32_t project_block(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                      const Family& f, bool variable_width) {
    Args a(b);
    Q4Projection p{};
    p.rows = a.constant(f.out_slot + 1);
    const uint32_t k_size = variable_width ? a.constant(f.out_slot + 2) : f.k_size;
    // the two input widths of the model: hidden (2048) and the attention / value width (4096)
    a.require(p.rows >= 1 && (k_size == kHidden || k_size == kGdnValueValues),
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
// attn_project_mfma_ms, gdn_project_mfma_ms, gdn_outproj_mfma_ms (no reference counterpart):
// the bindings and grids of the _ms forms, evaluated on the matrix unit by q4_wave_kernel -
// the same mathematics in another summation order, for decode waves of several lanes.
int32_t op_attn_project_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kAttnProject, false, true);
}
int32_t op_gdn_project_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kGdnProject, false, true);
}
int32_t op_gdn_outproj_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kOutProject, true, true);
}
// attn_project_rms_mfma_ms, gdn_project_rms_mfma_ms (no reference counterpart): the _mfma_ms
// forms on rows that have not been normed yet, + b13 / b16 the norm weight [2048]: every
// workgroup norms the rows while it stages them (rms_only_ms's bits), which takes the norm
// dispatch out of a decode layer.
int32_t op_attn_project_rms_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kAttnProject, false, true, WaveExtra::NormedInput);
}
int32_t op_gdn_project_rms_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kGdnProject, false, true, WaveExtra::NormedInput);
}
// gdn_outproj_residual_mfma_ms (no reference counterpart): gdn_outproj_mfma_ms + b8 the rows
// the projection is added to, [rows][c6]: output = bf16(residual + bf16(projection)), the sum
// residual_rms would form next (moe.metal:1-46); the output may be the residual buffer itself.
int32_t op_gdn_outproj_residual_mfma_ms(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_tiled(b, g, s, v, kOutProject, true, true, WaveExtra::ResidualOutput);
}
// outproj_blk: + c5 block rows, c6 input width (prefill_step.cpp:2063-2078).
int32_t op_outproj_blk(const Bindings& b, const Grid& g, hipStream_t s, bool v) {
    return project_block(b, g, s, v, kOutProject, true);
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side table of launchers
bool prepare_q4_kernels() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(q4_block_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               kBlockLdsBytes) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_rows_kernel<4, true>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               kRowsStagedBytes) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_rows_kernel<8, true>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               kRowsStagedBytes) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_wave_kernel<4>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               wave_lds_bytes<4>(kQ4BatchRowsMax)) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_wave_kernel<8>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               wave_lds_bytes<8>(kQ4BatchRowsMax)) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_wave_kernel<4, true, false>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               wave_lds_bytes<4>(kQ4BatchRowsMax)) == hipSuccess &&
           hipFuncSetAttribute(reinterpret_cast<const void*>(q4_wave_kernel<8, false, true>),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               wave_lds_bytes<8>(kQ4BatchRowsMax)) == hipSuccess;
}

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
    {"attn_project_mfma_ms", op_attn_project_mfma_ms},
    {"gdn_project_mfma_ms", op_gdn_project_mfma_ms},
    {"gdn_outproj_mfma_ms", op_gdn_outproj_mfma_ms},
    {"attn_project_rms_mfma_ms", op_attn_project_rms_mfma_ms},
    {"gdn_project_rms_mfma_ms", op_gdn_project_rms_mfma_ms},
    {"gdn_outproj_residual_mfma_ms", op_gdn_outproj_residual_mfma_ms},
};
const uint32_t kQ4ProjectKernelCount = sizeof(kQ4ProjectKernels) / sizeof(kQ4ProjectKernels[0]);
#endif

}  // namespace tt
