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
#include <algorithm>
#include <type_traits>

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

// The same for a block of rows, sized for the matrix unit.  One persistent workgroup of
// eight waves per compute unit; a workgroup owns tiles of 256 rows x 256 outputs (128 flop
// per operand byte it fetches) and walks K in units of 64 columns, two steps of 32 each:
//   * both operands go from global memory straight into LDS (16 bytes per lane and
//     transfer, whole 128-byte lines of a row, no registers), a ring of two units of
//     64 KiB.  The transfers are issued as assembly, so that the only waits are the ones
//     written below (M0 is used for nothing else in this kernel).  A ring row is one
//     row's 128 bytes of the unit; 16-byte piece p of row r sits in slot p ^ (r & 7), with
//     which the 16-byte fragment reads of a wave (sixteen consecutive rows, one piece per
//     quarter wave) were measured free of bank conflicts.
//   * wave (mh, nq) multiplies rows [128 mh, +128) with outputs [64 nq, +64) as 8 x 4 tiles
//     of v_mfma_f32_16x16x32_bf16 (twelve fragment reads for 32 products), the weights as
//     the left operand: a lane then holds four consecutive outputs of one row per tile and
//     stores them as 8 bytes.  The fragments of a step are read into registers while the
//     step before it is multiplied; one barrier per unit.
//   * the first two units of a workgroup's next tile are requested before it converts and
//     stores the sums of this one.
// Rows and outputs past the end are clamped on the way in and not stored.
constexpr uint32_t kDenseTileM = 256;
constexpr uint32_t kDenseTileN = 256;
constexpr uint32_t kDenseThreads = 512;
constexpr uint32_t kDenseRing = 2;
constexpr uint32_t kDenseUnitColumns = 64;
constexpr uint32_t kDenseRowBytes = kDenseUnitColumns * 2;
constexpr uint32_t kDenseXUnitBytes = kDenseTileM * kDenseRowBytes;
constexpr uint32_t kDenseUnitBytes = (kDenseTileM + kDenseTileN) * kDenseRowBytes;
constexpr uint32_t kDenseLdsBytes = kDenseRing * kDenseUnitBytes;      // 131072
static_assert(kDenseLdsBytes <= 160 * 1024, "one workgroup per compute unit");

// lane l's 16 bytes at base + offset land at lds_address + 16 l
__device__ __forceinline__ void dense_transfer(const uint8_t* base, uint32_t offset,
                                               uint32_t lds_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(offset), "s"(base)
                 : "memory");
}

// two sums to a packed bf16 pair: hardware round to nearest even, then results below the
// normal range flushed to signed zero
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
__device__ __forceinline__ uint32_t dense_pack(float a, float b) {
    const uint32_t pair = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
    const uint32_t keep = ((pair & 0x00007F80u) ? 0x0000FFFFu : 0x00008000u) |
                          ((pair & 0x7F800000u) ? 0xFFFF0000u : 0x80000000u);
    return pair & keep;
}

__global__ __launch_bounds__(kDenseThreads) void dense_block_kernel(const uint16_t* input,
                                                                   const uint16_t* weights,
                                                                   uint16_t* output, uint32_t rows,
                                                                   uint32_t in_dim, uint32_t out_dim) {
    extern __shared__ __align__(16) uint8_t dense_lds[];
    const uint32_t t = threadIdx.x;
    const uint32_t lane = t & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const uint32_t i16 = lane & 15, g = lane >> 4;
    const uint32_t units = in_dim / kDenseUnitColumns;
    const uint32_t n_tiles = (out_dim + kDenseTileN - 1) / kDenseTileN;
    const uint32_t tiles = n_tiles * ((rows + kDenseTileM - 1) / kDenseTileM);
    const uint32_t lds_base = static_cast<uint32_t>(
        reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)dense_lds));
    const uint32_t nq = wave & 3, mh = wave >> 2;

    // staging roles: transfers 0..3 of wave w fill x rows 32 w + 8 j .. + 7, transfers 4..7
    // the weight rows of the same numbers; lane l lands in row + (l >> 3), slot l & 7, so it
    // fetches piece (l & 7) ^ (l >> 3) of that row
    const uint8_t* x_base = reinterpret_cast<const uint8_t*>(input);
    const uint8_t* w_base = reinterpret_cast<const uint8_t*>(weights);
    const uint32_t piece = ((lane & 7) ^ (lane >> 3)) * 16;
    const uint32_t staged_row = 32 * wave + (lane >> 3);
    const uint32_t row_bytes = in_dim * 2;
    uint32_t m_aim = 0, n_aim = 0;   // first row and output of the tile the requests go to
    // Tiles are numbered along bands of eight tile rows, down a band's columns first, so that
    // a run of consecutive numbers is a compact patch (32 of them: eight rows x four columns,
    // twelve operand panels for 32 tiles).
    const uint32_t m_tiles = (rows + kDenseTileM - 1) / kDenseTileM;
    auto place = [&](uint32_t tile, uint32_t& m0, uint32_t& n0) {
        const uint32_t band = tile / (8 * n_tiles);
        const uint32_t band_rows = min(8u, m_tiles - 8 * band);
        const uint32_t within = tile - band * 8 * n_tiles;
        m0 = (8 * band + within % band_rows) * kDenseTileM;
        n0 = (within / band_rows) * kDenseTileN;
    };
    auto aim = [&](uint32_t tile) { place(tile, m_aim, n_aim); };
    // the lane offsets are worked out per request (a handful of instructions per 64
    // products) rather than held in eight registers the products need
    auto request = [&](uint32_t unit) {
        const uint32_t place = lds_base + (unit % kDenseRing) * kDenseUnitBytes;
        const uint8_t* x_unit = x_base + unit * kDenseRowBytes;   // uniform: scalar arithmetic
        const uint8_t* w_unit = w_base + unit * kDenseRowBytes;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t offset = min(m_aim + staged_row + 8 * j, rows - 1) * row_bytes + piece;
            dense_transfer(x_unit, offset, place + (32 * wave + 8 * j) * kDenseRowBytes);
        }
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            const uint32_t offset = min(n_aim + staged_row + 8 * j, out_dim - 1) * row_bytes + piece;
            dense_transfer(w_unit, offset,
                           place + kDenseXUnitBytes + (32 * wave + 8 * j) * kDenseRowBytes);
        }
    };

    // fragment of (row, step of the unit): piece 4 step + g, stored at slot piece ^ (row & 7)
    const uint32_t frag_row = i16 * kDenseRowBytes;
    const uint32_t frag_piece[2] = {(g ^ (i16 & 7)) * 16, ((4 + g) ^ (i16 & 7)) * 16};
    const uint32_t x_frag = 128 * mh * kDenseRowBytes + frag_row;
    const uint32_t w_frag = kDenseXUnitBytes + 64 * nq * kDenseRowBytes + frag_row;
    f32x4 acc[4][8];   // [tn][tm]

    struct Fragments {
        bf16x8 x[8], w[4];
    };
    auto read_fragments = [&](uint32_t unit, uint32_t step, Fragments& f) __attribute__((always_inline)) {
        const uint8_t* place = dense_lds + (unit % kDenseRing) * kDenseUnitBytes + frag_piece[step];
#pragma unroll
        for (uint32_t tile = 0; tile < 4; ++tile) {
            f.w[tile] = *reinterpret_cast<const bf16x8*>(place + w_frag + tile * 16 * kDenseRowBytes);
        }
#pragma unroll
        for (uint32_t tile = 0; tile < 8; ++tile) {
            f.x[tile] = *reinterpret_cast<const bf16x8*>(place + x_frag + tile * 16 * kDenseRowBytes);
        }
    };
    auto multiply = [&](const Fragments& f) __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t tm = 0; tm < 8; ++tm) {
#pragma unroll
            for (uint32_t tn = 0; tn < 4; ++tn) {
                acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.w[tn], f.x[tm], acc[tn][tm],
                                                                      0, 0, 0);
            }
        }
    };
    // issue order of a slot: a read, then two products, so that the eight waves' reads are
    // spread over the slot instead of queueing at the LDS while the matrix unit waits (left
    // alone the scheduler sinks each read to the product that needs it, a slot later).  No
    // branch between the reads and the products: at a join the compiler would wait for the
    // reads first.
    auto interleave = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (uint32_t i = 0; i < 12; ++i) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    // first step of `unit` (its fragments are in `first`): read the second step's while
    // multiplying; the unit was published a slot ago, so nothing to wait for
    auto first_step = [&](uint32_t unit, const Fragments& first, Fragments& second)
                          __attribute__((always_inline)) {
        __builtin_amdgcn_sched_barrier(0);
        read_fragments(unit, 1, second);
        multiply(first);
        interleave();
    };
    // second step of `unit`: the next unit (requested a unit ago) has landed - mine, then
    // everybody's -, and nobody reads the unit before this one any more, so the unit after
    // the next goes into its place; read the next unit's first fragments while multiplying
    auto second_step = [&](uint32_t unit, const Fragments& second, Fragments& first_of_next,
                           auto with_request) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
        __syncthreads();
        if constexpr (decltype(with_request)::value) request(unit + 2);
        __builtin_amdgcn_sched_barrier(0);
        read_fragments(unit + 1, 0, first_of_next);
        multiply(second);
        interleave();
    };
    using std::bool_constant;

    // Workgroup b of the dispatch order runs on XCD b mod 8, each XCD with an L2 of its own:
    // the workgroups of an XCD (b / 8 = 0, 1, ...) take a run of consecutive tiles together,
    // the XCDs take the runs in turn - the operand panels a patch shares are then fetched into
    // one L2 once instead of into several.  (A grid that is no multiple of eight - fewer tiles
    // than compute units - takes every gridDim.x-th tile.)
    const bool by_xcd = gridDim.x % 8 == 0;
    const uint32_t per_xcd = gridDim.x / 8;
    const uint32_t stride = by_xcd ? 8 * per_xcd : gridDim.x;
    uint32_t tile = by_xcd ? (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    if (tile >= tiles) return;
    aim(tile);
    request(0);
    if (units > 1) request(1);
    while (true) {
#pragma unroll
        for (uint32_t tn = 0; tn < 4; ++tn) {
#pragma unroll
            for (uint32_t tm = 0; tm < 8; ++tm) acc[tn][tm] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        // unit 0 has landed (the second unit may be in flight; so may the stores of the tile
        // before, and reads and writes do not retire in one order: wait for everything)
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __syncthreads();
        Fragments a, b;
        read_fragments(0, 0, a);
        uint32_t unit = 0;
        for (; unit + 2 < units; ++unit) {
            first_step(unit, a, b);
            second_step(unit, b, a, bool_constant<true>{});
        }
        if (units > 1) {   // unit == units - 2
            first_step(unit, a, b);
            second_step(unit, b, a, bool_constant<false>{});
            ++unit;
        }
        first_step(unit, a, b);
        multiply(b);

        uint32_t m0, n0;
        place(tile, m0, n0);
        const uint32_t next_tile = tile + stride;
        __syncthreads();   // nobody reads the stages any more
        if (next_tile < tiles) {
            aim(next_tile);
            request(0);
            if (units > 1) request(1);
        }
        // the lane holds outputs n0 + 64 nq + 16 tn + 4 g + j of row m0 + 128 mh + 16 tm + i16
        const bool wide = ((reinterpret_cast<uintptr_t>(output) | (out_dim * 2)) & 7) == 0;
#pragma unroll
        for (uint32_t tm = 0; tm < 8; ++tm) {
            const uint32_t row = m0 + 128 * mh + 16 * tm + i16;
            if (row >= rows) continue;
            uint16_t* out_row = output + static_cast<uint64_t>(row) * out_dim;
#pragma unroll
            for (uint32_t tn = 0; tn < 4; ++tn) {
                const uint32_t n = n0 + 64 * nq + 16 * tn + 4 * g;
                if (n >= out_dim) continue;
                const f32x4 v = acc[tn][tm];
                const u32x2 four = u32x2{dense_pack(v[0], v[1]), dense_pack(v[2], v[3])};
                if (wide && n + 4 <= out_dim) {
                    *reinterpret_cast<u32x2*>(out_row + n) = four;
                } else {
                    for (uint32_t j = 0; j < 4 && n + j < out_dim; ++j) {
                        out_row[n + j] = static_cast<uint16_t>(four[j >> 1] >> (16 * (j & 1)));
                    }
                }
            }
        }
        if (next_tile >= tiles) break;
        tile = next_tile;
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

// Compute units of the current device (one workgroup of the block kernel each); recorded
// when a library is created on the device.
uint32_t g_compute_units[64] = {};
uint32_t current_device_compute_units() {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
    return g_compute_units[device] != 0 ? g_compute_units[device] : 256;
}

// Blocks of more rows than this take the LDS-staged kernel (below it a 256-row tile is
// mostly padding).
constexpr uint32_t kDenseBlockRowsFrom = 64;
// What the block kernel assumes beyond the sizes: 16-byte pieces of both operands and
// 32-bit byte offsets into them.
bool dense_block_operands_fit(const uint16_t* input, const uint16_t* weights, uint32_t rows,
                              uint32_t in_dim, uint32_t out_dim) {
    return ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(weights)) & 15) == 0 &&
           static_cast<uint64_t>(rows) * in_dim * 2 < (1ull << 32) &&
           static_cast<uint64_t>(out_dim) * in_dim * 2 < (1ull << 32);
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
    } else if (rows > kDenseBlockRowsFrom && dense_block_operands_fit(input, weights, rows, in_dim, out_dim)) {
        const uint32_t tiles = ((out_dim + kDenseTileN - 1) / kDenseTileN) *
                               ((rows + kDenseTileM - 1) / kDenseTileM);
        hipLaunchKernelGGL(dense_block_kernel, dim3(std::min(tiles, current_device_compute_units())),
                           dim3(kDenseThreads), kDenseLdsBytes, stream, input, weights, output, rows,
                           in_dim, out_dim);
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
bool prepare_stack_kernels() {
    int device = 0, units = 0;
    if (hipGetDevice(&device) == hipSuccess && device >= 0 && device < 64 &&
        hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess &&
        units > 0) {
        g_compute_units[device] = static_cast<uint32_t>(units);
    }
    return hipFuncSetAttribute(reinterpret_cast<const void*>(dense_block_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               kDenseLdsBytes) == hipSuccess;
}
#endif

}  // namespace tt
