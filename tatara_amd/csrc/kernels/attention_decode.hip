// Full-attention decode for gfx950: qk-RMSNorm + partial rotary + cache append,
// split-K flash-decode over bf16 KV lanes, and the partial-record combine with
// the sigmoid output gate.
//
// Operators registered here, with the reference kernels whose argument tables
// they accept (src/backend/metal/kernels/attention.metal):
//   attn_qk_rope (:43), attn_qk_rope_ms (:119)
//   attention_decode (:200), attention_decode_ms (:283)
//   attention_decode_scores_values_gqa8 (:674), attention_decode_combine (:1086)
//   attention_decode_scores_gqa4 (:373), attention_decode_values_gqa8 (:995)
// plus the lane-batched split path the reference lacks (it re-dispatches the
// one-lane split path per long row, src/runtime/decode_step.cpp:1249-1259):
//   attention_decode_split_ms, attention_decode_combine_ms,
// and the same layer of a token wave in two dispatches instead of three - the qk-norm and
// rotation of attn_qk_rope_ms folded into the split-K walk, the token's own key and value
// folded in and appended by the finishing dispatch:
//   attention_decode_token_ms, attention_decode_token_finish_ms.
//
// Flash-decode layout.  One workgroup = 4 wave64 = one (row, kv head, key
// range).  Each wave owns every 4th block of 32 keys and keeps an online
// softmax state for the 8 query heads of the kv group:
//   S^T[key][head] = K[key][:] . Q[head][:]   v_mfma_f32_16x16x32_bf16,
//       A = K tile read from a per-wave LDS stage that HBM fills directly
//       (global_load_lds, no registers; row pairs padded to 1056 B so the
//       16-lane operand reads spread over the banks), B = Q^T in registers.
//       MFMA columns 8..15 repeat heads 0..7.
//   O^T[dim][head] += V^T[dim][key] P^T[key][head]
//       A = V^T built in registers: each lane loads 16 B runs of 8 value rows
//       (a 16-lane group reads 256 contiguous bytes of one row) and transposes
//       8x8 with v_perm_b32; B = P^T straight from the S^T accumulators.
//       Columns 0..7 carry bf16(p), columns 8..15 carry bf16(p - bf16(p)), so
//       the probability enters the product with ~16 mantissa bits at no extra
//       MFMA cost; the two column sets are added once at the end.
// HBM traffic is the K and V rows once each (1 KiB per key per kv head); the
// arithmetic runs at a few percent of MFMA peak, so the kernel is bound by how
// many loads are in flight, not by compute.
#include "../tt_internal.h"
#include "lane_sums.h"

#include <utility>

// Split records of tt_attention_decode_lanes_static: device memory that belongs to the
// code object, one copy per GPU the library is loaded on, held until the process ends.
// In host code this name is only a handle for hipGetSymbolAddress; the device address a
// kernel may use is the one static_scratch() returns.
static __device__ __align__(256) unsigned char scratch[TT_STATIC_SCRATCH_BYTES];

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr uint32_t kD = kAttnHeadDim;
constexpr uint32_t kBlockKeys = 32;         // keys per wave iteration
constexpr uint32_t kLdsPairBytes = 1056;    // key i row | key 16+i row | 32 B pad
constexpr uint32_t kWaveLdsBytes = 16 * kLdsPairBytes;  // 16896
constexpr uint32_t kWaves = 4;
constexpr uint32_t kHeadsPerWave = kAttnHeadsPerKv / kWaves;   // heads a wave norms and finishes
// Cache policy of the K transfers and V loads: every key and value byte is used once per
// dispatch, so it is requested nontemporal (the `nt` bit; V through
// __builtin_nontemporal_load) and does not displace what the caches hold.  Measured on the
// 4 x 32768 walk: 51.9 us with the default policy, 48.3 us with it.
constexpr uint32_t kStreamOnce = 2;
constexpr uint32_t kMergeTileFloats = 20;   // 16 accumulator words of one MFMA + 4 pad
constexpr uint32_t kMergeHeadFloats = 16 * kMergeTileFloats + 4;  // 324: head stride of the merge
// Bound of the rows a state table may carry (decode_step.cpp:1007-1009).
constexpr uint32_t kMaxBatchRows = 16;

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
// round-to-nearest-even, NaN/inf truncated; matches the host conversion
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
    const uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
__device__ __forceinline__ float round_bf16(float v) {
    return bf16_bits_to_f32(f32_to_bf16_bits(v));
}
__device__ __forceinline__ float sigmoid_gate(uint16_t g) {
    return 1.0f / (1.0f + __expf(-bf16_bits_to_f32(g)));
}

// ------------------------------------------------------------ rotation angle ---

// powf(1e7f, pair / 32.0f) for pair 0..31, the rotation's inverse frequencies as the
// reference's scalar model takes them (tests/native/kernel_reference.cpp:636-676 receives the
// cosines and sines its caller derived this way), written out so that every kernel uses
// the correctly rounded values whatever the device's powf returns.
// Selected with a tree of conditional moves on the bits of `pair`: a table in memory would
// put a load from the code object's constant data at the head of every kernel that rotates.
__device__ __forceinline__ float rope_inverse_frequency(uint32_t pair) {
    float f[kAttnRopePairs] = {
        0x1p+0f,        0x1.a7a218p+0f,  0x1.5e8488p+1f,  0x1.220578p+2f,  0x1.dfeeaap+2f,  0x1.8d19ap+3f,
        0x1.489062p+4f, 0x1.0fdb4ep+5f,  0x1.c1df8p+5f,   0x1.743a94p+6f,  0x1.33fc3cp+7f,  0x1.fda8ccp+7f,
        0x1.a5b24ep+8f, 0x1.5cea5p+9f,   0x1.20b20cp+10f, 0x1.ddbcfep+10f, 0x1.8b48e2p+11f, 0x1.470fdcp+12f,
        0x1.0e9d26p+13f, 0x1.bfd102p+13f, 0x1.7286f2p+14f, 0x1.3293ccp+15f, 0x1.fb5454p+15f, 0x1.a3c4c8p+16f,
        0x1.5b51f8p+17f, 0x1.1f602ep+18f, 0x1.db8de2p+18f, 0x1.897a46p+19f, 0x1.459116p+20f, 0x1.0d607p+21f,
        0x1.bdc4eap+21f, 0x1.70d55p+22f,
    };
#pragma unroll
    for (uint32_t level = 0; level < 5; ++level) {
        const bool odd = (pair >> level) & 1u;
#pragma unroll
        for (uint32_t i = 0; i < (kAttnRopePairs >> (level + 1)); ++i) f[i] = odd ? f[2 * i + 1] : f[2 * i];
    }
    return f[0];
}

// Cosine and sine of theta = position / inverse_frequency (the fp32 quotient, as the model
// forms it).  The quadrant reduction runs in fp64 - theta reaches 2.6e5 at the deepest
// cache position, where an fp32 reduction would lose the angle - and the two polynomials on
// [-pi/4, pi/4] in fp32, a few dozen instructions where the library's sincosf spends
// hundreds on an argument of this size.  Within 2 ulp of the correctly rounded values; the
// rotated values are rounded to bf16 next.
struct RopeAngle {
    float c, s;
};
__device__ __forceinline__ RopeAngle rope_angle_of(uint32_t position, float inverse_frequency) {
    const float theta = static_cast<float>(position) / inverse_frequency;
    const double t = static_cast<double>(theta);
    const double k = rint(t * 0.63661977236758134308);
    double r = fma(-k, 1.57079632679489655800e+00, t);
    r = fma(-k, 6.12323399573676603587e-17, r);
    const float x = static_cast<float>(r);
    const float z = x * x;
    const float sine = fmaf(((-1.9515295891e-4f * z + 8.3321608736e-3f) * z - 1.6666654611e-1f) * z, x, x);
    const float cosine =
        fmaf(((2.443315711809948e-5f * z - 1.388731625493765e-3f) * z + 4.166664568298827e-2f) * z, z,
             fmaf(-0.5f, z, 1.0f));
    const uint32_t quadrant = static_cast<uint32_t>(static_cast<int32_t>(k)) & 3u;
    RopeAngle a;
    a.s = (quadrant & 1u) ? cosine : sine;
    a.c = (quadrant & 1u) ? sine : cosine;
    if (quadrant == 1u || quadrant == 2u) a.c = -a.c;
    if (quadrant >= 2u) a.s = -a.s;
    return a;
}

// ---------------------------------------------------------------- qk rope ---

struct RopeArgs {
    const uint16_t* projection;
    const uint16_t* q_weight;
    const uint16_t* k_weight;
    uint16_t* q_out;
    uint16_t* gate_out;
    uint16_t* keys;
    uint16_t* values;
    const uint32_t* table;      // per row {kv element offset, context}; null = one lane
    uint32_t context;           // position of row 0 when table is null
    uint32_t capacity;
    uint32_t projection_stride; // elements between rows
    uint32_t query_stride;
    uint32_t position_per_row;  // 1: block prefill (row r sits at context + r)
    uint32_t rows;
    uint32_t rows_per_group;    // rows one workgroup walks (1 for decode)
};

// The squares of the 64 consecutive values a wave holds (one per lane), summed as the
// reference sums them: a quad sums its four squares in order (thread q of the reference's
// 64), then the adjacent-pairs tree over the slices runs over quads (mirrors of a half row
// and of a row: a quad holds one value), rows and the halves of the wave.
__device__ __forceinline__ float wave_square_slices(float sq) {
    float slices = ((quad_lane<0>(sq) + quad_lane<1>(sq)) + quad_lane<2>(sq)) + quad_lane<3>(sq);
    slices += lane_dpp<0x141>(slices);   // row_half_mirror: the neighbouring quad
    slices += lane_dpp<0x140>(slices);   // row_mirror: the neighbouring pair of quads
    slices += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(slices), 0x401F));  // lane ^ 16
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(slices), 0)) +
           __int_as_float(__builtin_amdgcn_readlane(__float_as_int(slices), 32));
}

// grid (18, ceil(rows / rows_per_group)) x 256: one head per workgroup, one
// dimension per thread.  Sum of squares as the reference takes it: 64 slices of 4
// values summed in order, a 32-slice adjacent-pairs tree per half, then the two
// halves added (attention.metal:63-88).
__global__ __launch_bounds__(256) void attn_qk_rope_kernel(RopeArgs a) {
    __shared__ float wave_squares[4];
    const uint32_t head = blockIdx.x;
    const uint32_t d = threadIdx.x;
    const bool is_query = head < kAttnQueryHeads;
    const uint32_t local = is_query ? head : head - kAttnQueryHeads;
    const uint32_t base = is_query ? head * 2 * kD : kAttnQGateRows + local * kD;
    const float weight = bf16_bits_to_f32(is_query ? a.q_weight[d] : a.k_weight[d]);
    const uint32_t pair = d & (kAttnRopePairs - 1);
    const float inverse_frequency = rope_inverse_frequency(pair);
    const uint32_t row_end = min(a.rows, (blockIdx.y + 1) * a.rows_per_group);
    for (uint32_t row = blockIdx.y * a.rows_per_group; row < row_end; ++row) {
        uint32_t position = a.context + (a.position_per_row ? row : 0u);
        uint64_t kv_offset = 0;
        if (a.table != nullptr) {
            kv_offset = a.table[row * 4];
            position = a.table[row * 4 + 1];
        }
        if (position >= a.capacity) continue;  // a bad table row must not write outside the cache
        const uint16_t* proj = a.projection + static_cast<uint64_t>(row) * a.projection_stride;
        const float x = bf16_bits_to_f32(proj[base + d]);
        // the gate (query heads) or value (kv heads) element this thread copies through:
        // requested with x, not after the rotation
        const uint16_t copied =
            proj[is_query ? head * 2 * kD + kD + d : kAttnVRowOffset + local * kD + d];
        // the rotation's cosine and sine depend on the position only: evaluated while the
        // loads above are in flight, not after the norm
        float c = 1.0f, s = 0.0f;
        if (d < 2 * kAttnRopePairs) {
            const RopeAngle angle = rope_angle_of(position, inverse_frequency);
            c = angle.c;
            s = angle.s;
        }
        // Sum of squares in registers: a quad sums its four squares in order (thread q of the
        // reference's 64), then the adjacent-pairs tree over the 64 slices runs over quads
        // (mirrors of a half row and of a row: a quad holds one value), rows, the halves of
        // the wave, and the four waves - one value per wave through LDS, one barrier.
        const float wave_slices = wave_square_slices(x * x);
        __syncthreads();  // the previous row's readers are done with the shared values
        if ((d & 63) == 0) wave_squares[d >> 6] = wave_slices;
        __syncthreads();
        const float total = (wave_squares[0] + wave_squares[1]) + (wave_squares[2] + wave_squares[3]);
        const float inverse = 1.0f / sqrtf(total / static_cast<float>(kD) + kRmsNormEpsilon);
        // w * bf16(x * inv), the product rounded to bf16 again
        const float n = round_bf16(weight * round_bf16(x * inverse));
        // the rotation's partner dimension sits 32 lanes away in the same wave
        const float partner = __shfl_xor(n, static_cast<int>(kAttnRopePairs), 64);
        float rotated = n;
        if (d < 2 * kAttnRopePairs) {
            rotated = d < kAttnRopePairs ? fmaf(-partner, s, n * c) : fmaf(partner, s, n * c);
        }
        const uint16_t stored = f32_to_bf16_bits(rotated);
        if (is_query) {
            const uint64_t at = static_cast<uint64_t>(row) * a.query_stride + head * kD + d;
            a.q_out[at] = stored;
            a.gate_out[at] = copied;
        } else {
            const uint64_t at =
                kv_offset + (static_cast<uint64_t>(local) * a.capacity + position) * kD + d;
            a.keys[at] = stored;
            a.values[at] = copied;
        }
    }
}

// Block form for rows that are consecutive positions of one lane: a lane owns 8
// adjacent dims (16-byte loads and stores), 32 lanes a head, a wave two heads, a
// workgroup of 192 lanes six of the 18 heads; grid (3, ceil(rows / rows_per_group)).
// Same arithmetic as attn_qk_rope_kernel: a lane's two runs of four squares are the
// partials of threads 2l and 2l+1 there, and the xor butterfly is its pair tree.  The
// 32 rotation angles of a row are the same for every head: lane p of each wave
// evaluates pair p once and the eight lanes that rotate fetch theirs by shuffle.
__global__ __launch_bounds__(192) void attn_qk_rope_block_kernel(RopeArgs a) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t head = blockIdx.x * 6 + (threadIdx.x >> 5);
    const uint32_t l = threadIdx.x & 31;  // dims 8l .. 8l+7
    const bool is_query = head < kAttnQueryHeads;
    const uint32_t local = is_query ? head : head - kAttnQueryHeads;
    const uint32_t base = (is_query ? head * 2 * kD : kAttnQGateRows + local * kD) + l * 8;
    const uint32_t extra = (is_query ? head * 2 * kD + kD : kAttnVRowOffset + local * kD) + l * 8;
    float weight[8];
    {
        const u32x4 bits =
            *reinterpret_cast<const u32x4*>((is_query ? a.q_weight : a.k_weight) + l * 8);
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            weight[j] = __uint_as_float((j & 1) ? (bits[j >> 1] & 0xFFFF0000u) : (bits[j >> 1] << 16));
        }
    }
    const float inverse_frequency = rope_inverse_frequency(lane & (kAttnRopePairs - 1));
    const bool rotates = l < 2 * kAttnRopePairs / 8;
    const uint32_t row_end = min(a.rows, (blockIdx.y + 1) * a.rows_per_group);
    for (uint32_t row = blockIdx.y * a.rows_per_group; row < row_end; ++row) {
        const uint32_t position = a.context + row;
        if (position >= a.capacity) continue;
        const uint16_t* proj = a.projection + static_cast<uint64_t>(row) * a.projection_stride;
        const u32x4 xb = *reinterpret_cast<const u32x4*>(proj + base);
        const u32x4 eb = *reinterpret_cast<const u32x4*>(proj + extra);
        float x[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            x[j] = __uint_as_float((j & 1) ? (xb[j >> 1] & 0xFFFF0000u) : (xb[j >> 1] << 16));
        }
        float run0 = 0.0f, run1 = 0.0f;
#pragma unroll
        for (uint32_t j = 0; j < 4; ++j) {
            run0 += x[j] * x[j];
            run1 += x[4 + j] * x[4 + j];
        }
        float acc = run0 + run1;
        acc = row_sum(acc);
        const float total = acc + __shfl_xor(acc, 16, 64);
        const float inverse = 1.0f / sqrtf(total / static_cast<float>(kD) + kRmsNormEpsilon);
        float n[8];
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) n[j] = round_bf16(weight[j] * round_bf16(x[j] * inverse));
        // pair p = lane & 31 of this row, shared by the wave's two heads
        const RopeAngle angle = rope_angle_of(position, inverse_frequency);
        const float c = angle.c;
        const float sn = angle.s;
        u32x4 packed;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            const uint32_t pair = (l * 8 + j) & (kAttnRopePairs - 1);
            const float cj = __shfl(c, pair, 64);
            const float sj = __shfl(sn, pair, 64);
            const float partner = __shfl_xor(n[j], kAttnRopePairs / 8, 64);  // dim +-32: lane l^4
            float rotated = n[j];
            if (rotates) {
                rotated = l < kAttnRopePairs / 8 ? fmaf(-partner, sj, n[j] * cj)
                                                 : fmaf(partner, sj, n[j] * cj);
            }
            const uint32_t bits = f32_to_bf16_bits(rotated);
            if (j & 1) {
                packed[j >> 1] |= bits << 16;
            } else {
                packed[j >> 1] = bits;
            }
        }
        if (head >= kAttnQueryHeads + kAttnKvHeads) continue;
        if (is_query) {
            const uint64_t at = static_cast<uint64_t>(row) * a.query_stride + head * kD + l * 8;
            *reinterpret_cast<u32x4*>(a.q_out + at) = packed;
            *reinterpret_cast<u32x4*>(a.gate_out + at) = eb;
        } else {
            const uint64_t at = (static_cast<uint64_t>(local) * a.capacity + position) * kD + l * 8;
            *reinterpret_cast<u32x4*>(a.keys + at) = packed;
            *reinterpret_cast<u32x4*>(a.values + at) = eb;
        }
    }
}

// ------------------------------------------- norm and rotation by one wave ---

// One head of 256 values through RMS norm, weight and rotation by one wave; lane l
// receives dims l, l + 64, l + 128, l + 192 as the fp32 of the stored bf16.  Operation for
// operation attn_qk_rope_kernel: lane l's four squares are thread l's there, the same
// half-wave tree, the same rounding points, the same cosine and sine.
struct HeadLoads {
    uint32_t run[2];      // values 4 l .. 4 l + 3 (sum of squares)
    uint16_t x[4];        // values l + 64 c
    uint16_t w[4];
    uint32_t x32[4];      // the registers of load_head_untracked, narrowed by heads_landed
    uint32_t w32[4];
};
// The loads of one head for a wave (lane l: the run of values 4 l .. 4 l + 3 for the sum
// of squares, values l + 64 c and their weights), issued as assembly, which the compiler
// does not count: the caller places them itself among the requests of a kernel's first
// microsecond and waits for them with heads_landed() (left to the compiler, a wait for
// these values would also wait for every request issued behind them: it does not wait for
// part of a queue that holds LDS transfers).
__device__ __forceinline__ HeadLoads load_head_untracked(const uint16_t* x, const uint16_t* weight,
                                                         uint32_t lane) {
    HeadLoads h;
    const uint16_t* words = x + lane * 4;
    u32x2 run;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(run) : "v"(words));
    h.run[0] = run[0];
    h.run[1] = run[1];
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) {
        uint32_t xv, wv;
        asm volatile("global_load_ushort %0, %1, off" : "=v"(xv) : "v"(x + lane + 64 * c));
        asm volatile("global_load_ushort %0, %1, off" : "=v"(wv) : "v"(weight + lane + 64 * c));
        h.x32[c] = xv;
        h.w32[c] = wv;
    }
    return h;
}
// Waits for every vector memory request of the wave and ties the registers of two
// load_head_untracked to the wait.
__device__ __forceinline__ void heads_landed(HeadLoads& a, HeadLoads& b) {
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(a.run[0]), "+v"(a.run[1]), "+v"(a.x32[0]), "+v"(a.x32[1]), "+v"(a.x32[2]),
                   "+v"(a.x32[3]), "+v"(a.w32[0]), "+v"(a.w32[1]), "+v"(a.w32[2]), "+v"(a.w32[3]),
                   "+v"(b.run[0]), "+v"(b.run[1]), "+v"(b.x32[0]), "+v"(b.x32[1]), "+v"(b.x32[2]),
                   "+v"(b.x32[3]), "+v"(b.w32[0]), "+v"(b.w32[1]), "+v"(b.w32[2]), "+v"(b.w32[3]));
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) {
        a.x[c] = static_cast<uint16_t>(a.x32[c]);
        a.w[c] = static_cast<uint16_t>(a.w32[c]);
        b.x[c] = static_cast<uint16_t>(b.x32[c]);
        b.w[c] = static_cast<uint16_t>(b.w32[c]);
    }
}
// Cosine and sine of the rotation of pair (lane & 31) at `position`: the same for every
// head of a row, so a wave evaluates them once (one shared argument reduction) for all the
// heads it norms.
__device__ __forceinline__ void norm_rope_head(const HeadLoads& h, const RopeAngle& angle,
                                               uint32_t lane, float (&out)[4]) {
    float acc = 0.0f;
#pragma unroll
    for (uint32_t j = 0; j < 4; ++j) {
        const float v = __uint_as_float((j & 1) ? (h.run[j >> 1] & 0xFFFF0000u)
                                                : (h.run[j >> 1] << 16));
        acc += v * v;
    }
    acc = half_wave_sum(acc);
    const float total = acc + __shfl_xor(acc, 32, 64);
    const float inverse = 1.0f / sqrtf(total / static_cast<float>(kD) + kRmsNormEpsilon);
#pragma unroll
    for (uint32_t c = 0; c < 4; ++c) {
        out[c] = round_bf16(bf16_bits_to_f32(h.w[c]) * round_bf16(bf16_bits_to_f32(h.x[c]) * inverse));
    }
    // dims below 64 rotate: lane l holds dim l, its partner (l ^ 32) the other half of the pair
    const float n = out[0];
    const float partner = __shfl_xor(n, kAttnRopePairs, 64);
    const float rotated = lane < kAttnRopePairs ? fmaf(-partner, angle.s, n * angle.c)
                                                : fmaf(partner, angle.s, n * angle.c);
    out[0] = round_bf16(rotated);
}

// ------------------------------------------------------------ flash decode ---

struct FlashArgs {
    const uint16_t* q;          // [rows][query_stride], head-major 16 x 256 per row
    const uint16_t* gate;       // same layout (final mode only)
    const uint16_t* keys;       // pool base; row r's cache at + kv element offset
    const uint16_t* values;
    const uint32_t* table;      // per row {kv element offset, context}; null = one lane
    const uint32_t* row_list;   // optional indirection blockIdx.z -> row
    float* partials;            // [row][16][record_splits][258]
    uint16_t* out;              // [rows][query_stride] (final mode only)
    uint32_t context;           // when table is null
    uint32_t capacity;
    uint32_t part;              // keys per workgroup
    uint32_t record_splits;     // record stride per head
    uint32_t query_stride;      // elements between rows of q / gate / out
    uint64_t partial_row_floats;
    uint32_t final_mode;        // 1: one workgroup sees every key, writes bf16 output
    uint32_t long_rows_only;    // 1: rows with a single partition are skipped
    uint32_t single_partition;  // keys of one reference partition (256)
    uint32_t row_limit;         // rows the q / gate / out / table operands hold
    uint32_t interleave;        // 1: a row's workgroups take its 32-key blocks in turn
    uint32_t compact;           // 1: the splits that hold keys lead the dispatch order
    uint32_t rotate;            // != 0: a workgroup starts (its place x rotate) blocks into its range
    // rope form (flash_decode_kernel<true>): q is null, the query heads come from the
    // projection rows and are normed and rotated by the workgroup itself
    const uint16_t* projection; // [rows][projection_stride]: {q | gate} x 16, K x 2, V x 2
    const uint16_t* q_weight;
    uint32_t projection_stride;
};

// value of lane (l ^ 8) within each row of 16 lanes
__device__ __forceinline__ float dpp_row_ror8(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128, 0xF, 0xF, false));
}

__device__ __forceinline__ uint32_t pack_low(uint32_t a, uint32_t b) {
    // {a.lo16, b.lo16}
    return __builtin_amdgcn_perm(b, a, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_high(uint32_t a, uint32_t b) {
    // {a.hi16, b.hi16}
    return __builtin_amdgcn_perm(b, a, 0x07060302u);
}

// kRope: the token's query heads are taken from its projection row - normed and rotated by
// the workgroup while its first blocks of keys and values are in flight - and the walk
// covers the `context` cached keys only; the token's own key and value never pass through
// the cache here, attention_finish_kernel folds them in and appends them.
// Transfer kI of the 16 that bring a block of 32 key rows into a wave's LDS stage: rows kI
// and 16 + kI (the lanes' halves), 1 KiB.  `from` = the block's first row + the lane's place.
// The row's offset travels as the instruction's immediate (at most 4095, so two bases 4 KiB
// apart); the hardware adds the immediate to the LDS address as well, so the destination is
// given less that much.
template <uint32_t kI>
__device__ __forceinline__ void key_row_transfer(const uint8_t* from, uint8_t* stage) {
    constexpr uint32_t kImmediate = (kI & 7) * kD * 2;
    __builtin_amdgcn_global_load_lds(
        (const __attribute__((address_space(1))) void*)(from + (kI >> 3) * 8 * kD * 2),
        (__attribute__((address_space(3))) void*)(stage + kI * kLdsPairBytes - kImmediate), 16,
        kImmediate, kStreamOnce);
}
template <uint32_t... kI>
__device__ __forceinline__ void key_block_transfers(const uint8_t* from, uint8_t* stage,
                                                    std::integer_sequence<uint32_t, kI...>) {
    (key_row_transfer<kI>(from, stage), ...);
}

// kFinal: one workgroup sees every key of its (row, kv head) and writes the gated bf16
// output itself instead of a split record.
template <bool kRope, bool kFinal = false>
__global__ __launch_bounds__(kWaves * 64, 2) void flash_decode_kernel(FlashArgs a) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    // (rope form) the rotation's inverse frequency of pair lane & 31
    float inverse_frequency = 1.0f;
    if constexpr (kRope) {
        inverse_frequency = rope_inverse_frequency(threadIdx.x & (kAttnRopePairs - 1));
        // The arguments of the rope form are fetched here, with the others: left to the
        // compiler they are fetched where they are first used, behind the state table, one
        // more trip to memory before the first block of keys can be requested.
        asm volatile("" ::"s"(a.projection), "s"(a.q_weight), "s"(a.projection_stride));
    }
    // (rope form) The wave's two query heads as the projection holds them.  Requested at
    // once where the grid position names the row, next to the state table; in the compact
    // order, where the table names it, right behind the table.  Either way they are here
    // before the walk's first requests go out: requested among those, they would wait in
    // the memory system's queues behind the first blocks of every workgroup.
    HeadLoads ql[kHeadsPerWave];
    auto request_heads = [&](uint32_t of_row, uint32_t of_kvh) {
        const uint16_t* proj = a.projection + static_cast<uint64_t>(of_row) * a.projection_stride;
#pragma unroll
        for (uint32_t i = 0; i < kHeadsPerWave; ++i) {
            ql[i] = load_head_untracked(
                proj + (of_kvh * kAttnHeadsPerKv + (threadIdx.x >> 6) * kHeadsPerWave + i) * 2 * kD, a.q_weight,
                threadIdx.x & 63);
        }
    };
    if constexpr (kRope) {
        if (!a.compact) request_heads(blockIdx.z, blockIdx.y);
    }
    uint32_t split = blockIdx.x;
    uint32_t kvh = blockIdx.y;
    uint32_t row = blockIdx.z;
    uint64_t kv_offset = 0;
    uint32_t context = a.context;
    if (a.compact) {
        // The grid covers the capacity of every row, but only ceil(keys / part) splits of a row
        // hold keys.  Taken by grid position, the empty ones lie between the others in the
        // dispatch order and the ones that work end up two to a compute unit while other units
        // hold none.  Here the workgroups that work are the first of the dispatch order, row
        // after row, head after head, split after split, and the rest of the grid leaves at
        // once: lane r counts the splits of row r, a prefix sum over the rows places this
        // workgroup.  (Launched with a state table, without a row list, never in final mode.)
        const uint32_t l = threadIdx.x & 63;
        const u32x2 entry = *reinterpret_cast<const u32x2*>(a.table + min(l, gridDim.z - 1) * 4);
        uint32_t mine = 0;
        if (l < gridDim.z && entry[1] < a.capacity) {
            const uint32_t keys = kRope ? entry[1] : entry[1] + 1;
            if (!(a.long_rows_only && keys <= a.single_partition)) mine = (keys + a.part - 1) / a.part;
        }
        uint32_t through = mine;   // splits of rows 0 .. l
        through += __builtin_amdgcn_update_dpp(0, through, 0x111, 0xF, 0xF, true);   // row_shr:1
        through += __builtin_amdgcn_update_dpp(0, through, 0x112, 0xF, 0xF, true);
        through += __builtin_amdgcn_update_dpp(0, through, 0x114, 0xF, 0xF, true);
        through += __builtin_amdgcn_update_dpp(0, through, 0x118, 0xF, 0xF, true);
        const uint32_t linear = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const uint64_t passed = __ballot(l < kMaxBatchRows && kAttnKvHeads * through <= linear);
        row = __builtin_popcountll(passed);
        if (row >= gridDim.z) return;
        const uint32_t row_splits = __builtin_amdgcn_readlane(mine, row);
        const uint32_t place = linear - kAttnKvHeads * (__builtin_amdgcn_readlane(through, row) - row_splits);
        kvh = place >= row_splits ? 1u : 0u;   // two kv heads
        split = place - kvh * row_splits;
        // (the builtin returns int: without the cast an offset past 2^31 elements would be
        // sign-extended into the 64-bit address)
        kv_offset = static_cast<uint32_t>(__builtin_amdgcn_readlane(entry[0], row));
        context = static_cast<uint32_t>(__builtin_amdgcn_readlane(entry[1], row));
    } else {
        if (a.row_list != nullptr) {
            row = a.row_list[row];
            if (row >= a.row_limit) return;  // a bad list entry must not index outside the slabs
        }
        if (a.table != nullptr) {
            kv_offset = a.table[row * 4];
            context = a.table[row * 4 + 1];
        }
    }
    if (context >= a.capacity) return;  // a bad table row must not read outside the cache
    const uint32_t n = kRope ? context : context + 1;
    if (a.long_rows_only && n <= a.single_partition) return;
    const uint32_t part = kFinal ? n : a.part;
    if (split * part >= n) return;
    // The workgroup's blocks of 32 keys: block b of its own is block first_block + b *
    // block_stride of the row.  Contiguous: the keys [split * part, + part).  Interleaved: the
    // row's ceil(n / part) workgroups take the row's blocks in turn, so that at any moment
    // they read one contiguous window of the cache and all get the same number of blocks.
    const uint32_t row_blocks = (n + kBlockKeys - 1) / kBlockKeys;
    const uint32_t row_splits = (n + part - 1) / part;
    const bool interleave = a.interleave != 0 && !kFinal;
    const uint32_t first_block = interleave ? split : split * (part / kBlockKeys);
    const uint32_t block_stride = interleave ? row_splits : 1;
    const uint32_t key_end = interleave ? n : min(n, split * part + part);

    // the wave index as a scalar: block numbers, key ranges and base addresses then stay in
    // scalar registers, and a request is one instruction (scalar base + lane offset +
    // immediate) instead of a 64-bit vector address computed per request
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;

    // B operand of S^T: Q^T, column m holds head (m & 7)
    bf16x8 qreg[8];
    if constexpr (kRope) {
        if (a.compact) request_heads(row, kvh);
        heads_landed(ql[0], ql[kHeadsPerWave - 1]);
    } else {
        const uint16_t* qh = a.q + static_cast<uint64_t>(row) * a.query_stride +
                             (kvh * kAttnHeadsPerKv + (m & 7)) * kD;
#pragma unroll
        for (uint32_t kb = 0; kb < 8; ++kb) {
            qreg[kb] = __builtin_bit_cast(
                bf16x8, *reinterpret_cast<const u32x4*>(qh + kb * 32 + g * 8));
        }
    }

    const uint16_t* kbase = a.keys + kv_offset + static_cast<uint64_t>(kvh) * a.capacity * kD;
    const uint16_t* vbase = a.values + kv_offset + static_cast<uint64_t>(kvh) * a.capacity * kD;
    uint8_t* stage = lds + wave * kWaveLdsBytes;

    f32x4 o[16];
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) o[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY;
    float l_run = 0.0f;

    const uint32_t nblocks =
        interleave ? (row_blocks - split + row_splits - 1) / row_splits
                   : (key_end - first_block * kBlockKeys + kBlockKeys - 1) / kBlockKeys;
    // Rotation: the workgroup walks its own blocks starting `turn` blocks in and wraps around
    // (the online softmax does not care about the order).  Workgroups that advance in step
    // through ranges a fixed stride apart then sit at different offsets of their ranges at any
    // moment, so how the stride between ranges falls on the memory channels no longer decides
    // whether their requests of the moment spread out or pile up.
    const uint32_t turn =
        (split + kvh * 5u + row * 11u) * a.rotate % nblocks;
    auto own_block = [&](uint32_t blk) {
        const uint32_t turned = blk + turn;
        return first_block + (turned >= nblocks ? turned - nblocks : turned) * block_stride;
    };

    // K rows go from HBM straight into the wave's LDS stage (no registers): one
    // instruction lands 1 KiB contiguous in LDS, lanes 0..31 fetching key i
    // (tile 0) and lanes 32..63 key 16+i (tile 1), so the two rows sharing LDS
    // banks are never read by the same operand load.
    // A whole block of 32 keys is requested from one scalar base per eight transfers, the
    // lane's place as a 32-bit offset and the row as the instruction's immediate (which the
    // hardware adds to the LDS address as well: the destination is given less that much).
    // Only a row's last, partial block takes the path that clamps every row to the last key.
    constexpr uint32_t kRowBytes = kD * 2;
    const uint32_t key_lane_bytes = (lane >> 5) * 16 * kRowBytes + (lane & 31) * 16;
    const uint32_t value_lane_bytes = g * 4 * kRowBytes + m * 16;
    const uint8_t* key_bytes = reinterpret_cast<const uint8_t*>(kbase);
    const uint8_t* value_bytes = reinterpret_cast<const uint8_t*>(vbase);
    auto stage_keys = [&](uint32_t blk) {
        const uint32_t key0 = own_block(blk) * kBlockKeys;
        const uint32_t valid = min(kBlockKeys, key_end - key0);
        if (valid == kBlockKeys) {
            const uint8_t* base = key_bytes + static_cast<uint64_t>(key0) * kRowBytes;
            key_block_transfers(base + key_lane_bytes, stage, std::make_integer_sequence<uint32_t, 16>{});
            return;
        }
#pragma unroll 1
        for (uint32_t i = 0; i < 16; ++i) {
            const uint32_t key = min(i + (lane >> 5) * 16, valid - 1);
            const uint16_t* src = kbase + static_cast<uint64_t>(key0 + key) * kD + (lane & 31) * 8;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(src),
                (__attribute__((address_space(3))) void*)(stage + i * kLdsPairBytes),
                16, 0, kStreamOnce);
        }
    };

    // V rows: contraction slot e of lane group g is key (e>>2)*16 + g*4 + (e&3);
    // one call fetches one 128-dim half (8 x 16 B per lane)
    auto load_values = [&](u32x4 (&vhalf)[8], uint32_t blk, uint32_t hh) {
        const uint32_t key0 = own_block(blk) * kBlockKeys;
        const uint32_t valid = min(kBlockKeys, key_end - key0);
        if (valid == kBlockKeys) {
            const uint8_t* base = value_bytes + static_cast<uint64_t>(key0) * kRowBytes + hh * 256;
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) {
                vhalf[e] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                    base + (e >> 2) * 16 * kRowBytes + (e & 3) * kRowBytes + value_lane_bytes));
            }
            return;
        }
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) {
            const uint32_t key = min((e >> 2) * 16 + g * 4 + (e & 3), valid - 1);
            vhalf[e] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(
                vbase + static_cast<uint64_t>(key0 + key) * kD + hh * 128 + m * 8));
        }
    };

    // Software pipeline per wave: the K transfer of block b+1 starts as soon as
    // the S^T operand reads of block b are done, and each V half of block b+1 is
    // requested as soon as the P.V products of block b have consumed that half's
    // registers, so a wave always has its next block in flight.
    u32x4 vreg[2][8];
    if constexpr (kRope) {
        // The first block is requested by every wave, also one whose range holds no block
        // for it (it fetches the last block again), so that no branch surrounds what
        // follows.  Its keys go out first; the norm and rotation of the wave's two query
        // heads run next, while the memory system is busy with them - a wave that has
        // issued all its requests cannot issue arithmetic any sooner, and one that still has
        // requests to issue is held at them by the queues - and the values after that.
        // Q^T reaches the operand layout through 4 KiB of LDS; the barrier waits for those
        // LDS writes only, not for the transfers in flight.
        const uint32_t first = min(wave, nblocks - 1);
        stage_keys(first);
        __builtin_amdgcn_sched_barrier(0);
        __shared__ __attribute__((aligned(16))) uint16_t qs[kAttnHeadsPerKv * kD];
        const RopeAngle angle = rope_angle_of(context, inverse_frequency);
#pragma unroll
        for (uint32_t i = 0; i < kHeadsPerWave; ++i) {
            float nr[4];
            norm_rope_head(ql[i], angle, lane, nr);
#pragma unroll
            for (uint32_t c = 0; c < 4; ++c) {
                qs[(wave * kHeadsPerWave + i) * kD + lane + 64 * c] = f32_to_bf16_bits(nr[c]);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        load_values(vreg[0], first, 0);
        load_values(vreg[1], first, 1);
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (uint32_t kb = 0; kb < 8; ++kb) {
            qreg[kb] = __builtin_bit_cast(
                bf16x8, *reinterpret_cast<const u32x4*>(qs + (m & 7) * kD + kb * 32 + g * 8));
        }
    } else if (wave < nblocks) {
        stage_keys(wave);
        load_values(vreg[0], wave, 0);
        load_values(vreg[1], wave, 1);
    }
    for (uint32_t blk = wave; blk < nblocks; blk += kWaves) {
        const uint32_t valid = min(kBlockKeys, key_end - own_block(blk) * kBlockKeys);
        const bool more = blk + kWaves < nblocks;
        // every transfer issued so far (this block's K and V) has landed
        __builtin_amdgcn_s_waitcnt(0x0F70);
        __builtin_amdgcn_wave_barrier();
        f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f};
        f32x4 s1 = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (uint32_t kb = 0; kb < 8; ++kb) {
            const bf16x8 a0 = __builtin_bit_cast(
                bf16x8, *reinterpret_cast<const u32x4*>(stage + m * kLdsPairBytes +
                                                        (kb * 4 + g) * 16));
            const bf16x8 a1 = __builtin_bit_cast(
                bf16x8, *reinterpret_cast<const u32x4*>(stage + m * kLdsPairBytes + 512 +
                                                        (kb * 4 + g) * 16));
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, qreg[kb], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, qreg[kb], s1, 0, 0, 0);
        }
        // scores of keys g*4+i (s0) and 16+g*4+i (s1) for head m&7; reading the
        // accumulators also retires every LDS operand read of this block
        float sc[8];
        float block_max = -INFINITY;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) {
            sc[i] = (g * 4 + i) < valid ? s0[i] * kAttnScale : -INFINITY;
            sc[4 + i] = (16 + g * 4 + i) < valid ? s1[i] * kAttnScale : -INFINITY;
            block_max = fmaxf(block_max, fmaxf(sc[i], sc[4 + i]));
        }
        __builtin_amdgcn_wave_barrier();
        // the stage is free again: start the next block's K transfer now
        if (more) stage_keys(blk + kWaves);
        block_max = fmaxf(block_max, __shfl_xor(block_max, 16, 64));
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32, 64));
        const float m_new = fmaxf(m_run, block_max);
        const float alpha = __expf(m_run - m_new);  // 0 on the first block
        float p[8];
        float block_sum = 0.0f;
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) {
            p[e] = __expf(sc[e] - m_new);
            block_sum += p[e];
        }
        block_sum += __shfl_xor(block_sum, 16, 64);
        block_sum += __shfl_xor(block_sum, 32, 64);
        l_run = l_run * alpha + block_sum;
        m_run = m_new;
        // P^T operand: columns 0..7 the bf16 head, columns 8..15 the residual
        uint32_t pw[4];
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c) {
            float x0 = p[2 * c];
            float x1 = p[2 * c + 1];
            if (m >= 8) {
                x0 -= round_bf16(x0);
                x1 -= round_bf16(x1);
            }
            pw[c] = static_cast<uint32_t>(f32_to_bf16_bits(x0)) |
                    (static_cast<uint32_t>(f32_to_bf16_bits(x1)) << 16);
        }
        const bf16x8 pb = __builtin_bit_cast(bf16x8, u32x4{pw[0], pw[1], pw[2], pw[3]});
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) o[j] *= alpha;
        }
        // O^T += V^T P^T; MFMA j covers dims (j>>3)*128 + row*8 + (j&7)
#pragma unroll
        for (uint32_t hh = 0; hh < 2; ++hh) {
#pragma unroll
            for (uint32_t dw = 0; dw < 4; ++dw) {
                u32x4 lo, hi;
                lo.x = pack_low(vreg[hh][0][dw], vreg[hh][1][dw]);
                lo.y = pack_low(vreg[hh][2][dw], vreg[hh][3][dw]);
                lo.z = pack_low(vreg[hh][4][dw], vreg[hh][5][dw]);
                lo.w = pack_low(vreg[hh][6][dw], vreg[hh][7][dw]);
                hi.x = pack_high(vreg[hh][0][dw], vreg[hh][1][dw]);
                hi.y = pack_high(vreg[hh][2][dw], vreg[hh][3][dw]);
                hi.z = pack_high(vreg[hh][4][dw], vreg[hh][5][dw]);
                hi.w = pack_high(vreg[hh][6][dw], vreg[hh][7][dw]);
                o[hh * 8 + 2 * dw] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, lo), pb, o[hh * 8 + 2 * dw], 0, 0, 0);
                o[hh * 8 + 2 * dw + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, hi), pb, o[hh * 8 + 2 * dw + 1], 0, 0, 0);
            }
            if (more) load_values(vreg[hh], blk + kWaves, hh);
        }
    }
    // every transfer into the stage has landed before the stage is reused below
    __builtin_amdgcn_s_waitcnt(0x0F70);

    // Fold the residual columns into the head columns (lanes m and m^8, a DPP
    // rotate by 8 inside each row of 16 lanes: no LDS traffic), then stage each
    // wave's {O[8][256], max, sum} in its own LDS region for the cross-wave
    // merge.  Stage layout per head: word j*20 + g*4 + i for MFMA j, lane group
    // g, accumulator element i (one 16-byte store per MFMA per lane); head
    // stride 324 words.  Both the stores and the strided reads of the merge
    // spread over the banks.
    float* merge = reinterpret_cast<float*>(stage);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (uint32_t j = 0; j < 16; ++j) {
        f32x4 total;
#pragma unroll
        for (uint32_t i = 0; i < 4; ++i) total[i] = o[j][i] + dpp_row_ror8(o[j][i]);
        if (m < 8) {
            *reinterpret_cast<f32x4*>(merge + m * kMergeHeadFloats + j * kMergeTileFloats +
                                      g * 4) = total;
        }
    }
    if (lane < 8) {
        merge[8 * kMergeHeadFloats + lane * 2] = m_run;
        merge[8 * kMergeHeadFloats + lane * 2 + 1] = l_run;
    }
    __syncthreads();

    // Cross-wave merge: wave w finishes heads 2w and 2w+1; lane l owns output
    // dimensions l, l+64, l+128, l+192 (coalesced stores).  Dimension d sits in
    // the stage at word ((d>>7)*8 + (d&7))*20 + ((d&127)>>3).
#pragma unroll
    for (uint32_t hl = 0; hl < kHeadsPerWave; ++hl) {
        const uint32_t h = wave * kHeadsPerWave + hl;
        float scale[kWaves];
        float gmax = -INFINITY;
        float lsum[kWaves];
#pragma unroll
        for (uint32_t w = 0; w < kWaves; ++w) {
            const float* wm = reinterpret_cast<const float*>(lds + w * kWaveLdsBytes);
            scale[w] = wm[8 * kMergeHeadFloats + h * 2];
            lsum[w] = wm[8 * kMergeHeadFloats + h * 2 + 1];
            gmax = fmaxf(gmax, scale[w]);
        }
        float denom = 0.0f;
#pragma unroll
        for (uint32_t w = 0; w < kWaves; ++w) {
            scale[w] = scale[w] == -INFINITY ? 0.0f : __expf(scale[w] - gmax);
            denom = fmaf(scale[w], lsum[w], denom);
        }
        const uint32_t head = kvh * kAttnHeadsPerKv + h;
        float* record = kFinal
                            ? nullptr
                            : a.partials + static_cast<uint64_t>(row) * a.partial_row_floats +
                                  (static_cast<uint64_t>(head) * a.record_splits + split) *
                                      kAttnRecordFloats;
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c) {
            const uint32_t d = lane + 64 * c;
            const uint32_t slot = ((d >> 7) * 8 + (d & 7)) * kMergeTileFloats + ((d & 127) >> 3);
            float acc = 0.0f;
#pragma unroll
            for (uint32_t w = 0; w < kWaves; ++w) {
                const float* wm = reinterpret_cast<const float*>(lds + w * kWaveLdsBytes);
                acc = fmaf(scale[w], wm[h * kMergeHeadFloats + slot], acc);
            }
            if constexpr (kFinal) {
                const uint64_t at = static_cast<uint64_t>(row) * a.query_stride + head * kD + d;
                a.out[at] = f32_to_bf16_bits((acc / denom) * sigmoid_gate(a.gate[at]));
            } else {
                // (nontemporal: the records are read once, by another dispatch, and a
                // dispatch that ends on cached stores ends on their write-back)
                __builtin_nontemporal_store(acc, record + d);
            }
        }
        if (!kFinal && lane == 0) {
            __builtin_nontemporal_store(gmax, record + kD);
            __builtin_nontemporal_store(denom, record + kD + 1);
        }
    }
}

// ----------------------------------------------------------------- combine ---

struct CombineArgs {
    const float* partials;   // [row][16][record_splits][258]
    const uint16_t* gate;
    uint16_t* out;
    const uint32_t* table;   // per row {kv offset, context}; null: nparts is explicit
    uint32_t nparts;
    uint32_t part;
    uint32_t record_splits;
    uint32_t query_stride;
    uint64_t partial_row_floats;
    uint32_t long_rows_only;
    uint32_t single_partition;
    uint32_t capacity;       // with a table: a row whose context is not a cache position is left alone
};

// Up to kParts partitions: every load is requested before the first is used - the
// numerators of all partitions by the lane that owns dimension d, their maxima and sums
// through uniform loads, the gate - so the kernel is one round trip to memory deep instead
// of one per stage (and, on the general path, one per eight partitions).
template <uint32_t kParts>
__device__ __forceinline__ void combine_few_parts(const float* base, uint32_t nparts, uint32_t d,
                                                  const uint16_t* gate_at, uint16_t* out_at) {
    __shared__ __attribute__((aligned(16))) float part_max[kParts];
    __shared__ __attribute__((aligned(16))) float part_sum[kParts];
    float numerator[kParts];
#pragma unroll
    for (uint32_t p = 0; p < kParts; ++p) {
        numerator[p] = base[static_cast<uint64_t>(min(p, nparts - 1)) * kAttnRecordFloats + d];
    }
    if (d < kParts) {
        const float* rec = base + static_cast<uint64_t>(min(d, nparts - 1)) * kAttnRecordFloats;
        part_max[d] = d < nparts ? rec[kD] : -INFINITY;
        part_sum[d] = rec[kD + 1];
    }
    const uint16_t gate = *gate_at;
    __syncthreads();
    float gmax = -INFINITY;
#pragma unroll
    for (uint32_t p = 0; p < kParts; p += 4) {
        const f32x4 m4 = *reinterpret_cast<const f32x4*>(part_max + p);
        gmax = fmaxf(fmaxf(gmax, m4[0]), fmaxf(fmaxf(m4[1], m4[2]), m4[3]));
    }
    float acc = 0.0f, denom = 0.0f;
#pragma unroll
    for (uint32_t p = 0; p < kParts; p += 4) {
        const f32x4 m4 = *reinterpret_cast<const f32x4*>(part_max + p);
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(part_sum + p);
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            if (p + u < nparts) {
                const float w = m4[u] == -INFINITY ? 0.0f : __expf(m4[u] - gmax);
                acc = fmaf(w, numerator[p + u], acc);
                denom += w * s4[u];
            }
        }
    }
    *out_at = f32_to_bf16_bits((acc / denom) * sigmoid_gate(gate));
}

// grid (16, rows) x 256.  out = bf16((sum_p w_p num_p / sum_p w_p sum_p) * sigmoid(gate)),
// w_p = exp(max_p - max) (attention.metal:1086-1108).
__global__ __launch_bounds__(256) void attention_combine_kernel(CombineArgs a) {
    const uint32_t head = blockIdx.x;
    const uint32_t row = blockIdx.y;
    const uint32_t d = threadIdx.x;
    uint32_t nparts = a.nparts;
    if (a.table != nullptr) {
        const uint32_t context = a.table[row * 4 + 1];
        // a table row the split kernel refused (its context is not a position of the cache)
        // has no records of this launch: its output is left alone, whatever earlier launches
        // left in the record buffer and whatever the context wraps to
        if (context >= a.capacity) return;
        const uint32_t n = context + 1;
        if (a.long_rows_only && n <= a.single_partition) return;
        nparts = (n + a.part - 1) / a.part;
        if (nparts > a.record_splits) return;
    }
    const float* base = a.partials + static_cast<uint64_t>(row) * a.partial_row_floats +
                        static_cast<uint64_t>(head) * a.record_splits * kAttnRecordFloats;
    const uint64_t at = static_cast<uint64_t>(row) * a.query_stride + head * kD + d;
    // 32 partitions are a 32k context in splits of 1024 keys, 128 a 100k context in splits of
    // 800; beyond that the general path below
    if (nparts <= 32) return combine_few_parts<32>(base, nparts, d, a.gate + at, a.out + at);
    if (nparts <= 64) return combine_few_parts<64>(base, nparts, d, a.gate + at, a.out + at);
    if (nparts <= 128) return combine_few_parts<128>(base, nparts, d, a.gate + at, a.out + at);
    __shared__ float red[256];
    __shared__ float weight[256];
    __shared__ float wsum[256];
    // global maximum: partitions strided over the threads, then a block reduction
    float local = -INFINITY;
    for (uint32_t p = d; p < nparts; p += 256) {
        local = fmaxf(local, base[static_cast<uint64_t>(p) * kAttnRecordFloats + kD]);
    }
    red[d] = local;
    __syncthreads();
    for (uint32_t off = 128; off; off >>= 1) {
        if (d < off) red[d] = fmaxf(red[d], red[d + off]);
        __syncthreads();
    }
    const float gmax = red[0];
    float acc = 0.0f;
    float denom = 0.0f;
    for (uint32_t chunk = 0; chunk < nparts; chunk += 256) {
        const uint32_t count = min(256u, nparts - chunk);
        __syncthreads();
        if (d < count) {
            const float* rec = base + static_cast<uint64_t>(chunk + d) * kAttnRecordFloats;
            const float pmax = rec[kD];
            const float w = pmax == -INFINITY ? 0.0f : __expf(pmax - gmax);
            weight[d] = w;
            wsum[d] = w * rec[kD + 1];
        }
        __syncthreads();
        const float* rec = base + static_cast<uint64_t>(chunk) * kAttnRecordFloats + d;
        uint32_t p = 0;
        for (; p + 8 <= count; p += 8) {
            float v[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                v[u] = rec[static_cast<uint64_t>(p + u) * kAttnRecordFloats];
            }
#pragma unroll
            for (uint32_t u = 0; u < 8; ++u) {
                acc = fmaf(weight[p + u], v[u], acc);
                denom += wsum[p + u];
            }
        }
        for (; p < count; ++p) {
            acc = fmaf(weight[p], rec[static_cast<uint64_t>(p) * kAttnRecordFloats], acc);
            denom += wsum[p];
        }
    }
    a.out[at] = f32_to_bf16_bits((acc / denom) * sigmoid_gate(a.gate[at]));
}

// ------------------------------------------- finish of the rope-form walk ----
//
// Second dispatch of the attention layer of a token wave whose first is
// flash_decode_kernel<true>: merges the split records over the cached keys, folds in the
// token itself - its key normed and rotated here, its value row as the projection holds
// it - as one more record {numerator = V row, max = its score, sum = 1}, applies the gate
// and appends the key and value rows to the cache.  Grid (16 heads, rows) x 256, thread d
// = dimension d.  The norm and the rotation are attn_qk_rope_kernel's, operation for
// operation, so the appended key row is that kernel's bit for bit.

struct FinishArgs {
    const uint16_t* projection;   // [rows][projection_stride]: {q | gate} x 16, K x 2, V x 2
    const uint16_t* q_weight;
    const uint16_t* k_weight;
    uint16_t* keys;               // pools; row r's cache at + table[4 r] elements
    uint16_t* values;
    const uint32_t* table;        // per row {kv element offset, context, -, -}
    const float* partials;        // [row][16][record_splits][258]
    uint16_t* out;                // [rows][query_stride]
    uint32_t capacity;
    uint32_t projection_stride;
    uint32_t query_stride;
    uint32_t part;
    uint32_t record_splits;
    uint32_t parts_hint;          // records per head the caller expects the deepest row to have
    uint64_t partial_row_floats;
};

struct MergedParts {
    float acc, denom, gmax;   // sum_p w_p num_p[d], sum_p w_p sum_p, w_p = exp(max_p - gmax)
};

// Numerators of up to kParts records requested at once by the thread that owns the
// dimension; their maxima and sums go through LDS (one thread per record).  `held` = how
// many records the buffer holds from `base` on (requests beyond it repeat the last one);
// which of them count is decided in reduce_parts, so nothing here waits for the state
// table.  The caller places a barrier between request_parts and reduce_parts.
template <uint32_t kParts>
__device__ __forceinline__ void request_parts(const float* base, uint32_t held, uint32_t d,
                                              float (&numerator)[kParts], float* part_max,
                                              float* part_sum) {
    const uint32_t last = held - 1;
#pragma unroll
    for (uint32_t p = 0; p < kParts; ++p) {
        numerator[p] = base[static_cast<uint64_t>(min(p, last)) * kAttnRecordFloats + d];
    }
    if (d < kParts) {
        const float* rec = base + static_cast<uint64_t>(min(d, last)) * kAttnRecordFloats;
        part_max[d] = rec[kD];
        part_sum[d] = rec[kD + 1];
    }
}
// Merge of the first `nparts` (at most kParts) of the requested records.
template <uint32_t kParts>
__device__ __forceinline__ MergedParts reduce_parts(const float (&numerator)[kParts], uint32_t nparts,
                                                    const float* part_max, const float* part_sum) {
    MergedParts r{0.0f, 0.0f, -INFINITY};
#pragma unroll
    for (uint32_t p = 0; p < kParts; p += 4) {
        const f32x4 m4 = *reinterpret_cast<const f32x4*>(part_max + p);
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            if (p + u < nparts) r.gmax = fmaxf(r.gmax, m4[u]);
        }
    }
#pragma unroll
    for (uint32_t p = 0; p < kParts; p += 4) {
        const f32x4 m4 = *reinterpret_cast<const f32x4*>(part_max + p);
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(part_sum + p);
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            if (p + u < nparts) {
                const float w = m4[u] == -INFINITY ? 0.0f : __expf(m4[u] - r.gmax);
                r.acc = fmaf(w, numerator[p + u], r.acc);
                r.denom += w * s4[u];
            }
        }
    }
    return r;
}

// One (row, head) by one workgroup.  Every load - the state table entry, the projection
// row's four slices, the two norm weights and the first kParts records - is requested
// before the first is used: the kernel is one trip to memory deep.
template <uint32_t kParts>
__device__ __forceinline__ void finish_row_head(const FinishArgs& a, uint32_t head, uint32_t row,
                                                uint32_t d) {
    __shared__ __attribute__((aligned(16))) float part_max[kParts];
    __shared__ __attribute__((aligned(16))) float part_sum[kParts];
    __shared__ float wave_values[3][4];   // squares of the query head, of the key head, q . k
    const uint32_t kvh = head / kAttnHeadsPerKv;
    const uint16_t* proj = a.projection + static_cast<uint64_t>(row) * a.projection_stride;
    const float* base = a.partials + static_cast<uint64_t>(row) * a.partial_row_floats +
                        static_cast<uint64_t>(head) * a.record_splits * kAttnRecordFloats;
    const u32x2 entry = *reinterpret_cast<const u32x2*>(a.table + row * 4);
    const float inverse_frequency = rope_inverse_frequency(d & (kAttnRopePairs - 1));
    const uint16_t xq = proj[head * 2 * kD + d];
    const uint16_t gate = proj[head * 2 * kD + kD + d];
    const uint16_t xk = proj[kAttnQGateRows + kvh * kD + d];
    const uint16_t vraw = proj[kAttnVRowOffset + kvh * kD + d];
    const uint16_t wq = a.q_weight[d];
    const uint16_t wk = a.k_weight[d];
    float numerator[kParts];
    request_parts<kParts>(base, min(kParts, a.record_splits), d, numerator, part_max, part_sum);

    const uint64_t kv_offset = entry[0];
    const uint32_t context = entry[1];
    // a row the table places outside its cache has no records and no slot to append to
    if (context >= a.capacity) return;
    const uint32_t nparts = (context + a.part - 1) / a.part;
    if (nparts > a.record_splits) return;
    float c = 1.0f, sn = 0.0f;
    if (d < 2 * kAttnRopePairs) {
        const RopeAngle angle = rope_angle_of(context, inverse_frequency);
        c = angle.c;
        sn = angle.s;
    }
    const float fq = bf16_bits_to_f32(xq);
    const float fk = bf16_bits_to_f32(xk);
    const float q_slices = wave_square_slices(fq * fq);
    const float k_slices = wave_square_slices(fk * fk);
    if ((d & 63) == 0) {
        wave_values[0][d >> 6] = q_slices;
        wave_values[1][d >> 6] = k_slices;
    }
    __syncthreads();   // also publishes the records' maxima and sums
    const float q_total = (wave_values[0][0] + wave_values[0][1]) + (wave_values[0][2] + wave_values[0][3]);
    const float k_total = (wave_values[1][0] + wave_values[1][1]) + (wave_values[1][2] + wave_values[1][3]);
    const float q_inverse = 1.0f / sqrtf(q_total / static_cast<float>(kD) + kRmsNormEpsilon);
    const float k_inverse = 1.0f / sqrtf(k_total / static_cast<float>(kD) + kRmsNormEpsilon);
    const float nq = round_bf16(bf16_bits_to_f32(wq) * round_bf16(fq * q_inverse));
    const float nk = round_bf16(bf16_bits_to_f32(wk) * round_bf16(fk * k_inverse));
    const float q_partner = __shfl_xor(nq, static_cast<int>(kAttnRopePairs), 64);
    const float k_partner = __shfl_xor(nk, static_cast<int>(kAttnRopePairs), 64);
    float q_rotated = nq, k_rotated = nk;
    if (d < 2 * kAttnRopePairs) {
        q_rotated = d < kAttnRopePairs ? fmaf(-q_partner, sn, nq * c) : fmaf(q_partner, sn, nq * c);
        k_rotated = d < kAttnRopePairs ? fmaf(-k_partner, sn, nk * c) : fmaf(k_partner, sn, nk * c);
    }
    const uint16_t k_bits = f32_to_bf16_bits(k_rotated);
    // the token's score from the stored (bf16) query and key, as the walk scores cached keys
    float dot = round_bf16(q_rotated) * bf16_bits_to_f32(k_bits);
    dot = half_wave_sum(dot);
    dot += __shfl_xor(dot, 32, 64);
    if ((d & 63) == 0) wave_values[2][d >> 6] = dot;
    MergedParts merged = reduce_parts<kParts>(numerator, min(nparts, kParts), part_max, part_sum);
    __syncthreads();
    {
        // more records than were requested up front (a context that has grown past the
        // caller's hint, or more than 128 records): the rest in batches, merged as they come
        for (uint32_t p0 = kParts; p0 < nparts; p0 += kParts) {
            const uint32_t count = min(kParts, nparts - p0);
            request_parts<kParts>(base + static_cast<uint64_t>(p0) * kAttnRecordFloats, count, d,
                                  numerator, part_max, part_sum);
            __syncthreads();
            const MergedParts next = reduce_parts<kParts>(numerator, count, part_max, part_sum);
            __syncthreads();
            const float g = fmaxf(merged.gmax, next.gmax);
            const float w_old = merged.gmax == -INFINITY ? 0.0f : __expf(merged.gmax - g);
            const float w_next = next.gmax == -INFINITY ? 0.0f : __expf(next.gmax - g);
            merged.acc = fmaf(w_old, merged.acc, w_next * next.acc);
            merged.denom = fmaf(w_old, merged.denom, w_next * next.denom);
            merged.gmax = g;
        }
    }
    const float s_new =
        ((wave_values[2][0] + wave_values[2][1]) + (wave_values[2][2] + wave_values[2][3])) * kAttnScale;
    const float gmax = fmaxf(merged.gmax, s_new);
    const float w_parts = merged.gmax == -INFINITY ? 0.0f : __expf(merged.gmax - gmax);
    const float w_new = __expf(s_new - gmax);
    const float acc = fmaf(w_new, bf16_bits_to_f32(vraw), w_parts * merged.acc);
    const float denom = fmaf(w_parts, merged.denom, w_new);
    const uint64_t at = static_cast<uint64_t>(row) * a.query_stride + head * kD + d;
    a.out[at] = f32_to_bf16_bits((acc / denom) * sigmoid_gate(gate));
    if (head % kAttnHeadsPerKv == 0) {
        const uint64_t slot = kv_offset + (static_cast<uint64_t>(kvh) * a.capacity + context) * kD + d;
        a.keys[slot] = k_bits;
        a.values[slot] = vraw;
    }
}

// The batch of records requested up front is sized by a launch constant - how many records
// the caller expects the deepest row to have, at most what the buffer holds per head - not
// by the contexts in the state table, which arrive with the records.
__global__ __launch_bounds__(256) void attention_finish_kernel(FinishArgs a) {
    const uint32_t head = blockIdx.x;
    const uint32_t row = blockIdx.y;
    const uint32_t d = threadIdx.x;
    const uint32_t expected = min(a.parts_hint == 0 ? a.record_splits : a.parts_hint, a.record_splits);
    if (expected <= 32) return finish_row_head<32>(a, head, row, d);
    if (expected <= 64) return finish_row_head<64>(a, head, row, d);
    return finish_row_head<128>(a, head, row, d);
}

// ---------------------------------------- separate score / value stages ------

// attention_decode_scores_gqa4: one workgroup per (head, partition); thread t
// scores key t of the partition; record = {p[0..255], max, sum}
// (attention.metal:373-448).  Scalar loads; this two-stage path exists for
// argument-table compatibility, the fused split path is the fast one.
__global__ __launch_bounds__(256) void attention_scores_kernel(const uint16_t* q,
                                                               const uint16_t* keys,
                                                               uint32_t context, uint32_t capacity,
                                                               uint32_t part, float* weights,
                                                               uint32_t nparts) {
    __shared__ float red[256];
    __shared__ float qs[kD];
    const uint32_t head = blockIdx.x;
    const uint32_t partition = blockIdx.y;
    const uint32_t t = threadIdx.x;
    const uint32_t n = context + 1;
    const uint32_t start = partition * part;
    const uint32_t count = start < n ? min(n - start, part) : 0u;
    qs[t] = bf16_bits_to_f32(q[head * kD + t]);
    __syncthreads();
    float s = -INFINITY;
    if (t < count) {
        const uint16_t* k =
            keys + (static_cast<uint64_t>(head / kAttnHeadsPerKv) * capacity + start + t) * kD;
        float dot = 0.0f;
        for (uint32_t d = 0; d < kD; d += 8) {
            const u32x4 w = *reinterpret_cast<const u32x4*>(k + d);
#pragma unroll
            for (uint32_t c = 0; c < 4; ++c) {
                dot = fmaf(qs[d + 2 * c], __uint_as_float(w[c] << 16), dot);
                dot = fmaf(qs[d + 2 * c + 1], __uint_as_float(w[c] & 0xFFFF0000u), dot);
            }
        }
        s = dot * kAttnScale;
    }
    red[t] = s;
    __syncthreads();
    for (uint32_t off = 128; off; off >>= 1) {
        if (t < off) red[t] = fmaxf(red[t], red[t + off]);
        __syncthreads();
    }
    const float pmax = red[0];
    __syncthreads();
    const float p = t < count ? __expf(s - pmax) : 0.0f;
    red[t] = p;
    __syncthreads();
    for (uint32_t off = 128; off; off >>= 1) {
        if (t < off) red[t] += red[t + off];
        __syncthreads();
    }
    float* record = weights + (static_cast<uint64_t>(head) * nparts + partition) * kAttnRecordFloats;
    record[t] = p;
    if (t == 0) {
        record[kD] = pmax;
        record[kD + 1] = red[0];
    }
}

// attention_decode_values_gqa8: one workgroup per (head, partition); thread d
// accumulates sum_p w_p V[p][d] in ascending p (attention.metal:995-1036).
__global__ __launch_bounds__(256) void attention_values_kernel(const float* weights,
                                                               const uint16_t* values,
                                                               uint32_t context, uint32_t capacity,
                                                               uint32_t part, float* partials,
                                                               uint32_t nparts) {
    __shared__ float w[256];
    const uint32_t head = blockIdx.x;
    const uint32_t partition = blockIdx.y;
    const uint32_t d = threadIdx.x;
    const uint32_t n = context + 1;
    const uint32_t start = partition * part;
    const uint32_t count = start < n ? min(n - start, part) : 0u;
    const uint64_t rec = (static_cast<uint64_t>(head) * nparts + partition) * kAttnRecordFloats;
    w[d] = weights[rec + d];
    __syncthreads();
    const uint16_t* v =
        values + (static_cast<uint64_t>(head / kAttnHeadsPerKv) * capacity + start) * kD + d;
    float acc = 0.0f;
    for (uint32_t p = 0; p < count; ++p) {
        acc = fmaf(w[p], bf16_bits_to_f32(v[static_cast<uint64_t>(p) * kD]), acc);
    }
    partials[rec + d] = acc;
    if (d == 0) {
        partials[rec + kD] = weights[rec + kD];
        partials[rec + kD + 1] = weights[rec + kD + 1];
    }
}

// ---------------------------------------------------------------- launchers --

constexpr uint64_t kQueryBytes = kAttnQueryValues * 2;

uint64_t cache_bytes(uint32_t capacity) {
    return static_cast<uint64_t>(kAttnKvHeads) * capacity * kD * 2;
}

int32_t launch_rope(const RopeArgs& args, uint32_t rows, hipStream_t stream) {
    RopeArgs r = args;
    r.rows = rows;
    r.rows_per_group = r.position_per_row ? 8u : 1u;  // blocks walk 8 rows per workgroup
    const uint32_t groups = (rows + r.rows_per_group - 1) / r.rows_per_group;
    if (r.position_per_row && r.table == nullptr && r.projection_stride % 8 == 0 &&
        r.query_stride % 8 == 0) {
        hipLaunchKernelGGL(attn_qk_rope_block_kernel, dim3(3, groups), dim3(192), 0, stream, r);
        return TT_OK;
    }
    hipLaunchKernelGGL(attn_qk_rope_kernel, dim3(kAttnQueryHeads + kAttnKvHeads, groups),
                       dim3(256), 0, stream, r);
    return TT_OK;
}

// attn_qk_rope: b0 projection, b1 q_w, b2 k_w, b3 q, b4 gate, b5 keys, b6 values,
// c7 context, c8 capacity; grid 18 x 256 (decode_step.cpp:713-723).
int32_t op_attn_qk_rope(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only) {
    Args a(b);
    RopeArgs r{};
    r.context = a.constant(7);
    r.capacity = a.constant(8);
    a.require(context_ok(r.context, r.capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    r.projection = a.buffer<const uint16_t>(0, kAttnProjectionRows * 2);
    r.q_weight = a.buffer<const uint16_t>(1, kD * 2);
    r.k_weight = a.buffer<const uint16_t>(2, kD * 2);
    r.q_out = a.buffer<uint16_t>(3, kQueryBytes);
    r.gate_out = a.buffer<uint16_t>(4, kQueryBytes);
    r.keys = a.buffer<uint16_t>(5, cache_bytes(r.capacity));
    r.values = a.buffer<uint16_t>(6, cache_bytes(r.capacity));
    r.projection_stride = kAttnProjectionRows;
    r.query_stride = kAttnQueryValues;
    a.require(grid_is(g, 18, 1, 1, 256, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_rope(r, 1, stream);
}

// attn_qk_rope_ms: b0 projection slab, b1 q_w, b2 k_w, b3 q slab, b4 gate slab,
// b5 keys_pool, b6 values_pool, c7 capacity, b8 state_table, c9 projection
// stride, c10 query stride; grid (18, rows) x 256 (decode_step.cpp:1231-1243).
// The per-row kv offsets and contexts live in device memory, so pool extents
// cannot be checked here; the runtime that writes the table guarantees
// offset + cache <= pool and context < capacity (decode_step.cpp:1022-1062).
int32_t op_attn_qk_rope_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                           bool validate_only) {
    Args a(b);
    RopeArgs r{};
    r.capacity = a.constant(7);
    r.projection_stride = a.constant(9);
    r.query_stride = a.constant(10);
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    a.require(g.gx == 18 && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1 && rows >= 1 &&
                  rows <= kMaxBatchRows,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(r.capacity != 0 && r.projection_stride >= kAttnProjectionRows &&
                  r.query_stride >= kAttnQueryValues,
              TT_CMD_INVALID_BUFFER);
    const uint64_t last = rows - 1;
    r.projection = a.buffer<const uint16_t>(0, (last * r.projection_stride + kAttnProjectionRows) * 2);
    r.q_weight = a.buffer<const uint16_t>(1, kD * 2);
    r.k_weight = a.buffer<const uint16_t>(2, kD * 2);
    r.q_out = a.buffer<uint16_t>(3, (last * r.query_stride + kAttnQueryValues) * 2);
    r.gate_out = a.buffer<uint16_t>(4, (last * r.query_stride + kAttnQueryValues) * 2);
    r.keys = a.buffer<uint16_t>(5, cache_bytes(r.capacity));
    r.values = a.buffer<uint16_t>(6, cache_bytes(r.capacity));
    r.table = a.buffer<const uint32_t>(8, rows * 16);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_rope(r, rows, stream);
}

}  // namespace

// attn_qk_rope_blk: b0 projection[rows][9216], b1 q_w, b2 k_w, b3 query[rows][16][256],
// b4 gate[rows][16][256], b5 keys, b6 values, c7 context of row 0, c8 capacity;
// grid (18, rows) x 256 (prefill_step.cpp:1450-1465; prefill_attention.metal:1-92).
int32_t op_attn_qk_rope_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only) {
    Args a(b);
    RopeArgs r{};
    r.context = a.constant(7);
    r.capacity = a.constant(8);
    const uint64_t rows = g.gy;
    a.require(g.gx == 18 && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1 && rows >= 1 &&
                  rows <= 65535,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(r.capacity != 0 && static_cast<uint64_t>(r.context) + rows <= r.capacity,
              TT_CMD_CONTEXT_OUT_OF_RANGE);
    r.projection = a.buffer<const uint16_t>(0, rows * kAttnProjectionRows * 2);
    r.q_weight = a.buffer<const uint16_t>(1, kD * 2);
    r.k_weight = a.buffer<const uint16_t>(2, kD * 2);
    r.q_out = a.buffer<uint16_t>(3, rows * kQueryBytes);
    r.gate_out = a.buffer<uint16_t>(4, rows * kQueryBytes);
    r.keys = a.buffer<uint16_t>(5, cache_bytes(r.capacity));
    r.values = a.buffer<uint16_t>(6, cache_bytes(r.capacity));
    r.projection_stride = kAttnProjectionRows;
    r.query_stride = kAttnQueryValues;
    r.position_per_row = 1;
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_rope(r, static_cast<uint32_t>(rows), stream);
}

namespace {

int32_t launch_flash(const FlashArgs& f, uint32_t splits, uint32_t rows, hipStream_t stream) {
    if (f.projection != nullptr) {
        hipLaunchKernelGGL(flash_decode_kernel<true>, dim3(splits, kAttnKvHeads, rows), dim3(kWaves * 64),
                           kWaves * kWaveLdsBytes, stream, f);
    } else if (f.final_mode) {
        hipLaunchKernelGGL((flash_decode_kernel<false, true>), dim3(splits, kAttnKvHeads, rows),
                           dim3(kWaves * 64), kWaves * kWaveLdsBytes, stream, f);
    } else {
        hipLaunchKernelGGL(flash_decode_kernel<false>, dim3(splits, kAttnKvHeads, rows), dim3(kWaves * 64),
                           kWaves * kWaveLdsBytes, stream, f);
    }
    return TT_OK;
}

// attention_decode: b0 q, b1 gate, b2 keys, b3 values, c4 context, b5 out,
// c6 capacity; grid 16 x 256 (decode_step.cpp:239-247).  Any context.
int32_t op_attention_decode(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only) {
    Args a(b);
    FlashArgs f{};
    f.context = a.constant(4);
    f.capacity = a.constant(6);
    a.require(context_ok(f.context, f.capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    f.q = a.buffer<const uint16_t>(0, kQueryBytes);
    f.gate = a.buffer<const uint16_t>(1, kQueryBytes);
    f.keys = a.buffer<const uint16_t>(2, cache_bytes(f.capacity));
    f.values = a.buffer<const uint16_t>(3, cache_bytes(f.capacity));
    f.out = a.buffer<uint16_t>(5, kQueryBytes);
    f.query_stride = kAttnQueryValues;
    f.final_mode = 1;
    a.require(grid_is(g, 16, 1, 1, 256, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_flash(f, 1, 1, stream);
}

// attention_decode_ms: b0 q slab, b1 gate slab, b2 keys_pool, b3 values_pool,
// b4 state_table, b5 out slab, c6 capacity, b7 bucket_rows, c8 query stride;
// grid (16, bucket_rows) x 256 (decode_step.cpp:1261-1272).
int32_t op_attention_decode_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                               bool validate_only) {
    Args a(b);
    FlashArgs f{};
    f.capacity = a.constant(6);
    f.query_stride = a.constant(8);
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    a.require(g.gx == 16 && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1 && rows >= 1 &&
                  rows <= kMaxBatchRows,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(f.capacity != 0 && f.query_stride >= kAttnQueryValues, TT_CMD_INVALID_BUFFER);
    f.q = a.buffer<const uint16_t>(0, kQueryBytes);
    f.gate = a.buffer<const uint16_t>(1, kQueryBytes);
    f.keys = a.buffer<const uint16_t>(2, cache_bytes(f.capacity));
    f.values = a.buffer<const uint16_t>(3, cache_bytes(f.capacity));
    f.table = a.buffer<const uint32_t>(4, kMaxBatchRows * 16);
    f.out = a.buffer<uint16_t>(5, kQueryBytes);
    f.row_list = a.buffer<const uint32_t>(7, rows * 4);
    f.final_mode = 1;
    // The row indices come from device memory: the kernel skips any that the smallest of
    // the three slabs does not hold, so a stale list entry cannot reach outside them.
    if (a.status == TT_OK) {
        uint64_t held = kMaxBatchRows;
        for (uint32_t index : {0u, 1u, 5u}) {
            const uint64_t values = a.buffer_bytes(index) / 2;
            held = std::min<uint64_t>(held, (values - kAttnQueryValues) / f.query_stride + 1);
        }
        f.row_limit = static_cast<uint32_t>(held);
        a.require(rows <= f.row_limit, TT_CMD_INVALID_BUFFER_OFFSET);
    }
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_flash(f, 1, rows, stream);
}

// attention_decode_scores_values_gqa8: b0 q, b1 keys, b2 values, c3 context,
// c4 capacity, c5 part, b6 partials[16][nparts][258], c7 nparts;
// grid (2, nparts) x (256, 4) (decode_step.cpp:296-306).  part may be any
// positive multiple of 32.
int32_t op_attention_scores_values(const Bindings& b, const Grid& g, hipStream_t stream,
                                   bool validate_only) {
    Args a(b);
    FlashArgs f{};
    f.context = a.constant(3);
    f.capacity = a.constant(4);
    f.part = a.constant(5);
    const uint32_t nparts = a.constant(7);
    a.require(context_ok(f.context, f.capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    a.require(f.part != 0 && f.part % kBlockKeys == 0 && nparts != 0 &&
                  static_cast<uint64_t>(nparts) * f.part >= static_cast<uint64_t>(f.context) + 1,
              TT_CMD_INVALID_BUFFER);
    a.require(g.gx == 2 && g.gy == nparts && g.gz == 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    f.q = a.buffer<const uint16_t>(0, kQueryBytes);
    f.keys = a.buffer<const uint16_t>(1, cache_bytes(f.capacity));
    f.values = a.buffer<const uint16_t>(2, cache_bytes(f.capacity));
    f.partials = a.buffer<float>(
        6, static_cast<uint64_t>(kAttnQueryHeads) * nparts * kAttnRecordFloats * 4);
    f.record_splits = nparts;
    f.query_stride = kAttnQueryValues;
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_flash(f, nparts, 1, stream);
}

// attention_decode_combine: b0 partials, b1 gate, c2 nparts, b3 out; grid 16 x 256
// (decode_step.cpp:332-337).
int32_t op_attention_combine(const Bindings& b, const Grid& g, hipStream_t stream,
                             bool validate_only) {
    Args a(b);
    CombineArgs c{};
    c.nparts = a.constant(2);
    a.require(c.nparts != 0, TT_CMD_INVALID_BUFFER);
    c.partials = a.buffer<const float>(
        0, static_cast<uint64_t>(kAttnQueryHeads) * c.nparts * kAttnRecordFloats * 4);
    c.gate = a.buffer<const uint16_t>(1, kQueryBytes);
    c.out = a.buffer<uint16_t>(3, kQueryBytes);
    c.record_splits = c.nparts;
    c.query_stride = kAttnQueryValues;
    a.require(grid_is(g, 16, 1, 1, 256, 1, 1), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_combine_kernel, dim3(kAttnQueryHeads, 1), dim3(256), 0, stream, c);
    return TT_OK;
}

// attention_decode_split_ms (no reference counterpart; folds every long row of
// a lane batch into one split-K grid): b0 q slab, b1 keys_pool, b2 values_pool,
// b3 state_table, b4 partials [rows][16][max_splits][258], c5 capacity,
// c6 query stride, c7 part (keys per workgroup, multiple of 32), c8 max_splits,
// c9 bit 0 long_rows_only (1: rows whose context fits one 256-key partition are left
// to attention_decode_ms), bit 1 interleave (1: a row's workgroups take its blocks of
// 32 keys in turn instead of `part` consecutive keys each), bit 2 compact (1: the
// workgroups whose splits hold keys are the first of the dispatch order, whatever the
// contexts; same records); grid (max_splits, 2, rows) x 256.
int32_t op_attention_split_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                              bool validate_only) {
    Args a(b);
    FlashArgs f{};
    f.capacity = a.constant(5);
    f.query_stride = a.constant(6);
    f.part = a.constant(7);
    f.record_splits = a.constant(8);
    f.long_rows_only = a.constant(9) & 1;
    f.interleave = (a.constant(9) >> 1) & 1;
    f.compact = (a.constant(9) >> 2) & 1;
    f.rotate = (a.constant(9) >> 3) & 31;
    f.single_partition = kAttnPartition;
    const uint32_t rows = static_cast<uint32_t>(g.gz);
    a.require(f.capacity != 0 && f.query_stride >= kAttnQueryValues && f.part != 0 &&
                  f.part % kBlockKeys == 0 && f.record_splits != 0 &&
                  static_cast<uint64_t>(f.record_splits) * f.part >= f.capacity,
              TT_CMD_INVALID_BUFFER);
    a.require(g.gx == f.record_splits && g.gy == 2 && rows >= 1 && rows <= kMaxBatchRows &&
                  g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t last = rows - 1;
    f.partial_row_floats =
        static_cast<uint64_t>(kAttnQueryHeads) * f.record_splits * kAttnRecordFloats;
    f.q = a.buffer<const uint16_t>(0, (last * f.query_stride + kAttnQueryValues) * 2);
    f.keys = a.buffer<const uint16_t>(1, cache_bytes(f.capacity));
    f.values = a.buffer<const uint16_t>(2, cache_bytes(f.capacity));
    f.table = a.buffer<const uint32_t>(3, rows * 16);
    f.partials = a.buffer<float>(4, f.partial_row_floats * rows * 4);
    // the compact order reads a table row as one 8-byte load
    a.require(!f.compact || reinterpret_cast<uintptr_t>(f.table) % 8 == 0, TT_CMD_INVALID_BUFFER_OFFSET);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_flash(f, f.record_splits, rows, stream);
}

// attention_decode_combine_ms: b0 partials, b1 gate slab, b2 state_table,
// b3 out slab, c4 part, c5 max_splits, c6 query stride, c7 long_rows_only, c8 capacity
// (the one the split dispatch ran with: rows it refused are left alone here too);
// grid (16, rows) x 256.
int32_t op_attention_combine_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                                bool validate_only) {
    Args a(b);
    CombineArgs c{};
    c.part = a.constant(4);
    c.record_splits = a.constant(5);
    c.query_stride = a.constant(6);
    c.long_rows_only = a.constant(7);
    c.capacity = a.constant(8);
    c.single_partition = kAttnPartition;
    const uint32_t rows = static_cast<uint32_t>(g.gy);
    a.require(c.part != 0 && c.record_splits != 0 && c.query_stride >= kAttnQueryValues &&
                  c.capacity != 0,
              TT_CMD_INVALID_BUFFER);
    a.require(g.gx == 16 && g.gz == 1 && rows >= 1 && rows <= kMaxBatchRows && g.tx == 256 &&
                  g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t last = rows - 1;
    c.partial_row_floats =
        static_cast<uint64_t>(kAttnQueryHeads) * c.record_splits * kAttnRecordFloats;
    c.partials = a.buffer<const float>(0, c.partial_row_floats * rows * 4);
    c.gate = a.buffer<const uint16_t>(1, (last * c.query_stride + kAttnQueryValues) * 2);
    c.table = a.buffer<const uint32_t>(2, rows * 16);
    c.out = a.buffer<uint16_t>(3, (last * c.query_stride + kAttnQueryValues) * 2);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_combine_kernel, dim3(kAttnQueryHeads, rows), dim3(256), 0, stream,
                       c);
    return TT_OK;
}

// Bindings shared by the two dispatches of a token wave's attention layer in the rope form:
// b0 projection slab [rows][projection stride], b1 q_w, b2 k_w, b3 keys_pool, b4 values_pool,
// b5 state_table, b6 split records [rows][16][max_splits][258] fp32, b7 out slab
// [rows][query stride], c8 capacity, c9 projection stride, c10 query stride, c11 part (keys
// per workgroup, multiple of 32), c12 max_splits, c13 bit 1 interleave, bit 2 compact, bits
// 3..7 rotate (as c9 of attention_decode_split_ms), c14 records per head the deepest row is
// expected to have (0: as many as the buffer holds; a hint that sizes the finishing
// dispatch's first batch of requests, any value gives the same result).
struct TokenLayer {
    FlashArgs walk;
    FinishArgs finish;
    uint32_t rows;
};
TokenLayer token_layer_args(Args& a, uint32_t rows) {
    TokenLayer t{};
    FlashArgs& f = t.walk;
    FinishArgs& n = t.finish;
    t.rows = rows;
    f.capacity = n.capacity = a.constant(8);
    f.projection_stride = n.projection_stride = a.constant(9);
    n.query_stride = a.constant(10);
    f.part = n.part = a.constant(11);
    f.record_splits = n.record_splits = a.constant(12);
    const uint32_t flags = a.constant(13);
    n.parts_hint = a.constant(14);
    f.interleave = (flags >> 1) & 1;
    f.compact = (flags >> 2) & 1;
    f.rotate = (flags >> 3) & 31;
    a.require(rows >= 1 && rows <= kMaxBatchRows, TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(f.capacity != 0 && f.projection_stride >= kAttnProjectionRows &&
                  f.projection_stride % 4 == 0 && n.query_stride >= kAttnQueryValues &&
                  f.part != 0 && f.part % kBlockKeys == 0 && f.record_splits != 0 &&
                  static_cast<uint64_t>(f.record_splits) * f.part >= f.capacity,
              TT_CMD_INVALID_BUFFER);
    if (a.status != TT_OK) return t;
    const uint64_t last = rows - 1;
    f.partial_row_floats = n.partial_row_floats =
        static_cast<uint64_t>(kAttnQueryHeads) * f.record_splits * kAttnRecordFloats;
    f.projection = n.projection =
        a.buffer<const uint16_t>(0, (last * f.projection_stride + kAttnProjectionRows) * 2);
    f.q_weight = n.q_weight = a.buffer<const uint16_t>(1, kD * 2);
    n.k_weight = a.buffer<const uint16_t>(2, kD * 2);
    n.keys = a.buffer<uint16_t>(3, cache_bytes(f.capacity));
    n.values = a.buffer<uint16_t>(4, cache_bytes(f.capacity));
    f.keys = n.keys;
    f.values = n.values;
    f.table = n.table = a.buffer<const uint32_t>(5, rows * 16);
    f.partials = a.buffer<float>(6, f.partial_row_floats * rows * 4);
    n.partials = f.partials;
    n.out = a.buffer<uint16_t>(7, (last * n.query_stride + kAttnQueryValues) * 2);
    // the table rows are read as 8-byte pairs
    a.require(reinterpret_cast<uintptr_t>(f.table) % 8 == 0, TT_CMD_INVALID_BUFFER_OFFSET);
    return t;
}

// attention_decode_token_ms (no reference counterpart; attn_qk_rope_ms and the split path of
// decode_step.cpp:1231-1259 for every row in one dispatch): bindings above; grid
// (max_splits, 2, rows) x 256.  Writes the split records over the cached keys; the token's
// own key and value are folded in, and appended, by attention_decode_token_finish_ms.
int32_t op_attention_token_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                              bool validate_only) {
    Args a(b);
    const uint32_t rows = static_cast<uint32_t>(std::min<uint64_t>(g.gz, 0xFFFF));
    TokenLayer t = token_layer_args(a, rows);
    a.require(g.gx == t.walk.record_splits && g.gy == 2 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    return launch_flash(t.walk, t.walk.record_splits, rows, stream);
}

// attention_decode_token_finish_ms: bindings above; grid (16, rows) x 256.
int32_t op_attention_token_finish_ms(const Bindings& b, const Grid& g, hipStream_t stream,
                                     bool validate_only) {
    Args a(b);
    const uint32_t rows = static_cast<uint32_t>(std::min<uint64_t>(g.gy, 0xFFFF));
    TokenLayer t = token_layer_args(a, rows);
    a.require(g.gx == kAttnQueryHeads && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_finish_kernel, dim3(kAttnQueryHeads, rows), dim3(256), 0, stream,
                       t.finish);
    return TT_OK;
}

// attention_decode_scores_gqa4: b0 q, b1 keys, c2 context, c3 capacity, c4 part,
// b5 weights[16][nparts][258], c6 nparts; grid (4, nparts) x (256, 4)
// (decode_step.cpp:309-318).
int32_t op_attention_scores(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only) {
    Args a(b);
    const uint32_t context = a.constant(2);
    const uint32_t capacity = a.constant(3);
    const uint32_t part = a.constant(4);
    const uint32_t nparts = a.constant(6);
    a.require(context_ok(context, capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    a.require(part != 0 && part <= 256 && nparts != 0, TT_CMD_INVALID_BUFFER);
    a.require(g.gx == 4 && g.gy == nparts && g.gz == 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint16_t* q = a.buffer<const uint16_t>(0, kQueryBytes);
    const uint16_t* keys = a.buffer<const uint16_t>(1, cache_bytes(capacity));
    float* weights = a.buffer<float>(
        5, static_cast<uint64_t>(kAttnQueryHeads) * nparts * kAttnRecordFloats * 4);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_scores_kernel, dim3(kAttnQueryHeads, nparts), dim3(256), 0, stream,
                       q, keys, context, capacity, part, weights, nparts);
    return TT_OK;
}

// attention_decode_values_gqa8: b0 weights, b1 values, c2 context, c3 capacity,
// c4 part, b5 partials, c6 nparts; grid (2, nparts) x (32, 4, 8)
// (decode_step.cpp:320-329).
int32_t op_attention_values(const Bindings& b, const Grid& g, hipStream_t stream,
                            bool validate_only) {
    Args a(b);
    const uint32_t context = a.constant(2);
    const uint32_t capacity = a.constant(3);
    const uint32_t part = a.constant(4);
    const uint32_t nparts = a.constant(6);
    a.require(context_ok(context, capacity), TT_CMD_CONTEXT_OUT_OF_RANGE);
    a.require(part != 0 && part <= 256 && nparts != 0, TT_CMD_INVALID_BUFFER);
    a.require(g.gx == 2 && g.gy == nparts && g.gz == 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    const uint64_t record_bytes =
        static_cast<uint64_t>(kAttnQueryHeads) * nparts * kAttnRecordFloats * 4;
    const float* weights = a.buffer<const float>(0, record_bytes);
    const uint16_t* values = a.buffer<const uint16_t>(1, cache_bytes(capacity));
    float* partials = a.buffer<float>(5, record_bytes);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_values_kernel, dim3(kAttnQueryHeads, nparts), dim3(256), 0, stream,
                       weights, values, context, capacity, part, partials, nparts);
    return TT_OK;
}

}  // namespace

// Host code that names `scratch` stays visible to the device pass of the compiler: that
// is how it learns that the host refers to the static device variable and gives it a
// symbol the runtime can resolve.
namespace {

constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};   // device address of `scratch`, per GPU
bool g_decode_ready[kMaxDevices] = {};

// Set-up of the current device, once per device: the large dynamic LDS opt-in of the
// split kernel and the device address of this GPU's copy of `scratch`.  Neither call
// allocates.  Called when a library is created and, for a caller that never created
// one, by the first direct launch on the device.
bool prepare_current_device() {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return false;
    }
    if (g_decode_ready[device]) return true;
    // 4 x 16.5 KiB of LDS is above the 64 KiB a kernel gets without opting in
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(flash_decode_kernel<false>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            kWaves * kWaveLdsBytes) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(flash_decode_kernel<false, true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            kWaves * kWaveLdsBytes) != hipSuccess ||
        hipFuncSetAttribute(reinterpret_cast<const void*>(flash_decode_kernel<true>),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            kWaves * kWaveLdsBytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    void* address = nullptr;
    if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess || address == nullptr) {
        (void)hipGetLastError();
        return false;
    }
    g_static_scratch[device] = address;
    g_decode_ready[device] = true;
    return true;
}

// Device address of the current GPU's `scratch`; null before prepare_current_device().
void* static_scratch() {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    return g_static_scratch[device];
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side tables of launchers
bool prepare_decode_kernels() { return prepare_current_device(); }

const KernelDesc kAttentionDecodeKernels[] = {
    {"attn_qk_rope", op_attn_qk_rope},
    {"attn_qk_rope_ms", op_attn_qk_rope_ms},
    {"attention_decode", op_attention_decode},
    {"attention_decode_ms", op_attention_decode_ms},
    {"attention_decode_scores_values_gqa8", op_attention_scores_values},
    {"attention_decode_combine", op_attention_combine},
    {"attention_decode_scores_gqa4", op_attention_scores},
    {"attention_decode_values_gqa8", op_attention_values},
    {"attention_decode_split_ms", op_attention_split_ms},
    {"attention_decode_combine_ms", op_attention_combine_ms},
    {"attention_decode_token_ms", op_attention_token_ms},
    {"attention_decode_token_finish_ms", op_attention_token_finish_ms},
};
const uint32_t kAttentionDecodeKernelCount =
    sizeof(kAttentionDecodeKernels) / sizeof(kAttentionDecodeKernels[0]);

#endif

}  // namespace tt

#if !defined(__HIP_DEVICE_COMPILE__)
// Direct launch of the lane-batched split-K decode with its records in `scratch`: the
// operand checks of op_attention_split_ms / op_attention_combine_ms on plain pointers,
// then the same two kernels.  No allocation on any path.
extern "C" int32_t tt_attention_decode_lanes_static(
    tt_queue* queue, const void* q, uint64_t q_bytes, const void* gate, uint64_t gate_bytes,
    const void* keys_pool, uint64_t keys_bytes, const void* values_pool, uint64_t values_bytes,
    const void* state_table, uint64_t table_bytes, void* out, uint64_t out_bytes, uint32_t rows,
    uint32_t capacity, uint32_t query_stride, uint32_t split_keys) {
    using namespace tt;
    hipStream_t stream = queue_stream(queue);
    if (queue == nullptr || stream == nullptr) return TT_CMD_INVALID_COMMAND_QUEUE;
    if (q == nullptr || gate == nullptr || keys_pool == nullptr || values_pool == nullptr ||
        state_table == nullptr || out == nullptr) {
        return TT_CMD_INVALID_BUFFER;
    }
    if (rows < 1 || rows > kMaxBatchRows || capacity == 0 || query_stride < kAttnQueryValues ||
        split_keys == 0 || split_keys % kBlockKeys != 0) {
        return TT_CMD_INVALID_DISPATCH_EXTENT;
    }
    const uint64_t slab_bytes =
        (static_cast<uint64_t>(rows - 1) * query_stride + kAttnQueryValues) * 2;
    if (q_bytes < slab_bytes || gate_bytes < slab_bytes || out_bytes < slab_bytes ||
        keys_bytes < cache_bytes(capacity) || values_bytes < cache_bytes(capacity) ||
        table_bytes < static_cast<uint64_t>(rows) * 16) {
        return TT_CMD_INVALID_BUFFER_OFFSET;
    }
    const uint32_t splits = (capacity + split_keys - 1) / split_keys;
    const uint64_t row_floats = static_cast<uint64_t>(kAttnQueryHeads) * splits * kAttnRecordFloats;
    if (row_floats * rows * 4 > TT_STATIC_SCRATCH_BYTES) return TT_CMD_STATIC_SCRATCH_EXCEEDED;
    // The device's one-time set-up is done when a queue is created; a caller that reaches
    // this point without it (a queue of another device made current by hand) gets it here,
    // unless the stream is capturing - the set-up calls are not capture-safe.
    if (static_scratch() == nullptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &capturing) != hipSuccess ||
            capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            return TT_CMD_INVALID_DEVICE;
        }
        if (!prepare_current_device()) return TT_CMD_INVALID_DEVICE;
    }
    float* records = static_cast<float*>(static_scratch());
    if (records == nullptr) return TT_CMD_INVALID_DEVICE;

    FlashArgs f{};
    f.q = static_cast<const uint16_t*>(q);
    f.keys = static_cast<const uint16_t*>(keys_pool);
    f.values = static_cast<const uint16_t*>(values_pool);
    f.table = static_cast<const uint32_t*>(state_table);
    f.partials = records;
    f.capacity = capacity;
    f.part = split_keys;
    f.record_splits = splits;
    f.query_stride = query_stride;
    f.partial_row_floats = row_floats;
    f.single_partition = kAttnPartition;
    // a grid larger than the chip may hold workgroups without keys: the ones with keys first
    // (the contexts are on the device, so this cannot be decided more finely here)
    const uint32_t units = queue_compute_units(queue);
    f.compact = static_cast<uint64_t>(splits) * kAttnKvHeads * rows > (units != 0 ? units : 256u) &&
                reinterpret_cast<uintptr_t>(state_table) % 8 == 0;
    f.rotate = 1;   // ranges walked from a rotated starting block, whatever the capacity
    launch_flash(f, splits, rows, stream);

    CombineArgs c{};
    c.partials = records;
    c.gate = static_cast<const uint16_t*>(gate);
    c.out = static_cast<uint16_t*>(out);
    c.table = f.table;
    c.part = split_keys;
    c.record_splits = splits;
    c.query_stride = query_stride;
    c.partial_row_floats = row_floats;
    c.single_partition = kAttnPartition;
    c.capacity = capacity;
    hipLaunchKernelGGL(attention_combine_kernel, dim3(kAttnQueryHeads, rows), dim3(256), 0, stream,
                       c);
    return hipGetLastError() == hipSuccess ? TT_OK : TT_CMD_INVALID_PENDING_EXECUTION;
}
#endif
