// Block-prefill full attention for gfx950: causal flash attention on bf16 MFMA
// with K/V tiles staged through LDS rings, plus the exact partial/combine control
// path.
//
// Operators registered here, with the reference kernels whose argument tables
// they accept (src/backend/metal/kernels/prefill_attention.metal):
//   attn_qk_rope_blk (:1)
//   attention_streaming_blk (:860), attention_flash_v2_blk (:1233)  -> flash kernel
//   attention_partial_blk (:97), attention_combine_blk (:207)        -> control path
//
// Flash kernel, in short (details above the kernel): one workgroup = 8 wave64 = 32
// consecutive query positions x the 8 query heads of one kv head; keys are walked
// in tiles of 32 up to the causal limit of the position tile.
//   S^T[key][pos] = K[key][:] . Q[pos][:]    v_mfma_f32_16x16x32_bf16,
//       A = K from LDS, B = Q^T held in registers for the whole walk.
//   O^T[dim][pos] += V^T[dim][key] P^T[key][pos]
//       A = V^T read from the row-major V stage with the transposing LDS load,
//       B = P^T = bf16 of the S^T accumulators, no LDS round trip.
// Row r of the dispatch sees keys [0, tile_context + r], which makes every row
// a decode step at context tile_context + r over the same cache
// (prefill_attention.metal:117-119).  Algorithmic work: 1024 flop per visible
// (query, key) pair per head.
#include "../tt_internal.h"

#include <type_traits>

namespace tt {
namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr uint32_t kD = kAttnHeadDim;
constexpr uint32_t kTileKeys = 32;
constexpr uint32_t kKeyPairBytes = 1056;                 // key i | key 16+i | 32 B pad
constexpr uint32_t kKeyStageBytes = 16 * kKeyPairBytes;  // 16896
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kReferenceSlackPower = 0x1p100f;   // a score may exceed the fixed reference by 100 log2 units

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float v) {
    const uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(2))) float f32x2;
// two probabilities to a packed bf16 pair (hardware round to nearest even)
__device__ __forceinline__ uint32_t pack_probabilities(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}

// One 1 KiB transfer HBM/L2 -> LDS: lane l's 16 bytes at base + offset go to LDS byte
// lds_address + 16 l.  Issued as assembly so that the waits on these transfers are
// exactly the s_waitcnt instructions written in the kernel: the compiler, seeing an
// LDS-writing load, would otherwise drain every transfer in flight before the next
// LDS read of the same array.
__device__ __forceinline__ void transfer_to_lds(const uint8_t* base, uint32_t offset,
                                                uint32_t lds_address) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_address)), "v"(offset), "s"(base)
                 : "memory");
}

struct FlashPrefillArgs {
    const uint16_t* query;   // [rows][16][256]
    const uint16_t* gate;    // [rows][16][256]
    const uint16_t* keys;    // [2][capacity][256]
    const uint16_t* values;
    uint16_t* out;           // [rows][16][256]
    uint32_t rows;
    uint32_t tile_context;   // cache position of row 0
    uint32_t capacity;
    uint32_t splits;         // workgroups that share the key walk of a position tile (grid z)
    uint8_t* scratch;        // splits > 1: arrival counts, then the partial results
};

// Key walk shared between workgroups.  A block of few rows is few position tiles - 2048 rows
// are 128 workgroups on 256 compute units - while each of them walks the whole prefix.  With
// splits > 1 the key tiles of a position tile are dealt to that many workgroups in equal
// ranges; each range is an ordinary walk with its own softmax reference.  A workgroup that is
// not the last of its position tile to finish leaves {O, reference, row sum} in scratch, fp32,
// in the register order of its lanes; the last one - told by an arrival count, nobody waits
// for anybody - adds the others' to its own with the usual reference change and writes the
// rows.  A walk of fewer than kMinTilesPerSplit key tiles per workgroup is shared by fewer.
constexpr uint32_t kMaxFlashSplits = 8;
constexpr uint32_t kMinTilesPerSplit = 4;
constexpr uint32_t kPartialBytes = 512 * 132 * 4;   // per lane 128 values of O, two references, two row-sum shares
constexpr uint32_t kArrivalBytesPerTile = 4;
__host__ __device__ constexpr uint64_t flash_arrival_bytes(uint32_t rows) {
    return ((static_cast<uint64_t>((rows + 31) / 32) * kAttnKvHeads * kArrivalBytesPerTile + 255) / 256) * 256;
}

// ---------------------------------------------------------- flash kernel ------
//
// Workgroup = 8 wave64 = 32 consecutive query positions x the 8 query heads of one
// kv head.  Wave w owns heads 2(w&3), 2(w&3)+1 at positions 16(w>>2)..+15: two 16x16
// blocks that share every K and V fragment the wave reads from LDS.  Two waves per
// SIMD (256 registers each): LDS operand reads are issued from eight waves and one
// wave's LDS round trips are covered by the other's products.  (The two waves of a SIMD
// pass every phase nearly together - the barrier keeps them in step - so the softmax
// itself is not hidden; forms that keep them a phase apart were measured and are slower,
// because a wave alone in its products waits for its own operand reads.)
//   K and V tiles: HBM/L2 -> LDS rings of 4 stages, three tiles ahead (global_load_lds), so
//   that a tile has landed one barrier before it is entered and its first operands can be
//   read while the tile before it is still being accumulated.
//   Both are stored as 16 row pairs (row i | row 16+i | 32 B pad): with pairs of 1056 bytes
//   both the 16-byte S^T operand reads (sixteen pairs, one piece per quarter wave) and the
//   transposing V reads were measured free of bank conflicts (pairs of 1040 bytes cost the
//   16-byte reads a second pass, pairs of 1024 seven).
//   V^T operands come straight from the row-major V stage with ds_read_b64_tr_b16:
//   16 lanes hand in the addresses of 4 key rows x 16 dims (4 lanes per row, 4 dims
//   each) and lane i receives dim i of the 4 rows - two such reads are the 8 contraction
//   slots of one MFMA operand, no register permutes and no transposed copy in LDS.
// One barrier per tile.  The softmax reference of a row is fixed by tile 0: with q and
// k RMS-normalised a later score cannot exceed it by 2^100, so the steady loop never
// rescales O and the accumulators are touched by MFMA only.  A tile that would exceed
// the slack leaves the steady loop for an exact online-softmax loop (running maximum
// raised per tile, O rescaled), which finishes the walk.
constexpr uint32_t kFlashWaves = 8;
constexpr uint32_t kTilePositions = 32;
constexpr uint32_t kRing = 4;
constexpr uint32_t kKeyRingBytes = kRing * kKeyStageBytes;             // 67584
constexpr uint32_t kValuePairBytes = 1056;                             // row i | row 16+i | 32 B pad
constexpr uint32_t kValuePairedStageBytes = 16 * kValuePairBytes;      // 16896
constexpr uint32_t kFlashLdsBytes = kKeyRingBytes + kRing * kValuePairedStageBytes;  // 135168

typedef __attribute__((ext_vector_type(4))) short s16x4;

__global__ __launch_bounds__(kFlashWaves * 64) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attention_flash_prefill_kernel(FlashPrefillArgs a) {
    constexpr uint32_t NB = 2;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    uint8_t* const key_ring = lds;
    uint8_t* const value_ring = lds + kKeyRingBytes;
    // longest key walks first: the last position tile is dispatched first
    const uint32_t tile = gridDim.x - 1 - blockIdx.x;
    const uint32_t kvh = blockIdx.y;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = lane & 15;
    const uint32_t g = lane >> 4;
    const uint32_t half = wave >> 2;
    const uint32_t head0 = kvh * kAttnHeadsPerKv + (wave & 3) * 2;
    const uint32_t p0 = tile * kTilePositions;
    const uint32_t tile_keys = a.tile_context + min(p0 + kTilePositions, a.rows);  // visible count
    const uint32_t walk_tiles = (tile_keys + kTileKeys - 1) / kTileKeys;
    // this workgroup's share of the walk: key tiles [kb_begin, nkb)
    const uint32_t sharers = min(a.splits, max(walk_tiles / kMinTilesPerSplit, 1u));
    const uint32_t share = blockIdx.z;
    if (share >= sharers) return;
    const uint32_t kb_begin = static_cast<uint32_t>(static_cast<uint64_t>(walk_tiles) * share / sharers);
    const uint32_t nkb = static_cast<uint32_t>(static_cast<uint64_t>(walk_tiles) * (share + 1) / sharers);
    // this lane's column: query row p0 + 16*half + m, whose last visible key is limit
    const uint32_t row = p0 + half * 16 + m;
    const uint32_t limit = a.tile_context + row;
    // tiles below first_masked lie entirely at or before the first column's limit
    const uint32_t first_masked = (a.tile_context + p0 + half * 16 + 1) / kTileKeys;

    bf16x8 q[NB][8];
    {
        const uint32_t pos = min(row, a.rows - 1);
#pragma unroll
        for (uint32_t t = 0; t < NB; ++t) {
            const uint16_t* qrow =
                a.query + (static_cast<uint64_t>(pos) * kAttnQueryHeads + head0 + t) * kD;
#pragma unroll
            for (uint32_t kk = 0; kk < 8; ++kk) {
                q[t][kk] = __builtin_bit_cast(
                    bf16x8, *reinterpret_cast<const u32x4*>(qrow + kk * 32 + g * 8));
            }
        }
    }

    // byte addresses inside one kv head stay below 2^32 (capacity * 512 B)
    const uint8_t* kbase =
        reinterpret_cast<const uint8_t*>(a.keys + static_cast<uint64_t>(kvh) * a.capacity * kD);
    const uint8_t* vbase =
        reinterpret_cast<const uint8_t*>(a.values + static_cast<uint64_t>(kvh) * a.capacity * kD);
    const uint32_t last_key = tile_keys - 1;
    const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
        (__attribute__((address_space(3))) uint8_t*)lds));  // LDS byte address of the key ring
    const uint32_t column_bytes = (lane & 31) * 16;
    // staging addresses are wave-uniform: give the compiler the wave index as a scalar
    const uint32_t swave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t key_lane = swave * 2 + (lane >> 5) * 16;    // + i: row pair 2w+i, second half +16

    // Each wave moves an eighth of a tile: 2 K transfers and 2 V transfers (row pairs
    // 2w, 2w+1), 1 KiB each.  Tiles past the walk re-read the last key, so every batch
    // has the same number of transfers.
    auto stage_tile = [&](uint32_t kb, uint32_t slot) {
        const uint32_t kstage = lds_base + slot * kKeyStageBytes + swave * 2 * kKeyPairBytes;
        const uint32_t vstage =
            lds_base + kKeyRingBytes + slot * kValuePairedStageBytes + swave * 2 * kValuePairBytes;
#pragma unroll
        for (uint32_t i = 0; i < 2; ++i) {
            const uint32_t key = min(kb * kTileKeys + i + key_lane, last_key);
            transfer_to_lds(kbase, key * 512u + column_bytes, kstage + i * kKeyPairBytes);
        }
#pragma unroll
        for (uint32_t i = 0; i < 2; ++i) {
            const uint32_t key = min(kb * kTileKeys + i + key_lane, last_key);
            transfer_to_lds(vbase, key * 512u + column_bytes, vstage + i * kValuePairBytes);
        }
    };

    f32x4 o[NB][16];
#pragma unroll
    for (uint32_t b = 0; b < NB; ++b) {
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) o[b][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    float m_run[NB], l_run[NB];  // reference in log2 units; this lane's share of the row sum
#pragma unroll
    for (uint32_t b = 0; b < NB; ++b) {
        m_run[b] = -INFINITY;
        l_run[b] = 0.0f;
    }
    const float scale = kAttnScale * kLog2e;

    const uint32_t key_read_bytes = m * kKeyPairBytes + g * 16;
    // The operands of a tile's first contraction step are requested while the tile before it
    // is still being accumulated (its keys have landed by then), those of the first V^T
    // product before the softmax: neither phase starts on an LDS round trip.
    u32x4 first_keys[2];
    auto request_first_keys = [&](uint32_t slot) {
        const uint8_t* stage = key_ring + slot * kKeyStageBytes + key_read_bytes;
        first_keys[0] = *reinterpret_cast<const u32x4*>(stage);
        first_keys[1] = *reinterpret_cast<const u32x4*>(stage + 512);
    };
    // S^T of the tile in key stage `slot`; operand reads run one contraction step ahead
    auto scores = [&](uint32_t slot, f32x4 (&s)[2][NB]) {
        const uint8_t* stage = key_ring + slot * kKeyStageBytes + key_read_bytes;
#pragma unroll
        for (uint32_t kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) s[kt][b] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
        u32x4 ka[2][2];
        ka[0][0] = first_keys[0];
        ka[0][1] = first_keys[1];
#pragma unroll
        for (uint32_t kk = 0; kk < 8; ++kk) {
            if (kk + 1 < 8) {
                ka[(kk + 1) & 1][0] = *reinterpret_cast<const u32x4*>(stage + (kk + 1) * 64);
                ka[(kk + 1) & 1][1] = *reinterpret_cast<const u32x4*>(stage + (kk + 1) * 64 + 512);
            }
#pragma unroll
            for (uint32_t kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (uint32_t b = 0; b < NB; ++b) {
                    s[kt][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, ka[kk & 1][kt]), q[b][kk], s[kt][b], 0, 0, 0);
                }
            }
        }
    };
    // O^T[dim][pos] += V^T[dim][slot] P^T[slot][pos]; MFMA j covers dims 16j..16j+15.
    // Contraction slot e of lane group g is key (e>>2)*16 + g*4 + (e&3), the order the
    // S^T accumulators hand the probabilities over in: lane (m, g) points at key row
    // g*4 + (m>>2), dims 16j + 4(m&3)..+3, once in the low and once in the high half
    // of the row pairs.
    const uint32_t value_read_bytes = (g * 4 + (m >> 2)) * kValuePairBytes + (m & 3) * 8;
    auto read_values = [&](const uint8_t* at) -> u32x4 {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(at));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (__attribute__((address_space(3))) s16x4*)(at + 512));
        const u32x2 l = __builtin_bit_cast(u32x2, lo);
        const u32x2 h = __builtin_bit_cast(u32x2, hi);
        return u32x4{l[0], l[1], h[0], h[1]};
    };
    u32x4 first_values;
    auto request_first_values = [&](uint32_t slot) {
        first_values = read_values(value_ring + slot * kValuePairedStageBytes + value_read_bytes);
    };
    auto accumulate = [&](uint32_t slot, const bf16x8 (&pb)[NB]) {
        const uint8_t* vt = value_ring + slot * kValuePairedStageBytes + value_read_bytes;
        u32x4 va[2];
        va[0] = first_values;
#pragma unroll
        for (uint32_t j = 0; j < 16; ++j) {
            if (j == 10) {
                // far enough from the barrier to have arrived by then, late enough for the
                // registers of the last score step to be free
                request_first_keys((slot + 1) & 3);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (j + 1 < 16) va[(j + 1) & 1] = read_values(vt + (j + 1) * 32);
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) {
                o[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    __builtin_bit_cast(bf16x8, va[j & 1]), pb[b], o[b][j], 0, 0, 0);
            }
        }
    };
    // exponent arguments of block b against the reference: s*scale - m_run, masked
    // keys at -inf.  Lane holds keys key0 + kt*16 + g*4 + i of its position column.
    auto arguments = [&](auto masked, uint32_t kb, const f32x4 (&s)[2][NB], uint32_t b,
                         float (&x)[8]) {
#pragma unroll
        for (uint32_t kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                float v = __builtin_fmaf(s[kt][b][i], scale, -m_run[b]);
                if (decltype(masked)::value && kb * kTileKeys + kt * 16 + g * 4 + i > limit) {
                    v = -INFINITY;
                }
                x[kt * 4 + i] = v;
            }
        }
    };
    auto probabilities = [&](const float (&x)[8], bf16x8& pb) -> float {
        float block_sum = 0.0f;
        uint32_t pw[4];
#pragma unroll
        for (uint32_t c = 0; c < 4; ++c) {
            const float x0 = __builtin_amdgcn_exp2f(x[2 * c]);
            const float x1 = __builtin_amdgcn_exp2f(x[2 * c + 1]);
            block_sum += x0 + x1;
            pw[c] = pack_probabilities(x0, x1);
        }
        pb = __builtin_bit_cast(bf16x8, u32x4{pw[0], pw[1], pw[2], pw[3]});
        return block_sum;
    };
    // Exact step of block b: scaled, masked scores; raises the reference to the
    // tile's maximum; returns the factor O and the row sum are scaled by.
    auto exact_step = [&](uint32_t kb, const f32x4 (&s)[2][NB], uint32_t b, float (&x)[8]) -> float {
        float block_max = -INFINITY;
#pragma unroll
        for (uint32_t kt = 0; kt < 2; ++kt) {
#pragma unroll
            for (uint32_t i = 0; i < 4; ++i) {
                float v = s[kt][b][i] * scale;
                if (kb * kTileKeys + kt * 16 + g * 4 + i > limit) v = -INFINITY;
                x[kt * 4 + i] = v;
                block_max = fmaxf(block_max, v);
            }
        }
        block_max = fmaxf(block_max, __shfl_xor(block_max, 16, 64));
        block_max = fmaxf(block_max, __shfl_xor(block_max, 32, 64));
        const float m_new = fmaxf(m_run[b], block_max);  // key 0 is visible: finite from tile 0 on
        const float alpha = __builtin_amdgcn_exp2f(m_run[b] - m_new);
        l_run[b] *= alpha;
        m_run[b] = m_new;
#pragma unroll
        for (uint32_t e = 0; e < 8; ++e) x[e] -= m_new;
        return alpha;
    };

    // Batch j, issued on entering the walk's tile j: keys and values of its tile j+3.
    stage_tile(kb_begin, 0);
    stage_tile(kb_begin + 1, 1);
    stage_tile(kb_begin + 2, 2);
    // Ring position of the tile being entered: kslot = (kb - kb_begin) % 4; tile kb+3 goes
    // to the stage tile kb-1 has just left.
    uint32_t kb = kb_begin;
    uint32_t kslot = 0;
    // Entering tile kb: batches up to kb-2 (tiles up to kb+1) have landed for every wave, so
    // the next tile's first operands may be read while this one is accumulated, and every
    // wave is done with tile kb-1.
    auto enter_tile = [&]() {
        __builtin_amdgcn_s_waitcnt(0x0F74);  // all but the 4 transfers of batch kb-1
        __syncthreads();
        stage_tile(kb + 3, (kslot + 3) & 3);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto advance = [&]() {
        ++kb;
        kslot = (kslot + 1) & 3;
    };

    bf16x8 pb[NB];
    enter_tile();
    request_first_keys(kslot);
    {
        f32x4 s[2][NB];
        scores(kslot, s);
        request_first_values(kslot);
#pragma unroll
        for (uint32_t b = 0; b < NB; ++b) {
            float x[8];
            (void)exact_step(kb, s, b, x);  // O and the sums are still zero
            l_run[b] += probabilities(x, pb[b]);
        }
        accumulate(kslot, pb);
    }
    advance();
    if (kb < nkb) enter_tile();
    // Steady state: the reference of every row stays where tile 0 put it (scores are
    // bounded by |q||k|/16 with RMS-normalised q and k), so O is touched by MFMA only.
    // A score beyond the slack leaves for the exact loop with tile kb entered and not
    // yet accumulated.
    auto steady = [&](auto masked, uint32_t end) -> bool {
        while (kb < end) {
            f32x4 s[2][NB];
            scores(kslot, s);
            request_first_values(kslot);
            __builtin_amdgcn_sched_barrier(0);
            float sums[NB];
            bf16x8 next[NB];
            float top = 0.0f;
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) {
                float x[8];
                arguments(masked, kb, s, b, x);
                sums[b] = probabilities(x, next[b]);
                top = fmaxf(top, sums[b]);
            }
            // an argument beyond the slack shows in the sum of its eight powers (2^slack at
            // the least; a sum that reaches it without such an argument leaves as well, which
            // costs time and nothing else): one comparison instead of a maximum over the arguments
            if (__builtin_amdgcn_ballot_w64(!(top < kReferenceSlackPower)) != 0) return true;
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) l_run[b] += sums[b];
            __builtin_amdgcn_sched_barrier(0);
            accumulate(kslot, next);
            advance();
            if (kb < nkb) enter_tile();
        }
        return false;
    };
    bool above = steady(std::false_type{}, min(first_masked, nkb));
    if (!above) above = steady(std::true_type{}, nkb);
    if (above) {
        // (a wave that leaves the steady loop has taken the scores of tile kb, so it asks for
        // that tile's first keys again)
        request_first_keys(kslot);
        for (;;) {
            f32x4 s[2][NB];
            scores(kslot, s);
            request_first_values(kslot);
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) {
                float x[8];
                const float alpha = exact_step(kb, s, b, x);
#pragma unroll
                for (uint32_t j = 0; j < 16; ++j) o[b][j] *= alpha;
                l_run[b] += probabilities(x, pb[b]);
            }
            accumulate(kslot, pb);
            advance();
            if (kb == nkb) break;
            enter_tile();
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);  // transfers of the tiles past the walk

    if (sharers > 1) {
        // Arrival: every workgroup but the last to finish leaves its result and goes; the
        // last one takes the others' in.  The count starts at zero (the launcher clears it).
        // Results travel as device-scope stores and loads of single words, which go through
        // to memory and come from it whatever the L2 of either side holds: the writer waits
        // for their acknowledgement before it counts itself in, and no cache is written back
        // or dropped (fences of that scope, one per wave, cost 60 us a launch: the L2s of
        // eight dies written back 2000 times).
        __shared__ uint32_t arrival;
        const uint32_t pair = tile * kAttnKvHeads + kvh;
        float* const partials = reinterpret_cast<float*>(a.scratch + flash_arrival_bytes(a.rows)) +
                                static_cast<uint64_t>(pair) * a.splits * (kPartialBytes / 4);
        const auto publish = [](float* at, float value) {
            __hip_atomic_store(reinterpret_cast<uint32_t*>(at), __float_as_uint(value), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        };
        const auto collect = [](const float* at) {
            return __uint_as_float(__hip_atomic_load(reinterpret_cast<const uint32_t*>(at),
                                                     __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        };
        // element e of a lane's 132 (O of head b, dim block j, value i at (b*16+j)*4+i, then
        // the two references and the two row-sum shares) lies at [e][thread]
        float* const mine = partials + static_cast<uint64_t>(share) * (kPartialBytes / 4) + threadIdx.x;
#pragma unroll
        for (uint32_t b = 0; b < NB; ++b) {
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
#pragma unroll
                for (uint32_t i = 0; i < 4; ++i) publish(mine + ((b * 16 + j) * 4 + i) * 512, o[b][j][i]);
            }
            publish(mine + (128 + b) * 512, m_run[b]);
            publish(mine + (130 + b) * 512, l_run[b]);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // every store of this wave acknowledged
        __syncthreads();
        if (threadIdx.x == 0) {
            arrival = __hip_atomic_fetch_add(reinterpret_cast<uint32_t*>(a.scratch) + pair, 1u,
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __syncthreads();
        if (arrival != sharers - 1) return;
        for (uint32_t other = 0; other < sharers; ++other) {
            if (other == share) continue;
            const float* theirs = partials + static_cast<uint64_t>(other) * (kPartialBytes / 4) + threadIdx.x;
#pragma unroll
            for (uint32_t b = 0; b < NB; ++b) {
                const float m_other = collect(theirs + (128 + b) * 512);
                const float l_other = collect(theirs + (130 + b) * 512);
                const float m_new = fmaxf(m_run[b], m_other);
                const float keep = __builtin_amdgcn_exp2f(m_run[b] - m_new);
                const float take = __builtin_amdgcn_exp2f(m_other - m_new);
                m_run[b] = m_new;
                l_run[b] = l_run[b] * keep + l_other * take;
#pragma unroll
                for (uint32_t j = 0; j < 16; ++j) {
#pragma unroll
                    for (uint32_t i = 0; i < 4; ++i) {
                        o[b][j][i] = o[b][j][i] * keep + collect(theirs + ((b * 16 + j) * 4 + i) * 512) * take;
                    }
                }
            }
        }
    }

    // out[(row*16 + head)*256 + dim] = bf16((O/l) * sigmoid(gate)); lane holds, for
    // position column m, dims 16j + 4g + i
    if (row < a.rows) {
#pragma unroll
        for (uint32_t b = 0; b < NB; ++b) {
            float l = l_run[b];
            l += __shfl_xor(l, 16, 64);
            l += __shfl_xor(l, 32, 64);
            const float inv = 1.0f / l;
            const uint64_t row_base = (static_cast<uint64_t>(row) * kAttnQueryHeads + head0 + b) * kD;
#pragma unroll
            for (uint32_t j = 0; j < 16; ++j) {
                const uint32_t dim = j * 16 + g * 4;
                const u32x2 gw = *reinterpret_cast<const u32x2*>(a.gate + row_base + dim);
                float r[4];
#pragma unroll
                for (uint32_t i = 0; i < 4; ++i) {
                    const float gate = __uint_as_float(
                        (i & 1) ? (gw[i >> 1] & 0xFFFF0000u) : (gw[i >> 1] << 16));
                    const float sig = 1.0f / (1.0f + __expf(-gate));
                    r[i] = (o[b][j][i] * inv) * sig;
                }
                u32x2 ow;
                ow[0] = static_cast<uint32_t>(f32_to_bf16_bits(r[0])) |
                        (static_cast<uint32_t>(f32_to_bf16_bits(r[1])) << 16);
                ow[1] = static_cast<uint32_t>(f32_to_bf16_bits(r[2])) |
                        (static_cast<uint32_t>(f32_to_bf16_bits(r[3])) << 16);
                *reinterpret_cast<u32x2*>(a.out + row_base + dim) = ow;
            }
        }
    }
}

// --------------------------------------------------- exact control path ------

// attention_partial_blk: grid (16, partitions, tile_rows) x 256; one record
// {numerator[256], max, sum} per (head, row, partition of 256 keys) with the
// causal limit visible = context + row + 1 (prefill_attention.metal:97-205).
// Scalar and simple on purpose: this is the reference the fast kernels are
// judged against, not a fast path.
__global__ __launch_bounds__(256) void attention_partial_blk_kernel(
    const uint16_t* query, const uint16_t* keys, const uint16_t* values, uint32_t context,
    uint32_t capacity, uint32_t partition, float* partials, uint32_t partition_count,
    uint32_t block) {
    __shared__ float scores[256];
    __shared__ float red[256];
    __shared__ float qs[kD];
    const uint32_t head = blockIdx.x;
    const uint32_t part = blockIdx.y;
    const uint32_t row = blockIdx.z;
    const uint32_t t = threadIdx.x;
    const uint32_t visible = context + row + 1;
    const uint32_t start = part * partition;
    const uint32_t end = min(visible, start + partition);
    const uint32_t kv = head / kAttnHeadsPerKv;
    qs[t] = bf16_bits_to_f32(query[(static_cast<uint64_t>(row) * kAttnQueryHeads + head) * kD + t]);
    float running = -INFINITY;
    float denom = 0.0f;
    float acc = 0.0f;
    __syncthreads();
    for (uint32_t tile = start; tile < end; tile += 256) {
        const uint32_t count = min(end - tile, 256u);
        float s = -INFINITY;
        if (t < count) {
            const uint16_t* k = keys + (static_cast<uint64_t>(kv) * capacity + tile + t) * kD;
            float dot = 0.0f;
            for (uint32_t d = 0; d < kD; ++d) dot = fmaf(qs[d], bf16_bits_to_f32(k[d]), dot);
            s = dot * kAttnScale;
        }
        red[t] = s;
        __syncthreads();
        for (uint32_t off = 128; off; off >>= 1) {
            if (t < off) red[t] = fmaxf(red[t], red[t + off]);
            __syncthreads();
        }
        const float next = fmaxf(running, red[0]);
        const float rescale = running == -INFINITY ? 0.0f : expf(running - next);
        __syncthreads();
        const float p = t < count ? expf(s - next) : 0.0f;
        scores[t] = p;
        red[t] = p;
        __syncthreads();
        for (uint32_t off = 128; off; off >>= 1) {
            if (t < off) red[t] += red[t + off];
            __syncthreads();
        }
        acc *= rescale;
        const uint16_t* v = values + (static_cast<uint64_t>(kv) * capacity + tile) * kD + t;
        for (uint32_t p2 = 0; p2 < count; ++p2) {
            acc = fmaf(scores[p2], bf16_bits_to_f32(v[static_cast<uint64_t>(p2) * kD]), acc);
        }
        denom = denom * rescale + red[0];
        running = next;
        __syncthreads();
    }
    float* dst = partials + ((static_cast<uint64_t>(head) * block + row) * partition_count + part) *
                                kAttnRecordFloats;
    dst[t] = acc;
    if (t == 0) {
        dst[kD] = running;
        dst[kD + 1] = denom;
    }
}

// attention_combine_blk: grid (16, tile_rows) x 256 (prefill_attention.metal:207-254);
// an all-masked partition (max = -inf) carries weight zero.
__global__ __launch_bounds__(256) void attention_combine_blk_kernel(const float* partials,
                                                                    const uint16_t* gate,
                                                                    uint32_t partition_count,
                                                                    uint16_t* out, uint32_t block) {
    const uint32_t head = blockIdx.x;
    const uint32_t row = blockIdx.y;
    const uint32_t d = threadIdx.x;
    const float* base = partials + (static_cast<uint64_t>(head) * block + row) * partition_count *
                                       kAttnRecordFloats;
    float gmax = -INFINITY;
    for (uint32_t p = 0; p < partition_count; ++p) {
        gmax = fmaxf(gmax, base[static_cast<uint64_t>(p) * kAttnRecordFloats + kD]);
    }
    float acc = 0.0f;
    float denom = 0.0f;
    for (uint32_t p = 0; p < partition_count; ++p) {
        const float* rec = base + static_cast<uint64_t>(p) * kAttnRecordFloats;
        const float w = rec[kD] == -INFINITY ? 0.0f : expf(rec[kD] - gmax);
        acc = fmaf(w, rec[d], acc);
        denom = fmaf(w, rec[kD + 1], denom);
    }
    const uint64_t at = (static_cast<uint64_t>(row) * kAttnQueryHeads + head) * kD + d;
    const float g = bf16_bits_to_f32(gate[at]);
    out[at] = f32_to_bf16_bits((acc / denom) * (1.0f / (1.0f + expf(-g))));
}

// ---------------------------------------------------------------- launchers --

}  // namespace

uint32_t flash_prefill_splits(uint32_t rows, uint32_t visible, uint32_t compute_units) {
    const uint64_t groups = static_cast<uint64_t>((rows + kTilePositions - 1) / kTilePositions) * kAttnKvHeads;
    // a longest walk that two workgroups would not share is not worth the clearing dispatch
    if (groups == 0 || (static_cast<uint64_t>(visible) + kTileKeys - 1) / kTileKeys < 4 * kMinTilesPerSplit) return 1;
    const uint64_t fit = compute_units / groups;
    return static_cast<uint32_t>(fit < 1 ? 1 : fit > kMaxFlashSplits ? kMaxFlashSplits : fit);
}

uint64_t stream_workspace_bytes(uint32_t compute_units) {
    // the shared walk never has more workgroups than compute units; their arrival counts
    // (at most one per two of them) stay under a page
    return 4096 + static_cast<uint64_t>(compute_units) * kPartialBytes;
}

uint64_t flash_prefill_scratch_bytes(uint32_t rows, uint32_t splits) {
    if (splits <= 1) return 0;
    const uint64_t groups = static_cast<uint64_t>((rows + kTilePositions - 1) / kTilePositions) * kAttnKvHeads;
    return flash_arrival_bytes(rows) + groups * splits * kPartialBytes;
}

namespace {

uint64_t cache_bytes(uint32_t capacity) {
    return static_cast<uint64_t>(kAttnKvHeads) * capacity * kD * 2;
}

// attention_streaming_blk / attention_flash_v2_blk: b0 query(+tile), b1 keys,
// b2 values, b3 gate(+tile), b4 attended(+tile), c5 visible, c6 capacity,
// c7 tile_rows, c8 tile_context; grid (16, ceil(tile_rows/16)) x 256
// (prefill_step.cpp:1657-1717).  tile_rows is not limited to the reference's
// 256-row query tile: one dispatch may cover a whole block.
__global__ void clear_arrivals_kernel(uint32_t* words, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) words[i] = 0;
}

int32_t flash_blk(const Bindings& b, const Grid& g, hipStream_t stream, bool validate_only,
                  bool shared_walk) {
    Args a(b);
    FlashPrefillArgs f{};
    const uint32_t visible = a.constant(5);
    f.capacity = a.constant(6);
    f.rows = a.constant(7);
    f.tile_context = a.constant(8);
    a.require(f.rows >= 1 && f.rows <= (1u << 24), TT_CMD_INVALID_DISPATCH_EXTENT);
    if (a.status != TT_OK) return a.status;
    // the reference dispatches one threadgroup per (head, 16 query rows)
    a.require(g.gx == 16 && g.gy == (f.rows + 15) / 16 && g.gz == 1 && g.tx == 256 && g.ty == 1 &&
                  g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    // the kernel addresses a kv head's rows with 32-bit byte offsets (512 B per key)
    a.require(f.capacity != 0 && f.capacity <= (1u << 23) &&
                  static_cast<uint64_t>(f.tile_context) + f.rows == visible &&
                  visible <= f.capacity,
              TT_CMD_CONTEXT_OUT_OF_RANGE);
    const uint64_t row_bytes = static_cast<uint64_t>(f.rows) * kAttnQueryValues * 2;
    f.query = a.buffer<const uint16_t>(0, row_bytes);
    f.keys = a.buffer<const uint16_t>(1, cache_bytes(f.capacity));
    f.values = a.buffer<const uint16_t>(2, cache_bytes(f.capacity));
    f.gate = a.buffer<const uint16_t>(3, row_bytes);
    f.out = a.buffer<uint16_t>(4, row_bytes);
    f.splits = 1;
    if (shared_walk) {
        f.splits = a.constant(10);
        a.require(f.splits >= 1 && f.splits <= kMaxFlashSplits, TT_CMD_INVALID_DISPATCH_EXTENT);
        if (a.status != TT_OK) return a.status;
        if (f.splits > 1) f.scratch = a.buffer<uint8_t>(9, flash_prefill_scratch_bytes(f.rows, f.splits));
    }
    if (a.status != TT_OK || validate_only) return a.status;
    if (!shared_walk) {
        // the reference's bindings carry no scratch: the walk is shared through the queue's
        // own workspace where the block is too few rows to fill the device
        const StreamWorkspace workspace = stream_workspace(stream);
        if (workspace.base != nullptr) {
            const uint32_t planned = flash_prefill_splits(f.rows, visible, workspace.compute_units);
            if (planned > 1 && flash_prefill_scratch_bytes(f.rows, planned) <= workspace.bytes) {
                f.splits = planned;
                f.scratch = workspace.base;
            }
        }
    }
    const uint32_t tiles = (f.rows + kTilePositions - 1) / kTilePositions;
    if (f.splits > 1) {
        const uint32_t words = tiles * kAttnKvHeads;
        hipLaunchKernelGGL(clear_arrivals_kernel, dim3((words + 255) / 256), dim3(256), 0, stream,
                           reinterpret_cast<uint32_t*>(f.scratch), words);
    }
    hipLaunchKernelGGL(attention_flash_prefill_kernel, dim3(tiles, kAttnKvHeads, f.splits),
                       dim3(kFlashWaves * 64), kFlashLdsBytes, stream, f);
    return TT_OK;
}

int32_t op_attention_flash_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                               bool validate_only) {
    return flash_blk(b, g, stream, validate_only, false);
}

// attention_flash_split_blk (no counterpart in the reference): the bindings, constants and
// grid of attention_flash_v2_blk, plus b9 scratch and c10 splits (1..8) - the workgroups that
// share each position tile's key walk.  tt_flash_prefill_splits gives the count that fills
// the device for a block of `rows` rows that sees `visible` keys, tt_flash_prefill_scratch_bytes the bytes b9 must hold
// (none for one split).  Same results as attention_flash_v2_blk up to the order of fp32 sums.
int32_t op_attention_flash_split_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                                     bool validate_only) {
    return flash_blk(b, g, stream, validate_only, true);
}

// attention_partial_blk: b0 query(+tile), b1 keys, b2 values, c3 tile_context,
// c4 capacity, c5 partition=256, b6 partials[16][tile_rows][parts][258],
// c7 partitions, c8 tile_rows; grid (16, partitions, tile_rows) x 256
// (prefill_step.cpp:1782-1800).
int32_t op_attention_partial_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                                 bool validate_only) {
    Args a(b);
    const uint32_t context = a.constant(3);
    const uint32_t capacity = a.constant(4);
    const uint32_t partition = a.constant(5);
    const uint32_t partitions = a.constant(7);
    const uint32_t rows = a.constant(8);
    a.require(rows >= 1 && rows <= 65535 && partitions >= 1 && partitions <= 65535 &&
                  partition >= 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(g.gx == 16 && g.gy == partitions && g.gz == rows && g.tx == 256 && g.ty == 1 &&
                  g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(capacity != 0 && static_cast<uint64_t>(context) + rows <= capacity,
              TT_CMD_CONTEXT_OUT_OF_RANGE);
    const uint16_t* query =
        a.buffer<const uint16_t>(0, static_cast<uint64_t>(rows) * kAttnQueryValues * 2);
    const uint16_t* keys = a.buffer<const uint16_t>(1, cache_bytes(capacity));
    const uint16_t* values = a.buffer<const uint16_t>(2, cache_bytes(capacity));
    float* partials = a.buffer<float>(
        6, static_cast<uint64_t>(kAttnQueryHeads) * rows * partitions * kAttnRecordFloats * 4);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_partial_blk_kernel, dim3(16, partitions, rows), dim3(256), 0,
                       stream, query, keys, values, context, capacity, partition, partials,
                       partitions, rows);
    return TT_OK;
}

// attention_combine_blk: b0 partials, b1 gate(+tile), c2 partitions,
// b3 attended(+tile), c4 tile_rows; grid (16, tile_rows) x 256
// (prefill_step.cpp:1802-1817).
int32_t op_attention_combine_blk(const Bindings& b, const Grid& g, hipStream_t stream,
                                 bool validate_only) {
    Args a(b);
    const uint32_t partitions = a.constant(2);
    const uint32_t rows = a.constant(4);
    a.require(rows >= 1 && rows <= 65535 && partitions >= 1, TT_CMD_INVALID_DISPATCH_EXTENT);
    a.require(g.gx == 16 && g.gy == rows && g.gz == 1 && g.tx == 256 && g.ty == 1 && g.tz == 1,
              TT_CMD_INVALID_DISPATCH_EXTENT);
    const float* partials = a.buffer<const float>(
        0, static_cast<uint64_t>(kAttnQueryHeads) * rows * partitions * kAttnRecordFloats * 4);
    const uint64_t row_bytes = static_cast<uint64_t>(rows) * kAttnQueryValues * 2;
    const uint16_t* gate = a.buffer<const uint16_t>(1, row_bytes);
    uint16_t* out = a.buffer<uint16_t>(3, row_bytes);
    if (a.status != TT_OK || validate_only) return a.status;
    hipLaunchKernelGGL(attention_combine_blk_kernel, dim3(16, rows), dim3(256), 0, stream, partials,
                       gate, partitions, out, rows);
    return TT_OK;
}

}  // namespace

#if !defined(__HIP_DEVICE_COMPILE__)  // host-side tables of launchers
bool prepare_prefill_kernels() {
    return hipFuncSetAttribute(reinterpret_cast<const void*>(attention_flash_prefill_kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize,
                               kFlashLdsBytes) == hipSuccess;
}

const KernelDesc kAttentionPrefillKernels[] = {
    {"attn_qk_rope_blk", op_attn_qk_rope_blk},
    {"attention_streaming_blk", op_attention_flash_blk},
    {"attention_flash_v2_blk", op_attention_flash_blk},
    {"attention_flash_split_blk", op_attention_flash_split_blk},
    {"attention_partial_blk", op_attention_partial_blk},
    {"attention_combine_blk", op_attention_combine_blk},
};
const uint32_t kAttentionPrefillKernelCount =
    sizeof(kAttentionPrefillKernels) / sizeof(kAttentionPrefillKernels[0]);
#endif

}  // namespace tt
