// Model and kernel constants of the attention-family path of Qwen3.6-35B-A3B.
// Values: reference catalog/model_packages/qwen36-35b-a3b/model.toml:9-34 and
// the kernel prelude literals of tools/generate_kernel_library.py:173-182,
// 1981-2015 (also pinned by tests/native/decode_geometry_test.cpp:31-50).
#pragma once

#include <stdint.h>

namespace tt {

constexpr uint32_t kLayers = 40;
constexpr uint32_t kHidden = 2048;

constexpr uint32_t kAttnQueryHeads = 16;
constexpr uint32_t kAttnKvHeads = 2;
constexpr uint32_t kAttnHeadsPerKv = kAttnQueryHeads / kAttnKvHeads;
constexpr uint32_t kAttnHeadDim = 256;
constexpr uint32_t kAttnRopePairs = kAttnHeadDim / 8;  // dims [0, 64) rotate
constexpr float kAttnRopeBase = 1.0e7f;
constexpr float kAttnScale = 0.0625f;  // 1/sqrt(256)
constexpr uint32_t kAttnQueryValues = kAttnQueryHeads * kAttnHeadDim;       // 4096
constexpr uint32_t kAttnQGateRows = kAttnQueryHeads * 2 * kAttnHeadDim;     // 8192
constexpr uint32_t kAttnVRowOffset = kAttnQGateRows + kAttnKvHeads * kAttnHeadDim;  // 8704
constexpr uint32_t kAttnProjectionRows = kAttnVRowOffset + kAttnKvHeads * kAttnHeadDim;  // 9216
constexpr uint32_t kAttnPartition = 256;
constexpr uint32_t kAttnRecordFloats = kAttnHeadDim + 2;  // numerators, max, sum

constexpr uint32_t kGdnValueHeads = 32;
constexpr uint32_t kGdnKeyHeads = 16;
constexpr uint32_t kGdnHeadDim = 128;
constexpr uint32_t kGdnConvWidth = 4;
constexpr uint32_t kGdnQkValues = 2 * kGdnKeyHeads * kGdnHeadDim;           // 4096
constexpr uint32_t kGdnValueValues = kGdnValueHeads * kGdnHeadDim;          // 4096
constexpr uint32_t kGdnConvChannels = kGdnQkValues + kGdnValueValues;       // 8192
constexpr uint32_t kGdnKOffset = kGdnKeyHeads * kGdnHeadDim;                // 2048
constexpr uint32_t kGdnBRowOffset = kGdnConvChannels + kGdnValueValues;     // 12288
constexpr uint32_t kGdnARowOffset = kGdnBRowOffset + kGdnValueHeads;        // 12320
constexpr uint32_t kGdnProjectionRows = kGdnARowOffset + kGdnValueHeads;    // 12352
constexpr uint32_t kGdnStateFloats = kGdnValueHeads * kGdnHeadDim * kGdnHeadDim;
constexpr uint16_t kGdnQueryScaleBits = 0x3C00;  // bf16(1/128)
constexpr uint16_t kGdnKeyScaleBits = 0x3DB5;    // bf16(1/sqrt(128)) = 0.08837890625
constexpr float kRmsNormEpsilon = 1.0e-6f;

// Rollback tape of a short verified block (tools/generate_kernel_library.py:2045-2049):
// per layer and block row the 32x128 delta values, then the 16x128 keys, then
// {decay, beta} per value head, each region sized for all 40 layers; the conv tape
// holds the conv window as it stands after each row.
constexpr uint32_t kGdnTapeRows = 16;
constexpr uint32_t kGdnTapeKeyOffset = kLayers * kGdnTapeRows * kGdnValueHeads * kGdnHeadDim;
constexpr uint32_t kGdnTapeGateOffset =
    kGdnTapeKeyOffset + kLayers * kGdnTapeRows * kGdnKeyHeads * kGdnHeadDim;
constexpr uint32_t kGdnTapeFloats = kGdnTapeGateOffset + kLayers * kGdnTapeRows * kGdnValueHeads * 2;
constexpr uint32_t kGdnConvTapeElements =
    kLayers * kGdnTapeRows * (kGdnConvWidth - 1) * kGdnConvChannels;

static_assert(kAttnProjectionRows == 9216 && kAttnQGateRows == 8192 && kAttnVRowOffset == 8704);
static_assert(kGdnProjectionRows == 12352 && kGdnBRowOffset == 12288 && kGdnARowOffset == 12320);
static_assert(kGdnTapeKeyOffset == 40u * 16u * 32u * 128u &&
              kGdnTapeGateOffset == 40u * 16u * 32u * 128u + 40u * 16u * 16u * 128u &&
              kGdnTapeFloats == 40u * 16u * (32u * 128u + 16u * 128u + 64u));
static_assert(kGdnConvChannels == 8192 && kGdnKOffset == 2048 && kAttnRopePairs == 32);

}  // namespace tt
