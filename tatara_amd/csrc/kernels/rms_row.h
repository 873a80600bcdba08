// The arithmetic of the RMS row norm (rms_only.metal:5-43), shared by the norm kernel and
// by the projections that apply the norm while they stage their input rows, so that both
// produce the same bits: four squares summed in order per 4-value slice, slices summed by
// the adjacent-pairs tree, out = bf16(w * bf16(x * inverse)).
#pragma once

#include <stdint.h>

#include <hip/hip_runtime.h>

#include "../tt_constants.h"

namespace tt {

__device__ __forceinline__ float rms_widen(uint16_t h) {
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}
// round to nearest even with subnormal results flushed to signed zero
__device__ __forceinline__ uint16_t rms_store16(float v) {
    uint32_t b = __float_as_uint(v);
    if ((b & 0x7F800000u) == 0) b &= 0x80000000u;
    if ((b & 0x7F800000u) == 0x7F800000u) return static_cast<uint16_t>(b >> 16);
    const uint16_t h = static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
    return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u);
}
__device__ __forceinline__ uint16_t rms_fz16(uint16_t h) {
    return (h & 0x7F80u) ? h : static_cast<uint16_t>(h & 0x8000u);
}

// squares of a slice of four values (two packed dwords), summed in order
__device__ __forceinline__ float rms_slice_squares(uint32_t low, uint32_t high) {
    const float x0 = __uint_as_float(low << 16), x1 = __uint_as_float(low & 0xFFFF0000u);
    const float x2 = __uint_as_float(high << 16), x3 = __uint_as_float(high & 0xFFFF0000u);
    float sum = 0.0f;
    sum += x0 * x0;
    sum += x1 * x1;
    sum += x2 * x2;
    sum += x3 * x3;
    return sum;
}

__device__ __forceinline__ float rms_inverse(float total, uint32_t hidden) {
    return 1.0f / sqrtf(total / static_cast<float>(hidden) + kRmsNormEpsilon);
}

// two values of a row and their weights, packed: bf16(w * bf16(x * inverse)) of each
__device__ __forceinline__ uint32_t rms_scale_pair(uint32_t x_pair, uint32_t w_pair, float inverse) {
    const float x0 = __uint_as_float(x_pair << 16), x1 = __uint_as_float(x_pair & 0xFFFF0000u);
    const uint16_t s0 = rms_store16(x0 * inverse), s1 = rms_store16(x1 * inverse);
    const uint16_t r0 = rms_store16(rms_widen(rms_fz16(static_cast<uint16_t>(w_pair))) * rms_widen(s0));
    const uint16_t r1 = rms_store16(rms_widen(rms_fz16(static_cast<uint16_t>(w_pair >> 16))) * rms_widen(s1));
    return r0 | (static_cast<uint32_t>(r1) << 16);
}

}  // namespace tt
