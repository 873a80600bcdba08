// Cross-lane sums of the kernels: butterflies over a half wave (32 lanes) and over a row
// (16 lanes), and the quad gather that feeds them.
#pragma once

#include <type_traits>

#include <hip/hip_runtime.h>

namespace tt {

template <int kControl>
__device__ __forceinline__ float lane_dpp(float v) {
    return __int_as_float(
        __builtin_amdgcn_update_dpp(0, __float_as_int(v), kControl, 0xF, 0xF, false));
}

// Sum over the 16 lanes of a row, every lane receiving it, as the xor butterfly (1, 2, 4,
// 8) - the adjacent-pairs tree.  The partner of the first two steps comes through quad
// permutes; after them a quad holds one value, so the mirror of a half row (lane 7 - i)
// and of a row (lane 15 - i) deliver what lanes i ^ 4 and i ^ 8 hold.  Same sums bit for
// bit as four __shfl_xor steps (fp addition commutes), without their LDS-permute round
// trips.
__device__ __forceinline__ float row_sum(float v) {
    v += lane_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
    v += lane_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
    v += lane_dpp<0x141>(v);   // row_half_mirror
    v += lane_dpp<0x140>(v);   // row_mirror
    return v;
}

// The same over the 32 lanes of a half wave (xor 1 .. 16): the last step swaps the two
// rows of the half wave with a bit-mask swizzle.
__device__ __forceinline__ float half_wave_sum(float v) {
    v = row_sum(v);
    v += __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), 0x401F));  // lane ^ 16
    return v;
}

// The value quad lane kLane holds, in every lane of its quad: on lane 4k that is what
// __shfl_down by kLane delivers.
template <int kLane>
__device__ __forceinline__ float quad_lane(float v) {
    return lane_dpp<kLane * 0x55>(v);
}

}  // namespace tt
