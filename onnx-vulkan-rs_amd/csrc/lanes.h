// Cross-lane reductions of a 64-wide wavefront on the vector unit alone (DPP row operations and
// v_readlane): no LDS round trip, a handful of instructions each.
#pragma once
#include <hip/hip_runtime.h>

namespace hipc {

template <int CTRL>
__device__ __forceinline__ float lean_dpp(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
// every lane ends with the sum (maximum) of its row of 16 lanes: neighbours, pairs, then rotations by 4 and 8
__device__ __forceinline__ float lean_row_sum(float v) {
    v += lean_dpp<0xB1>(v);    // quad_perm [1,0,3,2]
    v += lean_dpp<0x4E>(v);    // quad_perm [2,3,0,1]
    v += lean_dpp<0x124>(v);   // row_ror:4
    v += lean_dpp<0x128>(v);   // row_ror:8
    return v;
}
__device__ __forceinline__ float lean_row_max(float v) {
    v = fmaxf(v, lean_dpp<0xB1>(v));
    v = fmaxf(v, lean_dpp<0x4E>(v));
    v = fmaxf(v, lean_dpp<0x124>(v));
    v = fmaxf(v, lean_dpp<0x128>(v));
    return v;
}
__device__ __forceinline__ float lean_lane(float v, int l) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
}
__device__ __forceinline__ float lean_wave_sum(float v) {
    v = lean_row_sum(v);
    return (lean_lane(v, 0) + lean_lane(v, 16)) + (lean_lane(v, 32) + lean_lane(v, 48));
}
__device__ __forceinline__ float lean_wave_max(float v) {
    v = lean_row_max(v);
    return fmaxf(fmaxf(lean_lane(v, 0), lean_lane(v, 16)), fmaxf(lean_lane(v, 32), lean_lane(v, 48)));
}


}  // namespace hipc
