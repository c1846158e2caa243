// Wave64 cross-lane reductions for gfx950 built from DPP row operations, one ds_swizzle
// and two readlanes - no LDS traffic and no barriers inside a wave.
#pragma once
#include <hip/hip_runtime.h>

namespace mrk::dev {

struct MaxOp {
    __device__ static float apply(float a, float b) { return fmaxf(a, b); }
};
struct SumOp {
    __device__ static float apply(float a, float b) { return a + b; }
};

template <int kCtrl>
__device__ __forceinline__ float dpp_move(float v) {
    int i = __builtin_bit_cast(int, v);
    i = __builtin_amdgcn_update_dpp(i, i, kCtrl, 0xf, 0xf, false);
    return __builtin_bit_cast(float, i);
}

// All 64 lanes receive the reduction of `v` over the wave.
template <class Op>
__device__ __forceinline__ float wave_reduce(float v) {
    v = Op::apply(v, dpp_move<0xB1>(v));   // quad_perm [1,0,3,2]  : lane ^ 1
    v = Op::apply(v, dpp_move<0x4E>(v));   // quad_perm [2,3,0,1]  : lane ^ 2
    v = Op::apply(v, dpp_move<0x141>(v));  // row_half_mirror      : joins the two quads of 8
    v = Op::apply(v, dpp_move<0x140>(v));  // row_mirror           : joins the two halves of 16
    // swap with lane ^ 16 inside each group of 32: and_mask 0x1f, or 0, xor 0x10
    float w = __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));
    v = Op::apply(v, w);
    float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 0));
    float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 32));
    return Op::apply(lo, hi);
}

}  // namespace mrk::dev
