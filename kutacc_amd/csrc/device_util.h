// Small device-side helpers shared by the HIP translation units: storage-type loads/stores with
// the library's rounding rule (fp32 -> bf16 is round-to-nearest-even, bf16 -> fp32 is exact, as in
// reference src/wrapper/svcvt.h:23-37), wavefront reductions for 64-wide waves, error mapping.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kutacc_hip.h"

namespace kutacc_dev {

typedef __bf16 bf16_t;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v)
{
    return v;
}
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v)
{
    return (bf16_t)v; // v_cvt_pk_bf16_f32: round to nearest even
}

__device__ __forceinline__ float wave_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off, 64));
    }
    return v;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    return v;
}

// lane-group sums without LDS: a row spread over LPR consecutive lanes (LPR = 8, 16, 32 or 64)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v)
{
    const int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(moved);
}

// sum over the LPR lanes that hold one row; every lane of the group gets the total
template <int LPR>
__device__ __forceinline__ float group_sum(float v)
{
    v = dpp_add<0xB1>(v);  // quad_perm [1,0,3,2]: lane ^ 1
    v = dpp_add<0x4E>(v);  // quad_perm [2,3,0,1]: lane ^ 2
    v = dpp_add<0x141>(v); // row_half_mirror: pairs the two quads of 8 lanes
    if (LPR >= 16) {
        v = dpp_add<0x140>(v); // row_mirror: pairs the two halves of 16 lanes
    }
    if (LPR >= 32) {
        v += __shfl_xor(v, 16, 64);
    }
    if (LPR >= 64) {
        v += __shfl_xor(v, 32, 64);
    }
    return v;
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

} // namespace kutacc_dev
