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

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

} // namespace kutacc_dev
