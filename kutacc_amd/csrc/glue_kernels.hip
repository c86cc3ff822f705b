// Element-wise kernels that sit between the operators in an Evoformer block, where a caller of the
// reference runs framework code on the host side: the mask bias 1e9*(mask-1) (the convention of reference
// src/attention/global_attention.cpp:120-121), the exchange of the two leading axes of a [n0, n1, c]
// activation (the "ending node" orientation of triangle attention, and the layout change between the
// triangle equation and its output step), and the residual update.  All are HBM-bound copies with 16-byte
// accesses when shapes allow.
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "launch_internal.h"
#include "profiler.h"

namespace {
using namespace kutacc_dev;

// bias[i, j] = mask[i, j] * 1e9 - 1e9 in fp32 (one fused multiply-add, as the reference forms it), rounded to
// the storage type; transposed: bias[i, j] from mask[j, i] with mask stored [n1, n0]
template <typename T>
__global__ __launch_bounds__(256) void mask_bias_kernel(const T *__restrict__ mask, T *__restrict__ bias, int64_t n0,
                                                        int64_t n1, int transposed)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n0 * n1) {
        return;
    }
    const int64_t i = idx / n1, j = idx % n1;
    const float m = to_f32(mask[transposed ? j * n0 + i : idx]);
    bias[idx] = from_f32<T>(fmaf(m, 1e9f, -1e9f));
}

// out[j, i, :] = in[i, j, :]; one thread per 16-byte piece of the output, so writes are contiguous and reads come
// in runs of `inner` elements
template <typename V>
__global__ __launch_bounds__(256) void swap_axes_kernel(const V *__restrict__ in, V *__restrict__ out, int64_t n0, int64_t n1,
                                                        int64_t pieces)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n0 * n1 * pieces) {
        return;
    }
    const int64_t row = idx / pieces, piece = idx % pieces; // output row (j, i)
    const int64_t j = row / n0, i = row % n0;
    out[idx] = in[(i * n1 + j) * pieces + piece];
}

// acc[i, j, :] += delta[i, j, :] (or delta[j, i, :] when swapped, delta stored [n1, n0, c]); sum in fp32
template <typename T, int W>
__global__ __launch_bounds__(256) void residual_add_kernel(T *__restrict__ acc, const T *__restrict__ delta, int64_t n0,
                                                           int64_t n1, int64_t pieces, int swapped)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n0 * n1 * pieces) {
        return;
    }
    const int64_t row = idx / pieces, piece = idx % pieces;
    const int64_t i = row / n1, j = row % n1;
    const int64_t src = swapped ? (j * n0 + i) * pieces + piece : idx;
    struct alignas(sizeof(T) * W) Vec {
        T v[W];
    };
    Vec a = reinterpret_cast<const Vec *>(acc)[idx];
    const Vec d = reinterpret_cast<const Vec *>(delta)[src];
#pragma unroll
    for (int e = 0; e < W; ++e) {
        a.v[e] = from_f32<T>(to_f32(a.v[e]) + to_f32(d.v[e]));
    }
    reinterpret_cast<Vec *>(acc)[idx] = a;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline bool grid_for(int64_t work, unsigned &blocks)
{
    const int64_t b = (work + 255) / 256;
    if (b > INT32_MAX) {
        return false;
    }
    blocks = (unsigned)b;
    return true;
}
} // namespace

namespace kutacc_launch {

int mask_bias(const void *mask, void *bias, int64_t n0, int64_t n1, int transposed, int32_t dtype, hipStream_t stream)
{
    if (!mask || !bias || n0 <= 0 || n1 <= 0 || n0 > INT64_MAX / n1) {
        return KUTACC_HIP_EINVAL;
    }
    unsigned blocks;
    if (!grid_for(n0 * n1, blocks)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("mask_bias_kernel", 0.0, stream);
    if (dtype == KUTACC_DTYPE_BF16) {
        mask_bias_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t *)mask, (bf16_t *)bias, n0, n1, transposed);
    } else if (dtype == KUTACC_DTYPE_FP32) {
        mask_bias_kernel<float><<<blocks, 256, 0, stream>>>((const float *)mask, (float *)bias, n0, n1, transposed);
    } else {
        return KUTACC_HIP_EINVAL;
    }
    return kutacc_hip_status(hipGetLastError());
}

int swap_leading_axes(const void *in, void *out, int64_t n0, int64_t n1, int64_t inner, int32_t dtype, hipStream_t stream)
{
    if (!in || !out || in == out || n0 <= 0 || n1 <= 0 || inner <= 0 || n0 > INT64_MAX / n1 ||
        (dtype != KUTACC_DTYPE_BF16 && dtype != KUTACC_DTYPE_FP32)) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t esz = dtype == KUTACC_DTYPE_BF16 ? 2 : 4;
    const int64_t row_bytes = inner * esz;
    if (n0 * n1 > INT64_MAX / row_bytes) {
        return KUTACC_HIP_EINVAL;
    }
    unsigned blocks;
    kutacc_prof::KernelTimer t("swap_axes_kernel", 0.0, stream);
    if (row_bytes % 16 == 0 && aligned16(in) && aligned16(out)) {
        if (!grid_for(n0 * n1 * (row_bytes / 16), blocks)) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        swap_axes_kernel<uint4><<<blocks, 256, 0, stream>>>((const uint4 *)in, (uint4 *)out, n0, n1, row_bytes / 16);
    } else if (esz == 2) {
        if (!grid_for(n0 * n1 * inner, blocks)) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        swap_axes_kernel<uint16_t><<<blocks, 256, 0, stream>>>((const uint16_t *)in, (uint16_t *)out, n0, n1, inner);
    } else {
        if (!grid_for(n0 * n1 * inner, blocks)) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        swap_axes_kernel<uint32_t><<<blocks, 256, 0, stream>>>((const uint32_t *)in, (uint32_t *)out, n0, n1, inner);
    }
    return kutacc_hip_status(hipGetLastError());
}

int residual_add(void *acc, const void *delta, int64_t n0, int64_t n1, int64_t inner, int swapped, int32_t dtype,
                 hipStream_t stream)
{
    if (!acc || !delta || n0 <= 0 || n1 <= 0 || inner <= 0 || n0 > INT64_MAX / n1 || n0 * n1 > INT64_MAX / inner ||
        (dtype != KUTACC_DTYPE_BF16 && dtype != KUTACC_DTYPE_FP32)) {
        return KUTACC_HIP_EINVAL;
    }
    const int vw = dtype == KUTACC_DTYPE_BF16 ? 8 : 4; // elements per 16 bytes
    const bool vec = inner % vw == 0 && aligned16(acc) && aligned16(delta);
    unsigned blocks;
    if (!grid_for(n0 * n1 * (vec ? inner / vw : inner), blocks)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("residual_add_kernel", 0.0, stream);
    if (dtype == KUTACC_DTYPE_BF16) {
        if (vec) {
            residual_add_kernel<bf16_t, 8><<<blocks, 256, 0, stream>>>((bf16_t *)acc, (const bf16_t *)delta, n0, n1, inner / 8, swapped);
        } else {
            residual_add_kernel<bf16_t, 1><<<blocks, 256, 0, stream>>>((bf16_t *)acc, (const bf16_t *)delta, n0, n1, inner, swapped);
        }
    } else {
        if (vec) {
            residual_add_kernel<float, 4><<<blocks, 256, 0, stream>>>((float *)acc, (const float *)delta, n0, n1, inner / 4, swapped);
        } else {
            residual_add_kernel<float, 1><<<blocks, 256, 0, stream>>>((float *)acc, (const float *)delta, n0, n1, inner, swapped);
        }
    }
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch
