// Element-wise kernels that sit between the operators in an Evoformer block, where a caller of the
// reference runs framework code on the host side: the mask bias 1e9*(mask-1) (the convention of reference
// src/attention/global_attention.cpp:120-121), the exchange of the two leading axes of a [n0, n1, c]
// activation (the "ending node" orientation of triangle attention, and the layout change between the
// triangle equation and its output step), the residual update, and the LayerNorm that follows the triangle
// equation, whose input is channel-first and whose output the next GEMM wants channel-last.  All are HBM-bound
// with 16-byte accesses when shapes allow.
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "launch_internal.h"
#include "mfma_tiles.h"
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

// LayerNorm over the channel axis of a channel-first tensor x[c][p] (128 channels, p contiguous), written
// channel-last: out[p][c] = LN_c(x[:, p]) * gamma[c] + beta[c].  Same arithmetic as the row LayerNorm (reference
// src/normalization/layernorm_kernel.h:21-53: shift by the first element, fp32 sums, clamped variance).  A wave
// takes 64 positions: 16 loads per lane of 8 positions x 1 channel (whole 128-byte lines per channel), an 8 x 8
// transposition over lanes turns each into 8 channels x 1 position, after which a lane owns all 128 channels of
// its position -- the statistics need no cross-lane step.  Rows leave through LDS as 256-byte runs.
__global__ __launch_bounds__(256) void layernorm_channel_first_bf16_kernel(const bf16_t *__restrict__ x, int64_t ld_x,
                                                                           const float *__restrict__ gamma,
                                                                           const float *__restrict__ beta,
                                                                           bf16_t *__restrict__ out, int64_t ld_out,
                                                                           int64_t positions, float eps)
{
    constexpr int C = 128, ROW_SLOTS = 17; // 16 slots of 16 bytes per row + 1 of padding
    __shared__ uint4 tile[4][64 * ROW_SLOTS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int kk = lane >> 3, mc = lane & 7;
    const int64_t p0 = ((int64_t)blockIdx.x * 4 + wave) * 64;
    if (p0 >= positions) {
        return;
    }
    int64_t pl = p0 + 8 * mc;
    const bool inside = pl < positions; // positions is a multiple of 8: a chunk is inside or outside as a whole
    pl = inside ? pl : positions - 8;
    uint4 v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        v[j] = *reinterpret_cast<const uint4 *>(x + (int64_t)(8 * j + kk) * ld_x + pl);
    }
    const uint32_t sel = transpose8x8_selector(lane);
    float s1 = 0.f, s2 = 0.f, x0 = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        v[j] = transpose8x8_lanes(v[j], sel); // now channels 8j..8j+7 of position pl + kk
        const bf16x8 b = as_bf16x8(v[j]);
        if (j == 0) {
            x0 = to_f32(b[0]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float d = to_f32(b[e]) - x0;
            s1 += d;
            s2 = fmaf(d, d, s2);
        }
    }
    const float n = (float)C;
    const float mean = s1 / n + x0;
    const float var = fmaxf((s2 - s1 * s1 / n) / n, 0.f);
    const float rstd = 1.0f / sqrtf(var + eps);
    const float shift = -rstd * mean;
    uint4 *rows = tile[wave];
    const int lds_row = kk * 8 + mc; // 16 consecutive lanes write 16 consecutive rows: no bank conflicts
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const bf16x8 b = as_bf16x8(v[j]);
        bf16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            o[e] = (bf16_t)fmaf(fmaf(to_f32(b[e]), rstd, shift), gamma[8 * j + e], beta[8 * j + e]);
        }
        rows[lds_row * ROW_SLOTS + j] = as_uint4(o);
    }
    // (LDS rows are private to the wave: no barrier.)  Row r' = 8 kk + mc holds position p0 + 8 mc + kk.
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int idx = i * 64 + lane;
        const int r = idx >> 4, chunk = idx & 15;
        const int64_t pos = p0 + 8 * (r & 7) + (r >> 3);
        if (pos < positions) {
            *reinterpret_cast<uint4 *>(out + pos * ld_out + chunk * 8) = rows[r * ROW_SLOTS + chunk];
        }
    }
}

// any channel count, any alignment: one thread per position, two passes over its channels
template <typename T>
__global__ __launch_bounds__(256) void layernorm_channel_first_kernel(const T *__restrict__ x, int64_t ld_x,
                                                                      const float *__restrict__ gamma,
                                                                      const float *__restrict__ beta, T *__restrict__ out,
                                                                      int64_t ld_out, int64_t channels, int64_t positions,
                                                                      float eps)
{
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= positions) {
        return;
    }
    const float x0 = to_f32(x[p]);
    float s1 = 0.f, s2 = 0.f;
    for (int64_t c = 0; c < channels; ++c) {
        const float d = to_f32(x[c * ld_x + p]) - x0;
        s1 += d;
        s2 = fmaf(d, d, s2);
    }
    const float n = (float)channels;
    const float mean = s1 / n + x0;
    const float var = fmaxf((s2 - s1 * s1 / n) / n, 0.f);
    const float rstd = 1.0f / sqrtf(var + eps);
    const float shift = -rstd * mean;
    for (int64_t c = 0; c < channels; ++c) {
        out[p * ld_out + c] = from_f32<T>(fmaf(fmaf(to_f32(x[c * ld_x + p]), rstd, shift), gamma[c], beta[c]));
    }
}

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
    if (row_bytes % 16 == 0 && kutacc_hip_aligned16(in) && kutacc_hip_aligned16(out)) {
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
    const bool vec = inner % vw == 0 && kutacc_hip_aligned16(acc) && kutacc_hip_aligned16(delta);
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

int layernorm_channel_first(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                            int64_t channels, int64_t positions, float eps, int32_t dtype, hipStream_t stream)
{
    if (!x || !gamma || !beta || !out || channels <= 0 || positions <= 0 || ld_x < positions || ld_out < channels ||
        (dtype != KUTACC_DTYPE_BF16 && dtype != KUTACC_DTYPE_FP32)) {
        return KUTACC_HIP_EINVAL;
    }
    kutacc_prof::KernelTimer t("layernorm_channel_first_kernel", 0.0, stream);
    unsigned blocks;
    if (dtype == KUTACC_DTYPE_BF16 && channels == 128 && positions % 8 == 0 && ld_x % 8 == 0 && ld_out % 8 == 0 &&
        kutacc_hip_aligned16(x) && kutacc_hip_aligned16(out)) {
        if (!grid_for(positions, blocks)) { // 256 positions per workgroup
            return KUTACC_HIP_EUNSUPPORTED;
        }
        layernorm_channel_first_bf16_kernel<<<blocks, 256, 0, stream>>>((const bf16_t *)x, ld_x, gamma, beta, (bf16_t *)out,
                                                                         ld_out, positions, eps);
        return kutacc_hip_status(hipGetLastError());
    }
    if (!grid_for(positions, blocks)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    if (dtype == KUTACC_DTYPE_BF16) {
        layernorm_channel_first_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t *)x, ld_x, gamma, beta, (bf16_t *)out,
                                                                            ld_out, channels, positions, eps);
    } else {
        layernorm_channel_first_kernel<float><<<blocks, 256, 0, stream>>>((const float *)x, ld_x, gamma, beta, (float *)out,
                                                                           ld_out, channels, positions, eps);
    }
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch
