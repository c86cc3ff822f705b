// Row-wise HBM-bound kernels that sit in front of the attention operator: LayerNorm over the last
// axis, and the fused pair-bias producer LN(z) -> [H, c_z] projection -> [H, S, S] layout.
// Arithmetic follows reference src/normalization/layernorm_kernel.h:21-53 (shift by the first
// element, fp32 sum and sum of squares, clamped variance, rstd, then (x*rstd - rstd*mean)*gamma+beta)
// and reference src/linear/linear.cpp:21-42 (bf16 operands, result rounded to the storage type).
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "launch_internal.h"

using namespace kutacc_dev;

namespace {

constexpr int ROW_WAVES = 4; // rows per workgroup, one wavefront each

// Per-row statistics exactly as the reference forms them; every lane returns the same values.
template <typename T>
__device__ __forceinline__ void row_stats(const T *__restrict__ row, int64_t size, int lane, float eps, float &rstd,
                                          float &shift)
{
    const float delta = to_f32(row[0]);
    float s1 = 0.f, s2 = 0.f;
    for (int64_t i = lane; i < size; i += 64) {
        const float v = to_f32(row[i]) - delta;
        s1 += v;
        s2 = fmaf(v, v, s2);
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    const float n = (float)size;
    const float mean = s1 / n + delta;
    const float var = fmaxf((s2 - s1 * s1 / n) / n, 0.f);
    rstd = 1.0f / sqrtf(var + eps);
    shift = -rstd * mean;
}

template <typename T>
__global__ __launch_bounds__(64 * ROW_WAVES) void layernorm_rows_kernel(const T *__restrict__ x, int64_t ld_x,
                                                                       const float *__restrict__ gamma,
                                                                       const float *__restrict__ beta,
                                                                       T *__restrict__ out, int64_t ld_out,
                                                                       int64_t rows, int64_t size, float eps)
{
    const int lane = threadIdx.x % 64;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + threadIdx.x / 64;
    if (r >= rows) {
        return;
    }
    const T *row = x + r * ld_x;
    float rstd, shift;
    row_stats(row, size, lane, eps, rstd, shift);
    T *orow = out + r * ld_out;
    for (int64_t i = lane; i < size; i += 64) {
        const float v = fmaf(to_f32(row[i]), rstd, shift);
        orow[i] = from_f32<T>(fmaf(v, gamma[i], beta[i]));
    }
}

// One wavefront per (i, j) row of z.  The normalised row is rounded to the storage type first (that
// is what a caller of the reference would hand to kutacc_af2_linear), then dotted with each of the
// H weight rows; nb[h, i, j] is written in place of the caller-side [S, S, H] -> [H, S, S] permute.
template <typename T>
__global__ __launch_bounds__(64 * ROW_WAVES) void pair_bias_kernel(const T *__restrict__ z,
                                                                  const float *__restrict__ gamma,
                                                                  const float *__restrict__ beta,
                                                                  const T *__restrict__ w, T *__restrict__ nb,
                                                                  T *__restrict__ z_norm, int64_t rows_i,
                                                                  int64_t rows_j, int64_t c_z, int64_t nheads, float eps)
{
    const int lane = threadIdx.x % 64;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + threadIdx.x / 64;
    const int64_t rows = rows_i * rows_j;
    if (r >= rows) {
        return;
    }
    const T *row = z + r * c_z;
    float rstd, shift;
    row_stats(row, c_z, lane, eps, rstd, shift);
    for (int64_t h0 = 0; h0 < nheads; h0 += 8) {
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        for (int64_t c = lane; c < c_z; c += 64) {
            const float v = fmaf(to_f32(row[c]), rstd, shift);
            const T vn = from_f32<T>(fmaf(v, gamma[c], beta[c]));
            if (z_norm != nullptr && h0 == 0) {
                z_norm[r * c_z + c] = vn;
            }
            const float vf = to_f32(vn);
#pragma unroll
            for (int hh = 0; hh < 8; ++hh) {
                if (h0 + hh < nheads) {
                    acc[hh] = fmaf(vf, to_f32(w[(h0 + hh) * c_z + c]), acc[hh]);
                }
            }
        }
#pragma unroll
        for (int hh = 0; hh < 8; ++hh) {
            if (h0 + hh < nheads) {
                const float tot = wave_sum(acc[hh]);
                if (lane == 0) {
                    nb[(h0 + hh) * rows + r] = from_f32<T>(tot);
                }
            }
        }
    }
}

template <typename T>
int launch_layernorm(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                     int64_t rows, int64_t size, float eps, hipStream_t stream)
{
    const int64_t blocks = (rows + ROW_WAVES - 1) / ROW_WAVES;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    layernorm_rows_kernel<T><<<(unsigned)blocks, 64 * ROW_WAVES, 0, stream>>>((const T *)x, ld_x, gamma, beta, (T *)out,
                                                                               ld_out, rows, size, eps);
    return kutacc_hip_status(hipGetLastError());
}

template <typename T>
int launch_pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
                     int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, hipStream_t stream)
{
    const int64_t rows = rows_i * rows_j;
    const int64_t blocks = (rows + ROW_WAVES - 1) / ROW_WAVES;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    pair_bias_kernel<T><<<(unsigned)blocks, 64 * ROW_WAVES, 0, stream>>>(
        (const T *)z, gamma, beta, (const T *)w, (T *)nb, (T *)z_norm, rows_i, rows_j, c_z, nheads, eps);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace

namespace kutacc_launch {

int layernorm_rows(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                   int64_t rows, int64_t size, float eps, int32_t dtype, hipStream_t stream)
{
    if (!x || !gamma || !beta || !out || rows <= 0 || size <= 0 || ld_x < size || ld_out < size) {
        return KUTACC_HIP_EINVAL;
    }
    if (dtype == KUTACC_DTYPE_BF16) {
        return launch_layernorm<bf16_t>(x, ld_x, gamma, beta, out, ld_out, rows, size, eps, stream);
    }
    if (dtype == KUTACC_DTYPE_FP32) {
        return launch_layernorm<float>(x, ld_x, gamma, beta, out, ld_out, rows, size, eps, stream);
    }
    return KUTACC_HIP_EINVAL;
}

int pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
              int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int32_t dtype,
              hipStream_t stream)
{
    if (!z || !gamma || !beta || !w || !nb || rows_i <= 0 || rows_j <= 0 || c_z <= 0 || nheads <= 0) {
        return KUTACC_HIP_EINVAL;
    }
    if (dtype == KUTACC_DTYPE_BF16) {
        return launch_pair_bias<bf16_t>(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, stream);
    }
    if (dtype == KUTACC_DTYPE_FP32) {
        return launch_pair_bias<float>(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, stream);
    }
    return KUTACC_HIP_EINVAL;
}

} // namespace kutacc_launch
