// Shape-agnostic HIP kernels of the gated-attention operator: any head_size, any seq_len, bf16 or
// fp32 storage, fp32 arithmetic throughout.  They follow the reference's data flow one to one --
// four projections into the caller's scratch, per-(batch, head, query) softmax attention with the
// sigmoid gate applied to the weighted average, output projection (reference
// src/attention/gating_attention.cpp:47-66, 73-150, 152-157) -- and exist for what no MFMA kernel
// takes (fp32 tensors beyond the fp32 kernel's reach, head sizes that are no multiple of 8 or above 64,
// scratch layouts the reference's kernel would not view as matrices) and as an independent kernel
// family for the tests.
// Logits and probabilities stay in fp32 registers; only q/k/v/gate/avg/out are rounded to the
// storage type, at the points where the reference stores them.
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "launch_internal.h"
#include "profiler.h"

using namespace kutacc_dev;

namespace {

constexpr int GEMM_TILE = 64; // output tile edge per workgroup
constexpr int GEMM_KB = 16;   // k-slab staged in LDS

// C[m, n] = beta*C[m, n] + sum_k A[m, k] * W[n, k] (+ bias[n]); element (m, n) of C at
// c[m*c_rs + n*c_cs], so a transposed result (the reference's v layout) is a stride choice.
template <typename T>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const T *__restrict__ a, int64_t lda, const T *__restrict__ w,
                                                     int64_t ldw, const float *__restrict__ bias, T *__restrict__ c,
                                                     int64_t c_rs, int64_t c_cs, int64_t m, int64_t n, int64_t k,
                                                     float beta)
{
    __shared__ float a_s[GEMM_KB][GEMM_TILE + 1];
    __shared__ float w_s[GEMM_KB][GEMM_TILE + 1];

    const int tid = threadIdx.x;
    const int tx = tid % 16; // 4 output columns each
    const int ty = tid / 16; // 4 output rows each
    const int64_t m0 = (int64_t)blockIdx.x * GEMM_TILE;
    const int64_t n0 = (int64_t)blockIdx.y * GEMM_TILE;

    float acc[4][4] = {};
    for (int64_t k0 = 0; k0 < k; k0 += GEMM_KB) {
        // 64 rows x 16 k per operand = 1024 elements, 4 per thread, k fastest for coalescing
        for (int i = tid; i < GEMM_TILE * GEMM_KB; i += 256) {
            const int r = i / GEMM_KB;
            const int kk = i % GEMM_KB;
            const int64_t gk = k0 + kk;
            const int64_t gm = m0 + r;
            const int64_t gn = n0 + r;
            a_s[kk][r] = (gm < m && gk < k) ? to_f32(a[gm * lda + gk]) : 0.f;
            w_s[kk][r] = (gn < n && gk < k) ? to_f32(w[gn * ldw + gk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GEMM_KB; ++kk) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                av[i] = a_s[kk][ty * 4 + i];
                wv[i] = w_s[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t gm = m0 + ty * 4 + i;
        if (gm >= m) {
            continue;
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t gn = n0 + tx * 4 + j;
            if (gn >= n) {
                continue;
            }
            float r = acc[i][j];
            if (bias != nullptr) {
                r += bias[gn];
            }
            T *dst = c + gm * c_rs + gn * c_cs;
            if (beta != 0.f) {
                r += beta * to_f32(*dst);
            }
            *dst = from_f32<T>(r);
        }
    }
}

constexpr int ATT_WAVES = 4; // queries per workgroup, one wavefront each
constexpr int ATT_DB = 32;   // head-dim block accumulated per pass over the keys

struct AttnParams {
    const void *q, *k, *v, *gate, *bias, *nb;
    void *avg;
    int64_t q_sb, q_ss, q_sh;
    int64_t k_sb, k_ss, k_sh;
    int64_t g_sb, g_ss, g_sh;
    int64_t a_sb, a_ss, a_sh;
    int64_t v_sh, v_se, v_sb;
    int64_t bias_sb, nb_sh, nb_sq;
    int64_t batch, seq, heads, hd;
    float scale;
};

// One wavefront per (batch, head, query).  Lanes stride over the keys.  Pass 1 finds the row
// maximum of x = (q.k*scale + bias[b,k]) + nb[h,q,k] (same association as reference
// gating_attention.cpp:109-118); pass 2 re-evaluates x per 32-wide slice of the head dimension and
// accumulates exp(x-max) and exp(x-max)*v in lane-private registers, reduced across the wave once.
template <typename T>
__global__ __launch_bounds__(64 * ATT_WAVES) void attention_rows_kernel(AttnParams p)
{
    extern __shared__ float q_rows[]; // [ATT_WAVES][hd]
    const int wave = threadIdx.x / 64;
    const int lane = threadIdx.x % 64;
    const int64_t bh = blockIdx.x;
    const int64_t b = bh / p.heads;
    const int64_t h = bh % p.heads;
    const int64_t qi = (int64_t)blockIdx.y * ATT_WAVES + wave;
    const bool active = qi < p.seq;
    const int64_t hd = p.hd;
    float *qs = q_rows + (int64_t)wave * hd;
    if (active) {
        const T *qrow = (const T *)p.q + b * p.q_sb + qi * p.q_ss + h * p.q_sh;
        for (int64_t e = lane; e < hd; e += 64) {
            qs[e] = to_f32(qrow[e]);
        }
    }
    __syncthreads(); // the only block-level barrier; waves past the last query leave after it
    if (!active) {
        return;
    }

    const T *kbase = (const T *)p.k + b * p.k_sb + h * p.k_sh;
    const T *bias_row = (const T *)p.bias + b * p.bias_sb;
    const T *nb_row = p.nb ? (const T *)p.nb + h * p.nb_sh + qi * p.nb_sq : nullptr;

    auto logit = [&](int64_t key) -> float {
        const T *kr = kbase + key * p.k_ss;
        float s = 0.f;
        for (int64_t e = 0; e < hd; ++e) {
            s = fmaf(qs[e], to_f32(kr[e]), s);
        }
        float x = s * p.scale + to_f32(bias_row[key]);
        if (nb_row) {
            x += to_f32(nb_row[key]);
        }
        return x;
    };

    float m = -INFINITY;
    for (int64_t key = lane; key < p.seq; key += 64) {
        m = fmaxf(m, logit(key));
    }
    m = wave_max(m);

    const T *grow = (const T *)p.gate + b * p.g_sb + qi * p.g_ss + h * p.g_sh;
    T *arow = (T *)p.avg + b * p.a_sb + qi * p.a_ss + h * p.a_sh;
    for (int64_t d0 = 0; d0 < hd; d0 += ATT_DB) {
        float o[ATT_DB];
#pragma unroll
        for (int e = 0; e < ATT_DB; ++e) {
            o[e] = 0.f;
        }
        float lsum = 0.f;
        const T *vbase = (const T *)p.v + h * p.v_sh + b * p.v_sb;
        for (int64_t key = lane; key < p.seq; key += 64) {
            const float pr = expf(logit(key) - m);
            lsum += pr;
#pragma unroll
            for (int e = 0; e < ATT_DB; ++e) {
                if (d0 + e < hd) {
                    o[e] = fmaf(pr, to_f32(vbase[(d0 + e) * p.v_se + key]), o[e]);
                }
            }
        }
        const float inv = 1.0f / wave_sum(lsum);
        float mine = 0.f;
#pragma unroll
        for (int e = 0; e < ATT_DB; ++e) {
            const float tot = wave_sum(o[e]);
            if (lane == e) {
                mine = tot;
            }
        }
        if (lane < ATT_DB && d0 + lane < hd) {
            // the reference stores the weighted average in the storage type before gating
            // (gating_attention.cpp:128-133), then multiplies by sigmoid(gate) and stores again (:141-145)
            const float wavg = to_f32(from_f32<T>(mine * inv));
            const float g = to_f32(grow[d0 + lane]);
            arow[d0 + lane] = from_f32<T>(wavg * (1.0f / (1.0f + expf(-g))));
        }
    }
}

template <typename T>
int launch_gemm_nt(const void *a, int64_t lda, const void *w, int64_t ldw, const float *bias, void *c, int64_t c_rs,
                   int64_t c_cs, int64_t m, int64_t n, int64_t k, float beta, hipStream_t stream)
{
    if (m <= 0 || n <= 0 || k <= 0) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t gx = (m + GEMM_TILE - 1) / GEMM_TILE;
    const int64_t gy = (n + GEMM_TILE - 1) / GEMM_TILE;
    if (gx > INT32_MAX || gy > 65535) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    gemm_nt_kernel<T><<<dim3((unsigned)gx, (unsigned)gy), 256, 0, stream>>>((const T *)a, lda, (const T *)w, ldw, bias,
                                                                          (T *)c, c_rs, c_cs, m, n, k, beta);
    return kutacc_hip_status(hipGetLastError());
}

template <typename T>
int run_generic(const kutacc_hip_attention_args_t &g, hipStream_t stream)
{
    const int64_t B = g.batch, S = g.seq_len, H = g.nheads, hd = g.head_size, C = H * hd, M = B * S;
    if (!g.q || !g.k || !g.v || !g.gate || !g.avg) {
        return KUTACC_HIP_EINVAL;
    }
    // q/k/gate/avg must be viewable as [B*S, C] matrices and v as [C, B*S], exactly the views the
    // reference builds for its GEMMs (gating_attention.cpp:50,55,60,65,153).
    if (g.q_stride_b != S * g.q_stride_s || g.k_stride_b != S * g.k_stride_s ||
        g.gate_stride_b != S * g.gate_stride_s || g.avg_stride_b != S * g.avg_stride_s || g.q_stride_h != hd ||
        g.k_stride_h != hd || g.gate_stride_h != hd || g.avg_stride_h != hd || g.v_stride_h != hd * g.v_stride_e ||
        g.v_stride_b != S || g.v_stride_e < M) {
        return KUTACC_HIP_EINVAL;
    }
    int rc;
    const double proj_flops = 2.0 * (double)M * (double)C * (double)C;
    {
        kutacc_prof::KernelTimer t("generic_projections_qkvg", 4.0 * proj_flops, stream);
        if ((rc = launch_gemm_nt<T>(g.input, g.input_ld, g.query_w, C, nullptr, g.q, g.q_stride_s, 1, M, C, C, 0.f,
                                    stream))) {
            return rc;
        }
        if ((rc = launch_gemm_nt<T>(g.input, g.input_ld, g.key_w, C, nullptr, g.k, g.k_stride_s, 1, M, C, C, 0.f,
                                    stream))) {
            return rc;
        }
        if ((rc = launch_gemm_nt<T>(g.input, g.input_ld, g.value_w, C, nullptr, g.v, 1, g.v_stride_e, M, C, C, 0.f,
                                    stream))) {
            return rc;
        }
        if ((rc = launch_gemm_nt<T>(g.input, g.input_ld, g.gating_w, C, g.gating_b, g.gate, g.gate_stride_s, 1, M, C, C,
                                    0.f, stream))) {
            return rc;
        }
    }
    AttnParams p;
    p.q = g.q, p.k = g.k, p.v = g.v, p.gate = g.gate, p.bias = g.bias, p.nb = g.nonbatched_bias, p.avg = g.avg;
    p.q_sb = g.q_stride_b, p.q_ss = g.q_stride_s, p.q_sh = g.q_stride_h;
    p.k_sb = g.k_stride_b, p.k_ss = g.k_stride_s, p.k_sh = g.k_stride_h;
    p.g_sb = g.gate_stride_b, p.g_ss = g.gate_stride_s, p.g_sh = g.gate_stride_h;
    p.a_sb = g.avg_stride_b, p.a_ss = g.avg_stride_s, p.a_sh = g.avg_stride_h;
    p.v_sh = g.v_stride_h, p.v_se = g.v_stride_e, p.v_sb = g.v_stride_b;
    p.bias_sb = g.bias_stride_b, p.nb_sh = g.nb_stride_h, p.nb_sq = g.nb_stride_q;
    p.batch = B, p.seq = S, p.heads = H, p.hd = hd;
    // same evaluation as the reference: (float)(1 / sqrt(head_size)) in double (gating_attention.cpp:68)
    p.scale = (float)(1.0 / sqrt((double)hd));
    const int64_t qtiles = (S + ATT_WAVES - 1) / ATT_WAVES;
    if (B * H > INT32_MAX || qtiles > 65535 || hd * ATT_WAVES * 4 > 48 * 1024) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    {
        kutacc_prof::KernelTimer t("generic_attention_rows", 4.0 * (double)B * (double)S * (double)S * (double)C, stream);
        attention_rows_kernel<T><<<dim3((unsigned)(B * H), (unsigned)qtiles), 64 * ATT_WAVES,
                                   (size_t)(hd * ATT_WAVES * sizeof(float)), stream>>>(p);
        if ((rc = kutacc_hip_status(hipGetLastError()))) {
            return rc;
        }
    }
    kutacc_prof::KernelTimer t("generic_output_projection", proj_flops, stream);
    return launch_gemm_nt<T>(g.avg, g.avg_stride_s, g.output_w, C, g.output_b, g.out, g.out_ld, 1, M, C, C, 0.f, stream);
}

} // namespace

namespace kutacc_launch {

int gating_attention_generic(const kutacc_hip_attention_args_t &g, hipStream_t stream)
{
    if (g.dtype == KUTACC_DTYPE_BF16) {
        return run_generic<bf16_t>(g, stream);
    }
    if (g.dtype == KUTACC_DTYPE_FP32) {
        return run_generic<float>(g, stream);
    }
    return KUTACC_HIP_EINVAL;
}

int gemm_nt(int32_t dtype, const void *a, int64_t lda, const void *w, int64_t ldw, const float *bias, void *c,
            int64_t c_rs, int64_t c_cs, int64_t m, int64_t n, int64_t k, float beta, hipStream_t stream)
{
    if (dtype == KUTACC_DTYPE_BF16) {
        return launch_gemm_nt<bf16_t>(a, lda, w, ldw, bias, c, c_rs, c_cs, m, n, k, beta, stream);
    }
    if (dtype == KUTACC_DTYPE_FP32) {
        return launch_gemm_nt<float>(a, lda, w, ldw, bias, c, c_rs, c_cs, m, n, k, beta, stream);
    }
    return KUTACC_HIP_EINVAL;
}

} // namespace kutacc_launch
