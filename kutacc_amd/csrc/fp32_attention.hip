// Gated attention for fp32 storage on the fp32 matrix core (v_mfma_f32_32x32x2_f32), head_size 32, short sequences.
//
// The reference serves every call through its GEMM (src/linear/mm.cpp:77-86); the bf16 kernels of fused_attention.hip
// take bf16 storage only, and an fp32 tensor rounded to bf16 operands would miss the fp32 bar (1e-4 relative).  The
// fp32 MFMA multiplies fp32 operands exactly and accumulates in fp32, at a sixteenth of the bf16 rate -- enough for the
// small fp32 problems (the MSA-row benchmark shape is 0.74 GFLOP), which are bound by latency, not by arithmetic.
//
//   fp32_head_kernel     one workgroup of four waves per (batch row b, head h): the four projections of the head
//       (K, V, Q, gate -- one matrix per wave, the input rows staged through LDS 32 positions at a time), then
//       flash-style attention with a running maximum, one 32-query block per wave at a time, the sigmoid gate, and the
//       gated average stored where the reference leaves it (src/attention/gating_attention.cpp:47-66, 73-150).
//       q, k, v, gate, logits and probabilities never leave the chip.
//   fp32_rows_gemm_kernel   out[m, n] = sum_k a[m, k] * w[n, k] + bias[n], one 32 x 32 tile per wave: the output
//       projection (reference :152-157).
//
// Operand and accumulator layouts of the 32x32x2 MFMA: A is 32 x 2, lane l holds A[l % 32][l / 32]; B is 2 x 32, lane l
// holds B[l / 32][l % 32]; D[i][j] sits in lane j + 32 g, register v with i = 8 (v / 4) + 4 g + v % 4.  As in the bf16
// kernels, products are formed transposed (rows = keys or head dims, columns = queries) so that an accumulator is the
// next product's B operand as it stands: register v of the probabilities is the k-step of P.V whose two keys are the
// ones that register holds in the two halves of the wave.
#include <hip/hip_runtime.h>

#include <climits>
#include <cmath>

#include "device_util.h"
#include "launch_internal.h"
#include "profiler.h"

using namespace kutacc_dev;

namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int HEAD = 32;
constexpr int LDP = 33;            // row pitch of the [position][feature] arrays in LDS, in floats: odd, so a column read is conflict-free
constexpr int MAX_SEQ = 224;       // what the LDS holds of K, V, Q and gate of one head in fp32
constexpr int MAX_CHANNELS = 256;  // input rows are staged 32 positions x C channels at a time
constexpr float LOG2E_F = 1.44269504088896340736f;

__device__ __forceinline__ f32x16 mfma_f32(float a, float b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }

__device__ __forceinline__ float swap_halves_max(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float swap_halves_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

struct Fp32Params {
    const float *x, *wq, *wk, *wv, *wg, *bg, *bias, *nb;
    float *avg;
    int64_t x_ld, bias_sb, nb_sh, nb_sq, avg_sb, avg_ss, avg_sh;
    int B, S, H, C;
    int nb_vec; // pair-bias rows may be read with 16-byte loads
    float scale;
};

__global__ __launch_bounds__(256) void fp32_head_kernel(Fp32Params p)
{
    extern __shared__ float lds_f[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int S = p.S, C = p.C, NB = (S + 31) / 32, S32 = NB * 32;
    const int b = blockIdx.x / p.H, h = blockIdx.x % p.H;
    const int XP = C + 4; // staged input rows: 16 bytes of padding per row, so that 16 lanes reading 16 bytes of 16 rows hit 16 bank groups

    float *xs = lds_f;             // [32][XP]
    float *ks = xs + 32 * XP;      // [S32][LDP]
    float *vs = ks + S32 * LDP;    // [S32][LDP]
    float *qs = vs + S32 * LDP;    // [S32][LDP], scaled by 1/sqrt(d)
    float *gs = qs + S32 * LDP;    // [S32][LDP], sigmoid applied
    float *ms = gs + S32 * LDP;    // [S32] mask bias, -inf past S

    for (int k = tid; k < S32; k += 256) {
        ms[k] = k < S ? p.bias[(int64_t)b * p.bias_sb + k] : -INFINITY;
    }

    // ---- projections: wave w forms matrix w of the head for 32 positions at a time ----
    const float *xb = p.x + (int64_t)b * S * p.x_ld;
    const float *wmat = wave == 0 ? p.wk : wave == 1 ? p.wv : wave == 2 ? p.wq : p.wg;
    float *dst = wave == 0 ? ks : wave == 1 ? vs : wave == 2 ? qs : gs;
    const float *wrow = wmat + (int64_t)(h * HEAD + r) * C + 4 * g; // this lane's weight row, its half of every 8 channels
    const float gate_bias = p.bg[h * HEAD + r];
    const int c4 = C / 4;
    for (int t = 0; t < NB; ++t) {
        __syncthreads(); // the previous tile's readers are done with xs
        for (int idx = tid; idx < 32 * c4; idx += 256) {
            const int row = idx / c4, cc = idx % c4;
            const int pos = t * 32 + row < S ? t * 32 + row : S - 1;
            *reinterpret_cast<f32x4 *>(xs + row * XP + 4 * cc) = *reinterpret_cast<const f32x4 *>(xb + (int64_t)pos * p.x_ld + 4 * cc);
        }
        __syncthreads();
        f32x16 acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            acc[v] = wave == 3 ? gate_bias : 0.f; // D[position][feature]: a lane's registers all belong to feature r
        }
        const float *xrow = xs + r * XP + 4 * g;
#pragma unroll 4
        for (int c0 = 0; c0 < C; c0 += 8) {
            const f32x4 xa = *reinterpret_cast<const f32x4 *>(xrow + c0);
            const f32x4 wb = *reinterpret_cast<const f32x4 *>(wrow + c0);
            acc = mfma_f32(xa[0], wb[0], acc);
            acc = mfma_f32(xa[1], wb[1], acc);
            acc = mfma_f32(xa[2], wb[2], acc);
            acc = mfma_f32(xa[3], wb[3], acc);
        }
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float val = acc[v];
            if (wave == 2) {
                val *= p.scale;
            } else if (wave == 3) {
                val = 1.0f / (1.0f + __builtin_amdgcn_exp2f(-val * LOG2E_F));
            }
            dst[(t * 32 + 8 * (v >> 2) + 4 * g + (v & 3)) * LDP + r] = val;
        }
    }
    __syncthreads();

    // ---- attention: one 32-query block per wave at a time ----
    for (int qt = wave; qt < NB; qt += 4) {
        float qop[16]; // Q^T operand: this lane's query, head dims 2 i + g
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            qop[i] = qs[(qt * 32 + r) * LDP + 2 * i + g];
        }
        const int qpos = qt * 32 + r;
        const int qrow = qpos < S ? qpos : S - 1;
        const float *nbrow = p.nb != nullptr ? p.nb + (int64_t)h * p.nb_sh + (int64_t)qrow * p.nb_sq + 4 * g : nullptr;
        float m_run = -INFINITY, lsum = 0.f;
        f32x16 o;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            o[v] = 0.f;
        }
        for (int kt = 0; kt < NB; ++kt) {
            f32x16 x;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                x[v] = 0.f;
            }
            const float *krow = ks + (kt * 32 + r) * LDP + g;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                x = mfma_f32(krow[2 * i], qop[i], x); // logits^T: rows = keys, columns = queries
            }
            // (logit * scale + bias[b, k]) + nb[h, q, k], in that order (reference :109-118); register v holds key
            // 32 kt + 8 (v / 4) + 4 g + v % 4
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const int key0 = kt * 32 + 8 * a + 4 * g;
                const f32x4 mv = *reinterpret_cast<const f32x4 *>(ms + key0);
                f32x4 nv = {0.f, 0.f, 0.f, 0.f};
                if (nbrow != nullptr) {
                    if (p.nb_vec && key0 + 4 <= S) {
                        nv = *reinterpret_cast<const f32x4 *>(nbrow + kt * 32 + 8 * a);
                    } else {
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            nv[c] = key0 + c < S ? nbrow[kt * 32 + 8 * a + c] : 0.f;
                        }
                    }
                }
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x[4 * a + c] = (x[4 * a + c] + mv[c]) + nv[c];
                }
            }
            float mx = x[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) {
                mx = fmaxf(mx, x[v]);
            }
            mx = swap_halves_max(mx);
            const float m_new = fmaxf(m_run, mx); // finite: every tile has a key below S, whose bias is finite
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E_F);
            m_run = m_new;
            float psum = 0.f;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                x[v] = __builtin_amdgcn_exp2f((x[v] - m_new) * LOG2E_F);
                psum += x[v];
                o[v] *= alpha;
            }
            lsum = lsum * alpha + psum;
            // O^T += V^T . P^T: k-step v pairs the two keys register v holds in the two halves of the wave
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                o = mfma_f32(vs[(kt * 32 + 8 * (v >> 2) + 4 * g + (v & 3)) * LDP + r], x[v], o);
            }
        }
        const float inv = 1.0f / swap_halves_sum(lsum);
        if (qpos < S) {
            float *out = p.avg + (int64_t)b * p.avg_sb + (int64_t)qpos * p.avg_ss + (int64_t)h * p.avg_sh + 4 * g;
            const float *grow = gs + qpos * LDP + 4 * g;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                f32x4 ov;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    ov[c] = o[4 * a + c] * inv * grow[8 * a + c]; // register 4 a + c is head dim 8 a + 4 g + c
                }
                *reinterpret_cast<f32x4 *>(out + 8 * a) = ov;
            }
        }
    }
}

// out[m, n] = sum_k a[m, k] * w[n, k] + bias[n]; one 32 x 32 tile per wave, four tiles along n per workgroup.  k is a
// multiple of 8; rows are 16-byte aligned.
__global__ __launch_bounds__(256) void fp32_rows_gemm_kernel(const float *__restrict__ a, int64_t a_ld, const float *__restrict__ w,
                                                             int64_t w_ld, const float *__restrict__ bias, float *__restrict__ out,
                                                             int64_t out_ld, int64_t M, int N, int K)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int64_t m0 = (int64_t)blockIdx.x * 32;
    const int n0 = (blockIdx.y * 4 + wave) * 32;
    if (n0 >= N) {
        return;
    }
    const int64_t arow = m0 + r < M ? m0 + r : M - 1;
    const int wrow_i = n0 + r < N ? n0 + r : N - 1;
    const float *ap = a + arow * a_ld + 4 * g;
    const float *wp = w + (int64_t)wrow_i * w_ld + 4 * g;
    f32x16 acc;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        acc[v] = 0.f;
    }
#pragma unroll 4
    for (int k0 = 0; k0 < K; k0 += 8) {
        const f32x4 av = *reinterpret_cast<const f32x4 *>(ap + k0);
        const f32x4 wv = *reinterpret_cast<const f32x4 *>(wp + k0);
        acc = mfma_f32(av[0], wv[0], acc);
        acc = mfma_f32(av[1], wv[1], acc);
        acc = mfma_f32(av[2], wv[2], acc);
        acc = mfma_f32(av[3], wv[3], acc);
    }
    if (n0 + r < N) {
        const float bv = bias != nullptr ? bias[n0 + r] : 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int64_t m = m0 + 8 * (v >> 2) + 4 * g + (v & 3);
            if (m < M) {
                out[m * out_ld + n0 + r] = acc[v] + bv;
            }
        }
    }
}

inline bool aligned16(const void *ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

size_t head_kernel_lds(int S, int C)
{
    const int S32 = (S + 31) / 32 * 32;
    return (size_t)(32 * (C + 4) + 4 * S32 * LDP + S32) * sizeof(float);
}

} // namespace

namespace kutacc_launch {

bool fp32_attention_supports(const kutacc_hip_attention_args_t &a)
{
    if (a.dtype != KUTACC_DTYPE_FP32 || a.head_size != HEAD || a.batch <= 0 || a.seq_len <= 0 || a.seq_len > MAX_SEQ) {
        return false;
    }
    const int64_t C = a.nheads * a.head_size;
    if (C > MAX_CHANNELS || a.batch * a.nheads > INT32_MAX || a.batch * a.seq_len > INT32_MAX) {
        return false;
    }
    // 16-byte loads of input and weight rows, 16-byte stores of the gated average
    if (a.input_ld % 4 != 0 || a.avg_stride_b % 4 != 0 || a.avg_stride_s % 4 != 0 || a.avg_stride_h % 4 != 0 || !aligned16(a.input) ||
        !aligned16(a.query_w) || !aligned16(a.key_w) || !aligned16(a.value_w) || !aligned16(a.gating_w) || !aligned16(a.output_w) ||
        !aligned16(a.avg)) {
        return false;
    }
    // the output projection reads the gated average as [batch * seq_len] rows of C values
    return a.avg_stride_h == HEAD && a.avg_stride_b == a.seq_len * a.avg_stride_s && a.avg_stride_s >= C;
}

int gating_attention_fp32(const kutacc_hip_attention_args_t &a, hipStream_t stream)
{
    if (!fp32_attention_supports(a)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    const int C = (int)(a.nheads * a.head_size);
    Fp32Params p;
    p.x = (const float *)a.input, p.wq = (const float *)a.query_w, p.wk = (const float *)a.key_w, p.wv = (const float *)a.value_w;
    p.wg = (const float *)a.gating_w, p.bg = a.gating_b, p.bias = (const float *)a.bias, p.nb = (const float *)a.nonbatched_bias;
    p.avg = (float *)a.avg;
    p.x_ld = a.input_ld, p.bias_sb = a.bias_stride_b, p.nb_sh = a.nb_stride_h, p.nb_sq = a.nb_stride_q;
    p.avg_sb = a.avg_stride_b, p.avg_ss = a.avg_stride_s, p.avg_sh = a.avg_stride_h;
    p.B = (int)a.batch, p.S = (int)a.seq_len, p.H = (int)a.nheads, p.C = C;
    p.nb_vec = (p.nb != nullptr && aligned16(p.nb) && a.nb_stride_h % 4 == 0 && a.nb_stride_q % 4 == 0) ? 1 : 0;
    p.scale = (float)(1.0 / sqrt((double)a.head_size)); // reference gating_attention.cpp:68
    const size_t lds_bytes = head_kernel_lds(p.S, C);
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    {
        const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(fp32_head_kernel), lds_bytes, configured);
        if (e != hipSuccess) {
            return (int)e;
        }
    }
    const double BS = (double)a.batch * (double)a.seq_len;
    {
        kutacc_prof::KernelTimer t("fp32_head_kernel", 8.0 * BS * C * C + 4.0 * BS * (double)a.seq_len * C, stream);
        fp32_head_kernel<<<dim3((unsigned)(a.batch * a.nheads)), 256, lds_bytes, stream>>>(p);
        const int rc = kutacc_hip_status(hipGetLastError());
        if (rc != 0) {
            return rc;
        }
    }
    const int64_t M = a.batch * a.seq_len;
    kutacc_prof::KernelTimer t("fp32_rows_gemm_kernel", 2.0 * BS * C * C, stream);
    const dim3 grid((unsigned)((M + 31) / 32), (unsigned)((C / 32 + 3) / 4));
    fp32_rows_gemm_kernel<<<grid, 256, 0, stream>>>((const float *)a.avg, a.avg_stride_s, (const float *)a.output_w, C, a.output_b,
                                                    (float *)a.out, a.out_ld, M, C, C);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch
