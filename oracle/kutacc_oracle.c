/*
 * kutacc_oracle.c -- CPU restatement of the KuTACC gated-attention path.  TEST INFRASTRUCTURE ONLY:
 * it is the checker for the HIP kernels and the timed CPU baseline of the benchmark; nothing in the
 * shipped library links, loads or calls it.
 *
 * Two restatements of reference src/attention/gating_attention.cpp:33-158 are provided:
 *
 *   oracle_gating_attention_f32   "R32": fp32 operands, double accumulation, no intermediate
 *                                 rounding.  This is the parity oracle.
 *   oracle_gating_attention_bf16  "Rbf16": bf16 storage with a rounding step at every point where the
 *                                 reference stores bf16 (q, k, v, gate, logits, probabilities,
 *                                 weighted average, gated average, out), the same
 *                                 (batch, head, query-block) work decomposition and per-thread
 *                                 buffers, OpenMP.  This is the timed CPU baseline, and measures how
 *                                 far the reference itself sits from R32.
 *
 * plus the two row operators in front of the path (LayerNorm, Linear), an R32 restatement of the
 * global (extra-MSA column) attention, reference src/attention/global_attention.cpp:30-164, and R32
 * restatements of the transition (reference src/attention/transition.cpp:21-39) and of the steps of the
 * triangle multiplication (reference src/attention/triangle_multiplication.cpp:25-150).
 *
 * Pinning status (the reference ships no numeric test for any of this):
 *   - R32 (both attentions), layernorm, linear: pinned by tests/test_oracle_pinning.py against library routines
 *     (torch matmul / scaled_dot_product_attention / layer_norm / linear), a pure-Python brute
 *     force on tiny shapes, and closed-form invariants.
 *   - Rbf16 rounding points: pinned only relative to R32 (must agree within bf16 tolerances);
 *     the closed GEMM library's accumulation order is unknown -> bit-level parity unpinned.
 *   - exp_mode 1 (emulation of the SVE FEXPA based fast_exp, exported as oracle_ref_exp): the instruction itself cannot
 *     be run on this machine; the emulation is pinned by what the arithmetic of fast_exp.h:21-27 fixes (results are
 *     integer powers of 2^(1/64), the nearest one to exp(x) with ties away from zero, exactly 1 at 0, exactly 0 below
 *     the u32 saturation, constant above the clamp, monotone), tests/test_oracle_pinning.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- bf16 <-> fp32: widening is a 16-bit shift, narrowing is round-to-nearest-even
 *      (reference src/wrapper/svcvt.h:23-37) ---- */
static inline float bf16_to_f32(uint16_t v)
{
    uint32_t u = (uint32_t)v << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static inline uint16_t f32_to_bf16(float f)
{
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x40u); /* quiet NaN */
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

void oracle_f32_to_bf16(const float *src, uint16_t *dst, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        dst[i] = f32_to_bf16(src[i]);
    }
}

void oracle_bf16_to_f32(const uint16_t *src, float *dst, int64_t n)
{
    for (int64_t i = 0; i < n; ++i) {
        dst[i] = bf16_to_f32(src[i]);
    }
}

int oracle_num_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------------
 * R32: out = ((softmax_k(q.k^T*scale + bias[b,k] + nb[h,q,k]) . v) * sigmoid(gate)) . Wo^T + bo
 * with q,k,v = x.W^T and gate = x.Wg^T + bg (reference gating_attention.cpp:47-66, 97-157).
 * Weights are [out, in] row-major (the {1, C}-strided views at :49,:54,:64,:155; value_w is used as
 * the left operand un-transposed at :57).  bias is [B, S]; nb is [H, S, S] or NULL.
 * avg_out (optional) receives the gated weighted average [B*S, C].
 * ---------------------------------------------------------------------------------------------- */
static void project_f64(const float *x, const float *w, const float *b, int64_t rows, int64_t c, double *y)
{
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < rows; ++t) {
        for (int64_t o = 0; o < c; ++o) {
            double acc = 0.0;
            for (int64_t i = 0; i < c; ++i) {
                acc += (double)x[t * c + i] * (double)w[o * c + i];
            }
            y[t * c + o] = acc + (b ? (double)b[o] : 0.0);
        }
    }
}

void oracle_gating_attention_f32(const float *input, const float *wq, const float *wk, const float *wv,
                                 const float *wg, const float *bg, const float *wo, const float *bo,
                                 const float *bias, const float *nb, int64_t B, int64_t S, int64_t H, int64_t d,
                                 float *out, float *avg_out)
{
    const int64_t C = H * d, M = B * S;
    double *q = malloc(sizeof(double) * M * C), *k = malloc(sizeof(double) * M * C);
    double *v = malloc(sizeof(double) * M * C), *g = malloc(sizeof(double) * M * C);
    double *avg = malloc(sizeof(double) * M * C);
    project_f64(input, wq, NULL, M, C, q);
    project_f64(input, wk, NULL, M, C, k);
    project_f64(input, wv, NULL, M, C, v);
    project_f64(input, wg, bg, M, C, g);
    const double scale = 1.0 / sqrt((double)d);
#pragma omp parallel
    {
        double *x = malloc(sizeof(double) * S);
#pragma omp for collapse(2) schedule(static)
        for (int64_t b = 0; b < B; ++b) {
            for (int64_t h = 0; h < H; ++h) {
                for (int64_t qi = 0; qi < S; ++qi) {
                    const double *qr = q + (b * S + qi) * C + h * d;
                    double m = -INFINITY;
                    for (int64_t kj = 0; kj < S; ++kj) {
                        const double *kr = k + (b * S + kj) * C + h * d;
                        double s = 0.0;
                        for (int64_t e = 0; e < d; ++e) {
                            s += qr[e] * kr[e];
                        }
                        /* The two bias additions are fp32 additions, in the reference's order
                         * (gating_attention.cpp:113-117).  This matters: a -1e9 mask bias absorbs
                         * the logit in fp32, so a fully masked row attends uniformly. */
                        float xf = (float)(s * scale);
                        xf = xf + bias[b * S + kj];
                        if (nb) {
                            xf = xf + nb[(h * S + qi) * S + kj];
                        }
                        x[kj] = (double)xf;
                        if (x[kj] > m) {
                            m = x[kj];
                        }
                    }
                    double sum = 0.0;
                    for (int64_t kj = 0; kj < S; ++kj) {
                        x[kj] = exp(x[kj] - m);
                        sum += x[kj];
                    }
                    for (int64_t e = 0; e < d; ++e) {
                        double acc = 0.0;
                        for (int64_t kj = 0; kj < S; ++kj) {
                            acc += x[kj] * v[(b * S + kj) * C + h * d + e];
                        }
                        const double gate = 1.0 / (1.0 + exp(-g[(b * S + qi) * C + h * d + e]));
                        avg[(b * S + qi) * C + h * d + e] = acc / sum * gate;
                    }
                }
            }
        }
        free(x);
    }
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < M; ++t) {
        for (int64_t o = 0; o < C; ++o) {
            double acc = 0.0;
            for (int64_t i = 0; i < C; ++i) {
                acc += avg[t * C + i] * (double)wo[o * C + i];
            }
            out[t * C + o] = (float)(acc + (double)bo[o]);
        }
        if (avg_out) {
            for (int64_t i = 0; i < C; ++i) {
                avg_out[t * C + i] = (float)avg[t * C + i];
            }
        }
    }
    free(q), free(k), free(v), free(g), free(avg);
}

/* ------------------------------------------------------------------------------------------------
 * Global (extra-MSA column) attention, reference src/attention/global_attention.cpp:30-164.
 * One query per batch row and head, one key/value head shared by all heads:
 *   q_avg[b,:] = sum_s mask[b,s] x[b,s,:] / (sum_s mask[b,s] + 1e-10)                (:47-74)
 *   q[b] = q_avg[b].Wq^T viewed [H, d];  k[b,s] = Wk.x[b,s] (d);  v[b,s] = Wv.x[b,s] (d)   (:76-92)
 *   gate[b,s,:] = x[b,s,:].Wg^T + bg                                               (:93-97)
 *   logit[h,s] = (q[b,h].k[b,s]) * 1/sqrt(d) + (mask[b,s]*1e9 - 1e9)   fp32 adds      (:112-124)
 *   p = softmax_s(logit);  wavg[h,:] = sum_s p[h,s] v[b,s,:]                        (:126-132)
 *   gated[b,s,:] = sigmoid(gate[b,s,:]) * wavg (wavg flattened [H*d] = C)           (:133-153)
 *   out = gated.Wo^T + bo                                                           (:157-161)
 * Wq, Wg, Wo are [C, C] stored [out, in]; Wk, Wv are [d, C].  mask is [B, S].
 * R32: fp32 operands, double accumulation; the mask bias is formed and added in fp32 as the
 * reference does, so an all-zero mask row gives uniform attention.
 * ---------------------------------------------------------------------------------------------- */
void oracle_global_attention_f32(const float *x, const float *mask, const float *wq, const float *wk, const float *wv,
                                 const float *wg, const float *bg, const float *wo, const float *bo, int64_t B,
                                 int64_t S, int64_t H, int64_t d, float *out, float *q_avg_out)
{
    const int64_t C = H * d;
    const double scale = (double)(float)(1.0 / sqrt((double)d));
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < B; ++b) {
        double *qa = malloc(sizeof(double) * C), *q = malloc(sizeof(double) * C);
        double *k = malloc(sizeof(double) * S * d), *v = malloc(sizeof(double) * S * d);
        double *p = malloc(sizeof(double) * S), *wavg = malloc(sizeof(double) * C);
        double *gated = malloc(sizeof(double) * C);
        const float *xb = x + b * S * C;
        double msum = 0.0;
        for (int64_t c = 0; c < C; ++c) {
            qa[c] = 0.0;
        }
        for (int64_t s = 0; s < S; ++s) {
            msum += (double)mask[b * S + s];
            for (int64_t c = 0; c < C; ++c) {
                qa[c] += (double)mask[b * S + s] * (double)xb[s * C + c];
            }
        }
        for (int64_t c = 0; c < C; ++c) {
            qa[c] /= (msum + 1e-10);
            if (q_avg_out) {
                q_avg_out[b * C + c] = (float)qa[c];
            }
        }
        for (int64_t o = 0; o < C; ++o) {
            double acc = 0.0;
            for (int64_t c = 0; c < C; ++c) {
                acc += qa[c] * (double)wq[o * C + c];
            }
            q[o] = acc;
        }
        for (int64_t s = 0; s < S; ++s) {
            for (int64_t e = 0; e < d; ++e) {
                double ak = 0.0, av = 0.0;
                for (int64_t c = 0; c < C; ++c) {
                    ak += (double)xb[s * C + c] * (double)wk[e * C + c];
                    av += (double)xb[s * C + c] * (double)wv[e * C + c];
                }
                k[s * d + e] = ak;
                v[s * d + e] = av;
            }
        }
        for (int64_t h = 0; h < H; ++h) {
            double m = -INFINITY;
            for (int64_t s = 0; s < S; ++s) {
                double dot = 0.0;
                for (int64_t e = 0; e < d; ++e) {
                    dot += q[h * d + e] * k[s * d + e];
                }
                const float biasf = fmaf(mask[b * S + s], 1e9f, -1e9f);
                const float xf = (float)(dot * scale) + biasf;
                p[s] = (double)xf;
                if (p[s] > m) {
                    m = p[s];
                }
            }
            double sum = 0.0;
            for (int64_t s = 0; s < S; ++s) {
                p[s] = exp(p[s] - m);
                sum += p[s];
            }
            for (int64_t e = 0; e < d; ++e) {
                double acc = 0.0;
                for (int64_t s = 0; s < S; ++s) {
                    acc += p[s] * v[s * d + e];
                }
                wavg[h * d + e] = acc / sum;
            }
        }
        for (int64_t s = 0; s < S; ++s) {
            for (int64_t o = 0; o < C; ++o) {
                double acc = (double)bg[o];
                for (int64_t c = 0; c < C; ++c) {
                    acc += (double)xb[s * C + c] * (double)wg[o * C + c];
                }
                gated[o] = wavg[o] / (1.0 + exp(-acc));
            }
            for (int64_t o = 0; o < C; ++o) {
                double acc = (double)bo[o];
                for (int64_t c = 0; c < C; ++c) {
                    acc += gated[c] * (double)wo[o * C + c];
                }
                out[(b * S + s) * C + o] = (float)acc;
            }
        }
        free(qa), free(q), free(k), free(v), free(p), free(wavg), free(gated);
    }
}

/* ------------------------------------------------------------------------------------------------
 * Rbf16 building blocks
 * ---------------------------------------------------------------------------------------------- */

/* exp of the reference's fast_exp (src/math/fast_exp.h:21-27): 2^(n/64) with
 * n = round_half_away(min(x, 88.72284) * 92.33248 + 8128) - 8128, produced by the FEXPA instruction
 * from the integer n + 8128; a negative integer saturates to 0 in the u32 conversion and FEXPA(0)
 * is +0.0.  exp_mode 0 uses libm expf instead. */
static inline float ref_exp(float x, int exp_mode)
{
    if (exp_mode == 0) {
        return expf(x);
    }
    const float tf = fmaf(fminf(x, 88.72284f), 92.33248f, 8128.0f); /* svmad: single rounding */
    const float r = roundf(tf);                                     /* svrinta: ties away from zero */
    if (!(r > 0.0f)) {
        return 0.0f;
    }
    const uint32_t n = (uint32_t)r;
    const uint32_t frac = n & 63u, expo = (n >> 6) & 0xffu;
    /* table entry = the 23 fraction bits of 2^(frac/64) */
    const double mant = exp2((double)frac / 64.0);
    const float mf = (float)mant; /* in [1, 2) */
    uint32_t bits;
    memcpy(&bits, &mf, 4);
    bits = (bits & 0x007fffffu) | (expo << 23);
    float outv;
    memcpy(&outv, &bits, 4);
    return outv;
}

/* ref_exp over an array, for the tests that pin it. */
void oracle_ref_exp(const float *x, float *y, int64_t n, int exp_mode)
{
    for (int64_t i = 0; i < n; ++i) {
        y[i] = ref_exp(x[i], exp_mode);
    }
}

/* y[rows, n] (bf16, row stride ldy, col stride cs) = x[rows, kdim] . w[n, kdim]^T (+ bias[n]),
 * fp32 accumulation, one rounding to bf16 at the store -- the contract assumed for the closed
 * bf16 GEMM behind reference src/utils/blas.cpp:61-78 (row bias = per output column, :66,:157). */
static void gemm_nt_bf16(const uint16_t *x, int64_t ldx, const uint16_t *w, int64_t ldw, const float *bias,
                         uint16_t *y, int64_t y_rs, int64_t y_cs, int64_t rows, int64_t n, int64_t kdim)
{
    float *wf = malloc(sizeof(float) * n * kdim);
    for (int64_t o = 0; o < n; ++o) {
        for (int64_t i = 0; i < kdim; ++i) {
            wf[o * kdim + i] = bf16_to_f32(w[o * ldw + i]);
        }
    }
#pragma omp parallel
    {
        float *xf = malloc(sizeof(float) * kdim);
#pragma omp for schedule(static)
        for (int64_t t = 0; t < rows; ++t) {
            for (int64_t i = 0; i < kdim; ++i) {
                xf[i] = bf16_to_f32(x[t * ldx + i]);
            }
            for (int64_t o = 0; o < n; ++o) {
                const float *wr = wf + o * kdim;
                float acc = 0.f;
                for (int64_t i = 0; i < kdim; ++i) {
                    acc += xf[i] * wr[i];
                }
                if (bias) {
                    acc += bias[o];
                }
                y[t * y_rs + o * y_cs] = f32_to_bf16(acc);
            }
        }
        free(xf);
    }
    free(wf);
}

/*
 * Rbf16.  Scratch q,k,gate,avg are [B,S,H,d] dense, v is [H,d,B,S] dense (reference
 * gating_attention.cpp:57-61,123-127).  Loop structure: flat index over (b, h, query block) with
 * the block index fastest, contiguous chunks per thread, K and V of a (b,h) pair unpacked once per
 * pair (reference :73-150, src/utils/parallel.h:65-90, src/utils/collapse.h:31-58).
 */
void oracle_gating_attention_bf16(const uint16_t *input, const uint16_t *wq, const uint16_t *wk, const uint16_t *wv,
                                  const uint16_t *wg, const float *bg, const uint16_t *wo, const float *bo,
                                  const uint16_t *bias, const uint16_t *nb, int64_t B, int64_t S, int64_t H, int64_t d,
                                  int64_t block_size, int exp_mode, uint16_t *q, uint16_t *k, uint16_t *v,
                                  uint16_t *gate, uint16_t *avg, uint16_t *out)
{
    const int64_t C = H * d, M = B * S;
    gemm_nt_bf16(input, C, wq, C, NULL, q, C, 1, M, C, C);
    gemm_nt_bf16(input, C, wk, C, NULL, k, C, 1, M, C, C);
    gemm_nt_bf16(input, C, wv, C, NULL, v, 1, M, M, C, C); /* v^T: [C, B*S] */
    gemm_nt_bf16(input, C, wg, C, bg, gate, C, 1, M, C, C);

    const int64_t nblocks = (S + block_size - 1) / block_size;
    const float scale = (float)(1 / sqrt((double)d));
    const int64_t total = B * H * nblocks;
    int64_t nthreads = oracle_num_threads();
    const int64_t max_by_grain = (total + nblocks - 1) / nblocks;
    if (nthreads > max_by_grain) {
        nthreads = max_by_grain;
    }
    const int64_t chunk = (total + nthreads - 1) / nthreads;
#pragma omp parallel num_threads((int)nthreads)
    {
#ifdef _OPENMP
        const int64_t tid = omp_get_thread_num();
#else
        const int64_t tid = 0;
#endif
        const int64_t start = tid * chunk;
        const int64_t end = start + chunk < total ? start + chunk : total;
        if (start < end) {
            uint16_t *logits = malloc(sizeof(uint16_t) * block_size * S);
            float *sbuf = malloc(sizeof(float) * S);
            float *kbuf = malloc(sizeof(float) * S * d); /* [S, d] */
            float *vbuf = malloc(sizeof(float) * S * d); /* [d, S] */
            float *prow = malloc(sizeof(float) * S);
            int64_t kv_id = -1;
            for (int64_t it = start; it < end; ++it) {
                const int64_t blk = it % nblocks, hi = (it / nblocks) % H, bi = it / nblocks / H;
                const int64_t q0 = blk * block_size, q1 = q0 + block_size < S ? q0 + block_size : S;
                if (kv_id != bi * H + hi) {
                    for (int64_t s = 0; s < S; ++s) {
                        for (int64_t e = 0; e < d; ++e) {
                            kbuf[s * d + e] = bf16_to_f32(k[(bi * S + s) * C + hi * d + e]);
                            vbuf[e * S + s] = bf16_to_f32(v[(hi * d + e) * M + bi * S + s]);
                        }
                    }
                    kv_id = bi * H + hi;
                }
                /* logits block = bf16(Q_blk . K^T) */
                for (int64_t qi = q0; qi < q1; ++qi) {
                    float qf[512];
                    float *qrow = d <= 512 ? qf : malloc(sizeof(float) * d);
                    for (int64_t e = 0; e < d; ++e) {
                        qrow[e] = bf16_to_f32(q[(bi * S + qi) * C + hi * d + e]);
                    }
                    for (int64_t s = 0; s < S; ++s) {
                        float acc = 0.f;
                        for (int64_t e = 0; e < d; ++e) {
                            acc += qrow[e] * kbuf[s * d + e];
                        }
                        logits[(qi - q0) * S + s] = f32_to_bf16(acc);
                    }
                    if (qrow != qf) {
                        free(qrow);
                    }
                }
                for (int64_t qi = q0; qi < q1; ++qi) {
                    uint16_t *row = logits + (qi - q0) * S;
                    const uint16_t *nbrow = nb ? nb + (hi * S + qi) * S : NULL;
                    float m = -INFINITY;
                    for (int64_t s = 0; s < S; ++s) {
                        float x = bf16_to_f32(row[s]) * scale;
                        x = x + bf16_to_f32(bias[bi * S + s]);
                        if (nbrow) {
                            x = x + bf16_to_f32(nbrow[s]);
                        }
                        m = fmaxf(m, x);
                        sbuf[s] = x;
                    }
                    /* softmax_with_max (reference src/softmax/softmax.h:22-43) */
                    float sum = 0.f;
                    for (int64_t s = 0; s < S; ++s) {
                        sbuf[s] = ref_exp(sbuf[s] - m, exp_mode);
                        sum += sbuf[s];
                    }
                    const float inv = 1 / sum;
                    for (int64_t s = 0; s < S; ++s) {
                        row[s] = f32_to_bf16(sbuf[s] * inv);
                    }
                }
                /* weighted average = bf16(P . V), then gated in place */
                for (int64_t qi = q0; qi < q1; ++qi) {
                    const uint16_t *row = logits + (qi - q0) * S;
                    for (int64_t s = 0; s < S; ++s) {
                        prow[s] = bf16_to_f32(row[s]);
                    }
                    for (int64_t e = 0; e < d; ++e) {
                        const float *vr = vbuf + e * S;
                        float acc = 0.f;
                        for (int64_t s = 0; s < S; ++s) {
                            acc += prow[s] * vr[s];
                        }
                        const float wavg = bf16_to_f32(f32_to_bf16(acc));
                        const float gv = bf16_to_f32(gate[(bi * S + qi) * C + hi * d + e]);
                        /* Sigmoid::call (reference src/activation/sigmoid.h:30-35) */
                        const float sg = 1.0f / (ref_exp(-gv, exp_mode) + 1.0f);
                        avg[(bi * S + qi) * C + hi * d + e] = f32_to_bf16(wavg * sg);
                    }
                }
            }
            free(logits), free(sbuf), free(kbuf), free(vbuf), free(prow);
        }
    }
    gemm_nt_bf16(avg, C, wo, C, bo, out, C, 1, M, C, C);
}

/* ------------------------------------------------------------------------------------------------
 * LayerNorm of one row, bf16 in/out (reference src/normalization/layernorm_kernel.h:21-53):
 * shift by the first element, fp32 sums, clamped variance, then (x*rstd + (-rstd*mean))*gamma+beta
 * with the two fused multiply-adds the SVE code uses (:48-49).
 * ---------------------------------------------------------------------------------------------- */
void oracle_layernorm_bf16(const uint16_t *data, const float *gamma, const float *beta, int64_t size, float eps,
                           uint16_t *out)
{
    const float delta = bf16_to_f32(data[0]);
    float sum = 0.f, sum2 = 0.f;
    for (int64_t i = 0; i < size; ++i) {
        const float v = bf16_to_f32(data[i]) - delta;
        sum += v;
        sum2 = fmaf(v, v, sum2);
    }
    const float n = (float)size;
    const float mean = sum / n + delta;
    const float var = fmaxf((sum2 - sum * sum / n) / n, 0.f);
    const float rstd = 1 / sqrtf(var + eps);
    const float shift = -rstd * mean;
    for (int64_t i = 0; i < size; ++i) {
        const float v = fmaf(bf16_to_f32(data[i]), rstd, shift);
        out[i] = f32_to_bf16(fmaf(v, gamma[i], beta[i]));
    }
}

void oracle_layernorm_rows_bf16(const uint16_t *data, const float *gamma, const float *beta, int64_t rows,
                                int64_t size, float eps, uint16_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        oracle_layernorm_bf16(data + r * size, gamma, beta, size, eps, out + r * size);
    }
}

/* fp32-storage LayerNorm with double statistics: the oracle for the fp32 path. */
void oracle_layernorm_rows_f32(const float *data, const float *gamma, const float *beta, int64_t rows, int64_t size,
                               float eps, float *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const float *x = data + r * size;
        double s = 0.0, s2 = 0.0;
        for (int64_t i = 0; i < size; ++i) {
            s += x[i];
        }
        const double mean = s / (double)size;
        for (int64_t i = 0; i < size; ++i) {
            s2 += (x[i] - mean) * (x[i] - mean);
        }
        const double rstd = 1.0 / sqrt(s2 / (double)size + (double)eps);
        for (int64_t i = 0; i < size; ++i) {
            out[r * size + i] = (float)((x[i] - mean) * rstd * gamma[i] + beta[i]);
        }
    }
}

/* result[m, n] = bf16(beta*result + act[m, k].w[n, k]^T + bias[n]) (reference
 * src/linear/linear.cpp:21-42): fp32 accumulation, one rounding at the store. */
void oracle_linear_bf16(const uint16_t *act, int64_t ld_act, const uint16_t *w, int64_t ld_w, const float *bias,
                        uint16_t *result, int64_t m, int64_t n, int64_t k, float beta)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t o = 0; o < n; ++o) {
            double acc = 0.0;
            for (int64_t i = 0; i < k; ++i) {
                acc += (double)bf16_to_f32(act[r * ld_act + i]) * (double)bf16_to_f32(w[o * ld_w + i]);
            }
            float y = (float)acc;
            if (bias) {
                y += bias[o];
            }
            if (beta != 0.f) {
                y += beta * bf16_to_f32(result[r * n + o]);
            }
            result[r * n + o] = f32_to_bf16(y);
        }
    }
}

void oracle_linear_f32(const float *act, int64_t ld_act, const float *w, int64_t ld_w, const float *bias,
                       float *result, int64_t m, int64_t n, int64_t k, float beta)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < m; ++r) {
        for (int64_t o = 0; o < n; ++o) {
            double acc = 0.0;
            for (int64_t i = 0; i < k; ++i) {
                acc += (double)act[r * ld_act + i] * (double)w[o * ld_w + i];
            }
            if (bias) {
                acc += bias[o];
            }
            if (beta != 0.f) {
                acc += (double)beta * result[r * n + o];
            }
            result[r * n + o] = (float)acc;
        }
    }
}

/* ---- transition and triangle multiplication (R32: fp32 operands, double accumulation, no rounding) ---- */

/* mid = relu(x . w1^T + b1), out = mid . w2^T + b2 (reference src/attention/transition.cpp:31-38).
 * x [rows, c_o], w1 [c_i, c_o], w2 [c_o, c_i] stored [out, in]; mid [rows, c_i] may be NULL. */
void oracle_transition_f32(const float *x, const float *w1, const float *b1, const float *w2, const float *b2,
                           int64_t rows, int64_t c_o, int64_t c_i, float *out, float *mid)
{
#pragma omp parallel
    {
        double *h = (double *)malloc((size_t)c_i * sizeof(double));
#pragma omp for schedule(static)
        for (int64_t r = 0; r < rows; ++r) {
            for (int64_t j = 0; j < c_i; ++j) {
                double acc = b1[j];
                for (int64_t k = 0; k < c_o; ++k) {
                    acc += (double)x[r * c_o + k] * (double)w1[j * c_o + k];
                }
                h[j] = acc > 0.0 ? acc : 0.0;
                if (mid) {
                    mid[r * c_i + j] = (float)h[j];
                }
            }
            for (int64_t o = 0; o < c_o; ++o) {
                double acc = b2[o];
                for (int64_t j = 0; j < c_i; ++j) {
                    acc += h[j] * (double)w2[o * c_i + j];
                }
                out[r * c_o + o] = (float)acc;
            }
        }
        free(h);
    }
}

/* proj[c, i, j] = (x[i, j, :] . pw[c, :] + pb[c]) * mask[i, j] * sigmoid(x[i, j, :] . gw[c, :] + gb[c])
 * (reference src/attention/triangle_multiplication.cpp:37-66): x [n, c_o] with n = n_res*n_res_gather rows,
 * pw, gw [c_i, c_o], mask [n], proj [c_i, n] channel-first. */
void oracle_tm_calc_proj_f32(const float *x, const float *mask, const float *pw, const float *pb, const float *gw,
                             const float *gb, int64_t n, int64_t c_o, int64_t c_i, float *proj)
{
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < n; ++r) {
        for (int64_t c = 0; c < c_i; ++c) {
            double p = pb[c], g = gb[c];
            for (int64_t k = 0; k < c_o; ++k) {
                p += (double)x[r * c_o + k] * (double)pw[c * c_o + k];
                g += (double)x[r * c_o + k] * (double)gw[c * c_o + k];
            }
            proj[c * n + r] = (float)(p * (double)mask[r] / (1.0 + exp(-g)));
        }
    }
}

/* Per channel c of dense [channels, n, n] tensors (reference src/attention/triangle_multiplication.cpp:72-101):
 *   outgoing: center[c, i, j] = sum_k left[c, i, k] * right[c, j, k]
 *   incoming: center[c, i, j] = sum_k right[c, k, i] * left[c, k, j] */
void oracle_tm_equation_f32(const float *left, const float *right, int64_t channels, int64_t n, int incoming,
                            float *center)
{
#pragma omp parallel for schedule(static) collapse(2)
    for (int64_t c = 0; c < channels; ++c) {
        for (int64_t i = 0; i < n; ++i) {
            const float *l = left + c * n * n, *r = right + c * n * n;
            for (int64_t j = 0; j < n; ++j) {
                double acc = 0.0;
                if (!incoming) {
                    for (int64_t k = 0; k < n; ++k) {
                        acc += (double)l[i * n + k] * (double)r[j * n + k];
                    }
                } else {
                    for (int64_t k = 0; k < n; ++k) {
                        acc += (double)r[k * n + i] * (double)l[k * n + j];
                    }
                }
                center[(c * n + i) * n + j] = (float)acc;
            }
        }
    }
}
