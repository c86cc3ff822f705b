// Global (extra-MSA column) attention for gfx950, bf16 storage, 64 channels
// (reference src/attention/global_attention.cpp:30-164; nchannels == 64 is hard-wired there, :172).
//
// Per batch row b there is ONE query per head, the masked mean of the row's tokens, and ONE key/value
// head shared by all heads:
//   q_avg = sum_s mask[s] x[s,:] / (sum_s mask[s] + 1e-10);  q = q_avg.Wq^T  viewed [H, d]
//   logit[h,s] = q[h].(Wk x[s]) / sqrt(d) + (mask[s]*1e9 - 1e9);  p = softmax_s
//   wavg[h,:] = sum_s p[h,s] (Wv x[s]);  out[s,:] = (sigmoid(x[s].Wg^T + bg) * wavg).Wo^T + bo
// One workgroup (four waves) owns a batch row and walks it in 32-token tiles in three phases: (A) masked
// mean, (B) logits, online softmax and weighted average, (C) gate, gating and output projection.  Tiles
// arrive with whole-cache-line loads through the wave's LDS staging panel, the next one in flight while
// the current one is processed; up to seq_len 1024 a wave keeps the fragments of its tiles in registers
// after phase A, so the row is read from memory once.  Nothing but q_avg and out is written to memory.  All contractions are v_mfma_f32_32x32x16_bf16:
//   B: logits^T[s, h] = X[s, :] . QK^T with QK[h, :] = q[h].Wk / sqrt(d) folded per batch row (heads are the
//      columns, 8 of 32 used for H = 8); V[s, e] = X . Wv^T; O^T[e, h] += V^T . P^T -- the accumulators
//      of the first two products are directly the operands of the third, as in the gated attention
//      kernels (rows of a tile are the contraction index of the third product on both sides).
//   C: G^T[c, s] = Wg . X^T with the rows of Wg ordered so that a lane's accumulators are the k-slots of
//      the next product's B operand; OUT^T[o, s] = Wo . gated^T with the rows of Wo ordered so that a lane
//      holds 16 consecutive output features of its token (two 16-byte stores).
// The -1e9 mask bias is the accumulator's initial value and absorbs the logit in fp32, so a row whose mask
// is all zero attends uniformly, as in the reference.
#include <hip/hip_runtime.h>

#include <cmath>

#include "device_util.h"
#include "launch_internal.h"
#include "mfma_tiles.h"
#include "profiler.h"

using namespace kutacc_dev;

namespace {

constexpr int GC = 64;        // channels
constexpr int MERGE_LD = 18;  // floats per lane in the cross-wave merge area: m, l, 16 accumulators

struct GlobalParams {
    const bf16_t *x, *mask, *wq, *wk, *wv, *wg, *wo;
    const float *bg, *bo;
    bf16_t *q_avg, *out;
    int64_t x_sb, x_ss, mask_sb, qavg_sb, out_sb, out_ss;
    int B, S, H, d, NT;
    float scale;
};

// channel that accumulator register v of lane half g holds in row block rb of the gate product
__device__ __forceinline__ int gate_channel(int rb, int v, int g)
{
    const int idx = rb * 16 + v;
    return 16 * (idx >> 3) + 8 * g + (idx & 7);
}

// CACHED: the row has at most 32 tiles (seq_len <= 1024), so each wave keeps the fragments of its (at most 8) tiles
// in registers after phase A and the row is read from memory once; otherwise every phase streams the row again.
template <bool CACHED, int NW>
__global__ __launch_bounds__(64 * NW, 2) void global_attention_kernel(GlobalParams p)
{
    constexpr int NTHR = 64 * NW;
    constexpr int MAXI = CACHED ? 32 / NW : (1 << 24); // tiles per wave
    constexpr int UNR = CACHED ? 32 / NW : 1;          // the cached tile array needs compile-time indices
    bf16x8 xs[CACHED ? 32 / NW : 1][4];
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int b = blockIdx.x;
    const int S = p.S, NT = p.NT, H = p.H, d = p.d;
    const int spad = NT * 32;

    uint4 *qk_frag = lds;            // [4 k-steps][64 lanes]
    uint4 *wv_frag = qk_frag + 256;  // [4][64]
    uint4 *wg_frag = wv_frag + 256;  // [2 row blocks][4][64]
    uint4 *wo_frag = wg_frag + 512;  // [2 row blocks][4][64]
    uint4 *wk_rows = wo_frag + 512;  // the key weights as they lie in memory, [d][64 channels] bf16 (d <= 32)
    uint4 *panel = wk_rows + 256 + wave * 256;
    float *maskb = reinterpret_cast<float *>(wk_rows + 256 + NW * 256); // mask bias per token, -inf past S
    float *mask01 = maskb + spad;                                       // mask value per token, 0 past S
    float *part = mask01 + spad;                                        // [NW waves][68]: channel sums, mask sum
    float *qavg = part + NW * 68;                                        // [64]
    float *qv = qavg + GC;                                              // [64] q, bf16-rounded
    float *wavg = qv + GC;                                              // [64]
    float *merge = wavg + GC;                                           // [NW waves][64 lanes][MERGE_LD]

    const bf16_t *xb = p.x + (int64_t)b * p.x_sb;
    const uint32_t x_pitch = (uint32_t)p.x_ss; // tokens of a row by 32-bit byte offsets from xb (the launcher checks the range)

    // Requested before anything else, so that their latency passes under the staging of the weights: the first tiles of
    // the row (all of a wave's tiles when they are kept in registers and there are at most four) and this thread's slice
    // of the query weights (output o = tid / TPR, channels part * 64 / TPR ...).
    constexpr int PRE = CACHED ? (MAXI < 4 ? MAXI : 4) : 1;
    PanelRegs ahead[PRE];
#pragma unroll
    for (int i = 0; i < PRE; ++i) {
        const int t = wave + NW * i;
        ahead[i] = panel_load_near(xb, x_pitch, (t < NT ? t : NT - 1) * 32, S - 1, 0, lane);
    }
    constexpr int TPR = NTHR / GC, WQV = GC / TPR / 8; // threads per output of q, 16-byte pieces per thread
    uint4 wq_part[WQV];
#pragma unroll
    for (int v = 0; v < WQV; ++v) {
        wq_part[v] = *reinterpret_cast<const uint4 *>(p.wq + (tid / TPR) * GC + (tid % TPR) * (GC / TPR) + v * 8);
    }

    // ---- weights of phases B and C as MFMA fragments; mask ----
    for (int idx = tid; idx < d * 8; idx += NTHR) {
        wk_rows[idx] = reinterpret_cast<const uint4 *>(p.wk)[idx];
    }
    for (int idx = tid; idx < 256; idx += NTHR) {
        const int ks = idx >> 6, l = idx & 63, e = l & 31, gg = l >> 5;
        uint4 v = {0u, 0u, 0u, 0u};
        if (e < d) {
            v = *reinterpret_cast<const uint4 *>(p.wv + e * GC + ks * 16 + gg * 8);
        }
        wv_frag[idx] = v;
    }
    for (int idx = tid; idx < 512; idx += NTHR) {
        const int rb = idx >> 8, ks = (idx >> 6) & 3, l = idx & 63, i = l & 31, gg = l >> 5;
        const int ch = gate_channel(rb, 4 * (i >> 3) + (i & 3), (i >> 2) & 1);
        wg_frag[idx] = *reinterpret_cast<const uint4 *>(p.wg + ch * GC + ks * 16 + gg * 8);
        const int o = 32 * rb + pi_row(i);
        wo_frag[idx] = *reinterpret_cast<const uint4 *>(p.wo + o * GC + ks * 16 + gg * 8);
    }
    for (int s = tid; s < spad; s += NTHR) {
        float m = 0.f, mb = -INFINITY;
        if (s < S) {
            m = to_f32(p.mask[(int64_t)b * p.mask_sb + s]);
            mb = fmaf(m, 1e9f, -1e9f); // reference :120-121
        }
        mask01[s] = m;
        maskb[s] = mb;
    }
    __syncthreads();

    // ---- phase A: masked mean of the row, q, and the folded query-key matrix ----
    {
        float acc[4][8];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                acc[ks][e] = 0.f;
            }
        }
        float msum = 0.f;
        // the loads of the next PRE tiles are in flight while this one is summed
#pragma unroll(UNR)
        for (int i = 0; i < MAXI; ++i) {
            const int t = wave + NW * i;
            if (t >= NT) {
                break;
            }
            bf16x8 xf[4];
            panel_store(panel, lane, ahead[i % PRE]);
            if (!CACHED || i + PRE < MAXI) {
                const int tn = t + NW * PRE;
                ahead[i % PRE] = panel_load_near(xb, x_pitch, (tn < NT ? tn : NT - 1) * 32, S - 1, 0, lane);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                xf[ks] = as_bf16x8(panel[panel_slot(r, 2 * ks + g)]);
                if (CACHED) {
                    xs[i][ks] = xf[ks];
                }
            }
            const float m = mask01[t * 32 + r];
            msum += g == 0 ? m : 0.f;
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    acc[ks][e] = fmaf(m, to_f32(xf[ks][e]), acc[ks][e]);
                }
            }
        }
        // sum over the 32 lanes of each half (they hold different tokens of the same channels)
#pragma unroll
        for (int off = 16; off > 0; off >>= 1) {
            msum += __shfl_xor(msum, off, 64);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    acc[ks][e] += __shfl_xor(acc[ks][e], off, 64);
                }
            }
        }
        if (r == 0) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    part[wave * 68 + ks * 16 + g * 8 + e] = acc[ks][e];
                }
            }
            if (g == 0) {
                part[wave * 68 + 64] = msum;
            }
        }
    }
    __syncthreads();
    if (tid < GC) {
        float tot = 0.f, ms = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            tot += part[w * 68 + tid];
            ms += part[w * 68 + 64];
        }
        const bf16_t qa = (bf16_t)(tot * (1.0f / (ms + 1e-10f))); // reference :66-74
        qavg[tid] = to_f32(qa);
        if (p.q_avg != nullptr) {
            p.q_avg[(int64_t)b * p.qavg_sb + tid] = qa;
        }
    }
    __syncthreads();
    {
        // q[o] = sum_c q_avg[c] wq[o][c]: TPR neighbouring threads share an output, each with the slice it fetched at the start
        float a = 0.f;
#pragma unroll
        for (int v = 0; v < WQV; ++v) {
            const bf16x8 w8 = as_bf16x8(wq_part[v]);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                a = fmaf(qavg[(tid % TPR) * (GC / TPR) + v * 8 + e], to_f32(w8[e]), a);
            }
        }
#pragma unroll
        for (int off = TPR / 2; off > 0; off >>= 1) {
            a += __shfl_xor(a, off, 64);
        }
        if (tid % TPR == 0) {
            qv[tid / TPR] = to_f32((bf16_t)a); // the reference stores q as bf16 (:76-80)
        }
    }
    __syncthreads();
    if (tid < 256) {
        // B operand of the logits product: column h (zero for h >= H), 8 channels per lane and k-step
        const int ks = tid >> 6, h = r;
        float a[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (h < H) {
            for (int e = 0; e < d; ++e) {
                const bf16x8 w8 = as_bf16x8(wk_rows[e * 8 + ks * 2 + g]); // channels ks*16 + g*8 .. +8 of key row e
                const float qe = qv[h * d + e];
#pragma unroll
                for (int e8 = 0; e8 < 8; ++e8) {
                    a[e8] = fmaf(qe, to_f32(w8[e8]), a[e8]);
                }
            }
        }
        bf16x8 f;
#pragma unroll
        for (int e8 = 0; e8 < 8; ++e8) {
            f[e8] = (bf16_t)(a[e8] * p.scale);
        }
        qk_frag[ks * 64 + lane] = as_uint4(f);
    }
    __syncthreads();

    // ---- phase B: logits, online softmax, weighted average of V; one (m, l, O^T) state per wave ----
    {
        f32x16 o = zero16();
        float m_run = -1e30f, lsum = 0.f;
        PanelRegs nxt;
        if (!CACHED) {
            nxt = panel_load_near(xb, x_pitch, wave * 32, S - 1, 0, lane);
        }
#pragma unroll(UNR)
        for (int i = 0; i < MAXI; ++i) {
            const int t = wave + NW * i;
            if (t >= NT) {
                break;
            }
            bf16x8 xf[4];
            if (CACHED) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    xf[ks] = xs[i][ks];
                }
            } else {
                panel_store(panel, lane, nxt);
                nxt = panel_load_near(xb, x_pitch, (t + NW < NT ? t + NW : t) * 32, S - 1, 0, lane);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    xf[ks] = as_bf16x8(panel[panel_slot(r, 2 * ks + g)]);
                }
            }
            f32x16 x1, vv = zero16();
            const f32x4 *mb4 = reinterpret_cast<const f32x4 *>(maskb + t * 32 + 4 * g);
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 mv = mb4[2 * a];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x1[4 * a + c] = mv[c];
                }
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                x1 = mfma(xf[ks], as_bf16x8(qk_frag[ks * 64 + lane]), x1);
                vv = mfma(xf[ks], as_bf16x8(wv_frag[ks * 64 + lane]), vv);
            }
            float mx = x1[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) {
                mx = fmaxf(mx, x1[v]);
            }
            mx = half_swap_max(mx);
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
            lsum *= alpha;
            const float ml = -m_new * LOG2E;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                o[v] *= alpha;
                x1[v] = __builtin_amdgcn_exp2f(fmaf(x1[v], LOG2E, ml));
            }
            m_run = m_new;
            const bf16x8 p0 = pack8(x1, 0), p1 = pack8(x1, 8);
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                lsum += to_f32(p0[v]) + to_f32(p1[v]);
            }
            o = mfma(pack8(vv, 0), p0, o);
            o = mfma(pack8(vv, 8), p1, o);
        }
        float *mine = merge + (wave * 64 + lane) * MERGE_LD;
        mine[0] = m_run;
        mine[1] = half_swap_sum(lsum);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            mine[2 + v] = o[v];
        }
    }
    __syncthreads();
    if (wave == 0) {
        float mw[NW], lw[NW];
        float M = -1e30f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            mw[w] = merge[(w * 64 + lane) * MERGE_LD];
            lw[w] = merge[(w * 64 + lane) * MERGE_LD + 1];
            M = fmaxf(M, mw[w]);
        }
        float L = 0.f;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            mw[w] = __builtin_amdgcn_exp2f((mw[w] - M) * LOG2E);
            L = fmaf(lw[w], mw[w], L);
        }
        const float inv = 1.0f / L;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            float a = 0.f;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                a = fmaf(merge[(w * 64 + lane) * MERGE_LD + 2 + v], mw[w], a);
            }
            const int e = 8 * (v >> 2) + 4 * g + (v & 3);
            if (r < H && e < d) {
                wavg[r * d + e] = to_f32((bf16_t)(a * inv)); // the reference stores the weighted average as bf16 (:126-130)
            }
        }
    }
    __syncthreads();

    // ---- phase C: gate, gating, output projection ----
    {
        // per-channel constants of the gating, in the order the accumulators hold them
        float bgv[32], wv_[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            const int ch = gate_channel(i >> 4, i & 15, g);
            bgv[i] = p.bg[ch];
            wv_[i] = wavg[ch];
        }
        const float *bop = p.bo + 16 * g;
        PanelRegs nxt;
        if (!CACHED) {
            nxt = panel_load_near(xb, x_pitch, wave * 32, S - 1, 0, lane);
        }
#pragma unroll(UNR)
        for (int i = 0; i < MAXI; ++i) {
            const int t = wave + NW * i;
            if (t >= NT) {
                break;
            }
            bf16x8 xf[4];
            if (CACHED) {
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    xf[ks] = xs[i][ks];
                }
            } else {
                panel_store(panel, lane, nxt);
                nxt = panel_load_near(xb, x_pitch, (t + NW < NT ? t + NW : t) * 32, S - 1, 0, lane);
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    xf[ks] = as_bf16x8(panel[panel_slot(r, 2 * ks + g)]);
                }
            }
            bf16x8 gf[4];
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                f32x16 ga = zero16();
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    ga = mfma(as_bf16x8(wg_frag[(rb * 4 + ks) * 64 + lane]), xf[ks], ga);
                }
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    ga[v] = wv_[rb * 16 + v] * sigmoid_fast(ga[v] + bgv[rb * 16 + v]);
                }
                gf[2 * rb] = pack8(ga, 0);
                gf[2 * rb + 1] = pack8(ga, 8);
            }
            const int s = t * 32 + r;
#pragma unroll
            for (int ob = 0; ob < 2; ++ob) {
                f32x16 oa = zero16();
#pragma unroll
                for (int kk = 0; kk < 4; ++kk) {
                    oa = mfma(as_bf16x8(wo_frag[(ob * 4 + kk) * 64 + lane]), gf[kk], oa);
                }
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(bop + 32 * ob + 4 * a);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        oa[4 * a + c] += bv[c];
                    }
                }
                if (s < S) {
                    char *row_out = reinterpret_cast<char *>(p.out + (int64_t)b * p.out_sb + 32 * ob); // uniform
                    uint4 *dst = reinterpret_cast<uint4 *>(row_out + (__umul24((uint32_t)s, 2u * (uint32_t)p.out_ss) + 32u * g));
                    dst[0] = as_uint4(pack8(oa, 0));
                    dst[1] = as_uint4(pack8(oa, 8));
                }
            }
        }
    }
}

// Dynamic LDS of global_attention_kernel<., NW> for NT key tiles: staged weights and the waves' panels (16-byte units),
// then mask and logits rows, per-wave states and the merge area (floats).
constexpr size_t LDS_PER_WORKGROUP = 160 * 1024;
constexpr size_t lds_bytes_for(int nw, int nt)
{
    return (size_t)(256 + 256 + 512 + 512 + 256 + nw * 256) * 16 + (size_t)(2 * nt * 32 + nw * 68 + 3 * GC + nw * 64 * MERGE_LD) * 4;
}
constexpr int MAX_SEQ_LEN = 12288; // what the four-wave layout holds
static_assert(lds_bytes_for(4, MAX_SEQ_LEN / 32) <= LDS_PER_WORKGROUP && lds_bytes_for(4, MAX_SEQ_LEN / 32 + 1) > LDS_PER_WORKGROUP,
              "MAX_SEQ_LEN must be the longest row whose four-wave layout fits the LDS");

} // namespace

namespace kutacc_launch {

int global_attention(const kutacc_hip_global_attention_args_t &a, hipStream_t stream)
{
    if (a.batch <= 0 || a.seq_len <= 0 || a.nheads <= 0 || a.head_size <= 0 || !a.q_data || !a.q_mask || !a.query_w ||
        !a.key_w || !a.value_w || !a.gating_w || !a.output_w || !a.gating_b || !a.output_b || !a.out) {
        return KUTACC_HIP_EINVAL;
    }
    if (a.dtype != KUTACC_DTYPE_BF16 || a.nheads * a.head_size != GC || a.nheads > 32 || a.head_size > 32 ||
        a.batch > INT32_MAX || a.seq_len > MAX_SEQ_LEN) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    // tokens of a batch row are addressed by 32-bit byte offsets from its first one
    if (a.q_data_stride_s <= 0 || a.out_stride_s <= 0 || a.q_data_stride_s >= (1 << 22) || a.out_stride_s >= (1 << 22) ||
        a.seq_len >= (1 << 23) || (a.seq_len + 32) * a.q_data_stride_s * 2 >= ((int64_t)1 << 31) ||
        (a.seq_len + 32) * a.out_stride_s * 2 >= ((int64_t)1 << 31)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    // 16-byte row loads of x and the weights, 16-byte stores of out rows
    if (a.q_data_stride_s % 8 != 0 || a.q_data_stride_b % 8 != 0 || a.out_stride_s % 8 != 0 || a.out_stride_b % 8 != 0 ||
        !kutacc_hip_aligned16(a.q_data) || !kutacc_hip_aligned16(a.out) || !kutacc_hip_aligned16(a.query_w) || !kutacc_hip_aligned16(a.key_w) ||
        !kutacc_hip_aligned16(a.value_w) || !kutacc_hip_aligned16(a.gating_w) || !kutacc_hip_aligned16(a.output_w)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    GlobalParams p;
    p.x = (const bf16_t *)a.q_data, p.mask = (const bf16_t *)a.q_mask;
    p.wq = (const bf16_t *)a.query_w, p.wk = (const bf16_t *)a.key_w, p.wv = (const bf16_t *)a.value_w;
    p.wg = (const bf16_t *)a.gating_w, p.wo = (const bf16_t *)a.output_w;
    p.bg = a.gating_b, p.bo = a.output_b;
    p.q_avg = (bf16_t *)a.q_avg, p.out = (bf16_t *)a.out;
    p.x_sb = a.q_data_stride_b, p.x_ss = a.q_data_stride_s, p.mask_sb = a.q_mask_stride_b;
    p.qavg_sb = a.q_avg_stride_b, p.out_sb = a.out_stride_b, p.out_ss = a.out_stride_s;
    p.B = (int)a.batch, p.S = (int)a.seq_len, p.H = (int)a.nheads, p.d = (int)a.head_size;
    p.NT = (int)((a.seq_len + 31) / 32);
    p.scale = (float)(1.0 / sqrt((double)a.head_size)); // reference :98
    // A batch row is one workgroup and its three phases follow one another (load and mean, logits, gate and output), so what
    // overlaps them is other rows on the same CU.  With the row kept in registers (up to 1024 positions) four waves hold
    // 128 + 113 registers and two rows share a CU; eight waves hold half the tiles each (174 registers) and one row has the
    // CU to itself, which is faster only while there is no second row to put there -- batch <= CUs: 28.1 against 30.7 us at
    // 256 x 1024, 48.3 against 39.3 us at 384 x 1024.  Rows streamed three times (longer sequences) always take eight
    // waves: 220 against 282 us at 384 x 5120.
    const bool cached = p.NT <= 32;
    static int cu_table[KUTACC_DEVICE_SLOTS] = {};
    const int ncu = kutacc_device_attribute(hipDeviceAttributeMultiprocessorCount, 256, cu_table);
    // ... as long as the eight-wave layout fits the LDS: its fixed part is 36 KB larger than the four-wave one's, and
    // both grow by 256 bytes per key tile (7808 positions with eight waves, MAX_SEQ_LEN with four).
    int nw = (p.NT >= 16 && (!cached || a.batch <= ncu)) ? 8 : 4;
    if (nw == 8 && lds_bytes_for(8, p.NT) > LDS_PER_WORKGROUP) {
        nw = 4;
    }
    const size_t lds_bytes = lds_bytes_for(nw, p.NT);
    if (lds_bytes > LDS_PER_WORKGROUP) {
        return KUTACC_HIP_EUNSUPPORTED; // not reached while MAX_SEQ_LEN is what four waves can hold
    }
    static size_t configured[4][KUTACC_DEVICE_SLOTS] = {};
    const void *fn = nw == 8 ? (cached ? reinterpret_cast<const void *>(global_attention_kernel<true, 8>)
                                       : reinterpret_cast<const void *>(global_attention_kernel<false, 8>))
                             : (cached ? reinterpret_cast<const void *>(global_attention_kernel<true, 4>)
                                       : reinterpret_cast<const void *>(global_attention_kernel<false, 4>));
    {
        const hipError_t e = kutacc_opt_in_lds(fn, lds_bytes, configured[(nw == 8 ? 2 : 0) + (cached ? 1 : 0)]);
        if (e != hipSuccess) {
            return (int)e;
        }
    }
    const double BS = (double)a.batch * (double)a.seq_len;
    kutacc_prof::KernelTimer t("global_attention_kernel", BS * (4.0 * GC * a.head_size + 4.0 * GC * GC + 4.0 * GC), stream);
    const dim3 grid((unsigned)a.batch), block((unsigned)(64 * nw));
    if (nw == 8) {
        if (cached) {
            global_attention_kernel<true, 8><<<grid, block, lds_bytes, stream>>>(p);
        } else {
            global_attention_kernel<false, 8><<<grid, block, lds_bytes, stream>>>(p);
        }
    } else if (cached) {
        global_attention_kernel<true, 4><<<grid, block, lds_bytes, stream>>>(p);
    } else {
        global_attention_kernel<false, 4><<<grid, block, lds_bytes, stream>>>(p);
    }
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch
