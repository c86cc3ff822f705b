// Fused gated-attention kernels for gfx950 (CDNA4), bf16 storage, head_size 32.
//
// Two kernels compute the gated weighted average avg = softmax(q.k^T/sqrt(d) + bias + pair_bias).v *
// sigmoid(gate) for one (batch row b, head h) unit at a time; everything the reference materialises
// in memory between its GEMMs -- q, k, v, gate, the [bs, S] logits block, the probabilities
// (reference src/attention/gating_attention.cpp:47-66, 97-147) -- stays in LDS and registers:
//
//   persistent_head_kernel  seq_len <= 384 (C=128) / 256 (C=256).  One workgroup per CU keeps one head
//       for its lifetime (its four weight matrices staged once in LDS as MFMA fragments) and walks
//       batch rows; wave j owns sequence block j: it projects the block's K, V, Q and gate, then
//       attends its 32 queries against all keys of the row.
//   fused_head_kernel       any seq_len <= 1024.  One workgroup per unit; projections first (weights
//       staged through LDS in groups), then attention, up to four query blocks per wave.
//
// Both run the same attention blocks.  attend_block_l2 is the fast one (logits in log2 units, no running
// maximum, pair bias from a fragment-major copy made by pair_bias_fragments_kernel, row sums on the
// matrix core); attend_block and attend_block_direct are the general ones (running maximum with lazy
// rescale, pair bias read in place) for calls whose pair bias cannot be copied.
// A third kernel, output_projection_kernel, is the final GEMM with fp32 bias (reference :152-157).
//
// All contractions are v_mfma_f32_32x32x16_bf16 (fp32 accumulate); fragment and accumulator layouts
// are described in mfma_tiles.h.  Two consequences of those layouts are used everywhere below:
//   * a contraction index may be permuted freely as long as both operands agree, so an accumulator
//     can be fed back as the k-dimension of the next MFMA without any cross-lane movement: Q^T and
//     K^T share their head-dim order, and the probabilities share their key order with V;
//   * the sequence position handled by "row r" of a 32-row block is pi(r) = 16*((r>>2)&1) +
//     4*(r>>3) + (r&3), chosen so that the 16 logits a lane holds for its query are 16 CONSECUTIVE
//     keys (pair-bias row loads become two 16-byte loads).
#include <hip/hip_runtime.h>

#include <atomic>
#include <climits>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

#include "api_internal.h"
#include "device_util.h"
#include "launch_internal.h"
#include "mfma_tiles.h"
#include "profiler.h"

using namespace kutacc_dev;

namespace {

constexpr int HEAD = 32;            // head_size the MFMA kernels are written for
constexpr int WEIGHT_LOADS_IN_FLIGHT = 8; // per wave, while the weight fragments of a head are copied into LDS
constexpr int MAX_WAVES = 12;       // fused_head_kernel: 768 threads, 3 waves per SIMD, 168 VGPRs each
constexpr int FAIR_SLICE_SHIFT = 11;  // log2 of the clocks a wave keeps one issue priority (timeslice_priority); 2^8 to 2^13 measured alike
constexpr float RESCALE_GAP = 5.5f; // running max may lag the true max by this much (natural log units, ~8 octaves)

// Waves per workgroup a given fused_head_kernel instantiation may be launched with.  One query block
// per wave needs about 140 VGPRs at C=128, which fits three waves per SIMD; the variants that hold
// more state (more query blocks per wave, or 256 input channels in registers) get two per SIMD.
__host__ __device__ constexpr int max_waves(int C, int BPW) { return (C == 128 && BPW <= 2) ? MAX_WAVES : 8; }

enum Proj { PROJ_K = 0, PROJ_V = 1, PROJ_Q = 2, PROJ_G = 3 };

struct FusedParams {
    const bf16_t *x;
    const bf16_t *w[4]; // indexed by Proj
    const float *bg;
    const bf16_t *bias;
    const bf16_t *nb;
    bf16_t *avg;
    int64_t x_ld, x_sb, bias_sb, bias_sk, nb_sh, nb_sq, avg_sb, avg_ss, avg_sh; // x_sb: from one batch row of x to the next
    const float *ln_gamma, *ln_beta; // fused LayerNorm of the input rows (persistent kernel), else nullptr
    float ln_eps;
    int bias_is_mask; // bias holds the 0/1 mask; the kernels form 1e9*(mask-1) themselves
    int B, S, H, NB, NW, GW;
    int nb_vec;   // pair-bias rows may be read with 16-byte loads
    float qscale; // 1 / sqrt(head_size)
    int ngrp;     // persistent kernel: batch-row groups per XCD
    const uint4 *nbf; // pair bias * log2(e), fp16, in fragment-major order (pair_bias_fragments_kernel), or nullptr
    int NT;           // key tiles the LDS arrays are laid out for: NB rounded up to an even number (the log2-unit
                      // loop walks tile pairs; a phantom tile is all zeros behind a -inf mask)
    int l2mode;       // logits in log2 units (attend_block_l2); needs nbf when there is a pair bias
};

// 0/1 selection fragments that scatter the pair-bias words a lane loads (16 consecutive keys, 8 per
// MFMA) onto the logits rows: row i of a tile is key pi(i); k-slot 8*g+e of the first MFMA carries
// key 16*g+e, of the second key 16*g+8+e.
__device__ __forceinline__ void make_selectors(int lane, bf16x8 &sel0, bf16x8 &sel1)
{
    const int r = lane & 31, g = lane >> 5;
    const int gi = (r >> 2) & 1;          // which 16-key half row r belongs to
    const int w = 4 * (r >> 3) + (r & 3); // position of row r's key inside that half
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sel0[e] = (bf16_t)((gi == g && w == e) ? 1.0f : 0.0f);
        sel1[e] = (bf16_t)((gi == g && w == e + 8) ? 1.0f : 0.0f);
    }
}

// Pair-bias words on their way into a selector MFMA: -inf (and any negative NaN pattern) becomes the most negative finite
// bf16, since the MFMA multiplies every word by 0 or 1 and 0 x inf is a NaN.  As 16-bit unsigned numbers the negative
// values sort by magnitude, so this is one packed minimum per word; what the logit then holds is absorbed like a -inf.
__device__ __forceinline__ uint4 finite_bias_words(uint4 w)
{
    typedef __attribute__((ext_vector_type(2))) unsigned short u16x2;
    union {
        uint4 u;
        u16x2 h[4];
    } c;
    c.u = w;
    const u16x2 bound = {0xff7f, 0xff7f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        c.h[i] = __builtin_elementwise_min(c.h[i], bound);
    }
    return c.u;
}

// The same selectors with fp16 ones, for the log2-unit loop, whose pair-bias fragments are fp16.
__device__ __forceinline__ void make_selectors_f16(int lane, f16x8 &sel0, f16x8 &sel1)
{
    const int r = lane & 31, g = lane >> 5;
    const int gi = (r >> 2) & 1;
    const int w = 4 * (r >> 3) + (r & 3);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sel0[e] = (_Float16)((gi == g && w == e) ? 1.0f : 0.0f);
        sel1[e] = (_Float16)((gi == g && w == e + 8) ? 1.0f : 0.0f);
    }
}

// Mask bias of one batch row -> LDS as fp32 (keys past S get -inf), plus one flag bit per 32-key tile
// saying "this tile needs the mask added" (non-zero bias or ragged tail).  Wave w covers keys
// [64w, 64w+64); *flag_word must have been zeroed before, with a barrier in between.
// bias_row[k * stride_k] is the mask bias itself, or (from_mask) the 0/1 mask, turned into 1e9*(mask-1) here with the
// same multiply-add and bf16 rounding as the stand-alone mask-bias pass.
template <bool NEAR = false> // NEAR: S * stride_k < 2^31 and stride_k < 2^24 (checked on the host), 32-bit offsets
__device__ __forceinline__ void stage_mask_part(const bf16_t *bias_row, float *mask, uint32_t *flag_word, int S, int NB,
                                                int wave, int lane, float scale = 1.0f, int64_t stride_k = 1,
                                                bool from_mask = false)
{
    const int k = wave * 64 + lane;
    if (wave * 64 < NB * 32) {
        float mv = -INFINITY;
        if (k < S) {
            mv = to_f32(bias_row[NEAR ? (int64_t)__umul24((uint32_t)k, (uint32_t)stride_k) : k * stride_k]);
            if (from_mask) {
                mv = to_f32((bf16_t)fmaf(mv, 1e9f, -1e9f));
            }
            mv *= scale;
        }
        if (k < NB * 32) {
            mask[k] = mv;
        }
        const unsigned long long nz = __ballot(k < NB * 32 && mv != 0.f);
        const uint32_t bits = (((uint32_t)nz != 0u ? 1u : 0u) | ((uint32_t)(nz >> 32) != 0u ? 2u : 0u)) << (2 * wave);
        if (lane == 0 && bits != 0u) {
            atomicOr(flag_word, bits);
        }
    }
}

// stage_mask_part for the two-row kernel, which adds a row's mask bias to its logits with one more MFMA (a rank-one
// product of the per-key values with ones) instead of sixteen vector additions per tile: the value of key k is stored
// as two bf16, v = hi + lo to 2^-17 of |v|, the k-slots 0 and 1 of that MFMA's A operand.  -inf (keys past S): hi = -inf,
// lo = 0.
template <bool NEAR = false>
__device__ __forceinline__ void stage_mask_words(const bf16_t *bias_row, uint32_t *words, uint32_t *flag_word, int S, int NB,
                                                 int wave, int lane, float scale, int64_t stride_k, bool from_mask)
{
    const int k = wave * 64 + lane;
    if (wave * 64 < NB * 32) {
        float mv = -INFINITY;
        if (k < S) {
            mv = to_f32(bias_row[NEAR ? (int64_t)__umul24((uint32_t)k, (uint32_t)stride_k) : k * stride_k]);
            if (from_mask) {
                mv = to_f32((bf16_t)fmaf(mv, 1e9f, -1e9f));
            }
            mv *= scale;
        }
        if (k < NB * 32) {
            const bf16_t hi = (bf16_t)mv;
            const float hf = to_f32(hi);
            const float rest = (hf == mv || !(fabsf(hf) < INFINITY)) ? 0.f : mv - hf; // a NaN stays one through hi
            const bf16_t lo = (bf16_t)rest;
            bf16x2 pair;
            pair[0] = hi, pair[1] = lo;
            words[k] = __builtin_bit_cast(uint32_t, pair);
        }
        const unsigned long long nz = __ballot(k < NB * 32 && mv != 0.f);
        const uint32_t bits = (((uint32_t)nz != 0u ? 1u : 0u) | ((uint32_t)(nz >> 32) != 0u ? 2u : 0u)) << (2 * wave);
        if (lane == 0 && bits != 0u) {
            atomicOr(flag_word, bits);
        }
    }
}

__device__ __forceinline__ float mask_word_value(uint32_t w)
{
    return __uint_as_float(w << 16) + __uint_as_float(w & 0xffff0000u);
}

// The value stage_mask_part would store for key k, in two steps for kernels that fetch the mask early and store it
// later, so that nothing waits for the load where it is issued: the raw element of key min(k, S - 1) ...
__device__ __forceinline__ bf16_t mask_bias_fetch(const bf16_t *bias_row, int S, int k, int64_t stride_k)
{
    return bias_row[(k < S ? k : S - 1) * stride_k];
}

// ... and the value made of it where it is stored.
__device__ __forceinline__ float mask_bias_finish(bf16_t raw, bool in_range, float scale, bool from_mask)
{
    float mv = to_f32(raw);
    if (from_mask) {
        mv = to_f32((bf16_t)fmaf(mv, 1e9f, -1e9f));
    }
    return in_range ? mv * scale : -INFINITY;
}

// Flash-style attention of one 32-query block against all keys of the unit.
//   lds_k / lds_v : K and V fragments of the unit, [tile][kstep][lane] in 16-byte units
//   mask4         : fp32 mask bias in LDS, already offset by 16*g floats; flags: one bit per tile
//   nb_head       : pair bias of this head, [S, S] with row stride nb_sq (HAS_NB only); q0row = first
//                   query of the block
//   panel         : wave-private 4 KB staging panel, or nullptr to load the pair bias directly
//   q0, q1        : Q^T fragments scaled by 1/sqrt(d)
// Returns the unnormalised O^T accumulator and the row sum (identical in both lane halves).
// Per key tile: the logits accumulator starts at the mask bias (or 0); two MFMAs with the 0/1 selectors
// add the pair bias straight from its bf16 words (exact), two add q.k; the running maximum is
// refreshed only when some row's tile maximum exceeds it by RESCALE_GAP; probabilities go from the
// accumulator registers into the B operand of the P.V MFMAs without touching LDS.  The logits of
// tile t+1 are issued before the softmax of tile t so that the matrix core works under the VALU.
// Pair bias arrives two key tiles (64 keys = one 128-byte line per query) at a time through the
// staging panel, prefetched one pair ahead into registers; tiles of a ragged or unaligned tail are
// read directly.
template <bool HAS_NB>
__device__ __forceinline__ void attend_block(const uint4 *lds_k, const uint4 *lds_v, const f32x4 *mask4, uint32_t flags,
                                             const bf16_t *nb_head, int64_t nb_sq, int q0row, bool nb_vec, uint4 *panel,
                                             bf16x8 q0, bf16x8 q1, bf16x8 sel0, bf16x8 sel1, int NB, int S, int lane,
                                             f32x16 &o_out, float &l_out)
{
    const int r = lane & 31, g = lane >> 5;
    const int prow = pi_row(r);
    f32x16 o = zero16();
    float m_run = -1e30f; // finite, so the first rescale factor is exp2(-huge) = 0, never NaN
    float lsum = 0.f;     // this lane's share of the row sum; the two halves are added at the end
    bf16x2 one2;
    one2[0] = (bf16_t)1.0f, one2[1] = (bf16_t)1.0f;

    const int qrow = q0row + prow < S ? q0row + prow : S - 1;
    const bf16_t *nbrow = HAS_NB ? nb_head + (int64_t)qrow * nb_sq + 16 * g : nullptr;
    // number of leading tile pairs that go through the staging panel
    const int staged_pairs = (HAS_NB && panel != nullptr && nb_vec) ? S / 64 : 0;
    PanelRegs pf; // the next staged pair, in flight from global memory
    if (HAS_NB && staged_pairs > 0) {
        pf = panel_load(nb_head, nb_sq, q0row, S - 1, 0, lane);
    }

    // pair-bias words of key tile t for this lane (16 consecutive keys): B operands of the selector MFMAs
    auto nb_words = [&](int t, uint4 &w0, uint4 &w1) {
        const int pair = t >> 1;
        if (pair < staged_pairs) {
            if ((t & 1) == 0) {
                panel_store(panel, lane, pf); // the previous pair's reads were issued earlier in program order
                if (pair + 1 < staged_pairs) {
                    pf = panel_load(nb_head, nb_sq, q0row, S - 1, (pair + 1) * 64, lane);
                }
            }
            const int c = 4 * (t & 1) + 2 * g;
            w0 = panel[panel_slot(prow, c)];
            w1 = panel[panel_slot(prow, c + 1)];
        } else if (nb_vec && (t + 1) * 32 <= S) {
            w0 = *reinterpret_cast<const uint4 *>(nbrow + t * 32);
            w1 = *reinterpret_cast<const uint4 *>(nbrow + t * 32 + 8);
        } else {
            const uint16_t *s16 = reinterpret_cast<const uint16_t *>(nbrow + t * 32);
            const int key0 = t * 32 + 16 * g;
            uint32_t wds[8];
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const uint32_t a0 = key0 + 2 * v < S ? s16[2 * v] : 0u;
                const uint32_t a1 = key0 + 2 * v + 1 < S ? s16[2 * v + 1] : 0u;
                wds[v] = a0 | (a1 << 16);
            }
            w0.x = wds[0], w0.y = wds[1], w0.z = wds[2], w0.w = wds[3];
            w1.x = wds[4], w1.y = wds[5], w1.z = wds[6], w1.w = wds[7];
        }
    };
    // logits^T of key tile t (rows = keys, columns = this wave's 32 queries), natural-log units
    auto logits = [&](int t, f32x16 &x) {
        if ((flags >> t) & 1u) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 mv = mask4[t * 8 + a];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x[4 * a + c] = mv[c];
                }
            }
        } else {
            x = zero16();
        }
        if (HAS_NB) {
            uint4 w0, w1;
            nb_words(t, w0, w1);
            x = mfma(sel0, as_bf16x8(finite_bias_words(w0)), x);
            x = mfma(sel1, as_bf16x8(finite_bias_words(w1)), x);
        }
        x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), q0, x);
        x = mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), q1, x);
    };
    // online softmax of tile t held in xc, then O^T += V^T . P; before that, start tile t+1 into xn
    auto step = [&](int t, f32x16 &xc, f32x16 &xn) {
        if (t + 1 < NB) {
            logits(t + 1, xn);
        }
        float mx = xc[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) {
            mx = fmaxf(mx, xc[v]);
        }
        mx = half_swap_max(mx);
        if (__any(mx > m_run + RESCALE_GAP)) {
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
            lsum *= alpha;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                o[v] *= alpha;
            }
            m_run = m_new;
        }
        const float ml = -m_run * LOG2E;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            xc[v] = __builtin_amdgcn_exp2f(fmaf(xc[v], LOG2E, ml));
        }
        // the row sum is taken over the bf16-rounded probabilities, two per dot2 instruction
        const bf16x8 p0 = pack8(xc, 0), p1 = pack8(xc, 8);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bf16x2 a, c;
            a[0] = p0[2 * v], a[1] = p0[2 * v + 1];
            c[0] = p1[2 * v], c[1] = p1[2 * v + 1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(a, one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(c, one2, lsum, false);
        }
        o = mfma(as_bf16x8(lds_v[(t * 2 + 0) * 64 + lane]), p0, o);
        o = mfma(as_bf16x8(lds_v[(t * 2 + 1) * 64 + lane]), p1, o);
    };

    // softmax of a finished logits tile and its P.V accumulation (the part of `step` after the lookahead)
    auto softmax_pv = [&](int t, f32x16 &xc) {
        float mx = xc[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) {
            mx = fmaxf(mx, xc[v]);
        }
        mx = half_swap_max(mx);
        if (__any(mx > m_run + RESCALE_GAP)) {
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
            lsum *= alpha;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                o[v] *= alpha;
            }
            m_run = m_new;
        }
        const float ml = -m_run * LOG2E;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            xc[v] = __builtin_amdgcn_exp2f(fmaf(xc[v], LOG2E, ml));
        }
        const bf16x8 p0 = pack8(xc, 0), p1 = pack8(xc, 8);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bf16x2 a, c;
            a[0] = p0[2 * v], a[1] = p0[2 * v + 1];
            c[0] = p1[2 * v], c[1] = p1[2 * v + 1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(a, one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(c, one2, lsum, false);
        }
        o = mfma(as_bf16x8(lds_v[(t * 2 + 0) * 64 + lane]), p0, o);
        o = mfma(as_bf16x8(lds_v[(t * 2 + 1) * 64 + lane]), p1, o);
    };
    // logits of a tile whose pair bias sits in the staging panel; no branches, so that the scheduler
    // can spread the LDS reads, MFMAs and the neighbouring softmax over each other
    auto logits_staged = [&](int t, f32x16 &x, auto with_mask) {
        if (decltype(with_mask)::value) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 mv = mask4[t * 8 + a];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x[4 * a + c] = mv[c];
                }
            }
        } else {
            x = zero16();
        }
        const int c0 = 4 * (t & 1) + 2 * g;
        x = mfma(sel0, as_bf16x8(finite_bias_words(panel[panel_slot(prow, c0)])), x);
        x = mfma(sel1, as_bf16x8(finite_bias_words(panel[panel_slot(prow, c0 + 1)])), x);
        x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), q0, x);
        x = mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), q1, x);
    };

    f32x16 xa, xb;
    logits(0, xa);
    int t = 0;
    // main loop: two key tiles per iteration while a further staged pair follows; straight-line body
    auto main_loop = [&](auto with_mask) {
        for (int pair = 0; pair + 1 < staged_pairs; ++pair) {
            const int t0 = 2 * pair;
            logits_staged(t0 + 1, xb, with_mask);
            softmax_pv(t0, xa);
            panel_store(panel, lane, pf); // pair+1; the reads of this pair were issued above
            // prefetch pair+2 (clamped to the last staged pair: a harmless re-read instead of a branch)
            const int nxt = pair + 2 < staged_pairs ? pair + 2 : staged_pairs - 1;
            pf = panel_load(nb_head, nb_sq, q0row, S - 1, nxt * 64, lane);
            logits_staged(t0 + 2, xa, with_mask);
            softmax_pv(t0 + 1, xb);
        }
    };
    if (HAS_NB && staged_pairs > 1) {
        if (flags != 0u) {
            main_loop(std::true_type{});
        } else {
            main_loop(std::false_type{});
        }
        t = 2 * (staged_pairs - 1);
    }
    // remaining tiles (last staged pair, unstaged or ragged tail, or everything when nothing is staged)
    for (; t < NB; t += 2) {
        step(t, xa, xb);
        if (t + 1 < NB) {
            step(t + 1, xb, xa);
        }
    }
    o_out = o;
    l_out = half_swap_sum(lsum);
}

// ---- attention of one 32-query block in log2 units (the mode the persistent kernel runs in whenever
// it can) ----
// All inputs of the logits are pre-scaled by log2(e): the Q fragments by the kernel, the pair bias by
// pair_bias_fragments_kernel, the mask bias when it is staged.  The accumulator of the logits MFMAs is
// then the exponent itself, and the softmax of a tile is 16 v_exp_f32 and 8 packed converts -- the
// vector ALU no longer bounds the loop.  What the VALU used to do is done by the matrix core:
//  * no running maximum: the probabilities are 2^logit, unshifted.  Softmax is shift invariant and
//    fp32 and bf16 both carry 8 exponent bits, so this is exact in the same sense as the shifted form
//    as long as nothing overflows or the whole row underflows; the caller checks the row sum for
//    that (1e-30 < l < 1e30) and repeats the block with SHIFT = true and the true row maximum
//    (row_max_l2) when the check fails.  SHIFT costs one subtract per logit.
//  * the row sums come from a 16x16x32 MFMA whose A operand adds up the keys of each query
//    (rowsum_selector), fed with the same bf16 probabilities as the P.V product.
// Every operand of a tile is fetched ahead into registers that the loop carries: K and V fragments
// from LDS one tile ahead, pair-bias fragments from global memory two tiles ahead (two contiguous 1 KB
// loads per tile and wave).  The 8 MFMAs of a tile sit, fenced, between the exp/convert pieces of the
// neighbouring tile's softmax.  The loop runs one extra (clamped) logits computation at the end
// instead of a peeled epilogue.  Requires an even number of key tiles.
//   nbf : this wave's fragment-major pair bias, already offset by the lane: tile t at nbf[(2t+m)*64]
//   returns the row sum of every lane's query in l_out

// Issue priority of a wave among the (up to three) waves of its workgroup on one SIMD, by time slices of the clock they
// all see: in slice s the wave with turn (s + d) mod 3 gets priority 2 - d, so over three slices every wave is first,
// second and third once, however far it has come.  Left to the arbiter's oldest-first rule the oldest wave runs its
// attention almost alone and the youngest is left to finish by itself while the others wait at the barrier.  The
// branches sit inside one asm statement: as branches of a loop body they split the body into blocks, and the register
// allocator spills across them.  Call once per tile pair; reset with s_setprio 0 after the loop.
__device__ __forceinline__ void timeslice_priority(uint32_t turn, int shift)
{
    const uint32_t tick = ((uint32_t)__builtin_amdgcn_s_memtime() >> shift) & 0x3fffu;
    const uint32_t slice = tick - 3u * ((tick * 0x5556u) >> 16); // tick mod 3
    const uint32_t d = turn >= slice ? turn - slice : turn + 3u - slice;
    asm volatile("s_cmp_eq_u32 %0, 0\n\t"
                 "s_cbranch_scc1 .Lfirst_%=\n\t"
                 "s_cmp_eq_u32 %0, 1\n\t"
                 "s_cbranch_scc1 .Lsecond_%=\n\t"
                 "s_setprio 0\n\t"
                 "s_branch .Ldone_%=\n"
                 ".Lfirst_%=:\n\t"
                 "s_setprio 2\n\t"
                 "s_branch .Ldone_%=\n"
                 ".Lsecond_%=:\n\t"
                 "s_setprio 1\n"
                 ".Ldone_%=:"
                 :
                 : "s"(d)
                 : "scc");
}

// A operand of the row-sum MFMA (16x16x32: lane -> row lane&15, k-chunk lane>>4).  The B operand is a
// probability fragment of the 32x32x16 layout (lane -> query lane&31, 8 keys of half lane>>5), which the
// 16x16x32 shape reads as column lane&15, k-chunk lane>>4: chunks 0 and 2 belong to query n, chunks 1 and
// 3 to query n+16.  Row 0 of A therefore sums chunks 0 and 2, row 1 chunks 1 and 3; the sums of
// queries n and n+16 end up in lane n, accumulator registers 0 and 1.
__device__ __forceinline__ bf16x8 rowsum_selector(int lane)
{
    const int i = lane & 15, c = lane >> 4;
    const float v = ((i == 0 && (c & 1) == 0) || (i == 1 && (c & 1) == 1)) ? 1.0f : 0.0f;
    bf16x8 a;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (bf16_t)v;
    }
    return a;
}

__device__ __forceinline__ float rowsum_fetch(const f32x4 &lacc, int lane)
{
    const int q = lane & 31;
    const int src = (q & 15) * 4;
    const float a0 = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(lacc[0])));
    const float a1 = __int_as_float(__builtin_amdgcn_ds_bpermute(src, __float_as_int(lacc[1])));
    return (q >> 4) ? a1 : a0;
}

template <bool HAS_NB, bool WITH_MASK, bool SHIFT>
__device__ __forceinline__ void attend_block_l2(const uint4 *lds_k, const uint4 *lds_v, const f32x4 *mask4,
                                                const uint4 *nbf, bf16x8 q0, bf16x8 q1, f16x8 sel0, f16x8 sel1,
                                                bf16x8 sumsel, int NB, int lane, float shift, f32x16 &o_out, float &l_out,
                                                int prio_phase = -1, int fair_turn = -1)
{
    const int npairs = NB >> 1;
    const uint4 *kp = lds_k + lane;
    const uint4 *vp = lds_v + lane;

    auto init = [&](int t) {
        f32x16 x;
        if (WITH_MASK) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 mv = mask4[t * 8 + a];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x[4 * a + c] = mv[c];
                }
            }
        } else {
            x = zero16();
        }
        return x;
    };
    auto clampt = [&](int t) { return t < NB ? t : NB - 1; };

    // pair-bias words: wa* belong to even tiles, wb* to odd tiles
    uint4 wa0 = {}, wa1 = {}, wb0 = {}, wb1 = {}, k0, k1, v0, v1;
    if (HAS_NB) {
        wa0 = nbf[0], wa1 = nbf[64];
        wb0 = nbf[2 * 64], wb1 = nbf[3 * 64];
        // Pinned in this order, ahead of the reload of wa below: the loop then finds the loads in flight in the order it
        // leaves them in itself (odd tile's words older than the even tile's), and its wait at the top lets the two
        // newest stay in flight instead of draining the queue.
        __builtin_amdgcn_sched_barrier(0);
    }
    k0 = kp[0], k1 = kp[64];
    f32x16 xa = init(0), xb;
    if (HAS_NB) {
        xa = mfma_f16(sel0, as_f16x8(wa0), xa);
        xa = mfma_f16(sel1, as_f16x8(wa1), xa);
        wa0 = nbf[clampt(2) * 128], wa1 = nbf[clampt(2) * 128 + 64];
    }
    xa = mfma(as_bf16x8(k0), q0, xa);
    xa = mfma(as_bf16x8(k1), q1, xa);
    k0 = kp[2 * 64], k1 = kp[3 * 64];
    v0 = vp[0], v1 = vp[64];

    f32x16 o = zero16();
    f32x4 lacc = {0.f, 0.f, 0.f, 0.f};

    auto exp4 = [&](f32x16 &x, int base) {
#pragma unroll
        for (int v = base; v < base + 4; ++v) {
            x[v] = __builtin_amdgcn_exp2f(SHIFT ? x[v] - shift : x[v]);
        }
    };
    auto fence = [] { __builtin_amdgcn_sched_barrier(0); };
    // One half step: the softmax and P.V of the finished tile `xc`, with the logits MFMAs of the
    // following tile `xn` (pair-bias words w0, w1) spread between its pieces; t_w is the tile whose
    // pair-bias words replace w0, w1 once consumed, t_k the tile whose K fragments replace k0, k1.
    auto half_step = [&](f32x16 &xc, f32x16 &xn, int t_next, uint4 &w0, uint4 &w1, int t_w, int t_k) {
        bf16x8 p0, p1;
        xn = init(t_next);
        if (HAS_NB) {
            xn = mfma_f16(sel0, as_f16x8(w0), xn);
            exp4(xc, 0);
            fence();
            xn = mfma_f16(sel1, as_f16x8(w1), xn);
            w0 = nbf[t_w * 128], w1 = nbf[t_w * 128 + 64];
            exp4(xc, 4);
            p0 = pack8(xc, 0);
            fence();
        } else {
            exp4(xc, 0);
            exp4(xc, 4);
            p0 = pack8(xc, 0);
            fence();
        }
        xn = mfma(as_bf16x8(k0), q0, xn);
        o = mfma(as_bf16x8(v0), p0, o);
        exp4(xc, 8);
        fence();
        xn = mfma(as_bf16x8(k1), q1, xn);
        lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sumsel, p0, lacc, 0, 0, 0);
        k0 = kp[(t_k * 2 + 0) * 64], k1 = kp[(t_k * 2 + 1) * 64];
        exp4(xc, 12);
        p1 = pack8(xc, 8);
        fence();
        o = mfma(as_bf16x8(v1), p1, o);
        lacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(sumsel, p1, lacc, 0, 0, 0);
    };

    for (int pair = 0; pair < npairs; ++pair) {
        if (fair_turn >= 0) {
            timeslice_priority((uint32_t)fair_turn, FAIR_SLICE_SHIFT);
        }
        if (prio_phase >= 0) {
            // two waves of one workgroup share a SIMD in lock step; the arbiter prefers the older one, which then runs
            // ahead and leaves the other to finish alone.  Alternating the issue priority per tile pair keeps them level.
            if ((pair + prio_phase) & 1) {
                __builtin_amdgcn_s_setprio(1);
            } else {
                __builtin_amdgcn_s_setprio(0);
            }
        }
        const int t1 = 2 * pair + 1;
        const int tn = pair + 1 < npairs ? 2 * pair + 2 : 2 * pair; // next pair's first tile, clamped
        // ---- odd tile's logits under the even tile's softmax ----
        half_step(xa, xb, t1, wb0, wb1, clampt(t1 + 2), tn);
        v0 = vp[(t1 * 2 + 0) * 64], v1 = vp[(t1 * 2 + 1) * 64];
        fence();
        // ---- next pair's even tile under the odd tile's softmax ----
        half_step(xb, xa, tn, wa0, wa1, clampt(tn + 2), tn + 1);
        v0 = vp[(tn * 2 + 0) * 64], v1 = vp[(tn * 2 + 1) * 64];
        fence();
    }
    if (fair_turn >= 0) {
        __builtin_amdgcn_s_setprio(0);
    }
    o_out = o;
    l_out = rowsum_fetch(lacc, lane);
}

// Row maxima of the logits (log2 units) of one 32-query block over all key tiles: the shift for the
// repeat of attend_block_l2 after an overflow or underflow.  Not a hot path: operands are loaded at use.
template <bool HAS_NB>
__device__ __forceinline__ float row_max_l2(const uint4 *lds_k, const f32x4 *mask4, const uint4 *nbf, bf16x8 q0, bf16x8 q1,
                                            f16x8 sel0, f16x8 sel1, int NB, int lane)
{
    float mx = -INFINITY;
    for (int t = 0; t < NB; ++t) {
        f32x16 x;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const f32x4 mv = mask4[t * 8 + a];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                x[4 * a + c] = mv[c];
            }
        }
        if (HAS_NB) {
            x = mfma_f16(sel0, as_f16x8(nbf[t * 128]), x);
            x = mfma_f16(sel1, as_f16x8(nbf[t * 128 + 64]), x);
        }
        x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), q0, x);
        x = mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), q1, x);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            mx = fmaxf(mx, x[v]);
        }
    }
    mx = half_swap_max(mx);
    return mx; // finite: a fully masked row has -1e9*log2(e) everywhere
}

// The same attention of one 32-query block for kernels without a staging panel (long sequences, where
// K and V fill the LDS): every lane reads the pair bias of its own query row directly, 16 consecutive
// keys per tile, prefetched one tile ahead into registers.
template <bool HAS_NB>
__device__ __forceinline__ void attend_block_direct(const uint4 *lds_k, const uint4 *lds_v, const f32x4 *mask4,
                                                    uint32_t flags, const bf16_t *nbrow, bool nb_vec, bf16x8 q0,
                                                    bf16x8 q1, bf16x8 sel0, bf16x8 sel1, int NB, int S, int lane,
                                                    f32x16 &o_out, float &l_out)
{
    const int g = lane >> 5;
    f32x16 o = zero16();
    float m_run = -1e30f; // finite, so the first rescale factor is exp2(-huge) = 0, never NaN
    float lsum = 0.f;     // this lane's share of the row sum; the two halves are added at the end
    uint32_t nbw[8];      // pair-bias words of the NEXT tile to be turned into logits (prefetched)
    bf16x2 one2;
    one2[0] = (bf16_t)1.0f, one2[1] = (bf16_t)1.0f;

    // raw pair-bias of key tile t for this lane: 16 consecutive keys, two bf16 per word
    auto fetch_nb = [&](int t) {
        if (!HAS_NB) {
            return;
        }
        const bf16_t *src = nbrow + t * 32;
        if (nb_vec && (t + 1) * 32 <= S) {
            const uint4 lo = *reinterpret_cast<const uint4 *>(src);
            const uint4 hi = *reinterpret_cast<const uint4 *>(src + 8);
            nbw[0] = lo.x, nbw[1] = lo.y, nbw[2] = lo.z, nbw[3] = lo.w;
            nbw[4] = hi.x, nbw[5] = hi.y, nbw[6] = hi.z, nbw[7] = hi.w;
        } else {
            const uint16_t *s16 = reinterpret_cast<const uint16_t *>(src);
            const int key0 = t * 32 + 16 * g;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                const uint32_t a0 = key0 + 2 * v < S ? s16[2 * v] : 0u;
                const uint32_t a1 = key0 + 2 * v + 1 < S ? s16[2 * v + 1] : 0u;
                nbw[v] = a0 | (a1 << 16);
            }
        }
    };
    // logits^T of key tile t (rows = keys, columns = this wave's 32 queries), natural-log units
    auto logits = [&](int t, f32x16 &x) {
        if ((flags >> t) & 1u) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 mv = mask4[t * 8 + a];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    x[4 * a + c] = mv[c];
                }
            }
        } else {
            x = zero16();
        }
        if (HAS_NB) {
            uint4 w0, w1;
            w0.x = nbw[0], w0.y = nbw[1], w0.z = nbw[2], w0.w = nbw[3];
            w1.x = nbw[4], w1.y = nbw[5], w1.z = nbw[6], w1.w = nbw[7];
            x = mfma(sel0, as_bf16x8(finite_bias_words(w0)), x);
            x = mfma(sel1, as_bf16x8(finite_bias_words(w1)), x);
            if (t + 1 < NB) {
                fetch_nb(t + 1); // in flight while this tile's MFMAs and the previous tile's softmax run
            }
        }
        x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), q0, x);
        x = mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), q1, x);
    };
    // online softmax of tile t held in xc, then O^T += V^T . P; before that, start tile t+1 into xn
    auto step = [&](int t, f32x16 &xc, f32x16 &xn) {
        if (t + 1 < NB) {
            logits(t + 1, xn);
        }
        float mx = xc[0];
#pragma unroll
        for (int v = 1; v < 16; ++v) {
            mx = fmaxf(mx, xc[v]);
        }
        mx = half_swap_max(mx);
        if (__any(mx > m_run + RESCALE_GAP)) {
            const float m_new = fmaxf(m_run, mx);
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_new) * LOG2E);
            lsum *= alpha;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                o[v] *= alpha;
            }
            m_run = m_new;
        }
        const float ml = -m_run * LOG2E;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            xc[v] = __builtin_amdgcn_exp2f(fmaf(xc[v], LOG2E, ml));
        }
        // the row sum is taken over the bf16-rounded probabilities, two per dot2 instruction
        const bf16x8 p0 = pack8(xc, 0), p1 = pack8(xc, 8);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bf16x2 a, c;
            a[0] = p0[2 * v], a[1] = p0[2 * v + 1];
            c[0] = p1[2 * v], c[1] = p1[2 * v + 1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(a, one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(c, one2, lsum, false);
        }
        o = mfma(as_bf16x8(lds_v[(t * 2 + 0) * 64 + lane]), p0, o);
        o = mfma(as_bf16x8(lds_v[(t * 2 + 1) * 64 + lane]), p1, o);
    };

    f32x16 xa, xb;
    fetch_nb(0);
    logits(0, xa);
    for (int t = 0; t < NB; t += 2) {
        step(t, xa, xb);
        if (t + 1 < NB) {
            step(t + 1, xb, xa);
        }
    }
    o_out = o;
    l_out = half_swap_sum(lsum);
}

// avg[b, q, h, :] = O / l * gate for the 32 queries of one block; gate values in accumulator order
__device__ __forceinline__ void store_gated(bf16_t *dst, const f32x16 &o, float inv, const f32x16 &gate)
{
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        bf16x4 ov;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            ov[c] = (bf16_t)(o[4 * a + c] * inv * gate[4 * a + c]);
        }
        *reinterpret_cast<bf16x4 *>(dst + 8 * a) = ov;
    }
}

// Copies head h's rows of `count` weight matrices (first, first + 1, ...) into LDS in MFMA fragment order.  One
// fragment -- a matrix's 32 rows by 16 channels, 1 KB -- is one wave-wide copy, so the fragment index is wave-uniform
// and the matrix pointer is picked with scalar selects (indexing the pointer array per lane made every copy wait for a
// load of the pointer first).  Whole batches of eight fragments per wave go without a branch between the loads and the
// stores: eight L2 round trips overlap instead of queueing (one at a time they were 9 % of the long-sequence kernel).
// ------------------------------------------------------------------------------------------------
template <int C>
__device__ inline void stage_weight_fragments(uint4 *lds_w, const FusedParams &p, int first, int count, int h, int wave,
                                              int nwaves, int lane)
{
    constexpr int CK = C / 16;
    const int nfrag = count * CK;
    auto fragment = [&](int f) {
        const int m = first + f / CK, ks = f % CK;
        const bf16_t *w = m == 0 ? p.w[0] : m == 1 ? p.w[1] : m == 2 ? p.w[2] : p.w[3];
        return *reinterpret_cast<const uint4 *>(w + (int64_t)(h * HEAD + (lane & 31)) * C + ks * 16 + (lane >> 5) * 8);
    };
    int f = wave;
    for (; f + (WEIGHT_LOADS_IN_FLIGHT - 1) * nwaves < nfrag; f += WEIGHT_LOADS_IN_FLIGHT * nwaves) {
        uint4 t[WEIGHT_LOADS_IN_FLIGHT];
#pragma unroll
        for (int k = 0; k < WEIGHT_LOADS_IN_FLIGHT; ++k) {
            t[k] = fragment(f + k * nwaves);
        }
#pragma unroll
        for (int k = 0; k < WEIGHT_LOADS_IN_FLIGHT; ++k) {
            lds_w[(f + k * nwaves) * 64 + lane] = t[k];
        }
    }
    for (; f < nfrag; f += nwaves) {
        lds_w[f * 64 + lane] = fragment(f);
    }
}

// ------------------------------------------------------------------------------------------------
// fused_head_kernel: one workgroup per (b, h) unit
// LDS carve-up, in 16-byte units unless noted:
//   [0, GW*CK*64)               staged weight fragments  [slot][kstep][lane]
//   [.., +NT*2*64)              K fragments              [tile][kstep][lane]
//   [.., +NT*2*64)              V fragments              [tile][kstep][lane]
// The mask of the batch row (floats, -inf past S) and the tile flags are needed only by the attention phase and take
// the place of the weight fragments once the projections are done; every thread fetches its mask values at the start
// and keeps them in registers until then.  At 1024 keys that leaves room for all four weight matrices of a
// 128-channel head (two of a 256-channel one) beside K and V, so the input rows are read once (twice).
// ------------------------------------------------------------------------------------------------
template <int C, int BPW, bool HAS_NB>
__global__ __launch_bounds__(64 * max_waves(C, BPW)) void fused_head_kernel(FusedParams p)
{
    constexpr int CK = C / 16;
    constexpr bool V_ALIAS = C == 256 && BPW == 4; // second LDS layout, below
    constexpr bool ONE_GROUP = V_ALIAS || C == 128; // all four weight matrices staged at once, always (see make_plan)
    extern __shared__ uint4 lds[];

    // XCD-aware unit mapping: consecutive workgroup ids land on different XCDs (8 of them), so the H
    // heads of one batch row are placed 8 ids apart and share one XCD's L2 for their reads of x[b].
    const int u = blockIdx.x;
    const int xcd = u & 7;
    const int slot = u >> 3;
    const int h = slot % p.H;
    const int b = (slot / p.H) * 8 + xcd;
    if (b >= p.B) {
        return;
    }
    const int tid = threadIdx.x;
    const int nthreads = p.NW * 64;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform, kept in a scalar register
    const int r = lane & 31, g = lane >> 5;
    const int S = p.S, NB = p.NB, NT = p.NT, NW = p.NW, GW = ONE_GROUP ? 4 : p.GW;

    // Second layout (256 channels at the longest sequences, NT == NB): all four weight matrices (64 KB) lie on the V array,
    // whose fragments wait in registers until the projections are done; K, then V / weights, then one 4 KB input panel
    // per wave (the mask's place afterwards).  The input rows are then staged once for all four projections.
    uint4 *lds_w = lds;
    uint4 *lds_k = lds_w + GW * CK * 64;
    uint4 *lds_v = lds_k + NT * 2 * 64;
    uint4 *own_panel = nullptr;
    float *mask = reinterpret_cast<float *>(lds_w);
    if constexpr (V_ALIAS) {
        lds_k = lds, lds_v = lds_k + NT * 2 * 64, lds_w = lds_v;
        uint4 *panels = lds_v + (NT * 2 * 64 > 4 * CK * 64 ? NT * 2 * 64 : 4 * CK * 64); // past the longer of V and weights
        own_panel = panels + wave * 256;
        mask = reinterpret_cast<float *>(panels);
    }
    uint32_t *part_flags = reinterpret_cast<uint32_t *>(mask + NT * 32); // two flag bits per 64 keys, one word each
    uint4 vpark[V_ALIAS ? BPW : 1][2];

    if (NT > NB) { // phantom key tile: zero K and V fragments (V after the projections when the weights lie there)
        const uint4 z4 = {0u, 0u, 0u, 0u};
        for (int idx = tid; idx < 128; idx += nthreads) {
            lds_k[NB * 2 * 64 + idx] = z4;
            if constexpr (!V_ALIAS) {
                lds_v[NB * 2 * 64 + idx] = z4;
            }
        }
    }
    // wave w holds the mask of keys [64(w + q NW), +64): NT <= 4 NW + 1 tiles are at most 2 NW such parts
    constexpr int MASK_PARTS = (BPW + 1) / 2;
    bf16_t mask_raw[MASK_PARTS];
#pragma unroll
    for (int q = 0; q < MASK_PARTS; ++q) {
        mask_raw[q] = mask_bias_fetch(p.bias + (int64_t)b * p.bias_sb, S, (wave + q * NW) * 64 + lane, p.bias_sk);
    }

    const float qmul = p.l2mode ? p.qscale * LOG2E : p.qscale;
    // ---- projections, in groups of GW weight matrices staged through LDS ----
    bf16x8 qf[BPW][2];   // Q^T fragments (B operand of the logits MFMA), scaled by 1/sqrt(d)
    bf16x8 gate[BPW][2]; // sigmoid(gate) in accumulator order, packed
    const int npass = ONE_GROUP ? 1 : 4 / GW;
    // With at least two matrices per group K and V (matrices 0 and 1) share a group; the groups are then walked from the
    // last to the first, so that K and V come last and the K/V fragment slots of a block stay free until that block's
    // own results land in them.  That lets the input rows take the coalesced route: a 4 KB staging panel aliased onto
    // the block's K slot (rows 0-15) and V slot (rows 16-31), private to the wave that owns the block.  With one matrix
    // per group there is no such free space (LDS is full at that sequence length) and the fragments are loaded from
    // global memory directly.
    const bool staged_input = ONE_GROUP || GW >= 2;
    const int prow = pi_row(r);
    for (int pi = 0; pi < npass; ++pi) {
        const int pass = staged_input ? npass - 1 - pi : pi;
        if (pi > 0) {
            __syncthreads(); // previous group's fragments are no longer being read
        } else {
        }
        stage_weight_fragments<C>(lds_w, p, pass * GW, GW, h, wave, NW, lane);
        __syncthreads();
        if (pi == 0) {
        }
        if constexpr (C == 128 && BPW >= 3) {
            // Two blocks of the wave per walk over the weight fragments: the input fragments of both stay in registers
            // (64 of them) and every fragment of the weights is read from LDS once for the pair (1 KB per MFMA when the
            // blocks are projected one after the other); all rows of a pair are asked for at once.  A pair whose second
            // block does not exist projects the first one twice and stores it once.
#pragma unroll
            for (int i0 = 0; i0 < BPW; i0 += 2) {
                constexpr int PAIR = 2;
                int j0 = wave + i0 * NW;
                if (j0 >= NB) {
                    continue;
                }
                asm volatile("" : "+s"(j0)); // opaque, as below: addresses are formed per pair, not kept across the loop
                const bool second = i0 + 1 < BPW && j0 + NW < NB;
                const bf16_t *xb = p.x + (int64_t)b * p.x_sb;
                bf16x8 xf[PAIR][CK];
                int jn[PAIR];
                jn[0] = j0, jn[1] = second ? j0 + NW : j0;
                PanelRegs t[PAIR][CK / 4];
#pragma unroll
                for (int n = 0; n < PAIR; ++n) {
#pragma unroll
                    for (int c = 0; c < CK / 4; ++c) {
                        t[n][c] = panel_load_near(xb + c * 64, (uint32_t)p.x_ld, jn[n] * 32, S - 1, 0, lane);
                    }
                }
#pragma unroll
                for (int n = 0; n < PAIR; ++n) {
                    const int j = jn[n];
                    uint4 *kslot = lds_k + j * 128, *vslot = lds_v + j * 128 - 128; // panel slots 0-127 and 128-255
                    const uint4 *fsrc = prow < 16 ? kslot : vslot;
                    const int srow8 = lane >> 3, chunk = lane & 7;
#pragma unroll
                    for (int c = 0; c < CK / 4; ++c) {
                        kslot[panel_slot(srow8, chunk)] = t[n][c].r0;
                        kslot[panel_slot(srow8 + 8, chunk)] = t[n][c].r1;
                        vslot[panel_slot(srow8 + 16, chunk)] = t[n][c].r2;
                        vslot[panel_slot(srow8 + 24, chunk)] = t[n][c].r3;
#pragma unroll
                        for (int k = 0; k < 4; ++k) {
                            xf[n][4 * c + k] = as_bf16x8(fsrc[panel_slot(prow, 2 * k + g)]);
                        }
                    }
                }
#pragma unroll
                for (int m = 0; m < 4; ++m) {
                    const uint4 *wsrc = lds_w + m * CK * 64 + lane;
                    f32x16 acc[PAIR];
                    acc[0] = zero16(), acc[1] = zero16();
#pragma unroll
                    for (int ks = 0; ks < CK; ++ks) {
                        const bf16x8 wf = as_bf16x8(wsrc[ks * 64]);
#pragma unroll
                        for (int n = 0; n < PAIR; ++n) {
                            // V[s][d]: rows = sequence positions; the others W_h . x^T: rows = head-dim
                            acc[n] = m == PROJ_V ? mfma(xf[n][ks], wf, acc[n]) : mfma(wf, xf[n][ks], acc[n]);
                        }
                    }
#pragma unroll
                    for (int n = 0; n < PAIR; ++n) {
                        if (n == 1 && i0 + 1 >= BPW) {
                            continue;
                        }
                        const int i = i0 + n;
                        if (m == PROJ_V) {
                            if (n == 0 || second) {
                                lds_v[(jn[n] * 2 + 0) * 64 + lane] = as_uint4(pack8(acc[n], 0));
                                lds_v[(jn[n] * 2 + 1) * 64 + lane] = as_uint4(pack8(acc[n], 8));
                            }
                        } else if (m == PROJ_K) {
                            if (n == 0 || second) {
                                lds_k[(jn[n] * 2 + 0) * 64 + lane] = as_uint4(pack8(acc[n], 0));
                                lds_k[(jn[n] * 2 + 1) * 64 + lane] = as_uint4(pack8(acc[n], 8));
                            }
                        } else if (m == PROJ_Q) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                acc[n][v] *= qmul;
                            }
                            qf[i][0] = pack8(acc[n], 0);
                            qf[i][1] = pack8(acc[n], 8);
                        } else {
                            const float *bgp = p.bg + h * HEAD + 4 * g;
#pragma unroll
                            for (int a = 0; a < 4; ++a) {
                                const f32x4 bv = *reinterpret_cast<const f32x4 *>(bgp + 8 * a);
#pragma unroll
                                for (int c = 0; c < 4; ++c) {
                                    acc[n][4 * a + c] = sigmoid_fast(acc[n][4 * a + c] + bv[c]);
                                }
                            }
                            gate[i][0] = pack8(acc[n], 0);
                            gate[i][1] = pack8(acc[n], 8);
                        }
                    }
                }
            }
        } else {
#pragma unroll
        for (int i = 0; i < BPW; ++i) {
            int j = wave + i * NW;
            if (j >= NB) {
                continue;
            }
            // Opaque to the optimiser: otherwise the row addresses of every block of the wave are computed once, ahead
            // of the loop over the groups, and with three or four blocks of 256-channel rows they no longer fit the
            // registers -- each spilled address then costs a scratch round trip in front of the load it feeds.
            asm volatile("" : "+s"(j));
            bf16x8 xf[CK];
            if (staged_input) {
                const bf16_t *xb = p.x + (int64_t)b * p.x_sb;
                uint4 *kslot = lds_k + j * 128, *vslot = lds_v + j * 128 - 128; // panel slots 0-127 and 128-255
                if constexpr (V_ALIAS) {
                    kslot = vslot = own_panel;
                }
                const uint4 *fsrc = prow < 16 ? kslot : vslot;
                const int srow8 = lane >> 3, chunk = lane & 7;
                PanelRegs t = panel_load(xb, p.x_ld, j * 32, S - 1, 0, lane);
#pragma unroll
                for (int c = 0; c < CK / 4; ++c) {
                    kslot[panel_slot(srow8, chunk)] = t.r0;
                    kslot[panel_slot(srow8 + 8, chunk)] = t.r1;
                    vslot[panel_slot(srow8 + 16, chunk)] = t.r2;
                    vslot[panel_slot(srow8 + 24, chunk)] = t.r3;
                    if (c + 1 < CK / 4) {
                        t = panel_load(xb, p.x_ld, j * 32, S - 1, (c + 1) * 64, lane);
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        xf[4 * c + k] = as_bf16x8(fsrc[panel_slot(prow, 2 * k + g)]);
                    }
                }
            } else {
                int srow = j * 32 + prow;
                srow = srow < S ? srow : S - 1; // rows past the end repeat the last row; they are never stored
                const bf16_t *xrow = p.x + (int64_t)b * p.x_sb + (int64_t)srow * p.x_ld + g * 8;
#pragma unroll
                for (int ks = 0; ks < CK; ++ks) {
                    xf[ks] = as_bf16x8(*reinterpret_cast<const uint4 *>(xrow + ks * 16));
                }
            }
            for (int mm = 0; mm < GW; ++mm) {
                const int m = pass * GW + mm;
                const uint4 *wsrc = lds_w + mm * CK * 64 + lane;
                f32x16 acc = zero16();
                if (m == PROJ_V) {
                    // V[s][d]: rows = sequence positions, so a lane ends up with 16 keys of one head-dim
#pragma unroll
                    for (int ks = 0; ks < CK; ++ks) {
                        acc = mfma(xf[ks], as_bf16x8(wsrc[ks * 64]), acc);
                    }
                    if constexpr (V_ALIAS) {
                        vpark[i][0] = as_uint4(pack8(acc, 0));
                        vpark[i][1] = as_uint4(pack8(acc, 8));
                    } else {
                        lds_v[(j * 2 + 0) * 64 + lane] = as_uint4(pack8(acc, 0));
                        lds_v[(j * 2 + 1) * 64 + lane] = as_uint4(pack8(acc, 8));
                    }
                } else {
                    // W_h . x^T: rows = head-dim, columns = sequence positions
#pragma unroll
                    for (int ks = 0; ks < CK; ++ks) {
                        acc = mfma(as_bf16x8(wsrc[ks * 64]), xf[ks], acc);
                    }
                    if (m == PROJ_K) {
                        lds_k[(j * 2 + 0) * 64 + lane] = as_uint4(pack8(acc, 0));
                        lds_k[(j * 2 + 1) * 64 + lane] = as_uint4(pack8(acc, 8));
                    } else if (m == PROJ_Q) {
#pragma unroll
                        for (int v = 0; v < 16; ++v) {
                            acc[v] *= qmul;
                        }
                        qf[i][0] = pack8(acc, 0);
                        qf[i][1] = pack8(acc, 8);
                    } else {
                        const float *bgp = p.bg + h * HEAD + 4 * g;
#pragma unroll
                        for (int a = 0; a < 4; ++a) {
                            const f32x4 bv = *reinterpret_cast<const f32x4 *>(bgp + 8 * a);
#pragma unroll
                            for (int c = 0; c < 4; ++c) {
                                acc[4 * a + c] = sigmoid_fast(acc[4 * a + c] + bv[c]);
                            }
                        }
                        gate[i][0] = pack8(acc, 0);
                        gate[i][1] = pack8(acc, 8);
                    }
                }
            }
        }
        } // one block at a time
    }
    __syncthreads(); // K and V of the whole sequence are in LDS; the weight fragments are no longer read
    if constexpr (V_ALIAS) {
#pragma unroll
        for (int i = 0; i < BPW; ++i) {
            const int j = wave + i * NW;
            if (j < NB) {
                lds_v[(j * 2 + 0) * 64 + lane] = vpark[i][0];
                lds_v[(j * 2 + 1) * 64 + lane] = vpark[i][1];
            }
        }
        if (NT > NB && tid < 128) {
            lds_v[NB * 2 * 64 + tid] = uint4{0u, 0u, 0u, 0u};
        }
    }
#pragma unroll
    for (int q = 0; q < MASK_PARTS; ++q) {
        const int part = wave + q * NW;
        if (part * 64 < NT * 32) {
            const float mv = mask_bias_finish(mask_raw[q], part * 64 + lane < S, p.l2mode ? LOG2E : 1.0f, p.bias_is_mask != 0);
            mask[part * 64 + lane] = mv;
            const unsigned long long nz = __ballot(mv != 0.f);
            if (lane == 0) {
                part_flags[part] = ((uint32_t)nz != 0u ? 1u : 0u) | ((uint32_t)(nz >> 32) != 0u ? 2u : 0u);
            }
        }
    }
    __syncthreads();

    // ---- attention: each wave walks the key tiles for its own query blocks ----
    uint32_t flags = 0; // bit t: key tile t needs the mask added (non-zero bias or ragged tail)
    for (int part = 0; part * 64 < NT * 32; ++part) {
        flags |= part_flags[part] << (2 * part);
    }
    const f32x4 *mask4 = reinterpret_cast<const f32x4 *>(mask + 16 * g);
    // one pair of selector fragments, as bits: fp16 ones for the log2-unit loop (fp16 pair-bias fragments), bf16 ones otherwise
    uint4 selw0, selw1;
    if (p.l2mode) {
        f16x8 a, b;
        make_selectors_f16(lane, a, b);
        selw0 = as_uint4(a), selw1 = as_uint4(b);
    } else {
        bf16x8 a, b;
        make_selectors(lane, a, b);
        selw0 = as_uint4(a), selw1 = as_uint4(b);
    }
    const bf16x8 sumsel = rowsum_selector(lane);

#pragma unroll
    for (int i = 0; i < BPW; ++i) {
        const int j = wave + i * NW;
        if (j >= NB) {
            continue;
        }
        const int qpos = j * 32 + pi_row(r);
        const int qrow = qpos < S ? qpos : S - 1;
        f32x16 o;
        float l;
        if (p.l2mode) {
            const uint4 *nbf = HAS_NB ? p.nbf + ((int64_t)(h * NB + j) * NT * 2) * 64 + lane : nullptr;
            if (flags == 0u) {
                attend_block_l2<HAS_NB, false, false>(lds_k, lds_v, mask4, nbf, qf[i][0], qf[i][1], as_f16x8(selw0), as_f16x8(selw1), sumsel, NT,
                                                      lane, 0.f, o, l, (wave >> 2) & 1);
            } else {
                attend_block_l2<HAS_NB, true, false>(lds_k, lds_v, mask4, nbf, qf[i][0], qf[i][1], as_f16x8(selw0), as_f16x8(selw1), sumsel, NT,
                                                     lane, 0.f, o, l, (wave >> 2) & 1);
            }
            __builtin_amdgcn_s_setprio(0);
            if (__any(!(l > 1e-30f && l < 1e30f))) {
                // some probability overflowed or a whole row underflowed: shift by the true row maxima
                const float m = row_max_l2<HAS_NB>(lds_k, mask4, nbf, qf[i][0], qf[i][1], as_f16x8(selw0), as_f16x8(selw1), NT, lane);
                attend_block_l2<HAS_NB, true, true>(lds_k, lds_v, mask4, nbf, qf[i][0], qf[i][1], as_f16x8(selw0), as_f16x8(selw1), sumsel, NT,
                                                    lane, m, o, l);
            }
        } else {
            const bf16_t *nbrow = HAS_NB ? p.nb + (int64_t)h * p.nb_sh + (int64_t)qrow * p.nb_sq + 16 * g : nullptr;
            attend_block_direct<HAS_NB>(lds_k, lds_v, mask4, flags, nbrow, p.nb_vec != 0, qf[i][0], qf[i][1], as_bf16x8(selw0), as_bf16x8(selw1), NB,
                                        S, lane, o, l);
        }
        if (qpos < S) {
            f32x16 gv;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                gv[v] = to_f32(gate[i][v >> 3][v & 7]);
            }
            store_gated(p.avg + (int64_t)b * p.avg_sb + (int64_t)qpos * p.avg_ss + (int64_t)h * p.avg_sh + 4 * g, o,
                        __builtin_amdgcn_rcpf(l), gv);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// persistent_head_kernel: one workgroup per CU keeps one head for its lifetime and walks batch rows;
// wave j owns sequence block j (its K/V projection and its 32 queries).  Compared with one workgroup
// per (b, h) unit this stages the head's weights once, pays no workgroup launch per unit, and moves
// the two big streams -- input rows and pair bias -- through wave-private staging panels with fully
// coalesced loads.
// LDS, 16-byte units: W[4][CK][64]  K[NB][2][64]  V[NB][2][64]  panel[NB waves][256]  gate[NB waves][2][64];
// then floats mask[2][NB*32] and two uint32 of tile flags (both alternating by batch row).
// Per batch row: load and project (K, V, Q -> registers; gate -> LDS), barrier (previous row's attention
// is over everywhere), K and V -> LDS, barrier, attend.  A wave that finishes its attention early starts
// on the next row's loads and projections while the slower waves of its SIMD still attend, so the
// latency- and MFMA-bound projection phase overlaps the VALU-heavy attention phase.
// ------------------------------------------------------------------------------------------------
template <int C, bool HAS_NB, bool L2MODE, bool FUSED_LN>
__global__ __launch_bounds__(64 * max_waves(C, 1)) void persistent_head_kernel(FusedParams p)
{
    constexpr int CK = C / 16;
    constexpr int NP = CK / 4; // staging panels (64 channels each) per input row block
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform: values derived from it stay in scalar registers
    const int r = lane & 31, g = lane >> 5;
    const int S = p.S, NB = p.NB, NT = p.NT;
    const int nthreads = NB * 64;
    const int prow = pi_row(r);

    // workgroup -> (XCD, head, batch-row group): the H workgroups that share a batch-row sequence sit
    // on the same XCD (ids 8 apart) and walk it in step, so x[b] is read from HBM once per XCD
    const int w = blockIdx.x;
    const int xcd = w & 7;
    const int slot = w >> 3;
    const int h = slot % p.H;
    const int grp = slot / p.H;
    const int b0 = xcd + 8 * grp;
    const int bstep = 8 * p.ngrp;
    const int nrows = b0 < p.B ? (p.B - b0 + bstep - 1) / bstep : 0;

    uint4 *lds_w = lds;
    uint4 *lds_k = lds_w + 4 * CK * 64;
    uint4 *lds_v = lds_k + NT * 2 * 64;
    uint4 *panel = lds_v + NT * 2 * 64 + wave * 256;
    uint4 *gate_park_base = lds_v + NT * 2 * 64 + NB * 256 + wave * 128; // sigmoid(gate) waits here during attention
    float *mask_base = reinterpret_cast<float *>(lds_v + NT * 2 * 64 + NB * 256 + NB * 128); // two buffers of NT*32
    uint32_t *flag_words = reinterpret_cast<uint32_t *>(mask_base + 2 * NT * 32);            // two, alternating by batch row

    // the head's rows of the four weight matrices, in fragment order, for the whole kernel
    stage_weight_fragments<C>(lds_w, p, 0, 4, h, wave, nthreads >> 6, lane);
    if (tid == 0) {
        flag_words[0] = 0;
        flag_words[1] = 0;
    }
    if (NT > NB) { // phantom key tile: zero K and V fragments, never written again
        const uint4 z4 = {0u, 0u, 0u, 0u};
        for (int idx = tid; idx < 128; idx += nthreads) {
            lds_k[NB * 2 * 64 + idx] = z4;
            lds_v[NB * 2 * 64 + idx] = z4;
        }
    }
    std::conditional_t<L2MODE, f16x8, bf16x8> sel0, sel1; // fp16 ones for the log2-unit loop, whose pair-bias fragments are fp16
    if constexpr (L2MODE) {
        make_selectors_f16(lane, sel0, sel1);
    } else {
        make_selectors(lane, sel0, sel1);
    }
    __syncthreads();

    const int j = wave; // this wave's sequence block
    // With three waves per SIMD (128 channels) the waves take turns at the issue priorities during the attention; with two
    // (256 channels) the arbiter's own order measured 2 % faster.
    const int fair_turn = C == 128 ? wave >> 2 : -1;
    const float qmul = L2MODE ? p.qscale * LOG2E : p.qscale;
    const float mask_scale = L2MODE ? LOG2E : 1.0f;
    const bf16x8 sumsel = rowsum_selector(lane);
    for (int n = 0; n < nrows; ++n) {
        const int b = b0 + n * bstep;
        uint32_t *flag_word = flag_words + (n & 1);
        float *mask = mask_base + (n & 1) * NT * 32;
        // The lane index is opaque to the optimiser here: the row addresses and panel offsets derived from it are then
        // formed anew for every batch row (a few dozen vector instructions) instead of being kept across the attention
        // loop, where there is no register for them -- spilled, each costs a scratch round trip per batch row.
        int lane_x = lane;
        asm volatile("" : "+v"(lane_x));
        stage_mask_part<true>(p.bias + (int64_t)b * p.bias_sb, mask, flag_word, S, NT, wave, lane_x, mask_scale, p.bias_sk,
                              p.bias_is_mask != 0);

        // ---- input rows of the block -> fragments, 64 channels per staging panel ----
        const int prow_x = pi_row(lane_x & 31), g_x = lane_x >> 5;
        const bf16_t *xb = p.x + (int64_t)b * p.x_sb;
        const uint32_t x_pitch = (uint32_t)p.x_ld; // the host sends only near-addressable rows here
        bf16x8 xf[CK];
        if constexpr (FUSED_LN) {
            // The rows arrive un-normalised and are normalised between their load and their staging (arithmetic of
            // reference src/normalization/layernorm_kernel.h:21-53, result rounded to bf16 as the tensor it replaces
            // was).  A lane holds 8 channels per panel of four rows; a row's C channels sit in the 8 lanes that loaded
            // it, so its two sums cross three DPP steps.
            PanelRegs t[NP];
#pragma unroll
            for (int c = 0; c < NP; ++c) {
                t[c] = panel_load_near(xb + c * 64, x_pitch, j * 32, S - 1, 0, lane_x);
            }
            float gm[NP][8], bt[NP][8];
#pragma unroll
            for (int c = 0; c < NP; ++c) {
                const float *gsrc = p.ln_gamma + c * 64 + (lane_x & 7) * 8, *bsrc = p.ln_beta + c * 64 + (lane_x & 7) * 8;
#pragma unroll
                for (int e = 0; e < 8; e += 4) {
                    const f32x4 gv = *reinterpret_cast<const f32x4 *>(gsrc + e), bv = *reinterpret_cast<const f32x4 *>(bsrc + e);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        gm[c][e + k] = gv[k], bt[c][e + k] = bv[k];
                    }
                }
            }
            auto normalise_row = [&](uint4 (&words)[NP]) {
                float v[NP][8];
#pragma unroll
                for (int c = 0; c < NP; ++c) {
                    const bf16x8 in = as_bf16x8(words[c]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        v[c][e] = to_f32(in[e]);
                    }
                }
                const float x0 = __shfl(v[0][0], lane_x & ~7, 64); // first element of the row
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int c = 0; c < NP; ++c) {
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float d = v[c][e] - x0;
                        s1 += d;
                        s2 = fmaf(d, d, s2);
                    }
                }
                s1 = group_sum<8>(s1), s2 = group_sum<8>(s2);
                const float nch = (float)C;
                const float mean = s1 / nch + x0;
                const float var = fmaxf((s2 - s1 * s1 / nch) / nch, 0.f);
                const float rstd = __builtin_amdgcn_rsqf(var + p.ln_eps); // as the row kernels form it
                const float shift = -rstd * mean;
#pragma unroll
                for (int c = 0; c < NP; ++c) {
                    bf16x8 o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        o[e] = (bf16_t)fmaf(fmaf(v[c][e], rstd, shift), gm[c][e], bt[c][e]);
                    }
                    words[c] = as_uint4(o);
                }
            };
            {
                uint4 w0[NP], w1[NP], w2[NP], w3[NP];
#pragma unroll
                for (int c = 0; c < NP; ++c) {
                    w0[c] = t[c].r0, w1[c] = t[c].r1, w2[c] = t[c].r2, w3[c] = t[c].r3;
                }
                normalise_row(w0), normalise_row(w1), normalise_row(w2), normalise_row(w3);
#pragma unroll
                for (int c = 0; c < NP; ++c) {
                    t[c].r0 = w0[c], t[c].r1 = w1[c], t[c].r2 = w2[c], t[c].r3 = w3[c];
                }
            }
#pragma unroll
            for (int c = 0; c < NP; ++c) {
                panel_store(panel, lane_x, t[c]);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    xf[4 * c + k] = as_bf16x8(panel[panel_slot(prow_x, 2 * k + g_x)]);
                }
            }
        } else {
            PanelRegs ta, tb;
            ta = panel_load_near(xb, x_pitch, j * 32, S - 1, 0, lane_x);
#pragma unroll
            for (int c = 0; c < NP; c += 2) {
                if (c + 1 < NP) {
                    tb = panel_load_near(xb + (c + 1) * 64, x_pitch, j * 32, S - 1, 0, lane_x);
                }
                panel_store(panel, lane_x, ta);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    xf[4 * c + k] = as_bf16x8(panel[panel_slot(prow_x, 2 * k + g_x)]);
                }
                if (c + 1 < NP) {
                    if (c + 2 < NP) {
                        ta = panel_load_near(xb + (c + 2) * 64, x_pitch, j * 32, S - 1, 0, lane_x);
                    }
                    panel_store(panel, lane_x, tb);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        xf[4 * (c + 1) + k] = as_bf16x8(panel[panel_slot(prow_x, 2 * k + g_x)]);
                    }
                }
            }
        }
        // ---- four projections of the block ----
        bf16x8 q0, q1;
        uint4 kfrag0, kfrag1, vfrag0, vfrag1; // this block's K and V fragments, parked until the LDS arrays are free
        {
            uint4 *gate_park_x = gate_park_base + lane_x;
            const uint4 *wsrc = lds_w + lane_x;
            f32x16 acc = zero16();
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                acc = mfma(as_bf16x8(wsrc[(PROJ_K * CK + ks) * 64]), xf[ks], acc);
            }
            kfrag0 = as_uint4(pack8(acc, 0));
            kfrag1 = as_uint4(pack8(acc, 8));
            acc = zero16();
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                acc = mfma(xf[ks], as_bf16x8(wsrc[(PROJ_V * CK + ks) * 64]), acc);
            }
            vfrag0 = as_uint4(pack8(acc, 0));
            vfrag1 = as_uint4(pack8(acc, 8));
            acc = zero16();
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                acc = mfma(as_bf16x8(wsrc[(PROJ_Q * CK + ks) * 64]), xf[ks], acc);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[v] *= qmul;
            }
            q0 = pack8(acc, 0);
            q1 = pack8(acc, 8);
            // the gate's accumulator starts at its bias (register v of a lane holds feature 8 (v / 4) + 4 g + v % 4)
            const float *bgp = p.bg + h * HEAD + 4 * g_x;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 bv = *reinterpret_cast<const f32x4 *>(bgp + 8 * a);
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    acc[4 * a + c] = bv[c];
                }
            }
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                acc = mfma(as_bf16x8(wsrc[(PROJ_G * CK + ks) * 64]), xf[ks], acc);
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[v] = sigmoid_fast(acc[v]);
            }
            gate_park_x[0] = as_uint4(pack8(acc, 0));
            gate_park_x[64] = as_uint4(pack8(acc, 8));
        }
        __syncthreads(); // every wave is done with the previous row's attention: the K and V arrays are free
        lds_k[(j * 2 + 0) * 64 + lane] = kfrag0;
        lds_k[(j * 2 + 1) * 64 + lane] = kfrag1;
        lds_v[(j * 2 + 0) * 64 + lane] = vfrag0;
        lds_v[(j * 2 + 1) * 64 + lane] = vfrag1;
        if (tid == 0) {
            flag_words[(n + 1) & 1] = 0; // its readers (previous row) are done, its writers (next row) start after the next barrier
        }
        __syncthreads(); // K, V and the mask of this batch row are complete

        const f32x4 *mask4 = reinterpret_cast<const f32x4 *>(mask + 16 * g);
        f32x16 o;
        float l;
        const uint32_t flags = *flag_word;
        const bf16_t *nb_head = HAS_NB ? p.nb + (int64_t)h * p.nb_sh : nullptr;
        if constexpr (L2MODE) {
            const uint4 *nbf = HAS_NB ? p.nbf + ((int64_t)(h * NB + j) * NT * 2) * 64 + lane : nullptr;
            if (flags == 0u) {
                attend_block_l2<HAS_NB, false, false>(lds_k, lds_v, mask4, nbf, q0, q1, sel0, sel1, sumsel, NT, lane, 0.f, o,
                                                      l, -1, fair_turn);
            } else {
                attend_block_l2<HAS_NB, true, false>(lds_k, lds_v, mask4, nbf, q0, q1, sel0, sel1, sumsel, NT, lane, 0.f, o,
                                                     l, -1, fair_turn);
            }
            const bool ok = !__any(!(l > 1e-30f && l < 1e30f));
            if (!ok) {
                // some probability overflowed or a whole row underflowed: shift by the true row maxima
                const float m = row_max_l2<HAS_NB>(lds_k, mask4, nbf, q0, q1, sel0, sel1, NT, lane);
                attend_block_l2<HAS_NB, true, true>(lds_k, lds_v, mask4, nbf, q0, q1, sel0, sel1, sumsel, NT, lane, m, o, l);
            }
        } else {
            attend_block<HAS_NB>(lds_k, lds_v, mask4, flags, nb_head, p.nb_sq, j * 32, p.nb_vec != 0, panel, q0, q1, sel0,
                                 sel1, NB, S, lane, o, l);
        }
        int lane_o = lane; // as above: the addresses of the epilogue are not worth a register during the attention loop
        asm volatile("" : "+v"(lane_o));
        const int qpos = j * 32 + pi_row(lane_o & 31);
        if (qpos < S) {
            const uint4 *gate_park_o = gate_park_base + lane_o;
            const bf16x8 gate0 = as_bf16x8(gate_park_o[0]), gate1 = as_bf16x8(gate_park_o[64]);
            f32x16 gv;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                gv[v] = to_f32(gate0[v]);
                gv[8 + v] = to_f32(gate1[v]);
            }
            store_gated(p.avg + (int64_t)b * p.avg_sb + (int64_t)qpos * p.avg_ss + (int64_t)h * p.avg_sh + 4 * (lane_o >> 5), o,
                        __builtin_amdgcn_rcpf(l), gv);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// persistent_pair_kernel: persistent_head_kernel walking its batch rows two at a time (128 or 256 channels, log2 units).
// The pair bias of a (head, query block, key tile) is the same for every batch row, so a wave that attends the same query
// block of two rows at once fetches it once -- as fp32, in accumulator order, straight into the C operand of the logits
// MFMAs of both rows (pair_bias_tiles_kernel writes that copy).  Per row and key tile this moves the same bytes as the
// fp16 fragments of persistent_head_kernel and takes the two selector MFMAs out of the loop (matrix pipe 224 -> 160 clocks
// per tile); the two rows' instruction streams are independent, which gives the scheduler what a fourth wave per SIMD
// would; and every weight fragment read from LDS in the projection phase serves two rows.
// LDS, 16-byte units: W[4][CK][64]  K[2 rows][NT][2][64]  V[2 rows][NT][2][64]  panel[NB waves][128];
// then mask words mask[2 pairs in flight][2 rows][NT*32] (a key's mask bias as two bf16: the rows' masks enter the logits
// by one more MFMA per tile, see stage_mask_words) and four uint32 of tile flags.  At 128 channels and 384 positions that
// is 32 + 96 + 24 + 6 KB, at 256 channels and 256 positions 64 + 64 + 16 + 4 KB: the panels are half the size of
// persistent_head_kernel's (32 rows x 32 channels); during the attention a wave's panel holds the sigmoid of the first
// row's gate, the second row's waits in eight registers.
// ------------------------------------------------------------------------------------------------

// Wave-private 2 KB staging panel: 32 rows x 64 bytes in 16-byte slots, filled with two coalesced loads (lane l -> row
// l / 4 + 16 i, chunk l % 4) and read back in MFMA fragment order; the chunk index is XOR-swizzled by row so that both
// access patterns are free of LDS bank conflicts.
__device__ __forceinline__ int panel32_slot(int row, int chunk) { return row * 4 + (chunk ^ (((row >> 2) & 1) | (((row >> 4) & 1) << 1))); }

struct Panel32Regs {
    uint4 r0, r1;
};

// rows row0 .. row0 + 31 (clamped to last_row) of a row-major bf16 matrix, 32 columns from col0; 32-bit byte offsets from
// a wave-uniform base as in panel_load_near
__device__ __forceinline__ Panel32Regs panel32_load_near(const bf16_t *base, uint32_t ld, int row0, int last_row, int col0, int lane)
{
    const char *bytes = reinterpret_cast<const char *>(base);
    const uint32_t pitch = 2u * ld;
    const uint32_t col = 2u * (uint32_t)col0 + 16u * (uint32_t)(lane & 3);
    const uint32_t last = (uint32_t)last_row * pitch + col;
    const uint32_t first = __umul24((uint32_t)(row0 + (lane >> 2)), pitch) + col;
    Panel32Regs p;
    p.r0 = *reinterpret_cast<const uint4 *>(bytes + min(first, last));
    p.r1 = *reinterpret_cast<const uint4 *>(bytes + min(first + 16u * pitch, last));
    return p;
}

__device__ __forceinline__ void panel32_store(uint4 *panel, int lane, const Panel32Regs &p)
{
    const int row = lane >> 2, chunk = lane & 3;
    panel[panel32_slot(row, chunk)] = p.r0;
    panel[panel32_slot(row + 16, chunk)] = p.r1;
}

// Pair bias [H, S, S] -> fp32 tiles in accumulator order, in log2 units: for head h, query block j and key tile t,
// [h][j][t][4][64 lanes] x 16 bytes; lane (r, g) holds keys 32 t + 16 g .. + 15 of query 32 j + pi(r), four per 16-byte
// piece -- registers 4 a .. 4 a + 3 of the logits accumulator.  Queries past S repeat row S - 1, keys past S read as zero
// (their mask bias is -inf); -inf entries become the most negative finite value so that a row of them still has a
// finite maximum.
__global__ __launch_bounds__(64) void pair_bias_tiles_kernel(const bf16_t *__restrict__ nb, int64_t nb_sh, int64_t nb_sq, int S,
                                                             int NB, int NT, int vec, f32x4 *__restrict__ out)
{
    const int lane = threadIdx.x;
    const int r = lane & 31, g = lane >> 5;
    const int t = blockIdx.x % NT, j = blockIdx.x / NT, h = blockIdx.y;
    int q = 32 * j + pi_row(r);
    q = q < S ? q : S - 1;
    const int key0 = 32 * t + 16 * g;
    const bf16_t *src = nb + (int64_t)h * nb_sh + (int64_t)q * nb_sq + key0;
    float v[16];
    if (vec && key0 + 16 <= S) {
        const bf16x8 s0 = as_bf16x8(*reinterpret_cast<const uint4 *>(src)), s1 = as_bf16x8(*reinterpret_cast<const uint4 *>(src + 8));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[e] = to_f32(s0[e]), v[8 + e] = to_f32(s1[e]);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            v[e] = key0 + e < S ? to_f32(src[e]) : 0.f;
        }
    }
    f32x4 *dst = out + ((((int64_t)h * NB + j) * NT + t) * 4) * 64 + lane;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        f32x4 o;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const float x = v[4 * a + c] * LOG2E;
            o[c] = x < -3.0e38f ? -3.0e38f : x; // a comparison, not a max: a NaN stays a NaN
        }
        dst[a * 64] = o;
    }
}

// Attention of one 32-query block of two batch rows A and B (same head) in log2 units; see attend_block_l2 for the
// formulation.  Tiles are walked A(0) B(0) A(1) B(1) ...: while the softmax and P.V of one (row, tile) run on the vector
// ALU, the logits MFMAs of the next one are in the matrix pipe.
//   lds_kA/vA/kB/vB : K and V fragments of the two rows, [tile][kstep][lane]
//   mwA / mwB       : mask bias of the rows (log2 units) as hi/lo bf16 words (stage_mask_words), offset by the key the
//                     lane's accumulator row stands for; one more MFMA per tile adds them (WITH_MASK only)
//   nbc             : fp32 pair-bias tiles of this head and query block, offset by the lane: tile t, piece a at
//                     nbc[(4 t + a) * 64]; nullptr without a pair bias
//   MFMA_SUMS       : the row sums on the matrix pipe (one 16x16x32 MFMA per 16 keys and row) instead of four dot products
//                     on the vector ALU; costs ten more registers, which the 256-channel kernel (two waves per SIMD) has
template <bool HAS_NB, bool WITH_MASK, bool MFMA_SUMS>
__device__ __forceinline__ void attend_pair_l2(const uint4 *lds_kA, const uint4 *lds_vA, const uint4 *lds_kB, const uint4 *lds_vB,
                                               const uint32_t *mwA, const uint32_t *mwB, const f32x4 *nbc, bf16x8 qA0, bf16x8 qA1,
                                               bf16x8 qB0, bf16x8 qB1, int NB, int lane, f32x16 &oA_out,
                                               float &lA_out, f32x16 &oB_out, float &lB_out, int turn)
{
    const int npairs = NB >> 1;
    // The mask of a row as a rank-one MFMA: A holds (hi, lo) of the key of accumulator row i in k-slots 0 and 1, B holds
    // ones there, everything else is zero -- in the lanes of the upper half (k-slots 8..15) both operands are all zero,
    // so that an infinite mask value never meets a zero.
    const uint32_t lower = lane < 32 ? 0xffffffffu : 0u;
    uint4 ones4 = {0x3f803f80u & lower, 0u, 0u, 0u};
    const bf16x8 onesf = as_bf16x8(ones4);
    auto mask_fragment = [&](const uint32_t *mw, int t) {
        uint4 u = {0u, 0u, 0u, 0u};
        if constexpr (WITH_MASK) {
            u.x = mw[32 * t] & lower;
        }
        return as_bf16x8(u);
    };
    const uint4 *kA = lds_kA + lane, *vA = lds_vA + lane, *kB = lds_kB + lane, *vB = lds_vB + lane;
    auto clampt = [&](int t) { return t < NB ? t : NB - 1; };
    auto loadC = [&](int t) {
        f32x16 c;
        if constexpr (HAS_NB) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const f32x4 v = nbc[(t * 4 + a) * 64];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    c[4 * a + e] = v[e];
                }
            }
        } else {
            c = zero16();
        }
        return c;
    };
    f32x16 C0 = loadC(0), C1 = loadC(1);
    uint4 k0 = kA[0], k1 = kA[64], v0, v1;
    f32x16 xa, xb;
    xa = mfma(as_bf16x8(k0), qA0, C0);
    xa = mfma(as_bf16x8(k1), qA1, xa);
    if constexpr (WITH_MASK) {
        xa = mfma(mask_fragment(mwA, 0), onesf, xa);
    }
    k0 = kB[0], k1 = kB[64];
    v0 = vA[0], v1 = vA[64];
    f32x16 oA = zero16(), oB = zero16();
    float lsumA = 0.f, lsumB = 0.f; // this lane's share of the row sums; the two halves of the wave are added at the end
    // MFMA_SUMS: as in attend_block_l2 -- rowsum_selector's A operand sums the keys of each query in a 16x16x32 product
    // fed with the probability fragment; the sums of queries n and n + 16 end up in lane n, registers 0 and 1
    f32x4 sumsA = {0.f, 0.f, 0.f, 0.f}, sumsB = {0.f, 0.f, 0.f, 0.f};
    const bf16x8 ones_rows = rowsum_selector(lane);
    bf16x2 one2;
    one2[0] = (bf16_t)1.0f, one2[1] = (bf16_t)1.0f;
    // Probabilities -> bf16 by truncation: one byte permute per pair of values where the rounding conversion is a slower
    // instruction.  The row sums are taken over the same truncated values, so the bias (2^-9 on average) cancels in the
    // normalisation and what is left is a rounding error of up to 2^-8 per probability instead of 2^-9.
    auto pack_trunc = [&](const f32x16 &x, int base) {
        uint4 u;
        u.x = __builtin_amdgcn_perm(__float_as_uint(x[base + 1]), __float_as_uint(x[base + 0]), 0x07060302u);
        u.y = __builtin_amdgcn_perm(__float_as_uint(x[base + 3]), __float_as_uint(x[base + 2]), 0x07060302u);
        u.z = __builtin_amdgcn_perm(__float_as_uint(x[base + 5]), __float_as_uint(x[base + 4]), 0x07060302u);
        u.w = __builtin_amdgcn_perm(__float_as_uint(x[base + 7]), __float_as_uint(x[base + 6]), 0x07060302u);
        return as_bf16x8(u);
    };
    // row sums on the vector ALU, two probabilities per dot2: with two rows in flight the row-sum MFMAs of
    // attend_block_l2 (a selector fragment and an accumulator per row) cost more registers than the loop has
    auto rowsum = [&](float &lsum, f32x4 &sums, bf16x8 pv) {
        if constexpr (MFMA_SUMS) {
            sums = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones_rows, pv, sums, 0, 0, 0);
            return;
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bf16x2 a;
            a[0] = pv[2 * v], a[1] = pv[2 * v + 1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(a, one2, lsum, false);
        }
    };
    auto fence = [] { __builtin_amdgcn_sched_barrier(0); };
    auto exp4 = [&](f32x16 &x, int base) {
#pragma unroll
        for (int v = base; v < base + 4; ++v) {
            x[v] = __builtin_amdgcn_exp2f(x[v]);
        }
    };
    // softmax and P.V of the finished tile xc (into o, lacc); logits of the next tile into xn from seed C with query
    // fragments q0, q1; then k0, k1 <- knext[0], knext[64].  No scheduling fences inside: with two independent rows in
    // flight the compiler's own interleaving measured faster than a fixed one.  The empty asm keeps C live past the MFMA
    // that reads it: the compiler then writes xn to registers of its own (D != C) instead of computing it in place in
    // C's registers, which rotated the roles of the register blocks from one iteration to the next and cost 40 copies
    // per iteration, behind a wait for every load in flight.
    auto half_step = [&](f32x16 &xc, f32x16 &xn, const f32x16 &C, bf16x8 q0, bf16x8 q1, f32x16 &o, float &lsum, f32x4 &sums,
                         const uint4 *knext, const uint32_t *mw_next, int t_next) {
        bf16x8 p0, p1;
        const bf16x8 mnext = mask_fragment(mw_next, t_next); // requested first, used by the last MFMA of the step
        exp4(xc, 0);
        exp4(xc, 4);
        p0 = pack_trunc(xc, 0);
        xn = mfma(as_bf16x8(k0), q0, C);
        asm volatile("" ::"v"(C));
        o = mfma(as_bf16x8(v0), p0, o);
        exp4(xc, 8);
        xn = mfma(as_bf16x8(k1), q1, xn);
        if constexpr (WITH_MASK) {
            xn = mfma(mnext, onesf, xn);
        }
        rowsum(lsum, sums, p0);
        k0 = knext[0], k1 = knext[64];
        exp4(xc, 12);
        p1 = pack_trunc(xc, 8);
        o = mfma(as_bf16x8(v1), p1, o);
        rowsum(lsum, sums, p1);
    };
    for (int pair = 0; pair < npairs; ++pair) {
        if (turn >= 0) {
            timeslice_priority((uint32_t)turn, FAIR_SLICE_SHIFT);
        }
        const int t0 = 2 * pair, t1 = t0 + 1;
        const int tn = pair + 1 < npairs ? t0 + 2 : t0; // next pair's first tile, clamped
        // (A, t0) finished; logits of (B, t0) from C0
        half_step(xa, xb, C0, qB0, qB1, oA, lsumA, sumsA, kA + t1 * 128, mwB, t0);
        v0 = vB[t0 * 128], v1 = vB[t0 * 128 + 64];
        fence(); // the loads stay behind the last reader of the registers they fill
        C0 = loadC(clampt(t0 + 2));
        fence();
        // (B, t0) finished; logits of (A, t1) from C1
        half_step(xb, xa, C1, qA0, qA1, oB, lsumB, sumsB, kB + t1 * 128, mwA, t1);
        v0 = vA[t1 * 128], v1 = vA[t1 * 128 + 64];
        // (A, t1) finished; logits of (B, t1) from C1
        half_step(xa, xb, C1, qB0, qB1, oA, lsumA, sumsA, kA + tn * 128, mwB, t1);
        v0 = vB[t1 * 128], v1 = vB[t1 * 128 + 64];
        fence();
        C1 = loadC(clampt(t1 + 2));
        fence();
        // (B, t1) finished; logits of (A, tn) from C0
        half_step(xb, xa, C0, qA0, qA1, oB, lsumB, sumsB, kB + tn * 128, mwA, tn);
        v0 = vA[tn * 128], v1 = vA[tn * 128 + 64];
    }
    __builtin_amdgcn_s_setprio(0);
    oA_out = oA, oB_out = oB;
    if constexpr (MFMA_SUMS) {
        lA_out = rowsum_fetch(sumsA, lane), lB_out = rowsum_fetch(sumsB, lane);
    } else {
        lA_out = half_swap_sum(lsumA), lB_out = half_swap_sum(lsumB);
    }
}

// The repeat of one row's block after an overflow or underflow of the unshifted exponentials, with the pair bias as fp32
// tiles: a first pass over the key tiles for the true row maxima, a second one with them subtracted.  Not a hot path:
// one row, nothing prefetched, few registers.
template <bool HAS_NB>
__device__ __forceinline__ void attend_row_shifted(const uint4 *lds_k, const uint4 *lds_v, const uint32_t *words, const f32x4 *nbc, bf16x8 q0,
                                                bf16x8 q1, int NB, int lane, f32x16 &o_out, float &l_out)
{
    // words: the row's mask words (stage_mask_words), offset by 16 (lane >> 5): register 4 a + c stands for key 4 a + c of them
    auto logits = [&](int t) {
        f32x16 x;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const uint4 w4 = *reinterpret_cast<const uint4 *>(words + 32 * t + 4 * a);
            f32x4 mv = {mask_word_value(w4.x), mask_word_value(w4.y), mask_word_value(w4.z), mask_word_value(w4.w)};
            if constexpr (HAS_NB) {
                const f32x4 cv = nbc[(t * 4 + a) * 64];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    mv[c] += cv[c];
                }
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                x[4 * a + c] = mv[c];
            }
        }
        x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), q0, x);
        return mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), q1, x);
    };
    float mx = -INFINITY;
    for (int t = 0; t < NB; ++t) {
        const f32x16 x = logits(t);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            mx = fmaxf(mx, x[v]);
        }
    }
    mx = half_swap_max(mx); // finite: a fully masked row has -1e9*log2(e) everywhere
    f32x16 o = zero16();
    float lsum = 0.f;
    bf16x2 one2;
    one2[0] = (bf16_t)1.0f, one2[1] = (bf16_t)1.0f;
    for (int t = 0; t < NB; ++t) {
        f32x16 x = logits(t);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            x[v] = __builtin_amdgcn_exp2f(x[v] - mx);
        }
        const bf16x8 p0 = pack8(x, 0), p1 = pack8(x, 8);
        o = mfma(as_bf16x8(lds_v[(t * 2 + 0) * 64 + lane]), p0, o);
        o = mfma(as_bf16x8(lds_v[(t * 2 + 1) * 64 + lane]), p1, o);
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            bf16x2 a, c;
            a[0] = p0[2 * v], a[1] = p0[2 * v + 1];
            c[0] = p1[2 * v], c[1] = p1[2 * v + 1];
            lsum = __builtin_amdgcn_fdot2_f32_bf16(a, one2, lsum, false);
            lsum = __builtin_amdgcn_fdot2_f32_bf16(c, one2, lsum, false);
        }
    }
    o_out = o;
    l_out = half_swap_sum(lsum);
}

template <int C, bool HAS_NB>
__global__ __launch_bounds__(64 * max_waves(C, 1)) void persistent_pair_kernel(FusedParams p)
{
    constexpr int CK = C / 16;
    // the row sums on the matrix pipe where the registers are there: with 256 channels (two waves per SIMD) always, with
    // 128 (three) in the loop without mask products only -- the masked loop spills with them
    constexpr bool PAIR_MFMA_SUMS = C == 256;
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int S = p.S, NB = p.NB, NT = p.NT;
    const int nthreads = NB * 64;

    // workgroup -> (XCD, head, batch-row group) as in persistent_head_kernel
    const int w = blockIdx.x;
    const int xcd = w & 7;
    const int slot = w >> 3;
    const int h = slot % p.H;
    const int grp = slot / p.H;
    const int b0 = xcd + 8 * grp;
    const int bstep = 8 * p.ngrp;
    const int nrows = b0 < p.B ? (p.B - b0 + bstep - 1) / bstep : 0;

    uint4 *lds_w = lds;
    uint4 *lds_k = lds_w + 4 * CK * 64;     // [row of the pair][NT][2][64]
    uint4 *lds_v = lds_k + 2 * NT * 2 * 64; // likewise
    uint4 *panel = lds_v + 2 * NT * 2 * 64 + wave * 128;
    uint32_t *mask_base = reinterpret_cast<uint32_t *>(lds_v + 2 * NT * 2 * 64 + NB * 128); // [pair parity][row of the pair][NT*32] mask words
    uint32_t *flag_words = mask_base + 4 * NT * 32;                                         // [pair parity][row of the pair]

    stage_weight_fragments<C>(lds_w, p, 0, 4, h, wave, nthreads >> 6, lane);
    if (tid < 4) {
        flag_words[tid] = 0;
    }
    if (NT > NB) { // phantom key tile of both rows: zero K and V fragments, never written again
        const uint4 z4 = {0u, 0u, 0u, 0u};
        for (int idx = tid; idx < 256; idx += nthreads) {
            const int row = idx >> 7, i = idx & 127;
            lds_k[(row * NT + NB) * 128 + i] = z4;
            lds_v[(row * NT + NB) * 128 + i] = z4;
        }
    }
    __syncthreads();

    const int j = wave; // this wave's sequence block
    const int fair_turn = C == 128 ? wave >> 2 : -1; // time-sliced priorities pay with three waves per SIMD only
    const float qmul = p.qscale * LOG2E;
    const uint32_t x_pitch = (uint32_t)p.x_ld; // the host sends only near-addressable rows here
    for (int n = 0; n < nrows; n += 2) {
        const int par = (n >> 1) & 1;
        const bool have_b = n + 1 < nrows; // an odd row count: the last pair attends its one row twice and stores it once
        const int bA = b0 + n * bstep, bB = have_b ? bA + bstep : bA;
        uint32_t *flag_word = flag_words + 2 * par;
        uint32_t *mask = mask_base + par * 2 * NT * 32;
        // opaque lane index: addresses derived from it are formed anew per pair instead of living across the attention loop
        int lane_x = lane;
        asm volatile("" : "+v"(lane_x));
        stage_mask_words<true>(p.bias + (int64_t)bA * p.bias_sb, mask, flag_word, S, NT, wave, lane_x, LOG2E, p.bias_sk,
                               p.bias_is_mask != 0);
        stage_mask_words<true>(p.bias + (int64_t)bB * p.bias_sb, mask + NT * 32, flag_word + 1, S, NT, wave, lane_x, LOG2E, p.bias_sk,
                               p.bias_is_mask != 0);

        // ---- input rows of the block, both batch rows -> fragments, 32 channels per staging panel ----
        const int prow_x = pi_row(lane_x & 31), g_x = lane_x >> 5;
        const bf16_t *xA = p.x + (int64_t)bA * p.x_sb, *xB = p.x + (int64_t)bB * p.x_sb;
        bf16x8 xfA[CK], xfB[CK];
#pragma unroll
        for (int q = 0; q < C / 128; ++q) { // 128 channels of both rows at a time
            Panel32Regs ta[4], tb[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                ta[c] = panel32_load_near(xA, x_pitch, j * 32, S - 1, 128 * q + 32 * c, lane_x);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                tb[c] = panel32_load_near(xB, x_pitch, j * 32, S - 1, 128 * q + 32 * c, lane_x);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                panel32_store(panel, lane_x, ta[c]);
                xfA[8 * q + 2 * c] = as_bf16x8(panel[panel32_slot(prow_x, g_x)]);
                xfA[8 * q + 2 * c + 1] = as_bf16x8(panel[panel32_slot(prow_x, 2 + g_x)]);
            }
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                panel32_store(panel, lane_x, tb[c]);
                xfB[8 * q + 2 * c] = as_bf16x8(panel[panel32_slot(prow_x, g_x)]);
                xfB[8 * q + 2 * c + 1] = as_bf16x8(panel[panel32_slot(prow_x, 2 + g_x)]);
            }
        }
        // ---- four projections of the block, both rows per weight fragment ----
        // Gate first, then Q, K, V, each packed to bf16 as soon as it is complete;
        // the scheduling barriers keep the compiler from running the four loops into one another, which needs four
        // pairs of accumulators at once and spilled the input fragments.
        bf16x8 qA0, qA1, qB0, qB1;
        bf16x8 gateB0, gateB1;                                  // sigmoid(gate) of the second row, until the epilogue
        bf16x8 kfA0, kfA1, vfA0, vfA1, kfB0, kfB1, vfB0, vfB1; // parked until the LDS arrays are free
        {
            const uint4 *wsrc = lds_w + lane_x;
            auto project = [&](int proj, f32x16 &accA, f32x16 &accB, bool weights_left) {
#pragma unroll
                for (int ks = 0; ks < CK; ++ks) {
                    const bf16x8 wf = as_bf16x8(wsrc[(proj * CK + ks) * 64]);
                    if (weights_left) {
                        accA = mfma(wf, xfA[ks], accA);
                        accB = mfma(wf, xfB[ks], accB);
                    } else {
                        accA = mfma(xfA[ks], wf, accA);
                        accB = mfma(xfB[ks], wf, accB);
                    }
                }
            };
            __builtin_amdgcn_sched_barrier(0);
            {
                // the gate's accumulator starts at its bias (register v of a lane holds feature 8 (v / 4) + 4 g + v % 4)
                f32x16 accA, accB;
                const float *bgp = p.bg + h * HEAD + 4 * g_x;
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(bgp + 8 * a);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        accA[4 * a + c] = bv[c], accB[4 * a + c] = bv[c];
                    }
                }
                project(PROJ_G, accA, accB, true);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    accA[v] = sigmoid_fast(accA[v]), accB[v] = sigmoid_fast(accB[v]);
                }
                // the first row's into the wave's panel (its input rows are all staged), the second row's stay in registers
                panel[lane_x] = as_uint4(pack8(accA, 0));
                panel[64 + lane_x] = as_uint4(pack8(accA, 8));
                gateB0 = pack8(accB, 0), gateB1 = pack8(accB, 8);
                asm volatile("" : "+v"(gateB0), "+v"(gateB1));
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                f32x16 accA = zero16(), accB = zero16();
                project(PROJ_Q, accA, accB, true);
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    accA[v] *= qmul, accB[v] *= qmul;
                }
                qA0 = pack8(accA, 0), qA1 = pack8(accA, 8);
                qB0 = pack8(accB, 0), qB1 = pack8(accB, 8);
                asm volatile("" : "+v"(qA0), "+v"(qA1), "+v"(qB0), "+v"(qB1)); // packed here, not after the barrier
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                f32x16 accA = zero16(), accB = zero16();
                project(PROJ_K, accA, accB, true);
                kfA0 = pack8(accA, 0), kfA1 = pack8(accA, 8);
                kfB0 = pack8(accB, 0), kfB1 = pack8(accB, 8);
                asm volatile("" : "+v"(kfA0), "+v"(kfA1), "+v"(kfB0), "+v"(kfB1));
            }
            __builtin_amdgcn_sched_barrier(0);
            {
                f32x16 accA = zero16(), accB = zero16();
                project(PROJ_V, accA, accB, false);
                vfA0 = pack8(accA, 0), vfA1 = pack8(accA, 8);
                vfB0 = pack8(accB, 0), vfB1 = pack8(accB, 8);
                asm volatile("" : "+v"(vfA0), "+v"(vfA1), "+v"(vfB0), "+v"(vfB1));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads(); // every wave is done with the previous pair's attention: the K and V arrays are free
        {
            uint4 *ka = lds_k + (j * 2) * 64 + lane, *va = lds_v + (j * 2) * 64 + lane;
            ka[0] = as_uint4(kfA0), ka[64] = as_uint4(kfA1), va[0] = as_uint4(vfA0), va[64] = as_uint4(vfA1);
            ka[NT * 128] = as_uint4(kfB0), ka[NT * 128 + 64] = as_uint4(kfB1);
            va[NT * 128] = as_uint4(vfB0), va[NT * 128 + 64] = as_uint4(vfB1);
        }
        if (tid < 2) {
            flag_words[2 * (par ^ 1) + tid] = 0; // its readers (previous pair) are done, its writers (next pair) start after the next barrier
        }
        __syncthreads(); // K, V and the masks of this pair are complete

        // opaque once more: the loops' LDS and pair-bias addresses are formed here, per pair,
        // rather than hoisted out of the pair loop and spilled
        int lane_a = lane;
        asm volatile("" : "+v"(lane_a));
        const int g = lane_a >> 5;
        const uint32_t *mwA = mask + pi_row(lane_a & 31), *mwB = mwA + NT * 32; // accumulator row i of a tile is its key pi(i)
        const uint32_t flagsA = flag_word[0], flagsB = flag_word[1];
        const f32x4 *nbc = HAS_NB ? reinterpret_cast<const f32x4 *>(p.nbf) + ((int64_t)(h * NB + j) * NT * 4) * 64 + lane_a : nullptr;
        const uint4 *kA = lds_k, *vA = lds_v, *kB = lds_k + NT * 128, *vB = lds_v + NT * 128;
        f32x16 oA, oB;
        float lA, lB;
        if ((flagsA | flagsB) == 0u) {
            attend_pair_l2<HAS_NB, false, true>(kA, vA, kB, vB, mwA, mwB, nbc, qA0, qA1, qB0, qB1, NT, lane_a, oA, lA, oB, lB, fair_turn);
        } else {
            attend_pair_l2<HAS_NB, true, PAIR_MFMA_SUMS>(kA, vA, kB, vB, mwA, mwB, nbc, qA0, qA1, qB0, qB1, NT, lane_a, oA, lA, oB, lB, fair_turn);
        }
        // some probability overflowed or a whole row underflowed: repeat that row shifted by its true row maxima
        if (__any(!(lA > 1e-30f && lA < 1e30f))) {
            attend_row_shifted<HAS_NB>(kA, vA, mask + 16 * g, nbc, qA0, qA1, NT, lane_a, oA, lA);
        }
        if (__any(!(lB > 1e-30f && lB < 1e30f))) {
            attend_row_shifted<HAS_NB>(kB, vB, mask + NT * 32 + 16 * g, nbc, qB0, qB1, NT, lane_a, oB, lB);
        }
        int lane_o = lane; // as above: the addresses of the epilogue are not worth a register during the attention loop
        asm volatile("" : "+v"(lane_o));
        const int qpos = j * 32 + pi_row(lane_o & 31);
        if (qpos < S) {
            const int64_t off = (int64_t)qpos * p.avg_ss + (int64_t)h * p.avg_sh + 4 * (lane_o >> 5);
            const bf16x8 gateA0 = as_bf16x8(panel[lane_o]), gateA1 = as_bf16x8(panel[64 + lane_o]);
            f32x16 gv;
#pragma unroll
            for (int v = 0; v < 8; ++v) {
                gv[v] = to_f32(gateA0[v]), gv[8 + v] = to_f32(gateA1[v]);
            }
            store_gated(p.avg + (int64_t)bA * p.avg_sb + off, oA, __builtin_amdgcn_rcpf(lA), gv);
            if (have_b) {
#pragma unroll
                for (int v = 0; v < 8; ++v) {
                    gv[v] = to_f32(gateB0[v]), gv[8 + v] = to_f32(gateB1[v]);
                }
                store_gated(p.avg + (int64_t)bB * p.avg_sb + off, oB, __builtin_amdgcn_rcpf(lB), gv);
            }
        }
    }
}

// out[t][o] = sum_c avg[t][c] * Wo[o][c] + bo[o]  (reference src/attention/gating_attention.cpp:152-157).
// HBM-bound: each row of avg is read once and each row of out written once, both as whole cache
// lines through the wave-private staging panel.  A workgroup stages the fragments of a 128-feature
// slab of Wo once and its four waves walk 32-row tiles.  The product is formed transposed
// (rows = output features, columns = tokens), which leaves every lane with 4 consecutive features
// of its own token per accumulator group -- an 8-byte panel write.
// EPILOGUE 1 (gated residual): the rounded result is not stored but folded into `out`, out += result * sigmoid(gate),
// with gate and out read in the order they are written, 16 bytes per lane -- the last two steps of the triangle
// multiplication (reference src/attention/triangle_multiplication.cpp:129-150) and the residual update fused into
// its output projection.  EPILOGUE 2 (residual): out += result, where row (i, j) of the result goes to row (j, i)
// of `out` when swap_n != 0 (rows are pairs (i, j) of an [M / swap_n, swap_n] grid): the residual update of a triangle-attention block,
// transposed back for the ending node.
constexpr int EPILOGUE_STORE = 0, EPILOGUE_GATED_RESIDUAL = 1, EPILOGUE_RESIDUAL = 2;

// With 256 input features a workgroup has eight waves and keeps two 128-feature slabs of Wo (128 KB, the whole matrix of
// the attention's output projection), so a row is read once for all 256 output features; with 128 it has four waves,
// one slab, and two workgroups share a CU.
// NEAR_OUT (residual epilogue only): fewer than 2^24 rows, less than 2^31 bytes of `out`, swap_n zero or at least 32 (the
// launcher checks): the rows of `out` are found with 32-bit arithmetic -- one division of a wave-uniform row index per
// 32-row step and an add, a compare and two 24-bit multiplies per row -- where 64-bit division and remainder per lane
// and row are some 300 quarter-rate instructions per step.
template <int C, int EPILOGUE, bool NEAR_OUT = false>
__global__ __launch_bounds__(C == 128 ? 256 : 512, C == 128 ? 2 : 1) void output_projection_kernel(
    const bf16_t *__restrict__ avg, int64_t avg_ld, const bf16_t *__restrict__ wo, const float *__restrict__ bo,
    bf16_t *__restrict__ out, int64_t out_ld, int64_t M, int N, int rows_per_wave, const bf16_t *__restrict__ gate,
    int64_t gate_ld, int64_t swap_n)
{
    // row of `out` that receives row `row` of the result
    auto target_row = [&](int64_t row) -> int64_t {
        if constexpr (EPILOGUE == EPILOGUE_RESIDUAL) {
            return swap_n ? (row % swap_n) * (M / swap_n) + row / swap_n : row; // row (b, s) of [M / n, n] -> (s, b)
        }
        return row;
    };
    constexpr int CK = C / 16;
    constexpr int NP = CK / 4;
    constexpr int SLABS = C / 128, WAVES = 4 * SLABS, THREADS = 64 * WAVES;
    extern __shared__ uint4 lds[]; // W slabs [SLABS][4 feature blocks][CK][64 lanes], then one panel of 256 per wave
    constexpr bool NEAR = C == 128; // 32-bit row offsets from a wave-uniform base; measured slower with 256 features
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = NEAR ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int nbase = blockIdx.y * (128 * SLABS);               // first output feature of this workgroup
    // slabs it has: with two per workgroup the last workgroup of a row of them may have one
    const int nslab = (SLABS == 1 || N - nbase >= 128 * SLABS) ? SLABS : (N - nbase) / 128;
    uint4 *panel = lds + SLABS * 4 * CK * 64 + wave * 256;
    // Every wave owns a contiguous range of rows_per_wave rows (a multiple of 8), walked 32 rows at a
    // time; the last step of a range may be partial.  Equal ranges rather than whole 32-row tiles dealt
    // round robin: the kernel is short, and a wave with one tile more than its neighbours would set its
    // duration.  The first two panels of a step are fetched while the previous step is multiplied and
    // stored; those of the first step while the weight slab is staged.
    const int64_t start = ((int64_t)blockIdx.x * WAVES + wave) * rows_per_wave;
    const int64_t stop = start + rows_per_wave < M ? start + rows_per_wave : M;
    // With 128 features rows are addressed relative to the wave's first one: 32-bit byte offsets from a wave-uniform
    // base (the host keeps a wave's range below 2^31 bytes), no 64-bit multiply per row.
    const int last_rel = (int)(stop - 1 - start);
    const bf16_t *avg_w = avg + start * avg_ld;
    auto load_panel = [&](int rel_row, int c, int ln) { // 32 rows from rel_row (relative to start), channels 64 c .. 64 c + 63
        if constexpr (NEAR) {
            return panel_load_near(avg_w + c * 64, (uint32_t)avg_ld, rel_row, last_rel, 0, ln);
        } else {
            return panel_load(avg, avg_ld, (int)start + rel_row, (int)(stop - 1), c * 64, ln);
        }
    };
    PanelRegs ta, tb;
    if (start < stop) {
        ta = load_panel(0, 0, lane);
        tb = load_panel(0, 1, lane);
    }
    {
        constexpr int PER = SLABS * 4 * CK * 64 / THREADS; // weight fragments per thread, all loads issued before the first store
        uint4 wreg[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + i * THREADS;
            int nb_ = idx / (CK * 64);
            nb_ = nb_ < 4 * nslab ? nb_ : 0; // a slab this workgroup does not have: any valid rows, never used
            const int ks = (idx >> 6) % CK;
            const int ln = idx & 63;
            wreg[i] = *reinterpret_cast<const uint4 *>(wo + (int64_t)(nbase + nb_ * 32 + (ln & 31)) * C + ks * 16 + (ln >> 5) * 8);
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            lds[tid + i * THREADS] = wreg[i];
        }
    }
    __syncthreads();
    for (int64_t rbase = start; rbase < stop; rbase += 32) {
        const int row0 = (int)rbase, rel0 = (int)(rbase - start);
        // With 256 input features the lane index is opaque to the optimiser, so that addresses and panel offsets are
        // formed per step instead of being kept (and partly spilled) across the loop.  With 128 the kernel fits either
        // way, and the smaller footprint would let a third workgroup onto some CUs of a grid sized for two.
        int lv = lane;
        if constexpr (C > 128) {
            asm volatile("" : "+v"(lv));
        }
        const int rv = lv & 31, gv = lv >> 5;
        bf16x8 af[CK];
        panel_store(panel, lv, ta);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            af[k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
        }
        panel_store(panel, lv, tb);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            af[4 + k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
        }
#pragma unroll
        for (int c = 2; c < NP; ++c) {
            ta = load_panel(rel0, c, lv);
            panel_store(panel, lv, ta);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                af[4 * c + k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
        }
        uint32_t out_off[4]; // NEAR_OUT: byte offsets of this lane's four rows of `out` (rows past the end: the last one)
        if constexpr (EPILOGUE == EPILOGUE_RESIDUAL && NEAR_OUT) {
            const uint32_t n32 = (uint32_t)swap_n, nb32 = n32 ? (uint32_t)M / n32 : 0u;
            const uint32_t first = (uint32_t)__builtin_amdgcn_readfirstlane(row0);
            const uint32_t b0 = n32 ? first / n32 : 0u, s0 = first - b0 * n32; // row (b0, s0) of the [M / n, n] grid
            const uint32_t last_rel = (uint32_t)(stop - 1 - rbase);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint32_t pr = 8u * i + ((uint32_t)lv >> 3);
                pr = pr < last_rel ? pr : last_rel;
                uint32_t target = first + pr;
                if (n32) { // (b, s) -> (s, b); the 32 rows of a step wrap at most once (n >= 32)
                    uint32_t sq = s0 + pr, bq = b0;
                    if (sq >= n32) {
                        sq -= n32, bq += 1;
                    }
                    target = __umul24(sq, nb32) + bq;
                }
                out_off[i] = __umul24(target, 2u * (uint32_t)out_ld) + 16u * ((uint32_t)lv & 7u);
            }
        }
        {
            // clamped to the last step instead of a branch: one harmless re-read at the end
            const int rnext = rbase + 32 < stop ? rel0 + 32 : rel0;
            ta = load_panel(rnext, 0, lv);
            tb = load_panel(rnext, 1, lv);
        }
#pragma unroll 1
        for (int slab = 0; slab < nslab; ++slab) {
        const int n0 = nbase + slab * 128;
        const uint4 *wslab = lds + slab * 4 * CK * 64;
        const float *bias = bo + n0 + 4 * gv; // read per use: 16 cached loads per tile instead of 64 live registers
#pragma unroll
        for (int half = 0; half < 2; ++half) { // 64 output features per panel
            uint4 gq[4], zq[4];
            if constexpr (EPILOGUE != EPILOGUE_STORE) { // requested before the MFMAs, used after them
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    int64_t row = (int64_t)row0 + 8 * i + (lv >> 3);
                    row = row < stop ? row : stop - 1;
                    const int64_t col = n0 + half * 64 + (lv & 7) * 8;
                    if constexpr (EPILOGUE == EPILOGUE_GATED_RESIDUAL) {
                        gq[i] = *reinterpret_cast<const uint4 *>(gate + row * gate_ld + col);
                    }
                    if constexpr (EPILOGUE == EPILOGUE_RESIDUAL && NEAR_OUT) {
                        zq[i] = *reinterpret_cast<const uint4 *>(reinterpret_cast<const char *>(out + n0 + half * 64) + out_off[i]);
                    } else {
                        zq[i] = *reinterpret_cast<const uint4 *>(out + target_row(row) * out_ld + col);
                    }
                }
            }
            f32x16 acc[2];
            acc[0] = zero16(), acc[1] = zero16();
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
#pragma unroll
                for (int n = 0; n < 2; ++n) {
                    acc[n] = mfma(as_bf16x8(wslab[((2 * half + n) * CK + ks) * 64 + lv]), af[ks], acc[n]);
                }
            }
            // accumulators -> panel as bf16 [row][64 features], then whole-line stores
#pragma unroll
            for (int n = 0; n < 2; ++n) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(bias + (2 * half + n) * 32 + 8 * a);
                    bf16x4 ov;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        ov[c] = (bf16_t)(acc[n][4 * a + c] + bv[c]);
                    }
                    bf16x4 *dst = reinterpret_cast<bf16x4 *>(panel + panel_slot(rv, n * 4 + a)) + gv;
                    *dst = ov;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int prow_ = 8 * i + (lv >> 3);
                uint4 v = panel[panel_slot(prow_, lv & 7)];
                const int64_t row = (int64_t)row0 + prow_;
                if constexpr (EPILOGUE == EPILOGUE_GATED_RESIDUAL) {
                    const bf16x8 o = as_bf16x8(v), gt = as_bf16x8(gq[i]), z = as_bf16x8(zq[i]);
                    bf16x8 res;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        // bf16(out * sigmoid(gate)) as the reference stores it, then the residual sum in fp32
                        const float upd = to_f32((bf16_t)(to_f32(o[e]) * sigmoid_fast(to_f32(gt[e]))));
                        res[e] = (bf16_t)(to_f32(z[e]) + upd);
                    }
                    v = as_uint4(res);
                } else if constexpr (EPILOGUE == EPILOGUE_RESIDUAL) {
                    const bf16x8 o = as_bf16x8(v), z = as_bf16x8(zq[i]);
                    bf16x8 res;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        res[e] = (bf16_t)(to_f32(z[e]) + to_f32(o[e]));
                    }
                    v = as_uint4(res);
                }
                if (row < stop) {
                    if constexpr (EPILOGUE == EPILOGUE_RESIDUAL && NEAR_OUT) {
                        *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(out + n0 + half * 64) + out_off[i]) = v;
                    } else if constexpr (EPILOGUE == EPILOGUE_RESIDUAL || !NEAR) {
                        *reinterpret_cast<uint4 *>(out + target_row(row) * out_ld + n0 + half * 64 + (lv & 7) * 8) = v;
                    } else {
                        char *out_w = reinterpret_cast<char *>(out + start * out_ld + n0 + half * 64);
                        *reinterpret_cast<uint4 *>(out_w + (__umul24((uint32_t)(rel0 + prow_), 2u * (uint32_t)out_ld) + 16u * (lv & 7))) = v;
                    }
                }
            }
        }
        } // slabs
    }
}

// out[t][:] += bf16( bf16(x[t] . Wo^T + bo) * sigmoid(bf16(y[t] . Wg^T + bg)) ) for rows of 128 features in and out: the last
// three steps of the triangle multiplication with the gate projection folded in (reference
// src/attention/triangle_multiplication.cpp:106-150: gate = Linear(normalised input), out = Linear(normalised centre),
// out * sigmoid(gate), residual).  The gate tensor never exists in memory: against the separate gate projection this
// saves its write, its read and a launch.  Same structure as output_projection_kernel: both weight slabs stay in LDS
// (64 KB), every wave streams an equal range of rows 32 at a time, rows in and out as whole cache lines through its
// panel, the next step's rows requested while the current one is multiplied.  The gate goes first: its accumulators,
// rounded to bf16 as the reference stores them, wait as 32 packed registers for the projection of the same rows.
//
// X_CHANNEL_FIRST: x is the centre of the triangle multiplication as the equation leaves it, channel-first ([128, M],
// channel stride x_ld) and not yet normalised.  The kernel then takes the place of the channel-first LayerNorm too: a
// wave loads 64 channels x 32 positions (64 contiguous bytes per channel), stores them in its panel as they lie, gets
// its MFMA fragments -- 8 consecutive channels of one position per lane -- with the LDS transposing read, and normalises
// them in registers (a position's 128 channels sit in two lanes; the arithmetic is that of the LayerNorm kernels,
// reference src/normalization/layernorm_kernel.h:21-53, the result rounded to bf16 as the tensor it replaces was).
template <bool X_CHANNEL_FIRST>
__global__ __launch_bounds__(256, 2) void projected_gate_residual_kernel(
    const bf16_t *__restrict__ x, int64_t x_ld, const bf16_t *__restrict__ wo, const float *__restrict__ bo,
    const bf16_t *__restrict__ y, int64_t y_ld, const bf16_t *__restrict__ wg, const float *__restrict__ bg,
    bf16_t *__restrict__ out, int64_t out_ld, int64_t M, int rows_per_wave, const float *__restrict__ ln_gamma,
    const float *__restrict__ ln_beta, float ln_eps)
{
    constexpr int C = 128, CK = C / 16;
    extern __shared__ uint4 lds[]; // [Wo, Wg][4 feature blocks][CK][64 lanes], then 4 panels of 256
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform
    uint4 *panel = lds + 2 * 4 * CK * 64 + wave * 256;
    // The workgroup owns 4 * rows_per_wave consecutive rows and its waves take the 32-row steps of that range in turn
    // (wave w: steps w, w + 4, ...): neighbouring steps run at the same time, so the two 64-byte halves of a 128-byte
    // line of the channel-first tensor (32 positions each) are asked for together instead of a whole step apart, by
    // which time the line has left the L2.
    // Rows are addressed relative to the workgroup's first one, by 32-bit byte offsets from uniform bases; positions of
    // the channel-first tensor by 32-bit offsets from its first element (the launcher checks that both fit).
    const int64_t start = (int64_t)blockIdx.x * 4 * rows_per_wave;
    const int64_t stop = start + 4 * rows_per_wave < M ? start + 4 * rows_per_wave : M;
    const int64_t first = start + 32 * wave; // this wave's first step
    const int last_rel = (int)(stop - 1 - start);
    const bf16_t *y_w = y + start * y_ld, *x_w = x + start * x_ld;
    const uint32_t y_pitch = (uint32_t)y_ld, x_pitch = (uint32_t)x_ld, m32 = (uint32_t)M;
    // the first 64 features of the next step's rows of y and x are requested a step ahead; the second 64 at the top of
    // their own step, behind the first (four sets of registers held across a step do not fit)
    // channel-first x: 64 channels (from c0) x 32 positions (from p0), lane -> channel c0 + 16 i + lane / 4, positions
    // p0 + 8 (lane & 3) .. +7; a chunk past the end of the tensor repeats the last one (M is a multiple of 8)
    auto load_cf = [&](int c0, int64_t p0, int ln) {
        uint32_t pos = (uint32_t)p0 + 8u * (ln & 3);
        pos = pos + 8u <= m32 ? pos : m32 - 8u;
        PanelRegs t;
        const char *src = reinterpret_cast<const char *>(x + (int64_t)c0 * x_ld);
        const uint32_t off = 2u * (__umul24((uint32_t)(ln >> 2), x_pitch) + pos), step = 32u * x_pitch; // 16 channels on
        t.r0 = *reinterpret_cast<const uint4 *>(src + off);
        t.r1 = *reinterpret_cast<const uint4 *>(src + (off + step));
        t.r2 = *reinterpret_cast<const uint4 *>(src + (off + 2u * step));
        t.r3 = *reinterpret_cast<const uint4 *>(src + (off + 3u * step));
        return t;
    };
    PanelRegs ya, xa;
    if (first < stop) {
        ya = panel_load_near(y_w, y_pitch, 32 * wave, last_rel, 0, lane);
        if constexpr (X_CHANNEL_FIRST) {
            xa = load_cf(0, first, lane);
        } else {
            xa = panel_load_near(x_w, x_pitch, 32 * wave, last_rel, 0, lane);
        }
    }
    {
        constexpr int PER = 2 * 4 * CK * 64 / 256;
        uint4 wreg[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + i * 256;
            const int mat = idx / (4 * CK * 64), nb_ = (idx / (CK * 64)) % 4, ks = (idx >> 6) % CK, ln = idx & 63;
            const bf16_t *w = mat ? wg : wo;
            wreg[i] = *reinterpret_cast<const uint4 *>(w + (int64_t)(nb_ * 32 + (ln & 31)) * C + ks * 16 + (ln >> 5) * 8);
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            lds[tid + i * 256] = wreg[i];
        }
    }
    __syncthreads();
    const uint4 *wo_s = lds, *wg_s = lds + 4 * CK * 64;
    for (int64_t rbase = first; rbase < stop; rbase += 128) {
        const int rel0 = (int)(rbase - start);
        int lv = lane; // opaque: addresses and panel offsets are formed per step, not kept across the loop
        asm volatile("" : "+v"(lv));
        const int rv = lv & 31, gv = lv >> 5;
        const int rnext = rbase + 128 < stop ? rel0 + 128 : rel0; // clamped: one harmless re-read at the end
        // ---- gate: 128 features of the 32 rows, rounded to bf16, kept in accumulator order ----
        bf16x8 gate[4][2];
        {
            bf16x8 yf[CK];
            const PanelRegs yb = panel_load_near(y_w + 64, y_pitch, rel0, last_rel, 0, lv);
            panel_store(panel, lv, ya);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                yf[k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
            panel_store(panel, lv, yb);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                yf[4 + k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
            ya = panel_load_near(y_w, y_pitch, rnext, last_rel, 0, lv);
            const float *gbias = bg + 4 * gv;
#pragma unroll
            for (int nb_ = 0; nb_ < 4; ++nb_) {
                f32x16 acc = zero16();
#pragma unroll
                for (int ks = 0; ks < CK; ++ks) {
                    acc = mfma(as_bf16x8(wg_s[(nb_ * CK + ks) * 64 + lv]), yf[ks], acc);
                }
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(gbias + nb_ * 32 + 8 * a);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        gate[nb_][a >> 1][4 * (a & 1) + c] = (bf16_t)(acc[4 * a + c] + bv[c]);
                    }
                }
            }
        }
        // ---- projection of the same rows, gating, residual ----
        bf16x8 xf[CK];
        if constexpr (X_CHANNEL_FIRST) {
            const PanelRegs xb = load_cf(64, rbase, lv);
            // the panel holds [64 channels][32 positions], 64 bytes per channel, lane ln's pieces at slots ln + 64 i
            const lds_char *tile = (const lds_char *)panel;
            const int tr_off = ((lv >> 5) * 8 + ((lv & 15) >> 2)) * 64 + (4 * ((lv >> 4) & 1) + (lv & 3)) * 8;
            panel[lv] = xa.r0, panel[64 + lv] = xa.r1, panel[128 + lv] = xa.r2, panel[192 + lv] = xa.r3;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xf[k] = lds_transposed_fragment(tile + tr_off + k * 1024, tile + tr_off + k * 1024 + 256);
            }
            panel[lv] = xb.r0, panel[64 + lv] = xb.r1, panel[128 + lv] = xb.r2, panel[192 + lv] = xb.r3;
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xf[4 + k] = lds_transposed_fragment(tile + tr_off + k * 1024, tile + tr_off + k * 1024 + 256);
            }
            xa = load_cf(0, rbase + 128 < stop ? rbase + 128 : rbase, lv);
            // LayerNorm over the 128 channels of the lane's position: this lane holds channels 16 k + 8 g + 0..7
            float x0 = to_f32(xf[0][0]);
            x0 = __shfl(x0, lv & 31, 64); // channel 0 sits in the lane of the lower half
            float s1 = 0.f, s2 = 0.f;
#pragma unroll
            for (int k = 0; k < CK; ++k) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float d = to_f32(xf[k][e]) - x0;
                    s1 += d;
                    s2 = fmaf(d, d, s2);
                }
            }
            s1 = half_swap_sum(s1), s2 = half_swap_sum(s2);
            const float nch = (float)C;
            const float mean = s1 / nch + x0;
            const float var = fmaxf((s2 - s1 * s1 / nch) / nch, 0.f);
            const float rstd = 1.0f / sqrtf(var + ln_eps);
            const float shift = -rstd * mean;
#pragma unroll
            for (int k = 0; k < CK; ++k) {
                const float *gm = ln_gamma + 16 * k + 8 * gv, *bt = ln_beta + 16 * k + 8 * gv;
                const f32x4 g0 = *reinterpret_cast<const f32x4 *>(gm), g1 = *reinterpret_cast<const f32x4 *>(gm + 4);
                const f32x4 b0 = *reinterpret_cast<const f32x4 *>(bt), b1 = *reinterpret_cast<const f32x4 *>(bt + 4);
                bf16x8 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    o[e] = (bf16_t)fmaf(fmaf(to_f32(xf[k][e]), rstd, shift), g0[e], b0[e]);
                    o[4 + e] = (bf16_t)fmaf(fmaf(to_f32(xf[k][4 + e]), rstd, shift), g1[e], b1[e]);
                }
                xf[k] = o;
            }
        } else {
            const PanelRegs xb = panel_load_near(x_w + 64, x_pitch, rel0, last_rel, 0, lv);
            panel_store(panel, lv, xa);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xf[k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
            panel_store(panel, lv, xb);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xf[4 + k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
            xa = panel_load_near(x_w, x_pitch, rnext, last_rel, 0, lv);
        }
        const float *bias = bo + 4 * gv;
#pragma unroll
        for (int half = 0; half < 2; ++half) { // 64 output features per panel
            uint4 zq[4]; // the rows of `out` to add to, requested before the MFMAs
            char *out_w = reinterpret_cast<char *>(out + start * out_ld + half * 64);
            uint32_t out_off[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int rel = rel0 + 8 * i + (lv >> 3);
                rel = rel < last_rel ? rel : last_rel;
                out_off[i] = __umul24((uint32_t)rel, 2u * (uint32_t)out_ld) + 16u * (lv & 7);
                zq[i] = *reinterpret_cast<const uint4 *>(out_w + out_off[i]);
            }
            f32x16 acc[2];
            acc[0] = zero16(), acc[1] = zero16();
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
#pragma unroll
                for (int n = 0; n < 2; ++n) {
                    acc[n] = mfma(as_bf16x8(wo_s[((2 * half + n) * CK + ks) * 64 + lv]), xf[ks], acc[n]);
                }
            }
#pragma unroll
            for (int n = 0; n < 2; ++n) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(bias + (2 * half + n) * 32 + 8 * a);
                    bf16x4 ov;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        // bf16(out) * sigmoid(bf16(gate)), rounded to bf16: the reference's rounding points
                        const float o = to_f32((bf16_t)(acc[n][4 * a + c] + bv[c]));
                        const float gt = to_f32(gate[2 * half + n][a >> 1][4 * (a & 1) + c]);
                        ov[c] = (bf16_t)(o * sigmoid_fast(gt));
                    }
                    *(reinterpret_cast<bf16x4 *>(panel + panel_slot(rv, n * 4 + a)) + gv) = ov;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int prow_ = 8 * i + (lv >> 3);
                const bf16x8 u = as_bf16x8(panel[panel_slot(prow_, lv & 7)]), z = as_bf16x8(zq[i]);
                bf16x8 res;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    res[e] = (bf16_t)(to_f32(z[e]) + to_f32(u[e]));
                }
                if (rel0 + prow_ <= last_rel) {
                    *reinterpret_cast<uint4 *>(out_w + out_off[i]) = as_uint4(res);
                }
            }
        }
    }
}

// Pair bias [H, S, S] -> fragment-major order: for head h, query block j and key tile t the two B
// operands of the selector MFMAs, [h][j][t][2][64 lanes] x 16 bytes, so that a wave of the attention
// kernels fetches the pair bias of a tile with two contiguous 1 KB loads straight into registers.
// Lane (r, g) holds 16 consecutive keys 32t+16g.. of query row 32j+pi(r); queries past S repeat row
// S-1 and keys past S read as zero (their mask bias is -inf).  The pair bias is shared by every batch
// row, so this pass moves 2*H*S*S bytes once per call, against B times that in the attention kernel.
__global__ __launch_bounds__(64) void pair_bias_fragments_kernel(const bf16_t *__restrict__ nb, int64_t nb_sh,
                                                                 int64_t nb_sq, int S, int NB, int NT, int vec,
                                                                 uint4 *__restrict__ out)
{
    const int lane = threadIdx.x;
    const int r = lane & 31, g = lane >> 5;
    const int t = blockIdx.x % NT, j = blockIdx.x / NT, h = blockIdx.y;
    int q = 32 * j + pi_row(r);
    q = q < S ? q : S - 1;
    const int key0 = 32 * t + 16 * g;
    const bf16_t *src = nb + (int64_t)h * nb_sh + (int64_t)q * nb_sq + key0;
    uint4 w0, w1;
    if (vec && key0 + 16 <= S) {
        w0 = *reinterpret_cast<const uint4 *>(src);
        w1 = *reinterpret_cast<const uint4 *>(src + 8);
    } else {
        const uint16_t *s16 = reinterpret_cast<const uint16_t *>(src);
        uint32_t wds[8];
#pragma unroll
        for (int v = 0; v < 8; ++v) {
            const uint32_t a0 = key0 + 2 * v < S ? s16[2 * v] : 0u;
            const uint32_t a1 = key0 + 2 * v + 1 < S ? s16[2 * v + 1] : 0u;
            wds[v] = a0 | (a1 << 16);
        }
        w0.x = wds[0], w0.y = wds[1], w0.z = wds[2], w0.w = wds[3];
        w1.x = wds[4], w1.y = wds[5], w1.z = wds[6], w1.w = wds[7];
    }
    // into log2 units (the logits MFMAs of attend_block_l2 accumulate exponents of 2), as fp16: the product of a bf16 value
    // with log2(e) keeps eleven significant bits instead of eight, so the second rounding costs 2^-12 of the bias, not 2^-9
    const bf16x8 s0 = as_bf16x8(w0), s1 = as_bf16x8(w1);
    uint32_t d[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        d[e] = (uint32_t)pair_bias_log2_f16(to_f32(s0[2 * e])) | ((uint32_t)pair_bias_log2_f16(to_f32(s0[2 * e + 1])) << 16);
        d[4 + e] = (uint32_t)pair_bias_log2_f16(to_f32(s1[2 * e])) | ((uint32_t)pair_bias_log2_f16(to_f32(s1[2 * e + 1])) << 16);
    }
    uint4 *dst = out + ((((int64_t)h * NB + j) * NT + t) * 2) * 64 + lane;
    dst[0] = make_uint4(d[0], d[1], d[2], d[3]);
    dst[64] = make_uint4(d[4], d[5], d[6], d[7]);
}

// Tuning hooks (kutacc_hip_set_tuning): a forced plan of the long-sequence kernel, the fragment-major pair bias switched
// off, one line per call on stderr.  Plain atomics: set from a test or an experiment, read on every launch.
std::atomic<int> g_forced_bpw{0}, g_forced_gw{0}, g_no_fragments{0}, g_debug{0};
std::atomic<int> g_pair_mode{0}; // persistent_pair_kernel: 0 = where every workgroup has two batch rows or more, 1 = wherever it can run, 2 = never

bool fragments_disabled() { return g_no_fragments.load(std::memory_order_relaxed) != 0; }

struct Plan {
    bool persistent;
    int NB, NW, BPW, GW;
    size_t lds_bytes;
};

int max_lds_bytes()
{
    static int table[KUTACC_DEVICE_SLOTS] = {};
    return kutacc_device_attribute(hipDeviceAttributeMaxSharedMemoryPerBlock, 64 * 1024, table);
}

int num_cus()
{
    static int table[KUTACC_DEVICE_SLOTS] = {};
    return kutacc_device_attribute(hipDeviceAttributeMultiprocessorCount, 256, table);
}

// batch-row groups per XCD of the persistent kernels: one workgroup per CU at most; groups of 8*H workgroups share
// batch-row sequences across the XCDs
int persistent_groups(int B, int H)
{
    const int per_ring = 8 * H;
    int ngrp = num_cus() / per_ring;
    const int need = (B + 7) / 8;
    ngrp = ngrp < 1 ? 1 : ngrp;
    return ngrp > need ? need : ngrp;
}

size_t head_kernel_lds(int C, int NB, int GW, int NW, int BPW)
{
    const int NT = (NB + 1) & ~1; // key tiles, padded to a pair
    if (C == 256 && BPW == 4) {
        // second layout of fused_head_kernel: K, then V with all four weight matrices lying on it, then a 4 KB input
        // panel per wave (the mask's place later: 128 NT + 64 bytes always fit under 4 NW + 1 >= NT)
        const size_t kv = (size_t)NT * 2 * 64 * 16, wbytes = (size_t)4 * (C / 16) * 64 * 16;
        return kv + (kv > wbytes ? kv : wbytes) + (size_t)NW * 4096;
    }
    // weight fragments (the mask, 4 bytes per key, and 16 flag words take their place later), K and V
    return (size_t)GW * (C / 16) * 64 * 16 + (size_t)NT * 2 * 64 * 16 * 2;
}

size_t persistent_kernel_lds(int C, int NB)
{
    // all four weight matrices of the head, K and V of one batch row, per wave one 4 KB panel and 2 KB of
    // parked gate fragments, two mask buffers, flags
    const int NT = (NB + 1) & ~1; // key tiles, padded to a pair
    return (size_t)4 * (C / 16) * 64 * 16 + (size_t)NT * 2 * 64 * 16 * 2 + (size_t)NB * (4096 + 2048) +
           (size_t)2 * NT * 32 * 4 + 16;
}

size_t pair_kernel_lds(int C, int NB)
{
    // persistent_pair_kernel: the head's four weight matrices, K and V of two batch rows, per wave one 2 KB panel, two
    // pairs' masks of two rows each, flags
    const int NT = (NB + 1) & ~1;
    return (size_t)4 * (C / 16) * 64 * 16 + (size_t)2 * NT * 2 * 64 * 16 * 2 + (size_t)NB * 2048 + (size_t)4 * NT * 32 * 4 + 16;
}

bool make_plan(int64_t S, int C, Plan &pl)
{
    const int64_t NB = (S + 31) / 32;
    if (NB > 32) {
        return false;
    }
    pl.NB = (int)NB;
    pl.persistent = false;
    const size_t cap = (size_t)max_lds_bytes();
    const int forced_bpw = g_forced_bpw.load(std::memory_order_relaxed), forced_gw = g_forced_gw.load(std::memory_order_relaxed);
    // persistent kernel: one wave per sequence block, everything of one head resident in LDS
    const bool fits_persistent = NB <= max_waves(C, 1) && persistent_kernel_lds(C, (int)NB) <= cap;
    if (fits_persistent && forced_bpw == 0) {
        pl.persistent = true;
        pl.NW = (int)NB, pl.BPW = 1, pl.GW = 4, pl.lds_bytes = persistent_kernel_lds(C, (int)NB);
        return true;
    }
    if (forced_bpw != 0) {
        const int bpw = forced_bpw;
        const int gw = (C == 128 || bpw == 4) ? 4 : forced_gw; // those kernels are compiled for one group of four
        const int nw = (int)((NB + bpw - 1) / bpw);
        if (nw <= max_waves(C, bpw) && head_kernel_lds(C, pl.NB, gw, nw, bpw) <= cap) {
            pl.BPW = bpw, pl.NW = nw, pl.GW = gw, pl.lds_bytes = head_kernel_lds(C, pl.NB, gw, nw, bpw);
            return true;
        }
    }
    // fewest idle wave slots first, then fewest blocks per wave (more waves to overlap MFMA and VALU)
    int best_idle = 1 << 30;
    pl.BPW = 0;
    for (int bpw = 1; bpw <= 4; ++bpw) {
        const int nw = (int)((NB + bpw - 1) / bpw);
        if (nw > max_waves(C, bpw)) {
            continue;
        }
        const int idle = nw * bpw - (int)NB;
        if (idle < best_idle) {
            best_idle = idle, pl.BPW = bpw, pl.NW = nw;
        }
    }
    if (pl.BPW == 0) {
        return false;
    }
    // The 128-channel kernels and the 256-channel one with four blocks per wave are compiled for one group of four.
    const int gw_min = (C == 128 || pl.BPW == 4) ? 4 : 1;
    for (int gw = 4; gw >= gw_min; gw >>= 1) {
        const size_t need = head_kernel_lds(C, pl.NB, gw, pl.NW, pl.BPW);
        if (need <= cap) {
            pl.GW = gw, pl.lds_bytes = need;
            return true;
        }
    }
    return false;
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Bytes of the fragment-major copy of the pair bias: [nheads][NB query blocks][NB rounded up to even key tiles][2][64] x 16
int64_t fragment_bytes(int64_t nheads, int NB) { return nheads * NB * ((NB + 1) & ~1) * 2048; }

// Where the fast attention loop keeps its fragment-major copy of the pair bias, or nullptr when the call gets none: the
// workspace the options bring, else the caller's q scratch tensor when that is dense, aligned and large enough.
// `scale`: 1 for the fp16 fragments, 2 for the fp32 tiles of persistent_pair_kernel
void *fragment_home(const kutacc_hip_attention_args_t &a, int NB, const kutacc_launch::FusedAttentionOptions &opt, int scale = 1)
{
    if (a.nonbatched_bias == nullptr || fragments_disabled()) {
        return nullptr;
    }
    const int64_t nbf_bytes = fragment_bytes(a.nheads, NB) * scale;
    if (opt.fragment_workspace != nullptr) {
        return (aligned(opt.fragment_workspace, 16) && (uint64_t)nbf_bytes <= opt.fragment_workspace_bytes)
                   ? opt.fragment_workspace
                   : nullptr;
    }
    const int64_t C = a.nheads * a.head_size;
    const bool q_dense = a.q != nullptr && aligned(a.q, 16) && a.q_stride_h == a.head_size && a.q_stride_s == C &&
                         a.q_stride_b == a.seq_len * C;
    return (q_dense && nbf_bytes <= a.batch * a.seq_len * C * 2) ? a.q : nullptr;
}

// Two batch rows per step (persistent_pair_kernel): 128 channels, log2 units, a home for the fp32 tiles of the pair bias
// (twice the fragments' bytes), no LayerNorm inside the kernel and no ready-made fp16 fragments; by default only where
// every workgroup walks at least two rows.
bool pair_kernel_applies(const kutacc_hip_attention_args_t &a, const Plan &pl, const kutacc_launch::FusedAttentionOptions &opt)
{
    const int pair_mode = g_pair_mode.load(std::memory_order_relaxed);
    const int64_t C = a.nheads * a.head_size;
    return pl.persistent && (C == 128 || C == 256) && pair_mode != 2 && !fragments_disabled() && opt.ln_gamma == nullptr &&
           !opt.nb_fragments_ready && pair_kernel_lds((int)C, pl.NB) <= (size_t)max_lds_bytes() &&
           (a.nonbatched_bias == nullptr || fragment_home(a, pl.NB, opt, 2) != nullptr) &&
           (pair_mode == 1 || a.batch >= 16 * (int64_t)persistent_groups((int)a.batch, (int)a.nheads));
}

template <typename K>
int opt_in_lds(K kern, size_t bytes, size_t *table)
{
    return (int)kutacc_opt_in_lds(reinterpret_cast<const void *>(kern), bytes, table);
}

template <int C, int BPW, bool HAS_NB>
int launch_head_kernel(const FusedParams &p, const Plan &pl, hipStream_t stream)
{
    auto kern = fused_head_kernel<C, BPW, HAS_NB>;
    static size_t configured[KUTACC_DEVICE_SLOTS] = {}; // per instantiation and device: dynamic LDS opted into so far
    if (const int rc = opt_in_lds(kern, pl.lds_bytes, configured)) {
        return rc;
    }
    const int64_t units = ((int64_t)(p.B + 7) / 8) * 8 * p.H;
    kern<<<dim3((unsigned)units), dim3((unsigned)(pl.NW * 64)), pl.lds_bytes, stream>>>(p);
    return kutacc_hip_status(hipGetLastError());
}

template <int C, bool HAS_NB, bool L2MODE, bool FUSED_LN = false>
int launch_persistent_kernel(FusedParams p, const Plan &pl, hipStream_t stream)
{
    auto kern = persistent_head_kernel<C, HAS_NB, L2MODE, FUSED_LN>;
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    if (const int rc = opt_in_lds(kern, pl.lds_bytes, configured)) {
        return rc;
    }
    p.ngrp = persistent_groups(p.B, p.H);
    kern<<<dim3((unsigned)(8 * p.H * p.ngrp)), dim3((unsigned)(pl.NW * 64)), pl.lds_bytes, stream>>>(p);
    return kutacc_hip_status(hipGetLastError());
}

template <int C, bool HAS_NB>
int launch_pair_kernel(FusedParams p, const Plan &pl, hipStream_t stream)
{
    auto kern = persistent_pair_kernel<C, HAS_NB>;
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    const size_t lds_bytes = pair_kernel_lds(C, pl.NB);
    if (const int rc = opt_in_lds(kern, lds_bytes, configured)) {
        return rc;
    }
    p.ngrp = persistent_groups(p.B, p.H);
    kern<<<dim3((unsigned)(8 * p.H * p.ngrp)), dim3((unsigned)(pl.NW * 64)), lds_bytes, stream>>>(p);
    return kutacc_hip_status(hipGetLastError());
}

template <int C>
int dispatch_head_kernel(const FusedParams &p, const Plan &pl, hipStream_t stream)
{
    const bool nb = p.nb != nullptr;
    if (pl.persistent) {
        if (p.ln_gamma != nullptr) { // only asked for where fused_layernorm_supported says so: log2 units
            return nb ? launch_persistent_kernel<C, true, true, true>(p, pl, stream)
                      : launch_persistent_kernel<C, false, true, true>(p, pl, stream);
        }
        if (p.l2mode) {
            return nb ? launch_persistent_kernel<C, true, true>(p, pl, stream) : launch_persistent_kernel<C, false, true>(p, pl, stream);
        }
        return nb ? launch_persistent_kernel<C, true, false>(p, pl, stream) : launch_persistent_kernel<C, false, false>(p, pl, stream);
    }
    switch (pl.BPW) {
        case 1: return nb ? launch_head_kernel<C, 1, true>(p, pl, stream) : launch_head_kernel<C, 1, false>(p, pl, stream);
        case 2: return nb ? launch_head_kernel<C, 2, true>(p, pl, stream) : launch_head_kernel<C, 2, false>(p, pl, stream);
        case 3: return nb ? launch_head_kernel<C, 3, true>(p, pl, stream) : launch_head_kernel<C, 3, false>(p, pl, stream);
        case 4: return nb ? launch_head_kernel<C, 4, true>(p, pl, stream) : launch_head_kernel<C, 4, false>(p, pl, stream);
        default: return KUTACC_HIP_EUNSUPPORTED;
    }
}

// How output_projection_kernel<C, .> splits M rows: workgroups along the rows and rows per wave (a multiple of 8).  Two
// workgroups of four waves per CU, or one of eight: each wave with an equal share of the rows (a third resident
// workgroup, where the registers allow one, measured slower: the weight slab is staged per workgroup).
inline void output_projection_split(int C, int64_t M, int64_t &gx, int64_t &rpw)
{
    const int waves = 4 * (C / 128);
    const int64_t tiles = (M + 31) / 32;
    gx = (tiles + waves - 1) / waves;
    const int64_t cap = (int64_t)num_cus() * (C == 128 ? 2 : 1);
    gx = gx > cap ? cap : gx;
    rpw = ((M + gx * waves - 1) / (gx * waves) + 7) / 8 * 8;
}

// The kernel addresses a wave's rows with 32-bit byte offsets from the wave's first row: true when that range fits for
// these row pitches under the split the launcher will choose.
inline bool output_projection_rows_fit(int C, int64_t M, int64_t a_ld, int64_t out_ld)
{
    if (a_ld <= 0 || out_ld <= 0 || M <= 0) {
        return false;
    }
    int64_t gx, rpw;
    output_projection_split(C, M, gx, rpw);
    const int64_t pitch = a_ld > out_ld ? a_ld : out_ld;
    return pitch < (1 << 23) && (rpw + 32) * pitch * 2 < ((int64_t)1 << 31);
}

// out[M, N] = a[M, K] . w[N, K]^T + bias with K = C and N a multiple of 128 (one grid row per 128-feature slab)
template <int C, int EPILOGUE = EPILOGUE_STORE>
int launch_output_projection(const void *a, int64_t a_ld, const void *w, const float *bias, void *out, int64_t out_ld,
                             int64_t M, int64_t N, hipStream_t stream, const void *gate = nullptr, int64_t gate_ld = 0,
                             int64_t swap_n = 0)
{
    // the transposing residual epilogue finds its rows of `out` with 32-bit arithmetic where the tensor allows (without
    // the transposition there is no division to save, and the 64-bit form measured 1 us faster at 384 x 384 rows)
    const bool near_out = EPILOGUE == EPILOGUE_RESIDUAL && M < (1 << 24) && out_ld > 0 && out_ld < (1 << 22) &&
                          M * out_ld * 2 < ((int64_t)1 << 31) && swap_n >= 32 && M % swap_n == 0;
    auto kern = near_out ? output_projection_kernel<C, EPILOGUE, EPILOGUE == EPILOGUE_RESIDUAL> : output_projection_kernel<C, EPILOGUE, false>;
    constexpr int SLABS = C / 128, WAVES = 4 * SLABS;
    const size_t lds_bytes = (size_t)SLABS * 4 * (C / 16) * 64 * 16 + WAVES * 4096;
    static size_t configured[2][KUTACC_DEVICE_SLOTS] = {}; // one table per kernel the pointer may hold
    if (const int rc = opt_in_lds(kern, lds_bytes, configured[near_out ? 1 : 0])) {
        return rc;
    }
    if (!output_projection_rows_fit(C, M, a_ld, out_ld)) {
        return KUTACC_HIP_EUNSUPPORTED; // the callers' support checks ask the same question first
    }
    int64_t gx, rpw;
    output_projection_split(C, M, gx, rpw);
    const int64_t gy = (N / 128 + SLABS - 1) / SLABS;
    kern<<<dim3((unsigned)gx, (unsigned)gy), 64 * WAVES, lds_bytes, stream>>>(
        (const bf16_t *)a, a_ld, (const bf16_t *)w, bias, (bf16_t *)out, out_ld, M, (int)N, (int)rpw, (const bf16_t *)gate,
        gate_ld, swap_n);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace

namespace kutacc_launch {

bool fused_attention_fragment_layout(const kutacc_hip_attention_args_t &a, int *nb, int *nt)
{
    Plan pl;
    if (!fused_attention_supports(a) || !make_plan(a.seq_len, (int)(a.nheads * a.head_size), pl) ||
        fragment_home(a, pl.NB, FusedAttentionOptions()) == nullptr) {
        return false;
    }
    *nb = pl.NB, *nt = (pl.NB + 1) & ~1;
    return true;
}

bool fused_attention_tile_layout(const kutacc_hip_attention_args_t &a, const FusedAttentionOptions &opt, int *nb, int *nt)
{
    Plan pl;
    if (a.nonbatched_bias == nullptr || opt.nb_fragments_ready || !fused_attention_supports(a) ||
        !make_plan(a.seq_len, (int)(a.nheads * a.head_size), pl) || !pair_kernel_applies(a, pl, opt)) {
        return false;
    }
    *nb = pl.NB, *nt = (pl.NB + 1) & ~1;
    return true;
}

bool fused_layernorm_supported(const kutacc_hip_attention_args_t &a, const FusedAttentionOptions &opt)
{
    Plan pl;
    if (!fused_attention_supports(a) || !make_plan(a.seq_len, (int)(a.nheads * a.head_size), pl) || !pl.persistent ||
        fragments_disabled()) {
        return false;
    }
    // log2 units need the fragment-major pair bias (none without a pair bias)
    return a.nonbatched_bias == nullptr || fragment_home(a, pl.NB, opt) != nullptr;
}

bool fused_attention_supports(const kutacc_hip_attention_args_t &a)
{
    if (a.dtype != KUTACC_DTYPE_BF16 || a.head_size != HEAD) {
        return false;
    }
    const int64_t C = a.nheads * a.head_size;
    if (C != 128 && C != 256) {
        return false;
    }
    if (a.batch > (1 << 24) || a.seq_len > 1024) {
        return false;
    }
    // the kernels address the rows of one batch row (the output projection: of a wave's range) with 32-bit byte offsets
    if (a.input_ld <= 0 || a.input_ld > (1 << 19) || a.out_ld <= 0 || a.out_ld > (1 << 19) || a.avg_stride_s <= 0 ||
        a.avg_stride_s > (1 << 19)) {
        return false;
    }
    // 16-byte row loads of input and weights, 8-byte stores of avg/out rows
    if (a.input_ld % 8 != 0 || !aligned(a.input, 16) || !aligned(a.query_w, 16) || !aligned(a.key_w, 16) ||
        !aligned(a.value_w, 16) || !aligned(a.gating_w, 16) || !aligned(a.output_w, 16) || !aligned(a.gating_b, 16) ||
        !aligned(a.output_b, 16)) {
        return false;
    }
    if (a.avg_stride_h != HEAD || a.avg_stride_s % 8 != 0 || a.avg_stride_b != a.seq_len * a.avg_stride_s ||
        !aligned(a.avg, 16) || a.out_ld % 8 != 0 || !aligned(a.out, 16)) {
        return false;
    }
    // ... and the output projection a wave's range of the batch * seq_len rows of avg and out
    if (!output_projection_rows_fit((int)C, a.batch * a.seq_len, a.avg_stride_s, a.out_ld)) {
        return false;
    }
    Plan pl;
    return make_plan(a.seq_len, (int)C, pl);
}

int gating_attention_fused(const kutacc_hip_attention_args_t &a, hipStream_t stream, const FusedAttentionOptions &opt)
{
    const int residual = opt.out_mode;
    const int C = (int)(a.nheads * a.head_size);
    Plan pl;
    if (!make_plan(a.seq_len, C, pl)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    if (opt.bias_stride_k < 0 || opt.bias_stride_k > (1 << 20) || a.input_ld <= 0 || a.input_ld > (1 << 19)) {
        return KUTACC_HIP_EUNSUPPORTED; // 32-bit offsets within a batch row (fused_attention_supports checks input_ld too)
    }
    FusedParams p;
    p.x = (const bf16_t *)a.input;
    p.w[PROJ_K] = (const bf16_t *)a.key_w, p.w[PROJ_V] = (const bf16_t *)a.value_w;
    p.w[PROJ_Q] = (const bf16_t *)a.query_w, p.w[PROJ_G] = (const bf16_t *)a.gating_w;
    p.bg = a.gating_b;
    p.bias = (const bf16_t *)a.bias;
    p.nb = (const bf16_t *)a.nonbatched_bias;
    p.avg = (bf16_t *)a.avg;
    p.x_ld = a.input_ld, p.bias_sb = a.bias_stride_b, p.nb_sh = a.nb_stride_h, p.nb_sq = a.nb_stride_q;
    p.x_sb = opt.input_stride_b != 0 ? opt.input_stride_b : a.seq_len * a.input_ld;
    p.ln_gamma = nullptr, p.ln_beta = nullptr, p.ln_eps = 0.f;
    p.bias_sk = opt.bias_stride_k, p.bias_is_mask = opt.bias_is_mask ? 1 : 0;
    p.avg_sb = a.avg_stride_b, p.avg_ss = a.avg_stride_s, p.avg_sh = a.avg_stride_h;
    p.B = (int)a.batch, p.S = (int)a.seq_len, p.H = (int)a.nheads, p.NB = pl.NB, p.NW = pl.NW, p.GW = pl.GW;
    p.NT = (pl.NB + 1) & ~1;
    p.nb_vec = (p.nb != nullptr && aligned(p.nb, 16) && a.nb_stride_h % 8 == 0 && a.nb_stride_q % 8 == 0) ? 1 : 0;
    // (float)(1/sqrt(head_size)) as the reference forms it (gating_attention.cpp:68)
    p.qscale = (float)(1.0 / sqrt((double)a.head_size));
    p.ngrp = 1;
    p.nbf = nullptr;
    p.l2mode = 0;
    // Fragment-major copy of the pair bias for the fast attention loop.  It lives in the workspace the options bring or in
    // the caller's q scratch tensor (which this path does not otherwise use; its contents are unspecified after any
    // call) when that is dense, aligned and large enough; otherwise the kernels read the pair bias in place through the
    // staging panels.
    void *const fragments = fragment_home(a, pl.NB, opt);
    if (opt.fragment_workspace != nullptr && p.nb != nullptr && fragments == nullptr && !fragments_disabled()) {
        return KUTACC_HIP_EINVAL; // the caller's workspace cannot hold the copy
    }
    void *const tiles = fragment_home(a, pl.NB, opt, 2);
    const bool pair_kernel = pair_kernel_applies(a, pl, opt);
    if (opt.nb_tiles_ready && (!pair_kernel || p.nb == nullptr)) {
        return KUTACC_HIP_EINVAL; // the caller asks fused_attention_tile_layout under the same options and tuning first
    }

    const double BS = (double)a.batch * (double)a.seq_len;
    int rc;
    if (pair_kernel) {
        if (p.nb != nullptr && opt.nb_tiles_ready) {
            p.nbf = (const uint4 *)tiles; // the producer of the pair bias wrote the tiles
        } else if (p.nb != nullptr) {
            kutacc_prof::KernelTimer t("pair_bias_tiles_kernel", 0.0, stream);
            pair_bias_tiles_kernel<<<dim3((unsigned)(pl.NB * p.NT), (unsigned)a.nheads), 64, 0, stream>>>(
                p.nb, p.nb_sh, p.nb_sq, p.S, pl.NB, p.NT, p.nb_vec, (f32x4 *)tiles);
            rc = kutacc_hip_status(hipGetLastError());
            if (rc != 0) {
                return rc;
            }
            p.nbf = (const uint4 *)tiles;
        }
    } else if (fragments != nullptr && opt.nb_fragments_ready) {
        p.nbf = (const uint4 *)fragments; // the producer of the pair bias wrote the copy
    } else if (fragments != nullptr) {
        kutacc_prof::KernelTimer t("pair_bias_fragments_kernel", 0.0, stream);
        pair_bias_fragments_kernel<<<dim3((unsigned)(pl.NB * p.NT), (unsigned)a.nheads), 64, 0, stream>>>(
            p.nb, p.nb_sh, p.nb_sq, p.S, pl.NB, p.NT, p.nb_vec, (uint4 *)fragments);
        rc = kutacc_hip_status(hipGetLastError());
        if (rc != 0) {
            return rc;
        }
        p.nbf = (const uint4 *)fragments;
    }
    p.l2mode = ((p.nb == nullptr || p.nbf != nullptr) && !fragments_disabled()) ? 1 : 0;
    if (opt.ln_gamma != nullptr) {
        if (!pl.persistent || !p.l2mode || opt.ln_beta == nullptr || !aligned(opt.ln_gamma, 16) || !aligned(opt.ln_beta, 16)) {
            return KUTACC_HIP_EUNSUPPORTED; // the caller asks fused_layernorm_supported first
        }
        p.ln_gamma = opt.ln_gamma, p.ln_beta = opt.ln_beta, p.ln_eps = opt.ln_eps;
    }
    if (g_debug.load(std::memory_order_relaxed)) {
        fprintf(stderr,
                "[kutacc] fused plan: persistent=%d C=%d NB=%d NT=%d NW=%d BPW=%d GW=%d lds=%zu max_lds=%d cus=%d log2_units=%d "
                "fragments=%d row_pairs=%d\n",
                (int)pl.persistent, C, pl.NB, p.NT, pl.NW, pl.BPW, pl.GW, pl.lds_bytes, max_lds_bytes(), num_cus(), p.l2mode,
                p.nbf != nullptr ? 1 : 0, (int)pair_kernel);
    }
    {
        kutacc_prof::KernelTimer t(pair_kernel ? "persistent_pair_kernel" : pl.persistent ? "persistent_head_kernel" : "fused_head_kernel",
                                   8.0 * BS * C * C + 4.0 * BS * (double)a.seq_len * C, stream);
        rc = pair_kernel ? (C == 128 ? (p.nb != nullptr ? launch_pair_kernel<128, true>(p, pl, stream) : launch_pair_kernel<128, false>(p, pl, stream))
                                     : (p.nb != nullptr ? launch_pair_kernel<256, true>(p, pl, stream) : launch_pair_kernel<256, false>(p, pl, stream)))
             : (C == 128) ? dispatch_head_kernel<128>(p, pl, stream)
                          : dispatch_head_kernel<256>(p, pl, stream);
        if (rc != 0) {
            return rc;
        }
    }
    const int64_t M = a.batch * a.seq_len;
    if (residual != FUSED_OUT_STORE) {
        // out += result, row (b, s) of the result going to row (s, b) of out ([seq_len, batch, C]) in the transposed form
        const int64_t swap_n = residual == FUSED_OUT_ADD_TRANSPOSED ? a.seq_len : 0;
        kutacc_prof::KernelTimer t("output_projection_kernel<residual>", 2.0 * BS * C * C, stream);
        return (C == 128) ? launch_output_projection<128, EPILOGUE_RESIDUAL>(a.avg, a.avg_stride_s, a.output_w, a.output_b, a.out,
                                                                             a.out_ld, M, C, stream, nullptr, 0, swap_n)
                          : launch_output_projection<256, EPILOGUE_RESIDUAL>(a.avg, a.avg_stride_s, a.output_w, a.output_b, a.out,
                                                                             a.out_ld, M, C, stream, nullptr, 0, swap_n);
    }
    kutacc_prof::KernelTimer t("output_projection_kernel", 2.0 * BS * C * C, stream);
    return (C == 128) ? launch_output_projection<128>(a.avg, a.avg_stride_s, a.output_w, a.output_b, a.out, a.out_ld, M, C, stream)
                      : launch_output_projection<256>(a.avg, a.avg_stride_s, a.output_w, a.output_b, a.out, a.out_ld, M, C, stream);
}

// The attention's output-projection kernel on its own: out[m, n] = sum_k a[m, k] * w[n, k] + bias[n] for rows of
// 128 or 256 input features (w dense [n, k]) and n a multiple of 128.  HBM-bound; every row is read and written
// once per 128-feature slab of the output.
bool row_projection_supports(const void *a, int64_t a_ld, const void *w, const float *bias, const void *out, int64_t out_ld,
                             int64_t m, int64_t n, int64_t k)
{
    // row pitches the kernel's 32-bit offsets within a wave's range of rows can take under the launcher's split of m rows
    if (k != 128 && k != 256) {
        return false;
    }
    const bool pitches = a_ld > 0 && out_ld > 0 && a_ld <= (1 << 19) && out_ld <= (1 << 19) && m > 0 &&
                         output_projection_rows_fit((int)k, m, a_ld, out_ld);
    return n > 0 && n % 128 == 0 && n / 128 <= 65535 && m > 0 && m <= INT32_MAX - 64 && bias && pitches &&
           a_ld % 8 == 0 && out_ld % 8 == 0 && aligned(a, 16) && aligned(w, 16) && aligned(bias, 16) && aligned(out, 16);
}

int row_projection(const void *a, int64_t a_ld, const void *w, const float *bias, void *out, int64_t out_ld, int64_t m,
                   int64_t n, int64_t k, hipStream_t stream)
{
    if (!row_projection_supports(a, a_ld, w, bias, out, out_ld, m, n, k)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("output_projection_kernel", 2.0 * (double)m * (double)n * (double)k, stream);
    return k == 128 ? launch_output_projection<128>(a, a_ld, w, bias, out, out_ld, m, n, stream)
                    : launch_output_projection<256>(a, a_ld, w, bias, out, out_ld, m, n, stream);
}

// acc[m, n] += bf16(sum_k a[m, k] * w[n, k] + bias[n]) * sigmoid(gate[m, n]): same shapes as row_projection
int row_projection_gated_residual(const void *a, int64_t a_ld, const void *w, const float *bias, const void *gate,
                                  int64_t gate_ld, void *acc, int64_t acc_ld, int64_t m, int64_t n, int64_t k,
                                  hipStream_t stream)
{
    if (!row_projection_supports(a, a_ld, w, bias, acc, acc_ld, m, n, k) || !gate || gate_ld % 8 != 0 || !aligned(gate, 16)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("output_projection_kernel<gated residual>", 2.0 * (double)m * (double)n * (double)k, stream);
    return k == 128 ? launch_output_projection<128, EPILOGUE_GATED_RESIDUAL>(a, a_ld, w, bias, acc, acc_ld, m, n, stream, gate, gate_ld)
                    : launch_output_projection<256, EPILOGUE_GATED_RESIDUAL>(a, a_ld, w, bias, acc, acc_ld, m, n, stream, gate, gate_ld);
}

// acc[m, 128] += bf16(bf16(a . w^T + bias) * sigmoid(bf16(y . wg^T + bg))), a and y rows of 128 features: the gate
// projection inside the kernel (no gate tensor)
bool row_projection_projected_gate_supports(const void *a, int64_t a_ld, const void *w, const float *bias, const void *y,
                                            int64_t y_ld, const void *wg, const float *bg, const void *acc, int64_t acc_ld,
                                            int64_t m, int64_t n, int64_t k, int64_t ky)
{
    // the kernel addresses rows by 32-bit byte offsets: of a wave's rows from its first one, of a channel-first `a`
    // (a_ld >= m) from its first element
    const int64_t lim = (int64_t)1 << 31;
    const bool near = m < (1 << 23) && a_ld > 0 && a_ld < (1 << 23) && y_ld > 0 && acc_ld > 0 && m * y_ld * 2 < lim &&
                      m * acc_ld * 2 < lim && (a_ld >= m || m * a_ld * 2 < lim);
    return k == 128 && ky == 128 && n == 128 && m > 0 && near && bias && bg && y && wg && a_ld % 8 == 0 &&
           y_ld % 8 == 0 && acc_ld % 8 == 0 && aligned(a, 16) && aligned(w, 16) && aligned(bias, 16) && aligned(y, 16) &&
           aligned(wg, 16) && aligned(bg, 16) && aligned(acc, 16);
}

// ln_gamma != nullptr: `a` is channel-first ([128, m], channel stride a_ld, m a multiple of 8) and not yet normalised;
// the kernel applies LayerNorm(ln_gamma, ln_beta, ln_eps) over its 128 channels on the way in
int row_projection_projected_gate_residual(const void *a, int64_t a_ld, const void *w, const float *bias, const void *y,
                                           int64_t y_ld, const void *wg, const float *bg, void *acc, int64_t acc_ld, int64_t m,
                                           hipStream_t stream, const float *ln_gamma, const float *ln_beta, float ln_eps)
{
    if (!row_projection_projected_gate_supports(a, a_ld, w, bias, y, y_ld, wg, bg, acc, acc_ld, m, 128, 128, 128)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    const bool cf = ln_gamma != nullptr;
    if (cf && (!ln_beta || m % 8 != 0 || m < 8 || !aligned(ln_gamma, 16) || !aligned(ln_beta, 16))) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    constexpr size_t lds_bytes = (size_t)2 * 4 * 8 * 64 * 16 + 4 * 4096;
    static size_t configured[2][KUTACC_DEVICE_SLOTS] = {};
    if (const int rc = cf ? opt_in_lds(projected_gate_residual_kernel<true>, lds_bytes, configured[1])
                          : opt_in_lds(projected_gate_residual_kernel<false>, lds_bytes, configured[0])) {
        return rc;
    }
    kutacc_prof::KernelTimer t(cf ? "projected_gate_residual_kernel<channel-first>" : "projected_gate_residual_kernel",
                               4.0 * (double)m * 128.0 * 128.0, stream);
    const int64_t tiles = (m + 31) / 32;
    int64_t gx = (tiles + 3) / 4;
    const int64_t cap = (int64_t)num_cus() * 2; // two workgroups per CU, each wave with an equal share of the rows
    gx = gx > cap ? cap : gx;
    const int64_t rpw = ((m + gx * 4 - 1) / (gx * 4) + 7) / 8 * 8; // a workgroup's range, 4 rpw rows, is whole 32-row steps
    auto kern = cf ? projected_gate_residual_kernel<true> : projected_gate_residual_kernel<false>;
    kern<<<dim3((unsigned)gx), 256, lds_bytes, stream>>>((const bf16_t *)a, a_ld, (const bf16_t *)w, bias, (const bf16_t *)y, y_ld,
                                                         (const bf16_t *)wg, bg, (bf16_t *)acc, acc_ld, m, (int)rpw, ln_gamma,
                                                         ln_beta, ln_eps);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch

// ------------------------------------------------------------------------------------------------
// Entry point that allocates nothing: the fragment-major copy of the pair bias -- the one scratch buffer of the fused
// path, which kutacc_hip_gating_attention keeps in the caller's q tensor -- lives in a device array that is part of the
// library image.  Every GPU the library runs on holds its own copy of the array, at its own address, until the process
// ends; the address is asked for once per device and kept.
// ------------------------------------------------------------------------------------------------
namespace {
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)KUTACC_HIP_STATIC_SCRATCH_BYTES;
}
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

namespace {
std::atomic<void *> g_scratch_ptr[KUTACC_DEVICE_SLOTS];

// device address of `scratch` on the current device (the array's name is a host-side stand-in, never a device address)
int static_scratch_address(void **out)
{
    const int slot = kutacc_device_slot();
    if (slot < 0) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    void *ptr = g_scratch_ptr[slot].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            return e != hipSuccess ? (int)e : KUTACC_HIP_EUNSUPPORTED;
        }
        g_scratch_ptr[slot].store(ptr, std::memory_order_release); // every thread gets the same answer for a device
    }
    *out = ptr;
    return 0;
}
} // namespace

extern "C" kutacc_export int kutacc_hip_gating_attention_static(const kutacc_hip_attention_args_t *a, void *stream)
{
    if (!a || !a->input || !a->query_w || !a->key_w || !a->value_w || !a->gating_w || !a->output_w || !a->gating_b ||
        !a->output_b || !a->bias || !a->out || !a->avg) {
        return KUTACC_HIP_EINVAL;
    }
    if (a->batch <= 0 || a->seq_len <= 0 || a->nheads <= 0 || a->head_size <= 0 || a->batch > INT32_MAX / a->seq_len ||
        a->nheads > INT32_MAX / a->head_size) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t C = a->nheads * a->head_size;
    if (a->input_ld < C || a->out_ld < C) {
        return KUTACC_HIP_EINVAL;
    }
    if (!kutacc_launch::fused_attention_supports(*a)) {
        return KUTACC_HIP_EUNSUPPORTED; // the shape-agnostic kernels need the caller's q, k, v and gate tensors
    }
    kutacc_launch::FusedAttentionOptions opt;
    if (a->nonbatched_bias != nullptr) {
        const int64_t need = fragment_bytes(a->nheads, (int)((a->seq_len + 31) / 32));
        if ((uint64_t)need > STATIC_SCRATCH_BYTES) {
            fprintf(stderr,
                    "kutacc_hip_gating_attention_static: the pair bias of %lld heads x %lld positions needs %lld bytes of "
                    "scratch, the library's static array holds %zu\n",
                    (long long)a->nheads, (long long)a->seq_len, (long long)need, STATIC_SCRATCH_BYTES);
            return KUTACC_HIP_EINVAL;
        }
        void *ptr = nullptr;
        if (const int rc = static_scratch_address(&ptr)) {
            return rc;
        }
        opt.fragment_workspace = ptr;
        opt.fragment_workspace_bytes = STATIC_SCRATCH_BYTES;
    }
    kutacc_prof::Suppress no_events;
    return kutacc_launch::gating_attention_fused(*a, stream ? (hipStream_t)stream : kutacc_api::default_stream(), opt);
}

// Tuning hooks for tests and experiments: "plan" = "bpw,gw" forces the long-sequence kernel with that many query blocks
// per wave and weight matrices per group where it fits (anything else: the planner decides), "fragments" = "0" keeps the
// kernels off the fragment-major pair bias (general attention blocks), "debug" = "1" prints the plan of every call.
int kutacc_launch::fused_attention_tuning(const char *name, const char *value)
{
    const bool on = value && value[0] != '\0' && value[0] != '0';
    if (!strcmp(name, "plan")) {
        int bpw = 0, gw = 0;
        if (value && sscanf(value, "%d,%d", &bpw, &gw) == 2 && bpw >= 1 && bpw <= 4 && (gw == 1 || gw == 2 || gw == 4)) {
            g_forced_gw.store(gw), g_forced_bpw.store(bpw);
        } else {
            g_forced_bpw.store(0), g_forced_gw.store(0);
        }
        return 0;
    }
    if (!strcmp(name, "row_pairs")) { // "1": wherever the two-row kernel can run, "0": never, anything else: the default rule
        g_pair_mode.store(value && value[0] == '1' ? 1 : (value && value[0] == '0' ? 2 : 0));
        return 0;
    }
    if (!strcmp(name, "fragments")) {
        g_no_fragments.store((value && value[0] == '0') ? 1 : 0);
        return 0;
    }
    if (!strcmp(name, "debug")) {
        g_debug.store(on ? 1 : 0);
        return 0;
    }
    return KUTACC_HIP_EINVAL;
}
