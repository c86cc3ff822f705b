// Fused gated-attention kernels for gfx950 (CDNA4), bf16 storage, head_size 32.
//
// Kernel 1, fused_head_kernel: one workgroup per (batch row b, head h).  It reads the rows of
// `input` once per staged weight group, projects K_h and V_h for the whole sequence into LDS, keeps
// Q_h and sigmoid(gate_h) of each wave's own query blocks in registers, runs flash-style attention
// with online softmax over 32-key tiles (logits never leave registers) and writes the gated weighted
// average.  Everything that the reference materialises in memory between its GEMMs -- q, k, v, gate,
// the [bs, S] logits block, the probabilities (reference src/attention/gating_attention.cpp:47-66,
// 97-147) -- stays on chip.  Kernel 2, output_projection_kernel, is the final GEMM with fp32 bias
// (reference :152-157).
//
// All contractions are v_mfma_f32_32x32x16_bf16 (fp32 accumulate).  Operand fragments use one
// format throughout: a [32 rows x 16 k] slab, lane l holding row (l & 31), k-chunk (l >> 5)*8..+8,
// i.e. 16 contiguous bytes of a row-major bf16 matrix.  Results come out as D[i][j] with
// j = l & 31 and i = 8*(v/4) + 4*(l>>5) + (v&3) for accumulator register v.  Two consequences are
// used everywhere below:
//   * a contraction index may be permuted freely as long as both operands agree, so an accumulator
//     (rows i scattered as above) can be fed back as the k-dimension of the next MFMA without any
//     cross-lane movement: Q^T and K^T share their head-dim order, and the probabilities share
//     their key order with V;
//   * the sequence position handled by "row r" of a 32-row block is pi(r) = 16*((r>>2)&1) +
//     4*(r>>3) + (r&3), chosen so that the 16 logits a lane holds for its query are 16 CONSECUTIVE
//     keys (pair-bias row loads become two 16-byte loads).
#include <hip/hip_runtime.h>

#include "device_util.h"
#include "launch_internal.h"
#include "profiler.h"

using namespace kutacc_dev;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float LOG2E = 1.44269504088896340736f;
constexpr int HEAD = 32;          // head_size the MFMA kernels are written for
constexpr int MAX_WAVES = 12;     // 768 threads: 3 waves per SIMD, 168 VGPRs each

// Waves per workgroup a given instantiation may be launched with.  One query block per wave needs
// about 150 VGPRs at C=128, which fits three waves per SIMD; the variants that hold more state
// (more query blocks per wave, or 256 input channels in registers) get two waves per SIMD.
__host__ __device__ constexpr int max_waves(int C, int BPW) { return (C == 128 && BPW <= 2) ? MAX_WAVES : 8; }
constexpr float RESCALE_GAP = 8.f; // running max may lag the true max by this many octaves

enum Proj { PROJ_K = 0, PROJ_V = 1, PROJ_Q = 2, PROJ_G = 3 };

struct FusedParams {
    const bf16_t *x;
    const bf16_t *w[4]; // indexed by Proj
    const float *bg;
    const bf16_t *bias;
    const bf16_t *nb;
    bf16_t *avg;
    int64_t x_ld, bias_sb, nb_sh, nb_sq, avg_sb, avg_ss, avg_sh;
    int B, S, H, NB, NW, GW;
    int nb_vec; // pair-bias rows may be read with 16-byte loads
    float qscale; // log2(e) / sqrt(head_size)
};

__device__ __forceinline__ int pi_row(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

__device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ bf16x8 pack8(const f32x16 &v, int base)
{
    bf16x8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        r[i] = (bf16_t)v[base + i];
    }
    return r;
}

__device__ __forceinline__ bf16x8 as_bf16x8(uint4 u)
{
    union {
        uint4 u;
        bf16x8 b;
    } c;
    c.u = u;
    return c.b;
}

__device__ __forceinline__ uint4 as_uint4(bf16x8 b)
{
    union {
        uint4 u;
        bf16x8 b;
    } c;
    c.b = b;
    return c.u;
}

// combine the two 32-lane halves of a wave: returns op(x[lane], x[lane ^ 32]) in every lane
__device__ __forceinline__ float half_swap_max(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_swap_sum(float x)
{
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// LDS carve-up, in 16-byte units unless noted:
//   [0, GW*CK*64)               staged weight fragments  [slot][kstep][lane]
//   [.., +NB*2*64)              K fragments              [tile][kstep][lane]
//   [.., +NB*2*64)              V fragments              [tile][kstep][lane]
//   then floats: mask[NB*32] (log2-scaled, -inf past S), then ints: tile_flag[NB]
template <int C, int BPW>
__global__ __launch_bounds__(64 * max_waves(C, BPW)) void fused_head_kernel(FusedParams p)
{
    constexpr int CK = C / 16;
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
    const int lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int S = p.S, NB = p.NB, NW = p.NW, GW = p.GW;

    uint4 *lds_w = lds;
    uint4 *lds_k = lds_w + GW * CK * 64;
    uint4 *lds_v = lds_k + NB * 2 * 64;
    float *mask = reinterpret_cast<float *>(lds_v + NB * 2 * 64);
    int *tile_flag = reinterpret_cast<int *>(mask + NB * 32);

    // ---- mask bias -> LDS, pre-multiplied by log2(e); keys past S get -inf ----
    for (int t = tid; t < NB; t += nthreads) {
        tile_flag[t] = ((t + 1) * 32 > S) ? 1 : 0; // ragged last tile always takes the masked path
    }
    __syncthreads();
    for (int k = tid; k < NB * 32; k += nthreads) {
        float mv = -INFINITY;
        if (k < S) {
            mv = to_f32(p.bias[(int64_t)b * p.bias_sb + k]) * LOG2E;
            if (mv != 0.f) {
                atomicOr(&tile_flag[k >> 5], 1);
            }
        }
        mask[k] = mv;
    }

    // ---- projections, in groups of GW weight matrices staged through LDS ----
    bf16x8 qf[BPW][2];   // Q^T fragments (B operand of the logits MFMA), scaled by log2(e)/sqrt(d)
    bf16x8 gate[BPW][2]; // sigmoid(gate) in accumulator order, packed
    const int npass = 4 / GW;
    for (int pass = 0; pass < npass; ++pass) {
        __syncthreads(); // previous group's fragments are no longer being read
        for (int idx = tid; idx < GW * CK * 64; idx += nthreads) {
            const int mm = idx / (CK * 64);
            const int ks = (idx >> 6) % CK;
            const int ln = idx & 63;
            const bf16_t *src = p.w[pass * GW + mm] + (int64_t)(h * HEAD + (ln & 31)) * C + ks * 16 + (ln >> 5) * 8;
            lds_w[idx] = *reinterpret_cast<const uint4 *>(src);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < BPW; ++i) {
            const int j = wave + i * NW;
            if (j >= NB) {
                continue;
            }
            int srow = j * 32 + pi_row(r);
            srow = srow < S ? srow : S - 1; // rows past the end repeat the last row; they are never stored
            const bf16_t *xrow = p.x + ((int64_t)b * S + srow) * p.x_ld + g * 8;
            bf16x8 xf[CK];
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                xf[ks] = as_bf16x8(*reinterpret_cast<const uint4 *>(xrow + ks * 16));
            }
            for (int mm = 0; mm < GW; ++mm) {
                const int m = pass * GW + mm;
                const uint4 *wsrc = lds_w + mm * CK * 64 + lane;
                f32x16 acc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                if (m == PROJ_V) {
                    // V[s][d]: rows = sequence positions, so a lane ends up with 16 keys of one head-dim
#pragma unroll
                    for (int ks = 0; ks < CK; ++ks) {
                        acc = mfma(xf[ks], as_bf16x8(wsrc[ks * 64]), acc);
                    }
                    lds_v[(j * 2 + 0) * 64 + lane] = as_uint4(pack8(acc, 0));
                    lds_v[(j * 2 + 1) * 64 + lane] = as_uint4(pack8(acc, 8));
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
                            acc[v] *= p.qscale;
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
                                const float gv = acc[4 * a + c] + bv[c];
                                acc[4 * a + c] = 1.0f / (1.0f + __builtin_amdgcn_exp2f(-gv * LOG2E));
                            }
                        }
                        gate[i][0] = pack8(acc, 0);
                        gate[i][1] = pack8(acc, 8);
                    }
                }
            }
        }
    }
    __syncthreads(); // K and V of the whole sequence are in LDS

    // ---- attention: each wave walks the key tiles for its own query blocks ----
#pragma unroll
    for (int i = 0; i < BPW; ++i) {
        const int j = wave + i * NW;
        if (j >= NB) {
            continue;
        }
        const int qpos = j * 32 + pi_row(r);
        const int qrow = qpos < S ? qpos : S - 1;
        const bf16_t *nbrow = p.nb ? p.nb + (int64_t)h * p.nb_sh + (int64_t)qrow * p.nb_sq + 16 * g : nullptr;
        f32x16 o = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float m_run = -1e30f; // finite, so the first rescale factor is exp2(-huge) = 0, never NaN
        float lsum = 0.f;     // this lane's share of the row sum; the two halves are added at the end
        for (int t = 0; t < NB; ++t) {
            f32x16 x;
            const bool ragged = (t + 1) * 32 > S;
            if (nbrow != nullptr) {
                if (p.nb_vec && !ragged) {
                    const uint4 lo = *reinterpret_cast<const uint4 *>(nbrow + t * 32);
                    const uint4 hi = *reinterpret_cast<const uint4 *>(nbrow + t * 32 + 8);
                    const uint32_t wds[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
                    for (int v = 0; v < 8; ++v) {
                        x[2 * v] = __uint_as_float(wds[v] << 16) * LOG2E;
                        x[2 * v + 1] = __uint_as_float(wds[v] & 0xffff0000u) * LOG2E;
                    }
                } else {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int key = t * 32 + 16 * g + v;
                        x[v] = key < S ? to_f32(nbrow[t * 32 + v]) * LOG2E : 0.f;
                    }
                }
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    x[v] = 0.f;
                }
            }
            if (tile_flag[t]) {
                const f32x4 *mp = reinterpret_cast<const f32x4 *>(mask + t * 32 + 16 * g);
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 mv = mp[a];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        x[4 * a + c] += mv[c];
                    }
                }
            }
            // logits^T tile: rows = keys of tile t, columns = this wave's 32 queries
            x = mfma(as_bf16x8(lds_k[(t * 2 + 0) * 64 + lane]), qf[i][0], x);
            x = mfma(as_bf16x8(lds_k[(t * 2 + 1) * 64 + lane]), qf[i][1], x);

            float mx = x[0];
#pragma unroll
            for (int v = 1; v < 16; ++v) {
                mx = fmaxf(mx, x[v]);
            }
            mx = half_swap_max(mx);
            if (__any(mx > m_run + RESCALE_GAP)) {
                const float m_new = fmaxf(m_run, mx);
                const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
                lsum *= alpha;
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    o[v] *= alpha;
                }
                m_run = m_new;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                x[v] = __builtin_amdgcn_exp2f(x[v] - m_run);
                lsum += x[v];
            }
            // weighted sum: O^T[d][q] += V^T[d][keys] . P[keys][q]; P goes straight from registers
            o = mfma(as_bf16x8(lds_v[(t * 2 + 0) * 64 + lane]), pack8(x, 0), o);
            o = mfma(as_bf16x8(lds_v[(t * 2 + 1) * 64 + lane]), pack8(x, 8), o);
        }
        const float inv = 1.0f / half_swap_sum(lsum);
        if (qpos < S) {
            bf16_t *dst = p.avg + (int64_t)b * p.avg_sb + (int64_t)qpos * p.avg_ss + (int64_t)h * p.avg_sh + 4 * g;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                bf16x4 ov;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int v = 4 * a + c;
                    const float gv = to_f32(gate[i][v >> 3][v & 7]);
                    ov[c] = (bf16_t)(o[v] * inv * gv);
                }
                *reinterpret_cast<bf16x4 *>(dst + 8 * a) = ov;
            }
        }
    }
}

// out[t][o] = sum_c avg[t][c] * Wo[o][c] + bo[o].  Computed transposed (rows = output features,
// columns = tokens) so that each lane owns one token row and stores 4 consecutive features at a time.
// One workgroup stages the fragments of a 128-feature slab of Wo in LDS and walks row tiles.
template <int C>
__global__ __launch_bounds__(256) void output_projection_kernel(const bf16_t *__restrict__ avg, int64_t avg_ld,
                                                                const bf16_t *__restrict__ wo,
                                                                const float *__restrict__ bo, bf16_t *__restrict__ out,
                                                                int64_t out_ld, int64_t M, int tiles_per_wg)
{
    constexpr int CK = C / 16;
    constexpr int NSLAB = 128;
    extern __shared__ uint4 lds[]; // [4 row blocks of 32 features][CK][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int n0 = blockIdx.y * NSLAB;
    for (int idx = tid; idx < 4 * CK * 64; idx += 256) {
        const int nb_ = idx / (CK * 64);
        const int ks = (idx >> 6) % CK;
        const int ln = idx & 63;
        const bf16_t *src = wo + (int64_t)(n0 + nb_ * 32 + (ln & 31)) * C + ks * 16 + (ln >> 5) * 8;
        lds[idx] = *reinterpret_cast<const uint4 *>(src);
    }
    __syncthreads();
    const int64_t tile0 = (int64_t)blockIdx.x * tiles_per_wg;
    for (int tt = wave; tt < tiles_per_wg; tt += 4) {
        const int64_t row0 = (tile0 + tt) * 32;
        if (row0 >= M) {
            break;
        }
        int64_t row = row0 + r;
        const bool live = row < M;
        row = live ? row : M - 1;
        const bf16_t *arow = avg + row * avg_ld + g * 8;
        f32x16 acc[4];
#pragma unroll
        for (int n = 0; n < 4; ++n) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                acc[n][v] = 0.f;
            }
        }
#pragma unroll
        for (int ks = 0; ks < CK; ++ks) {
            const bf16x8 af = as_bf16x8(*reinterpret_cast<const uint4 *>(arow + ks * 16));
#pragma unroll
            for (int n = 0; n < 4; ++n) {
                acc[n] = mfma(as_bf16x8(lds[(n * CK + ks) * 64 + lane]), af, acc[n]);
            }
        }
        if (live) {
            bf16_t *orow = out + row * out_ld + n0 + 4 * g;
            const float *brow = bo + n0 + 4 * g;
#pragma unroll
            for (int n = 0; n < 4; ++n) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(brow + n * 32 + 8 * a);
                    bf16x4 ov;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        ov[c] = (bf16_t)(acc[n][4 * a + c] + bv[c]);
                    }
                    *reinterpret_cast<bf16x4 *>(orow + n * 32 + 8 * a) = ov;
                }
            }
        }
    }
}

struct Plan {
    int NB, NW, BPW, GW;
    size_t lds_bytes;
};

int max_lds_bytes()
{
    static int cached = -1;
    if (cached < 0) {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess) {
            (void)hipGetLastError();
            v = 64 * 1024;
        }
        cached = v;
    }
    return cached;
}

size_t head_kernel_lds(int C, int NB, int GW)
{
    return (size_t)GW * (C / 16) * 64 * 16 + (size_t)NB * 2 * 64 * 16 * 2 + (size_t)NB * 32 * 4 + (size_t)NB * 4;
}

bool make_plan(int64_t S, int C, Plan &pl)
{
    const int64_t NB = (S + 31) / 32;
    if (NB > 32) {
        return false;
    }
    pl.NB = (int)NB;
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
    const size_t cap = (size_t)max_lds_bytes();
    for (int gw = 4; gw >= 1; gw >>= 1) {
        const size_t need = head_kernel_lds(C, pl.NB, gw);
        if (need <= cap) {
            pl.GW = gw, pl.lds_bytes = need;
            return true;
        }
    }
    return false;
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

template <int C, int BPW>
int launch_head_kernel(const FusedParams &p, const Plan &pl, hipStream_t stream)
{
    auto kern = fused_head_kernel<C, BPW>;
    static size_t configured = 0; // per instantiation: largest dynamic LDS size opted into so far
    if (pl.lds_bytes > configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)pl.lds_bytes);
        if (e != hipSuccess) {
            return (int)e;
        }
        configured = pl.lds_bytes;
    }
    const int64_t units = ((int64_t)(p.B + 7) / 8) * 8 * p.H;
    kern<<<dim3((unsigned)units), dim3((unsigned)(pl.NW * 64)), pl.lds_bytes, stream>>>(p);
    return kutacc_hip_status(hipGetLastError());
}

template <int C>
int dispatch_head_kernel(const FusedParams &p, const Plan &pl, hipStream_t stream)
{
    switch (pl.BPW) {
        case 1: return launch_head_kernel<C, 1>(p, pl, stream);
        case 2: return launch_head_kernel<C, 2>(p, pl, stream);
        case 3: return launch_head_kernel<C, 3>(p, pl, stream);
        case 4: return launch_head_kernel<C, 4>(p, pl, stream);
        default: return KUTACC_HIP_EUNSUPPORTED;
    }
}

template <int C>
int launch_output_projection(const kutacc_hip_attention_args_t &a, hipStream_t stream)
{
    auto kern = output_projection_kernel<C>;
    const size_t lds_bytes = (size_t)4 * (C / 16) * 64 * 16;
    static bool configured = false;
    if (!configured) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);
        if (e != hipSuccess) {
            return (int)e;
        }
        configured = true;
    }
    const int64_t M = a.batch * a.seq_len;
    const int64_t tiles = (M + 31) / 32;
    const int tiles_per_wg = 16;
    const int64_t gx = (tiles + tiles_per_wg - 1) / tiles_per_wg;
    kern<<<dim3((unsigned)gx, (unsigned)(C / 128)), 256, lds_bytes, stream>>>(
        (const bf16_t *)a.avg, a.avg_stride_s, (const bf16_t *)a.output_w, a.output_b, (bf16_t *)a.out, a.out_ld, M,
        tiles_per_wg);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace

namespace kutacc_launch {

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
    // 16-byte row loads of input and weights, 8-byte stores of avg/out rows
    if (a.input_ld % 8 != 0 || !aligned(a.input, 16) || !aligned(a.query_w, 16) || !aligned(a.key_w, 16) ||
        !aligned(a.value_w, 16) || !aligned(a.gating_w, 16) || !aligned(a.output_w, 16) || !aligned(a.gating_b, 16) ||
        !aligned(a.output_b, 16)) {
        return false;
    }
    if (a.avg_stride_h != HEAD || a.avg_stride_s % 8 != 0 || a.avg_stride_b != a.seq_len * a.avg_stride_s ||
        !aligned(a.avg, 16) || a.out_ld % 4 != 0 || !aligned(a.out, 8)) {
        return false;
    }
    Plan pl;
    return make_plan(a.seq_len, (int)C, pl);
}

int gating_attention_fused(const kutacc_hip_attention_args_t &a, hipStream_t stream)
{
    const int C = (int)(a.nheads * a.head_size);
    Plan pl;
    if (!make_plan(a.seq_len, C, pl)) {
        return KUTACC_HIP_EUNSUPPORTED;
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
    p.avg_sb = a.avg_stride_b, p.avg_ss = a.avg_stride_s, p.avg_sh = a.avg_stride_h;
    p.B = (int)a.batch, p.S = (int)a.seq_len, p.H = (int)a.nheads, p.NB = pl.NB, p.NW = pl.NW, p.GW = pl.GW;
    p.nb_vec = (p.nb != nullptr && aligned(p.nb, 16) && a.nb_stride_h % 8 == 0 && a.nb_stride_q % 8 == 0) ? 1 : 0;
    // (float)(1/sqrt(head_size)) as the reference forms it (gating_attention.cpp:68), times log2(e)
    p.qscale = (float)(1.0 / sqrt((double)a.head_size)) * LOG2E;

    const double BS = (double)a.batch * (double)a.seq_len;
    int rc;
    {
        kutacc_prof::KernelTimer t("fused_head_kernel", 8.0 * BS * C * C + 4.0 * BS * (double)a.seq_len * C, stream);
        rc = (C == 128) ? dispatch_head_kernel<128>(p, pl, stream) : dispatch_head_kernel<256>(p, pl, stream);
        if (rc != 0) {
            return rc;
        }
    }
    kutacc_prof::KernelTimer t("output_projection_kernel", 2.0 * BS * C * C, stream);
    return (C == 128) ? launch_output_projection<128>(a, stream) : launch_output_projection<256>(a, stream);
}

} // namespace kutacc_launch
