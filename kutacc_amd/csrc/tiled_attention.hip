// Gated attention for the bf16 shapes the fused head kernels do not take: any sequence length, head sizes that are
// multiples of 8 up to 64, any number of channels.  The data flow is the reference's own (reference
// src/attention/gating_attention.cpp:47-66, 73-150, 152-157): four projections into the caller's q, k, v and gate
// tensors (v transposed to [channels, batch * seq_len], the gate with its bias), attention per (batch row, head) with
// the sigmoid gate applied to the weighted average, output projection -- so this route also leaves the scratch
// tensors as the reference's kernel does.  The projections run on the strided MFMA GEMM of the pair stack; the
// attention is the kernel below: MFMA products for q.k and p.v, softmax in fp32 (unshifted in log2 units where a row's
// sums allow it, with a running maximum where they do not), keys streamed through LDS in chunks of 64, so that the
// logits of a row never exist and nothing depends on the row's length.
//
// Rounding points: q, k, v, gate as bf16 in memory (the reference's), logits
// x = (q.k * scale + bias[b, key]) + nonbatched_bias[h, query, key] in fp32 with that association
// (gating_attention.cpp:109-118), probabilities in fp32 (rounded to bf16 as MFMA operands of p.v, their sum taken in
// fp32), weighted average rounded to bf16 before the gate multiplies it and once more after (:128-145).
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <type_traits>

#include "device_util.h"
#include "launch_internal.h"
#include "mfma_tiles.h"
#include "profiler.h"

namespace {
using namespace kutacc_dev;

struct TileParams {
    const bf16_t *q, *k, *v, *gate, *bias, *nb;
    bf16_t *avg;
    int64_t q_sb, q_ss, q_sh;
    int64_t k_sb, k_ss, k_sh;
    int64_t g_sb, g_ss, g_sh;
    int64_t a_sb, a_ss, a_sh;
    int64_t v_se, v_sb; // v[(h * hd + e) * v_se + b * v_sb + key]
    int64_t bias_sb, nb_sh, nb_sq;
    int B, S, H, hd;
    int groups, groups_q, query_blocks; // placement of workgroups, below
    int v_vec, nb_vec;                  // rows of v / of the pair bias can be read 16 bytes at a time
    float scale;
};

constexpr int QUERIES = 128; // per workgroup: four waves of 32
constexpr int CHUNK = 64;    // keys per LDS stage
constexpr int GROUP_ROWS = 8, GROUP_QBLOCKS = 8;

// The logits MFMA puts key (row) i of a 32-key block into accumulator register 4 a + c of lane half g with
// i = 8 a + 4 g + c.  The p.v MFMA wants, per lane half and k-step of 16 keys, 8 consecutive keys in 8 consecutive
// registers.  Both hold if row i of the K fragment is key swap23(i) of the block (bits 2 and 3 of the index exchanged):
// register 8 j + e of lane half g is then key 16 j + 8 g + e.
__device__ __forceinline__ int swap23(int i) { return (i & ~12) | ((i & 4) << 1) | ((i & 8) >> 1); }

__device__ __forceinline__ uint4 zero_u4() { return make_uint4(0u, 0u, 0u, 0u); }

// eight bf16 at src[0 .. 7]; elements from `valid` on are zero (never read)
__device__ __forceinline__ uint4 load8_checked(const bf16_t *src, int valid)
{
    union {
        uint4 u;
        bf16_t e[8];
    } c;
    c.u = zero_u4();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (i < valid) {
            c.e[i] = src[i];
        }
    }
    return c.u;
}

// acc + the sum of eight bf16: four dot products of a pair with (1, 1)
__device__ __forceinline__ float pair_sums(bf16x8 v, float acc)
{
    typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
    const pair_t ones = {(__bf16)1.0f, (__bf16)1.0f};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const pair_t pr = {v[2 * i], v[2 * i + 1]};
        acc = __builtin_amdgcn_fdot2_f32_bf16(pr, ones, acc, false);
    }
    return acc;
}

// KS: k-steps of 16 of the q.k product (head_size <= 16 KS, zero padded); the head's values span DB = ceil(KS / 2)
// blocks of 32 MFMA rows.
//
// One workgroup = 128 queries of one (batch row, head): wave w owns queries 32 w .. 32 w + 31, keeps their q fragments,
// running sum (and maximum, in the second pass) and the head_size x 32 accumulator of p.v in registers, and walks all keys.  The
// workgroup stages each chunk of 64 keys once (K in fragment order with the row permutation above, V^T as it lies in
// the caller's tensor: key-contiguous rows, which is the fragment order of the p.v product; mask bias as fp32, -inf
// for keys past the end, which is all the handling a ragged length needs), two stages, one barrier per chunk; the
// pair bias is per (query, key): each lane fetches its own query's keys into registers, one chunk ahead.
//
// Placement: workgroup ids are dealt round robin over the 8 XCDs; the id is decoded so that each XCD works on groups of
// 8 batch rows x 8 query blocks of one head at a time.  The 64 workgroups of a group sweep the keys roughly together,
// so the group's K/V (8 rows) and pair bias (8 query blocks) come from HBM once and from the XCD's L2 seven times.
template <int KS, bool HAS_NB>
__global__ __launch_bounds__(256, 2) void attention_tiles_kernel(const TileParams p)
{
    constexpr int DB = (KS + 1) / 2;
    constexpr int K_SLOTS = 2 * KS * 64, V_SLOTS = DB * 4 * 64, STAGE_SLOTS = K_SLOTS + V_SLOTS + CHUNK / 4;
    constexpr int K_PIECES = CHUNK * 2 * KS, PK = (K_PIECES + 255) / 256; // 16-byte pieces of a K chunk, per thread
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;

    const uint32_t bid = blockIdx.x;
    const int group = (int)(bid >> 9) * 8 + (int)(bid & 7), member = (int)(bid >> 3) & 63;
    if (group >= p.groups) {
        return;
    }
    const int h = group % p.H;
    const int b = ((group / p.H) / p.groups_q) * GROUP_ROWS + (member & 7);
    const int qb = ((group / p.H) % p.groups_q) * GROUP_QBLOCKS + (member >> 3);
    if (b >= p.B || qb >= p.query_blocks) {
        return;
    }
    const int S = p.S, hd = p.hd;
    const int q0 = qb * QUERIES + wave * 32;
    const bool active = q0 < S; // a wave past the end only helps staging
    const int query = q0 + r < S ? q0 + r : S - 1;

    bf16x8 qf[KS];
    {
        const bf16_t *qp = p.q + (int64_t)b * p.q_sb + (int64_t)query * p.q_ss + (int64_t)h * p.q_sh;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const int d0 = 16 * ks + 8 * g;
            qf[ks] = as_bf16x8(d0 < hd ? *reinterpret_cast<const uint4 *>(qp + d0) : zero_u4());
        }
    }
    const bf16_t *kbase = p.k + (int64_t)b * p.k_sb + (int64_t)h * p.k_sh;
    const bf16_t *vbase = p.v + (int64_t)h * hd * p.v_se + (int64_t)b * p.v_sb;
    const bf16_t *bias_row = p.bias + (int64_t)b * p.bias_sb;
    const bf16_t *nb_row = HAS_NB ? p.nb + (int64_t)h * p.nb_sh + (int64_t)query * p.nb_sq : nullptr;

    // What a thread stages of every chunk: PK 16-byte pieces of K (key kap, values 8 o .. 8 o + 7 of the head) and DB of
    // V^T (value d, keys 8 ko .. 8 ko + 7 of the chunk); pieces that lie in the padding are stored as zeros.
    int k_kap[PK], k_slot[PK], v_slot[DB];
    int64_t k_off[PK], v_off[DB];
    bool k_real[PK], v_real[DB];
#pragma unroll
    for (int i = 0; i < PK; ++i) {
        const int idx = tid + 256 * i;
        const int o = idx % (2 * KS), kap = (idx / (2 * KS)) % CHUNK;
        k_kap[i] = kap;
        k_real[i] = 8 * o < hd; // (an index past the last piece repeats piece idx - K_PIECES: same data, same slot)
        k_off[i] = k_real[i] ? 8 * o : 0;
        k_slot[i] = ((kap >> 5) * KS + (o >> 1)) * 64 + swap23(kap & 31) + 32 * (o & 1);
    }
#pragma unroll
    for (int i = 0; i < DB; ++i) {
        const int idx = tid + 256 * i;
        const int d = idx >> 3, ko = idx & 7;
        v_real[i] = d < hd;
        v_off[i] = (int64_t)(v_real[i] ? d : 0) * p.v_se + 8 * ko;
        v_slot[i] = K_SLOTS + ((d >> 5) * 4 + (ko >> 1)) * 64 + (d & 31) + 32 * (ko & 1);
    }
    auto keep = [](uint4 v, bool ok) { // a select, not a branch around the load
        const uint32_t m = ok ? 0xffffffffu : 0u;
        return make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
    };
    // Two forms of the loads of a chunk.  PLAIN: every key of the chunk exists and every row can be read 16 bytes at a
    // time -- no condition anywhere (a thread without a piece of its own repeats another thread's, to the same slot), so
    // that the loop made of such chunks is one basic block per phase and the loads stay in flight across the compute
    // phase.  Otherwise: the checked form (clamped rows, element-wise reads past alignment or the end).  Nothing touches
    // what a load returns before park(): a use right behind the load makes the wave wait out the memory latency.
    uint4 kreg[PK], vreg[DB];
    bool k_keep[PK];
    bf16_t bias_raw = (bf16_t)0.f;
    bool bias_keep = false;
    auto fetch = [&](int c, auto plain_tag) {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        const int kc0 = c * CHUNK;
#pragma unroll
        for (int i = 0; i < PK; ++i) {
            const int key = kc0 + k_kap[i], key_c = PLAIN || key < S ? key : S - 1;
            kreg[i] = *reinterpret_cast<const uint4 *>(kbase + (int64_t)key_c * p.k_ss + k_off[i]);
            k_keep[i] = k_real[i] && (PLAIN || key < S);
        }
        if constexpr (PLAIN) {
#pragma unroll
            for (int i = 0; i < DB; ++i) {
                vreg[i] = *reinterpret_cast<const uint4 *>(vbase + v_off[i] + kc0);
            }
            bias_raw = bias_row[kc0 + (tid & (CHUNK - 1))];
            bias_keep = true;
        } else {
#pragma unroll
            for (int i = 0; i < DB; ++i) {
                const int key = kc0 + 8 * ((tid + 256 * i) & 7);
                vreg[i] = zero_u4();
                if (v_real[i] && key < S) {
                    const bf16_t *src = vbase + v_off[i] + kc0;
                    vreg[i] = (p.v_vec && key + 8 <= S) ? *reinterpret_cast<const uint4 *>(src) : load8_checked(src, S - key);
                }
            }
            const int key = kc0 + (tid & (CHUNK - 1));
            bias_raw = bias_row[key < S ? key : S - 1];
            bias_keep = key < S;
        }
    };
    auto park = [&](uint4 *stage) {
#pragma unroll
        for (int i = 0; i < PK; ++i) {
            stage[k_slot[i]] = keep(kreg[i], k_keep[i]);
        }
#pragma unroll
        for (int i = 0; i < DB; ++i) {
            stage[v_slot[i]] = keep(vreg[i], v_real[i]); // (the element-wise form has zeroed what it must already)
        }
        reinterpret_cast<float *>(stage + K_SLOTS + V_SLOTS)[tid & (CHUNK - 1)] = bias_keep ? to_f32(bias_raw) * LOG2E : -INFINITY;
    };
    // Pair bias of this lane's query for the keys of chunk c, in accumulator order: [key block][j] holds keys
    // 32 kb + 16 j + 8 g .. + 7.  Straight from global memory into registers: a load instruction touches 32 rows, a quarter
    // of a cache line each, and the other three loads touch the same lines again.  (Whole 128-byte rows through a
    // wave-private LDS panel, read back in this order, measured the same and cost 8 KB of LDS traffic per wave and chunk.)
    struct NbRegs {
        uint4 v[2][2];
    };
    auto fetch_nb = [&](int c, auto plain_tag) -> NbRegs {
        constexpr bool PLAIN = decltype(plain_tag)::value;
        NbRegs f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                f.v[kb][j] = zero_u4();
                if constexpr (HAS_NB) {
                    const int key = c * CHUNK + 32 * kb + 16 * j + 8 * g;
                    if constexpr (PLAIN) {
                        f.v[kb][j] = *reinterpret_cast<const uint4 *>(nb_row + key);
                    } else if (key < S) {
                        f.v[kb][j] = (p.nb_vec && key + 8 <= S) ? *reinterpret_cast<const uint4 *>(nb_row + key)
                                                                : load8_checked(nb_row + key, S - key);
                    }
                }
            }
        }
        return f;
    };

    f32x16 oacc[DB];
    float m_run, l_run; // running maximum (log2 units; SAFE only) and this lane's share of the sum (its half of the keys)
    const int chunks = (S + CHUNK - 1) / CHUNK;
    const float scale2 = p.scale * LOG2E;
    // One pass over all keys.  Everything is in log2 units: x = q.k * (scale * log2 e) + bias * log2 e + nb * log2 e,
    // p = 2^x.  The fast pass takes 2^x as it stands -- a softmax does not depend on a common shift, and fp32 and bf16
    // hold 2^-126 .. 2^127 -- and the caller checks the sums afterwards; the SAFE pass keeps a running maximum and
    // serves the rows the fast one could not (logits beyond that range, rows with every key masked).
    auto sweep = [&](auto safe_tag) {
        constexpr bool SAFE = decltype(safe_tag)::value;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            oacc[db] = zero16();
        }
        m_run = -INFINITY, l_run = 0.f;
        NbRegs nb_cur, nb_next;
        // chunks [0, plain) take the PLAIN loads
        const int plain = (p.v_vec && (!HAS_NB || p.nb_vec)) ? S / CHUNK : 0;
        if (plain > 0) {
            fetch(0, std::true_type{});
            nb_cur = fetch_nb(0, std::true_type{});
        } else {
            fetch(0, std::false_type{});
            nb_cur = fetch_nb(0, std::false_type{});
        }
        park(lds);
        __syncthreads();
        // chunk c from its stage, with the loads of chunk c + 1 (if `more`) in flight meanwhile
        auto step = [&](int c, bool more, auto plain_tag) {
            const uint4 *stage = lds + (c & 1) * STAGE_SLOTS;
            if (more) {
                fetch(c + 1, plain_tag);
                nb_next = fetch_nb(c + 1, plain_tag);
            }
            if (active) {
                const float *mask_bias = reinterpret_cast<const float *>(stage + K_SLOTS + V_SLOTS);
                f32x16 x[2];
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    x[kb] = zero16();
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) {
                        x[kb] = mfma(as_bf16x8(stage[(kb * KS + ks) * 64 + lane]), qf[ks], x[kb]);
                    }
                }
                float mx = -INFINITY;
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const f32x4 b0 = *reinterpret_cast<const f32x4 *>(mask_bias + 32 * kb + 16 * j + 8 * g);
                        const f32x4 b1 = *reinterpret_cast<const f32x4 *>(mask_bias + 32 * kb + 16 * j + 8 * g + 4);
                        const bf16x8 nbv = as_bf16x8(nb_cur.v[kb][j]);
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            float v = fmaf(x[kb][8 * j + e], scale2, e < 4 ? b0[e & 3] : b1[e & 3]);
                            if constexpr (HAS_NB) {
                                v = fmaf(to_f32(nbv[e]), LOG2E, v);
                            }
                            x[kb][8 * j + e] = v;
                            if constexpr (SAFE) {
                                mx = fmaxf(mx, v);
                            }
                        }
                    }
                }
                float m_ref = 0.f;
                if constexpr (SAFE) {
                    const float m_new = fmaxf(m_run, half_swap_max(mx));
                    // every key so far at -inf: any finite reference point keeps the arithmetic free of inf - inf
                    m_ref = m_new == -INFINITY ? 0.f : m_new;
                    if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
                        const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
                        l_run *= alpha;
#pragma unroll
                        for (int db = 0; db < DB; ++db) {
#pragma unroll
                            for (int v = 0; v < 16; ++v) {
                                oacc[db][v] *= alpha;
                            }
                        }
                        m_run = m_new;
                    }
                }
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        // SAFE: (x - m) is exact where x = m, whatever their size (a masked row sits at -1.4e9)
                        x[kb][v] = __builtin_amdgcn_exp2f(SAFE ? x[kb][v] - m_ref : x[kb][v]);
                    }
                    const bf16x8 p0 = pack8(x[kb], 0), p1 = pack8(x[kb], 8);
                    l_run = pair_sums(p0, pair_sums(p1, l_run)); // of the rounded values, the ones p.v multiplies
#pragma unroll
                    for (int db = 0; db < DB; ++db) {
                        oacc[db] = mfma(as_bf16x8(stage[K_SLOTS + (db * 4 + 2 * kb) * 64 + lane]), p0, oacc[db]);
                        oacc[db] = mfma(as_bf16x8(stage[K_SLOTS + (db * 4 + 2 * kb + 1) * 64 + lane]), p1, oacc[db]);
                    }
                }
            }
            if (more) {
                park(lds + ((c + 1) & 1) * STAGE_SLOTS); // its last readers passed the barrier that ended the previous chunk
                nb_cur = nb_next;
            }
            __syncthreads();
        };
        int c = 0;
        for (; c + 1 < plain; ++c) {
            step(c, true, std::true_type{});
        }
        for (; c < chunks; ++c) {
            step(c, c + 1 < chunks, std::false_type{});
        }
        l_run = half_swap_sum(l_run);
    };
    sweep(std::false_type{});
    // a sum outside [1e-30, 1e30] (or not a number): the row's logits left the range in which 2^x and the products with
    // v are safe in fp32, or every key is masked.  The keys are staged by the whole workgroup, so it repeats as one.
    const bool fast_failed = active && q0 + r < S && !(l_run >= 1e-30f && l_run <= 1e30f);
    if (__syncthreads_or(fast_failed ? 1 : 0)) {
        sweep(std::true_type{});
    }
    if (!active || q0 + r >= S) {
        return;
    }
    // weighted average -> bf16, x sigmoid(gate) -> bf16; register 4 a + c of lane half g is value 32 db + 8 a + 4 g + c
    const float inv = 1.0f / l_run;
    const int64_t row = (int64_t)(q0 + r);
    const bf16_t *gp = p.gate + (int64_t)b * p.g_sb + row * p.g_ss + (int64_t)h * p.g_sh;
    bf16_t *ap = p.avg + (int64_t)b * p.a_sb + row * p.a_ss + (int64_t)h * p.a_sh;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int d0 = 32 * db + 8 * a + 4 * g;
            if (d0 < hd) {
                const bf16x4 gv = *reinterpret_cast<const bf16x4 *>(gp + d0);
                bf16x4 ov;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float wavg = to_f32((bf16_t)(oacc[db][4 * a + c] * inv));
                    ov[c] = (bf16_t)(wavg * sigmoid_f32(to_f32(gv[c])));
                }
                *reinterpret_cast<bf16x4 *>(ap + d0) = ov;
            }
        }
    }
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int KS, bool HAS_NB>
hipError_t launch_tiles(const TileParams &p, int64_t blocks, hipStream_t stream)
{
    constexpr int DB = (KS + 1) / 2;
    constexpr size_t lds_bytes = 2 * (2 * KS * 64 + DB * 4 * 64 + CHUNK / 4) * 16;
    static_assert(lds_bytes <= 64 * 1024, "two stages fit the LDS a kernel may use without opting in");
    attention_tiles_kernel<KS, HAS_NB><<<dim3((unsigned)blocks), 256, lds_bytes, stream>>>(p);
    return hipGetLastError();
}

int project(const void *a, int64_t a_sm, int64_t m, const void *b, int64_t b_sn, int64_t n, int64_t k, void *c, int64_t c_sm,
            const float *bias, hipStream_t stream)
{
    kutacc_hip_gemm_args_t g = {};
    g.m = m, g.n = n, g.k = k, g.batches = 1;
    g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_AUTO;
    g.a = a, g.a_stride_m = a_sm, g.a_stride_k = 1, g.a_stride_batch = 0;
    g.b = b, g.b_stride_n = b_sn, g.b_stride_k = 1, g.b_stride_batch = 0;
    g.c = c, g.c_stride_m = c_sm, g.c_stride_batch = 0;
    g.bias = bias, g.bias_axis = bias ? 1 : 0;
    return kutacc_launch::pair_gemm(g, stream);
}

} // namespace

namespace kutacc_launch {

bool tiled_attention_supports(const kutacc_hip_attention_args_t &a)
{
    if (a.dtype != KUTACC_DTYPE_BF16 || a.head_size % 8 != 0 || a.head_size > 64 || a.batch <= 0 || a.seq_len <= 0 || a.nheads <= 0) {
        return false;
    }
    if (!a.q || !a.k || !a.v || !a.gate || !a.avg) {
        return false;
    }
    const int64_t S = a.seq_len, hd = a.head_size, M = a.batch * S;
    // q, k, gate and avg as [batch * seq_len, channels] matrices and v as [channels, batch * seq_len], the views the
    // reference hands to its GEMMs (gating_attention.cpp:50, 55, 60, 65, 153)
    if (a.q_stride_b != S * a.q_stride_s || a.k_stride_b != S * a.k_stride_s || a.gate_stride_b != S * a.gate_stride_s ||
        a.avg_stride_b != S * a.avg_stride_s || a.q_stride_h != hd || a.k_stride_h != hd || a.gate_stride_h != hd ||
        a.avg_stride_h != hd || a.v_stride_h != hd * a.v_stride_e || a.v_stride_b != S || a.v_stride_e < M) {
        return false;
    }
    // 16-byte loads of q and k rows, 8-byte loads of gate rows and stores of avg rows
    if (a.q_stride_s % 8 != 0 || a.k_stride_s % 8 != 0 || a.gate_stride_s % 4 != 0 || a.avg_stride_s % 4 != 0 || !aligned16(a.q) ||
        !aligned16(a.k) || !aligned16(a.gate) || !aligned16(a.avg)) {
        return false;
    }
    const int64_t query_blocks = (S + QUERIES - 1) / QUERIES;
    const int64_t groups = a.nheads * ((a.batch + GROUP_ROWS - 1) / GROUP_ROWS) * ((query_blocks + GROUP_QBLOCKS - 1) / GROUP_QBLOCKS);
    return S <= (1 << 24) && a.batch <= (1 << 24) && (groups + 7) / 8 * 8 * 64 <= INT32_MAX;
}

int gating_attention_tiled(const kutacc_hip_attention_args_t &a, hipStream_t stream)
{
    if (!tiled_attention_supports(a)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    const int64_t B = a.batch, S = a.seq_len, H = a.nheads, hd = a.head_size, C = H * hd, M = B * S;
    int rc;
    if ((rc = project(a.input, a.input_ld, M, a.query_w, C, C, C, a.q, a.q_stride_s, nullptr, stream)) ||
        (rc = project(a.input, a.input_ld, M, a.key_w, C, C, C, a.k, a.k_stride_s, nullptr, stream)) ||
        (rc = project(a.value_w, C, C, a.input, a.input_ld, M, C, a.v, a.v_stride_e, nullptr, stream)) ||
        (rc = project(a.input, a.input_ld, M, a.gating_w, C, C, C, a.gate, a.gate_stride_s, a.gating_b, stream))) {
        return rc;
    }
    TileParams p;
    p.q = (const bf16_t *)a.q, p.k = (const bf16_t *)a.k, p.v = (const bf16_t *)a.v, p.gate = (const bf16_t *)a.gate;
    p.bias = (const bf16_t *)a.bias, p.nb = (const bf16_t *)a.nonbatched_bias, p.avg = (bf16_t *)a.avg;
    p.q_sb = a.q_stride_b, p.q_ss = a.q_stride_s, p.q_sh = a.q_stride_h;
    p.k_sb = a.k_stride_b, p.k_ss = a.k_stride_s, p.k_sh = a.k_stride_h;
    p.g_sb = a.gate_stride_b, p.g_ss = a.gate_stride_s, p.g_sh = a.gate_stride_h;
    p.a_sb = a.avg_stride_b, p.a_ss = a.avg_stride_s, p.a_sh = a.avg_stride_h;
    p.v_se = a.v_stride_e, p.v_sb = a.v_stride_b;
    p.bias_sb = a.bias_stride_b, p.nb_sh = a.nb_stride_h, p.nb_sq = a.nb_stride_q;
    p.B = (int)B, p.S = (int)S, p.H = (int)H, p.hd = (int)hd;
    p.query_blocks = (int)((S + QUERIES - 1) / QUERIES);
    p.groups_q = (p.query_blocks + GROUP_QBLOCKS - 1) / GROUP_QBLOCKS;
    p.groups = (int)(H * ((B + GROUP_ROWS - 1) / GROUP_ROWS) * p.groups_q);
    p.v_vec = (aligned16(a.v) && a.v_stride_e % 8 == 0 && a.v_stride_b % 8 == 0) ? 1 : 0;
    p.nb_vec = (p.nb != nullptr && aligned16(p.nb) && a.nb_stride_h % 8 == 0 && a.nb_stride_q % 8 == 0) ? 1 : 0;
    // (float)(1 / sqrt(head_size)) as the reference forms it (gating_attention.cpp:68)
    p.scale = (float)(1.0 / sqrt((double)hd));
    const int64_t blocks = ((int64_t)p.groups + 7) / 8 * 8 * 64;
    {
        kutacc_prof::KernelTimer t("attention_tiles_kernel", 4.0 * (double)B * (double)S * (double)S * (double)C, stream);
        const int ks = (int)(hd + 15) / 16;
        hipError_t e;
        if (p.nb != nullptr) {
            e = ks == 1 ? launch_tiles<1, true>(p, blocks, stream) : ks == 2 ? launch_tiles<2, true>(p, blocks, stream)
                : ks == 3 ? launch_tiles<3, true>(p, blocks, stream) : launch_tiles<4, true>(p, blocks, stream);
        } else {
            e = ks == 1 ? launch_tiles<1, false>(p, blocks, stream) : ks == 2 ? launch_tiles<2, false>(p, blocks, stream)
                : ks == 3 ? launch_tiles<3, false>(p, blocks, stream) : launch_tiles<4, false>(p, blocks, stream);
        }
        if ((rc = kutacc_hip_status(e))) {
            return rc;
        }
    }
    return project(a.avg, a.avg_stride_s, M, a.output_w, C, C, C, a.out, a.out_ld, a.output_b, stream);
}

} // namespace kutacc_launch
