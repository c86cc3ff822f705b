// Row-wise HBM-bound kernels that sit in front of the attention operator: LayerNorm over the last
// axis, and the fused pair-bias producer LN(z) -> [H, c_z] projection -> [H, S, S] layout.
// Arithmetic follows reference src/normalization/layernorm_kernel.h:21-53 (shift by the first
// element, fp32 sum and sum of squares, clamped variance, rstd, then (x*rstd - rstd*mean)*gamma+beta)
// and reference src/linear/linear.cpp:21-42 (bf16 operands, result rounded to the storage type).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "device_util.h"
#include "launch_internal.h"
#include "mfma_tiles.h"

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
                                                                       int64_t rows, int64_t size, float eps, int64_t swap_j)
{
    const int lane = threadIdx.x % 64;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + threadIdx.x / 64;
    if (r >= rows) {
        return;
    }
    // swap_j != 0: rows are pairs (i, j) of an [rows / swap_j, swap_j] grid and output row (i, j) is computed from
    // input row (j, i) of the transposed grid
    const T *row = x + (swap_j ? (r % swap_j) * (rows / swap_j) + r / swap_j : r) * ld_x;
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
                                                                  int64_t rows_j, int64_t c_z, int64_t nheads, float eps,
                                                                  int transposed)
{
    const int lane = threadIdx.x % 64;
    const int64_t r = (int64_t)blockIdx.x * ROW_WAVES + threadIdx.x / 64;
    const int64_t rows = rows_i * rows_j;
    if (r >= rows) {
        return;
    }
    // transposed: output row (i, j) is computed from row (j, i) of z, stored [rows_j, rows_i, c_z]
    const T *row = z + (transposed ? (r % rows_j) * rows_i + r / rows_j : r) * c_z;
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


// ---------------------------------------------------------------------------------------------
// bf16 fast paths (row length a multiple of 8 with row_len/8 in {8, 16, 32, 64} lanes per row, rows
// and tensors 16-byte aligned).  A row is spread over LPR = row_len/8 lanes, 16 bytes each, so every
// load and store instruction moves whole cache lines and 64/LPR rows; sums run over the LPR lanes
// with DPP adds (no LDS traffic) up to 16 lanes and lane shuffles above.  Same arithmetic as the
// generic kernels: shift by the row's first element, fp32 sums, clamped variance.
// ---------------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

union Pack16 {
    uint4 u;
    bf16x8 b;
    bf16x2 p[4];
};

// statistics of one row held as 8 values per lane; x0 = first element of the row
template <int LPR>
__device__ __forceinline__ void group_stats(const float (&x)[8], float x0, float n, float eps, float &rstd, float &shift)
{
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float v = x[e] - x0;
        s1 += v;
        s2 = fmaf(v, v, s2);
    }
    s1 = group_sum<LPR>(s1);
    s2 = group_sum<LPR>(s2);
    const float mean = s1 / n + x0;
    const float var = fmaxf((s2 - s1 * s1 / n) / n, 0.f);
    // The hardware's reciprocal square root (1 ulp) instead of an IEEE square root and division: every lane of a row
    // forms it, the two correctly rounded operations expand to some 25 instructions per lane and row, and the normalised
    // value is rounded to bf16 afterwards.
    rstd = __builtin_amdgcn_rsqf(var + eps);
    shift = -rstd * mean;
}

// NEAR: fewer than 2^24 rows, row pitches below 2^23 elements and less than 2^31 bytes from the first row to the end of
// the last (the launcher checks): rows are counted in 32 bits and addressed by 32-bit byte offsets from the tensors'
// first elements -- a 24-bit multiply per row where 64-bit pointer arithmetic spends three quarter-rate ones.
template <int LPR, bool NEAR>
__global__ __launch_bounds__(256) void layernorm_rows_bf16_kernel(const bf16_t *__restrict__ x, int64_t ld_x,
                                                                  const float *__restrict__ gamma,
                                                                  const float *__restrict__ beta, bf16_t *__restrict__ out,
                                                                  int64_t ld_out, int64_t rows, float eps, int64_t swap_j)
{
    constexpr int RPS = 64 / LPR; // rows per step of a wave
    constexpr int U = 4;          // steps in flight
    const int lane = threadIdx.x & 63;
    const int sub = lane % LPR, grp = lane / LPR;
    const int wave_in_block = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform
    float gm[8], bt[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        gm[e] = gamma[sub * 8 + e];
        bt[e] = beta[sub * 8 + e];
    }
    using index_t = std::conditional_t<NEAR, uint32_t, int64_t>;
    const index_t nrows = (index_t)rows, swap = (index_t)swap_j;
    const index_t r0 = ((index_t)blockIdx.x * 4 + wave_in_block) * (RPS * U);
    auto row_ptr = [&](auto *base, int64_t ld, index_t r) {
        if constexpr (NEAR) {
            using byte_t = std::conditional_t<std::is_const_v<std::remove_pointer_t<decltype(base)>>, const char, char>;
            return reinterpret_cast<decltype(base)>(reinterpret_cast<byte_t *>(base) +
                                                    (__umul24(r, 2u * (uint32_t)ld) + 16u * (uint32_t)sub));
        } else {
            return base + r * ld + sub * 8;
        }
    };
    Pack16 in[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        index_t r = r0 + u * RPS + grp;
        r = r < nrows ? r : nrows - 1;
        r = swap ? (r % swap) * (nrows / swap) + r / swap : r; // input row (j, i) for output row (i, j)
        in[u].u = *reinterpret_cast<const uint4 *>(row_ptr(x, ld_x, r));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const index_t r = r0 + u * RPS + grp;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[e] = (float)in[u].b[e];
        }
        const float x0 = __shfl(v[0], grp * LPR, 64);
        float rstd, shift;
        group_stats<LPR>(v, x0, (float)(LPR * 8), eps, rstd, shift);
        Pack16 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            o.b[e] = (bf16_t)fmaf(fmaf(v[e], rstd, shift), gm[e], bt[e]);
        }
        if (r < nrows) {
            *reinterpret_cast<uint4 *>(row_ptr(out, ld_out, r)) = o.u;
        }
    }
}

// Pair-bias producer, bf16, c_z = 128 (16 lanes per row), H <= 8.  A wave owns 32 consecutive rows of
// z; its four 16-lane groups walk 8 rows each (all loads of a lane are issued up front: 8 KB in
// flight per wave, and the small LDS tile leaves room for five workgroups per CU).  The normalised row is rounded to bf16, as a caller of the reference would hand it
// to kutacc_af2_linear, written out (if wanted) and parked in a wave-private LDS tile; when the rows
// are done, the [H, c_z] projection of all of them is 8 MFMAs (heads as MFMA rows, z rows as columns,
// fp32 accumulation), whose result has one z row per lane: every head's 32 values leave as one 64-byte store.
// The vector ALU, which bounds this kernel, is left with the LayerNorm alone.
constexpr int PAIR_BIAS_ROWS_PER_WAVE = 32; // a multiple of 32; LDS per workgroup = 1 KB per row

template <int H>
__global__ __launch_bounds__(256) void pair_bias_bf16_kernel(const bf16_t *__restrict__ z, const float *__restrict__ gamma,
                                                             const float *__restrict__ beta, const bf16_t *__restrict__ w,
                                                             bf16_t *__restrict__ nb, bf16_t *__restrict__ z_norm,
                                                             int64_t rows, float eps, int64_t rows_i, int64_t rows_j,
                                                             int transposed, uint4 *__restrict__ nbf, int frag_nb,
                                                             int frag_nt, int frag_tiles)
{
    constexpr int LPR = 16, CZ = 128, STEPS = PAIR_BIAS_ROWS_PER_WAVE / 4, RB = PAIR_BIAS_ROWS_PER_WAVE / 32;
    __shared__ uint4 tiles[4][RB * 2 * 256]; // per wave: its rows x 128 channels as 32 x 64 panels
    const int lane = threadIdx.x & 63;
    const int sub = lane & 15, grp = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6); // uniform: the wave's first row stays in scalar registers
    // Rows are counted in 32 bits and addressed by 32-bit byte offsets from the tensors' first elements (the launcher
    // sends at most 2^23 rows here: 2 GiB of z), not by 64-bit products per lane and row.
    const uint32_t nrows = (uint32_t)rows, ncol = (uint32_t)rows_j, nrow_i = (uint32_t)rows_i;
    const uint32_t r0 = ((uint32_t)blockIdx.x * 4 + wave) * PAIR_BIAS_ROWS_PER_WAVE;
    if (r0 >= nrows) {
        return;
    }
    const char *zbytes = reinterpret_cast<const char *>(z);
    uint4 *tile = tiles[wave];
    Pack16 in[STEPS];
    {
        // transposed: output row (i, j) is computed from row (j, i) of z, stored [rows_j, rows_i, c_z]; the walk
        // over consecutive output rows then steps through z with stride rows_i rows
        uint32_t r = r0 + grp * STEPS;
        uint32_t i = transposed ? r / ncol : 0, j = transposed ? r % ncol : 0;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            uint32_t src = transposed ? j * nrow_i + i : r;
            src = r < nrows ? src : 0;
            in[s].u = *reinterpret_cast<const uint4 *>(zbytes + (src * (2u * CZ) + 16u * sub));
            ++r;
            if (++j == ncol) {
                j = 0, ++i;
            }
        }
    }
    float gm[8], bt[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        gm[e] = gamma[sub * 8 + e];
        bt[e] = beta[sub * 8 + e];
    }
    // weight fragments, heads as MFMA rows (rows >= H are zero): lane (head, g) holds w[head][16 ks + 8 g .. + 8]
    kutacc_dev::bf16x8 wf[8];
    {
        const int head = lane & 31, g = lane >> 5;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            uint4 v = make_uint4(0u, 0u, 0u, 0u);
            if (head < H) {
                v = *reinterpret_cast<const uint4 *>(w + head * CZ + ks * 16 + g * 8);
            }
            wf[ks] = kutacc_dev::as_bf16x8(v);
        }
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
        const int row_local = grp * STEPS + s;
        const uint32_t r = r0 + row_local;
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[e] = (float)in[s].b[e];
        }
        const float x0 = __shfl(v[0], grp * 16, 64);
        float rstd, shift;
        group_stats<LPR>(v, x0, (float)CZ, eps, rstd, shift);
        Pack16 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            o.b[e] = (bf16_t)fmaf(fmaf(v[e], rstd, shift), gm[e], bt[e]);
        }
        if (z_norm != nullptr && r < nrows) {
            *reinterpret_cast<uint4 *>(reinterpret_cast<char *>(z_norm) + (r * (2u * CZ) + 16u * sub)) = o.u;
        }
        tile[((row_local >> 5) * 2 + (sub >> 3)) * 256 + kutacc_dev::panel_slot(row_local & 31, sub & 7)] = o.u;
    }
    // the tile is private to the wave and LDS operations of a wave complete in order: no barrier
    const int col = lane & 31, g = lane >> 5;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        kutacc_dev::f32x16 acc = kutacc_dev::zero16();
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const uint4 zf = tile[(rb * 2 + (ks >> 2)) * 256 + kutacc_dev::panel_slot(col, 2 * (ks & 3) + g)];
            acc = kutacc_dev::mfma(wf[ks], kutacc_dev::as_bf16x8(zf), acc);
        }
        // accumulator v < 4 of lane (col, g) is head 4 g + v of z row r0 + 32 rb + col
        const uint32_t r = r0 + rb * 32 + col;
        if (r < nrows) {
            char *nbytes = reinterpret_cast<char *>(nb);
            const uint32_t first = 2u * (__umul24(4u * g, nrows) + r); // head 4 g of row r, in bytes; H * rows * 2 < 2^28
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (4 * g + v < H) {
                    *reinterpret_cast<bf16_t *>(nbytes + (first + 2u * v * nrows)) = (bf16_t)acc[v];
                }
            }
        }
        if (nbf != nullptr && frag_tiles) {
            // The copy the two-row attention kernel reads: fp32 tiles in the order of its logits accumulators, in log2 units,
            // [head][query block][key tile][4][64 lanes] x 16 bytes -- lane (pi^-1(q mod 32), g') holds keys 16 g' .. + 15 of
            // the tile for query q, four per piece.  Through the wave's tile: [head][32 keys] fp32, of which a lane takes
            // the four keys of one piece.
            static_assert(RB == 1 && H <= 8, "one lane per piece: 8 pieces per head");
            float *t32 = reinterpret_cast<float *>(tile);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (4 * g + v < H) {
                    const float x = (float)(bf16_t)acc[v] * kutacc_dev::LOG2E;
                    t32[(4 * g + v) * 32 + col] = x < -3.0e38f ? -3.0e38f : x; // -inf: the most negative finite value
                }
            }
            __builtin_amdgcn_wave_barrier(); // other lanes' stores: keep the loads below behind them
            if (lane < 8 * H) {
                const int h = lane >> 3, c = lane & 7; // piece c: keys 4 c .. 4 c + 3 = half g' = c >> 2, piece a = c & 3
                const uint4 val = *reinterpret_cast<const uint4 *>(t32 + h * 32 + c * 4);
                const uint32_t r0b = r0 + rb * 32;
                const int q = (int)(r0b / ncol), t = (int)(r0b % ncol) >> 5, qr = q & 31;
                const int qlane = (qr & 3) | (((qr >> 4) & 1) << 2) | (((qr >> 2) & 3) << 3);
                uint4 *dst = nbf + ((((int64_t)h * frag_nb + (q >> 5)) * frag_nt + t) * 4 + (c & 3)) * 64 + qlane + 32 * (c >> 2);
                *dst = val;
                if (t + 1 == frag_nb && frag_nt > frag_nb) { // the phantom tile that pads the key tiles to a pair
                    dst[256] = make_uint4(0u, 0u, 0u, 0u);
                }
            }
        } else if (nbf != nullptr) {
            // The copy the attention kernels read (rows_j a multiple of 32: the wave's rows are key tile t of one query
            // q): for head h, query block j, key tile t, 16-key half g' and 8-key half e the 16 bytes of lane
            // (pi^-1(q mod 32), g'), pi being the row order of the attention's accumulators; values in log2 units as
            // fp16 (the bf16 pair bias times log2(e), eleven significant bits kept).  Through the wave's tile, which nobody
            // reads any more: [head][32 keys].
            static_assert(RB == 1, "the transposing buffer lies on the first row block of the tile");
            uint16_t *t16 = reinterpret_cast<uint16_t *>(tile);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                if (4 * g + v < H) {
                    t16[(4 * g + v) * 32 + col] = kutacc_dev::pair_bias_log2_f16((float)(bf16_t)acc[v]);
                }
            }
            __builtin_amdgcn_wave_barrier(); // other lanes' stores: keep the loads below behind them
            if (lane < 4 * H) {
                const int h = lane >> 2, c = lane & 3;
                const uint4 val = *reinterpret_cast<const uint4 *>(t16 + h * 32 + c * 8);
                const uint32_t r0b = r0 + rb * 32;
                const int q = (int)(r0b / ncol), t = (int)(r0b % ncol) >> 5, qr = q & 31;
                const int qlane = (qr & 3) | (((qr >> 4) & 1) << 2) | (((qr >> 2) & 3) << 3);
                uint4 *dst = nbf + ((((int64_t)h * frag_nb + (q >> 5)) * frag_nt + t) * 2 + (c & 1)) * 64 + qlane + 32 * (c >> 1);
                *dst = val;
                if (t + 1 == frag_nb && frag_nt > frag_nb) { // the phantom tile that pads the key tiles to a pair
                    dst[128] = make_uint4(0u, 0u, 0u, 0u);
                }
            }
        }
    }
}

template <typename T>
int launch_layernorm(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                     int64_t rows, int64_t size, float eps, int64_t swap_j, hipStream_t stream)
{
    if (sizeof(T) == 2 && (size == 64 || size == 128 || size == 256 || size == 512) && ld_x % 8 == 0 && ld_out % 8 == 0 &&
        (reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) % 16 == 0) {
        const int lpr = (int)(size / 8);
        const int64_t rows_per_block = 4 * 4 * (64 / lpr);
        const int64_t nblk = (rows + rows_per_block - 1) / rows_per_block;
        if (nblk > INT32_MAX) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        const bf16_t *xi = (const bf16_t *)x;
        bf16_t *oi = (bf16_t *)out;
        const int64_t pitch = ld_x > ld_out ? ld_x : ld_out;
        const bool near = rows < (1 << 24) && pitch < (1 << 23) && rows * pitch * 2 < ((int64_t)1 << 31);
        auto launch = [&](auto kernel) { kernel<<<(unsigned)nblk, 256, 0, stream>>>(xi, ld_x, gamma, beta, oi, ld_out, rows, eps, swap_j); };
        switch (lpr) {
            case 8: near ? launch(layernorm_rows_bf16_kernel<8, true>) : launch(layernorm_rows_bf16_kernel<8, false>); break;
            case 16: near ? launch(layernorm_rows_bf16_kernel<16, true>) : launch(layernorm_rows_bf16_kernel<16, false>); break;
            case 32: near ? launch(layernorm_rows_bf16_kernel<32, true>) : launch(layernorm_rows_bf16_kernel<32, false>); break;
            default: near ? launch(layernorm_rows_bf16_kernel<64, true>) : launch(layernorm_rows_bf16_kernel<64, false>); break;
        }
        return kutacc_hip_status(hipGetLastError());
    }
    const int64_t blocks = (rows + ROW_WAVES - 1) / ROW_WAVES;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    layernorm_rows_kernel<T><<<(unsigned)blocks, 64 * ROW_WAVES, 0, stream>>>((const T *)x, ld_x, gamma, beta, (T *)out,
                                                                               ld_out, rows, size, eps, swap_j);
    return kutacc_hip_status(hipGetLastError());
}

template <typename T>
int launch_pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
                     int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int transposed,
                     hipStream_t stream, void *fragments, int frag_nb, int frag_nt, int frag_tiles)
{
    const int64_t rows = rows_i * rows_j;
    if (fragments != nullptr &&
        (!kutacc_launch::pair_bias_writes_fragments(z, w, z_norm, rows_i, rows_j, c_z, nheads,
                                                    sizeof(T) == 2 ? KUTACC_DTYPE_BF16 : KUTACC_DTYPE_FP32) ||
         frag_nb != rows_j / 32 || frag_nt != ((frag_nb + 1) & ~1))) {
        return KUTACC_HIP_EINVAL;
    }
    // the MFMA kernel counts rows and byte offsets in 32 bits: at most 2^23 rows of 256 bytes
    if (sizeof(T) == 2 && c_z == 128 && (nheads == 4 || nheads == 8) && rows <= ((int64_t)1 << 23) &&
        (reinterpret_cast<uintptr_t>(z) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(z_norm)) % 16 == 0) {
        const int64_t nblk = (rows + 4 * PAIR_BIAS_ROWS_PER_WAVE - 1) / (4 * PAIR_BIAS_ROWS_PER_WAVE);
        if (nblk > INT32_MAX) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        if (nheads == 4) {
            pair_bias_bf16_kernel<4><<<(unsigned)nblk, 256, 0, stream>>>((const bf16_t *)z, gamma, beta, (const bf16_t *)w,
                                                                        (bf16_t *)nb, (bf16_t *)z_norm, rows, eps, rows_i, rows_j,
                                                                        transposed, (uint4 *)fragments, frag_nb, frag_nt, frag_tiles);
        } else {
            pair_bias_bf16_kernel<8><<<(unsigned)nblk, 256, 0, stream>>>((const bf16_t *)z, gamma, beta, (const bf16_t *)w,
                                                                        (bf16_t *)nb, (bf16_t *)z_norm, rows, eps, rows_i, rows_j,
                                                                        transposed, (uint4 *)fragments, frag_nb, frag_nt, frag_tiles);
        }
        return kutacc_hip_status(hipGetLastError());
    }
    const int64_t blocks = (rows + ROW_WAVES - 1) / ROW_WAVES;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    pair_bias_kernel<T><<<(unsigned)blocks, 64 * ROW_WAVES, 0, stream>>>(
        (const T *)z, gamma, beta, (const T *)w, (T *)nb, (T *)z_norm, rows_i, rows_j, c_z, nheads, eps, transposed);
    return kutacc_hip_status(hipGetLastError());
}

} // namespace

namespace kutacc_launch {

int layernorm_rows(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                   int64_t rows, int64_t size, float eps, int32_t dtype, hipStream_t stream, int64_t swap_j)
{
    if (!x || !gamma || !beta || !out || rows <= 0 || size <= 0 || ld_x < size || ld_out < size || swap_j < 0 ||
        (swap_j > 0 && rows % swap_j != 0)) {
        return KUTACC_HIP_EINVAL;
    }
    if (dtype == KUTACC_DTYPE_BF16) {
        return launch_layernorm<bf16_t>(x, ld_x, gamma, beta, out, ld_out, rows, size, eps, swap_j, stream);
    }
    if (dtype == KUTACC_DTYPE_FP32) {
        return launch_layernorm<float>(x, ld_x, gamma, beta, out, ld_out, rows, size, eps, swap_j, stream);
    }
    return KUTACC_HIP_EINVAL;
}

bool pair_bias_writes_fragments(const void *z, const void *w, const void *z_norm, int64_t rows_i, int64_t rows_j, int64_t c_z,
                                int64_t nheads, int32_t dtype)
{
    // the MFMA producer, whose waves own 32 consecutive rows: whole key tiles of one query when the grid is square
    // and its side a multiple of 32
    return dtype == KUTACC_DTYPE_BF16 && c_z == 128 && (nheads == 4 || nheads == 8) && rows_i == rows_j && rows_j % 32 == 0 &&
           (reinterpret_cast<uintptr_t>(z) | reinterpret_cast<uintptr_t>(w) | reinterpret_cast<uintptr_t>(z_norm)) % 16 == 0;
}

int pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
              int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int32_t dtype, int transposed,
              hipStream_t stream, void *fragments, int frag_nb, int frag_nt, int frag_tiles)
{
    if (!z || !gamma || !beta || !w || !nb || rows_i <= 0 || rows_j <= 0 || c_z <= 0 || nheads <= 0) {
        return KUTACC_HIP_EINVAL;
    }
    if (dtype == KUTACC_DTYPE_BF16) {
        return launch_pair_bias<bf16_t>(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, transposed, stream,
                                        fragments, frag_nb, frag_nt, frag_tiles);
    }
    if (dtype == KUTACC_DTYPE_FP32) {
        return launch_pair_bias<float>(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, transposed, stream,
                                       fragments, frag_nb, frag_nt, frag_tiles);
    }
    return KUTACC_HIP_EINVAL;
}

} // namespace kutacc_launch
