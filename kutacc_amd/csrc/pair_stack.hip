// bf16 matrix products with fused epilogues for the operators next to the attention on the pair and
// MSA stacks: transition (reference src/attention/transition.cpp:21-39) and the four steps of the
// triangle multiplication (reference src/attention/triangle_multiplication.cpp:25-150).  All of them are
// C = epilogue(A * B^T) on strided bf16 views with fp32 accumulation, which is what the reference hands
// to its GEMM backend through addmm (src/linear/mm.cpp:46-86).
//
// One kernel covers them.  A workgroup of four waves owns a 128 x 128 tile of C and walks K in steps of
// 64: each wave fetches a quarter of both operand tiles with whole-cache-line loads one step ahead,
// parks it in registers while the current step is multiplied, and stores it into the other half of a
// double-buffered LDS tile in MFMA fragment order (one barrier per step).  Operands may be stored
// K-major (rows contiguous in k) or M-major (the "incoming" triangle equation contracts over the leading
// index of both operands; those tiles are transposed in registers, eight lanes at a time, on their way
// into LDS).  The product is formed transposed (MFMA rows = columns of C) so that every lane
// ends up with four consecutive columns of its own row of C; the tile is rounded to bf16 into LDS and
// leaves as whole rows of 256 bytes.
//
// Epilogues: bias per column or per row of C, ReLU, and the gated form of the triangle projections,
// where one launch multiplies the same B tile with 64 rows of the projection weights and the matching
// 64 rows of the gate weights and writes bf16(bf16(proj) * mask * sigmoid(bf16(gate))) -- the rounding
// points of the reference, which rounds both GEMM results to bf16 before its element-wise pass
// (triangle_multiplication.cpp:37-66).
//
// Shapes the MFMA kernel does not take (k, n or a leading dimension not a multiple of 8, pointers not
// 16-byte aligned) run on a scalar kernel with the same epilogues.
//
// The batched product of the triangle equation, where its sides are whole large tiles and there are enough of them,
// runs on persistent kernels with 256 x 256 (or 192 x 192) tiles per workgroup: pair_gemm_direct_kernel, whose
// operands go straight from global memory into the LDS, and pair_gemm_big_kernel, which stages them through
// registers.  The transition keeps its hidden layer on chip (transition_fused_kernel); the gated projections of 128
// channels have kernels of their own that read the activation once (gated_projection_blocks_kernel, and
// gated_projection_kernel behind a tuning switch).
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>
#include <type_traits>
#include <utility>

#include "launch_internal.h"
#include "mfma_tiles.h"
#include "profiler.h"

namespace {
using namespace kutacc_dev;

struct GemmParams {
    const bf16_t *a, *a_gate, *b;
    bf16_t *c;
    int64_t a_sm, a_sk, a_sb; // A(m, k) at a + m*a_sm + k*a_sk + batch*a_sb
    int64_t b_sn, b_sk, b_sb; // B(n, k)
    int64_t c_sm, c_sb;       // C(m, n) at c + m*c_sm + n + batch*c_sb
    const float *bias, *bias_gate;
    const bf16_t *mask; // gated epilogue: multiplier per column of C
    int64_t mask_sb;
    int M, N, K, batches;
    int bias_axis; // 0 none, 1 per column n, 2 per row m
    int relu;
    int MT, NT; // tiles along m and n
    // gated form with two batches that share B and the mask: weights, biases and result of batch 1 (else null).  The two
    // sides of the triangle multiplication's projections in one launch: the activation tile is fetched from HBM once.
    const bf16_t *a_alt, *a_gate_alt;
    const float *bias_alt, *bias_gate_alt;
    bf16_t *c_alt;
};

constexpr int TILE = 128, KSTEP = 64;
constexpr int OPERAND_SLOTS = 4 * 256;          // four 32-row panels of 256 16-byte slots
constexpr int STAGE_SLOTS = 2 * OPERAND_SLOTS;  // A and B
constexpr int CT_LD = 136;                      // bf16 elements per row of the C tile in LDS (272 bytes)
// One operand stage (two barriers per k-step) that the C tile takes over at the end: 34 KB, three workgroups per CU.
// With a second stage only two fit, and the third workgroup hides more of a short tile's prologue and epilogue than
// the second stage did (triangle-multiplication products at 384 residues: 30.7 -> 26.6 us, gated projection 32 -> 27).
constexpr size_t GEMM_LDS = TILE * CT_LD * 2 > STAGE_SLOTS * 16 ? TILE * CT_LD * 2 : STAGE_SLOTS * 16;

// K-major operand: rows row0..row0+31 (clamped), 64 k from k0; chunks past K read as zero
__device__ __forceinline__ PanelRegs load_kmajor(const bf16_t *base, int64_t ld, int row0, int last_row, int k0, int K, int lane)
{
    const int col = k0 + (lane & 7) * 8;
    const bool ok = col < K;
    const int colc = ok ? col : 0;
    PanelRegs p;
    uint4 *dst[4] = {&p.r0, &p.r1, &p.r2, &p.r3};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int row = row0 + 8 * i + (lane >> 3);
        row = row < last_row ? row : last_row;
        uint4 v = *reinterpret_cast<const uint4 *>(base + (int64_t)row * ld + colc);
        if (!ok) {
            v = make_uint4(0u, 0u, 0u, 0u);
        }
        *dst[i] = v;
    }
    return p;
}

// M-major operand (element (m, k) at base + k*ld + m).  Its tile goes to LDS the way it lies in memory, 64 rows k of
// 128 m (256 bytes), and the MFMA fragments -- 8 consecutive k of one m per lane -- come out of the LDS transposing
// read of gfx950, ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i & 3) of the 8-byte chunks that lanes
// 4j + (i >> 2), j = 0..3, point at.  With lane s of the group pointing at row k0 + (s >> 2), m = m0 + 4 (s & 3), lane
// i ends up with k0..k0+3 of m0 + i: a 4 x 16 block transposed per group and instruction, two instructions per
// fragment.  The 8-byte chunk index of a row is XOR-ed with 8 (k & 3), which spreads the four rows a group reads over
// all banks; writes are whole 16-byte pieces of a row.
//
// Loading: 64 m from m0, 32 k from k0 per wave.  Lane (kk, mc) takes 8 consecutive m of row k0 + 8i + mm_row(kk); a
// load instruction covers 8 k x 128 contiguous bytes.  mm_row orders the rows so that the 16 lanes that store together
// hold rows with different k & 3 (different bank halves after the swizzle).
__device__ __forceinline__ int mm_row(int kk) { return (kk & 4) | ((kk & 1) << 1) | ((kk >> 1) & 1); }

__device__ __forceinline__ PanelRegs load_mmajor(const bf16_t *base, int64_t ld, int m0, int rows, int k0, int K, int lane)
{
    int m = m0 + (lane & 7) * 8;
    m = m + 8 <= rows ? m : rows - 8; // rows past the end are never stored; any valid address will do
    PanelRegs p;
    uint4 *dst[4] = {&p.r0, &p.r1, &p.r2, &p.r3};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int k = k0 + 8 * i + mm_row(lane >> 3);
        const bool ok = k < K;
        uint4 v = *reinterpret_cast<const uint4 *>(base + (int64_t)(ok ? k : 0) * ld + m);
        if (!ok) {
            v = make_uint4(0u, 0u, 0u, 0u);
        }
        *dst[i] = v;
    }
    return p;
}

// what load_mmajor fetched -> operand tile [64 k][128 m], m columns mcol0.., rows krow0..
__device__ __forceinline__ void store_mmajor(uint4 *operand, int mcol0, int krow0, int lane, const PanelRegs &p)
{
    const int chunk = (mcol0 >> 2) + 2 * (lane & 7); // 8-byte chunk of the row: 4 m each
    const uint4 regs[4] = {p.r0, p.r1, p.r2, p.r3};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int k = krow0 + 8 * i + mm_row(lane >> 3);
        operand[k * 16 + ((chunk ^ (8 * (k & 3))) >> 1)] = regs[i];
    }
}

// byte offset, inside an m-major operand tile, of the chunk a lane points ds_read_b64_tr_b16 at for the 32-row block
// mblk of the tile: row (lane >> 5) * 8 + ((lane & 15) >> 2) of a 16-k step, m = 32 mblk + 16 ((lane >> 4) & 1) + 4 (lane & 3)
__device__ __forceinline__ int mm_fragment_offset(int mblk, int lane)
{
    const int a = (lane & 15) >> 2;
    const int chunk = 8 * mblk + 4 * ((lane >> 4) & 1) + (lane & 3);
    return ((lane >> 5) * 8 + a) * 256 + ((chunk ^ (8 * a)) * 8);
}

// fragment of k-step s (16 k) from an m-major operand tile: k = 16 s + 8 (lane >> 5) + 0..7 of the lane's m
__device__ __forceinline__ bf16x8 mm_fragment(const lds_char *operand, int lane_off, int s)
{
    return lds_transposed_fragment(operand + lane_off + s * 4096, operand + lane_off + s * 4096 + 1024);
}

template <bool A_MMAJOR, bool B_MMAJOR, bool GATED>
__global__ __launch_bounds__(256, (A_MMAJOR && B_MMAJOR) ? 4 : 3) void pair_gemm_kernel(const GemmParams p)
{
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    // Workgroup ids are dealt round robin over the 8 XCDs; give each XCD a contiguous run of tiles so
    // that neighbours in the walk (which share an operand tile) share an L2.
    int64_t bid = blockIdx.x;
    {
        const int64_t total = gridDim.x, per = total / 8;
        if (bid < per * 8) {
            bid = (bid % 8) * per + bid / 8;
        }
    }
    const int64_t tiles = (int64_t)p.MT * p.NT;
    int batch = (int)(bid / tiles);
    int t = (int)(bid % tiles);
    if (GATED && p.a_alt != nullptr) { // two sides of one B: neighbours in the walk, so that they share its tile in the L2
        batch = (int)(bid & 1), t = (int)(bid >> 1);
    }
    // the dimension with fewer tiles runs fastest: consecutive workgroups then share the tile of the larger operand
    int mt, nt;
    if (p.MT <= p.NT) {
        mt = t % p.MT, nt = t / p.MT;
    } else {
        nt = t % p.NT, mt = t / p.NT;
    }
    constexpr int MROWS = GATED ? 64 : 128; // rows of C per tile
    const int m0 = mt * MROWS, n0 = nt * TILE;

    const bool alt = GATED && p.a_alt != nullptr && batch == 1;
    const bf16_t *a = alt ? p.a_alt : p.a + (int64_t)batch * p.a_sb;
    const bf16_t *a_gate = GATED ? (alt ? p.a_gate_alt : p.a_gate + (int64_t)batch * p.a_sb) : nullptr;
    const bf16_t *b = p.b + (int64_t)batch * p.b_sb;

    auto fetch_a = [&](int k0) -> PanelRegs {
        if constexpr (A_MMAJOR) {
            return load_mmajor(a, p.a_sk, m0 + 64 * (wave & 1), p.M, k0 + 32 * (wave >> 1), p.K, lane);
        } else if constexpr (GATED) {
            return load_kmajor(wave < 2 ? a : a_gate, p.a_sm, m0 + 32 * (wave & 1), p.M - 1, k0, p.K, lane);
        } else {
            return load_kmajor(a, p.a_sm, m0 + 32 * wave, p.M - 1, k0, p.K, lane);
        }
    };
    auto fetch_b = [&](int k0) -> PanelRegs {
        if constexpr (B_MMAJOR) {
            return load_mmajor(b, p.b_sk, n0 + 64 * (wave & 1), p.N, k0 + 32 * (wave >> 1), p.K, lane);
        } else {
            return load_kmajor(b, p.b_sn, n0 + 32 * wave, p.N - 1, k0, p.K, lane);
        }
    };
    auto park = [&](uint4 *stage, const PanelRegs &ra, const PanelRegs &rb) {
        if constexpr (A_MMAJOR) {
            store_mmajor(stage, 64 * (wave & 1), 32 * (wave >> 1), lane, ra);
        } else {
            panel_store(stage + wave * 256, lane, ra);
        }
        if constexpr (B_MMAJOR) {
            store_mmajor(stage + OPERAND_SLOTS, 64 * (wave & 1), 32 * (wave >> 1), lane, rb);
        } else {
            panel_store(stage + OPERAND_SLOTS + wave * 256, lane, rb);
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            acc[i][j] = zero16();
        }
    }

    // m-major operands: where this lane points the transposing reads for the wave's two row blocks and two column blocks
    const int mm_a0 = mm_fragment_offset(2 * wm, lane), mm_a1 = mm_fragment_offset(2 * wm + 1, lane);
    const int mm_b0 = mm_fragment_offset(2 * wn, lane), mm_b1 = mm_fragment_offset(2 * wn + 1, lane);

    const int KT = (p.K + KSTEP - 1) / KSTEP;
    PanelRegs ra = fetch_a(0), rb = fetch_b(0);
    for (int kt = 0; kt < KT; ++kt) {
        uint4 *stage = lds;
        if (kt > 0) {
            __syncthreads(); // the stage is no longer being read
        }
        park(stage, ra, rb);
        __syncthreads();
        if (kt + 1 < KT) {
            ra = fetch_a((kt + 1) * KSTEP);
            rb = fetch_b((kt + 1) * KSTEP);
        }
        const uint4 *oa = stage + (2 * wm) * 256;
        const uint4 *ob = stage + OPERAND_SLOTS + (2 * wn) * 256;
        const lds_char *ta = (const lds_char *)stage, *tb = (const lds_char *)(stage + OPERAND_SLOTS);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int slot = panel_slot(r, 2 * s + g);
            bf16x8 a0, a1, b0, b1;
            if constexpr (A_MMAJOR) {
                a0 = mm_fragment(ta, mm_a0, s), a1 = mm_fragment(ta, mm_a1, s);
            } else {
                a0 = as_bf16x8(oa[slot]), a1 = as_bf16x8(oa[256 + slot]);
            }
            if constexpr (B_MMAJOR) {
                b0 = mm_fragment(tb, mm_b0, s), b1 = mm_fragment(tb, mm_b1, s);
            } else {
                b0 = as_bf16x8(ob[slot]), b1 = as_bf16x8(ob[256 + slot]);
            }
            acc[0][0] = mfma(b0, a0, acc[0][0]);
            acc[0][1] = mfma(b1, a0, acc[0][1]);
            acc[1][0] = mfma(b0, a1, acc[1][0]);
            acc[1][1] = mfma(b1, a1, acc[1][1]);
        }
    }
    __syncthreads(); // every wave is done with the operand tiles; the C tile takes their place

    // accumulators (+ bias, ReLU) -> bf16 C tile in LDS: lane = row of C, four consecutive columns per group
    bf16_t *ct = reinterpret_cast<bf16_t *>(lds);
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int trow = 64 * wm + 32 * i + r; // row of the LDS tile
        // gated form: rows 64-127 of the tile are the gate product, with its own bias and no ReLU
        const bool gate_rows = GATED && wm == 1;
        const float *bsrc = gate_rows ? (alt ? p.bias_gate_alt : p.bias_gate) : (alt ? p.bias_alt : p.bias);
        float row_bias = 0.f;
        if (p.bias_axis == 2) {
            const int gm = GATED ? m0 + 32 * i + r : m0 + trow;
            row_bias = gm < p.M ? bsrc[gm] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int tcol = 64 * wn + 32 * j + 8 * q + 4 * g;
                f32x4 bv = {row_bias, row_bias, row_bias, row_bias};
                if (p.bias_axis == 1 && n0 + tcol + 4 <= p.N) {
                    bv = *reinterpret_cast<const f32x4 *>(bsrc + n0 + tcol);
                }
                bf16x4 ov;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float x = acc[i][j][4 * q + c] + bv[c];
                    if (p.relu && !gate_rows) {
                        x = fmaxf(x, 0.f);
                    }
                    ov[c] = (bf16_t)x;
                }
                *reinterpret_cast<bf16x4 *>(ct + trow * CT_LD + tcol) = ov;
            }
        }
    }
    __syncthreads();

    bf16_t *c = alt ? p.c_alt : p.c + (int64_t)batch * p.c_sb;
    if constexpr (GATED) {
        const bf16_t *mask = p.mask + (int64_t)batch * p.mask_sb;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = tid + 256 * i;
            const int row = piece >> 4, chunk = piece & 15;
            const int gm = m0 + row, gn = n0 + chunk * 8;
            if (gm < p.M && gn < p.N) {
                const bf16x8 pv = *reinterpret_cast<const bf16x8 *>(ct + row * CT_LD + chunk * 8);
                const bf16x8 gv = *reinterpret_cast<const bf16x8 *>(ct + (64 + row) * CT_LD + chunk * 8);
                const bf16x8 mv = *reinterpret_cast<const bf16x8 *>(mask + gn);
                bf16x8 ov;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    ov[e] = (bf16_t)(to_f32(pv[e]) * to_f32(mv[e]) * sigmoid_fast(to_f32(gv[e])));
                }
                *reinterpret_cast<bf16x8 *>(c + (int64_t)gm * p.c_sm + gn) = ov;
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int piece = tid + 256 * i;
            const int row = piece >> 4, chunk = piece & 15;
            const int gm = m0 + row, gn = n0 + chunk * 8;
            if (gm < p.M && gn < p.N) {
                *reinterpret_cast<uint4 *>(c + (int64_t)gm * p.c_sm + gn) =
                    *reinterpret_cast<const uint4 *>(ct + row * CT_LD + chunk * 8);
            }
        }
    }
}

// ---- square products with many tiles: 256 x 256 of C per workgroup, 128 x 128 per wave ----
//
// At 64 x 64 per wave the four MFMAs of a k-step need four operand fragments from the LDS, and with the stores that
// stage the tiles the LDS moves 1.5 KB per MFMA: more than it can deliver at the matrix cores' rate.  Here a wave
// multiplies 4 x 4 blocks (eight fragments for sixteen MFMAs) and a workgroup stages 512 rows of operands for 256
// MFMAs, 0.75 KB per MFMA.  The 256 accumulator registers leave room for one wave per SIMD, so nothing but the
// wave's own instruction order hides a latency: operands are requested two k-steps ahead, fragments one quarter step
// ahead, and the order is pinned with scheduling barriers (one workgroup barrier per step).  An operand stage holds
// four sub-tiles of 128 rows x 64 k (16 KB each: A rows 0-127, A rows 128-255, B likewise) in the layout the
// 128 x 128 kernel uses for that orientation; wave w stages sub-tile w.  Both operands in the same orientation, no
// epilogue but the rounding: the triangle-multiplication equation.
constexpr int BIG_TILE = 256;
constexpr int SUB_SLOTS = 1024;
constexpr int BIG_STAGE_SLOTS = 4 * SUB_SLOTS;
constexpr size_t BIG_GEMM_LDS = 2 * BIG_STAGE_SLOTS * 16;

// The registers, or zeros, by a mask: a conditional assignment becomes a branch, and a branch inside the k-loop splits
// the basic block whose instruction order the loop depends on.
__device__ __forceinline__ PanelRegs keep_if(const PanelRegs &p, bool ok)
{
    const uint32_t keep = ok ? 0xffffffffu : 0u;
    auto m = [&](uint4 v) { return make_uint4(v.x & keep, v.y & keep, v.z & keep, v.w & keep); };
    return PanelRegs{m(p.r0), m(p.r1), m(p.r2), m(p.r3)};
}

struct TilePlace {
    int batch, m0, n0;
};

// Where tile `index` of a persistent workgroup's walk lies (tiles of `side` x `side`).  Workgroup ids are dealt round
// robin over the 8 XCDs, and id + gridDim.x lands on the same XCD when the grid is a multiple of 8: each XCD gets a
// contiguous run of tiles, so that neighbours in the walk (which share an operand tile) share an L2; within a batch the
// dimension with fewer tiles runs fastest.  An index past the last tile gives the last one: a valid address, never used.
// (The launchers keep the number of tiles within 32 bits: 64-bit divisions cost a few thousand clocks per tile.)
__device__ __forceinline__ TilePlace walk_place(const GemmParams &p, int64_t total_tiles, int64_t index, int side)
{
    uint32_t v = (uint32_t)(index < total_tiles ? index : total_tiles - 1);
    const uint32_t per = (uint32_t)total_tiles / 8;
    if (v < per * 8) {
        v = (v % 8) * per + v / 8;
    }
    const uint32_t tiles_per_batch = (uint32_t)p.MT * (uint32_t)p.NT;
    const int batch = (int)(v / tiles_per_batch), t = (int)(v % tiles_per_batch);
    int mt, nt;
    if (p.MT <= p.NT) {
        mt = t % p.MT, nt = t / p.MT;
    } else {
        nt = t % p.NT, mt = t / p.NT;
    }
    return TilePlace{batch, mt * side, nt * side};
}

// The order of one quarter (k-step of 16) of pair_gemm_big_kernel's k-loop, as scheduling-group barriers, whose sizes
// must be integer constants: NMFMA MFMAs in pairs, with this quarter's LDS reads, global loads or LDS stores dealt
// evenly between them.
template <int COUNT, int SLOT, int SLOTS>
constexpr int slot_share() { return (COUNT * (SLOT + 1)) / SLOTS - (COUNT * SLOT) / SLOTS; }

template <int NMFMA, int READS, int LOADS, int STORES, int SLOT>
__device__ __forceinline__ void quarter_slot()
{
    constexpr int SLOTS = (NMFMA + 1) / 2;
    if constexpr (slot_share<READS, SLOT, SLOTS>() > 0) {
        __builtin_amdgcn_sched_group_barrier(0x100, slot_share<READS, SLOT, SLOTS>(), 0); // LDS reads
    }
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); // MFMA
    if constexpr (slot_share<LOADS, SLOT, SLOTS>() > 0) {
        __builtin_amdgcn_sched_group_barrier(0x020, slot_share<LOADS, SLOT, SLOTS>(), 0); // global loads
    }
    if constexpr (slot_share<STORES, SLOT, SLOTS>() > 0) {
        __builtin_amdgcn_sched_group_barrier(0x200, slot_share<STORES, SLOT, SLOTS>(), 0); // LDS stores
    }
    if constexpr (2 * SLOT + 1 < NMFMA) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    }
}

template <int NMFMA, int READS, int LOADS, int STORES, int... SLOT>
__device__ __forceinline__ void quarter_order(std::integer_sequence<int, SLOT...>)
{
    (quarter_slot<NMFMA, READS, LOADS, STORES, SLOT>(), ...);
}

template <int NMFMA, int READS, int LOADS, int STORES>
__device__ __forceinline__ void quarter_order()
{
    quarter_order<NMFMA, READS, LOADS, STORES>(std::make_integer_sequence<int, (NMFMA + 1) / 2>{});
}

// Persistent: one workgroup per CU walks tiles blockIdx.x, blockIdx.x + gridDim.x, ... and its operand pipeline runs
// on across the tile boundary -- the last two k-steps of a tile request the first two of the next, and the store of
// the finished tile goes out under the next tile's MFMAs.
//
// BW = 4: 256 x 256 per workgroup (128 x 128 per wave).  BW = 3: 192 x 192 (96 x 96 per wave), for sides that are
// multiples of 192 but not of 256 (384 residues: four tiles per channel, two per CU, where the 128 x 128 tiles leave
// the chip one eighth of a round short).  A stage keeps its layout of four 16 KB sub-tiles; with BW = 3 the second
// sub-tile of each operand is half used.  The operand loads of a step come in pieces of a quarter sub-tile (k-major: 32
// rows x 64 k; m-major: 64 m x 32 k), 4 BW per step, BW per wave.
template <bool MMAJOR, int BW>
__global__ __launch_bounds__(256, 1) void pair_gemm_big_kernel(const GemmParams p, const int64_t total_tiles)
{
    constexpr int TILE_SIDE = 64 * BW; // rows of C per workgroup, and columns
    constexpr int WAVE_SIDE = 32 * BW;
    constexpr int NMFMA = BW * BW;     // per wave and k-step of 16
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    auto place = [&](int64_t index) -> TilePlace { return walk_place(p, total_tiles, index, TILE_SIDE); };

    // The pieces this wave stages: piece e = wave * BW + i of the step's 4 BW; pieces 0 .. 2 BW - 1 belong to A, the rest
    // to B.  M, N and K are whole tiles and steps here, so an address is a wave-uniform pointer (tile, k-step, piece:
    // scalar arithmetic) plus one 32-bit byte offset per lane that never changes; the loads cost no vector instructions
    // beyond themselves, which matters with one wave per SIMD, where every vector instruction between two MFMAs comes out
    // of the matrix pipe's time.
    const int64_t lda = MMAJOR ? p.a_sk : p.a_sm, ldb = MMAJOR ? p.b_sk : p.b_sn;
    auto piece_is_a = [&](int i) { return wave * BW + i < 2 * BW; };
    auto piece_index = [&](int i) { const int e = wave * BW + i; return e < 2 * BW ? e : e - 2 * BW; }; // within its operand
    uint32_t lane_bytes[BW];
#pragma unroll
    for (int i = 0; i < BW; ++i) {
        const int64_t ld = piece_is_a(i) ? lda : ldb;
        lane_bytes[i] = (uint32_t)(((MMAJOR ? mm_row(lane >> 3) : (lane >> 3)) * ld + (lane & 7) * 8) * 2);
    }
    struct Sources {
        const char *a, *b; // element (row 0 of the tile, k = 0) of each operand
    };
    auto sources = [&](const TilePlace &tp) -> Sources {
        const bf16_t *a = p.a + (int64_t)tp.batch * p.a_sb, *b = p.b + (int64_t)tp.batch * p.b_sb;
        return Sources{reinterpret_cast<const char *>(MMAJOR ? a + tp.m0 : a + (int64_t)tp.m0 * lda),
                       reinterpret_cast<const char *>(MMAJOR ? b + tp.n0 : b + (int64_t)tp.n0 * ldb)};
    };
    // piece i of this wave for the k-step at k0; a step past K (an odd number of steps is rounded up) reads step 0
    // instead and is cleared on its way to the LDS
    auto fetch_piece = [&](const Sources &src, int i, int k0) -> PanelRegs {
        const int k0c = k0 < p.K ? k0 : 0;
        const bool is_a = piece_is_a(i);
        const int64_t ld = is_a ? lda : ldb;
        const int e = piece_index(i);
        // k-major: rows 32 e .. + 31, 64 k from k0c; m-major: 64 m from 64 (e / 2), k = k0c + 32 (e % 2) .. + 31
        const char *base = is_a ? src.a : src.b;
        const char *q = MMAJOR ? base + ((int64_t)(k0c + 32 * (e & 1)) * ld + 64 * (e >> 1)) * 2 : base + ((int64_t)32 * e * ld + k0c) * 2;
        PanelRegs f;
        f.r0 = *reinterpret_cast<const uint4 *>(q + lane_bytes[i]);
        f.r1 = *reinterpret_cast<const uint4 *>(q + 16 * ld + lane_bytes[i]);
        f.r2 = *reinterpret_cast<const uint4 *>(q + 32 * ld + lane_bytes[i]);
        f.r3 = *reinterpret_cast<const uint4 *>(q + 48 * ld + lane_bytes[i]);
        return f;
    };
    // what fetch_piece(.., i, k0) brought, zeros for a step past K, into its place in a stage: operand o's rows live in
    // sub-tiles 2 o and 2 o + 1, 128 rows each
    auto park_piece = [&](uint4 *stage, const PanelRegs &f, int i, int k0) {
        const PanelRegs q = keep_if(f, k0 < p.K);
        const int e = piece_index(i);
        uint4 *operand = stage + (piece_is_a(i) ? 0 : 2 * SUB_SLOTS);
        if constexpr (MMAJOR) {
            const int mchunk = e >> 1; // 64 m each
            store_mmajor(operand + (mchunk >> 1) * SUB_SLOTS, 64 * (mchunk & 1), 32 * (e & 1), lane, q);
        } else {
            panel_store(operand + (e >> 2) * SUB_SLOTS + (e & 3) * 256, lane, q);
        }
    };
    struct Pieces {
        PanelRegs q[BW];
    };
    auto fetch = [&](const Sources &src, int k0) -> Pieces {
        Pieces f;
#pragma unroll
        for (int i = 0; i < BW; ++i) {
            f.q[i] = fetch_piece(src, i, k0);
        }
        return f;
    };
    auto park = [&](uint4 *stage, const Pieces &f, int k0) {
#pragma unroll
        for (int i = 0; i < BW; ++i) {
            park_piece(stage, f.q[i], i, k0);
        }
    };

    f32x16 acc[BW][BW];
    int mm_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mm_off[i] = mm_fragment_offset(i, lane);
    }

    // Fragments of k-step s + 1 are requested while the MFMAs of step s issue (two register sets), the next stage's
    // stores go behind the MFMAs of the last step, and the scheduler is told the interleaving: left to itself it
    // puts every LDS read directly in front of the MFMAs that need it, and with one wave per SIMD nothing else
    // covers that latency.
    bf16x8 af[2][BW], bq[2][BW];
    auto fragments = [&](int set, const uint4 *stage, int s) {
        const int slot = panel_slot(r, 2 * s + g);
#pragma unroll
        for (int i = 0; i < BW; ++i) {
            const int ba = wm * BW + i, bb = wn * BW + i; // 32-row blocks of the operands' 192 or 256 rows
            const uint4 *sa = stage + (ba >> 2) * SUB_SLOTS, *sb = stage + (2 + (bb >> 2)) * SUB_SLOTS;
            if constexpr (MMAJOR) {
                af[set][i] = mm_fragment((const lds_char *)sa, mm_off[ba & 3], s);
                bq[set][i] = mm_fragment((const lds_char *)sb, mm_off[bb & 3], s);
            } else {
                af[set][i] = as_bf16x8(sa[(ba & 3) * 256 + slot]);
                bq[set][i] = as_bf16x8(sb[(bb & 3) * 256 + slot]);
            }
        }
    };
    // The fragments arrive in the order a0 b0 a1 b1 ..., the last ones shortly before the quarter that uses them
    // begins: the MFMAs go in the order in which their operands arrive, those that need the last fragment last.
    auto multiply = [&](int set) {
#pragma unroll
        for (int m = 0; m < BW; ++m) { // all pairs (i, j) with max(i, j) = m
#pragma unroll
            for (int j = 0; j < m; ++j) {
                acc[m][j] = mfma(bq[set][j], af[set][m], acc[m][j]);
            }
#pragma unroll
            for (int i = 0; i <= m; ++i) {
                acc[i][m] = mfma(bq[set][m], af[set][i], acc[i][m]);
            }
        }
    };
    constexpr int READS = (MMAJOR ? 4 : 2) * BW; // LDS read instructions per k-step of 16
    // One k-step of 64 from `stage`.  Operands travel two steps ahead of the MFMAs: the step requests the tiles of the
    // step after next (of `src`, at k_fetch) into `fill` and stores `ahead`, requested a step earlier for k_park, into
    // the other stage.  The loads are spread over the MFMAs of the first three quarters: issued together they hold the
    // wave, and with it the matrix pipe, for as long as the CU's memory path takes to accept 64 KB (1500 to 2400 clocks of
    // a step of 2048 MFMA clocks, measured).
    auto k_step = [&](const uint4 *stage, uint4 *other, const Sources &src, int k_fetch, int k_park, const Pieces &ahead, Pieces &fill) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if (s < 3) {
                fragments((s + 1) & 1, stage, s + 1);
            }
            // BW = 4: pieces 0 and 1, then 2, then 3; BW = 3: one piece per quarter
            if (s == 0) {
                fill.q[0] = fetch_piece(src, 0, k_fetch);
                if constexpr (BW == 4) {
                    fill.q[1] = fetch_piece(src, 1, k_fetch);
                }
            } else if (s < 3) {
                fill.q[BW - 3 + s] = fetch_piece(src, BW - 3 + s, k_fetch);
            }
            multiply(s & 1);
            if (s == 3) {
                park(other, ahead, k_park); // every wave left that stage before the barrier that ended the previous step
            }
            if (s == 0) {
                quarter_order<NMFMA, READS, 4 * (BW - 2), 0>();
            } else if (s < 3) {
                quarter_order<NMFMA, READS, 4, 0>();
            } else {
                quarter_order<NMFMA, 0, 0, 4 * BW>();
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        fragments(0, other, 0);
    };

    // Steps go in pairs with one body, so that the accumulators and the two register sets keep their places; an odd
    // number of steps ends with a step whose operands, past K, were cleared on their way to the LDS.
    const int KT2 = ((p.K + KSTEP - 1) / KSTEP + 1) & ~1;
    uint4 *stage0 = lds, *stage1 = lds + BIG_STAGE_SLOTS;
    int64_t v = blockIdx.x;
    TilePlace cur = place(v);
    Sources cur_src = sources(cur);
    Pieces even, odd; // tiles of an even / odd k-step on their way to the LDS
    even = fetch(cur_src, 0);
    odd = fetch(cur_src, KSTEP);
    park(stage0, even, 0);
    __syncthreads();
    fragments(0, stage0, 0);
    for (; v < total_tiles; v += gridDim.x) {
        const Sources next_src = sources(place(v + gridDim.x));
#pragma unroll
        for (int i = 0; i < BW; ++i) {
#pragma unroll
            for (int j = 0; j < BW; ++j) {
                acc[i][j] = zero16();
            }
        }
        for (int kt = 0; kt < KT2; kt += 2) {
            const bool last = kt + 2 == KT2; // the requests go on to the next tile
            const Sources src = last ? next_src : cur_src;
            k_step(stage0, stage1, src, last ? 0 : (kt + 2) * KSTEP, (kt + 1) * KSTEP, odd, even);
            k_step(stage1, stage0, src, last ? KSTEP : (kt + 3) * KSTEP, last ? 0 : (kt + 2) * KSTEP, even, odd);
        }

        // Each wave rounds its block to bf16 through a 32-row strip in the stage the last step read (the other one
        // already holds the next tile's first step; a wave's LDS accesses complete in order, so the strip needs no
        // barrier) and writes whole pieces of rows.  The strips lie in sub-tile `wave` of that stage.  With BW = 4 that
        // sub-tile is also the only place this wave's next stores go, so a wave that is ahead cannot reach a slower one's
        // strip; with BW = 3 the pieces of a wave spread over sub-tiles, and a barrier keeps the next step's stores behind
        // every wave's strip.
        bf16_t *ct = reinterpret_cast<bf16_t *>(stage1 + wave * SUB_SLOTS);
        bf16_t *c = p.c + (int64_t)cur.batch * p.c_sb;
        constexpr int CHUNKS = WAVE_SIDE / 8; // 16-byte pieces per row of the wave's block
#pragma unroll
        for (int i = 0; i < BW; ++i) {
#pragma unroll
            for (int j = 0; j < BW; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    bf16x4 ov;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        ov[e] = (bf16_t)acc[i][j][4 * q + e];
                    }
                    *reinterpret_cast<bf16x4 *>(ct + r * CT_LD + 32 * j + 8 * q + 4 * g) = ov;
                }
            }
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int e = 0; e < (32 * CHUNKS) / 64; ++e) {
                const int piece = lane + 64 * e;
                const int row = piece / CHUNKS, chunk = piece % CHUNKS;
                const int64_t gm = cur.m0 + WAVE_SIDE * wm + 32 * i + row, gn = cur.n0 + WAVE_SIDE * wn + chunk * 8;
                *reinterpret_cast<uint4 *>(c + gm * p.c_sm + gn) = *reinterpret_cast<const uint4 *>(ct + row * CT_LD + chunk * 8);
            }
            __builtin_amdgcn_wave_barrier();
        }
        if constexpr (BW != 4) {
            __syncthreads();
        }
        cur = place(v + gridDim.x);
        cur_src = next_src;
    }
}

// The 256 x 256 tiles with the operands loaded straight into the LDS (global_load_lds_dwordx4: a wave's 64 lanes
// write 1 KB of consecutive LDS, each from its own global address), no registers and no LDS store instructions on the
// way.  The stage is 32 k deep (32 KB: A's 256 rows, then B's), four of them form a ring and a stage is requested three
// stages ahead of its MFMAs: a wave asks for its eight 1 KB units of stage t + 3 among the MFMAs of stage t, waits at the
// end of stage t until its units of stage t + 2 have landed (at most the eight youngest loads still in flight) and
// meets the others at the barrier; after it every wave may read stage t + 2 and overwrite stage t - 1.
//
// K-major operand: a unit is 16 rows x 64 bytes, lane l -> row l / 4, 16-byte slot l % 4, and the lane fetches the
// chunk that the slot holds after the swizzle (chunk ^ direct_swizzle(row)), under which the fragment reads (lane ->
// its own row, chunk 2 s + g) are free of bank conflicts.  M-major operand: a unit is 4 k x 128 m (256 bytes a row),
// rows as they lie in memory with the 16-byte slots of row k XOR-ed with 4 (k & 3): the layout the transposing reads
// of the other kernels expect, with 32 rows per sub-tile.
constexpr int DIRECT_KSTEP = 32;
constexpr int DIRECT_STAGE_SLOTS = 2048;
constexpr int DIRECT_RING = 4;
constexpr int DIRECT_STRIP_LD = 72; // bf16 per row of a wave's output strip: 64 columns and 16 bytes of padding
constexpr size_t DIRECT_STRIP_BYTES = 32 * DIRECT_STRIP_LD * 2;
constexpr size_t DIRECT_GEMM_LDS = DIRECT_RING * DIRECT_STAGE_SLOTS * 16 + 4 * DIRECT_STRIP_BYTES;

// 64-byte rows: rows two apart start in the same banks (32 banks of 4 bytes), so the eight rows that eight consecutive
// lanes read take four different slots per parity
__device__ __forceinline__ int direct_swizzle(int row) { return ((row >> 1) & 3) ^ ((row >> 3) & 1); }

// The sixteen MFMAs of a quarter, blocks (i, j) in the order in which the fragments a0 b0 a1 b1 ... arrive.
__device__ constexpr int DIRECT_MI[16] = {0, 1, 0, 1, 2, 2, 0, 1, 2, 3, 3, 3, 0, 1, 2, 3};
__device__ constexpr int DIRECT_MJ[16] = {0, 0, 1, 1, 0, 1, 2, 2, 2, 0, 1, 2, 3, 3, 3, 3};

template <bool MMAJOR>
__global__ __launch_bounds__(256, 1) void pair_gemm_direct_kernel(const GemmParams p, const int64_t total_tiles)
{
    typedef __attribute__((address_space(3))) void *lds_ptr;
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 31, g = lane >> 5;
    const int wm = wave >> 1, wn = wave & 1;

    auto place = [&](int64_t index) -> TilePlace { return walk_place(p, total_tiles, index, BIG_TILE); };

    // Waves 0 and 1 bring A, waves 2 and 3 B: unit u = 8 (wave & 1) + i of the operand's sixteen per stage.  An address
    // is a wave-uniform pointer (tile, stage, unit) plus a 32-bit byte offset per lane that never changes.
    const bool brings_a = wave < 2;
    const int64_t ld = brings_a ? (MMAJOR ? p.a_sk : p.a_sm) : (MMAJOR ? p.b_sk : p.b_sn);
    // byte offsets of this lane's 16 bytes of unit i from the stage's first element of the operand: the unit's place
    // in the stage and the lane's in the unit; they never change, so a request costs its own instruction, the LDS
    // address in M0 and nothing else (with one wave per SIMD every instruction issued comes out of the MFMAs' time)
    uint32_t unit_bytes[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int u = (wave & 1) * 8 + i;
        if constexpr (MMAJOR) {
            unit_bytes[i] = (uint32_t)((((lane >> 4) + 4 * (u & 7)) * ld + 8 * ((lane & 15) ^ (4 * (lane >> 4))) + 128 * (u >> 3)) * 2);
        } else {
            const int row = lane >> 2;
            unit_bytes[i] = (uint32_t)(((16 * u + row) * ld + 8 * ((lane & 3) ^ direct_swizzle(row))) * 2);
        }
    }
    const int64_t stage_pitch = MMAJOR ? DIRECT_KSTEP * ld * 2 : DIRECT_KSTEP * 2; // bytes from one stage's elements to the next's
    auto operand_of = [&](const TilePlace &tp) -> const char * { // element (first row of the tile, k = 0) of this wave's operand
        if (brings_a) {
            const bf16_t *a = p.a + (int64_t)tp.batch * p.a_sb;
            return reinterpret_cast<const char *>(MMAJOR ? a + tp.m0 : a + (int64_t)tp.m0 * ld);
        }
        const bf16_t *b = p.b + (int64_t)tp.batch * p.b_sb;
        return reinterpret_cast<const char *>(MMAJOR ? b + tp.n0 : b + (int64_t)tp.n0 * ld);
    };
    // The load is written out: as a builtin the compiler takes every LDS read behind it for a possible reader of its
    // data and waits for all loads in flight first.  Nothing the compiler generates depends on these loads; the waits
    // for them are the explicit ones at the end of a stage.  `from`: the stage's first element of the operand; `to`:
    // LDS byte address of this wave's first unit in the stage.
    auto request = [&](const char *from, uint32_t to, int i) {
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(to + i * 1024u), "v"(unit_bytes[i]), "s"(from) : "memory");
    };
    const uint32_t ring_bytes = (uint32_t)(uintptr_t)(lds_ptr)lds + (brings_a ? 0u : DIRECT_STAGE_SLOTS * 8u) + (wave & 1) * 8192u;

    f32x16 acc[4][4];
    int mm_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        mm_off[i] = mm_fragment_offset(i, lane);
    }
    const int frag_slot[2] = {r * 4 + (g ^ direct_swizzle(r)), r * 4 + ((2 + g) ^ direct_swizzle(r))};
    bf16x8 af[2][4], bq[2][4];
    // fragment n of a quarter's eight, in the order a0 b0 a1 b1 ...
    auto fragment = [&](int set, const uint4 *stage, int s, int n) {
        const int i = n >> 1;
        const int ba = wm * 4 + i, bb = wn * 4 + i; // 32-row blocks of the operands' 256 rows
        if (!(n & 1)) {
            if constexpr (MMAJOR) {
                af[set][i] = mm_fragment((const lds_char *)(stage + (ba >> 2) * 512), mm_off[ba & 3], s);
            } else {
                af[set][i] = as_bf16x8(stage[ba * 128 + frag_slot[s]]);
            }
        } else {
            if constexpr (MMAJOR) {
                bq[set][i] = mm_fragment((const lds_char *)(stage + DIRECT_STAGE_SLOTS / 2 + (bb >> 2) * 512), mm_off[bb & 3], s);
            } else {
                bq[set][i] = as_bf16x8(stage[DIRECT_STAGE_SLOTS / 2 + bb * 128 + frag_slot[s]]);
            }
        }
    };
    // One quarter in a fixed order: per pair of MFMAs on `set` one fragment for the other set (quarter s_next of
    // `stage`) in front, and behind the pair's first MFMA what `issue` requests for pair n.  `fresh`: a tile's first
    // quarter, which touches every block once, starts the sums (a zero operand costs nothing; clearing 256 accumulator
    // registers is 512 instructions a tile).
    auto quarter = [&](int set, const uint4 *stage, int s_next, auto issue, auto fresh) {
#pragma unroll
        for (int n = 0; n < 8; ++n) {
            fragment(set ^ 1, stage, s_next, n);
            acc[DIRECT_MI[2 * n]][DIRECT_MJ[2 * n]] =
                mfma(bq[set][DIRECT_MJ[2 * n]], af[set][DIRECT_MI[2 * n]], decltype(fresh)::value ? zero16() : acc[DIRECT_MI[2 * n]][DIRECT_MJ[2 * n]]);
            issue(n);
            acc[DIRECT_MI[2 * n + 1]][DIRECT_MJ[2 * n + 1]] = mfma(bq[set][DIRECT_MJ[2 * n + 1]], af[set][DIRECT_MI[2 * n + 1]],
                                                                 decltype(fresh)::value ? zero16() : acc[DIRECT_MI[2 * n + 1]][DIRECT_MJ[2 * n + 1]]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto ring_step = [](int slot, int d) { return slot + d >= DIRECT_RING ? slot + d - DIRECT_RING : slot + d; };

    const int KT = p.K / DIRECT_KSTEP; // at least three (the launcher sees to it)
    int64_t v = blockIdx.x;
    TilePlace cur = place(v);
    const char *cur_operand = operand_of(cur), *next_operand = cur_operand;
#pragma unroll
    for (int t = 0; t < 3; ++t) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            request(cur_operand + t * stage_pitch, ring_bytes + t * DIRECT_STAGE_SLOTS * 16u, i);
        }
    }
    asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
#pragma unroll
    for (int n = 0; n < 8; ++n) {
        fragment(0, lds, 0, n);
    }
    int slot = 0; // of the ring, where the current stage lies
    for (; v < total_tiles; v += gridDim.x) {
        const TilePlace next = place(v + gridDim.x);
        next_operand = operand_of(next);
        auto stage = [&](int kt, auto fresh) {
            const bool over = kt + 3 >= KT; // the requests go on to the next tile
            const char *from = (over ? next_operand : cur_operand) + (over ? kt + 3 - KT : kt + 3) * stage_pitch;
            const uint32_t to = ring_bytes + ring_step(slot, 3) * DIRECT_STAGE_SLOTS * 16u;
            quarter(0, lds + slot * DIRECT_STAGE_SLOTS, 1, [&](int n) {
                if (n & 1) {
                    request(from, to, n >> 1);
                }
            }, fresh);
            quarter(1, lds + ring_step(slot, 1) * DIRECT_STAGE_SLOTS, 0, [&](int n) {
                if (n & 1) {
                    request(from, to, 4 + (n >> 1));
                }
            }, std::false_type{});
            // this wave's units of the stage after next have landed when at most the eight requests of this stage are
            // in flight; behind the barrier every wave's have, and every wave has left the stage before this one
            asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory");
            slot = ring_step(slot, 1);
        };
        stage(0, std::true_type{});
        for (int kt = 1; kt < KT; ++kt) {
            stage(kt, std::false_type{});
        }

        // Each wave rounds its block to bf16 through a strip of its own (32 rows x 64 columns) behind the ring and
        // writes whole 128-byte pieces of rows; a wave's LDS accesses complete in order, so the strip needs no barrier.
        bf16_t *ct = reinterpret_cast<bf16_t *>(reinterpret_cast<char *>(lds + DIRECT_RING * DIRECT_STAGE_SLOTS) + wave * DIRECT_STRIP_BYTES);
        bf16_t *c = p.c + (int64_t)cur.batch * p.c_sb;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        bf16x4 ov;
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            ov[e] = (bf16_t)acc[i][2 * jh + jj][4 * q + e];
                        }
                        *reinterpret_cast<bf16x4 *>(ct + r * DIRECT_STRIP_LD + 32 * jj + 8 * q + 4 * g) = ov;
                    }
                }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int piece = lane + 64 * e;
                    const int row = piece >> 3, chunk = piece & 7;
                    const int64_t gm = cur.m0 + 128 * wm + 32 * i + row, gn = cur.n0 + 128 * wn + 64 * jh + chunk * 8;
                    *reinterpret_cast<uint4 *>(c + gm * p.c_sm + gn) = *reinterpret_cast<const uint4 *>(ct + row * DIRECT_STRIP_LD + chunk * 8);
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
        cur = next;
        cur_operand = next_operand;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the requests for a tile past the last one: let them land before the LDS is given back
}

// Transition with the hidden layer kept on chip: out = relu(x . W1^T + b1) . W2^T + b2 for row tiles of x
// (reference src/attention/transition.cpp:31-38 runs two GEMMs through a [rows, c_i] intermediate; with
// c_i = 4 c_o that intermediate is four fifths of the HBM traffic).  A wave owns RB blocks of 32 rows, whose
// input fragments stay in registers; the workgroup streams the two weight matrices through LDS in slices
// of 64 hidden units, double buffered, one barrier per slice.  Both products are formed transposed
// (MFMA rows = hidden units, then output channels; columns = rows of x): the accumulators of the first,
// after bias, ReLU and rounding to bf16 (the reference's rounding point: its intermediate is a bf16
// tensor), are the B operand of the second without leaving the registers.  For that the lane that feeds
// MFMA row i with a row of W1 takes hidden unit sigma(i) (bits 2 and 3 of i swapped), which makes the
// eight values a lane holds per k-step consecutive hidden units.
typedef __attribute__((ext_vector_type(2))) float f32x2;

__device__ __forceinline__ int sigma_row(int r) { return (r & 0x13) | ((r & 4) << 1) | ((r & 8) >> 1); }

//
// BLOCK: the whole transition block of an Evoformer layer in place, out += transition(LayerNorm(out)) with x == out.
// The rows are normalised between their coalesced load and the fragment staging (a row's 16-byte chunks sit in the 8
// lanes that loaded them: sums by DPP adds, arithmetic of reference src/normalization/layernorm_kernel.h:21-53), and
// the epilogue re-reads the rows in the order it writes them and adds.  One read and one write of the activation
// for LayerNorm, both linears and the residual.
template <int CO, int RB, bool BLOCK, int WAVES = 4>
__global__ __launch_bounds__(64 * WAVES, 1) void transition_fused_kernel(const bf16_t *__restrict__ x,
                                                                 const bf16_t *__restrict__ w1,
                                                                 const float *__restrict__ b1,
                                                                 const bf16_t *__restrict__ w2,
                                                                 const float *__restrict__ b2, bf16_t *__restrict__ out,
                                                                 int64_t rows, int c_i, const float *__restrict__ ln_gamma,
                                                                 const float *__restrict__ ln_beta, float ln_eps)
{
    constexpr int KS = CO / 16; // k-steps of the first product
    constexpr int CP = CO / 64; // 64-column panels across a row of x or W1
    constexpr int CB = CO / 32; // 32-channel blocks of the output
    constexpr int W1_PANELS = 2 * CP, STAGE_PANELS = W1_PANELS + CB, PPW = STAGE_PANELS / WAVES;
    static_assert(STAGE_PANELS % WAVES == 0, "every wave stages the same number of weight panels");
    extern __shared__ uint4 lds[]; // [2 stages][STAGE_PANELS][256 slots], one private panel per wave, b1 as fp32
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, g = lane >> 5, sr = sigma_row(r);
    uint4 *xpanel = lds + 2 * STAGE_PANELS * 256 + wave * 256;
    float *b1s = reinterpret_cast<float *>(lds + 2 * STAGE_PANELS * 256 + WAVES * 256);
    for (int i = tid; i < c_i; i += 64 * WAVES) {
        b1s[i] = b1[i]; // visible after the first barrier of the slice loop
    }

    int64_t row0 = ((int64_t)blockIdx.x * WAVES + wave) * (32 * RB);
    const bool active = row0 < rows;
    if (!active) {
        row0 = rows - 1; // keeps every address valid; nothing is stored
    }
    const int last_local = (int)((rows - row0 < 32 * RB ? rows - row0 : 32 * RB) - 1);
    const bf16_t *xb = x + row0 * CO;

    auto fetch = [&](int jc, PanelRegs *wr) {
        const int h0 = jc * 64;
#pragma unroll
        for (int i = 0; i < PPW; ++i) {
            const int pnl = wave * PPW + i;
            if (pnl < W1_PANELS) {
                wr[i] = panel_load(w1 + (int64_t)(h0 + 32 * (pnl / CP)) * CO, CO, 0, 31, (pnl % CP) * 64, lane);
            } else {
                wr[i] = panel_load(w2 + (int64_t)((pnl - W1_PANELS) * 32) * c_i, c_i, 0, 31, h0, lane);
            }
        }
    };
    PanelRegs wr[PPW];
    fetch(0, wr);

    bf16x8 xf[RB][KS];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        PanelRegs t[CP];
#pragma unroll
        for (int cp = 0; cp < CP; ++cp) {
            t[cp] = panel_load(xb, CO, rb * 32, last_local, cp * 64, lane);
        }
        if constexpr (BLOCK) {
            // lane (lane >> 3, lane & 7) holds chunk lane & 7 of every 64-channel panel of rows 8i + (lane >> 3)
            float gm[CP][8], bt[CP][8];
#pragma unroll
            for (int cp = 0; cp < CP; ++cp) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    gm[cp][e] = ln_gamma[cp * 64 + (lane & 7) * 8 + e];
                    bt[cp][e] = ln_beta[cp * 64 + (lane & 7) * 8 + e];
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                uint4 *regs[CP];
#pragma unroll
                for (int cp = 0; cp < CP; ++cp) {
                    regs[cp] = i == 0 ? &t[cp].r0 : i == 1 ? &t[cp].r1 : i == 2 ? &t[cp].r2 : &t[cp].r3;
                }
                const float x0 = __shfl(to_f32(as_bf16x8(*regs[0])[0]), lane & ~7, 64); // first element of the row
                float s1 = 0.f, s2 = 0.f;
#pragma unroll
                for (int cp = 0; cp < CP; ++cp) {
                    const bf16x8 b = as_bf16x8(*regs[cp]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float d = to_f32(b[e]) - x0;
                        s1 += d;
                        s2 = fmaf(d, d, s2);
                    }
                }
                s1 = group_sum<8>(s1);
                s2 = group_sum<8>(s2);
                const float n = (float)CO;
                const float mean = s1 / n + x0;
                const float var = fmaxf((s2 - s1 * s1 / n) / n, 0.f);
                const float rstd = 1.0f / sqrtf(var + ln_eps);
                const float shift = -rstd * mean;
#pragma unroll
                for (int cp = 0; cp < CP; ++cp) {
                    const bf16x8 b = as_bf16x8(*regs[cp]);
                    bf16x8 o;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        o[e] = (bf16_t)fmaf(fmaf(to_f32(b[e]), rstd, shift), gm[cp][e], bt[cp][e]);
                    }
                    *regs[cp] = as_uint4(o);
                }
            }
        }
#pragma unroll
        for (int cp = 0; cp < CP; ++cp) {
            panel_store(xpanel, lane, t[cp]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                xf[rb][cp * 4 + k] = as_bf16x8(xpanel[panel_slot(r, 2 * k + g)]);
            }
        }
    }

    f32x16 oacc[RB][CB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
            oacc[rb][cb] = zero16();
        }
    }

    // Blocks of 32 hidden units, t = 0 .. c_i/32 - 1; block t lives in slice t/2.  The loop is software-pipelined by
    // hand: while the matrix core runs the first product of block t+1, the vector ALU turns the finished accumulators
    // of block t into the bf16 operand of its second product (bias, ReLU, rounding), whose MFMAs follow.  Fences keep
    // the compiler from pulling the two instruction streams apart again.
    auto first_product = [&](const uint4 *stage, int hb, f32x16 (&hn)[RB]) {
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            hn[rb] = zero16();
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 a = as_bf16x8(stage[(hb * CP + ks / 4) * 256 + panel_slot(sr, 2 * (ks % 4) + g)]);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                hn[rb] = mfma(a, xf[rb][ks], hn[rb]);
            }
        }
    };
    // element pair q of k-step s2 of block t: + b1, ReLU, round to bf16 (the pair form maps onto one conversion)
    auto convert_pair = [&](const f32x16 (&hc)[RB], const float *bp, int s2, int q, bf16x2 (&w)[RB][2][4]) {
        const f32x2 bias = *reinterpret_cast<const f32x2 *>(bp + 16 * s2 + 2 * q);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
            const f32x2 pr = {fmaxf(hc[rb][8 * s2 + 2 * q] + bias[0], 0.f), fmaxf(hc[rb][8 * s2 + 2 * q + 1] + bias[1], 0.f)};
            w[rb][s2][q] = __builtin_convertvector(pr, bf16x2);
        }
    };
    // first product of the next block (if any) interleaved with the conversion of the current one
    auto overlap = [&](const uint4 *stage_next, int hb_next, bool have_next, f32x16 (&hn)[RB], const f32x16 (&hc)[RB], int t,
                       bf16x8 (&hf)[RB][2]) {
        const float *bp = b1s + t * 32 + 8 * g;
        bf16x2 w[RB][2][4];
        if (have_next) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
                hn[rb] = zero16();
            }
            constexpr int PER = KS / 8; // k-steps per converted pair
            // all weight fragments of the block are requested up front: with one wave per SIMD nothing else hides an
            // LDS round trip, and the fences below would otherwise pin each read right in front of its MFMA
            bf16x8 af[KS];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                af[ks] = as_bf16x8(stage_next[(hb_next * CP + ks / 4) * 256 + panel_slot(sr, 2 * (ks % 4) + g)]);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const bf16x8 a = af[ks];
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    hn[rb] = mfma(a, xf[rb][ks], hn[rb]);
                }
                if (ks % PER == 0) {
                    convert_pair(hc, bp, (ks / PER) >> 2, (ks / PER) & 3, w);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                convert_pair(hc, bp, i >> 2, i & 3, w);
            }
        }
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                const bf16x8 all = {w[rb][s2][0][0], w[rb][s2][0][1], w[rb][s2][1][0], w[rb][s2][1][1],
                                    w[rb][s2][2][0], w[rb][s2][2][1], w[rb][s2][3][0], w[rb][s2][3][1]};
                hf[rb][s2] = all;
            }
        }
    };
    auto second_fragments = [&](const uint4 *stage, int hb, bf16x8 (&a2)[CB][2]) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
                a2[cb][s2] = as_bf16x8(stage[(W1_PANELS + cb) * 256 + panel_slot(r, 2 * (2 * hb + s2) + g)]);
            }
        }
    };
    auto second_product = [&](const bf16x8 (&a2)[CB][2], const bf16x8 (&hf)[RB][2]) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) {
#pragma unroll
            for (int s2 = 0; s2 < 2; ++s2) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) {
                    oacc[rb][cb] = mfma(a2[cb][s2], hf[rb][s2], oacc[rb][cb]);
                }
            }
        }
    };

    const int NJ = c_i / 64;
#pragma unroll
    for (int i = 0; i < PPW; ++i) {
        panel_store(lds + (wave * PPW + i) * 256, lane, wr[i]);
    }
    __syncthreads();
    if (NJ > 1) {
        fetch(1, wr);
    }
    f32x16 ha[RB], hb_[RB];
    first_product(lds, 0, ha);
    for (int jc = 0; jc < NJ; ++jc) {
        const uint4 *stage = lds + (jc & 1) * STAGE_PANELS * 256;
        uint4 *other = lds + ((jc + 1) & 1) * STAGE_PANELS * 256;
        const bool more = jc + 1 < NJ;
        // every wave is done with the other stage (its last readers were the second products of the previous slice)
        __syncthreads();
        if (more) {
#pragma unroll
            for (int i = 0; i < PPW; ++i) {
                panel_store(other + (wave * PPW + i) * 256, lane, wr[i]);
            }
            if (jc + 2 < NJ) {
                fetch(jc + 2, wr);
            }
        }
        bf16x8 hf[RB][2], a2[CB][2];
        second_fragments(stage, 0, a2); // on their way while the first product of the next block runs
        overlap(stage, 1, true, hb_, ha, 2 * jc, hf);
        second_product(a2, hf);
        __syncthreads(); // the other stage is complete and visible before the first product of its block 0 reads it
        second_fragments(stage, 1, a2);
        overlap(other, 0, more, ha, hb_, 2 * jc + 1, hf);
        second_product(a2, hf);
    }

    // accumulators (+ b2) -> bf16 through the private panel, 64 channels at a time, out as whole 128-byte runs
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
        for (int half = 0; half < CB / 2; ++half) {
#pragma unroll
            for (int n = 0; n < 2; ++n) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    const f32x4 bv = *reinterpret_cast<const f32x4 *>(b2 + (2 * half + n) * 32 + 8 * a + 4 * g);
                    bf16x4 ov;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        ov[c] = (bf16_t)(oacc[rb][2 * half + n][4 * a + c] + bv[c]);
                    }
                    *(reinterpret_cast<bf16x4 *>(xpanel + panel_slot(r, n * 4 + a)) + g) = ov;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int prow = 8 * i + (lane >> 3);
                uint4 v = xpanel[panel_slot(prow, lane & 7)];
                if (active && rb * 32 + prow <= last_local) {
                    bf16_t *dst = out + (row0 + rb * 32 + prow) * CO + half * 64 + (lane & 7) * 8;
                    if constexpr (BLOCK) { // residual: the row as it was before the LayerNorm
                        const bf16x8 o = as_bf16x8(v), z = as_bf16x8(*reinterpret_cast<const uint4 *>(dst));
                        bf16x8 res;
#pragma unroll
                        for (int e = 0; e < 8; ++e) {
                            res[e] = (bf16_t)(to_f32(z[e]) + to_f32(o[e]));
                        }
                        v = as_uint4(res);
                    }
                    *reinterpret_cast<uint4 *>(dst) = v;
                }
            }
        }
    }
}

// Gated projection of the triangle multiplication for 128 pair channels and 128 projected channels
// (reference src/attention/triangle_multiplication.cpp:37-66):
//   out[c][p] = bf16( bf16(x[p] . wp[c] + bp[c]) * mask[p] * sigmoid(x[p] . wg[c] + bg[c]) )
// over positions p of the pair tensor, written channel-first (the gate is not rounded to bf16 on its way into the
// sigmoid as it is in the reference, which stores it; the result is the closer one to exact arithmetic).  HBM-bound (256 bytes in, 256 bytes out per
// position), so the layout follows the row-projection kernel of the attention: both weight matrices stay in
// LDS in fragment order for the life of the workgroup (64 KB), every wave streams ranges of 64 positions whose
// rows it fetches as whole cache lines one step ahead, and the products are formed with positions as MFMA rows
// and channels as columns: a lane then owns one channel and four consecutive positions per accumulator group,
// which is the order of the channel-first output -- an 8-byte panel write, then 128-byte runs per channel.
// SIDES = 2: the left and the right projection of the triangle multiplication in one pass over the activation (a
// workgroup of eight waves, all four weight matrices in LDS: 128 KB + eight panels, the whole 160 KB).
struct GatedSide {
    const bf16_t *wp, *wg;
    const float *bp, *bg;
    bf16_t *out;
};

template <int SIDES>
__global__ __launch_bounds__(256 * SIDES, 2 / SIDES) void gated_projection_kernel(const bf16_t *__restrict__ x, GatedSide s0,
                                                                                 GatedSide s1,
                                                                                 const bf16_t *__restrict__ mask,
                                                                                 int64_t out_ld, int64_t n_pos, int pos_per_wave)
{
    constexpr int C = 128, CK = C / 16, WAVES = 4 * SIDES, THREADS = 64 * WAVES;
    extern __shared__ uint4 lds[]; // [SIDES][2 matrices][4 channel blocks][CK][64 lanes], then one panel per wave
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    uint4 *panel = lds + SIDES * 2 * 4 * CK * 64 + wave * 256;
    const int64_t start = ((int64_t)blockIdx.x * WAVES + wave) * pos_per_wave;
    const int64_t stop = start + pos_per_wave < n_pos ? start + pos_per_wave : n_pos;
    const int last = (int)(stop - start) - 1; // last valid position of the range, relative to start
    const bf16_t *xb = x + start * C;
    // two 32-row blocks x two 64-column halves per step; the first three are asked for a step ahead, the fourth at the
    // top of its own step (a fourth set of registers held across the channel loop does not fit)
    PanelRegs t[4];
    if (start < stop) {
#pragma unroll
        for (int q = 0; q < 3; ++q) {
            t[q] = panel_load(xb, C, (q >> 1) * 32, last, (q & 1) * 64, lane);
        }
    }
    {
        constexpr int PER = SIDES * 2 * 4 * CK * 64 / THREADS;
        uint4 wreg[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + i * THREADS;
            const int mat = idx / (4 * CK * 64), nb_ = (idx / (CK * 64)) % 4, ks = (idx >> 6) % CK, ln = idx & 63;
            const GatedSide &sd = (SIDES == 2 && mat >= 2) ? s1 : s0;
            const bf16_t *w = (mat & 1) ? sd.wg : sd.wp;
            wreg[i] = *reinterpret_cast<const uint4 *>(w + (int64_t)(nb_ * 32 + (ln & 31)) * C + ks * 16 + (ln >> 5) * 8);
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            lds[tid + i * THREADS] = wreg[i];
        }
    }
    __syncthreads();
    for (int64_t base = start; base < stop; base += 64) {
        const int rel = (int)(base - start);
        // the lane index is opaque to the optimiser inside a step, so that panel offsets and store addresses are formed
        // where they are used instead of being kept (and spilled) across the loop
        int lv = lane;
        asm volatile("" : "+v"(lv));
        const int rv = lv & 31, gv = lv >> 5;
        bf16x8 af[2][CK];
        t[3] = panel_load(xb, C, rel + 32, last, 64, lv);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            panel_store(panel, lv, t[q]);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                af[q >> 1][(q & 1) * 4 + k] = as_bf16x8(panel[panel_slot(rv, 2 * k + gv)]);
            }
        }
        {
            const int nrel = base + 64 < stop ? rel + 64 : rel; // clamped: one harmless re-read at the end
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                t[q] = panel_load(xb, C, nrel + (q >> 1) * 32, last, (q & 1) * 64, lv);
            }
        }
#pragma unroll 1
        for (int sn = 0; sn < 4 * SIDES; ++sn) { // 32 channels of one side at a time
            const int n = sn & 3;
            const GatedSide &sd = (SIDES == 2 && sn >= 4) ? s1 : s0;
            const uint4 *wside = lds + (sn >> 2) * 2 * 4 * CK * 64;
            bf16_t *out = sd.out;
            // projection first, rounded to bf16 and parked as packed pairs, then the gate: half the accumulators live
            const float pbias = sd.bp[n * 32 + rv], gneg = -LOG2E * sd.bg[n * 32 + rv];
            bf16x8 pp[2][2];
            {
                f32x16 pa[2];
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
                    pa[rb] = zero16();
                }
#pragma unroll
                for (int ks = 0; ks < CK; ++ks) {
                    const bf16x8 wpf = as_bf16x8(wside[(n * CK + ks) * 64 + lv]);
#pragma unroll
                    for (int rb = 0; rb < 2; ++rb) {
                        pa[rb] = mfma(af[rb][ks], wpf, pa[rb]);
                    }
                }
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        pa[rb][v] += pbias;
                    }
                    pp[rb][0] = pack8(pa[rb], 0), pp[rb][1] = pack8(pa[rb], 8);
                }
            }
            f32x16 ga[2];
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                ga[rb] = zero16();
            }
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                const bf16x8 wgf = as_bf16x8(wside[((4 + n) * CK + ks) * 64 + lv]);
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
                    ga[rb] = mfma(af[rb][ks], wgf, ga[rb]);
                }
            }
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
                for (int a = 0; a < 4; ++a) {
                    // mask of the lv's four consecutive positions (re-read per channel block: it stays in the L1)
                    int64_t p0 = base + rb * 32 + 8 * a + 4 * gv;
                    p0 = p0 + 4 <= n_pos ? p0 : n_pos - 4; // positions past the end are never stored
                    const bf16x4 mk = *reinterpret_cast<const bf16x4 *>(mask + p0);
                    bf16x4 ov;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float pv = to_f32(pp[rb][a >> 1][4 * (a & 1) + c]) * to_f32(mk[c]);
                        // sigmoid(gate + bias) = 1 / (1 + 2^-(gate*log2e + bias*log2e)); the gate stays in fp32
                        const float e = __builtin_amdgcn_exp2f(fmaf(ga[rb][4 * a + c], -LOG2E, gneg));
                        ov[c] = (bf16_t)(pv * __builtin_amdgcn_rcpf(1.0f + e));
                    }
                    *(reinterpret_cast<bf16x4 *>(panel + panel_slot(rv, rb * 4 + a)) + gv) = ov;
                }
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ch = 8 * i + (lv >> 3);
                const uint4 v = panel[panel_slot(ch, lv & 7)];
                const int64_t p0 = base + (lv & 7) * 8;
                if (p0 < stop) {
                    *reinterpret_cast<uint4 *>(out + (int64_t)(n * 32 + ch) * out_ld + p0) = v;
                }
            }
        }
    }
}

// The gated projection with the weights in registers and the activation shared through the LDS.  In the kernel above
// every wave multiplies its own positions by all four weight matrices, whose fragments it reads from the LDS for every
// step: 128 KB of LDS reads per wave and step of 64 positions, and whole steps as the unit of work (at 384 x 384
// positions a CU has nine steps for eight waves).  Here a workgroup takes the steps one after the other and a wave owns
// 32 output channels of one side: its two 32 x 128 weight blocks (projection and gate) stay in 64 registers, and per
// step it reads the 64 x 128 activation (16 KB, loaded once per workgroup straight into the LDS, a ring of stages
// requested RING - 1 steps ahead) and the mask (128 bytes, each wave's own copy), multiplies, gates and writes 32
// channels x 128 bytes.  Eight equal shares of every step, an eighth of the LDS reads.  Same arithmetic in the same
// order as the kernel above: the results are bit-identical.
template <int SIDES>
__global__ __launch_bounds__(256 * SIDES, 2 / SIDES) void gated_projection_blocks_kernel(const bf16_t *__restrict__ x, GatedSide s0, GatedSide s1,
                                                                                        const bf16_t *__restrict__ mask, int64_t out_ld,
                                                                                        int64_t n_pos, int steps_per_group)
{
    typedef __attribute__((address_space(3))) void *lds_ptr;
    constexpr int C = 128, CK = C / 16, WAVES = 4 * SIDES, RING = SIDES == 2 ? 4 : 3, UNITS = 16 / WAVES;
    constexpr int STAGE_SLOTS = 1024; // 64 positions x 256 bytes
    constexpr int WAVE_SLOTS = 256 + RING * 16; // a panel for the way out, and RING mask rows of 256 bytes
    extern __shared__ uint4 lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rv = lane & 31, gv = lane >> 5;
    const GatedSide &sd = (SIDES == 2 && wave >= 4) ? s1 : s0;
    const int cb = wave & 3; // this wave's 32 channels
    uint4 *panel = lds + RING * STAGE_SLOTS + wave * WAVE_SLOTS;
    const uint4 *mask_rows = panel + 256;

    const int64_t total_steps = (n_pos + 63) / 64;
    const int64_t first = (int64_t)blockIdx.x * steps_per_group;
    const int64_t stop = first + steps_per_group < total_steps ? first + steps_per_group : total_steps;
    if (first >= stop) {
        return;
    }

    // A stage holds its 64 rows of 256 bytes with the 16-byte slots of row r XOR-ed with r % 8 (the fragment reads, lane
    // -> its own row, then hit eight different bank groups per eight lanes).  A request is a unit of four rows: lane l
    // writes slot l % 16 of row l / 16 and fetches the chunk that belongs there.  Units past the last position fetch the
    // last four positions again (their results are never stored), so every wave issues the same number of requests,
    // which the waits below count.
    uint32_t lane_bytes[2]; // for even and odd units
#pragma unroll
    for (int par = 0; par < 2; ++par) {
        lane_bytes[par] = (uint32_t)((lane >> 4) * 256 + (((lane & 15) ^ ((4 * par + (lane >> 4)) & 7)) * 16));
    }
    const uint32_t x_lds = (uint32_t)(uintptr_t)(lds_ptr)lds, mask_lds = (uint32_t)(uintptr_t)(lds_ptr)mask_rows;
    auto request = [&](int64_t step, int slot) {
#pragma unroll
        for (int i = 0; i < UNITS; ++i) {
            const int u = wave * UNITS + i;
            int64_t pos = step * 64 + 4 * u;
            pos = pos + 4 <= n_pos ? pos : n_pos - 4;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(x_lds + slot * (STAGE_SLOTS * 16u) + u * 1024u),
                         "v"(lane_bytes[i & 1]), "s"(x + pos * C)
                         : "memory");
        }
        // the mask of the step's positions, two per lane (lanes 32-63 repeat lanes 0-31); past the end: the last two
        const uint32_t last_pair = (uint32_t)(n_pos - step * 64 - 2) * 2u;
        const uint32_t mine = 4u * (uint32_t)(lane & 31);
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2" ::"s"(mask_lds + slot * 256u), "v"(mine < last_pair ? mine : last_pair),
                     "s"(mask + step * 64)
                     : "memory");
    };
    auto ring = [](int slot) { return slot >= RING ? slot - RING : slot; };

    // requests are issued RING - 1 steps ahead; a step that lies past this workgroup's last one fetches the last one again
#pragma unroll
    for (int d = 0; d < RING - 1; ++d) {
        request(first + d < stop ? first + d : stop - 1, d);
    }
    bf16x8 wp[CK], wg[CK];
#pragma unroll
    for (int ks = 0; ks < CK; ++ks) {
        wp[ks] = *reinterpret_cast<const bf16x8 *>(sd.wp + (int64_t)(cb * 32 + rv) * C + ks * 16 + gv * 8);
        wg[ks] = *reinterpret_cast<const bf16x8 *>(sd.wg + (int64_t)(cb * 32 + rv) * C + ks * 16 + gv * 8);
    }
    float pbias = sd.bp[cb * 32 + rv], gneg = -LOG2E * sd.bg[cb * 32 + rv];
    // The weights are asked for behind the first requests and waited for here, before the loop: the compiler does not
    // know of the requests, and a wait it places for one of its own loads waits for every request issued before that
    // load -- once, here, that is one memory round trip for both; inside the loop it would stall every step.
#pragma unroll
    for (int ks = 0; ks < CK; ++ks) {
        asm volatile("" : "+v"(wp[ks]), "+v"(wg[ks]));
    }
    asm volatile("" : "+v"(pbias), "+v"(gneg));

    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
    int slot = 0;
    for (int64_t step = first; step < stop; ++step) {
        {
            const int64_t ahead = step + RING - 1;
            request(ahead < stop ? ahead : stop - 1, ring(slot + RING - 1));
        }
        const uint4 *stage = lds + slot * STAGE_SLOTS;
        const char *mrow = reinterpret_cast<const char *>(mask_rows + slot * 16);
        const int64_t base = step * 64;
        bf16x8 af[2][CK];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
                af[rb][ks] = as_bf16x8(stage[(rb * 32 + rv) * 16 + ((2 * ks + gv) ^ (rv & 7))]);
            }
        }
        // projection first, rounded to bf16 and parked as packed pairs, then the gate: half the accumulators live
        bf16x8 pp[2][2];
        {
            f32x16 pa[2];
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                pa[rb] = zero16();
            }
#pragma unroll
            for (int ks = 0; ks < CK; ++ks) {
#pragma unroll
                for (int rb = 0; rb < 2; ++rb) {
                    pa[rb] = mfma(af[rb][ks], wp[ks], pa[rb]);
                }
            }
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    pa[rb][v] += pbias;
                }
                pp[rb][0] = pack8(pa[rb], 0), pp[rb][1] = pack8(pa[rb], 8);
            }
        }
        f32x16 ga[2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            ga[rb] = zero16();
        }
#pragma unroll
        for (int ks = 0; ks < CK; ++ks) {
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                ga[rb] = mfma(af[rb][ks], wg[ks], ga[rb]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const bf16x4 mk = *reinterpret_cast<const bf16x4 *>(mrow + 2 * (rb * 32 + 8 * a + 4 * gv)); // the lane's four consecutive positions
                bf16x4 ov;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float pv = to_f32(pp[rb][a >> 1][4 * (a & 1) + c]) * to_f32(mk[c]);
                    // sigmoid(gate + bias) = 1 / (1 + 2^-(gate*log2e + bias*log2e)); the gate stays in fp32
                    const float e = __builtin_amdgcn_exp2f(fmaf(ga[rb][4 * a + c], -LOG2E, gneg));
                    ov[c] = (bf16_t)(pv * __builtin_amdgcn_rcpf(1.0f + e));
                }
                *(reinterpret_cast<bf16x4 *>(panel + panel_slot(rv, rb * 4 + a)) + gv) = ov;
            }
        }
        {
            // 32 channels x eight 16-byte pieces of 8 positions; the pieces past the last position repeat the last valid
            // one (same data to the same address), so that the stores, too, are the same number in every step
            const int64_t left = n_pos - base;
            const int valid = left >= 64 ? 8 : (int)(left >> 3);
            const int piece = (lane & 7) < valid ? (lane & 7) : valid - 1;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int ch = 8 * i + (lane >> 3);
                const uint4 v = panel[panel_slot(ch, piece)];
                *reinterpret_cast<uint4 *>(sd.out + (int64_t)(cb * 32 + ch) * out_ld + base + piece * 8) = v;
            }
        }
        // The next step's stage has landed when nothing older than what this wave has issued since its request is in
        // flight: the requests of the steps after it (UNITS + 1 each) and four stores per step gone by.  Behind the
        // barrier every wave's part of it has, and every wave has left this step's stage.
        const int64_t gone = step - first;
        if constexpr (RING == 4) {
            if (gone == 0) {
                asm volatile("s_waitcnt vmcnt(10)\n\ts_barrier" ::: "memory");
            } else if (gone == 1) {
                asm volatile("s_waitcnt vmcnt(14)\n\ts_barrier" ::: "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(18)\n\ts_barrier" ::: "memory");
            }
        } else {
            if (gone == 0) {
                asm volatile("s_waitcnt vmcnt(9)\n\ts_barrier" ::: "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(13)\n\ts_barrier" ::: "memory");
            }
        }
        slot = ring(slot + 1);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // requests repeated past the last step: let them land before the LDS is given back
}

// Any strides, any sizes: one thread per element of C, same epilogues and rounding points.
__global__ __launch_bounds__(256) void pair_gemm_scalar_kernel(const GemmParams p)
{
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t per = (int64_t)p.M * p.N;
    if (idx >= per * p.batches) {
        return;
    }
    const int batch = (int)(idx / per);
    const int m = (int)((idx % per) / p.N), n = (int)(idx % p.N);
    const bf16_t *a = p.a + (int64_t)batch * p.a_sb + (int64_t)m * p.a_sm;
    const bf16_t *b = p.b + (int64_t)batch * p.b_sb + (int64_t)n * p.b_sn;
    float s = 0.f, sg = 0.f;
    for (int k = 0; k < p.K; ++k) {
        const float bv = to_f32(b[(int64_t)k * p.b_sk]);
        s = fmaf(to_f32(a[(int64_t)k * p.a_sk]), bv, s);
        if (p.a_gate) {
            sg = fmaf(to_f32(p.a_gate[(int64_t)batch * p.a_sb + (int64_t)m * p.a_sm + (int64_t)k * p.a_sk]), bv, sg);
        }
    }
    const int bi = p.bias_axis == 1 ? n : m;
    if (p.bias_axis != 0) {
        s += p.bias[bi];
    }
    if (p.relu) {
        s = fmaxf(s, 0.f);
    }
    float out = s;
    if (p.a_gate) {
        if (p.bias_axis != 0) {
            sg += p.bias_gate[bi];
        }
        const float mv = to_f32(p.mask[(int64_t)batch * p.mask_sb + n]);
        out = to_f32((bf16_t)s) * mv * sigmoid_fast(to_f32((bf16_t)sg));
    }
    p.c[(int64_t)batch * p.c_sb + (int64_t)m * p.c_sm + n] = (bf16_t)out;
}

// out[r][c] *= sigmoid(gate[r][c]) over rows r = (i, j) of two strided [n0, n1, size] tensors
// (reference triangle_multiplication.cpp:129-150).
template <bool VEC>
__global__ __launch_bounds__(256) void sigmoid_gate_rows_kernel(bf16_t *__restrict__ out, int64_t out_s0, int64_t out_s1,
                                                                const bf16_t *__restrict__ gate, int64_t gate_s0,
                                                                int64_t gate_s1, int64_t n0, int64_t n1, int size)
{
    constexpr int W = VEC ? 8 : 1;
    const int per_row = (size + W - 1) / W;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n0 * n1 * per_row) {
        return;
    }
    const int64_t row = idx / per_row;
    const int col = (int)(idx % per_row) * W;
    const int64_t i = row / n1, j = row % n1;
    bf16_t *o = out + i * out_s0 + j * out_s1 + col;
    const bf16_t *gt = gate + i * gate_s0 + j * gate_s1 + col;
    if constexpr (VEC) {
        const bf16x8 ov = *reinterpret_cast<const bf16x8 *>(o), gv = *reinterpret_cast<const bf16x8 *>(gt);
        bf16x8 res;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            res[e] = (bf16_t)(to_f32(ov[e]) * sigmoid_fast(to_f32(gv[e])));
        }
        *reinterpret_cast<bf16x8 *>(o) = res;
    } else {
        *o = (bf16_t)(to_f32(*o) * sigmoid_fast(to_f32(*gt)));
    }
}

// does this operand suit the 16-byte loads of the MFMA kernel?  rows = extent of the non-k index
bool operand_ok(const void *ptr, int64_t s_row, int64_t s_k, int64_t s_batch, int64_t rows, int64_t K, bool &mmajor)
{
    if (!kutacc_hip_aligned16(ptr) || s_batch % 8 != 0) {
        return false;
    }
    if (s_k == 1) {
        mmajor = false;
        return s_row % 8 == 0 && K % 8 == 0;
    }
    if (s_row == 1) {
        mmajor = true;
        return s_k % 8 == 0 && rows % 8 == 0 && rows >= 8;
    }
    return false;
}

template <bool AM, bool BM, bool G>
hipError_t launch_tiles(const GemmParams &p, int64_t blocks, hipStream_t stream)
{
    static size_t configured[KUTACC_DEVICE_SLOTS] = {}; // per instantiation and device: dynamic LDS is set through the opt-in
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&pair_gemm_kernel<AM, BM, G>), GEMM_LDS, configured)) {
        return e;
    }
    pair_gemm_kernel<AM, BM, G><<<dim3((unsigned)blocks), 256, GEMM_LDS, stream>>>(p);
    return hipGetLastError();
}

template <bool MM, int BW>
hipError_t launch_big_tiles(const GemmParams &p, int64_t blocks, hipStream_t stream)
{
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&pair_gemm_big_kernel<MM, BW>), BIG_GEMM_LDS, configured)) {
        return e;
    }
    int device = 0, cus = 0;
    if (hipError_t e = hipGetDevice(&device)) {
        return e;
    }
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device)) {
        return e;
    }
    // one workgroup per CU; a multiple of 8, so that a workgroup's tiles stay on its XCD's share of the walk
    const int64_t grid = blocks < cus ? blocks : (cus >= 8 ? cus / 8 * 8 : cus);
    pair_gemm_big_kernel<MM, BW><<<dim3((unsigned)grid), 256, BIG_GEMM_LDS, stream>>>(p, blocks);
    return hipGetLastError();
}

template <bool MM>
hipError_t launch_direct_tiles(const GemmParams &p, int64_t blocks, hipStream_t stream)
{
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&pair_gemm_direct_kernel<MM>), DIRECT_GEMM_LDS, configured)) {
        return e;
    }
    int device = 0, cus = 0;
    if (hipError_t e = hipGetDevice(&device)) {
        return e;
    }
    if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device)) {
        return e;
    }
    const int64_t grid = blocks < cus ? blocks : (cus >= 8 ? cus / 8 * 8 : cus);
    pair_gemm_direct_kernel<MM><<<dim3((unsigned)grid), 256, DIRECT_GEMM_LDS, stream>>>(p, blocks);
    return hipGetLastError();
}

// 0: the 256 x 256 tiles with operands loaded straight into the LDS where every CU gets at least two of them (measured
// at 128 channels, outgoing / incoming, against the next best form: 512 x 512 46 / 44 us against 49-56 / 58; 768 x 768
// 150 / 134 against 154 / 158; 1024 x 1024 281-289 / 270 against 308 / 322; 256 x 256, one tile per two CUs, loses:
// 14.3 against 12.4), else the 192 x 192 tiles where every CU gets at least two (384 x 384: 24.6 us against 25.8-26.6;
// 576 x 576: 74-78 against 79-86; 192 x 192 loses), else the 128 x 128 tiles; 4: the direct 256 x 256 tiles wherever the
// shape has whole ones; 1: the 256 x 256 tiles staged through registers wherever it has; 3: 192 x 192 likewise; 2: none
// of them
std::atomic<int> g_big_tile_mode{0};
constexpr int64_t BIG_TILE_MIN_WORKGROUPS = 1024;

// which kernel takes a gated projection that gated_projection_fits(): 0 (default) and 1: the one with the weights in
// registers ("blocks"); 2: the streaming kernel; 3: the tiled kernel
std::atomic<int> g_gated_mode{0};

// the dedicated kernel of the gated projection: 128 -> 128 channels, dense operands, positions in whole 16-byte runs
bool gated_projection_fits(const kutacc_hip_gemm_args_t &g)
{
    return g.a_gate && g.mask && g.bias_axis == 2 && g.bias && g.bias_gate && g.batches == 1 && g.m == 128 && g.k == 128 &&
           g.a_stride_k == 1 && g.a_stride_m == 128 && g.b_stride_k == 1 && g.b_stride_n == 128 && g.n % 8 == 0 && g.n >= 8 &&
           g.c_stride_m % 8 == 0 && kutacc_hip_aligned16(g.a) && kutacc_hip_aligned16(g.a_gate) && kutacc_hip_aligned16(g.b) && kutacc_hip_aligned16(g.c) &&
           (reinterpret_cast<uintptr_t>(g.mask) & 7u) == 0 && !g.relu;
}

template <int SIDES>
hipError_t launch_gated_projection(const kutacc_hip_gemm_args_t &g, const kutacc_hip_gemm_args_t *second, hipStream_t stream)
{
    constexpr int WAVES = 4 * SIDES;
    constexpr size_t lds_bytes = (size_t)SIDES * 2 * 4 * 8 * 64 * 16 + WAVES * 4096;
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    static int cu_table[KUTACC_DEVICE_SLOTS] = {};
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&gated_projection_kernel<SIDES>), lds_bytes, configured)) {
        return e;
    }
    const int cus = kutacc_device_attribute(hipDeviceAttributeMultiprocessorCount, 256, cu_table);
    // eight resident waves per CU (two workgroups of four, or one of eight), every wave an equal range of positions (a
    // multiple of 8; the last step of a range may be partial)
    const int64_t tiles = (g.n + 63) / 64;
    int64_t gx = (tiles + WAVES - 1) / WAVES;
    const int64_t cap = (int64_t)cus * (2 / SIDES);
    gx = gx > cap ? cap : gx;
    const int64_t ppw = ((g.n + gx * WAVES - 1) / (gx * WAVES) + 7) / 8 * 8;
    const GatedSide s0 = {(const bf16_t *)g.a, (const bf16_t *)g.a_gate, g.bias, g.bias_gate, (bf16_t *)g.c};
    GatedSide s1 = s0;
    if (SIDES == 2) {
        s1 = GatedSide{(const bf16_t *)second->a, (const bf16_t *)second->a_gate, second->bias, second->bias_gate, (bf16_t *)second->c};
    }
    gated_projection_kernel<SIDES><<<dim3((unsigned)gx), 64 * WAVES, lds_bytes, stream>>>(
        (const bf16_t *)g.b, s0, s1, (const bf16_t *)g.mask, g.c_stride_m, g.n, (int)ppw);
    return hipGetLastError();
}

template <int SIDES>
hipError_t launch_gated_projection_blocks(const kutacc_hip_gemm_args_t &g, const kutacc_hip_gemm_args_t *second, hipStream_t stream)
{
    constexpr int WAVES = 4 * SIDES, RING = SIDES == 2 ? 4 : 3;
    constexpr size_t lds_bytes = (size_t)(RING * 1024 + WAVES * (256 + RING * 16)) * 16;
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    static int cu_table[KUTACC_DEVICE_SLOTS] = {};
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&gated_projection_blocks_kernel<SIDES>), lds_bytes, configured)) {
        return e;
    }
    const int cus = kutacc_device_attribute(hipDeviceAttributeMultiprocessorCount, 256, cu_table);
    // eight resident waves per CU (two workgroups of four, or one of eight); every workgroup an equal run of steps
    const int64_t steps = (g.n + 63) / 64;
    const int64_t cap = (int64_t)cus * (2 / SIDES);
    const int64_t groups = steps < cap ? steps : cap;
    const int64_t per_group = (steps + groups - 1) / groups;
    const GatedSide s0 = {(const bf16_t *)g.a, (const bf16_t *)g.a_gate, g.bias, g.bias_gate, (bf16_t *)g.c};
    GatedSide s1 = s0;
    if (SIDES == 2) {
        s1 = GatedSide{(const bf16_t *)second->a, (const bf16_t *)second->a_gate, second->bias, second->bias_gate, (bf16_t *)second->c};
    }
    gated_projection_blocks_kernel<SIDES><<<dim3((unsigned)((steps + per_group - 1) / per_group)), 64 * WAVES, lds_bytes, stream>>>(
        (const bf16_t *)g.b, s0, s1, (const bf16_t *)g.mask, g.c_stride_m, g.n, (int)per_group);
    return hipGetLastError();
}

constexpr int MAX_HIDDEN = 2048; // hidden units whose bias fits next to the weight stages in LDS

template <int CO, int RB, bool BLOCK, int WAVES = 4>
hipError_t launch_transition(const void *x, const void *w1, const float *b1, const void *w2, const float *b2, void *out,
                             int64_t rows, int c_i, const float *ln_gamma, const float *ln_beta, float ln_eps,
                             hipStream_t stream)
{
    constexpr int STAGE_PANELS = 2 * (CO / 64) + CO / 32;
    const size_t lds_bytes = (size_t)(2 * STAGE_PANELS + WAVES) * 4096 + (size_t)c_i * sizeof(float);
    static size_t configured[KUTACC_DEVICE_SLOTS] = {};
    if (const hipError_t e = kutacc_opt_in_lds(reinterpret_cast<const void *>(&transition_fused_kernel<CO, RB, BLOCK, WAVES>),
                                               (size_t)(2 * STAGE_PANELS + WAVES) * 4096 + MAX_HIDDEN * sizeof(float), configured)) {
        return e;
    }
    const int64_t per_group = 32 * RB * WAVES;
    const int64_t blocks = (rows + per_group - 1) / per_group;
    transition_fused_kernel<CO, RB, BLOCK, WAVES><<<dim3((unsigned)blocks), 64 * WAVES, lds_bytes, stream>>>(
        (const bf16_t *)x, (const bf16_t *)w1, b1, (const bf16_t *)w2, b2, (bf16_t *)out, rows, c_i, ln_gamma, ln_beta, ln_eps);
    return hipGetLastError();
}
} // namespace

namespace kutacc_launch {

bool transition_fused_supports(int64_t rows, int64_t c_o, int64_t c_i, const void *x, const void *w1, const float *b1,
                               const void *w2, const float *b2, const void *out)
{
    return (c_o == 128 || c_o == 256) && c_i >= 64 && c_i % 64 == 0 && c_i <= MAX_HIDDEN && rows > 0 &&
           rows <= ((int64_t)1 << 31) * 64 && kutacc_hip_aligned16(x) && kutacc_hip_aligned16(w1) && kutacc_hip_aligned16(b1) && kutacc_hip_aligned16(w2) &&
           kutacc_hip_aligned16(b2) && kutacc_hip_aligned16(out);
}

// 128 channels: eight waves of 32 rows each per workgroup (one workgroup per CU, two waves per SIMD, which hide each
// other's LDS round trips and barriers).  Measured against four waves of 64 rows, which reads every weight fragment from
// LDS half as often but leaves a SIMD to one wave: 12 % faster for the transition at n = 384, 14 % for the block with
// its LayerNorm and residual, 5 % and 17 % at n = 1024.  (With the four-wave kernel a separate, smaller-workgroup launch
// for the rows of a last, partial round of workgroups paid off; with this one it no longer does.)
template <bool BLOCK>
static hipError_t launch_transition_128(const void *x, const void *w1, const float *b1, const void *w2, const float *b2, void *out,
                                        int64_t rows, int c_i, const float *ln_gamma, const float *ln_beta, float ln_eps,
                                        hipStream_t stream)
{
    return launch_transition<128, 1, BLOCK, 8>(x, w1, b1, w2, b2, out, rows, c_i, ln_gamma, ln_beta, ln_eps, stream);
}

int transition_fused(const void *x, const void *w1, const float *b1, const void *w2, const float *b2, void *out,
                     int64_t rows, int64_t c_o, int64_t c_i, hipStream_t stream)
{
    if (!transition_fused_supports(rows, c_o, c_i, x, w1, b1, w2, b2, out)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("transition_fused_kernel", 4.0 * (double)rows * (double)c_o * (double)c_i, stream);
    const hipError_t e = c_o == 128 ? launch_transition_128<false>(x, w1, b1, w2, b2, out, rows, (int)c_i, nullptr, nullptr, 0.f, stream)
                                    : launch_transition<256, 1, false>(x, w1, b1, w2, b2, out, rows, (int)c_i, nullptr, nullptr, 0.f, stream);
    return kutacc_hip_status(e);
}

// act += transition(LayerNorm(act)) in place, one kernel
int transition_block_fused(void *act, const float *ln_gamma, const float *ln_beta, float ln_eps, const void *w1, const float *b1,
                           const void *w2, const float *b2, int64_t rows, int64_t c_o, int64_t c_i, hipStream_t stream)
{
    if (!ln_gamma || !ln_beta || !transition_fused_supports(rows, c_o, c_i, act, w1, b1, w2, b2, act)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("transition_fused_kernel<block>", 4.0 * (double)rows * (double)c_o * (double)c_i, stream);
    const hipError_t e =
        c_o == 128 ? launch_transition_128<true>(act, w1, b1, w2, b2, act, rows, (int)c_i, ln_gamma, ln_beta, ln_eps, stream)
                   : launch_transition<256, 1, true>(act, w1, b1, w2, b2, act, rows, (int)c_i, ln_gamma, ln_beta, ln_eps, stream);
    return kutacc_hip_status(e);
}

int pair_gemm_tuning(const char *name, const char *value)
{
    if (!std::strcmp(name, "gemm_tile")) { // "128", "256", "192", "direct": see g_big_tile_mode; anything else: the default rule
        g_big_tile_mode.store(value && !std::strcmp(value, "256") ? 1 : (value && !std::strcmp(value, "128") ? 2 : (value && !std::strcmp(value, "192") ? 3 : (value && !std::strcmp(value, "direct") ? 4 : 0))));
        return 0;
    }
    if (!std::strcmp(name, "gated_projection")) { // "blocks", "streaming", "tiled": see g_gated_mode; anything else: the default rule
        g_gated_mode.store(value && !std::strcmp(value, "blocks") ? 1 : (value && !std::strcmp(value, "streaming") ? 2 : (value && !std::strcmp(value, "tiled") ? 3 : 0)));
        return 0;
    }
    return KUTACC_HIP_EINVAL;
}

int pair_gemm(const kutacc_hip_gemm_args_t &g, hipStream_t stream, const kutacc_hip_gemm_args_t *second)
{
    if (g.m <= 0 || g.n <= 0 || g.k <= 0 || g.batches <= 0 || !g.a || !g.b || !g.c || g.dtype != KUTACC_DTYPE_BF16) {
        return KUTACC_HIP_EINVAL;
    }
    if (g.m > INT32_MAX / 2 || g.n > INT32_MAX / 2 || g.k > INT32_MAX / 2 || g.batches > INT32_MAX ||
        g.bias_axis < 0 || g.bias_axis > 2 || (g.bias_axis != 0 && !g.bias)) {
        return KUTACC_HIP_EINVAL;
    }
    const bool gated = g.a_gate != nullptr;
    if (gated && (!g.mask || (g.bias_axis != 0 && !g.bias_gate))) {
        return KUTACC_HIP_EINVAL;
    }
    GemmParams p;
    p.a = (const bf16_t *)g.a, p.a_gate = (const bf16_t *)g.a_gate, p.b = (const bf16_t *)g.b, p.c = (bf16_t *)g.c;
    p.a_sm = g.a_stride_m, p.a_sk = g.a_stride_k, p.a_sb = g.a_stride_batch;
    p.b_sn = g.b_stride_n, p.b_sk = g.b_stride_k, p.b_sb = g.b_stride_batch;
    p.c_sm = g.c_stride_m, p.c_sb = g.c_stride_batch;
    p.bias = g.bias, p.bias_gate = g.bias_gate, p.mask = (const bf16_t *)g.mask, p.mask_sb = g.mask_stride_batch;
    p.M = (int)g.m, p.N = (int)g.n, p.K = (int)g.k, p.batches = (int)g.batches;
    p.bias_axis = g.bias_axis, p.relu = g.relu ? 1 : 0;
    p.a_alt = p.a_gate_alt = nullptr, p.bias_alt = p.bias_gate_alt = nullptr, p.c_alt = nullptr;

    bool am = false, bm = false;
    bool mfma_ok = operand_ok(g.a, g.a_stride_m, g.a_stride_k, g.a_stride_batch, g.m, g.k, am) &&
                   operand_ok(g.b, g.b_stride_n, g.b_stride_k, g.b_stride_batch, g.n, g.k, bm) && kutacc_hip_aligned16(g.c) &&
                   g.c_stride_m % 8 == 0 && g.c_stride_batch % 8 == 0 && g.n % 8 == 0 &&
                   (g.bias_axis != 1 || kutacc_hip_aligned16(g.bias));
    if (gated) {
        mfma_ok = mfma_ok && !am && !bm && kutacc_hip_aligned16(g.a_gate) && kutacc_hip_aligned16(g.mask) && g.mask_stride_batch % 8 == 0 &&
                  (g.bias_axis != 1 || kutacc_hip_aligned16(g.bias_gate));
    }
    if (g.path == KUTACC_HIP_PATH_GENERIC) {
        mfma_ok = false;
    } else if (g.path == KUTACC_HIP_PATH_FUSED && !mfma_ok) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    // Gated projections of 128 channels on dense operands have kernels of their own (gated_projection_fits): by default
    // the one with the weights in registers, at every size (one side, us, against the tiled kernel up to 384 x 384
    // positions and the streaming kernel beyond: 256 x 256 12.7 against 14.2; 384 x 384 23-25 against 28; 512 x 512 30.5
    // against 39.7; 768 x 768 61 against 91; 1024 x 1024 143 against 144-147).
    if (second != nullptr) {
        // a second gated projection of the same B and mask (other weights, biases and result) rides along as batch 1 of
        // the tiled kernel, so that the tile of B both need comes from HBM once; any other route: the caller runs the two
        // separately
        const kutacc_hip_gemm_args_t &h = *second;
        const bool same = h.a_gate && h.m == g.m && h.n == g.n && h.k == g.k && h.batches == 1 && g.batches == 1 && h.b == g.b &&
                          h.mask == g.mask && h.a_stride_m == g.a_stride_m && h.a_stride_k == g.a_stride_k &&
                          h.b_stride_n == g.b_stride_n && h.b_stride_k == g.b_stride_k && h.c_stride_m == g.c_stride_m &&
                          h.bias_axis == g.bias_axis && h.relu == g.relu && h.dtype == g.dtype && h.a && h.c &&
                          (g.bias_axis == 0 || (h.bias && h.bias_gate)) &&
                          (g.bias_axis != 1 || (kutacc_hip_aligned16(h.bias) && kutacc_hip_aligned16(h.bias_gate))) && kutacc_hip_aligned16(h.a) &&
                          kutacc_hip_aligned16(h.a_gate) && kutacc_hip_aligned16(h.c);
        const int gated_mode = g_gated_mode.load();
        const bool dedicated = gated && gated_mode != 3 && gated_projection_fits(g) && gated_projection_fits(h) && g.n <= INT32_MAX / 2;
        if (!same || !gated || g.path == KUTACC_HIP_PATH_GENERIC) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        if (dedicated) { // both sides in one pass over the activation
            if (gated_mode == 2) {
                kutacc_prof::KernelTimer t("gated_projection_kernel<2>", 8.0 * (double)g.m * (double)g.n * (double)g.k, stream);
                return kutacc_hip_status(launch_gated_projection<2>(g, second, stream));
            }
            kutacc_prof::KernelTimer t("gated_projection_blocks_kernel<2>", 8.0 * (double)g.m * (double)g.n * (double)g.k, stream);
            return kutacc_hip_status(launch_gated_projection_blocks<2>(g, second, stream));
        }
        // (one that fits a dedicated kernel by itself: the caller runs the two separately)
        if (!mfma_ok || (gated_mode != 3 && gated_projection_fits(g))) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        p.a_alt = (const bf16_t *)h.a, p.a_gate_alt = (const bf16_t *)h.a_gate, p.bias_alt = h.bias, p.bias_gate_alt = h.bias_gate;
        p.c_alt = (bf16_t *)h.c;
        p.batches = 2;
    }
    if (g.path != KUTACC_HIP_PATH_GENERIC && gated && second == nullptr && g_gated_mode.load() != 3 && gated_projection_fits(g) &&
        g.n <= INT32_MAX / 2) {
        if (g_gated_mode.load() == 2) {
            kutacc_prof::KernelTimer t("gated_projection_kernel", 4.0 * (double)g.m * (double)g.n * (double)g.k, stream);
            return kutacc_hip_status(launch_gated_projection<1>(g, nullptr, stream));
        }
        kutacc_prof::KernelTimer t("gated_projection_blocks_kernel", 4.0 * (double)g.m * (double)g.n * (double)g.k, stream);
        return kutacc_hip_status(launch_gated_projection_blocks<1>(g, nullptr, stream));
    }
    // rows of 128 or 256 features against a dense weight matrix: the attention's output-projection kernel keeps
    // the weight slab in LDS and streams the rows, which suits these HBM-bound shapes better than square tiles
    if (mfma_ok && !gated && !am && !bm && g.batches == 1 && g.bias_axis == 1 && !g.relu && g.b_stride_n == g.k &&
        kutacc_launch::row_projection_supports(g.a, g.a_stride_m, g.b, g.bias, g.c, g.c_stride_m, g.m, g.n, g.k)) {
        return kutacc_launch::row_projection(g.a, g.a_stride_m, g.b, g.bias, g.c, g.c_stride_m, g.m, g.n, g.k, stream);
    }
    const double flops = 2.0 * (double)g.m * (double)g.n * (double)g.k * (double)p.batches * (gated ? 2.0 : 1.0);
    if (!mfma_ok) {
        const int64_t total = g.m * g.n * g.batches;
        const int64_t blocks = (total + 255) / 256;
        if (blocks > INT32_MAX) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        kutacc_prof::KernelTimer t("pair_gemm_scalar_kernel", flops, stream);
        pair_gemm_scalar_kernel<<<dim3((unsigned)blocks), 256, 0, stream>>>(p);
        return kutacc_hip_status(hipGetLastError());
    }
    // (whole tiles and k-steps, and lane offsets within 32 bits: the kernel's addresses are a uniform pointer plus a lane constant)
    const int tile_mode = g_big_tile_mode.load();
    if (!gated && am == bm && g.bias_axis == 0 && !g.relu && g.k % KSTEP == 0 && (am ? g.a_stride_k : g.a_stride_m) < (1 << 26) &&
        (bm ? g.b_stride_k : g.b_stride_n) < (1 << 26) && tile_mode != 2) {
        // (the direct kernel's lane offsets span the tile's 256 rows: pitches below 2^22 elements keep them in 32 bits)
        if ((tile_mode == 4 || tile_mode == 0) && (am ? g.a_stride_k : g.a_stride_m) < (1 << 22) && (bm ? g.b_stride_k : g.b_stride_n) < (1 << 22) &&
            g.m % BIG_TILE == 0 && g.n % BIG_TILE == 0 && g.k >= 3 * DIRECT_KSTEP && g.m / BIG_TILE * (g.n / BIG_TILE) * p.batches <= INT32_MAX &&
            (tile_mode == 4 || g.m / BIG_TILE * (g.n / BIG_TILE) * p.batches >= BIG_TILE_MIN_WORKGROUPS / 2)) {
            p.MT = (int)(g.m / BIG_TILE), p.NT = (int)(g.n / BIG_TILE);
            const int64_t big_blocks = (int64_t)p.MT * p.NT * p.batches;
            kutacc_prof::KernelTimer t(am ? "pair_gemm_direct_kernel<m-major>" : "pair_gemm_direct_kernel", flops, stream);
            return kutacc_hip_status(am ? launch_direct_tiles<true>(p, big_blocks, stream) : launch_direct_tiles<false>(p, big_blocks, stream));
        }
        // 256 x 256 tiles where every CU gets at least four; else 192 x 192 where every CU gets at least two
        for (const int side : {BIG_TILE, 192}) {
            const bool forced = tile_mode == (side == BIG_TILE ? 1 : 3);
            if (g.m % side != 0 || g.n % side != 0 || (!forced && tile_mode != 0)) {
                continue;
            }
            p.MT = (int)(g.m / side), p.NT = (int)(g.n / side);
            const int64_t big_blocks = (int64_t)p.MT * p.NT * p.batches;
            const int64_t enough = side == BIG_TILE ? BIG_TILE_MIN_WORKGROUPS : BIG_TILE_MIN_WORKGROUPS / 2;
            if (big_blocks <= INT32_MAX && (big_blocks >= enough || forced)) {
                kutacc_prof::KernelTimer t(side == BIG_TILE ? (am ? "pair_gemm_big_kernel<m-major>" : "pair_gemm_big_kernel")
                                                            : (am ? "pair_gemm_big_kernel<m-major, 192>" : "pair_gemm_big_kernel<192>"),
                                           flops, stream);
                const hipError_t e = side == BIG_TILE ? (am ? launch_big_tiles<true, 4>(p, big_blocks, stream) : launch_big_tiles<false, 4>(p, big_blocks, stream))
                                                      : (am ? launch_big_tiles<true, 3>(p, big_blocks, stream) : launch_big_tiles<false, 3>(p, big_blocks, stream));
                return kutacc_hip_status(e);
            }
        }
    }
    p.MT = (int)((g.m + (gated ? 64 : 128) - 1) / (gated ? 64 : 128));
    p.NT = (int)((g.n + 127) / 128);
    const int64_t blocks = (int64_t)p.MT * p.NT * p.batches;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t(gated ? "pair_gemm_kernel<gated>" : (am || bm ? "pair_gemm_kernel<m-major>" : "pair_gemm_kernel"),
                               flops, stream);
    hipError_t e;
    if (gated) {
        e = launch_tiles<false, false, true>(p, blocks, stream);
    } else if (am && bm) {
        e = launch_tiles<true, true, false>(p, blocks, stream);
    } else if (am) {
        e = launch_tiles<true, false, false>(p, blocks, stream);
    } else if (bm) {
        e = launch_tiles<false, true, false>(p, blocks, stream);
    } else {
        e = launch_tiles<false, false, false>(p, blocks, stream);
    }
    return kutacc_hip_status(e);
}

int sigmoid_gate_rows(void *out, int64_t out_s0, int64_t out_s1, const void *gate, int64_t gate_s0, int64_t gate_s1,
                      int64_t n0, int64_t n1, int64_t size, hipStream_t stream)
{
    if (!out || !gate || n0 <= 0 || n1 <= 0 || size <= 0 || size > INT32_MAX) {
        return KUTACC_HIP_EINVAL;
    }
    const bool vec = size % 8 == 0 && kutacc_hip_aligned16(out) && kutacc_hip_aligned16(gate) && out_s0 % 8 == 0 && out_s1 % 8 == 0 &&
                     gate_s0 % 8 == 0 && gate_s1 % 8 == 0;
    const int64_t per_row = vec ? size / 8 : size;
    if (n0 > INT64_MAX / n1 || n0 * n1 > INT64_MAX / per_row) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t blocks = (n0 * n1 * per_row + 255) / 256;
    if (blocks > INT32_MAX) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    kutacc_prof::KernelTimer t("sigmoid_gate_rows_kernel", 0.0, stream);
    if (vec) {
        sigmoid_gate_rows_kernel<true><<<dim3((unsigned)blocks), 256, 0, stream>>>(
            (bf16_t *)out, out_s0, out_s1, (const bf16_t *)gate, gate_s0, gate_s1, n0, n1, (int)size);
    } else {
        sigmoid_gate_rows_kernel<false><<<dim3((unsigned)blocks), 256, 0, stream>>>(
            (bf16_t *)out, out_s0, out_s1, (const bf16_t *)gate, gate_s0, gate_s1, n0, n1, (int)size);
    }
    return kutacc_hip_status(hipGetLastError());
}

} // namespace kutacc_launch
