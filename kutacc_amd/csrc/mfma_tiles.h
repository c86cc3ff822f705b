// MFMA tile helpers shared by the attention kernels (gfx950, bf16 operands, fp32 accumulation).
//
// Operand fragments use one format throughout: a [32 rows x 16 k] slab, lane l holding row (l & 31),
// k-chunk (l >> 5)*8..+8, i.e. 16 contiguous bytes of a row-major bf16 matrix.  Results of
// v_mfma_f32_32x32x16_bf16 come out as D[i][j] with j = l & 31 and i = 8*(v/4) + 4*(l>>5) + (v&3) for
// accumulator register v.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_util.h"

namespace kutacc_dev {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;


constexpr float LOG2E = 1.44269504088896340736f;

__device__ __forceinline__ int pi_row(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

__device__ __forceinline__ f32x16 mfma(bf16x8 a, bf16x8 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// The same product with fp16 operands (same operand and accumulator layout, same rate): used where an operand needs the
// eleven significand bits of fp16 rather than the eight of bf16.
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;

__device__ __forceinline__ f32x16 mfma_f16(f16x8 a, f16x8 b, f32x16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ f16x8 as_f16x8(uint4 u)
{
    union {
        uint4 u;
        f16x8 h;
    } c;
    c.u = u;
    return c.h;
}

__device__ __forceinline__ uint4 as_uint4(f16x8 h)
{
    union {
        uint4 u;
        f16x8 h;
    } c;
    c.h = h;
    return c.u;
}

// nb * log2(e) as an fp16 bit pattern, for the fragment-major pair bias: magnitudes past fp16's range (|nb| > 45 403,
// infinities included) act as that bound -- 2^-65504 is zero all the same, and the selector products stay finite
__device__ __forceinline__ uint16_t pair_bias_log2_f16(float nb)
{
    float t = nb * LOG2E;
    t = t > 65504.0f ? 65504.0f : (t < -65504.0f ? -65504.0f : t); // comparisons, not min/max: a NaN stays a NaN
    union {
        _Float16 h;
        uint16_t u;
    } c;
    c.h = (_Float16)t;
    return c.u;
}

__device__ __forceinline__ f32x16 zero16()
{
    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    return z;
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

// Wave-private staging panel in LDS: 32 rows x 128 bytes, in 16-byte slots.  A panel is filled with
// four fully coalesced loads (each instruction reads 8 rows x 128 contiguous bytes = 8 whole cache
// lines, lane l -> row 8i + l/8, slot l%8) and read back in MFMA fragment order (lane -> its own
// row).  Loading fragments straight from global memory would touch 32 different cache lines per
// instruction, four times the L1 tag traffic.  The slot index is XOR-swizzled by row so that both
// access patterns are free of LDS bank conflicts.
__device__ __forceinline__ int panel_slot(int row, int chunk)
{
    return row * 8 + (chunk ^ ((row & 7) ^ ((row >> 4) & 1)));
}

// issue the four coalesced loads of a panel: rows row0 .. row0+31 (clamped to last_row) of a
// row-major bf16 matrix with leading dimension ld, 64 columns starting at col0
struct PanelRegs {
    uint4 r0, r1, r2, r3; // named members rather than an array, so that they always live in registers
};

__device__ __forceinline__ uint4 panel_load_one(const bf16_t *base, int64_t ld, int row, int last_row, int col0, int lane)
{
    row = row < last_row ? row : last_row;
    return *reinterpret_cast<const uint4 *>(base + (int64_t)row * ld + col0 + (lane & 7) * 8);
}

__device__ __forceinline__ PanelRegs panel_load(const bf16_t *base, int64_t ld, int row0, int last_row, int col0, int lane)
{
    PanelRegs p;
    const int row = row0 + (lane >> 3);
    p.r0 = panel_load_one(base, ld, row, last_row, col0, lane);
    p.r1 = panel_load_one(base, ld, row + 8, last_row, col0, lane);
    p.r2 = panel_load_one(base, ld, row + 16, last_row, col0, lane);
    p.r3 = panel_load_one(base, ld, row + 24, last_row, col0, lane);
    return p;
}

// The same four loads for a matrix whose last wanted element lies less than 2^31 bytes past `base` and whose row pitch
// is below 2^23 elements (the host checks both before it picks a kernel that calls this): the lane's part of each
// address is then a 32-bit byte offset from the wave-uniform base -- one 24-bit multiply, and an add and a min per
// row -- where 64-bit pointer arithmetic spends three quarter-rate multiplies per row.
__device__ __forceinline__ PanelRegs panel_load_near(const bf16_t *base, uint32_t ld, int row0, int last_row, int col0, int lane)
{
    const char *bytes = reinterpret_cast<const char *>(base);
    const uint32_t pitch = 2u * ld;
    const uint32_t col = 2u * (uint32_t)col0 + 16u * (uint32_t)(lane & 7);
    const uint32_t last = (uint32_t)last_row * pitch + col;
    const uint32_t first = __umul24((uint32_t)(row0 + (lane >> 3)), pitch) + col;
    PanelRegs p;
    p.r0 = *reinterpret_cast<const uint4 *>(bytes + min(first, last));
    p.r1 = *reinterpret_cast<const uint4 *>(bytes + min(first + 8u * pitch, last));
    p.r2 = *reinterpret_cast<const uint4 *>(bytes + min(first + 16u * pitch, last));
    p.r3 = *reinterpret_cast<const uint4 *>(bytes + min(first + 24u * pitch, last));
    return p;
}

__device__ __forceinline__ void panel_store(uint4 *panel, int lane, const PanelRegs &p)
{
    // panel_slot(lane / 8 + 8 i, lane % 8) for i = 0..3, written out: rows 0..7 swizzle by the row itself, and rows
    // 16..31 flip bit 0 on top of that
    const int s0 = (lane & 0x38) | ((lane ^ (lane >> 3)) & 7);
    panel[s0] = p.r0;
    panel[s0 + 64] = p.r1;
    panel[(s0 ^ 1) + 128] = p.r2;
    panel[(s0 ^ 1) + 192] = p.r3;
}

// 8 x 8 transposition of 16-bit elements over the eight lanes that differ in lane bits 3, 4, 5 (same lane & 7).
// Before: lane with index kk = lane >> 3 holds elements (kk, 0..7) as four dwords; after: elements (0..7, kk).
// Three exchange steps in registers: halves of a dword against lane bit 3 (row rotation by 8 + byte permute;
// `sel` must be transpose8x8_selector(lane)), dword pairs against lane bit 4 (v_permlane16_swap) and against lane
// bit 5 (v_permlane32_swap).  Used where memory is contiguous along the index an MFMA fragment (or a row kernel)
// wants spread over lanes.
__device__ __forceinline__ uint32_t transpose8x8_selector(int lane)
{
    // even lanes of bit 3 keep their low halves and take the partner's low halves on top; odd ones the high halves
    return (lane & 8) ? 0x03020706u : 0x05040100u;
}

__device__ __forceinline__ uint4 transpose8x8_lanes(uint4 v, uint32_t sel)
{
    uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const uint32_t partner = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)d[j], 0x128, 0xf, 0xf, false); // lane ^ 8
        d[j] = __builtin_amdgcn_perm(partner, d[j], sel);
    }
#pragma unroll
    for (int j = 0; j < 4; j += 2) {
        const auto sw = __builtin_amdgcn_permlane16_swap(d[j], d[j + 1], false, false);
        d[j] = sw[0], d[j + 1] = sw[1];
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const auto sw = __builtin_amdgcn_permlane32_swap(d[j], d[j + 2], false, false);
        d[j] = sw[0], d[j + 2] = sw[1];
    }
    return make_uint4(d[0], d[1], d[2], d[3]);
}

// LDS transposing read of gfx950 (ds_read_b64_tr_b16).  Within 16 lanes, lane i receives element (i & 3) of the 8-byte
// chunks that lanes 4j + (i >> 2), j = 0..3, point at.  With lane s of a group pointing at row k0 + (s >> 2), columns
// m0 + 4 (s & 3) .. +3 of a tile stored [k][m], lane i ends up with k0..k0+3 of column m0 + i: a 4 x 16 block
// transposed per group and instruction.  Two of them (k0 and k0 + 4) make the 8 consecutive k of an MFMA fragment.
typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ bf16x8 lds_transposed_fragment(const lds_char *lo, const lds_char *hi)
{
    const v4i16 a =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<__attribute__((address_space(3))) v4i16 *>(const_cast<lds_char *>(lo)));
    const v4i16 b =
        __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<__attribute__((address_space(3))) v4i16 *>(const_cast<lds_char *>(hi)));
    union {
        v4i16 h[2];
        bf16x8 f;
    } u;
    u.h[0] = a, u.h[1] = b;
    return u.f;
}

__device__ __forceinline__ float sigmoid_fast(float x)
{
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-x * LOG2E));
}

} // namespace kutacc_dev
