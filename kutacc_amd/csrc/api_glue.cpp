// extern "C" layer of the glue between operators (mask bias, axis swap, residual update, the pair-bias
// producer reading a transposed pair tensor) and of the triangle-attention block built from them:
//   pair_act += attention(LayerNorm(pair_act))        along rows (starting node) or columns (ending node)
// with the pair bias projected from the same normalised tensor.  The reference leaves these steps to its
// caller (a PyTorch extension that is not part of the repository); the operator calls in between are
// kutacc_af2_layernorm / kutacc_af2_linear (reference src/normalization/layernorm.cpp:17-20,
// src/linear/linear.cpp:45-50) and kutacc_af2_gating_attention (reference src/attention/gating_attention.cpp:160-200).
// The triangle-multiplication block is assembled the same way from the steps of reference
// src/attention/triangle_multiplication.cpp:25-150, with the two LayerNorms and the residual a caller adds around them.
// Everything here runs on the device, on one stream, without host round trips.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstring>

#include "api_internal.h"
#include "kutacc_hip.h"
#include "launch_internal.h"

namespace {
constexpr int64_t HEAD = 32;

inline int64_t align256(int64_t v) { return (v + 255) / 256 * 256; }

struct Workspace {
    int64_t z_norm, nb, bias, q, avg, k, v, gate, out, total; // byte offsets (k .. out: the tiled route only)
};

// fused_ln: the head kernel normalises the rows of the pair tensor itself, so no normalised copy is kept.
// tiled: rows beyond the fused head kernels (more than 1024 residues) -- the operator runs on the tiled MFMA route, which
// forms k, v and gate in memory, and its result is added to the pair activation by a pass of its own.
Workspace layout(int64_t n, int64_t heads, bool fused_ln, bool tiled = false)
{
    const int64_t c = heads * HEAD, act = align256(n * n * c * 2);
    Workspace w;
    w.z_norm = 0;
    w.nb = w.z_norm + (fused_ln ? 0 : act);
    w.bias = w.nb + align256(heads * n * n * 2);
    w.q = w.bias + align256(n * n * 2);
    w.avg = w.q + act;
    w.k = w.v = w.gate = w.out = w.total = w.avg + act;
    if (tiled) {
        w.v = w.k + act, w.gate = w.v + act, w.out = w.gate + act, w.total = w.out + act;
    }
    return w;
}
// Argument block of the attention call inside the triangle-attention block, on a workspace laid out by layout();
// `ws` may be a null base when only the plan is of interest (the offsets are then the pointers).
kutacc_hip_attention_args_t triangle_attention_call(const kutacc_hip_triangle_attention_args_t *a, char *ws, const Workspace &w,
                                                    bool fused_ln)
{
    const int64_t n = a->n_res, heads = a->nheads, c = heads * HEAD;
    const bool ending = a->ending_node != 0;
    kutacc_hip_attention_args_t g;
    std::memset(&g, 0, sizeof(g));
    g.batch = n, g.seq_len = n, g.nheads = heads, g.head_size = HEAD;
    g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_FUSED;
    if (fused_ln) {
        // the un-normalised pair tensor itself: row (b, s) of the attention's input is row (s, b) of it for the ending node
        g.input = a->pair_act, g.input_ld = ending ? n * c : c;
    } else {
        g.input = ws + w.z_norm, g.input_ld = c;
    }
    g.query_w = a->query_w, g.key_w = a->key_w, g.value_w = a->value_w, g.gating_w = a->gating_w, g.output_w = a->output_w;
    g.gating_b = a->gating_b, g.output_b = a->output_b;
    g.bias = a->pair_mask, g.bias_stride_b = ending ? 1 : n;
    g.nonbatched_bias = ws + w.nb, g.nb_stride_h = n * n, g.nb_stride_q = n;
    g.q = ws + w.q, g.q_stride_b = n * c, g.q_stride_s = c, g.q_stride_h = HEAD;
    g.avg = ws + w.avg, g.avg_stride_b = n * c, g.avg_stride_s = c, g.avg_stride_h = HEAD;
    g.out = a->pair_act, g.out_ld = c;
    return g;
}

// Whether the block at this size lets the head kernel do the LayerNorm: asked with stand-in pointers (only sizes,
// strides and alignment matter to the plan).
// The policy both blocks share.  Inside the head kernel the LayerNorm is repeated by every head's workgroup and sits on
// the kernel's critical path (the projection phase of the wave that finishes its attention last, which is latency bound);
// against that stands one write and one read of the normalised activation, a pass the memory system does in 6-15 us.
// Measured on one MI355X the fused form is slower at both block shapes (triangle attention, 384 residues x 128
// channels: 133-140 against 119 us; MSA row-wise, 512 x 256 x 256 channels: 238 against 221 us), so the separate pass is
// the default and the fused form is for callers who want the workspace without the normalised copy.
bool layernorm_policy_allows(int64_t)
{
    return kutacc_api::block_layernorm_mode() == 1;
}

// the operator's call with the scratch tensors and the separate result of the tiled route
kutacc_hip_attention_args_t tiled_call(kutacc_hip_attention_args_t g, char *ws, int64_t k, int64_t v, int64_t gate, int64_t out,
                                       int64_t bias, int64_t bias_stride_b)
{
    const int64_t c = g.nheads * g.head_size, m = g.batch * g.seq_len;
    g.path = KUTACC_HIP_PATH_TILED;
    g.bias = ws + bias, g.bias_stride_b = bias_stride_b; // the mask bias as a tensor of its own
    g.k = ws + k, g.k_stride_b = g.seq_len * c, g.k_stride_s = c, g.k_stride_h = g.head_size;
    g.gate = ws + gate, g.gate_stride_b = g.seq_len * c, g.gate_stride_s = c, g.gate_stride_h = g.head_size;
    g.v = ws + v, g.v_stride_h = g.head_size * m, g.v_stride_e = m, g.v_stride_b = g.seq_len;
    g.out = ws + out, g.out_ld = c;
    return g;
}

// The sizes the fused head kernels are written for (fused_attention_supports asks the same of the shape, and more of the
// pointers): blocks of any other size take the tiled route.  By shape alone, so that the workspace functions answer the
// same with and without a device.
bool beyond_fused_kernels(int64_t seq_len, int64_t heads)
{
    const int64_t c = heads * HEAD;
    return (c != 128 && c != 256) || seq_len > 1024;
}
bool triangle_block_is_tiled(int64_t n, int64_t heads) { return beyond_fused_kernels(n, heads); }

bool triangle_block_fuses_layernorm(int64_t n, int64_t heads)
{
    if (!layernorm_policy_allows(heads * HEAD) || triangle_block_is_tiled(n, heads)) {
        return false;
    }
    kutacc_hip_triangle_attention_args_t a;
    std::memset(&a, 0, sizeof(a));
    char *fake = reinterpret_cast<char *>(uintptr_t(1) << 20);
    a.n_res = n, a.nheads = heads, a.dtype = KUTACC_DTYPE_BF16;
    a.pair_act = fake, a.pair_mask = fake;
    a.query_w = a.key_w = a.value_w = a.gating_w = a.output_w = fake;
    a.gating_b = a.output_b = reinterpret_cast<const float *>(fake);
    const Workspace w = layout(n, heads, true);
    const kutacc_hip_attention_args_t g = triangle_attention_call(&a, fake, w, true);
    return kutacc_launch::fused_layernorm_supported(g, kutacc_launch::FusedAttentionOptions());
}
} // namespace

extern "C" {

int kutacc_hip_pair_bias_transposed(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
                                    int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int32_t dtype,
                                    void *stream)
{
    return kutacc_launch::pair_bias(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, dtype, 1,
                                    kutacc_api::stream_or_default(stream));
}

int kutacc_hip_mask_bias(const void *mask, void *bias, int64_t n0, int64_t n1, int32_t transposed, int32_t dtype, void *stream)
{
    return kutacc_launch::mask_bias(mask, bias, n0, n1, transposed != 0, dtype, kutacc_api::stream_or_default(stream));
}

int kutacc_hip_swap_leading_axes(const void *in, void *out, int64_t n0, int64_t n1, int64_t inner, int32_t dtype, void *stream)
{
    return kutacc_launch::swap_leading_axes(in, out, n0, n1, inner, dtype, kutacc_api::stream_or_default(stream));
}

int kutacc_hip_residual_add(void *acc, const void *delta, int64_t n0, int64_t n1, int64_t inner, int32_t swapped, int32_t dtype,
                            void *stream)
{
    return kutacc_launch::residual_add(acc, delta, n0, n1, inner, swapped != 0, dtype, kutacc_api::stream_or_default(stream));
}

int64_t kutacc_hip_triangle_attention_workspace(int64_t n_res, int64_t nheads)
{
    if (n_res <= 0 || nheads <= 0 || n_res > 65536 || nheads > 64) {
        return -1;
    }
    return layout(n_res, nheads, triangle_block_fuses_layernorm(n_res, nheads), triangle_block_is_tiled(n_res, nheads)).total;
}

int kutacc_hip_triangle_attention(const kutacc_hip_triangle_attention_args_t *a, void *stream)
{
    if (!a || !a->pair_act || !a->pair_mask || !a->ln_gamma || !a->ln_beta || !a->bias_w || !a->query_w || !a->key_w ||
        !a->value_w || !a->gating_w || !a->output_w || !a->gating_b || !a->output_b || !a->workspace) {
        return KUTACC_HIP_EINVAL;
    }
    if (a->dtype != KUTACC_DTYPE_BF16 || a->n_res <= 0 || a->n_res > 65536 || a->nheads <= 0 || a->nheads > 64) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t n = a->n_res, heads = a->nheads, c = heads * HEAD;
    // Where the persistent head kernel takes the call, it normalises the rows of the pair tensor itself (LayerNorm is
    // then the first link of the fused chain, and the workspace holds no normalised copy); elsewhere the producer below
    // writes one.
    const bool fused_ln = triangle_block_fuses_layernorm(n, heads), tiled = triangle_block_is_tiled(n, heads);
    const Workspace w = layout(n, heads, fused_ln, tiled);
    if (a->workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(a->workspace) & 255u) != 0) {
        return KUTACC_HIP_EINVAL;
    }
    char *ws = static_cast<char *>(a->workspace);
    hipStream_t s = kutacc_api::stream_or_default(stream);
    const int ending = a->ending_node != 0;

    const kutacc_hip_attention_args_t g = triangle_attention_call(a, ws, w, fused_ln);
    if (tiled) {
        // Rows beyond the fused head kernels: the same chain as separate passes -- LayerNorm + pair bias (read transposed
        // for the ending node), mask bias, the operator on the tiled MFMA route, residual sum (transposed back).
        const kutacc_hip_attention_args_t t = tiled_call(g, ws, w.k, w.v, w.gate, w.out, w.bias, n);
        if (!kutacc_launch::tiled_attention_supports(t)) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        int rc = kutacc_launch::pair_bias(a->pair_act, a->ln_gamma, a->ln_beta, a->bias_w, ws + w.nb, ws + w.z_norm, n, n, c, heads,
                                          a->ln_eps, KUTACC_DTYPE_BF16, ending, s);
        if (rc == 0) {
            rc = kutacc_launch::mask_bias(a->pair_mask, ws + w.bias, n, n, ending, KUTACC_DTYPE_BF16, s);
        }
        if (rc == 0) {
            rc = kutacc_launch::gating_attention_tiled(t, s);
        }
        if (rc == 0) {
            rc = kutacc_launch::residual_add(a->pair_act, ws + w.out, n, n, c, ending, KUTACC_DTYPE_BF16, s);
        }
        return rc;
    }
    if (!kutacc_launch::fused_attention_supports(g)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    // The operator forms the mask bias from the pair mask itself, and its output projection adds straight into the pair
    // activation (transposed back for the ending node), so neither costs a pass of its own.
    kutacc_launch::FusedAttentionOptions opt;
    opt.out_mode = ending ? kutacc_launch::FUSED_OUT_ADD_TRANSPOSED : kutacc_launch::FUSED_OUT_ADD;
    opt.bias_is_mask = true; // element (b, k) of the mask bias comes from mask[b, k], or mask[k, b] for the ending node
    opt.bias_stride_k = ending ? n : 1;
    if (fused_ln) {
        opt.ln_gamma = a->ln_gamma, opt.ln_beta = a->ln_beta, opt.ln_eps = a->ln_eps;
        opt.input_stride_b = ending ? c : n * c;
    }
    // 1. LayerNorm + pair-bias projection in one pass over the pair tensor; the ending node reads it transposed
    //    -- and, where the grid allows it, writes the copy the attention kernel will read as well: fp32 tiles where
    //    the operator takes the two-row kernel, fp16 fragments otherwise
    void *z_norm = fused_ln ? nullptr : ws + w.z_norm;
    int frag_nb = 0, frag_nt = 0;
    const bool writes = kutacc_launch::pair_bias_writes_fragments(a->pair_act, a->bias_w, z_norm, n, n, c, heads, KUTACC_DTYPE_BF16);
    const bool tiles = writes && heads <= 8 && kutacc_launch::fused_attention_tile_layout(g, opt, &frag_nb, &frag_nt);
    const bool fragments = !tiles && writes && kutacc_launch::fused_attention_fragment_layout(g, &frag_nb, &frag_nt);
    int rc = kutacc_launch::pair_bias(a->pair_act, a->ln_gamma, a->ln_beta, a->bias_w, ws + w.nb, z_norm, n, n, c, heads,
                                      a->ln_eps, KUTACC_DTYPE_BF16, ending, s, (tiles || fragments) ? g.q : nullptr, frag_nb,
                                      frag_nt, tiles ? 1 : 0);
    if (rc != 0) {
        return rc;
    }
    // 2. the operator
    opt.nb_tiles_ready = tiles;
    opt.nb_fragments_ready = fragments;
    return kutacc_launch::gating_attention_fused(g, s, opt);
}

int kutacc_hip_layernorm_channel_first(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out,
                                       int64_t ld_out, int64_t channels, int64_t positions, float eps, int32_t dtype,
                                       void *stream)
{
    return kutacc_launch::layernorm_channel_first(x, ld_x, gamma, beta, out, ld_out, channels, positions, eps, dtype,
                                                  kutacc_api::stream_or_default(stream));
}

int kutacc_hip_gated_residual_projection(const void *a, int64_t a_ld, const void *w, const float *bias, const void *gate,
                                         int64_t gate_ld, void *acc, int64_t acc_ld, int64_t m, int64_t n, int64_t k,
                                         int32_t dtype, void *stream)
{
    if (!a || !w || !bias || !gate || !acc || m <= 0 || n <= 0 || k <= 0 || dtype != KUTACC_DTYPE_BF16) {
        return KUTACC_HIP_EINVAL;
    }
    return kutacc_launch::row_projection_gated_residual(a, a_ld, w, bias, gate, gate_ld, acc, acc_ld, m, n, k,
                                                        kutacc_api::stream_or_default(stream));
}

// The channel-first intermediates of the block (projections and centre: one n x n plane per channel) keep their planes
// 17 cache lines further apart than the positions need.  At 1024 residues a plane is exactly 2 MB, every step of the
// kernels that write or read them touches the same offset of all 128 planes, and addresses 2 MB apart fall on the same
// memory channel: one gated projection at 1024 x 1024 positions 145-151 us dense, 119-127 us padded.
constexpr int64_t TM_PLANE_PAD = 1088;

int64_t kutacc_hip_triangle_multiplication_workspace(int64_t n_res, int64_t c_z, int64_t c_i)
{
    if (n_res <= 0 || c_z <= 0 || c_i <= 0 || n_res > 65536 || c_z > 4096 || c_i > 4096) {
        return -1;
    }
    return 4 * align256((n_res * n_res + TM_PLANE_PAD) * (c_z > c_i ? c_z : c_i) * 2);
}

int kutacc_hip_triangle_multiplication(const kutacc_hip_triangle_multiplication_args_t *a, void *stream)
{
    if (!a || !a->pair_act || !a->pair_mask || !a->ln_in_gamma || !a->ln_in_beta || !a->left_proj_w || !a->left_proj_b ||
        !a->left_gate_w || !a->left_gate_b || !a->right_proj_w || !a->right_proj_b || !a->right_gate_w || !a->right_gate_b ||
        !a->ln_center_gamma || !a->ln_center_beta || !a->output_w || !a->output_b || !a->gating_w || !a->gating_b ||
        !a->workspace) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t need = kutacc_hip_triangle_multiplication_workspace(a->n_res, a->c_z, a->c_i);
    if (a->dtype != KUTACC_DTYPE_BF16 || need < 0 || a->workspace_bytes < need ||
        (reinterpret_cast<uintptr_t>(a->workspace) & 255u) != 0) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t n = a->n_res, cz = a->c_z, ci = a->c_i, rows = n * n, buf = need / 4, plane = rows + TM_PLANE_PAD;
    char *ws = static_cast<char *>(a->workspace);
    void *act = ws, *left = ws + buf, *right = ws + 2 * buf, *center_cf = ws + 3 * buf;
    void *center = left, *gate = right, *out = center_cf; // each is free again by the time its second tenant arrives
    hipStream_t s = kutacc_api::stream_or_default(stream);

    // 1. layer_norm_input
    int rc = kutacc_launch::layernorm_rows(a->pair_act, cz, a->ln_in_gamma, a->ln_in_beta, act, cz, rows, cz, a->ln_eps,
                                           KUTACC_DTYPE_BF16, s);
    // 2. gated projections, channel-first: both sides in one launch where the tiled kernel takes them, else one after
    //    the other
    if (rc == 0) {
        kutacc_hip_gemm_args_t g[2];
        for (int side = 0; side < 2; ++side) {
            std::memset(&g[side], 0, sizeof(g[side]));
            g[side].dtype = KUTACC_DTYPE_BF16, g[side].path = KUTACC_HIP_PATH_AUTO, g[side].batches = 1;
            g[side].m = ci, g[side].n = rows, g[side].k = cz;
            g[side].a = side ? a->right_proj_w : a->left_proj_w, g[side].a_gate = side ? a->right_gate_w : a->left_gate_w;
            g[side].a_stride_m = cz, g[side].a_stride_k = 1;
            g[side].b = act, g[side].b_stride_n = cz, g[side].b_stride_k = 1;
            g[side].c = side ? right : left, g[side].c_stride_m = plane;
            g[side].bias = side ? a->right_proj_b : a->left_proj_b, g[side].bias_gate = side ? a->right_gate_b : a->left_gate_b;
            g[side].bias_axis = 2, g[side].mask = a->pair_mask;
        }
        rc = kutacc_launch::pair_gemm(g[0], s, &g[1]);
        if (rc == KUTACC_HIP_EUNSUPPORTED) {
            rc = kutacc_launch::pair_gemm(g[0], s);
            if (rc == 0) {
                rc = kutacc_launch::pair_gemm(g[1], s);
            }
        }
    }
    // 3. the equation, one n x n product per channel
    if (rc == 0) {
        kutacc_hip_gemm_args_t g;
        std::memset(&g, 0, sizeof(g));
        g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_AUTO;
        g.m = g.n = g.k = n, g.batches = ci;
        if (!a->incoming) {
            g.a = left, g.a_stride_m = n, g.a_stride_k = 1, g.b = right, g.b_stride_n = n, g.b_stride_k = 1;
        } else {
            g.a = right, g.a_stride_m = 1, g.a_stride_k = n, g.b = left, g.b_stride_n = 1, g.b_stride_k = n;
        }
        g.a_stride_batch = g.b_stride_batch = g.c_stride_batch = plane;
        g.c = center_cf, g.c_stride_m = n;
        rc = kutacc_launch::pair_gemm(g, s);
    }
    // The last kernel can form the gate itself (128 channels in and out: the gate tensor is then never written), and with
    // positions in whole 16-byte runs it also reads the centre channel-first and normalises it on the way in
    const bool gate_inside = kutacc_launch::row_projection_projected_gate_supports(
        center, ci, a->output_w, a->output_b, act, cz, a->gating_w, a->gating_b, a->pair_act, cz, rows, cz, ci, cz);
    const bool norm_inside = gate_inside && rows % 8 == 0 && kutacc_hip_aligned16(a->ln_center_gamma) &&
                             kutacc_hip_aligned16(a->ln_center_beta);
    // 4. center_layer_norm, channel-first in, channel-last out
    if (rc == 0 && !norm_inside) {
        rc = kutacc_launch::layernorm_channel_first(center_cf, plane, a->ln_center_gamma, a->ln_center_beta, center, ci, ci, rows,
                                                    a->ln_eps, KUTACC_DTYPE_BF16, s);
    }
    // 5. gate from the normalised input
    if (rc == 0 && !gate_inside) {
        kutacc_hip_gemm_args_t g;
        std::memset(&g, 0, sizeof(g));
        g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_AUTO, g.batches = 1;
        g.m = rows, g.n = cz, g.k = cz;
        g.a = act, g.a_stride_m = cz, g.a_stride_k = 1;
        g.b = a->gating_w, g.b_stride_n = cz, g.b_stride_k = 1;
        g.c = gate, g.c_stride_m = cz;
        g.bias = a->gating_b, g.bias_axis = 1;
        rc = kutacc_launch::pair_gemm(g, s);
    }
    // 6. output projection of the normalised centre, times sigmoid(gate), added to the pair activation: one kernel
    //    when the shape allows, else projection, gating and residual as three passes
    if (rc == 0 && norm_inside) {
        rc = kutacc_launch::row_projection_projected_gate_residual(center_cf, plane, a->output_w, a->output_b, act, cz,
                                                                   a->gating_w, a->gating_b, a->pair_act, cz, rows, s,
                                                                   a->ln_center_gamma, a->ln_center_beta, a->ln_eps);
    } else if (rc == 0 && gate_inside) {
        rc = kutacc_launch::row_projection_projected_gate_residual(center, ci, a->output_w, a->output_b, act, cz, a->gating_w,
                                                                   a->gating_b, a->pair_act, cz, rows, s);
    } else if (rc == 0) {
        rc = kutacc_launch::row_projection_gated_residual(center, ci, a->output_w, a->output_b, gate, cz, a->pair_act, cz, rows,
                                                          cz, ci, s);
        if (rc == KUTACC_HIP_EUNSUPPORTED) {
            kutacc_hip_gemm_args_t g;
            std::memset(&g, 0, sizeof(g));
            g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_AUTO, g.batches = 1;
            g.m = rows, g.n = cz, g.k = ci;
            g.a = center, g.a_stride_m = ci, g.a_stride_k = 1;
            g.b = a->output_w, g.b_stride_n = ci, g.b_stride_k = 1;
            g.c = out, g.c_stride_m = cz;
            g.bias = a->output_b, g.bias_axis = 1;
            rc = kutacc_launch::pair_gemm(g, s);
            if (rc == 0) {
                rc = kutacc_launch::sigmoid_gate_rows(out, n * cz, cz, gate, n * cz, cz, n, n, cz, s);
            }
            if (rc == 0) {
                rc = kutacc_launch::residual_add(a->pair_act, out, n, n, cz, 0, KUTACC_DTYPE_BF16, s);
            }
        }
    }
    return rc;
}

int64_t kutacc_hip_transition_block_workspace(int64_t rows, int64_t c_o, int64_t c_i)
{
    if (rows <= 0 || c_o <= 0 || c_i <= 0 || rows > INT64_MAX / 4 / (c_o + c_i)) {
        return -1;
    }
    if ((c_o == 128 || c_o == 256) && c_i % 64 == 0 && c_i <= 2048) {
        return 0; // the one-kernel form needs none
    }
    return align256(rows * c_o * 2) + align256(rows * c_i * 2);
}

int kutacc_hip_transition_block(void *act, const float *ln_gamma, const float *ln_beta, float ln_eps, const void *w1,
                                const float *b1, const void *w2, const float *b2, void *workspace, int64_t workspace_bytes,
                                int64_t rows, int64_t c_o, int64_t c_i, int32_t dtype, void *stream)
{
    if (!act || !ln_gamma || !ln_beta || !w1 || !b1 || !w2 || !b2 || rows <= 0 || c_o <= 0 || c_i <= 0 ||
        dtype != KUTACC_DTYPE_BF16) {
        return KUTACC_HIP_EINVAL;
    }
    hipStream_t s = kutacc_api::stream_or_default(stream);
    int rc = kutacc_launch::transition_block_fused(act, ln_gamma, ln_beta, ln_eps, w1, b1, w2, b2, rows, c_o, c_i, s);
    if (rc != KUTACC_HIP_EUNSUPPORTED) {
        return rc;
    }
    // three passes through the workspace: LayerNorm, the transition (its result takes the place of its input), residual
    const int64_t norm_bytes = align256(rows * c_o * 2), need = norm_bytes + align256(rows * c_i * 2);
    if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u) != 0) {
        return KUTACC_HIP_EINVAL;
    }
    char *ws = static_cast<char *>(workspace);
    rc = kutacc_launch::layernorm_rows(act, c_o, ln_gamma, ln_beta, ws, c_o, rows, c_o, ln_eps, KUTACC_DTYPE_BF16, s);
    if (rc == 0) {
        rc = kutacc_hip_transition(ws, w1, b1, w2, b2, ws + norm_bytes, ws, rows, c_o, c_i, KUTACC_DTYPE_BF16, KUTACC_HIP_PATH_GENERIC,
                                   s);
    }
    if (rc == 0) {
        rc = kutacc_launch::residual_add(act, ws, rows, 1, c_o, 0, KUTACC_DTYPE_BF16, s);
    }
    return rc;
}

int kutacc_hip_layernorm_rows_transposed(const void *x, const float *gamma, const float *beta, void *out, int64_t rows_i,
                                         int64_t rows_j, int64_t size, float eps, int32_t dtype, void *stream)
{
    if (rows_i <= 0 || rows_j <= 0 || rows_i > INT64_MAX / rows_j) {
        return KUTACC_HIP_EINVAL;
    }
    return kutacc_launch::layernorm_rows(x, size, gamma, beta, out, size, rows_i * rows_j, size, eps, dtype,
                                         kutacc_api::stream_or_default(stream), rows_j);
}

namespace {
struct MsaWorkspace {
    int64_t m_norm, nb, bias, q, avg, k, v, gate, out, total; // (k .. out: the tiled route only)
};

// fused_ln: the head kernel normalises the msa rows itself, so no normalised copy is kept; tiled: as for the
// triangle-attention block
MsaWorkspace msa_layout(int64_t n_seq, int64_t n_res, int64_t heads, bool column, bool fused_ln, bool tiled = false)
{
    const int64_t act = align256(n_seq * n_res * heads * HEAD * 2);
    MsaWorkspace w;
    w.m_norm = 0;
    w.nb = w.m_norm + (fused_ln ? 0 : act);
    w.bias = w.nb + (column ? 0 : align256(heads * n_res * n_res * 2));
    w.q = w.bias + align256(n_seq * n_res * 2);
    w.avg = w.q + act;
    w.k = w.v = w.gate = w.out = w.total = w.avg + act;
    if (tiled) {
        w.v = w.k + act, w.gate = w.v + act, w.out = w.gate + act, w.total = w.out + act;
    }
    return w;
}
// Argument block of the attention call inside the MSA attention block (see triangle_attention_call)
kutacc_hip_attention_args_t msa_attention_call(const kutacc_hip_msa_attention_args_t *a, char *ws, const MsaWorkspace &w,
                                               bool fused_ln)
{
    const bool column = a->column != 0;
    const int64_t n_seq = a->n_seq, n_res = a->n_res, heads = a->nheads, c = heads * HEAD;
    // row-wise: every sequence attends over the residues; column-wise: every residue attends over the sequences,
    // i.e. the same operator on the msa with its two leading axes exchanged
    const int64_t batch = column ? n_res : n_seq, seq = column ? n_seq : n_res;
    kutacc_hip_attention_args_t g;
    std::memset(&g, 0, sizeof(g));
    g.batch = batch, g.seq_len = seq, g.nheads = heads, g.head_size = HEAD;
    g.dtype = KUTACC_DTYPE_BF16, g.path = KUTACC_HIP_PATH_FUSED;
    if (fused_ln) {
        // the un-normalised msa itself; column-wise, row (b, s) of the attention's input is row (s, b) of it
        g.input = a->msa_act, g.input_ld = column ? n_res * c : c;
    } else {
        g.input = ws + w.m_norm, g.input_ld = c;
    }
    g.query_w = a->query_w, g.key_w = a->key_w, g.value_w = a->value_w, g.gating_w = a->gating_w, g.output_w = a->output_w;
    g.gating_b = a->gating_b, g.output_b = a->output_b;
    g.bias = a->msa_mask, g.bias_stride_b = column ? 1 : n_res;
    if (!column) {
        g.nonbatched_bias = ws + w.nb, g.nb_stride_h = n_res * n_res, g.nb_stride_q = n_res;
    }
    g.q = ws + w.q, g.q_stride_b = seq * c, g.q_stride_s = c, g.q_stride_h = HEAD;
    g.avg = ws + w.avg, g.avg_stride_b = seq * c, g.avg_stride_s = c, g.avg_stride_h = HEAD;
    g.out = a->msa_act, g.out_ld = c;
    return g;
}

bool msa_block_is_tiled(int64_t n_seq, int64_t n_res, int64_t heads, bool column)
{
    return beyond_fused_kernels(column ? n_seq : n_res, heads);
}

bool msa_block_fuses_layernorm(int64_t n_seq, int64_t n_res, int64_t heads, bool column)
{
    if (!layernorm_policy_allows(heads * HEAD) || msa_block_is_tiled(n_seq, n_res, heads, column)) {
        return false;
    }
    kutacc_hip_msa_attention_args_t a;
    std::memset(&a, 0, sizeof(a));
    char *fake = reinterpret_cast<char *>(uintptr_t(1) << 20);
    a.n_seq = n_seq, a.n_res = n_res, a.nheads = heads, a.dtype = KUTACC_DTYPE_BF16, a.column = column ? 1 : 0;
    a.msa_act = fake, a.msa_mask = fake;
    a.query_w = a.key_w = a.value_w = a.gating_w = a.output_w = fake;
    a.gating_b = a.output_b = reinterpret_cast<const float *>(fake);
    const MsaWorkspace w = msa_layout(n_seq, n_res, heads, column, true);
    const kutacc_hip_attention_args_t g = msa_attention_call(&a, fake, w, true);
    return kutacc_launch::fused_layernorm_supported(g, kutacc_launch::FusedAttentionOptions());
}
} // namespace

int64_t kutacc_hip_msa_attention_workspace(int64_t n_seq, int64_t n_res, int64_t nheads, int32_t column)
{
    if (n_seq <= 0 || n_res <= 0 || nheads <= 0 || n_seq > 1 << 20 || n_res > 65536 || nheads > 64) {
        return -1;
    }
    return msa_layout(n_seq, n_res, nheads, column != 0, msa_block_fuses_layernorm(n_seq, n_res, nheads, column != 0),
                      msa_block_is_tiled(n_seq, n_res, nheads, column != 0))
        .total;
}

int kutacc_hip_msa_attention(const kutacc_hip_msa_attention_args_t *a, void *stream)
{
    if (!a || !a->msa_act || !a->msa_mask || !a->ln_gamma || !a->ln_beta || !a->query_w || !a->key_w || !a->value_w ||
        !a->gating_w || !a->output_w || !a->gating_b || !a->output_b || !a->workspace) {
        return KUTACC_HIP_EINVAL;
    }
    const bool column = a->column != 0;
    if (!column && (!a->pair_act || !a->pair_ln_gamma || !a->pair_ln_beta || !a->bias_w || a->c_z <= 0)) {
        return KUTACC_HIP_EINVAL;
    }
    if (a->dtype != KUTACC_DTYPE_BF16 || kutacc_hip_msa_attention_workspace(a->n_seq, a->n_res, a->nheads, a->column) < 0) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t n_seq = a->n_seq, n_res = a->n_res, heads = a->nheads, c = heads * HEAD;
    // where the persistent head kernel takes the call it normalises the msa rows itself: no normalised copy, no LayerNorm pass
    const bool fused_ln = msa_block_fuses_layernorm(n_seq, n_res, heads, column), tiled = msa_block_is_tiled(n_seq, n_res, heads, column);
    const MsaWorkspace w = msa_layout(n_seq, n_res, heads, column, fused_ln, tiled);
    if (a->workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(a->workspace) & 255u) != 0) {
        return KUTACC_HIP_EINVAL;
    }
    char *ws = static_cast<char *>(a->workspace);
    hipStream_t s = kutacc_api::stream_or_default(stream);
    const kutacc_hip_attention_args_t g = msa_attention_call(a, ws, w, fused_ln);
    if (tiled) {
        // Rows beyond the fused head kernels (more than 1024 keys): LayerNorm (read transposed column-wise), pair bias
        // (row-wise), mask bias, the operator on the tiled MFMA route, residual sum (transposed back column-wise).
        const int64_t batch = column ? n_res : n_seq, seq = column ? n_seq : n_res;
        const kutacc_hip_attention_args_t t = tiled_call(g, ws, w.k, w.v, w.gate, w.out, w.bias, seq);
        if (!kutacc_launch::tiled_attention_supports(t)) {
            return KUTACC_HIP_EUNSUPPORTED;
        }
        int rc = kutacc_launch::layernorm_rows(a->msa_act, c, a->ln_gamma, a->ln_beta, ws + w.m_norm, c, n_seq * n_res, c, a->ln_eps,
                                               KUTACC_DTYPE_BF16, s, column ? n_seq : 0);
        if (rc == 0 && !column) {
            rc = kutacc_launch::pair_bias(a->pair_act, a->pair_ln_gamma, a->pair_ln_beta, a->bias_w, ws + w.nb, nullptr, n_res, n_res,
                                          a->c_z, heads, a->ln_eps, KUTACC_DTYPE_BF16, 0, s);
        }
        if (rc == 0) {
            rc = kutacc_launch::mask_bias(a->msa_mask, ws + w.bias, batch, seq, column ? 1 : 0, KUTACC_DTYPE_BF16, s);
        }
        if (rc == 0) {
            rc = kutacc_launch::gating_attention_tiled(t, s);
        }
        if (rc == 0) {
            rc = kutacc_launch::residual_add(a->msa_act, ws + w.out, n_seq, n_res, c, column ? 1 : 0, KUTACC_DTYPE_BF16, s);
        }
        return rc;
    }
    if (!kutacc_launch::fused_attention_supports(g)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    // 1. LayerNorm of the msa rows, read transposed for the column-wise form (unless the head kernel does it)
    int rc = fused_ln ? 0
                      : kutacc_launch::layernorm_rows(a->msa_act, c, a->ln_gamma, a->ln_beta, ws + w.m_norm, c, n_seq * n_res, c,
                                                      a->ln_eps, KUTACC_DTYPE_BF16, s, column ? n_seq : 0);
    // The operator forms the mask bias from the msa mask on the fly, and its output projection adds into the msa
    // (transposed back for the column-wise form).
    kutacc_launch::FusedAttentionOptions opt;
    opt.out_mode = column ? kutacc_launch::FUSED_OUT_ADD_TRANSPOSED : kutacc_launch::FUSED_OUT_ADD;
    opt.bias_is_mask = true; // msa_mask[s, r] is element (b = s, k = r) row-wise and (b = r, k = s) column-wise
    opt.bias_stride_k = column ? n_res : 1;
    if (fused_ln) {
        opt.ln_gamma = a->ln_gamma, opt.ln_beta = a->ln_beta, opt.ln_eps = a->ln_eps;
        opt.input_stride_b = column ? c : n_res * c;
    }
    // 2. pair bias from the pair activation (row-wise form only)
    //    -- with the copy the attention kernel will read, where the grid allows it: fp32 tiles for the two-row kernel,
    //    fp16 fragments otherwise
    if (rc == 0 && !column) {
        int frag_nb = 0, frag_nt = 0;
        const bool writes = kutacc_launch::pair_bias_writes_fragments(a->pair_act, a->bias_w, nullptr, n_res, n_res, a->c_z, heads,
                                                                      KUTACC_DTYPE_BF16);
        const bool tiles = writes && heads <= 8 && kutacc_launch::fused_attention_tile_layout(g, opt, &frag_nb, &frag_nt);
        const bool fragments = !tiles && writes && kutacc_launch::fused_attention_fragment_layout(g, &frag_nb, &frag_nt);
        rc = kutacc_launch::pair_bias(a->pair_act, a->pair_ln_gamma, a->pair_ln_beta, a->bias_w, ws + w.nb, nullptr, n_res, n_res,
                                      a->c_z, heads, a->ln_eps, KUTACC_DTYPE_BF16, 0, s, (tiles || fragments) ? g.q : nullptr,
                                      frag_nb, frag_nt, tiles ? 1 : 0);
        opt.nb_tiles_ready = tiles;
        opt.nb_fragments_ready = fragments;
    }
    // 3. the operator
    if (rc == 0) {
        rc = kutacc_launch::gating_attention_fused(g, s, opt);
    }
    return rc;
}

} // extern "C"
