/*
 * kutacc_hip.h -- the C-ABI launch layer between the C++ host side of libkutacc and its HIP kernels.
 *
 * Everything here is extern "C" with plain pointers and sizes: no C++ types, no torch types, no
 * tensor handles.  The handle-based entry points of kutacc.h unpack their arguments and call these;
 * an FFI user (ctypes, cgo, JNI) can call them directly on device memory.
 *
 * Conventions
 *   - every data pointer is a HIP DEVICE pointer on the current device unless stated otherwise;
 *   - `dtype` is a kutacc::DType value: 1 = bf16 storage, 2 = fp32 storage;
 *   - `stream` is a hipStream_t passed as void* (NULL = the library stream, see
 *     kutacc_hip_set_stream); launches are asynchronous, the caller synchronises;
 *   - the return value is 0 on success, a hipError_t value if a HIP call failed, or a negative
 *     KUTACC_HIP_E* code if the arguments were rejected before anything was launched.
 *   - strides are in elements.
 */
#ifndef KUTACC_HIP_H
#define KUTACC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifndef kutacc_export
#define kutacc_export __attribute__((visibility("default")))
#endif

#ifdef __cplusplus
extern "C" {
#endif

#define KUTACC_HIP_EINVAL (-2)      /* bad shape / stride / dtype / null pointer          */
#define KUTACC_HIP_EUNSUPPORTED (-3) /* request is valid but no kernel on this backend takes it */

#define KUTACC_DTYPE_BF16 1
#define KUTACC_DTYPE_FP32 2

/* Kernel family selection for kutacc_hip_gating_attention. */
#define KUTACC_HIP_PATH_AUTO 0    /* fused MFMA kernels when the shape allows, else tiled, else generic */
#define KUTACC_HIP_PATH_GENERIC 1 /* shape-agnostic scalar kernels (any head_size, bf16 or fp32)  */
#define KUTACC_HIP_PATH_FUSED 2   /* MFMA kernels only (fused, fp32, tiled); EUNSUPPORTED if none takes the shape */
#define KUTACC_HIP_PATH_TILED 3   /* the tiled MFMA route; EUNSUPPORTED if it does not take the shape */
/* The fused MFMA kernels cover bf16, head_size 32, nheads * 32 in {128, 256}, seq_len <= 1024, 16-byte aligned operands
 * with leading dimensions that are multiples of 8, and an input row pitch of at most 2^19 elements (they address the
 * rows of a batch row with 32-bit byte offsets).
 * The tiled MFMA route covers the other bf16 shapes: any seq_len, head sizes that are multiples of 8 up to 64, any number
 * of heads; q, k, v, gate and avg laid out as the reference's kernel views them (dense [batch * seq_len, channels]
 * matrices with row pitches that are multiples of 8, v as [channels, batch * seq_len]).  It follows the reference's data
 * flow -- projections into q, k, v, gate on the MFMA GEMM, attention on MFMA tiles with an online softmax, output
 * projection -- and so leaves those tensors as the reference does. */

/*
 * Flat argument block of the gated-attention operator.  Replaces, for the launch layer, the
 * (Tensor&, ...) parameter list of kutacc::gating_attention_kernel
 * (reference src/attention/gating_attention.cpp:33-37); field meaning follows that function.
 */
typedef struct kutacc_hip_attention_args {
    int64_t batch;     /* B */
    int64_t seq_len;   /* S */
    int64_t nheads;    /* H */
    int64_t head_size; /* d;  nchannels C = H*d */
    int32_t dtype;     /* storage type of input, weights matrices, biases tensors, scratch and out */
    int32_t path;      /* KUTACC_HIP_PATH_* */

    const void *input;    /* [B*S, C], row stride input_ld                                   */
    int64_t input_ld;
    const void *query_w;  /* [C, C] stored [out, in], row stride C                           */
    const void *key_w;
    const void *value_w;
    const void *gating_w;
    const void *output_w;
    const float *gating_b; /* fp32 [C]                                                       */
    const float *output_b; /* fp32 [C]                                                       */

    const void *bias;      /* mask bias, element (b,k) at bias[b*bias_stride_b + k]          */
    int64_t bias_stride_b;
    const void *nonbatched_bias; /* pair bias, element (h,q,k) at h*nb_stride_h + q*nb_stride_q + k; NULL = absent */
    int64_t nb_stride_h;
    int64_t nb_stride_q;

    /* Caller scratch.  k/v/gate are written only by the generic and the tiled path; q is written by those
     * and may be used as workspace by the fused path (a fragment-major copy of the pair bias), so
     * its contents are unspecified after any call; avg (gated weighted average, [B,S,H,d]) is
     * written by every path.  Element (b,s,h,e) of q,k,gate,avg lives at
     * b*stride_b + s*stride_s + h*stride_h + e; v is [H,d,B,S]: (h,e,b,s) at
     * h*v_stride_h + e*v_stride_e + b*v_stride_b + s. */
    void *q, *k, *v, *gate, *avg;
    int64_t q_stride_b, q_stride_s, q_stride_h;
    int64_t k_stride_b, k_stride_s, k_stride_h;
    int64_t gate_stride_b, gate_stride_s, gate_stride_h;
    int64_t avg_stride_b, avg_stride_s, avg_stride_h;
    int64_t v_stride_h, v_stride_e, v_stride_b;

    void *out;          /* [B*S, C], row stride out_ld                                       */
    int64_t out_ld;
} kutacc_hip_attention_args_t;

/* Enqueue the whole operator on `stream`.  Replaces kutacc::gating_attention_kernel
 * (reference src/attention/gating_attention.cpp:33-158). */
kutacc_export int kutacc_hip_gating_attention(const kutacc_hip_attention_args_t *args, void *stream);

/*
 * kutacc_hip_gating_attention for callers that cannot allocate device memory or lend scratch: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  The one
 * scratch buffer of the MFMA kernels, a fragment-major copy of the pair bias, lives in a device array inside the
 * library image (KUTACC_HIP_STATIC_SCRATCH_BYTES; each GPU the library runs on holds it until the process ends), so
 * args->q, k, v and gate are neither read nor written and may be NULL.  Nothing on this path calls hipMalloc, hipFree
 * or any allocating routine; per-kernel profiling events are not recorded for it.  Only shapes the MFMA kernels take
 * (bf16, head_size 32, nheads*32 in {128, 256}, seq_len <= 1024): others return KUTACC_HIP_EUNSUPPORTED.  A pair bias
 * whose copy, nheads * ceil(S/32) * 2*ceil(S/64) * 2048 bytes, exceeds the array is rejected with KUTACC_HIP_EINVAL
 * and a line on stderr (16 MiB holds 8 heads at 1024 positions).  All calls on one GPU share the array, which keeps
 * the last call's contents: every call rewrites the part it reads, and calls that overlap in time on one GPU race.
 * The first call on a device looks up the array's address (hipGetSymbolAddress) and the first call of a kernel
 * variant raises its dynamic-LDS limit (hipFuncSetAttribute, device-attribute queries); neither may be recorded into
 * a graph, so make one warm-up call per device and shape outside stream capture before capturing this entry point.
 */
#define KUTACC_HIP_STATIC_SCRATCH_BYTES (16u << 20)
kutacc_export int kutacc_hip_gating_attention_static(const kutacc_hip_attention_args_t *args, void *stream);

/* Global (extra-MSA column) attention, reference src/attention/global_attention.cpp:30-164 (kernel) and
 * :167-205 (entry).  One query per batch row and head (the masked mean of the row), one key/value head
 * shared by all heads.  bf16 storage, nheads*head_size == 64 (the reference hard-wires nchannels == 64,
 * :172), nheads <= 32, head_size <= 32.  The reference's scratch tensors q, k, v, gate are not needed and
 * not touched; q_avg ([B, 64], may be NULL) receives the masked mean as the reference leaves it in `avg`.
 * seq_len <= 12288 (what a workgroup's LDS holds of a row's mask and logits; longer rows return
 * KUTACC_HIP_EUNSUPPORTED before anything is launched); the tokens of a batch row must lie within 2 GiB of its first one in q_data and in out (32-bit
 * offsets in the kernel), else KUTACC_HIP_EUNSUPPORTED. */
typedef struct kutacc_hip_global_attention_args {
    int64_t batch;     /* B */
    int64_t seq_len;   /* S */
    int64_t nheads;    /* H */
    int64_t head_size; /* d;  H*d == 64 */
    int32_t dtype;     /* KUTACC_DTYPE_BF16 */
    int32_t reserved;

    const void *q_data;       /* element (b,s,c) at b*q_data_stride_b + s*q_data_stride_s + c */
    int64_t q_data_stride_b;
    int64_t q_data_stride_s;
    const void *q_mask;       /* element (b,s) at b*q_mask_stride_b + s */
    int64_t q_mask_stride_b;
    const void *query_w;      /* [64, 64] stored [out, in] */
    const void *key_w;        /* [d, 64]  stored [out, in] */
    const void *value_w;      /* [d, 64]  stored [out, in] */
    const void *gating_w;     /* [64, 64] stored [out, in] */
    const void *output_w;     /* [64, 64] stored [out, in] */
    const float *gating_b;    /* fp32 [64] */
    const float *output_b;    /* fp32 [64] */

    void *q_avg;              /* [B, 64], row stride q_avg_stride_b; NULL = not wanted */
    int64_t q_avg_stride_b;
    void *out;                /* element (b,s,c) at b*out_stride_b + s*out_stride_s + c */
    int64_t out_stride_b;
    int64_t out_stride_s;
} kutacc_hip_global_attention_args_t;

kutacc_export int kutacc_hip_global_attention(const kutacc_hip_global_attention_args_t *args, void *stream);

/* Name of the kernel family the last successful kutacc_hip_gating_attention call used on this
 * thread: "fused_mfma", "fp32_mfma", "tiled_mfma" or "generic".  Static storage. */
kutacc_export const char *kutacc_hip_last_path(void);

/*
 * LayerNorm over the last axis of `rows` rows (row r at x + r*ld_x, out + r*ld_out), fp32 gamma and
 * beta of length `size`.  Batched form of kutacc_af2_layernorm (reference
 * src/normalization/layernorm_kernel.h:21-53), which handles exactly one row per call.
 */
kutacc_export int kutacc_hip_layernorm_rows(const void *x, int64_t ld_x, const float *gamma, const float *beta,
                                            void *out, int64_t ld_out, int64_t rows, int64_t size, float eps,
                                            int32_t dtype, void *stream);

/*
 * result[m,n] = beta*result[m,n] + sum_k act[m,k]*weight[n,k] (+ bias[n]); act row stride ld_act,
 * weight row stride ld_w, result dense [m,n].  Replaces kutacc::linear_kernel
 * (reference src/linear/linear.cpp:21-42).  bias may be NULL.
 */
kutacc_export int kutacc_hip_linear(const void *act, int64_t ld_act, const void *weight, int64_t ld_w,
                                    const float *bias, void *result, int64_t m, int64_t n, int64_t k, float beta,
                                    int32_t dtype, void *stream);

/*
 * Pair-bias producer: nb[h,i,j] = sum_c LN(z[i,j,:])[c] * w[h,c], written directly in the [H,S,S]
 * layout kutacc_af2_gating_attention expects.  One pass over z ([rows_i, rows_j, c_z], dense).
 * Fuses what a caller of the reference does with kutacc_af2_layernorm per row
 * (reference src/normalization/layernorm.cpp:17-20), kutacc_af2_linear
 * (reference src/linear/linear.cpp:45-50) and a [S,S,H]->[H,S,S] permute.  gamma/beta fp32 [c_z];
 * w is [H, c_z] in `dtype`.  If `z_norm` is non-NULL the normalised rows are also written there
 * (dense, same shape as z) so the attention input comes out of the same pass.
 */
kutacc_export int kutacc_hip_pair_bias(const void *z, const float *gamma, const float *beta, const void *w,
                                       void *nb, void *z_norm, int64_t rows_i, int64_t rows_j, int64_t c_z,
                                       int64_t nheads, float eps, int32_t dtype, void *stream);

/*
 * Strided bf16 matrix product with a fused epilogue: what kutacc::addmm (reference src/linear/mm.cpp:46-86) plus
 * the BlasExtendParams epilogue flags (reference include/kutacc.h:474-482) hand to the GEMM backend, and the
 * engine behind the transition and triangle-multiplication entry points below.
 *   C(m, n) = epilogue( sum_k A(m, k) * B(n, k) ),  fp32 accumulation, result rounded to bf16
 * A(m, k) sits at a + batch*a_stride_batch + m*a_stride_m + k*a_stride_k (one of the two strides must be 1 for
 * the MFMA kernel; anything else runs on a scalar kernel), B(n, k) likewise, C(m, n) at
 * c + batch*c_stride_batch + m*c_stride_m + n.  Epilogue: + bias (bias_axis 1: bias[n], the reference's
 * row_bias; 2: bias[m], its col_bias; 0: none), then ReLU if `relu`.  Gated form (a_gate != NULL, used by the
 * triangle projections, reference src/attention/triangle_multiplication.cpp:25-67): a second product
 * G = A_gate * B^T (A_gate laid out like A, bias_gate like bias) and
 *   C = bf16( bf16(A*B^T + bias) * mask[n] * sigmoid(bf16(G + bias_gate)) ),  mask bf16 at mask + batch*mask_stride_batch + n.
 */
typedef struct kutacc_hip_gemm_args {
    int64_t m, n, k, batches;
    int32_t dtype; /* KUTACC_DTYPE_BF16 */
    int32_t path;  /* KUTACC_HIP_PATH_*: AUTO, GENERIC (scalar kernel), FUSED (MFMA kernel or EUNSUPPORTED) */
    const void *a;
    int64_t a_stride_m, a_stride_k, a_stride_batch;
    const void *b;
    int64_t b_stride_n, b_stride_k, b_stride_batch;
    void *c;
    int64_t c_stride_m, c_stride_batch;
    const float *bias; /* fp32, NULL with bias_axis 0 */
    int32_t bias_axis;
    int32_t relu;
    const void *a_gate; /* NULL = plain epilogue */
    const float *bias_gate;
    const void *mask;
    int64_t mask_stride_batch;
} kutacc_hip_gemm_args_t;

kutacc_export int kutacc_hip_gemm(const kutacc_hip_gemm_args_t *args, void *stream);

/*
 * Transition: out = relu(x . w1^T + b1) . w2^T + b2 over `rows` dense rows (x, out [rows, c_o]; w1 [c_i, c_o] and
 * w2 [c_o, c_i] stored [out, in]; b1 fp32 [c_i], b2 fp32 [c_o]).  Replaces kutacc::transition_kernel (reference
 * src/attention/transition.cpp:21-39).  path AUTO: one kernel that keeps the hidden layer on chip when c_o is 128
 * or 256 and c_i a multiple of 64 (`intermediate` is then not touched and may be NULL), else two kutacc_hip_gemm
 * launches through `intermediate` ([rows, c_i], required); GENERIC: always the two launches; FUSED: the one kernel
 * or KUTACC_HIP_EUNSUPPORTED.
 */
kutacc_export int kutacc_hip_transition(const void *x, const void *w1, const float *b1, const void *w2, const float *b2,
                                        void *intermediate, void *out, int64_t rows, int64_t c_o, int64_t c_i,
                                        int32_t dtype, int32_t path, void *stream);

/* out[i, j, c] *= sigmoid(gate[i, j, c]) for c < size; element (i, j, c) of either tensor at i*stride0 + j*stride1 + c.
 * The element-wise pass of kutacc::last (reference src/attention/triangle_multiplication.cpp:129-150). */
kutacc_export int kutacc_hip_sigmoid_gate_rows(void *out, int64_t out_stride0, int64_t out_stride1, const void *gate,
                                               int64_t gate_stride0, int64_t gate_stride1, int64_t n0, int64_t n1,
                                               int64_t size, int32_t dtype, void *stream);

/* ---- between the operators: what a caller of the reference does in its framework, here on the device ---- */

/* kutacc_hip_pair_bias reading the pair tensor transposed: output row (i, j) (of nb[h, i, j] and of z_norm[i, j, :])
 * is computed from z[j, i, :], z dense [rows_j, rows_i, c_z].  This is the "ending node" orientation of triangle
 * attention without a separate pass that swaps the axes of z. */
kutacc_export int kutacc_hip_pair_bias_transposed(const void *z, const float *gamma, const float *beta, const void *w,
                                                  void *nb, void *z_norm, int64_t rows_i, int64_t rows_j, int64_t c_z,
                                                  int64_t nheads, float eps, int32_t dtype, void *stream);

/* bias[i, j] = 1e9 * (mask[i, j] - 1), formed as one fp32 multiply-add (the convention of reference
 * src/attention/global_attention.cpp:120-121) and rounded to `dtype`; dense [n0, n1].  transposed != 0 reads
 * mask[j, i] from a dense [n1, n0] mask.  The result is the `bias` argument of kutacc_af2_gating_attention. */
kutacc_export int kutacc_hip_mask_bias(const void *mask, void *bias, int64_t n0, int64_t n1, int32_t transposed,
                                       int32_t dtype, void *stream);

/* out[j, i, :] = in[i, j, :] for dense in [n0, n1, inner], out [n1, n0, inner]; in != out. */
kutacc_export int kutacc_hip_swap_leading_axes(const void *in, void *out, int64_t n0, int64_t n1, int64_t inner,
                                               int32_t dtype, void *stream);

/* acc[i, j, :] += delta[i, j, :], or delta[j, i, :] (delta dense [n1, n0, inner]) when swapped != 0; fp32 sum. */
kutacc_export int kutacc_hip_residual_add(void *acc, const void *delta, int64_t n0, int64_t n1, int64_t inner,
                                          int32_t swapped, int32_t dtype, void *stream);

/*
 * One triangle-attention block of the pair stack, in place:
 *   pair_act += gating_attention(input = LN(pair_act), nonbatched_bias = LN(pair_act) . bias_w^T, bias = 1e9*(pair_mask-1))
 * around the starting node (ending_node == 0: row i attends over j) or the ending node (ending_node != 0: the same
 * on the transposed pair tensor, result transposed back).  Four device passes on `stream`: LayerNorm + pair-bias
 * projection (one read of pair_act), mask bias, the attention operator, residual update.  bf16, head_size 32,
 * c_z = nheads * 32.  With c_z in {128, 256} and n_res <= 1024 (the shapes of the fused MFMA attention kernels) the
 * mask bias and the residual update happen inside the operator: three launches.  Any other size runs the chain as
 * separate passes with the operator on the tiled MFMA route (KUTACC_HIP_PATH_TILED), which needs four more
 * activation-sized buffers -- the workspace function answers for the size it is asked about.  `workspace`: device memory,
 * 256-byte aligned, at least kutacc_hip_triangle_attention_workspace(n_res, nheads) bytes; contents unspecified afterwards.
 */
typedef struct kutacc_hip_triangle_attention_args {
    int64_t n_res;
    int64_t nheads;
    int32_t dtype;       /* KUTACC_DTYPE_BF16 */
    int32_t ending_node; /* 0 starting node, 1 ending node */
    void *pair_act;        /* [n_res, n_res, c_z], updated in place */
    const void *pair_mask; /* [n_res, n_res], 1 = valid, 0 = padding */
    const float *ln_gamma; /* fp32 [c_z] */
    const float *ln_beta;  /* fp32 [c_z] */
    float ln_eps;
    int32_t reserved;
    const void *bias_w;    /* [nheads, c_z] pair-bias projection, stored [out, in] */
    const void *query_w, *key_w, *value_w, *gating_w, *output_w; /* [c_z, c_z] stored [out, in] */
    const float *gating_b, *output_b;                             /* fp32 [c_z] */
    void *workspace;
    int64_t workspace_bytes;
} kutacc_hip_triangle_attention_args_t;

kutacc_export int64_t kutacc_hip_triangle_attention_workspace(int64_t n_res, int64_t nheads);
kutacc_export int kutacc_hip_triangle_attention(const kutacc_hip_triangle_attention_args_t *args, void *stream);

/* LayerNorm over the channel axis of a channel-first tensor, written channel-last: out[p, c] = LN_c(x[c, p]) * gamma[c]
 * + beta[c], x element (c, p) at c*ld_x + p, out row stride ld_out.  The step between the triangle equation, which
 * leaves [c_i, n, n], and the output projection, which reads [n, n, c_i]; arithmetic as kutacc_af2_layernorm
 * (reference src/normalization/layernorm_kernel.h:21-53). */
kutacc_export int kutacc_hip_layernorm_channel_first(const void *x, int64_t ld_x, const float *gamma, const float *beta,
                                                     void *out, int64_t ld_out, int64_t channels, int64_t positions,
                                                     float eps, int32_t dtype, void *stream);

/* acc[m, n] += bf16(sum_k a[m, k] * w[n, k] + bias[n]) * sigmoid(gate[m, n]) in one pass: the output projection of the
 * triangle multiplication with its gating (kutacc::last, reference src/attention/triangle_multiplication.cpp:129-150)
 * and the residual update folded into the epilogue.  bf16; k in {128, 256}, n a multiple of 128, w dense [n, k], row
 * strides multiples of 8 elements, 16-byte aligned pointers; otherwise KUTACC_HIP_EUNSUPPORTED (run
 * kutacc_hip_gemm, kutacc_hip_sigmoid_gate_rows and kutacc_hip_residual_add instead). */
kutacc_export int kutacc_hip_gated_residual_projection(const void *a, int64_t a_ld, const void *w, const float *bias,
                                                       const void *gate, int64_t gate_ld, void *acc, int64_t acc_ld,
                                                       int64_t m, int64_t n, int64_t k, int32_t dtype, void *stream);

/*
 * One triangle-multiplication block of the pair stack, in place (outgoing or incoming edges):
 *   act    = LN_in(pair_act)
 *   left   = mask * (act . left_proj_w^T + left_proj_b) * sigmoid(act . left_gate_w^T + left_gate_b)       (right alike)
 *   center = sum_k left[i, k] * right[j, k]   (outgoing)      or      sum_k right[k, i] * left[k, j]   (incoming)
 *   pair_act += (LN_center(center) . output_w^T + output_b) * sigmoid(act . gating_w^T + gating_b)
 * i.e. the four kutacc_af2_triangle_multiplication_* steps (reference src/attention/triangle_multiplication.cpp:25-150)
 * with the two LayerNorms, the layout change and the residual a caller of the reference adds around them; seven
 * launches on `stream` (the output projection, its gating and the residual are one kernel when c_i is 128 or 256
 * and c_z a multiple of 128; with c_i = c_z = 128 that kernel projects the gate as well and, when n_res^2 is a multiple
 * of 8, normalises the centre on its way in: five launches, four when both gated projections share one).  bf16; weights stored [out, in]: *_proj_w, *_gate_w [c_i, c_z], output_w [c_z, c_i], gating_w
 * [c_z, c_z]; all biases and LayerNorm parameters fp32.  `workspace`: device memory, 256-byte aligned, at least
 * kutacc_hip_triangle_multiplication_workspace(n_res, c_z, c_i) bytes.
 */
typedef struct kutacc_hip_triangle_multiplication_args {
    int64_t n_res;
    int64_t c_z; /* channels of the pair activation */
    int64_t c_i; /* projected channels */
    int32_t dtype;    /* KUTACC_DTYPE_BF16 */
    int32_t incoming; /* 0 outgoing edges, 1 incoming edges */
    void *pair_act;        /* [n_res, n_res, c_z], updated in place */
    const void *pair_mask; /* [n_res, n_res] */
    const float *ln_in_gamma, *ln_in_beta; /* [c_z] */
    float ln_eps;
    int32_t reserved;
    const void *left_proj_w;
    const float *left_proj_b;
    const void *left_gate_w;
    const float *left_gate_b;
    const void *right_proj_w;
    const float *right_proj_b;
    const void *right_gate_w;
    const float *right_gate_b;
    const float *ln_center_gamma, *ln_center_beta; /* [c_i] */
    const void *output_w;
    const float *output_b;
    const void *gating_w;
    const float *gating_b;
    void *workspace;
    int64_t workspace_bytes;
} kutacc_hip_triangle_multiplication_args_t;

kutacc_export int64_t kutacc_hip_triangle_multiplication_workspace(int64_t n_res, int64_t c_z, int64_t c_i);
kutacc_export int kutacc_hip_triangle_multiplication(const kutacc_hip_triangle_multiplication_args_t *args, void *stream);

/*
 * One transition block in place: act += relu(LN(act) . w1^T + b1) . w2^T + b2 over `rows` dense rows of c_o channels
 * (kutacc_af2_transition, reference src/attention/transition.cpp:21-39, with the LayerNorm in front of it and the
 * residual behind it that a caller of the reference runs itself).  bf16.  With c_o in {128, 256} and c_i a multiple of
 * 64 (<= 2048) this is one kernel and one read and one write of the activation; `workspace` may then be NULL.
 * Other shapes run LayerNorm, the two GEMMs and the residual as separate passes through `workspace` (256-byte
 * aligned, kutacc_hip_transition_block_workspace(rows, c_o, c_i) bytes).
 */
kutacc_export int64_t kutacc_hip_transition_block_workspace(int64_t rows, int64_t c_o, int64_t c_i);
kutacc_export int kutacc_hip_transition_block(void *act, const float *ln_gamma, const float *ln_beta, float ln_eps,
                                              const void *w1, const float *b1, const void *w2, const float *b2,
                                              void *workspace, int64_t workspace_bytes, int64_t rows, int64_t c_o,
                                              int64_t c_i, int32_t dtype, void *stream);

/* kutacc_hip_layernorm_rows on a grid of rows read transposed: out row (i, j) of a dense [rows_i, rows_j, size] tensor is
 * the LayerNorm of row (j, i) of the dense [rows_j, rows_i, size] input.  The column-wise MSA attention's input without
 * a separate pass that swaps the axes of the msa. */
kutacc_export int kutacc_hip_layernorm_rows_transposed(const void *x, const float *gamma, const float *beta, void *out,
                                                       int64_t rows_i, int64_t rows_j, int64_t size, float eps,
                                                       int32_t dtype, void *stream);

/*
 * One MSA attention block, in place on msa_act [n_seq, n_res, c_m] (c_m = nheads * 32):
 *   column == 0, row-wise with pair bias: msa_act += gating_attention(LN(msa_act), bias from msa_mask,
 *                nonbatched_bias = LN_pair(pair_act) . bias_w^T), every sequence attending over the residues;
 *   column != 0, column-wise: the same operator without pair bias on the msa with its leading axes exchanged, every
 *                residue attending over the sequences; no transposed copy of the msa is made (the LayerNorm reads it
 *                transposed, the output projection adds its result back transposed).
 * bf16.  With c_m in {128, 256} and an attended axis of at most 1024 (the shapes of the fused MFMA attention kernels) mask
 * bias and residual update happen inside the operator; any other size runs them as passes of their own around the operator
 * on the tiled MFMA route, with four more activation-sized buffers in the workspace.
 * pair_act [n_res, n_res, c_z], its LayerNorm parameters and bias_w [nheads, c_z] are read by the row-wise form only.
 */
typedef struct kutacc_hip_msa_attention_args {
    int64_t n_seq;
    int64_t n_res;
    int64_t nheads;
    int64_t c_z;     /* channels of pair_act (row-wise form) */
    int32_t dtype;   /* KUTACC_DTYPE_BF16 */
    int32_t column;  /* 0 row-wise with pair bias, 1 column-wise */
    void *msa_act;          /* [n_seq, n_res, c_m], updated in place */
    const void *msa_mask;   /* [n_seq, n_res], 1 = valid */
    const float *ln_gamma, *ln_beta; /* [c_m] */
    float ln_eps;
    int32_t reserved;
    const void *pair_act;
    const float *pair_ln_gamma, *pair_ln_beta; /* [c_z] */
    const void *bias_w;
    const void *query_w, *key_w, *value_w, *gating_w, *output_w; /* [c_m, c_m] stored [out, in] */
    const float *gating_b, *output_b;
    void *workspace;
    int64_t workspace_bytes; /* >= kutacc_hip_msa_attention_workspace(n_seq, n_res, nheads, column), 256-byte aligned */
} kutacc_hip_msa_attention_args_t;

kutacc_export int64_t kutacc_hip_msa_attention_workspace(int64_t n_seq, int64_t n_res, int64_t nheads, int32_t column);
kutacc_export int kutacc_hip_msa_attention(const kutacc_hip_msa_attention_args_t *args, void *stream);

/* ---- runtime control (no counterpart in the reference; the CPU library has no device) ---- */

/* Stream used when a `stream` argument is NULL and by the handle-based API of kutacc.h.
 * Default: the HIP null stream.  The setting belongs to the calling host thread (like a framework's current
 * stream): threads that drive the library on different streams each set their own.  A thread that has never set one
 * uses the value set last by any thread, so worker threads of a host that configured the library once inherit it. */
kutacc_export void kutacc_hip_set_stream(void *stream);
kutacc_export void *kutacc_hip_get_stream(void);

/* 1 (default): the handle-based API blocks until the device work has finished, as the CPU library
 * does.  0: it returns after enqueueing when all operands are device pointers.  Per host thread, inherited like the stream. */
kutacc_export void kutacc_hip_set_blocking(int blocking);

/* Calls on host pointers run on device copies of their operands; those copies are kept between calls (a repeated
 * shape allocates once).  This frees them and returns the number of bytes released.  Call it when no such call is
 * in flight. */
kutacc_export int64_t kutacc_hip_release_staging(void);

/* Per-kernel timing for benchmarks.  While enabled, each kernel launched by this library is
 * bracketed by hipEvents on its stream.  kutacc_hip_profile_read(i, ...) waits for the recorded
 * events and returns entry i (0 on success, -1 past the last entry): kernel name, summed
 * milliseconds, number of launches and the algorithmic flops of one launch.  Enabling clears the
 * previous totals. */
kutacc_export void kutacc_hip_profile_enable(int on);
kutacc_export int kutacc_hip_profile_read(int index, char *name, int name_len, double *total_ms, int64_t *launches,
                                          double *flops_per_launch);

/* Tuning hooks for tests and experiments; name/value strings, 0 on success, KUTACC_HIP_EINVAL for an unknown name.
 *   "plan"      "bpw,gw": force the long-sequence attention kernel with bpw (1-4) query blocks per wave and gw (1, 2, 4)
 *               weight matrices per LDS group where that fits the device; anything else: the planner decides (default)
 *   "fragments" "0": keep the attention kernels off the fragment-major pair bias (general softmax blocks); "1": default
 *   "debug"     "1": one line per fused call on stderr with the plan taken; "0": default
 *   "row_pairs" "0": never the attention kernel that walks two batch rows per step (128 channels up to 384 positions,
 *               256 channels up to 256);
 *               "1": wherever it can run; anything else (default): where every workgroup has at least two batch rows
 *   "gemm_tile" "128" / "256" / "192" / "direct": the batched products of kutacc_af2_triangle_multiplication_equation
 *               always on 128 x 128 tiles / on 256 x 256 tiles staged through registers wherever the shape has whole
 *               ones / on 192 x 192 tiles wherever it has / on 256 x 256 tiles whose operands are loaded straight into
 *               the LDS wherever it has (and k is at least 96); anything else (default): the direct 256 x 256 tiles
 *               where every CU gets at least two, else 192 x 192 where every CU gets at least two, else 128 x 128
 *   "gated_projection" "streaming" / "tiled": the gated projections of kutacc_af2_triangle_multiplication_calc_proj and
 *               of kutacc_hip_triangle_multiplication at 128 channels on the kernel that gives every wave its own positions
 *               and keeps the weights in the LDS / on the tiled kernel of the general products; "blocks" or anything else
 *               (default): on the kernel that keeps a wave's weights in registers and shares the activation through
 *               the LDS
 *   "layernorm" "fused": kutacc_hip_triangle_attention and kutacc_hip_msa_attention let the attention kernel normalise its
 *               input rows itself where it can (sequence lengths of the persistent kernel), which drops the normalised
 *               copy from the workspace and costs 8-15 % of the block's time; "separate" or "auto" (default): the
 *               LayerNorm runs as a pass of its own.  The workspace functions answer for the mode in force when they are
 *               called: query and call under the same setting.
 *   "scratch"   "reference": kutacc_af2_gating_attention runs on the tiled MFMA route (KUTACC_HIP_PATH_TILED; the
 *               shape-agnostic kernels where that route does not take the call), which fills the caller's q, k, v and
 *               gate tensors as the reference's kernel does (src/attention/gating_attention.cpp:47-66) -- for callers or
 *               tests that read them; about twice the time of the fused kernels.  Anything else (default): the fused MFMA
 *               kernels where they apply, which leave k, v and gate untouched and use q as workspace.
 *   "pointer_checks" "0": the handle-based attention entry points classify only `input` (host or device) and take the
 *               caller's word that every other operand lives in the same place, which saves about fifteen driver
 *               queries per call; "1": every operand is checked and mixed calls are rejected (default) */
kutacc_export int kutacc_hip_set_tuning(const char *name, const char *value);

/* The process-wide sticky error flag behind KUTACC_CHECK (reference src/utils/check.cpp:16 keeps it
 * hidden and never resets it).  Reading/clearing it is an addition for tests and long-lived hosts. */
kutacc_export int kutacc_hip_error_flag(void);
kutacc_export void kutacc_hip_clear_error(void);

/* Tensor descriptors for callers that cannot run the C++ TensorWrapper constructor
 * (reference include/kutacc.h:484-497).  The returned handle is what get_tensor() returns. */
kutacc_export void *kutacc_hip_tensor_create(void *data, const int64_t *sizes, const int64_t *strides, int64_t dim,
                                             int32_t dtype);
kutacc_export void kutacc_hip_tensor_destroy(void *handle);

#ifdef __cplusplus
}
#endif
#endif /* KUTACC_HIP_H */
