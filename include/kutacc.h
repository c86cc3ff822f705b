/*
 * kutacc.h -- public interface of the MI355X (gfx950) build of the KuTACC gated-attention path.
 *
 * Interface contract: every name, argument order, struct layout and enum value below is the one a
 * caller of the Kunpeng library already compiles against (reference include/kutacc.h), restricted
 * to the entry points that feed or form the fused gated-attention operator.  A program built
 * against the reference header links and runs against this library for those entry points; the
 * remaining kutacc_af2_* / kutacc_comm_* symbols are exported as "not implemented on this
 * backend" stubs (see kutacc_amd/csrc/unsupported.cpp) so that the shared object still resolves.
 *
 * Differences a caller can observe, all additive:
 *   - DType gains kFP32 (value 2, after kBF16) so that fp32 tensors can be described.
 *   - data pointers may be HIP device pointers (fast path) or host pointers (staged through the
 *     device); the two kinds must not be mixed within one call.
 *   - "prepacked" operands are plain row-major: the pack routines below are identity copies.
 *
 * Requires a compiler that knows the __bf16 type (ROCm clang++ / hipcc).
 */
#ifndef KUTACC_H
#define KUTACC_H

#include <cstddef>
#include <cstdint>
#include <vector>

#define kutacc_export __attribute__((visibility("default")))

/* Status codes; only kutacc_get_version returns one (reference include/kutacc.h:28-29). */
#define KUTACC_OK 0
#define KUTACC_ERROR (-1)

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque tensor descriptor; produced by kutacc::TensorWrapper::get_tensor()
 * (reference include/kutacc.h:49). */
typedef void *kutacc_tensor_h;

/* Version record, six C strings owned by the library (reference include/kutacc.h:32-39). */
typedef struct kutacc_version {
    const char *product_name;
    const char *product_version;
    const char *component_name;
    const char *component_version;
    const char *component_abi_version;
    const char *component_appendinfo;
} kutacc_version_t;

/* Fills *version; returns KUTACC_ERROR for a null argument
 * (reference include/kutacc.h:47, src/version/version.cpp:28-35). */
kutacc_export int kutacc_get_version(kutacc_version_t *version);

/* Rank bookkeeping of the reference's shared-memory collectives (reference include/kutacc.h:51-53).
 * Exported for link compatibility; this single-GPU build never changes them. */
kutacc_export extern int64_t world_size;
kutacc_export extern int64_t rank;

/* Weights of one gated-attention block (reference include/kutacc.h:77-89).
 *   query_w/key_w/value_w/gating_w/output_w : [nchannels, nchannels], stored [out, in] row-major
 *   gating_b/output_b                       : fp32 [nchannels]
 *   nchannels == nheads * head_size */
typedef struct kutacc_af2_attention_weights {
    int64_t nchannels;
    int64_t nheads;
    int64_t head_size;

    kutacc_tensor_h query_w;
    kutacc_tensor_h key_w;
    kutacc_tensor_h value_w;
    kutacc_tensor_h gating_w;
    kutacc_tensor_h gating_b;
    kutacc_tensor_h output_w;
    kutacc_tensor_h output_b;
} kutacc_af2_attention_weights_t;

/* Problem extent plus caller-owned scratch tensors (reference include/kutacc.h:95-104).
 *   q, k, gate, avg : [batch, seq_len, nheads, head_size]
 *   v               : [nheads, head_size, batch, seq_len]  (transposed, as the reference writes it,
 *                     src/attention/gating_attention.cpp:57-61,123-127)
 * The library may overwrite them; after a call `avg` holds the gated weighted average. */
typedef struct kutacc_af2_attention_inputs {
    int64_t batch;
    int64_t seq_len;

    kutacc_tensor_h q;
    kutacc_tensor_h k;
    kutacc_tensor_h v;
    kutacc_tensor_h gate;
    kutacc_tensor_h avg;
} kutacc_af2_attention_inputs_t;

/*
 * Fused Evoformer gated attention with pair bias (reference include/kutacc.h:297-300,
 * src/attention/gating_attention.cpp:33-200):
 *
 *   q,k,v = input.Wq^T, input.Wk^T, input.Wv^T         gate = input.Wg^T + gating_b
 *   p     = softmax_k(q.k^T / sqrt(head_size) + bias[b,k] + nonbatched_bias[h,q,k])
 *   out   = ((p.v) * sigmoid(gate)).Wo^T + output_b
 *
 *   input            [batch*seq_len, nchannels], already layer-normalised
 *   bias             [batch, 1, 1, seq_len] mask bias (0 or -1e9), element (b,k) at b*strides[0]+k
 *   nonbatched_bias  [nheads, seq_len, seq_len]; a tensor whose sizes[0]==0 means "absent".  Entries of -inf or below
 *                    -45 000 exclude a (query, key) pair, as in the reference.  One corner differs: for a query that
 *                    has no key left whose mask bias is 0 and whose pair bias is above that bound, the reference
 *                    attends uniformly over the keys the mask bias excludes, the MFMA kernels over the keys the pair
 *                    bias excludes (they carry such entries as the largest fp16 magnitude, which lies above -1e9)
 *   out              [batch, seq_len, nchannels]
 *   block_size       query tiling of the CPU implementation; validated (>0), otherwise advisory
 *
 * All six pointer arguments must be non-null.  Violations print one KUTACC_CHECK line on stderr,
 * latch the process-wide error flag and return without touching `out`.
 */
kutacc_export void kutacc_af2_gating_attention(kutacc_tensor_h input, kutacc_af2_attention_inputs_t *q_based_ptr,
                                               kutacc_tensor_h bias, kutacc_tensor_h nonbatched_bias,
                                               kutacc_af2_attention_weights_t *weight_ptr, kutacc_tensor_h out,
                                               int64_t block_size);

/**
 * @brief global (extra-MSA column) attention: one query per batch row and head (the masked mean of the row),
 *        one key/value head shared by all heads.  Reference include/kutacc.h:292-307 (declaration),
 *        src/attention/global_attention.cpp:167-205 (entry), :30-164 (kernel).
 * @param [in] q_based_ptr batch, seq_len and the scratch tensors q [batch, nchannels], k [batch*seq_len, head_size],
 *             v [head_size, batch*seq_len], gate [batch, seq_len, nchannels], avg = q_avg [batch, nchannels];
 *             this backend writes only avg (the masked mean) and leaves q, k, v, gate untouched
 * @param [in] q_data shape [batch, seq_len, nchannels], bf16
 * @param [in] q_mask shape [batch, seq_len, 1], bf16
 * @param [in] weight_ptr nchannels must be 64; query_w, gating_w, output_w [64, 64], key_w, value_w [head_size, 64],
 *             all stored [out, in]; gating_b, output_b fp32 [64]
 * @param [out] out shape [batch, seq_len, nchannels], bf16
 */
kutacc_export void kutacc_af2_global_attention(kutacc_af2_attention_inputs_t *q_based_ptr, kutacc_tensor_h q_data,
                                               kutacc_tensor_h q_mask, kutacc_af2_attention_weights_t *weight_ptr,
                                               kutacc_tensor_h out);

/* ---- transition and triangle multiplication: the pair/MSA-stack operators around the attention ---- */

/* Weights of the transition (reference include/kutacc.h:194-202).  c_o = channels of the activation,
 * c_i = channels of the hidden layer; linear1_w [c_i, c_o] and linear2_w [c_o, c_i] stored [out, in],
 * linear1_b fp32 [c_i], linear2_b fp32 [c_o]. */
typedef struct kutacc_af2_trans_weights {
    int64_t c_o;
    int64_t c_i;

    kutacc_tensor_h linear1_w;
    kutacc_tensor_h linear1_b;
    kutacc_tensor_h linear2_w;
    kutacc_tensor_h linear2_b;
} kutacc_af2_trans_weights_t;

/* Activations of the transition (reference include/kutacc.h:208-214): input_act dense [batch*n_res, c_o]
 * (already layer-normalised), intermediate_act dense [batch*n_res, c_i] caller-owned scratch that receives
 * relu(input_act . linear1_w^T + linear1_b). */
typedef struct kutacc_af2_trans_act_inputs {
    int64_t batch;
    int64_t n_res;

    kutacc_tensor_h input_act;
    kutacc_tensor_h intermediate_act;
} kutacc_af2_trans_act_inputs_t;

/*
 * out = relu(input_act . linear1_w^T + linear1_b) . linear2_w^T + linear2_b, out dense [batch*n_res, c_o]
 * (reference include/kutacc.h:321-322, src/attention/transition.cpp:21-67).  Device pointers only.
 */
kutacc_export void kutacc_af2_transition(kutacc_af2_trans_act_inputs_t *trans_inputs_ptr,
                                         kutacc_af2_trans_weights_t *trans_weights_ptr, kutacc_tensor_h out);

/* Weights of one triangle projection, left or right (reference include/kutacc.h:154-162): proj_w and gate_w
 * [c_i, c_o] stored [out, in] (c_o = channels of the pair activation, c_i = projected channels), proj_b and
 * gate_b fp32 [c_i]. */
typedef struct kutacc_af2_tm_proj_weights {
    int64_t c_o;
    int64_t c_i;

    kutacc_tensor_h proj_w;
    kutacc_tensor_h proj_b;
    kutacc_tensor_h gate_w;
    kutacc_tensor_h gate_b;
} kutacc_af2_tm_proj_weights_t;

/* Activations of the triangle multiplication (reference include/kutacc.h:168-175): input_act dense
 * [n_res, n_res_gather, c_o] (layer-normalised pair activation), proj_act [c_i, n_res, n_res_gather] channel-first
 * output of the projection step, proj_act_gate a scratch tensor of the same shape. */
typedef struct kutacc_af2_tm_act_inputs {
    int64_t n_res;
    int64_t n_res_gather;

    kutacc_tensor_h proj_act;
    kutacc_tensor_h input_act;
    kutacc_tensor_h proj_act_gate;
} kutacc_af2_tm_act_inputs_t;

/* Weights of the output step (reference include/kutacc.h:181-189): gating_w [c_o, c_o], output_proj_w [c_o, c_i],
 * both stored [out, in]; gating_b, output_proj_b fp32 [c_o]. */
typedef struct kutacc_af2_tm_linear_weights {
    int64_t c_o;
    int64_t c_i;

    kutacc_tensor_h gating_w;
    kutacc_tensor_h gating_b;
    kutacc_tensor_h output_proj_w;
    kutacc_tensor_h output_proj_b;
} kutacc_af2_tm_linear_weights_t;

/*
 * proj_act[c, i, j] = (input_act[i, j, :] . proj_w[c, :] + proj_b[c]) * mask[i, j] * sigmoid(input_act[i, j, :] . gate_w[c, :] + gate_b[c])
 * (reference include/kutacc.h:426-429, src/attention/triangle_multiplication.cpp:25-67, 152-178).
 * mask bf16 [n_res, n_res_gather].  This backend forms both products in one kernel and leaves proj_act_gate
 * untouched; `input_prepack` (a layout hint of the CPU GEMM) is ignored.  Device pointers only.
 */
kutacc_export void kutacc_af2_triangle_multiplication_calc_proj(kutacc_af2_tm_act_inputs_t *tm_acts_ptr,
                                                                kutacc_tensor_h mask,
                                                                kutacc_af2_tm_proj_weights_t *tm_weights_ptr,
                                                                bool input_prepack);

/*
 * Per channel c of [c_i, n_res_gather, n_res_gather] tensors (reference include/kutacc.h:436-439,
 * src/attention/triangle_multiplication.cpp:72-101, 180-195):
 *   outgoing (is_incoming == false): center[c, i, j] = sum_k left[c, i, k] * right[c, j, k]
 *   incoming (is_incoming == true) : center[c, i, j] = sum_k right[c, k, i] * left[c, k, j]
 */
kutacc_export void kutacc_af2_triangle_multiplication_equation(kutacc_tensor_h center_act,
                                                               kutacc_tensor_h left_proj_act,
                                                               kutacc_tensor_h right_proj_act, int64_t n_res_gather,
                                                               bool is_incoming);

/*
 * gate = input_act . gating_w^T + gating_b and out = center_act . output_proj_w^T + output_proj_b, rows (i, j) of
 * [n_res, n_res_gather, .] tensors; center_act is the channel-last, layer-normalised result of the equation
 * (reference include/kutacc.h:446-448, src/attention/triangle_multiplication.cpp:106-127, 197-224).
 */
kutacc_export void kutacc_af2_triangle_multiplication_gate_and_out_linear(
    kutacc_tensor_h gate, kutacc_tensor_h out, kutacc_af2_tm_act_inputs_t *tm_acts_ptr, kutacc_tensor_h center_act,
    kutacc_af2_tm_linear_weights_t *tm_weights_ptr, bool input_prepack);

/*
 * out[i, j, :c_o] *= sigmoid(gate[i, j, :c_o]) (reference include/kutacc.h:455-456,
 * src/attention/triangle_multiplication.cpp:129-150, 226-240).
 */
kutacc_export void kutacc_af2_triangle_multiplication_last(kutacc_tensor_h out, kutacc_tensor_h gate, int64_t n_res,
                                                           int64_t n_res_gather, int64_t c_o);

/*
 * LayerNorm of ONE row of `size` elements, bf16 in/out, fp32 gamma/beta
 * (reference include/kutacc.h:334, src/normalization/layernorm_kernel.h:21-53).
 * Raw pointers, not handles.  See kutacc_hip_layernorm_rows in kutacc_hip.h for the batched form.
 */
kutacc_export void kutacc_af2_layernorm(__bf16 *data, float *gamma, float *beta, int64_t size, float eps, __bf16 *out);

/*
 * result[m,n] = beta*result + act[m,k].weight[n,k]^T (+ bias_data[n]), bf16 operands and result
 * (reference include/kutacc.h:399-400, src/linear/linear.cpp:21-50).  m = numel(act)/k,
 * k = last dim of act, n = numel(weight)/k; result is written contiguously as [m,n].
 */
kutacc_export void kutacc_af2_linear(kutacc_tensor_h act, kutacc_tensor_h weight, float *bias_data,
                                     kutacc_tensor_h result, int64_t beta);

/*
 * "Pre-pack" a [n,k] bf16 matrix with leading dimension ldb (reference include/kutacc.h:407-408,
 * src/linear/mm.cpp:94-110).  On this backend the packed layout is dense row-major [n,k], so this
 * is a strided copy; num_threads is accepted and ignored.
 */
kutacc_export void kutacc_af2_linear_weight_prepack(const __bf16 *weight, __bf16 *result, int64_t n, int64_t k,
                                                    int64_t ldb, int64_t num_threads = 0);

/*
 * Element count of a packed operand: m*k for identifier 'A', k*n for 'B'
 * (reference include/kutacc.h:418, src/utils/blas.cpp:93-98).
 */
kutacc_export size_t kutacc_af2_gemm_pack_get_size(char identifier, char transa, char transb, int m, int n, int k);

#ifdef __cplusplus
}
#endif

#ifdef __cplusplus
namespace kutacc {

/* Element type tag carried by a tensor descriptor (reference include/kutacc.h:467-471).
 * kFP32 is new on this backend and sits after the reference's values. */
typedef enum TensorDataType {
    kInt64 = 0,
    kBF16 = 1,
    kFP32 = 2,
    kNumTypes
} DType;

/* GEMM epilogue switches of the reference's BLAS shim (reference include/kutacc.h:474-482).
 * Kept so that callers naming the type still compile; this backend reads none of it. */
struct BlasExtendParams {
    int64_t num_threads;
    bool prepack_a;
    bool prepack_b;
    bool row_bias;
    bool col_bias;
    void *bias;
    bool relu;
};

/* Owns one strided, non-owning view {data, sizes, strides (in elements), dim, dtype} and hands it
 * out as a kutacc_tensor_h (reference include/kutacc.h:484-497, src/tensor/tensor.cpp:20-30,88-92).
 * As in the reference, copying a TensorWrapper is not supported. */
struct kutacc_export TensorWrapper {
private:
    kutacc_tensor_h tensor_;

public:
    TensorWrapper(void *data_ptr, std::vector<int64_t> &&sizes, std::vector<int64_t> &&strides, int64_t dim,
                  DType dtype);
    TensorWrapper();
    kutacc_tensor_h get_tensor()
    {
        return tensor_;
    }
    ~TensorWrapper();
};
} // namespace kutacc
#endif

#endif /* KUTACC_H */
