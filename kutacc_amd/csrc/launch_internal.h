// C++-side declarations of the per-translation-unit launchers behind the extern "C" layer of
// kutacc_hip.h.  Each returns the same int convention as that layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kutacc_hip.h"

// Turn a HIP status into the int the C ABI returns (0 = success, else the hipError_t value).
static inline int kutacc_hip_status(hipError_t e) { return e == hipSuccess ? 0 : (int)e; }

// 16-byte alignment of a pointer: what the vector loads and stores of the fast kernels need
static inline bool kutacc_hip_aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// One-time kernel set-up and device properties are per device (hipFuncSetAttribute applies to the current device only),
// and a process may drive several: the launchers keep what they have done in small tables indexed by the device ordinal.
constexpr int KUTACC_DEVICE_SLOTS = 64;

// ordinal of the current device, or -1 when it cannot be had or does not fit the tables (then nothing is remembered)
static inline int kutacc_device_slot()
{
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    return (dev >= 0 && dev < KUTACC_DEVICE_SLOTS) ? dev : -1;
}

// Opt a kernel into `bytes` of dynamic LDS on the current device unless the table says it already has that much.
// `table` is a zero-initialised array of KUTACC_DEVICE_SLOTS entries owned by the caller, one per kernel instantiation.
static inline hipError_t kutacc_opt_in_lds(const void *kernel, size_t bytes, size_t *table)
{
    const int slot = kutacc_device_slot();
    if (slot < 0 || bytes > table[slot]) {
        const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess) {
            return e;
        }
        if (slot >= 0) {
            table[slot] = bytes;
        }
    }
    return hipSuccess;
}

// an integer attribute of the current device, remembered per device in `table` (zero-initialised, values are positive)
static inline int kutacc_device_attribute(hipDeviceAttribute_t attr, int fallback, int *table)
{
    const int slot = kutacc_device_slot();
    if (slot >= 0 && table[slot] > 0) {
        return table[slot];
    }
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, attr, dev) != hipSuccess || v <= 0) {
        (void)hipGetLastError();
        return fallback;
    }
    if (slot >= 0) {
        table[slot] = v;
    }
    return v;
}

namespace kutacc_launch {

// generic_kernels.hip
int gating_attention_generic(const kutacc_hip_attention_args_t &args, hipStream_t stream);
int gemm_nt(int32_t dtype, const void *a, int64_t lda, const void *w, int64_t ldw, const float *bias, void *c,
            int64_t c_rs, int64_t c_cs, int64_t m, int64_t n, int64_t k, float beta, hipStream_t stream);

// tiled_attention.hip: bf16, any seq_len, head sizes 8 .. 64; projections into the caller's q, k, v, gate as the reference
// leaves them, attention on MFMA tiles with an online softmax
bool tiled_attention_supports(const kutacc_hip_attention_args_t &args);
int gating_attention_tiled(const kutacc_hip_attention_args_t &args, hipStream_t stream);

// fp32_attention.hip: fp32 storage on the fp32 matrix core (head_size 32, up to 256 channels, up to 224 positions)
bool fp32_attention_supports(const kutacc_hip_attention_args_t &args);
int gating_attention_fp32(const kutacc_hip_attention_args_t &args, hipStream_t stream);

// fused_attention.hip
bool fused_attention_supports(const kutacc_hip_attention_args_t &args);
// `residual`: what the output projection does with its result -- store it in args.out (the operator as the reference
// defines it), add it to args.out, or add row (b, s) of it to row (s, b) of args.out, then [seq_len, batch, C]
constexpr int FUSED_OUT_STORE = 0, FUSED_OUT_ADD = 1, FUSED_OUT_ADD_TRANSPOSED = 2;
// bias_is_mask: args.bias holds the 0/1 mask instead of the mask bias, element (b, k) at b*bias_stride_b + k*bias_stride_k,
// and the kernels form 1e9*(mask-1) themselves (no separate mask-bias pass; a transposed mask is a stride choice)
struct FusedAttentionOptions {
    int out_mode = FUSED_OUT_STORE;
    bool bias_is_mask = false;
    int64_t bias_stride_k = 1;
    // the fragment-major copy of the pair bias already lies in args.q (written by pair_bias with the layout
    // fused_attention_fragment_layout reports): the pass that makes it is skipped
    bool nb_fragments_ready = false;
    // the fp32 tiles of the pair bias that the two-row kernel reads already lie there (written by pair_bias with the
    // layout fused_attention_tile_layout reports for the same options): the pass that makes them is skipped
    bool nb_tiles_ready = false;
    // device memory (16-byte aligned) that takes the fragment-major copy of the pair bias instead of args.q, which is then
    // neither read nor written; a call whose copy does not fit is rejected with KUTACC_HIP_EINVAL
    void *fragment_workspace = nullptr;
    size_t fragment_workspace_bytes = 0;
    // LayerNorm of the input rows inside the head kernel (args.input is then the un-normalised tensor): fp32 gamma and
    // beta of nheads*head_size values, 16-byte aligned.  Only where fused_layernorm_supported says so.
    const float *ln_gamma = nullptr, *ln_beta = nullptr;
    float ln_eps = 0.f;
    // elements from one batch row of args.input to the next; 0 = seq_len * input_ld (dense).  With input_ld as the
    // stride between sequence positions this lets the kernels read an [S, B, C] tensor as [B, S, C] without a copy.
    int64_t input_stride_b = 0;
};
// Whether gating_attention_fused can normalise the input rows itself for this call (the persistent kernel in log2 units)
bool fused_layernorm_supported(const kutacc_hip_attention_args_t &args, const FusedAttentionOptions &opt);
// Whether gating_attention_fused would keep a fragment-major copy of the pair bias in args.q, and the copy's extent:
// [nheads][*nb query blocks][*nt key tiles][2][64 lanes] x 16 bytes.
bool fused_attention_fragment_layout(const kutacc_hip_attention_args_t &args, int *nb, int *nt);
// Whether gating_attention_fused would run the two-row kernel on this call under these options (and the tuning in force)
// and keep the fp32 tiles of the pair bias in args.q or the options' workspace, and their extent:
// [nheads][*nb query blocks][*nt key tiles][4][64 lanes] x 16 bytes.
bool fused_attention_tile_layout(const kutacc_hip_attention_args_t &args, const FusedAttentionOptions &opt, int *nb, int *nt);
int gating_attention_fused(const kutacc_hip_attention_args_t &args, hipStream_t stream,
                           const FusedAttentionOptions &opt = FusedAttentionOptions());

// "plan" / "fragments" / "debug" hooks of the attention launcher (kutacc_hip_set_tuning); KUTACC_HIP_EINVAL for other names
int fused_attention_tuning(const char *name, const char *value);
// "gemm_tile" hook of the matrix products of the pair stack; KUTACC_HIP_EINVAL for other names
int pair_gemm_tuning(const char *name, const char *value);

bool row_projection_supports(const void *a, int64_t a_ld, const void *w, const float *bias, const void *out, int64_t out_ld,
                             int64_t m, int64_t n, int64_t k);
int row_projection(const void *a, int64_t a_ld, const void *w, const float *bias, void *out, int64_t out_ld, int64_t m,
                   int64_t n, int64_t k, hipStream_t stream);

int row_projection_gated_residual(const void *a, int64_t a_ld, const void *w, const float *bias, const void *gate,
                                  int64_t gate_ld, void *acc, int64_t acc_ld, int64_t m, int64_t n, int64_t k,
                                  hipStream_t stream);
// the same with the gate projected inside the kernel from rows y of 128 features (no gate tensor); 128 features in and out
bool row_projection_projected_gate_supports(const void *a, int64_t a_ld, const void *w, const float *bias, const void *y,
                                            int64_t y_ld, const void *wg, const float *bg, const void *acc, int64_t acc_ld,
                                            int64_t m, int64_t n, int64_t k, int64_t ky);
// ln_gamma != nullptr: `a` is channel-first ([128, m], channel stride a_ld) and is normalised over its channels on the way in
int row_projection_projected_gate_residual(const void *a, int64_t a_ld, const void *w, const float *bias, const void *y,
                                           int64_t y_ld, const void *wg, const float *bg, void *acc, int64_t acc_ld, int64_t m,
                                           hipStream_t stream, const float *ln_gamma = nullptr, const float *ln_beta = nullptr,
                                           float ln_eps = 0.f);

// global_attention.hip
int global_attention(const kutacc_hip_global_attention_args_t &args, hipStream_t stream);

// pair_stack.hip
// `second`: a second gated projection of the same B and mask to run in the same launch (KUTACC_HIP_EUNSUPPORTED, with
// nothing launched, when the two cannot share one: the caller then makes two calls)
int pair_gemm(const kutacc_hip_gemm_args_t &args, hipStream_t stream, const kutacc_hip_gemm_args_t *second = nullptr);
bool transition_fused_supports(int64_t rows, int64_t c_o, int64_t c_i, const void *x, const void *w1, const float *b1,
                               const void *w2, const float *b2, const void *out);
int transition_fused(const void *x, const void *w1, const float *b1, const void *w2, const float *b2, void *out,
                     int64_t rows, int64_t c_o, int64_t c_i, hipStream_t stream);
int transition_block_fused(void *act, const float *ln_gamma, const float *ln_beta, float ln_eps, const void *w1, const float *b1,
                           const void *w2, const float *b2, int64_t rows, int64_t c_o, int64_t c_i, hipStream_t stream);
int sigmoid_gate_rows(void *out, int64_t out_s0, int64_t out_s1, const void *gate, int64_t gate_s0, int64_t gate_s1,
                      int64_t n0, int64_t n1, int64_t size, hipStream_t stream);

// glue_kernels.hip
int mask_bias(const void *mask, void *bias, int64_t n0, int64_t n1, int transposed, int32_t dtype, hipStream_t stream);
int swap_leading_axes(const void *in, void *out, int64_t n0, int64_t n1, int64_t inner, int32_t dtype, hipStream_t stream);
int residual_add(void *acc, const void *delta, int64_t n0, int64_t n1, int64_t inner, int swapped, int32_t dtype,
                 hipStream_t stream);

int layernorm_channel_first(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                            int64_t channels, int64_t positions, float eps, int32_t dtype, hipStream_t stream);

// row_kernels.hip
// swap_j != 0: rows are pairs (i, j) of an [rows / swap_j, swap_j] grid and output row (i, j) is computed from input
// row (j, i) of the transposed grid
int layernorm_rows(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out, int64_t ld_out,
                   int64_t rows, int64_t size, float eps, int32_t dtype, hipStream_t stream, int64_t swap_j = 0);
// fragments != nullptr: the copy the attention kernels read is written as well, values times log2(e): fp16 fragments
// [nheads][frag_nb][frag_nt][2][64] x 16 bytes, or with frag_tiles != 0 the fp32 tiles of the two-row kernel,
// [nheads][frag_nb][frag_nt][4][64] x 16 bytes; only where pair_bias_writes_fragments says so, else KUTACC_HIP_EINVAL
int pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
              int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int32_t dtype, int transposed,
              hipStream_t stream, void *fragments = nullptr, int frag_nb = 0, int frag_nt = 0, int frag_tiles = 0);
bool pair_bias_writes_fragments(const void *z, const void *w, const void *z_norm, int64_t rows_i, int64_t rows_j, int64_t c_z,
                                int64_t nheads, int32_t dtype);

} // namespace kutacc_launch
