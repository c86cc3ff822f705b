// A caller of libkutacc.so written the way the reference's own consumers are (reference
// test/functest/cal/gating_attention_test.cpp:18-264 and the external PyTorch extension its header mentions): a C++
// translation unit that includes kutacc.h, wraps raw pointers in kutacc::TensorWrapper through the
// std::vector<int64_t>&& constructor, fills the two POD argument structs and calls kutacc_af2_gating_attention.
// It is compiled twice from this one file -- against the reference's include/kutacc.h and against this repository's --
// and each build is loaded into the test process, which proves that a program compiled with the Kunpeng header links
// and runs against this library unchanged.  Test infrastructure only.
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <vector>

#include "kutacc.h"

// Struct layouts of the interface, as this repository's header declares them (LP64).  Compiled against the reference
// header these assertions check that both headers describe the same memory.
static_assert(sizeof(kutacc_version_t) == 48 && offsetof(kutacc_version_t, component_appendinfo) == 40, "kutacc_version_t");
static_assert(sizeof(kutacc_af2_attention_weights_t) == 80 && offsetof(kutacc_af2_attention_weights_t, nheads) == 8 &&
                  offsetof(kutacc_af2_attention_weights_t, head_size) == 16 && offsetof(kutacc_af2_attention_weights_t, query_w) == 24 &&
                  offsetof(kutacc_af2_attention_weights_t, key_w) == 32 && offsetof(kutacc_af2_attention_weights_t, value_w) == 40 &&
                  offsetof(kutacc_af2_attention_weights_t, gating_w) == 48 && offsetof(kutacc_af2_attention_weights_t, gating_b) == 56 &&
                  offsetof(kutacc_af2_attention_weights_t, output_w) == 64 && offsetof(kutacc_af2_attention_weights_t, output_b) == 72,
              "kutacc_af2_attention_weights_t");
static_assert(sizeof(kutacc_af2_attention_inputs_t) == 56 && offsetof(kutacc_af2_attention_inputs_t, seq_len) == 8 &&
                  offsetof(kutacc_af2_attention_inputs_t, q) == 16 && offsetof(kutacc_af2_attention_inputs_t, k) == 24 &&
                  offsetof(kutacc_af2_attention_inputs_t, v) == 32 && offsetof(kutacc_af2_attention_inputs_t, gate) == 40 &&
                  offsetof(kutacc_af2_attention_inputs_t, avg) == 48,
              "kutacc_af2_attention_inputs_t");
static_assert(sizeof(kutacc_af2_tm_proj_weights_t) == 48 && offsetof(kutacc_af2_tm_proj_weights_t, c_i) == 8 &&
                  offsetof(kutacc_af2_tm_proj_weights_t, proj_w) == 16 && offsetof(kutacc_af2_tm_proj_weights_t, proj_b) == 24 &&
                  offsetof(kutacc_af2_tm_proj_weights_t, gate_w) == 32 && offsetof(kutacc_af2_tm_proj_weights_t, gate_b) == 40,
              "kutacc_af2_tm_proj_weights_t");
static_assert(sizeof(kutacc_af2_tm_act_inputs_t) == 40 && offsetof(kutacc_af2_tm_act_inputs_t, n_res_gather) == 8 &&
                  offsetof(kutacc_af2_tm_act_inputs_t, proj_act) == 16 && offsetof(kutacc_af2_tm_act_inputs_t, input_act) == 24 &&
                  offsetof(kutacc_af2_tm_act_inputs_t, proj_act_gate) == 32,
              "kutacc_af2_tm_act_inputs_t");
static_assert(sizeof(kutacc_af2_tm_linear_weights_t) == 48 && offsetof(kutacc_af2_tm_linear_weights_t, c_i) == 8 &&
                  offsetof(kutacc_af2_tm_linear_weights_t, gating_w) == 16 && offsetof(kutacc_af2_tm_linear_weights_t, gating_b) == 24 &&
                  offsetof(kutacc_af2_tm_linear_weights_t, output_proj_w) == 32 &&
                  offsetof(kutacc_af2_tm_linear_weights_t, output_proj_b) == 40,
              "kutacc_af2_tm_linear_weights_t");
static_assert(sizeof(kutacc_af2_trans_weights_t) == 48 && offsetof(kutacc_af2_trans_weights_t, c_i) == 8 &&
                  offsetof(kutacc_af2_trans_weights_t, linear1_w) == 16 && offsetof(kutacc_af2_trans_weights_t, linear1_b) == 24 &&
                  offsetof(kutacc_af2_trans_weights_t, linear2_w) == 32 && offsetof(kutacc_af2_trans_weights_t, linear2_b) == 40,
              "kutacc_af2_trans_weights_t");
static_assert(sizeof(kutacc_af2_trans_act_inputs_t) == 32 && offsetof(kutacc_af2_trans_act_inputs_t, n_res) == 8 &&
                  offsetof(kutacc_af2_trans_act_inputs_t, input_act) == 16 &&
                  offsetof(kutacc_af2_trans_act_inputs_t, intermediate_act) == 24,
              "kutacc_af2_trans_act_inputs_t");
static_assert(sizeof(kutacc::TensorWrapper) == sizeof(void *), "TensorWrapper holds exactly one handle");
static_assert((int)kutacc::kInt64 == 0 && (int)kutacc::kBF16 == 1, "DType values");
static_assert(sizeof(kutacc::BlasExtendParams) == 32 && offsetof(kutacc::BlasExtendParams, bias) == 16, "BlasExtendParams");
static_assert(KUTACC_OK == 0 && KUTACC_ERROR == -1, "status codes");

namespace {
using kutacc::TensorWrapper;

std::vector<int64_t> dims(std::initializer_list<int64_t> v) { return std::vector<int64_t>(v); }
} // namespace

extern "C" {

// sizeof of every interface struct followed by the offset of its last member, for comparing the two builds at run time
__attribute__((visibility("default"))) int dropin_layout(int64_t *out, int cap)
{
    const int64_t v[] = {
        (int64_t)sizeof(kutacc_version_t), (int64_t)offsetof(kutacc_version_t, component_appendinfo),
        (int64_t)sizeof(kutacc_af2_attention_weights_t), (int64_t)offsetof(kutacc_af2_attention_weights_t, output_b),
        (int64_t)sizeof(kutacc_af2_attention_inputs_t), (int64_t)offsetof(kutacc_af2_attention_inputs_t, avg),
        (int64_t)sizeof(kutacc_af2_tm_proj_weights_t), (int64_t)offsetof(kutacc_af2_tm_proj_weights_t, gate_b),
        (int64_t)sizeof(kutacc_af2_tm_act_inputs_t), (int64_t)offsetof(kutacc_af2_tm_act_inputs_t, proj_act_gate),
        (int64_t)sizeof(kutacc_af2_tm_linear_weights_t), (int64_t)offsetof(kutacc_af2_tm_linear_weights_t, output_proj_b),
        (int64_t)sizeof(kutacc_af2_trans_weights_t), (int64_t)offsetof(kutacc_af2_trans_weights_t, linear2_b),
        (int64_t)sizeof(kutacc_af2_trans_act_inputs_t), (int64_t)offsetof(kutacc_af2_trans_act_inputs_t, intermediate_act),
        (int64_t)sizeof(kutacc::TensorWrapper), (int64_t)sizeof(kutacc::BlasExtendParams), (int64_t)kutacc::kBF16,
    };
    const int n = (int)(sizeof(v) / sizeof(v[0]));
    for (int i = 0; i < n && i < cap; ++i) {
        out[i] = v[i];
    }
    return n;
}

// The seven argument-validation cases the reference's tests hold for this operator: `which` = 1..6 passes a null pointer
// as the which-th pointer argument (input, q_based_ptr, bias, nonbatched_bias, weight_ptr, out), 7 a negative block_size;
// every other handle is, as there, the address of some float -- not a tensor -- so the library must reject the call before
// it looks inside any handle.  Returns 0 when the call came back.
__attribute__((visibility("default"))) int dropin_validation_case(int which)
{
    float one = 1.5f;
    float grid[2][2][2] = {{{1.f, 2.f}, {3.f, 4.f}}, {{7.f, 8.f}, {9.f, 10.f}}};
    void *h = &one, *x = &grid;
    kutacc_af2_attention_weights_t weights = {2, 1, 2, x, x, x, x, x, x, x};
    kutacc_af2_attention_inputs_t inputs = {2, 2, x, x, x, x, x};
    if (which < 1 || which > 7) {
        return -1;
    }
    kutacc_af2_gating_attention(which == 1 ? nullptr : h, which == 2 ? nullptr : &inputs, which == 3 ? nullptr : h,
                                which == 4 ? nullptr : (which == 7 ? x : h), which == 5 ? nullptr : &weights,
                                which == 6 ? nullptr : h, which == 7 ? -5 : 5);
    return 0;
}

// kutacc_get_version through the header's struct
__attribute__((visibility("default"))) const char *dropin_component_name()
{
    static kutacc_version_t v;
    return kutacc_get_version(&v) == KUTACC_OK ? v.component_name : nullptr;
}

// One real call on the caller's memory (bf16 storage, fp32 biases), tensors described exactly as the reference's
// operator reads them (reference src/attention/gating_attention.cpp:47-66, 90, 103-106, 156): q, k, gate, avg
// [batch, seq_len, nheads, head_size]; v [nheads, head_size, batch, seq_len]; bias [batch, 1, 1, seq_len];
// nonbatched_bias [nheads, seq_len, seq_len], or a tensor whose first size is 0 when there is none.
__attribute__((visibility("default"))) int dropin_gating_attention(void *input, void *q, void *k, void *v, void *gate, void *avg,
                                                                  void *bias, void *nonbatched_bias, void *query_w, void *key_w,
                                                                  void *value_w, void *gating_w, void *gating_b, void *output_w,
                                                                  void *output_b, void *out, int64_t batch, int64_t seq_len,
                                                                  int64_t nheads, int64_t head_size, int64_t block_size)
{
    const int64_t B = batch, S = seq_len, H = nheads, d = head_size, C = H * d;
    const kutacc::DType bf16 = kutacc::kBF16;
    TensorWrapper t_in(input, dims({B, S, C}), dims({S * C, C, 1}), 3, bf16);
    TensorWrapper t_q(q, dims({B, S, H, d}), dims({S * C, C, d, 1}), 4, bf16);
    TensorWrapper t_k(k, dims({B, S, H, d}), dims({S * C, C, d, 1}), 4, bf16);
    TensorWrapper t_v(v, dims({H, d, B, S}), dims({d * B * S, B * S, S, 1}), 4, bf16);
    TensorWrapper t_gate(gate, dims({B, S, H, d}), dims({S * C, C, d, 1}), 4, bf16);
    TensorWrapper t_avg(avg, dims({B, S, H, d}), dims({S * C, C, d, 1}), 4, bf16);
    TensorWrapper t_bias(bias, dims({B, 1, 1, S}), dims({S, S, S, 1}), 4, bf16);
    TensorWrapper t_nb(nonbatched_bias, nonbatched_bias ? dims({H, S, S}) : dims({0}),
                       nonbatched_bias ? dims({S * S, S, 1}) : dims({1}), nonbatched_bias ? 3 : 1, bf16);
    TensorWrapper t_wq(query_w, dims({C, C}), dims({C, 1}), 2, bf16), t_wk(key_w, dims({C, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_wv(value_w, dims({C, C}), dims({C, 1}), 2, bf16), t_wg(gating_w, dims({C, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_wo(output_w, dims({C, C}), dims({C, 1}), 2, bf16);
    // the reference's DType has no fp32 tag; its bias handles carry the pointer only
    TensorWrapper t_bg(gating_b, dims({C}), dims({1}), 1, bf16), t_bo(output_b, dims({C}), dims({1}), 1, bf16);
    TensorWrapper t_out(out, dims({B, S, C}), dims({S * C, C, 1}), 3, bf16);

    kutacc_af2_attention_weights_t weights = {C,
                                              H,
                                              d,
                                              t_wq.get_tensor(),
                                              t_wk.get_tensor(),
                                              t_wv.get_tensor(),
                                              t_wg.get_tensor(),
                                              t_bg.get_tensor(),
                                              t_wo.get_tensor(),
                                              t_bo.get_tensor()};
    kutacc_af2_attention_inputs_t inputs = {B,
                                            S,
                                            t_q.get_tensor(),
                                            t_k.get_tensor(),
                                            t_v.get_tensor(),
                                            t_gate.get_tensor(),
                                            t_avg.get_tensor()};
    kutacc_af2_gating_attention(t_in.get_tensor(), &inputs, t_bias.get_tensor(), t_nb.get_tensor(), &weights, t_out.get_tensor(),
                                block_size);
    // a default-constructed wrapper, as a caller holds before it has a tensor: must construct and destruct cleanly
    TensorWrapper unset;
    return unset.get_tensor() == nullptr ? 0 : 1;
}

// kutacc_af2_global_attention on the caller's memory, tensors described as the reference's operator reads them (reference
// src/attention/global_attention.cpp:30-164, include/kutacc.h:292-307): q_data [batch, seq_len, 64], q_mask
// [batch, seq_len, 1], query/gating/output weights [64, 64], key/value weights [head_size, 64], scratch q and avg
// [batch, 64], k [batch*seq_len, head_size], v [head_size, batch*seq_len], gate [batch, seq_len, 64].
__attribute__((visibility("default"))) int dropin_global_attention(void *q_data, void *q_mask, void *q, void *k, void *v,
                                                                  void *gate, void *avg, void *query_w, void *key_w,
                                                                  void *value_w, void *gating_w, void *gating_b, void *output_w,
                                                                  void *output_b, void *out, int64_t batch, int64_t seq_len,
                                                                  int64_t nheads, int64_t head_size)
{
    const int64_t B = batch, S = seq_len, H = nheads, d = head_size, C = H * d;
    const kutacc::DType bf16 = kutacc::kBF16;
    TensorWrapper t_x(q_data, dims({B, S, C}), dims({S * C, C, 1}), 3, bf16);
    TensorWrapper t_mask(q_mask, dims({B, S, 1}), dims({S, 1, 1}), 3, bf16);
    TensorWrapper t_q(q, dims({B, C}), dims({C, 1}), 2, bf16), t_avg(avg, dims({B, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_k(k, dims({B * S, d}), dims({d, 1}), 2, bf16), t_v(v, dims({d, B * S}), dims({B * S, 1}), 2, bf16);
    TensorWrapper t_gate(gate, dims({B, S, C}), dims({S * C, C, 1}), 3, bf16);
    TensorWrapper t_wq(query_w, dims({C, C}), dims({C, 1}), 2, bf16), t_wk(key_w, dims({d, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_wv(value_w, dims({d, C}), dims({C, 1}), 2, bf16), t_wg(gating_w, dims({C, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_wo(output_w, dims({C, C}), dims({C, 1}), 2, bf16);
    TensorWrapper t_bg(gating_b, dims({C}), dims({1}), 1, bf16), t_bo(output_b, dims({C}), dims({1}), 1, bf16);
    TensorWrapper t_out(out, dims({B, S, C}), dims({S * C, C, 1}), 3, bf16);
    kutacc_af2_attention_weights_t weights = {C,
                                              H,
                                              d,
                                              t_wq.get_tensor(),
                                              t_wk.get_tensor(),
                                              t_wv.get_tensor(),
                                              t_wg.get_tensor(),
                                              t_bg.get_tensor(),
                                              t_wo.get_tensor(),
                                              t_bo.get_tensor()};
    kutacc_af2_attention_inputs_t inputs = {B,
                                            S,
                                            t_q.get_tensor(),
                                            t_k.get_tensor(),
                                            t_v.get_tensor(),
                                            t_gate.get_tensor(),
                                            t_avg.get_tensor()};
    kutacc_af2_global_attention(&inputs, t_x.get_tensor(), t_mask.get_tensor(), &weights, t_out.get_tensor());
    return 0;
}

// kutacc_af2_transition on the caller's memory (reference src/attention/transition.cpp:21-67, include/kutacc.h:194-214,
// 321-322): input_act and out [batch, n_res, c_o], linear1_w [c_i, c_o], linear2_w [c_o, c_i], fp32 biases,
// intermediate_act [batch*n_res, c_i].
__attribute__((visibility("default"))) int dropin_transition(void *input_act, void *intermediate_act, void *linear1_w,
                                                            void *linear1_b, void *linear2_w, void *linear2_b, void *out,
                                                            int64_t batch, int64_t n_res, int64_t c_o, int64_t c_i)
{
    const kutacc::DType bf16 = kutacc::kBF16;
    TensorWrapper t_x(input_act, dims({batch, n_res, c_o}), dims({n_res * c_o, c_o, 1}), 3, bf16);
    TensorWrapper t_mid(intermediate_act, dims({batch * n_res, c_i}), dims({c_i, 1}), 2, bf16);
    TensorWrapper t_w1(linear1_w, dims({c_i, c_o}), dims({c_o, 1}), 2, bf16), t_w2(linear2_w, dims({c_o, c_i}), dims({c_i, 1}), 2, bf16);
    TensorWrapper t_b1(linear1_b, dims({c_i}), dims({1}), 1, bf16), t_b2(linear2_b, dims({c_o}), dims({1}), 1, bf16);
    TensorWrapper t_out(out, dims({batch, n_res, c_o}), dims({n_res * c_o, c_o, 1}), 3, bf16);
    kutacc_af2_trans_act_inputs_t inputs = {batch, n_res, t_x.get_tensor(), t_mid.get_tensor()};
    kutacc_af2_trans_weights_t weights = {c_o, c_i, t_w1.get_tensor(), t_b1.get_tensor(), t_w2.get_tensor(), t_b2.get_tensor()};
    kutacc_af2_transition(&inputs, &weights, t_out.get_tensor());
    return 0;
}

// kutacc_af2_linear_weight_prepack through the header's prototype, default argument included
__attribute__((visibility("default"))) void dropin_prepack(const void *weight, void *result, int64_t n, int64_t k, int64_t ldb)
{
    kutacc_af2_linear_weight_prepack((const __bf16 *)weight, (__bf16 *)result, n, k, ldb);
}

} // extern "C"
