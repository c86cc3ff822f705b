// Handle-based entry points of the transition and the triangle multiplication, and the extern "C"
// launch layer under them.  Check order and messages follow reference src/attention/transition.cpp:21-67
// and src/attention/triangle_multiplication.cpp:25-240: pointer checks in the entry, then the scalar
// checks of the kernel function, both before any tensor handle is looked into; after that the operand
// checks of addmm (reference src/linear/mm.cpp:23-35,80-82: bf16 dtype, non-null data).
//
// Every step is one or two launches of the strided bf16 GEMM of pair_stack.hip; the views below are
// the ones the reference builds for its addmm calls.  Device pointers run in place; host pointers (the reference's
// callers pass host tensors) are mirrored on the device for the call and the results copied back -- all operands of a
// call must live on the same side.
#include <hip/hip_runtime.h>

#include <climits>
#include <cstring>
#include <initializer_list>
#include <string>

#include "api_internal.h"
#include "check.h"
#include "kutacc.h"
#include "kutacc_hip.h"
#include "launch_internal.h"
#include "staging.h"
#include "tensor_view.h"

namespace {
using kutacc::TensorView;

bool handles_present(const char *who, std::initializer_list<kutacc_tensor_h> handles)
{
    for (kutacc_tensor_h h : handles) {
        KUTACC_CHECK(h != nullptr, who, ": tensor handle inside argument struct is null");
    }
    return !KUTACC_FAILED();
}

// the operand checks of addmm, plus the memory-space rule of these operators: all on the device or all on the host
bool operands_ok(const char *who, std::initializer_list<const TensorView *> bf16_views,
                 std::initializer_list<const TensorView *> fp32_views, bool *on_host)
{
    for (const TensorView *v : bf16_views) {
        KUTACC_CHECK(v->dtype == kutacc::kBF16, "addmm dtype invalid, a: [", (int)v->dtype, "]");
        KUTACC_CHECK(v->data != nullptr, "addmm input invalid");
    }
    for (const TensorView *v : fp32_views) {
        KUTACC_CHECK(v->data != nullptr, "addmm input invalid");
    }
    if (KUTACC_FAILED()) {
        return false;
    }
    const bool device = kutacc_api::on_device((*bf16_views.begin())->data);
    for (const TensorView *v : bf16_views) {
        KUTACC_CHECK(kutacc_api::on_device(v->data) == device, who, ": host and device pointers mixed in one call");
    }
    for (const TensorView *v : fp32_views) {
        KUTACC_CHECK(kutacc_api::on_device(v->data) == device, who, ": host and device pointers mixed in one call");
    }
    *on_host = !device;
    return !KUTACC_FAILED();
}

// Operands of one call.  Device pointers pass through; host ranges get a device mirror (uploaded for inputs, copied
// back for outputs; `preload` uploads an output first, for ranges the kernels only partly overwrite).
struct Operands {
    bool host;
    hipStream_t stream;
    kutacc_api::Stager st;
    Operands(bool on_host, hipStream_t s) : host(on_host), stream(s), st(s) {}
    const void *in(const void *p, size_t elems, size_t elem_bytes = 2) { return host ? st.in(p, elems * elem_bytes) : p; }
    const float *in_f32(const void *p, size_t elems) { return (const float *)in(p, elems, sizeof(float)); }
    void *out(void *p, size_t elems, bool preload) { return host ? st.out(p, elems * 2, preload) : p; }
    void *scratch(void *p, size_t elems) { return host ? st.scratch(elems * 2) : p; }
    bool ready() const { return !host || st.rc == 0; }
    // ends the call: blocking-mode synchronisation on the device side, copy-back and release on the host side
    int finish(int rc)
    {
        if (!host) {
            return kutacc_api::finish(rc, stream);
        }
        if (rc == 0) {
            rc = st.rc;
        }
        const int rc2 = st.finish();
        return rc != 0 ? rc : rc2;
    }
};

// highest element offset of a [n0, n1, n2] access with unit inner stride, plus one
inline size_t span3(int64_t n0, int64_t s0, int64_t n1, int64_t s1, int64_t n2)
{
    return (size_t)((n0 - 1) * s0 + (n1 - 1) * s1 + n2);
}

void report(const char *who, int rc)
{
    KUTACC_CHECK(rc == 0, who, ": launch layer returned ", rc,
                 rc > 0 ? std::string(" (") + hipGetErrorString((hipError_t)rc) + ")" : std::string());
}

kutacc_hip_gemm_args_t blank_gemm()
{
    kutacc_hip_gemm_args_t g;
    std::memset(&g, 0, sizeof(g));
    g.dtype = KUTACC_DTYPE_BF16;
    g.path = KUTACC_HIP_PATH_AUTO;
    g.batches = 1;
    return g;
}
} // namespace

extern "C" {

int kutacc_hip_gemm(const kutacc_hip_gemm_args_t *args, void *stream)
{
    if (args == nullptr) {
        return KUTACC_HIP_EINVAL;
    }
    return kutacc_launch::pair_gemm(*args, kutacc_api::stream_or_default(stream));
}

int kutacc_hip_sigmoid_gate_rows(void *out, int64_t out_stride0, int64_t out_stride1, const void *gate,
                                 int64_t gate_stride0, int64_t gate_stride1, int64_t n0, int64_t n1, int64_t size,
                                 int32_t dtype, void *stream)
{
    if (dtype != KUTACC_DTYPE_BF16) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    return kutacc_launch::sigmoid_gate_rows(out, out_stride0, out_stride1, gate, gate_stride0, gate_stride1, n0, n1, size,
                                            kutacc_api::stream_or_default(stream));
}

int kutacc_hip_transition(const void *x, const void *w1, const float *b1, const void *w2, const float *b2, void *intermediate,
                          void *out, int64_t rows, int64_t c_o, int64_t c_i, int32_t dtype, int32_t path, void *stream)
{
    if (!x || !w1 || !b1 || !w2 || !b2 || !out || rows <= 0 || c_o <= 0 || c_i <= 0 || dtype != KUTACC_DTYPE_BF16) {
        return KUTACC_HIP_EINVAL;
    }
    hipStream_t s = kutacc_api::stream_or_default(stream);
    const bool fused_ok = kutacc_launch::transition_fused_supports(rows, c_o, c_i, x, w1, b1, w2, b2, out);
    if (path == KUTACC_HIP_PATH_FUSED && !fused_ok) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    if (path != KUTACC_HIP_PATH_GENERIC && fused_ok) {
        return kutacc_launch::transition_fused(x, w1, b1, w2, b2, out, rows, c_o, c_i, s);
    }
    if (!intermediate) {
        return KUTACC_HIP_EINVAL;
    }
    kutacc_hip_gemm_args_t g = blank_gemm();
    g.m = rows, g.n = c_i, g.k = c_o;
    g.a = x, g.a_stride_m = c_o, g.a_stride_k = 1;
    g.b = w1, g.b_stride_n = c_o, g.b_stride_k = 1;
    g.c = intermediate, g.c_stride_m = c_i;
    g.bias = b1, g.bias_axis = 1, g.relu = 1;
    int rc = kutacc_launch::pair_gemm(g, s);
    if (rc != 0) {
        return rc;
    }
    g = blank_gemm();
    g.m = rows, g.n = c_o, g.k = c_i;
    g.a = intermediate, g.a_stride_m = c_i, g.a_stride_k = 1;
    g.b = w2, g.b_stride_n = c_i, g.b_stride_k = 1;
    g.c = out, g.c_stride_m = c_o;
    g.bias = b2, g.bias_axis = 1;
    return kutacc_launch::pair_gemm(g, s);
}

void kutacc_af2_transition(kutacc_af2_trans_act_inputs_t *trans_inputs_ptr, kutacc_af2_trans_weights_t *trans_weights_ptr,
                           kutacc_tensor_h out)
{
    KUTACC_CHECK(trans_inputs_ptr != nullptr && trans_weights_ptr != nullptr && out != nullptr,
                 "af2_transition: input args nullptr error\n");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t batch = trans_inputs_ptr->batch, n_res = trans_inputs_ptr->n_res;
    const int64_t c_o = trans_weights_ptr->c_o, c_i = trans_weights_ptr->c_i;
    KUTACC_CHECK(batch > 0 && n_res > 0 && c_o > 0 && c_i > 0 && batch <= INT64_MAX / n_res && c_o <= INT32_MAX &&
                     c_i <= INT32_MAX,
                 "input param <= 0 or overflow");
    if (KUTACC_FAILED()) {
        return;
    }
    if (!handles_present("kutacc_af2_transition",
                         {trans_inputs_ptr->input_act, trans_inputs_ptr->intermediate_act, trans_weights_ptr->linear1_w,
                          trans_weights_ptr->linear1_b, trans_weights_ptr->linear2_w, trans_weights_ptr->linear2_b})) {
        return;
    }
    const TensorView &x = *kutacc::as_view(trans_inputs_ptr->input_act), &mid = *kutacc::as_view(trans_inputs_ptr->intermediate_act),
                     &w1 = *kutacc::as_view(trans_weights_ptr->linear1_w), &b1 = *kutacc::as_view(trans_weights_ptr->linear1_b),
                     &w2 = *kutacc::as_view(trans_weights_ptr->linear2_w), &b2 = *kutacc::as_view(trans_weights_ptr->linear2_b),
                     &o = *kutacc::as_view(out);
    bool on_host = false;
    if (!operands_ok("kutacc_af2_transition", {&x, &mid, &w1, &w2, &o}, {&b1, &b2}, &on_host)) {
        return;
    }
    hipStream_t s = kutacc_api::default_stream();
    Operands ops(on_host, s);
    // the reference's views: every tensor dense with its channel count as the row stride (transition.cpp:31-38)
    const int64_t rows = batch * n_res;
    const void *xd = ops.in(x.data, (size_t)(rows * c_o)), *w1d = ops.in(w1.data, (size_t)(c_i * c_o)),
               *w2d = ops.in(w2.data, (size_t)(c_o * c_i));
    const float *b1d = ops.in_f32(b1.data, (size_t)c_i), *b2d = ops.in_f32(b2.data, (size_t)c_o);
    void *midd = ops.scratch(mid.data, (size_t)(rows * c_i)), *od = ops.out(o.data, (size_t)(rows * c_o), false);
    int rc = 0;
    if (ops.ready()) {
        rc = kutacc_hip_transition(xd, w1d, b1d, w2d, b2d, midd, od, rows, c_o, c_i, KUTACC_DTYPE_BF16, KUTACC_HIP_PATH_AUTO, s);
    }
    report("kutacc_af2_transition", ops.finish(rc));
}

void kutacc_af2_triangle_multiplication_calc_proj(kutacc_af2_tm_act_inputs_t *tm_acts_ptr, kutacc_tensor_h mask,
                                                  kutacc_af2_tm_proj_weights_t *tm_weights_ptr, bool input_prepack)
{
    (void)input_prepack; // operand layout hint of the CPU GEMM; operands are plain row-major here
    KUTACC_CHECK(tm_acts_ptr != nullptr && mask != nullptr && tm_weights_ptr != nullptr,
                 "kutacc_af2_triangle_multiplication_calc_proj: input args nullptr error\n");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t n_res = tm_acts_ptr->n_res, n_res_gather = tm_acts_ptr->n_res_gather;
    const int64_t c_o = tm_weights_ptr->c_o, c_i = tm_weights_ptr->c_i;
    KUTACC_CHECK(n_res > 0 && n_res_gather > 0 && c_o > 0 && c_i > 0 && n_res <= INT64_MAX / n_res_gather &&
                     n_res <= INT64_MAX / c_i && c_o <= INT32_MAX,
                 "input param <= 0 or overflow");
    if (KUTACC_FAILED()) {
        return;
    }
    if (!handles_present("kutacc_af2_triangle_multiplication_calc_proj",
                         {tm_acts_ptr->proj_act, tm_acts_ptr->input_act, tm_weights_ptr->proj_w, tm_weights_ptr->proj_b,
                          tm_weights_ptr->gate_w, tm_weights_ptr->gate_b})) {
        return;
    }
    const TensorView &pa = *kutacc::as_view(tm_acts_ptr->proj_act), &x = *kutacc::as_view(tm_acts_ptr->input_act),
                     &mk = *kutacc::as_view(mask), &pw = *kutacc::as_view(tm_weights_ptr->proj_w),
                     &pb = *kutacc::as_view(tm_weights_ptr->proj_b), &gw = *kutacc::as_view(tm_weights_ptr->gate_w),
                     &gb = *kutacc::as_view(tm_weights_ptr->gate_b);
    bool on_host = false;
    if (!operands_ok("kutacc_af2_triangle_multiplication_calc_proj", {&pa, &x, &mk, &pw, &gw}, {&pb, &gb}, &on_host)) {
        return;
    }
    KUTACC_CHECK(pa.dim >= 2 && mk.dim >= 1, "kutacc_af2_triangle_multiplication_calc_proj: proj_act needs rank >= 2, mask rank >= 1");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = kutacc_api::default_stream();
    // proj_act^T = proj_w . input_act^T with a per-row (channel) bias: the reference's first two addmm calls
    // (triangle_multiplication.cpp:37-45), and its element-wise pass (:47-66) as the epilogue
    Operands ops(on_host, s);
    const int64_t pa_s1 = pa.dim >= 3 ? pa.stride(1) : n_res_gather;
    const size_t pa_span = span3(c_i, pa.stride(0), n_res, pa_s1, n_res_gather);
    kutacc_hip_gemm_args_t g = blank_gemm();
    g.m = c_i, g.k = c_o;
    g.a = ops.in(pw.data, (size_t)(c_i * c_o)), g.a_gate = ops.in(gw.data, (size_t)(c_i * c_o)), g.a_stride_m = c_o, g.a_stride_k = 1;
    g.b = ops.in(x.data, (size_t)(n_res * n_res_gather * c_o)), g.b_stride_n = c_o, g.b_stride_k = 1;
    g.c = ops.out(pa.data, pa_span, pa_span != (size_t)(c_i * n_res * n_res_gather)), g.c_stride_m = pa.stride(0);
    g.bias = ops.in_f32(pb.data, (size_t)c_i), g.bias_gate = ops.in_f32(gb.data, (size_t)c_i), g.bias_axis = 2;
    g.mask = ops.in(mk.data, (size_t)((n_res - 1) * mk.stride(0) + n_res_gather));
    if (pa_s1 == n_res_gather && mk.stride(0) == n_res_gather) {
        g.n = n_res * n_res_gather; // rows (i, j) of the pair tensor are one flat, dense index
    } else {
        g.n = n_res_gather, g.batches = n_res;
        g.b_stride_batch = n_res_gather * c_o, g.c_stride_batch = pa_s1, g.mask_stride_batch = mk.stride(0);
    }
    report("kutacc_af2_triangle_multiplication_calc_proj", ops.finish(ops.ready() ? kutacc_launch::pair_gemm(g, s) : 0));
}

void kutacc_af2_triangle_multiplication_equation(kutacc_tensor_h center_act, kutacc_tensor_h left_proj_act,
                                                 kutacc_tensor_h right_proj_act, int64_t n_res_gather, bool is_incoming)
{
    KUTACC_CHECK(center_act != nullptr && left_proj_act != nullptr && right_proj_act != nullptr,
                 "kutacc_af2_triangle_multiplication_equation: input args nullptr error\n");
    KUTACC_CHECK(n_res_gather > 0, "kutacc_af2_triangle_multiplication_equation: input args int values error, values "
                                   "are less than or equal to zero\n");
    if (KUTACC_FAILED()) {
        return;
    }
    const TensorView &ce = *kutacc::as_view(center_act), &le = *kutacc::as_view(left_proj_act),
                     &ri = *kutacc::as_view(right_proj_act);
    bool on_host = false;
    if (!operands_ok("kutacc_af2_triangle_multiplication_equation", {&ce, &le, &ri}, {}, &on_host)) {
        return;
    }
    KUTACC_CHECK(ce.dim >= 2 && le.dim >= 2 && ri.dim >= 2 && le.size(0) > 0,
                 "kutacc_af2_triangle_multiplication_equation: tensors need rank >= 2 and at least one channel");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = kutacc_api::default_stream();
    kutacc_hip_gemm_args_t g = blank_gemm();
    g.m = g.n = g.k = n_res_gather;
    g.batches = le.size(0); // one product per channel (triangle_multiplication.cpp:74)
    Operands ops(on_host, s);
    const int64_t nch = le.size(0), n = n_res_gather;
    const void *led = ops.in(le.data, span3(nch, le.stride(0), n, le.stride(1), n)),
               *rid = ops.in(ri.data, span3(nch, ri.stride(0), n, ri.stride(1), n));
    const size_t ce_span = span3(nch, ce.stride(0), n, ce.stride(1), n);
    if (!is_incoming) {
        // center[i, j] = sum_k left[i, k] * right[j, k]  (:77-86)
        g.a = led, g.a_stride_m = le.stride(1), g.a_stride_k = 1, g.a_stride_batch = le.stride(0);
        g.b = rid, g.b_stride_n = ri.stride(1), g.b_stride_k = 1, g.b_stride_batch = ri.stride(0);
    } else {
        // center[i, j] = sum_k right[k, i] * left[k, j]  (:88-97)
        g.a = rid, g.a_stride_m = 1, g.a_stride_k = ri.stride(1), g.a_stride_batch = ri.stride(0);
        g.b = led, g.b_stride_n = 1, g.b_stride_k = le.stride(1), g.b_stride_batch = le.stride(0);
    }
    g.c = ops.out(ce.data, ce_span, ce_span != (size_t)(nch * n * n)), g.c_stride_m = ce.stride(1), g.c_stride_batch = ce.stride(0);
    report("kutacc_af2_triangle_multiplication_equation", ops.finish(ops.ready() ? kutacc_launch::pair_gemm(g, s) : 0));
}

void kutacc_af2_triangle_multiplication_gate_and_out_linear(kutacc_tensor_h gate, kutacc_tensor_h out,
                                                            kutacc_af2_tm_act_inputs_t *tm_acts_ptr,
                                                            kutacc_tensor_h center_act,
                                                            kutacc_af2_tm_linear_weights_t *tm_weights_ptr,
                                                            bool input_prepack)
{
    (void)input_prepack;
    KUTACC_CHECK(gate != nullptr && out != nullptr && tm_acts_ptr != nullptr && center_act != nullptr &&
                     tm_weights_ptr != nullptr,
                 "kutacc_af2_triangle_multiplication_gate_and_out_linear: input args nullptr error\n");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t n_res = tm_acts_ptr->n_res, n_res_gather = tm_acts_ptr->n_res_gather;
    const int64_t c_o = tm_weights_ptr->c_o, c_i = tm_weights_ptr->c_i;
    KUTACC_CHECK(n_res > 0 && n_res_gather > 0 && c_o > 0 && c_i > 0 && n_res <= INT64_MAX / n_res_gather &&
                     c_o <= INT32_MAX && c_i <= INT32_MAX,
                 "input param <= 0 or overflow");
    if (KUTACC_FAILED()) {
        return;
    }
    if (!handles_present("kutacc_af2_triangle_multiplication_gate_and_out_linear",
                         {tm_acts_ptr->input_act, tm_weights_ptr->gating_w, tm_weights_ptr->gating_b,
                          tm_weights_ptr->output_proj_w, tm_weights_ptr->output_proj_b})) {
        return;
    }
    const TensorView &gt = *kutacc::as_view(gate), &o = *kutacc::as_view(out), &x = *kutacc::as_view(tm_acts_ptr->input_act),
                     &ce = *kutacc::as_view(center_act), &gw = *kutacc::as_view(tm_weights_ptr->gating_w),
                     &gb = *kutacc::as_view(tm_weights_ptr->gating_b), &ow = *kutacc::as_view(tm_weights_ptr->output_proj_w),
                     &ob = *kutacc::as_view(tm_weights_ptr->output_proj_b);
    bool on_host = false;
    if (!operands_ok("kutacc_af2_triangle_multiplication_gate_and_out_linear", {&gt, &o, &x, &ce, &gw, &ow}, {&gb, &ob},
                     &on_host)) {
        return;
    }
    KUTACC_CHECK(gt.dim >= 2 && o.dim >= 2 && ce.dim >= 2,
                 "kutacc_af2_triangle_multiplication_gate_and_out_linear: gate, out and center_act need rank >= 2");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = kutacc_api::default_stream();
    const int64_t rows = n_res * n_res_gather;
    Operands ops(on_host, s);
    const size_t gt_span = (size_t)((rows - 1) * gt.stride(1) + c_o), o_span = (size_t)((rows - 1) * o.stride(1) + c_o);
    // gate = input_act . gating_w^T + gating_b  (triangle_multiplication.cpp:115-119)
    kutacc_hip_gemm_args_t g = blank_gemm();
    g.m = rows, g.n = c_o, g.k = c_o;
    g.a = ops.in(x.data, (size_t)(rows * c_o)), g.a_stride_m = c_o, g.a_stride_k = 1;
    g.b = ops.in(gw.data, (size_t)(c_o * c_o)), g.b_stride_n = c_o, g.b_stride_k = 1;
    g.c = ops.out(gt.data, gt_span, gt_span != (size_t)(rows * c_o)), g.c_stride_m = gt.stride(1);
    g.bias = ops.in_f32(gb.data, (size_t)c_o), g.bias_axis = 1;
    // out = center_act . output_proj_w^T + output_proj_b  (:121-126)
    kutacc_hip_gemm_args_t g2 = blank_gemm();
    g2.m = rows, g2.n = c_o, g2.k = c_i;
    g2.a = ops.in(ce.data, (size_t)((rows - 1) * ce.stride(1) + c_i)), g2.a_stride_m = ce.stride(1), g2.a_stride_k = 1;
    g2.b = ops.in(ow.data, (size_t)(c_o * c_i)), g2.b_stride_n = c_i, g2.b_stride_k = 1;
    g2.c = ops.out(o.data, o_span, o_span != (size_t)(rows * c_o)), g2.c_stride_m = o.stride(1);
    g2.bias = ops.in_f32(ob.data, (size_t)c_o), g2.bias_axis = 1;
    int rc = 0;
    if (ops.ready()) {
        rc = kutacc_launch::pair_gemm(g, s);
        if (rc == 0) {
            rc = kutacc_launch::pair_gemm(g2, s);
        }
    }
    report("kutacc_af2_triangle_multiplication_gate_and_out_linear", ops.finish(rc));
}

void kutacc_af2_triangle_multiplication_last(kutacc_tensor_h out, kutacc_tensor_h gate, int64_t n_res, int64_t n_res_gather,
                                             int64_t c_o)
{
    KUTACC_CHECK(out != nullptr && gate != nullptr, "kutacc_af2_triangle_multiplication_last: input args nullptr error\n");
    KUTACC_CHECK(n_res > 0 && n_res_gather > 0 && c_o > 0 && n_res <= INT64_MAX / n_res_gather,
                 "kutacc_af2_triangle_multiplication_last: input args int values error, values are less than or equal "
                 "to zero, or overflow\n");
    if (KUTACC_FAILED()) {
        return;
    }
    const TensorView &o = *kutacc::as_view(out), &gt = *kutacc::as_view(gate);
    bool on_host = false;
    if (!operands_ok("kutacc_af2_triangle_multiplication_last", {&o, &gt}, {}, &on_host)) {
        return;
    }
    KUTACC_CHECK(o.dim >= 2 && gt.dim >= 2, "kutacc_af2_triangle_multiplication_last: out and gate need rank >= 2");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = kutacc_api::default_stream();
    Operands ops(on_host, s);
    // `out` is read and rewritten in place (triangle_multiplication.cpp:129-150): its mirror is always uploaded first
    void *od = ops.out(o.data, span3(n_res, o.stride(0), n_res_gather, o.stride(1), c_o), true);
    const void *gd = ops.in(gt.data, span3(n_res, gt.stride(0), n_res_gather, gt.stride(1), c_o));
    int rc = 0;
    if (ops.ready()) {
        rc = kutacc_launch::sigmoid_gate_rows(od, o.stride(0), o.stride(1), gd, gt.stride(0), gt.stride(1), n_res, n_res_gather,
                                              c_o, s);
    }
    report("kutacc_af2_triangle_multiplication_last", ops.finish(rc));
}

} // extern "C"
