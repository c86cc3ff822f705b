// Host side of libkutacc for MI355X: the handle-based entry points of kutacc.h, the tensor
// descriptor, the sticky-error convention, and the extern "C" launch layer of kutacc_hip.h.
// Validation order and error behaviour mirror reference src/attention/gating_attention.cpp:160-200
// (pointer checks), :39-45 and :69 (scalar checks, all before any handle is dereferenced) and
// reference src/linear/mm.cpp:23-35,80-82 (shape / stride / dtype checks of the GEMM operands).
#include <hip/hip_runtime.h>

#include <atomic>
#include <climits>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <mutex>
#include <vector>

#include "check.h"
#include "kutacc.h"
#include "kutacc_hip.h"
#include "api_internal.h"
#include "staging.h"
#include "launch_internal.h"
#include "tensor_view.h"

// ---------------------------------------------------------------------------------------------
// error flag, version, rank globals
// ---------------------------------------------------------------------------------------------
namespace kutacc {
bool kutacc_check_err_set = false;

namespace internal {
void emit_check_failure(const char *func, const char *file, int line, const std::string &detail)
{
    // same line shape as reference src/utils/check.h:38-45: header, message, blank line
    std::ostringstream os;
    os << "KUTACC_CHECK fail in " << func << " at " << file << ":" << line << " , " << detail << "\n\n";
    std::cerr << os.str();
    kutacc_check_err_set = true;
}
} // namespace internal
} // namespace kutacc

kutacc_export int64_t world_size = 1;
kutacc_export int64_t rank = 0;

namespace {
const kutacc_version_t k_version = {
    "Kunpeng HPCKit", "26.1.RC1", "KuTACC", "26.1.RC1", "1", "hip-gfx950",
};

// Stream and blocking mode belong to the calling host thread (as a framework's "current stream" does): two threads
// that each set theirs do not see each other's settings.  A thread that never set one (a worker of a pool whose owner
// configured the library) inherits the value set last by any thread.
std::atomic<hipStream_t> g_shared_stream{nullptr};
std::atomic<bool> g_shared_blocking{true};
thread_local bool t_own_stream = false, t_own_blocking = false;
thread_local hipStream_t t_stream = nullptr;
thread_local bool t_blocking = true;
inline hipStream_t current_stream() { return t_own_stream ? t_stream : g_shared_stream.load(std::memory_order_relaxed); }
inline bool current_blocking() { return t_own_blocking ? t_blocking : g_shared_blocking.load(std::memory_order_relaxed); }
thread_local const char *t_last_path = "none";
// 0: the handle-based entry points take the caller's word that all operands of a call live where `input` lives
std::atomic<int> g_pointer_checks{1};
std::atomic<int> g_block_layernorm{0};
std::atomic<int> g_reference_scratch{0}; // kutacc_af2_gating_attention fills q, k, v, gate as the reference does

inline hipStream_t pick_stream(void *s) { return s ? (hipStream_t)s : current_stream(); }

// Where does a data pointer live?  Plain malloc memory is unknown to HIP (the query fails and leaves
// a sticky error behind, which is cleared here); pinned host memory counts as host.
enum class Space { Host, Device };
Space space_of(const void *p)
{
    hipPointerAttribute_t attr;
    std::memset(&attr, 0, sizeof(attr));
    const hipError_t e = hipPointerGetAttributes(&attr, p);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return Space::Host;
    }
    return (attr.type == hipMemoryTypeDevice || attr.type == hipMemoryTypeManaged) ? Space::Device : Space::Host;
}

using kutacc_api::g_staging;
using kutacc_api::Stager;
} // namespace

kutacc_api::StagingPool kutacc_api::g_staging;

int kutacc_get_version(kutacc_version_t *version)
{
    if (version == nullptr) {
        return KUTACC_ERROR;
    }
    *version = k_version;
    return KUTACC_OK;
}

// ---------------------------------------------------------------------------------------------
// tensor descriptors
// ---------------------------------------------------------------------------------------------
namespace kutacc {
static TensorView *make_view(void *data_ptr, std::vector<int64_t> &&sizes, std::vector<int64_t> &&strides, int64_t dim,
                             DType dtype)
{
    TensorView *t = new TensorView();
    t->data = data_ptr;
    t->sizes = std::move(sizes);
    t->strides = std::move(strides);
    t->dim = dim;
    t->dtype = dtype;
    // rank must agree with both vectors (reference src/tensor/tensor.h:32-33)
    KUTACC_CHECK(dim == (int64_t)t->sizes.size(), dim, " ", t->sizes.size());
    KUTACC_CHECK(dim == (int64_t)t->strides.size(), dim, " ", t->strides.size());
    return t;
}

TensorWrapper::TensorWrapper(void *data_ptr, std::vector<int64_t> &&sizes, std::vector<int64_t> &&strides, int64_t dim,
                             DType dtype)
{
    tensor_ = make_view(data_ptr, std::move(sizes), std::move(strides), dim, dtype);
}

TensorWrapper::TensorWrapper() { tensor_ = nullptr; }

TensorWrapper::~TensorWrapper() { delete static_cast<TensorView *>(tensor_); }
} // namespace kutacc

void *kutacc_hip_tensor_create(void *data, const int64_t *sizes, const int64_t *strides, int64_t dim, int32_t dtype)
{
    if (dim < 0 || (dim > 0 && (!sizes || !strides))) {
        return nullptr;
    }
    return kutacc::make_view(data, std::vector<int64_t>(sizes, sizes + dim), std::vector<int64_t>(strides, strides + dim),
                             dim, (kutacc::DType)dtype);
}

void kutacc_hip_tensor_destroy(void *handle) { delete static_cast<kutacc::TensorView *>(handle); }

// ---------------------------------------------------------------------------------------------
// runtime control
// ---------------------------------------------------------------------------------------------
int64_t kutacc_hip_release_staging(void) { return (int64_t)g_staging.release(); }

// the hooks of the attention launcher live with it; "pointer_checks" belongs to the entry points here
namespace kutacc_launch {
int fused_attention_tuning(const char *name, const char *value);
int pair_gemm_tuning(const char *name, const char *value);
}
int kutacc_hip_set_tuning(const char *name, const char *value)
{
    if (!name) {
        return KUTACC_HIP_EINVAL;
    }
    if (!std::strcmp(name, "pointer_checks")) {
        g_pointer_checks.store((value && value[0] == '0') ? 0 : 1);
        return 0;
    }
    if (!std::strcmp(name, "scratch")) {
        g_reference_scratch.store(value && !std::strcmp(value, "reference") ? 1 : 0);
        return 0;
    }
    if (!std::strcmp(name, "layernorm")) {
        g_block_layernorm.store(value && !std::strcmp(value, "fused") ? 1 : (value && !std::strcmp(value, "separate") ? 2 : 0));
        return 0;
    }
    if (kutacc_launch::pair_gemm_tuning(name, value) == 0) {
        return 0;
    }
    return kutacc_launch::fused_attention_tuning(name, value);
}

void kutacc_hip_set_stream(void *stream)
{
    t_stream = (hipStream_t)stream, t_own_stream = true;
    g_shared_stream.store(t_stream, std::memory_order_relaxed);
}
void *kutacc_hip_get_stream(void) { return (void *)current_stream(); }
void kutacc_hip_set_blocking(int blocking)
{
    t_blocking = blocking != 0, t_own_blocking = true;
    g_shared_blocking.store(t_blocking, std::memory_order_relaxed);
}
int kutacc_hip_error_flag(void) { return kutacc::kutacc_check_err_set ? 1 : 0; }
void kutacc_hip_clear_error(void) { kutacc::kutacc_check_err_set = false; }
const char *kutacc_hip_last_path(void) { return t_last_path; }

// ---------------------------------------------------------------------------------------------
// launch layer
// ---------------------------------------------------------------------------------------------
int kutacc_hip_gating_attention(const kutacc_hip_attention_args_t *a, void *stream)
{
    if (!a || !a->input || !a->query_w || !a->key_w || !a->value_w || !a->gating_w || !a->output_w || !a->gating_b ||
        !a->output_b || !a->bias || !a->out || !a->avg) {
        return KUTACC_HIP_EINVAL;
    }
    if (a->batch <= 0 || a->seq_len <= 0 || a->nheads <= 0 || a->head_size <= 0 || a->batch > INT32_MAX / a->seq_len ||
        a->nheads > INT32_MAX / a->head_size) {
        return KUTACC_HIP_EINVAL;
    }
    const int64_t C = a->nheads * a->head_size;
    if (a->input_ld < C || a->out_ld < C || (a->dtype != KUTACC_DTYPE_BF16 && a->dtype != KUTACC_DTYPE_FP32)) {
        return KUTACC_HIP_EINVAL;
    }
    hipStream_t s = pick_stream(stream);
    const bool fused_ok = kutacc_launch::fused_attention_supports(*a);
    const bool fp32_ok = !fused_ok && kutacc_launch::fp32_attention_supports(*a);
    const bool tiled_ok = kutacc_launch::tiled_attention_supports(*a);
    if ((a->path == KUTACC_HIP_PATH_FUSED && !fused_ok && !fp32_ok && !tiled_ok) || (a->path == KUTACC_HIP_PATH_TILED && !tiled_ok)) {
        return KUTACC_HIP_EUNSUPPORTED;
    }
    int rc;
    if (tiled_ok && (a->path == KUTACC_HIP_PATH_TILED || (!fused_ok && a->path != KUTACC_HIP_PATH_GENERIC))) {
        rc = kutacc_launch::gating_attention_tiled(*a, s);
        if (rc == 0) {
            t_last_path = "tiled_mfma";
        }
    } else if (fp32_ok && a->path != KUTACC_HIP_PATH_GENERIC) {
        rc = kutacc_launch::gating_attention_fp32(*a, s);
        if (rc == 0) {
            t_last_path = "fp32_mfma";
        }
    } else if (fused_ok && a->path != KUTACC_HIP_PATH_GENERIC) {
        rc = kutacc_launch::gating_attention_fused(*a, s);
        if (rc == 0) {
            t_last_path = "fused_mfma";
        }
    } else {
        rc = kutacc_launch::gating_attention_generic(*a, s);
        if (rc == 0) {
            t_last_path = "generic";
        }
    }
    return rc;
}

int kutacc_hip_layernorm_rows(const void *x, int64_t ld_x, const float *gamma, const float *beta, void *out,
                              int64_t ld_out, int64_t rows, int64_t size, float eps, int32_t dtype, void *stream)
{
    return kutacc_launch::layernorm_rows(x, ld_x, gamma, beta, out, ld_out, rows, size, eps, dtype, pick_stream(stream));
}

int kutacc_hip_linear(const void *act, int64_t ld_act, const void *weight, int64_t ld_w, const float *bias, void *result,
                      int64_t m, int64_t n, int64_t k, float beta, int32_t dtype, void *stream)
{
    if (!act || !weight || !result || ld_act < k || ld_w < k) {
        return KUTACC_HIP_EINVAL;
    }
    return kutacc_launch::gemm_nt(dtype, act, ld_act, weight, ld_w, bias, result, n, 1, m, n, k, beta,
                                  pick_stream(stream));
}

int kutacc_hip_pair_bias(const void *z, const float *gamma, const float *beta, const void *w, void *nb, void *z_norm,
                         int64_t rows_i, int64_t rows_j, int64_t c_z, int64_t nheads, float eps, int32_t dtype,
                         void *stream)
{
    return kutacc_launch::pair_bias(z, gamma, beta, w, nb, z_norm, rows_i, rows_j, c_z, nheads, eps, dtype, 0,
                                    pick_stream(stream));
}

// ---------------------------------------------------------------------------------------------
// handle-based API
// ---------------------------------------------------------------------------------------------
namespace {
using kutacc::TensorView;

// Highest element offset a strided [rows, cols] access with unit inner stride touches, plus one.
inline size_t span2(int64_t rows, int64_t row_stride, int64_t cols) { return (size_t)((rows - 1) * row_stride + cols); }

int finish_device_call(int rc, hipStream_t s)
{
    if (rc == 0 && current_blocking()) {
        rc = kutacc_hip_status(hipStreamSynchronize(s));
    }
    return rc;
}
} // namespace

namespace kutacc_api {
hipStream_t default_stream() { return current_stream(); }
hipStream_t stream_or_default(void *s) { return pick_stream(s); }
bool on_device(const void *p) { return space_of(p) == Space::Device; }
int finish(int rc, hipStream_t s) { return finish_device_call(rc, s); }
int block_layernorm_mode() { return g_block_layernorm.load(std::memory_order_relaxed); }
} // namespace kutacc_api

void kutacc_af2_gating_attention(kutacc_tensor_h input, kutacc_af2_attention_inputs_t *q_based_ptr, kutacc_tensor_h bias,
                                 kutacc_tensor_h nonbatched_bias, kutacc_af2_attention_weights_t *weight_ptr,
                                 kutacc_tensor_h out, int64_t block_size)
{
    KUTACC_CHECK(input != nullptr && q_based_ptr != nullptr && bias != nullptr && nonbatched_bias != nullptr &&
                     weight_ptr != nullptr && out != nullptr,
                 "kutacc_af2_gating_attention: input args nullptr error");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t batch = q_based_ptr->batch, seq_len = q_based_ptr->seq_len;
    const int64_t head_size = weight_ptr->head_size, nheads = weight_ptr->nheads, nchannels = weight_ptr->nchannels;

    // scalar checks come before the first look inside any tensor handle: the reference's own tests
    // pass arbitrary non-tensor pointers as handles together with an invalid block_size
    KUTACC_CHECK(batch > 0 && seq_len > 0 && block_size > 0 && head_size > 0 && nheads > 0 && nchannels > 0 &&
                     batch <= INT32_MAX / seq_len && seq_len <= INT32_MAX && nchannels <= INT32_MAX &&
                     head_size <= INT32_MAX && block_size <= INT64_MAX / seq_len,
                 "input param <= 0 or overflow");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t nblocks = (seq_len + block_size - 1) / block_size;
    KUTACC_CHECK(batch <= INT64_MAX / nheads / nblocks, "parallel end overflow");
    KUTACC_CHECK(nchannels == nheads * head_size, "nchannels != nheads * head_size: ", nchannels, " vs ", nheads, "*",
                 head_size);
    if (KUTACC_FAILED()) {
        return;
    }

    kutacc_tensor_h handles[] = {q_based_ptr->q,      q_based_ptr->k,       q_based_ptr->v,       q_based_ptr->gate,
                                 q_based_ptr->avg,    weight_ptr->query_w,  weight_ptr->key_w,    weight_ptr->value_w,
                                 weight_ptr->gating_w, weight_ptr->gating_b, weight_ptr->output_w, weight_ptr->output_b};
    for (kutacc_tensor_h h : handles) {
        KUTACC_CHECK(h != nullptr, "kutacc_af2_gating_attention: tensor handle inside argument struct is null");
    }
    if (KUTACC_FAILED()) {
        return;
    }
    TensorView &in = *kutacc::as_view(input), &bs = *kutacc::as_view(bias), &nb = *kutacc::as_view(nonbatched_bias),
               &ot = *kutacc::as_view(out);
    TensorView &q = *kutacc::as_view(q_based_ptr->q), &k = *kutacc::as_view(q_based_ptr->k),
               &v = *kutacc::as_view(q_based_ptr->v), &gt = *kutacc::as_view(q_based_ptr->gate),
               &av = *kutacc::as_view(q_based_ptr->avg);
    TensorView &wq = *kutacc::as_view(weight_ptr->query_w), &wk = *kutacc::as_view(weight_ptr->key_w),
               &wv = *kutacc::as_view(weight_ptr->value_w), &wg = *kutacc::as_view(weight_ptr->gating_w),
               &bg = *kutacc::as_view(weight_ptr->gating_b), &wo = *kutacc::as_view(weight_ptr->output_w),
               &bo = *kutacc::as_view(weight_ptr->output_b);

    const kutacc::DType dt = in.dtype;
    KUTACC_CHECK(dt == kutacc::kBF16 || dt == kutacc::kFP32, "addmm dtype invalid, a: [", (int)dt, "]");
    KUTACC_CHECK(bs.dtype == dt && ot.dtype == dt && q.dtype == dt && k.dtype == dt && v.dtype == dt && gt.dtype == dt &&
                     av.dtype == dt && wq.dtype == dt && wk.dtype == dt && wv.dtype == dt && wg.dtype == dt &&
                     wo.dtype == dt && (nb.dim == 0 || nb.dtype == dt),
                 "kutacc_af2_gating_attention: tensors of one call must share one dtype");
    KUTACC_CHECK(in.data && bs.data && ot.data && q.data && k.data && v.data && gt.data && av.data && wq.data &&
                     wk.data && wv.data && wg.data && bg.data && wo.data && bo.data,
                 "addmm input invalid");
    KUTACC_CHECK(q.dim >= 3 && k.dim >= 3 && v.dim >= 3 && gt.dim >= 3 && av.dim >= 3 && ot.dim >= 2 && bs.dim >= 1,
                 "kutacc_af2_gating_attention: scratch tensors need rank >= 3, out rank >= 2, bias rank >= 1");
    const bool has_nb = nb.dim >= 1 && nb.size(0) != 0;
    KUTACC_CHECK(!has_nb || (nb.dim >= 2 && nb.data != nullptr), "nonbatched_bias needs rank >= 2 and data");
    if (KUTACC_FAILED()) {
        return;
    }

    kutacc_hip_attention_args_t a;
    std::memset(&a, 0, sizeof(a));
    a.batch = batch, a.seq_len = seq_len, a.nheads = nheads, a.head_size = head_size;
    // "scratch" = "reference": a route that leaves q, k, v and gate as the reference's kernel does
    // (src/attention/gating_attention.cpp:47-66) -- the tiled MFMA route where it takes the call (decided below, once the
    // strides are known), else the shape-agnostic kernels; the fused MFMA kernels never form them in memory
    const bool reference_scratch = g_reference_scratch.load(std::memory_order_relaxed) != 0;
    a.dtype = (int32_t)dt, a.path = KUTACC_HIP_PATH_AUTO;
    a.input = in.data, a.input_ld = nchannels;
    a.query_w = wq.data, a.key_w = wk.data, a.value_w = wv.data, a.gating_w = wg.data, a.output_w = wo.data;
    a.gating_b = (const float *)bg.data, a.output_b = (const float *)bo.data;
    a.bias = bs.data, a.bias_stride_b = bs.stride(0);
    a.nonbatched_bias = has_nb ? nb.data : nullptr;
    a.nb_stride_h = has_nb ? nb.stride(0) : 0, a.nb_stride_q = has_nb ? nb.stride(1) : 0;
    a.q = q.data, a.k = k.data, a.v = v.data, a.gate = gt.data, a.avg = av.data;
    a.q_stride_b = q.stride(0), a.q_stride_s = q.stride(1), a.q_stride_h = q.stride(2);
    a.k_stride_b = k.stride(0), a.k_stride_s = k.stride(1), a.k_stride_h = k.stride(2);
    a.gate_stride_b = gt.stride(0), a.gate_stride_s = gt.stride(1), a.gate_stride_h = gt.stride(2);
    a.avg_stride_b = av.stride(0), a.avg_stride_s = av.stride(1), a.avg_stride_h = av.stride(2);
    a.v_stride_h = v.stride(0), a.v_stride_e = v.stride(1), a.v_stride_b = v.stride(2);
    a.out = ot.data, a.out_ld = ot.stride(ot.dim >= 3 ? 1 : 0);
    // The MFMA kernels may use q as workspace for a copy of the pair bias and take its extent from batch, seq_len and
    // the strides: a handle that describes fewer elements than that must not be written through.
    if (q.numel() < batch * seq_len * nchannels && kutacc_launch::fused_attention_supports(a)) {
        a.q = nullptr;
    }
    auto pick_path = [&]() {
        if (reference_scratch) {
            a.path = kutacc_launch::tiled_attention_supports(a) ? KUTACC_HIP_PATH_TILED : KUTACC_HIP_PATH_GENERIC;
        }
    };
    pick_path();

    hipStream_t s = current_stream();
    const Space sp = space_of(in.data);
    const void *all_ptrs[] = {bs.data, ot.data, q.data, k.data, v.data, gt.data, av.data, wq.data,
                              wk.data, wv.data, wg.data, bg.data, wo.data, bo.data, has_nb ? nb.data : in.data};
    if (g_pointer_checks.load(std::memory_order_relaxed)) {
        for (const void *p : all_ptrs) {
            KUTACC_CHECK(space_of(p) == sp, "kutacc_af2_gating_attention: host and device pointers mixed in one call");
        }
    }
    if (KUTACC_FAILED()) {
        return;
    }

    int rc;
    if (sp == Space::Device) {
        rc = finish_device_call(kutacc_hip_gating_attention(&a, s), s);
    } else {
        // Staged path: mirror every operand on the device, run, copy `out` and `avg` back.
        const size_t e = kutacc::dtype_bytes(dt);
        const int64_t M = batch * seq_len, C = nchannels;
        Stager st(s);
        a.input = st.in(in.data, (size_t)(M * C) * e);
        a.query_w = st.in(wq.data, (size_t)(C * C) * e);
        a.key_w = st.in(wk.data, (size_t)(C * C) * e);
        a.value_w = st.in(wv.data, (size_t)(C * C) * e);
        a.gating_w = st.in(wg.data, (size_t)(C * C) * e);
        a.output_w = st.in(wo.data, (size_t)(C * C) * e);
        a.gating_b = (const float *)st.in(bg.data, (size_t)C * sizeof(float));
        a.output_b = (const float *)st.in(bo.data, (size_t)C * sizeof(float));
        a.bias = st.in(bs.data, span2(batch, a.bias_stride_b, seq_len) * e);
        if (has_nb) {
            a.nonbatched_bias =
                st.in(nb.data, (size_t)((nheads - 1) * a.nb_stride_h + (seq_len - 1) * a.nb_stride_q + seq_len) * e);
        }
        // scratch: dense device copies in the layouts the header documents
        a.q = st.scratch((size_t)(M * C) * e), a.k = st.scratch((size_t)(M * C) * e);
        a.v = st.scratch((size_t)(M * C) * e), a.gate = st.scratch((size_t)(M * C) * e);
        a.q_stride_b = a.k_stride_b = a.gate_stride_b = seq_len * C;
        a.q_stride_s = a.k_stride_s = a.gate_stride_s = C;
        a.q_stride_h = a.k_stride_h = a.gate_stride_h = head_size;
        a.v_stride_h = head_size * M, a.v_stride_e = M, a.v_stride_b = seq_len;
        const bool avg_dense_rows = a.avg_stride_b == seq_len * a.avg_stride_s && a.avg_stride_h == head_size;
        KUTACC_CHECK(avg_dense_rows, "avg must be viewable as a [batch*seq_len, nchannels] matrix");
        a.avg = avg_dense_rows ? st.out(av.data, span2(M, a.avg_stride_s, C) * e, false) : nullptr;
        a.out = st.out(ot.data, span2(M, a.out_ld, C) * e, a.out_ld != C);
        pick_path();
        rc = st.rc;
        if (rc == 0 && !KUTACC_FAILED()) {
            rc = kutacc_hip_gating_attention(&a, s);
        }
        const int rc2 = st.finish();
        if (rc == 0) {
            rc = rc2;
        }
    }
    KUTACC_CHECK(rc == 0, "kutacc_af2_gating_attention: launch layer returned ", rc,
                 rc > 0 ? std::string(" (") + hipGetErrorString((hipError_t)rc) + ")" : std::string());
}

int kutacc_hip_global_attention(const kutacc_hip_global_attention_args_t *a, void *stream)
{
    if (!a) {
        return KUTACC_HIP_EINVAL;
    }
    const int rc = kutacc_launch::global_attention(*a, pick_stream(stream));
    if (rc == 0) {
        t_last_path = "global_mfma";
    }
    return rc;
}

void kutacc_af2_global_attention(kutacc_af2_attention_inputs_t *q_based_ptr, kutacc_tensor_h q_data, kutacc_tensor_h q_mask,
                                 kutacc_af2_attention_weights_t *weight_ptr, kutacc_tensor_h out)
{
    // same first check as the reference, including the hard-wired channel count (global_attention.cpp:171-173)
    KUTACC_CHECK(q_based_ptr != nullptr && q_data != nullptr && q_mask != nullptr && weight_ptr != nullptr &&
                     out != nullptr && weight_ptr->nchannels == 64,
                 "kutacc_af2_gating_attention: input args nullptr error or invalid int value error");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t batch = q_based_ptr->batch, seq_len = q_based_ptr->seq_len;
    const int64_t head_size = weight_ptr->head_size, nheads = weight_ptr->nheads, nchannels = weight_ptr->nchannels;
    // scalar checks before any handle is looked into (global_attention.cpp:37-44)
    KUTACC_CHECK(batch > 0 && seq_len > 0 && nchannels > 0 && nheads > 0 && head_size > 0 && batch <= INT32_MAX / seq_len &&
                     seq_len <= INT32_MAX && nchannels <= INT32_MAX && head_size <= INT32_MAX &&
                     nheads <= INT64_MAX / seq_len && nheads <= INT64_MAX / head_size,
                 "input param <= 0 or overflow");
    if (KUTACC_FAILED()) {
        return;
    }
    KUTACC_CHECK(nchannels == nheads * head_size, "nchannels != nheads * head_size: ", nchannels, " vs ", nheads, "*",
                 head_size);
    kutacc_tensor_h handles[] = {q_based_ptr->avg,     weight_ptr->query_w,  weight_ptr->key_w,    weight_ptr->value_w,
                                 weight_ptr->gating_w, weight_ptr->gating_b, weight_ptr->output_w, weight_ptr->output_b};
    for (kutacc_tensor_h h : handles) {
        KUTACC_CHECK(h != nullptr, "kutacc_af2_global_attention: tensor handle inside argument struct is null");
    }
    if (KUTACC_FAILED()) {
        return;
    }
    TensorView &x = *kutacc::as_view(q_data), &mk = *kutacc::as_view(q_mask), &ot = *kutacc::as_view(out),
               &qa = *kutacc::as_view(q_based_ptr->avg);
    TensorView &wq = *kutacc::as_view(weight_ptr->query_w), &wk = *kutacc::as_view(weight_ptr->key_w),
               &wv = *kutacc::as_view(weight_ptr->value_w), &wg = *kutacc::as_view(weight_ptr->gating_w),
               &bg = *kutacc::as_view(weight_ptr->gating_b), &wo = *kutacc::as_view(weight_ptr->output_w),
               &bo = *kutacc::as_view(weight_ptr->output_b);
    KUTACC_CHECK(x.dtype == kutacc::kBF16 && mk.dtype == kutacc::kBF16 && ot.dtype == kutacc::kBF16 &&
                     qa.dtype == kutacc::kBF16 && wq.dtype == kutacc::kBF16 && wk.dtype == kutacc::kBF16 &&
                     wv.dtype == kutacc::kBF16 && wg.dtype == kutacc::kBF16 && wo.dtype == kutacc::kBF16,
                 "addmm dtype invalid, a: [", (int)x.dtype, "]");
    KUTACC_CHECK(x.data && mk.data && ot.data && qa.data && wq.data && wk.data && wv.data && wg.data && bg.data &&
                     wo.data && bo.data,
                 "addmm input invalid");
    KUTACC_CHECK(ot.dim >= 2 && mk.dim >= 1 && qa.dim >= 1, "kutacc_af2_global_attention: out needs rank >= 2, q_mask and avg rank >= 1");
    if (KUTACC_FAILED()) {
        return;
    }

    kutacc_hip_global_attention_args_t a;
    std::memset(&a, 0, sizeof(a));
    a.batch = batch, a.seq_len = seq_len, a.nheads = nheads, a.head_size = head_size;
    a.dtype = KUTACC_DTYPE_BF16;
    // q_data is read as a dense [batch, seq_len, nchannels] array, as the reference does (:53, :81)
    a.q_data = x.data, a.q_data_stride_b = seq_len * nchannels, a.q_data_stride_s = nchannels;
    a.q_mask = mk.data, a.q_mask_stride_b = mk.stride(0);
    a.query_w = wq.data, a.key_w = wk.data, a.value_w = wv.data, a.gating_w = wg.data, a.output_w = wo.data;
    a.gating_b = (const float *)bg.data, a.output_b = (const float *)bo.data;
    a.q_avg = qa.data, a.q_avg_stride_b = nchannels;
    a.out = ot.data, a.out_stride_s = ot.stride(ot.dim >= 3 ? 1 : 0), a.out_stride_b = seq_len * a.out_stride_s;

    hipStream_t s = current_stream();
    const Space sp = space_of(x.data);
    const void *all_ptrs[] = {mk.data, ot.data, qa.data, wq.data, wk.data, wv.data, wg.data, bg.data, wo.data, bo.data};
    if (g_pointer_checks.load(std::memory_order_relaxed)) {
        for (const void *ptr : all_ptrs) {
            KUTACC_CHECK(space_of(ptr) == sp, "kutacc_af2_global_attention: host and device pointers mixed in one call");
        }
    }
    if (KUTACC_FAILED()) {
        return;
    }
    int rc;
    if (sp == Space::Device) {
        rc = finish_device_call(kutacc_hip_global_attention(&a, s), s);
    } else {
        // Staged path: mirror every operand on the device, run, copy out and q_avg back.
        const size_t e = 2;
        const int64_t M = batch * seq_len, C = nchannels;
        Stager st(s);
        a.q_data = st.in(x.data, (size_t)(M * C) * e);
        a.q_mask = st.in(mk.data, span2(batch, a.q_mask_stride_b, seq_len) * e);
        a.query_w = st.in(wq.data, (size_t)(C * C) * e);
        a.key_w = st.in(wk.data, (size_t)(head_size * C) * e);
        a.value_w = st.in(wv.data, (size_t)(head_size * C) * e);
        a.gating_w = st.in(wg.data, (size_t)(C * C) * e);
        a.output_w = st.in(wo.data, (size_t)(C * C) * e);
        a.gating_b = (const float *)st.in(bg.data, (size_t)C * sizeof(float));
        a.output_b = (const float *)st.in(bo.data, (size_t)C * sizeof(float));
        a.q_avg = st.out(qa.data, (size_t)(batch * C) * e, false);
        a.out = st.out(ot.data, span2(M, a.out_stride_s, C) * e, a.out_stride_s != C);
        rc = st.rc;
        if (rc == 0) {
            rc = kutacc_hip_global_attention(&a, s);
        }
        const int rc2 = st.finish();
        if (rc == 0) {
            rc = rc2;
        }
    }
    KUTACC_CHECK(rc == 0, "kutacc_af2_global_attention: launch layer returned ", rc,
                 rc > 0 ? std::string(" (") + hipGetErrorString((hipError_t)rc) + ")" : std::string());
}

void kutacc_af2_layernorm(__bf16 *data, float *gamma, float *beta, int64_t size, float eps, __bf16 *out)
{
    // The reference dereferences unconditionally (src/normalization/layernorm.cpp:17-20); a device
    // launch deserves the check.
    KUTACC_CHECK(data != nullptr && gamma != nullptr && beta != nullptr && out != nullptr && size > 0,
                 "kutacc_af2_layernorm: null pointer or size <= 0");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = current_stream();
    int rc;
    if (space_of(data) == Space::Device) {
        rc = finish_device_call(
            kutacc_hip_layernorm_rows(data, size, gamma, beta, out, size, 1, size, eps, KUTACC_DTYPE_BF16, s), s);
    } else {
        Stager st(s);
        const void *dx = st.in(data, (size_t)size * 2);
        const float *dg = (const float *)st.in(gamma, (size_t)size * 4);
        const float *db = (const float *)st.in(beta, (size_t)size * 4);
        void *dout = st.out(out, (size_t)size * 2, false);
        rc = st.rc;
        if (rc == 0) {
            rc = kutacc_hip_layernorm_rows(dx, size, dg, db, dout, size, 1, size, eps, KUTACC_DTYPE_BF16, s);
        }
        const int rc2 = st.finish();
        rc = rc ? rc : rc2;
    }
    KUTACC_CHECK(rc == 0, "kutacc_af2_layernorm: launch layer returned ", rc);
}

void kutacc_af2_linear(kutacc_tensor_h act, kutacc_tensor_h weight, float *bias_data, kutacc_tensor_h result,
                       int64_t beta)
{
    KUTACC_CHECK(act != nullptr && weight != nullptr && result != nullptr, "kutacc_af2_linear: input args nullptr error");
    if (KUTACC_FAILED()) {
        return;
    }
    TensorView &a = *kutacc::as_view(act), &w = *kutacc::as_view(weight), &r = *kutacc::as_view(result);
    KUTACC_CHECK(a.dim >= 2 && w.dim >= 2 && r.dim >= 1, "dim invalid, a: [", a.dim, "], b: [", w.dim, "], c: [", r.dim,
                 "]");
    KUTACC_CHECK(a.data != nullptr && w.data != nullptr && r.data != nullptr, "addmm input invalid");
    KUTACC_CHECK((a.dtype == kutacc::kBF16 || a.dtype == kutacc::kFP32) && w.dtype == a.dtype && r.dtype == a.dtype,
                 "addmm dtype invalid, a: [", (int)a.dtype, "], b: [", (int)w.dtype, "], c: [", (int)r.dtype, "]");
    if (KUTACC_FAILED()) {
        return;
    }
    // m, n, k and leading dimensions exactly as reference src/linear/linear.cpp:23-31 derives them
    const int64_t k = a.sizes.back();
    KUTACC_CHECK(k > 0 && w.sizes.back() == k, "shape invalid, a: [", a.numel() / (k ? k : 1), ", ", k, "], b: [",
                 w.sizes.back(), ", ", w.numel() / (w.sizes.back() ? w.sizes.back() : 1), "]");
    if (KUTACC_FAILED()) {
        return;
    }
    const int64_t m = a.numel() / k, n = w.numel() / k;
    const int64_t lda = a.stride(a.dim - 2), ldw = w.stride(w.dim - 2);
    KUTACC_CHECK(m > 0 && n > 0 && r.numel() >= m * n, "shape invalid, a: [", m, ", ", k, "], b: [", k, ", ", n,
                 "], c: [", r.numel(), "]");
    KUTACC_CHECK(a.stride(a.dim - 1) == 1 && lda >= k, "a strides invalid: [", lda, ", ", a.stride(a.dim - 1), "]");
    KUTACC_CHECK(w.stride(w.dim - 1) == 1 && ldw >= k, "b strides invalid: [", ldw, ", ", w.stride(w.dim - 1), "]");
    if (KUTACC_FAILED()) {
        return;
    }
    // the reference converts the integer beta to bf16 before use (linear.cpp:29)
    const float beta_f = (float)(__bf16)(float)beta;
    const Space sp = space_of(a.data);
    KUTACC_CHECK(space_of(w.data) == sp && space_of(r.data) == sp && (!bias_data || space_of(bias_data) == sp),
                 "kutacc_af2_linear: host and device pointers mixed in one call");
    if (KUTACC_FAILED()) {
        return;
    }
    hipStream_t s = current_stream();
    int rc;
    if (sp == Space::Device) {
        rc = finish_device_call(
            kutacc_hip_linear(a.data, lda, w.data, ldw, bias_data, r.data, m, n, k, beta_f, (int32_t)a.dtype, s), s);
    } else {
        const size_t e = kutacc::dtype_bytes(a.dtype);
        Stager st(s);
        const void *da = st.in(a.data, span2(m, lda, k) * e);
        const void *dw = st.in(w.data, span2(n, ldw, k) * e);
        const float *db = bias_data ? (const float *)st.in(bias_data, (size_t)n * 4) : nullptr;
        void *dr = st.out(r.data, (size_t)(m * n) * e, beta != 0);
        rc = st.rc;
        if (rc == 0) {
            rc = kutacc_hip_linear(da, lda, dw, ldw, db, dr, m, n, k, beta_f, (int32_t)a.dtype, s);
        }
        const int rc2 = st.finish();
        rc = rc ? rc : rc2;
    }
    KUTACC_CHECK(rc == 0, "kutacc_af2_linear: launch layer returned ", rc);
}

void kutacc_af2_linear_weight_prepack(const __bf16 *weight, __bf16 *result, int64_t n, int64_t k, int64_t ldb,
                                      int64_t num_threads)
{
    (void)num_threads;
    KUTACC_CHECK(weight != nullptr && result != nullptr && n > 0 && k > 0 && ldb >= k,
                 "kutacc_af2_linear_weight_prepack: null pointer or invalid n/k/ldb");
    if (KUTACC_FAILED()) {
        return;
    }
    // Packed layout on this backend = dense row-major [n, k]: a pitched copy, host or device.
    const Space sp = space_of(weight);
    KUTACC_CHECK(space_of(result) == sp, "kutacc_af2_linear_weight_prepack: host and device pointers mixed");
    if (KUTACC_FAILED()) {
        return;
    }
    if (sp == Space::Host) {
        for (int64_t r = 0; r < n; ++r) {
            std::memcpy((void *)(result + r * k), (const void *)(weight + r * ldb), (size_t)k * 2);
        }
        return;
    }
    hipError_t e = hipMemcpy2DAsync(result, (size_t)k * 2, weight, (size_t)ldb * 2, (size_t)k * 2, (size_t)n,
                                    hipMemcpyDeviceToDevice, current_stream());
    if (e == hipSuccess && current_blocking()) {
        e = hipStreamSynchronize(current_stream());
    }
    KUTACC_CHECK(e == hipSuccess, "kutacc_af2_linear_weight_prepack: ", hipGetErrorString(e));
}

size_t kutacc_af2_gemm_pack_get_size(char identifier, char transa, char transb, int m, int n, int k)
{
    (void)transa;
    (void)transb;
    // 'A' packs the [m, k] operand, 'B' the [k, n] one (reference include/kutacc.h:411-418)
    if (m < 0 || n < 0 || k < 0) {
        return 0;
    }
    if (identifier == 'A' || identifier == 'a') {
        return (size_t)m * (size_t)k;
    }
    if (identifier == 'B' || identifier == 'b') {
        return (size_t)k * (size_t)n;
    }
    return 0;
}
