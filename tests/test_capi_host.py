"""Host-side behaviour of libkutacc.so that needs no GPU: the library loads and exports every
declared symbol, and the argument-validation contract of the operator -- the seven cases of the
reference's own test file (test/functest/cal/gating_attention_test.cpp:18-264: each pointer
argument null in turn, and a negative block_size with non-tensor handles) plus the sticky error
flag (reference src/utils/check.h:50-56)."""
import ctypes
import os
import re

import numpy as np
import pytest

from kutacc_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    for name in capi.DECLARED_SYMBOLS:
        assert hasattr(L, name) or ctypes.c_void_p.in_dll(L, name) is not None, name


def test_headers_and_binding_agree_on_symbol_list():
    """Every kutacc_export declaration in include/*.h is in the binding's list (and so checked above)."""
    text = ""
    for h in ("kutacc.h", "kutacc_hip.h"):
        with open(os.path.join(ROOT, "include", h)) as f:
            text += f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"#define[^\n]*", "", text)
    names = set(re.findall(r"kutacc_export\s+[\w\s\*]*?\b(\w+)\s*\(", text))
    names |= set(re.findall(r"kutacc_export\s+extern\s+int64_t\s+(\w+)\s*;", text))
    names.discard("TensorWrapper")
    assert names, "no declarations parsed"
    missing = sorted(n for n in names if n not in capi.DECLARED_SYMBOLS)
    assert not missing, missing


def test_unimplemented_operators_resolve_and_report():
    L = capi.lib()
    for name in ("kutacc_af2_invariant_point", "kutacc_af2_transpose", "kutacc_comm_init",
                 "kutacc_af2_outer_product_mean_chunk"):
        assert hasattr(L, name), name
    L.kutacc_af2_transpose(None, None)
    assert capi.error_flag()


def test_version():
    v = capi.get_version()
    assert v["component_name"] == "KuTACC" and v["component_abi_version"] == "1"
    assert capi.lib().kutacc_get_version(None) == capi.KUTACC_ERROR


def test_world_size_and_rank_globals():
    L = capi.lib()
    assert ctypes.c_int64.in_dll(L, "world_size").value == 1
    assert ctypes.c_int64.in_dll(L, "rank").value == 0


def test_pack_size_query():
    L = capi.lib()
    assert L.kutacc_af2_gemm_pack_get_size(b"A", b"N", b"N", 3, 4, 5) == 15
    assert L.kutacc_af2_gemm_pack_get_size(b"B", b"T", b"N", 3, 4, 5) == 20


def test_prepack_is_row_major_copy_on_host():
    src = np.arange(6 * 10, dtype=np.uint16).reshape(6, 10)  # n=6 rows, ldb=10, k=7 used
    dst = np.zeros((6, 7), dtype=np.uint16)
    capi.lib().kutacc_af2_linear_weight_prepack(src.ctypes.data, dst.ctypes.data, 6, 7, 10, 0)
    assert not capi.error_flag()
    np.testing.assert_array_equal(dst, src[:, :7])


def _reference_style_arguments():
    """The argument set of the reference's tests: plain floats behind every handle."""
    a = (ctypes.c_float * 1)(1.5)
    x = (ctypes.c_float * 8)(1, 2, 3, 4, 7, 8, 9, 10)
    xp = ctypes.addressof(x)
    weights = capi.AttentionWeights(2, 1, 2, xp, xp, xp, xp, xp, xp, xp)
    inputs = capi.AttentionInputs(2, 2, xp, xp, xp, xp, xp)
    return a, x, ctypes.addressof(a), xp, weights, inputs


@pytest.mark.parametrize("null_index", range(6))
def test_each_null_pointer_is_rejected(null_index, capfd):
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    args = [ap, ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap]
    args[null_index] = None
    capi.lib().kutacc_af2_gating_attention(*args, 5)
    assert capi.error_flag()
    err = capfd.readouterr().err
    assert "KUTACC_CHECK fail in kutacc_af2_gating_attention" in err and "nullptr" in err


def test_negative_block_size_is_rejected_before_any_handle_is_read(capfd):
    # the handles are not tensors at all: reading them would crash, so the scalar check must come first
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    capi.lib().kutacc_af2_gating_attention(ap, ctypes.byref(inputs), ap, xp, ctypes.byref(weights), ap, -5)
    assert capi.error_flag()
    assert "input param <= 0 or overflow" in capfd.readouterr().err


@pytest.mark.parametrize("field,value", [("batch", 0), ("seq_len", -1), ("batch", 2 ** 31)])
def test_bad_extents_are_rejected(field, value):
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    setattr(inputs, field, value)
    capi.lib().kutacc_af2_gating_attention(ap, ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap, 5)
    assert capi.error_flag()


def test_channel_mismatch_is_rejected():
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    weights.nchannels = 3
    capi.lib().kutacc_af2_gating_attention(ap, ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap, 5)
    assert capi.error_flag()


def test_error_flag_is_sticky_until_cleared(capfd):
    """After one failed check every later call returns at its first check, silently for valid
    arguments too (each entry re-tests the flag, reference gating_attention.cpp:168)."""
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    L = capi.lib()
    L.kutacc_af2_gating_attention(None, ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap, 5)
    assert capi.error_flag()
    capfd.readouterr()
    src = np.arange(12, dtype=np.uint16).reshape(3, 4)
    dst = np.zeros((3, 4), dtype=np.uint16)
    L.kutacc_af2_linear_weight_prepack(src.ctypes.data, dst.ctypes.data, 3, 4, 4, 0)
    assert not dst.any(), "a call after a latched error must be a no-op"
    assert capfd.readouterr().err == ""
    capi.clear_error()
    L.kutacc_af2_linear_weight_prepack(src.ctypes.data, dst.ctypes.data, 3, 4, 4, 0)
    np.testing.assert_array_equal(dst, src)


def test_tensor_rank_mismatch_sets_flag():
    arr = (ctypes.c_int64 * 2)(2, 3)
    h = capi.lib().kutacc_hip_tensor_create(None, arr, arr, 2, capi.K_BF16)
    assert h and not capi.error_flag()
    capi.lib().kutacc_hip_tensor_destroy(h)


def test_launch_layer_rejects_bad_arguments_without_a_device():
    L = capi.lib()
    assert L.kutacc_hip_gating_attention(None, None) == capi.EINVAL
    a = capi.HipAttentionArgs()
    assert L.kutacc_hip_gating_attention(ctypes.byref(a), None) == capi.EINVAL
    assert L.kutacc_hip_layernorm_rows(None, 1, None, None, None, 1, 1, 1, 1e-5, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_linear(None, 1, None, 1, None, None, 1, 1, 1, 0.0, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_pair_bias(None, None, None, None, None, None, 1, 1, 1, 1, 1e-5, capi.K_BF16, None) == capi.EINVAL


# ---- kutacc_af2_global_attention: the five null-pointer cases of reference test/functest/cal/global_attention_test.cpp:18-190
@pytest.mark.parametrize("null_index", range(5))
def test_global_attention_null_pointers_are_rejected(null_index, capfd):
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    weights.nchannels = 64
    args = [ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap]
    args[null_index] = None
    capi.lib().kutacc_af2_global_attention(*args)
    assert capi.error_flag()
    assert "nullptr error or invalid int value error" in capfd.readouterr().err


def test_global_attention_needs_64_channels_and_checks_scalars_before_handles(capfd):
    # handles are plain floats, as in the reference's tests: nothing may be read through them
    a, x, ap, xp, weights, inputs = _reference_style_arguments()
    capi.lib().kutacc_af2_global_attention(ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap)  # nchannels == 2
    assert capi.error_flag()
    capi.clear_error()
    weights.nchannels = 64
    inputs.batch = 0
    capi.lib().kutacc_af2_global_attention(ctypes.byref(inputs), ap, ap, ctypes.byref(weights), ap)
    assert capi.error_flag()
    assert "input param <= 0 or overflow" in capfd.readouterr().err


# ---- transition: reference test/functest/cal/transition_test.cpp:18-106 (each pointer null in turn) -------------
def _pair_stack_arguments():
    a = (ctypes.c_float * 1)(0.8)
    x = (ctypes.c_float * 8)(1, 2, 3, 4, 7, 8, 9, 10)
    ap, xp = ctypes.addressof(a), ctypes.addressof(x)
    keep = (a, x)
    return keep, ap, xp


@pytest.mark.parametrize("null_index", range(3))
def test_transition_null_pointers_are_rejected(null_index, capfd):
    keep, ap, xp = _pair_stack_arguments()
    inputs = capi.TransActInputs(2, 2, xp, xp)
    weights = capi.TransWeights(2, 2, xp, xp, xp, xp)
    args = [ctypes.byref(inputs), ctypes.byref(weights), ap]
    args[null_index] = None
    capi.lib().kutacc_af2_transition(*args)
    assert capi.error_flag()
    assert "af2_transition: input args nullptr error" in capfd.readouterr().err


def test_transition_checks_scalars_before_any_handle_is_read(capfd):
    keep, ap, xp = _pair_stack_arguments()
    inputs = capi.TransActInputs(2, 0, xp, xp)  # handles are plain floats: nothing may be read through them
    weights = capi.TransWeights(2, 2, xp, xp, xp, xp)
    capi.lib().kutacc_af2_transition(ctypes.byref(inputs), ctypes.byref(weights), ap)
    assert capi.error_flag()
    assert "input param <= 0 or overflow" in capfd.readouterr().err


# ---- triangle multiplication: reference test/functest/cal/triangle_multiplication_test.cpp:18-354 ---------------
@pytest.mark.parametrize("null_index", range(3))
def test_tm_calc_proj_null_pointers_are_rejected(null_index, capfd):
    keep, ap, xp = _pair_stack_arguments()
    acts = capi.TmActInputs(2, 2, xp, xp, xp)
    weights = capi.TmProjWeights(2, 2, xp, xp, xp, xp)
    args = [ctypes.byref(acts), ap, ctypes.byref(weights)]
    args[null_index] = None
    capi.lib().kutacc_af2_triangle_multiplication_calc_proj(*args, True)
    assert capi.error_flag()
    assert "kutacc_af2_triangle_multiplication_calc_proj: input args nullptr error" in capfd.readouterr().err


@pytest.mark.parametrize("null_index", range(3))
def test_tm_equation_null_pointers_are_rejected(null_index, capfd):
    keep, ap, xp = _pair_stack_arguments()
    args = [ap, ap, ap]
    args[null_index] = None
    capi.lib().kutacc_af2_triangle_multiplication_equation(*args, 5, True)
    assert capi.error_flag()
    assert "kutacc_af2_triangle_multiplication_equation: input args nullptr error" in capfd.readouterr().err


def test_tm_equation_negative_extent_is_rejected_before_any_handle_is_read(capfd):
    keep, ap, xp = _pair_stack_arguments()
    capi.lib().kutacc_af2_triangle_multiplication_equation(ap, ap, ap, -5, True)
    assert capi.error_flag()
    assert "less than or equal to zero" in capfd.readouterr().err


@pytest.mark.parametrize("null_index", range(5))
def test_tm_gate_and_out_linear_null_pointers_are_rejected(null_index, capfd):
    keep, ap, xp = _pair_stack_arguments()
    acts = capi.TmActInputs(2, 2, xp, xp, xp)
    weights = capi.TmLinearWeights(2, 2, xp, xp, xp, xp)
    args = [ap, ap, ctypes.byref(acts), ap, ctypes.byref(weights)]
    args[null_index] = None
    capi.lib().kutacc_af2_triangle_multiplication_gate_and_out_linear(*args, True)
    assert capi.error_flag()
    assert "kutacc_af2_triangle_multiplication_gate_and_out_linear: input args nullptr error" in capfd.readouterr().err


@pytest.mark.parametrize("null_index", range(2))
def test_tm_last_null_pointers_are_rejected(null_index, capfd):
    keep, ap, xp = _pair_stack_arguments()
    args = [ap, ap]
    args[null_index] = None
    capi.lib().kutacc_af2_triangle_multiplication_last(*args, 5, 5, 5)
    assert capi.error_flag()
    assert "kutacc_af2_triangle_multiplication_last: input args nullptr error" in capfd.readouterr().err


@pytest.mark.parametrize("extents", [(-5, 5, 5), (5, -5, 5), (5, 5, -5)])
def test_tm_last_negative_extents_are_rejected_before_any_handle_is_read(extents, capfd):
    keep, ap, xp = _pair_stack_arguments()
    capi.lib().kutacc_af2_triangle_multiplication_last(ap, ap, *extents)
    assert capi.error_flag()
    assert "less than or equal" in capfd.readouterr().err


def test_gemm_launch_layer_rejects_bad_arguments_without_a_device():
    L = capi.lib()
    assert L.kutacc_hip_gemm(None, None) == capi.EINVAL
    g = capi.HipGemmArgs()
    g.m, g.n, g.k, g.batches, g.dtype = 4, 4, 4, 1, capi.K_BF16
    assert L.kutacc_hip_gemm(ctypes.byref(g), None) == capi.EINVAL  # null operands
    assert L.kutacc_hip_sigmoid_gate_rows(None, 1, 1, None, 1, 1, 1, 1, 1, capi.K_BF16, None) == capi.EINVAL


def test_glue_launch_layer_rejects_bad_arguments_without_a_device():
    L = capi.lib()
    assert L.kutacc_hip_mask_bias(None, None, 4, 4, 0, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_swap_leading_axes(None, None, 4, 4, 8, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_residual_add(None, None, 4, 4, 8, 0, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_pair_bias_transposed(None, None, None, None, None, None, 1, 1, 1, 1, 1e-5, capi.K_BF16, None) == capi.EINVAL
    assert L.kutacc_hip_triangle_attention(None, None) == capi.EINVAL
    # activation, pair bias, mask bias and two scratch activations, each rounded up to 256 bytes
    n, h = 384, 4
    act = n * n * h * 32 * 2
    assert L.kutacc_hip_triangle_attention_workspace(n, h) == 3 * act + h * n * n * 2 + n * n * 2
    assert L.kutacc_hip_triangle_attention_workspace(-1, h) == -1


def test_global_attention_launch_layer_rejects_long_rows_before_any_launch():
    """A row's mask and logits must fit the workgroup's LDS: 12288 positions.  Longer rows are refused by the argument
    checks, before any HIP call, so this runs without a GPU (the pointers are never dereferenced)."""
    a = capi.HipGlobalAttentionArgs()
    fake = 1 << 20  # 16-byte aligned, non-null
    a.batch, a.nheads, a.head_size, a.dtype = 2, 8, 8, capi.K_BF16
    for f in ("q_data", "q_mask", "query_w", "key_w", "value_w", "gating_w", "output_w", "gating_b", "output_b", "out"):
        setattr(a, f, fake)
    a.q_data_stride_s = a.out_stride_s = 64
    for seq_len in (12320, 16384):
        a.seq_len = seq_len
        a.q_data_stride_b = a.out_stride_b = 64 * seq_len
        a.q_mask_stride_b = seq_len
        assert capi.lib().kutacc_hip_global_attention(ctypes.byref(a), None) == capi.EUNSUPPORTED


def test_stream_and_blocking_are_inherited_by_threads_that_never_set_them():
    """A thread that sets a stream keeps its own; one that never did sees the value set last by anyone (a host that
    configures the library on one thread and calls it from pool workers).  No GPU needed: the stream is only stored."""
    import threading
    lib = capi.lib()
    lib.kutacc_hip_get_stream.restype = ctypes.c_void_p
    seen = {}
    try:
        lib.kutacc_hip_set_stream(ctypes.c_void_p(0x1000))

        def fresh():
            seen["fresh"] = lib.kutacc_hip_get_stream()

        def own():
            lib.kutacc_hip_set_stream(ctypes.c_void_p(0x2000))
            seen["own"] = lib.kutacc_hip_get_stream()

        for fn in (fresh, own, fresh):
            t = threading.Thread(target=fn)
            t.start()
            t.join()
            if fn is fresh and "first" not in seen:
                seen["first"] = seen.pop("fresh")
        assert seen["first"] == 0x1000        # inherited from the configuring thread
        assert seen["own"] == 0x2000          # a thread's own setting
        assert seen["fresh"] == 0x2000        # a later fresh thread inherits the value set last
        assert lib.kutacc_hip_get_stream() == 0x1000  # and this thread keeps its own
    finally:
        lib.kutacc_hip_set_stream(None)
        assert not lib.kutacc_hip_get_stream()
