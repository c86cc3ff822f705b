"""ctypes binding of libkutacc.so: the handle-based operator API of include/kutacc.h and the
pointer-level launch layer of include/kutacc_hip.h.

The Python functions keep the C names and argument order (reference include/kutacc.h:297-300, :334,
:399-400, :407-408, :418, :47) so that tests read like calls into the C library.  torch is used only
to own device memory and streams; nothing here computes.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libkutacc.so")

KUTACC_OK = 0
KUTACC_ERROR = -1
K_INT64, K_BF16, K_FP32 = 0, 1, 2
PATH_AUTO, PATH_GENERIC, PATH_FUSED, PATH_TILED = 0, 1, 2, 3
EINVAL, EUNSUPPORTED = -2, -3

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_i32 = ctypes.c_int32
_f32p = ctypes.POINTER(ctypes.c_float)


class Version(ctypes.Structure):
    _fields_ = [(n, ctypes.c_char_p) for n in ("product_name", "product_version", "component_name",
                                                "component_version", "component_abi_version",
                                                "component_appendinfo")]


class AttentionWeights(ctypes.Structure):
    """kutacc_af2_attention_weights_t"""
    _fields_ = [("nchannels", _i64), ("nheads", _i64), ("head_size", _i64), ("query_w", _vp), ("key_w", _vp),
                ("value_w", _vp), ("gating_w", _vp), ("gating_b", _vp), ("output_w", _vp), ("output_b", _vp)]


class AttentionInputs(ctypes.Structure):
    """kutacc_af2_attention_inputs_t"""
    _fields_ = [("batch", _i64), ("seq_len", _i64), ("q", _vp), ("k", _vp), ("v", _vp), ("gate", _vp), ("avg", _vp)]


class HipAttentionArgs(ctypes.Structure):
    """kutacc_hip_attention_args_t"""
    _fields_ = [
        ("batch", _i64), ("seq_len", _i64), ("nheads", _i64), ("head_size", _i64), ("dtype", _i32), ("path", _i32),
        ("input", _vp), ("input_ld", _i64),
        ("query_w", _vp), ("key_w", _vp), ("value_w", _vp), ("gating_w", _vp), ("output_w", _vp),
        ("gating_b", _vp), ("output_b", _vp),
        ("bias", _vp), ("bias_stride_b", _i64),
        ("nonbatched_bias", _vp), ("nb_stride_h", _i64), ("nb_stride_q", _i64),
        ("q", _vp), ("k", _vp), ("v", _vp), ("gate", _vp), ("avg", _vp),
        ("q_stride_b", _i64), ("q_stride_s", _i64), ("q_stride_h", _i64),
        ("k_stride_b", _i64), ("k_stride_s", _i64), ("k_stride_h", _i64),
        ("gate_stride_b", _i64), ("gate_stride_s", _i64), ("gate_stride_h", _i64),
        ("avg_stride_b", _i64), ("avg_stride_s", _i64), ("avg_stride_h", _i64),
        ("v_stride_h", _i64), ("v_stride_e", _i64), ("v_stride_b", _i64),
        ("out", _vp), ("out_ld", _i64),
    ]


class HipGlobalAttentionArgs(ctypes.Structure):
    """kutacc_hip_global_attention_args_t"""
    _fields_ = [
        ("batch", _i64), ("seq_len", _i64), ("nheads", _i64), ("head_size", _i64), ("dtype", _i32), ("reserved", _i32),
        ("q_data", _vp), ("q_data_stride_b", _i64), ("q_data_stride_s", _i64),
        ("q_mask", _vp), ("q_mask_stride_b", _i64),
        ("query_w", _vp), ("key_w", _vp), ("value_w", _vp), ("gating_w", _vp), ("output_w", _vp),
        ("gating_b", _vp), ("output_b", _vp),
        ("q_avg", _vp), ("q_avg_stride_b", _i64),
        ("out", _vp), ("out_stride_b", _i64), ("out_stride_s", _i64),
    ]


class HipGemmArgs(ctypes.Structure):
    """kutacc_hip_gemm_args_t"""
    _fields_ = [
        ("m", _i64), ("n", _i64), ("k", _i64), ("batches", _i64), ("dtype", _i32), ("path", _i32),
        ("a", _vp), ("a_stride_m", _i64), ("a_stride_k", _i64), ("a_stride_batch", _i64),
        ("b", _vp), ("b_stride_n", _i64), ("b_stride_k", _i64), ("b_stride_batch", _i64),
        ("c", _vp), ("c_stride_m", _i64), ("c_stride_batch", _i64),
        ("bias", _vp), ("bias_axis", _i32), ("relu", _i32),
        ("a_gate", _vp), ("bias_gate", _vp), ("mask", _vp), ("mask_stride_batch", _i64),
    ]


class TransWeights(ctypes.Structure):
    """kutacc_af2_trans_weights_t"""
    _fields_ = [("c_o", _i64), ("c_i", _i64), ("linear1_w", _vp), ("linear1_b", _vp), ("linear2_w", _vp), ("linear2_b", _vp)]


class TransActInputs(ctypes.Structure):
    """kutacc_af2_trans_act_inputs_t"""
    _fields_ = [("batch", _i64), ("n_res", _i64), ("input_act", _vp), ("intermediate_act", _vp)]


class TmProjWeights(ctypes.Structure):
    """kutacc_af2_tm_proj_weights_t"""
    _fields_ = [("c_o", _i64), ("c_i", _i64), ("proj_w", _vp), ("proj_b", _vp), ("gate_w", _vp), ("gate_b", _vp)]


class TmActInputs(ctypes.Structure):
    """kutacc_af2_tm_act_inputs_t"""
    _fields_ = [("n_res", _i64), ("n_res_gather", _i64), ("proj_act", _vp), ("input_act", _vp), ("proj_act_gate", _vp)]


class TmLinearWeights(ctypes.Structure):
    """kutacc_af2_tm_linear_weights_t"""
    _fields_ = [("c_o", _i64), ("c_i", _i64), ("gating_w", _vp), ("gating_b", _vp), ("output_proj_w", _vp),
                ("output_proj_b", _vp)]


class HipTriangleAttentionArgs(ctypes.Structure):
    """kutacc_hip_triangle_attention_args_t"""
    _fields_ = [
        ("n_res", _i64), ("nheads", _i64), ("dtype", _i32), ("ending_node", _i32),
        ("pair_act", _vp), ("pair_mask", _vp), ("ln_gamma", _vp), ("ln_beta", _vp), ("ln_eps", ctypes.c_float),
        ("reserved", _i32), ("bias_w", _vp),
        ("query_w", _vp), ("key_w", _vp), ("value_w", _vp), ("gating_w", _vp), ("output_w", _vp),
        ("gating_b", _vp), ("output_b", _vp), ("workspace", _vp), ("workspace_bytes", _i64),
    ]


class HipTriangleMultiplicationArgs(ctypes.Structure):
    """kutacc_hip_triangle_multiplication_args_t"""
    _fields_ = [
        ("n_res", _i64), ("c_z", _i64), ("c_i", _i64), ("dtype", _i32), ("incoming", _i32),
        ("pair_act", _vp), ("pair_mask", _vp), ("ln_in_gamma", _vp), ("ln_in_beta", _vp), ("ln_eps", ctypes.c_float),
        ("reserved", _i32),
        ("left_proj_w", _vp), ("left_proj_b", _vp), ("left_gate_w", _vp), ("left_gate_b", _vp),
        ("right_proj_w", _vp), ("right_proj_b", _vp), ("right_gate_w", _vp), ("right_gate_b", _vp),
        ("ln_center_gamma", _vp), ("ln_center_beta", _vp),
        ("output_w", _vp), ("output_b", _vp), ("gating_w", _vp), ("gating_b", _vp),
        ("workspace", _vp), ("workspace_bytes", _i64),
    ]


class HipMsaAttentionArgs(ctypes.Structure):
    """kutacc_hip_msa_attention_args_t"""
    _fields_ = [
        ("n_seq", _i64), ("n_res", _i64), ("nheads", _i64), ("c_z", _i64), ("dtype", _i32), ("column", _i32),
        ("msa_act", _vp), ("msa_mask", _vp), ("ln_gamma", _vp), ("ln_beta", _vp), ("ln_eps", ctypes.c_float), ("reserved", _i32),
        ("pair_act", _vp), ("pair_ln_gamma", _vp), ("pair_ln_beta", _vp), ("bias_w", _vp),
        ("query_w", _vp), ("key_w", _vp), ("value_w", _vp), ("gating_w", _vp), ("output_w", _vp),
        ("gating_b", _vp), ("output_b", _vp), ("workspace", _vp), ("workspace_bytes", _i64),
    ]


# every symbol the two public headers declare; tests check that the library exports all of them
DECLARED_SYMBOLS = [
    "kutacc_get_version", "kutacc_af2_gating_attention", "kutacc_af2_global_attention", "kutacc_af2_layernorm",
    "kutacc_af2_linear", "kutacc_af2_transition", "kutacc_af2_triangle_multiplication_calc_proj",
    "kutacc_af2_triangle_multiplication_equation", "kutacc_af2_triangle_multiplication_gate_and_out_linear",
    "kutacc_af2_triangle_multiplication_last", "kutacc_hip_gemm", "kutacc_hip_sigmoid_gate_rows", "kutacc_hip_transition",
    "kutacc_hip_pair_bias_transposed", "kutacc_hip_mask_bias", "kutacc_hip_swap_leading_axes", "kutacc_hip_residual_add",
    "kutacc_hip_triangle_attention_workspace", "kutacc_hip_triangle_attention", "kutacc_hip_layernorm_channel_first",
    "kutacc_hip_triangle_multiplication_workspace", "kutacc_hip_triangle_multiplication",
    "kutacc_hip_gated_residual_projection", "kutacc_hip_transition_block_workspace", "kutacc_hip_transition_block",
    "kutacc_hip_layernorm_rows_transposed", "kutacc_hip_msa_attention_workspace", "kutacc_hip_msa_attention",
    "kutacc_af2_linear_weight_prepack", "kutacc_af2_gemm_pack_get_size", "world_size", "rank",
    "_ZN6kutacc13TensorWrapperC1EPvOSt6vectorIlSaIlEES5_lNS_14TensorDataTypeE",
    "_ZN6kutacc13TensorWrapperC1Ev", "_ZN6kutacc13TensorWrapperD1Ev",
    "kutacc_hip_gating_attention", "kutacc_hip_global_attention", "kutacc_hip_last_path", "kutacc_hip_layernorm_rows", "kutacc_hip_linear",
    "kutacc_hip_pair_bias", "kutacc_hip_set_stream", "kutacc_hip_get_stream", "kutacc_hip_set_blocking",
    "kutacc_hip_error_flag", "kutacc_hip_clear_error", "kutacc_hip_tensor_create", "kutacc_hip_tensor_destroy",
    "kutacc_hip_profile_enable", "kutacc_hip_profile_read", "kutacc_hip_set_tuning",
    "kutacc_hip_gating_attention_static", "kutacc_hip_release_staging",
]

_lib = None


def lib() -> ctypes.CDLL:
    """Load the built library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m kutacc_amd.build` "
                           "(the HIP library is the only implementation; there is no CPU path)")
    # One HIP runtime per process: PyTorch ships its own libamdhip64, and a library loaded before it would bind the
    # system copy instead -- a second runtime, which on a GPU box reports "no device" for every call made through it.
    # Loading torch first makes the dynamic loader hand this library the runtime torch already mapped.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    L.kutacc_get_version.argtypes = [ctypes.POINTER(Version)]
    L.kutacc_get_version.restype = ctypes.c_int
    L.kutacc_af2_gating_attention.argtypes = [_vp, ctypes.POINTER(AttentionInputs), _vp, _vp,
                                              ctypes.POINTER(AttentionWeights), _vp, _i64]
    L.kutacc_af2_gating_attention.restype = None
    L.kutacc_af2_global_attention.argtypes = [ctypes.POINTER(AttentionInputs), _vp, _vp, ctypes.POINTER(AttentionWeights),
                                              _vp]
    L.kutacc_af2_global_attention.restype = None
    L.kutacc_hip_global_attention.argtypes = [ctypes.POINTER(HipGlobalAttentionArgs), _vp]
    L.kutacc_hip_global_attention.restype = ctypes.c_int
    L.kutacc_af2_layernorm.argtypes = [_vp, _vp, _vp, _i64, ctypes.c_float, _vp]
    L.kutacc_af2_layernorm.restype = None
    L.kutacc_af2_linear.argtypes = [_vp, _vp, _vp, _vp, _i64]
    L.kutacc_af2_linear.restype = None
    L.kutacc_af2_linear_weight_prepack.argtypes = [_vp, _vp, _i64, _i64, _i64, _i64]
    L.kutacc_af2_linear_weight_prepack.restype = None
    L.kutacc_af2_gemm_pack_get_size.argtypes = [ctypes.c_char, ctypes.c_char, ctypes.c_char, ctypes.c_int,
                                                ctypes.c_int, ctypes.c_int]
    L.kutacc_af2_gemm_pack_get_size.restype = ctypes.c_size_t
    L.kutacc_hip_gating_attention.argtypes = [ctypes.POINTER(HipAttentionArgs), _vp]
    L.kutacc_hip_gating_attention.restype = ctypes.c_int
    L.kutacc_hip_last_path.restype = ctypes.c_char_p
    L.kutacc_hip_layernorm_rows.argtypes = [_vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_float, _i32, _vp]
    L.kutacc_hip_layernorm_rows.restype = ctypes.c_int
    L.kutacc_hip_linear.argtypes = [_vp, _i64, _vp, _i64, _vp, _vp, _i64, _i64, _i64, ctypes.c_float, _i32, _vp]
    L.kutacc_hip_linear.restype = ctypes.c_int
    L.kutacc_hip_pair_bias.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_float, _i32, _vp]
    L.kutacc_hip_pair_bias.restype = ctypes.c_int
    L.kutacc_hip_gemm.argtypes = [ctypes.POINTER(HipGemmArgs), _vp]
    L.kutacc_hip_gemm.restype = ctypes.c_int
    L.kutacc_hip_sigmoid_gate_rows.argtypes = [_vp, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _i32, _vp]
    L.kutacc_hip_sigmoid_gate_rows.restype = ctypes.c_int
    L.kutacc_hip_transition.argtypes = [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp]
    L.kutacc_hip_transition.restype = ctypes.c_int
    L.kutacc_af2_transition.argtypes = [ctypes.POINTER(TransActInputs), ctypes.POINTER(TransWeights), _vp]
    L.kutacc_af2_transition.restype = None
    L.kutacc_af2_triangle_multiplication_calc_proj.argtypes = [ctypes.POINTER(TmActInputs), _vp,
                                                               ctypes.POINTER(TmProjWeights), ctypes.c_bool]
    L.kutacc_af2_triangle_multiplication_calc_proj.restype = None
    L.kutacc_af2_triangle_multiplication_equation.argtypes = [_vp, _vp, _vp, _i64, ctypes.c_bool]
    L.kutacc_af2_triangle_multiplication_equation.restype = None
    L.kutacc_af2_triangle_multiplication_gate_and_out_linear.argtypes = [_vp, _vp, ctypes.POINTER(TmActInputs), _vp,
                                                                         ctypes.POINTER(TmLinearWeights), ctypes.c_bool]
    L.kutacc_af2_triangle_multiplication_gate_and_out_linear.restype = None
    L.kutacc_af2_triangle_multiplication_last.argtypes = [_vp, _vp, _i64, _i64, _i64]
    L.kutacc_af2_triangle_multiplication_last.restype = None
    L.kutacc_hip_pair_bias_transposed.argtypes = L.kutacc_hip_pair_bias.argtypes
    L.kutacc_hip_pair_bias_transposed.restype = ctypes.c_int
    L.kutacc_hip_mask_bias.argtypes = [_vp, _vp, _i64, _i64, _i32, _i32, _vp]
    L.kutacc_hip_mask_bias.restype = ctypes.c_int
    L.kutacc_hip_swap_leading_axes.argtypes = [_vp, _vp, _i64, _i64, _i64, _i32, _vp]
    L.kutacc_hip_swap_leading_axes.restype = ctypes.c_int
    L.kutacc_hip_residual_add.argtypes = [_vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp]
    L.kutacc_hip_residual_add.restype = ctypes.c_int
    L.kutacc_hip_triangle_attention_workspace.argtypes = [_i64, _i64]
    L.kutacc_hip_triangle_attention_workspace.restype = _i64
    L.kutacc_hip_triangle_attention.argtypes = [ctypes.POINTER(HipTriangleAttentionArgs), _vp]
    L.kutacc_hip_triangle_attention.restype = ctypes.c_int
    L.kutacc_hip_layernorm_channel_first.argtypes = [_vp, _i64, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_float, _i32, _vp]
    L.kutacc_hip_layernorm_channel_first.restype = ctypes.c_int
    L.kutacc_hip_triangle_multiplication_workspace.argtypes = [_i64, _i64, _i64]
    L.kutacc_hip_triangle_multiplication_workspace.restype = _i64
    L.kutacc_hip_triangle_multiplication.argtypes = [ctypes.POINTER(HipTriangleMultiplicationArgs), _vp]
    L.kutacc_hip_triangle_multiplication.restype = ctypes.c_int
    L.kutacc_hip_gated_residual_projection.argtypes = [_vp, _i64, _vp, _vp, _vp, _i64, _vp, _i64, _i64, _i64, _i64, _i32, _vp]
    L.kutacc_hip_gated_residual_projection.restype = ctypes.c_int
    L.kutacc_hip_transition_block_workspace.argtypes = [_i64, _i64, _i64]
    L.kutacc_hip_transition_block_workspace.restype = _i64
    L.kutacc_hip_transition_block.argtypes = [_vp, _vp, _vp, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64,
                                              _i32, _vp]
    L.kutacc_hip_transition_block.restype = ctypes.c_int
    L.kutacc_hip_layernorm_rows_transposed.argtypes = [_vp, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_float, _i32, _vp]
    L.kutacc_hip_layernorm_rows_transposed.restype = ctypes.c_int
    L.kutacc_hip_msa_attention_workspace.argtypes = [_i64, _i64, _i64, _i32]
    L.kutacc_hip_msa_attention_workspace.restype = _i64
    L.kutacc_hip_msa_attention.argtypes = [ctypes.POINTER(HipMsaAttentionArgs), _vp]
    L.kutacc_hip_msa_attention.restype = ctypes.c_int
    L.kutacc_hip_set_stream.argtypes = [_vp]
    L.kutacc_hip_get_stream.restype = _vp
    L.kutacc_hip_set_blocking.argtypes = [ctypes.c_int]
    L.kutacc_hip_error_flag.restype = ctypes.c_int
    L.kutacc_hip_tensor_create.argtypes = [_vp, ctypes.POINTER(_i64), ctypes.POINTER(_i64), _i64, _i32]
    L.kutacc_hip_tensor_create.restype = _vp
    L.kutacc_hip_tensor_destroy.argtypes = [_vp]
    L.kutacc_hip_profile_enable.argtypes = [ctypes.c_int]
    L.kutacc_hip_profile_read.argtypes = [ctypes.c_int, ctypes.c_char_p, ctypes.c_int, ctypes.POINTER(ctypes.c_double),
                                          ctypes.POINTER(_i64), ctypes.POINTER(ctypes.c_double)]
    L.kutacc_hip_profile_read.restype = ctypes.c_int
    L.kutacc_hip_gating_attention_static.argtypes = [ctypes.POINTER(HipAttentionArgs), _vp]
    L.kutacc_hip_gating_attention_static.restype = ctypes.c_int
    L.kutacc_hip_release_staging.restype = _i64
    L.kutacc_hip_set_tuning.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    L.kutacc_hip_set_tuning.restype = ctypes.c_int
    _lib = L
    return L


def get_version() -> dict:
    v = Version()
    rc = lib().kutacc_get_version(ctypes.byref(v))
    assert rc == KUTACC_OK
    return {n: getattr(v, n).decode() for n, _ in Version._fields_}


def error_flag() -> bool:
    return bool(lib().kutacc_hip_error_flag())


def clear_error() -> None:
    lib().kutacc_hip_clear_error()


def last_path() -> str:
    return lib().kutacc_hip_last_path().decode()


def set_stream(stream_ptr: int | None) -> None:
    lib().kutacc_hip_set_stream(_vp(stream_ptr or 0))


def set_blocking(blocking: bool) -> None:
    lib().kutacc_hip_set_blocking(1 if blocking else 0)


def set_tuning(name: str, value: str | None) -> int:
    """kutacc_hip_set_tuning: the hooks include/kutacc_hip.h lists ("plan", "fragments", "debug", "row_pairs",
    "gemm_tile", "gated_projection", "layernorm", "scratch", "pointer_checks"); None = the default of that hook."""
    return lib().kutacc_hip_set_tuning(name.encode(), None if value is None else value.encode())


class TensorHandle:
    """Owns one kutacc_tensor_h (the C++ side's TensorWrapper) and keeps the backing array alive."""

    def __init__(self, data_ptr: int, sizes, strides, dtype: int, keepalive=None):
        self.sizes = [int(s) for s in sizes]
        self.strides = [int(s) for s in strides]
        n = len(self.sizes)
        arr = _i64 * max(n, 1)
        self._h = lib().kutacc_hip_tensor_create(_vp(data_ptr), arr(*self.sizes), arr(*self.strides), n, dtype)
        self._keep = keepalive
        self.dtype = dtype

    @property
    def handle(self) -> int:
        return self._h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h and _lib is not None:
            _lib.kutacc_hip_tensor_destroy(_vp(h))


def _torch_dtype_code(t) -> int:
    import torch
    if t.dtype == torch.bfloat16:
        return K_BF16
    if t.dtype == torch.float32:
        return K_FP32
    if t.dtype == torch.int64:
        return K_INT64
    raise TypeError(f"unsupported tensor dtype {t.dtype}")


def tensor(t, dtype: int | None = None) -> TensorHandle:
    """Handle for a torch tensor (device or host memory) or a numpy array (host memory).
    numpy uint16 arrays are taken as bf16 bit patterns."""
    if isinstance(t, np.ndarray):
        code = dtype if dtype is not None else {np.dtype(np.uint16): K_BF16, np.dtype(np.float32): K_FP32,
                                                 np.dtype(np.int64): K_INT64}[t.dtype]
        return TensorHandle(t.ctypes.data, t.shape, [s // t.itemsize for s in t.strides], code, keepalive=t)
    code = dtype if dtype is not None else _torch_dtype_code(t)
    return TensorHandle(t.data_ptr(), list(t.shape), list(t.stride()), code, keepalive=t)


def empty_tensor(dtype: int = K_BF16) -> TensorHandle:
    """A rank-1 tensor with sizes[0] == 0: how a caller says "no nonbatched_bias"
    (reference src/attention/gating_attention.cpp:103)."""
    return TensorHandle(0, [0], [1], dtype)


def kutacc_af2_gating_attention(input, q_based: AttentionInputs, bias, nonbatched_bias, weights: AttentionWeights, out,
                                block_size: int) -> None:
    """Arguments as in the C API; tensor arguments are TensorHandle objects (or None for a null handle)."""
    h = lambda t: _vp(t.handle) if t is not None else None  # noqa: E731
    lib().kutacc_af2_gating_attention(h(input), ctypes.byref(q_based) if q_based is not None else None, h(bias),
                                      h(nonbatched_bias), ctypes.byref(weights) if weights is not None else None,
                                      h(out), block_size)


class GatedAttention:
    """Convenience owner of everything one kutacc_af2_gating_attention call needs, for tensors that
    already live where the call should run (torch tensors on the GPU, or numpy arrays on the host).
    Builds the handles once; `run()` is exactly one C call."""

    def __init__(self, x, wq, wk, wv, wg, bg, wo, bo, bias, nb, nheads, out, scratch, block_size=64):
        B, S, C = x.shape
        self.keep = dict(x=x, wq=wq, wk=wk, wv=wv, wg=wg, bg=bg, wo=wo, bo=bo, bias=bias, nb=nb, out=out, **scratch)
        dt = tensor(x).dtype
        self.h = {k: tensor(v) for k, v in self.keep.items() if v is not None and k not in ("bg", "bo")}
        self.h["bg"] = tensor(bg, K_FP32)
        self.h["bo"] = tensor(bo, K_FP32)
        self.h_nb = self.h["nb"] if nb is not None else empty_tensor(dt)
        self.weights = AttentionWeights(C, nheads, C // nheads, self.h["wq"].handle, self.h["wk"].handle,
                                        self.h["wv"].handle, self.h["wg"].handle, self.h["bg"].handle,
                                        self.h["wo"].handle, self.h["bo"].handle)
        self.inputs = AttentionInputs(B, S, self.h["q"].handle, self.h["k"].handle, self.h["v"].handle,
                                      self.h["gate"].handle, self.h["avg"].handle)
        self.block_size = block_size

    def run(self) -> None:
        kutacc_af2_gating_attention(self.h["x"], self.inputs, self.h["bias"], self.h_nb, self.weights, self.h["out"],
                                    self.block_size)


def kutacc_af2_global_attention(q_based: AttentionInputs, q_data, q_mask, weights: AttentionWeights, out) -> None:
    """Arguments as in the C API; tensor arguments are TensorHandle objects (or None for a null handle)."""
    h = lambda t: _vp(t.handle) if t is not None else None  # noqa: E731
    lib().kutacc_af2_global_attention(ctypes.byref(q_based) if q_based is not None else None, h(q_data), h(q_mask),
                                      ctypes.byref(weights) if weights is not None else None, h(out))


class GlobalAttention:
    """Owner of everything one kutacc_af2_global_attention call needs (torch tensors on the GPU or numpy arrays
    on the host).  x [B,S,64]; mask [B,S,1]; wq, wg, wo [64,64]; wk, wv [d,64]; bg, bo fp32 [64]; out [B,S,64];
    scratch: dict with q [B,64], k [B*S,d], v [d,B*S], gate [B,S,64], avg [B,64]."""

    def __init__(self, x, mask, wq, wk, wv, wg, bg, wo, bo, nheads, out, scratch):
        B, S, C = x.shape
        self.keep = dict(x=x, mask=mask, wq=wq, wk=wk, wv=wv, wg=wg, bg=bg, wo=wo, bo=bo, out=out, **scratch)
        self.h = {k: tensor(v) for k, v in self.keep.items() if k not in ("bg", "bo")}
        self.h["bg"] = tensor(bg, K_FP32)
        self.h["bo"] = tensor(bo, K_FP32)
        self.weights = AttentionWeights(C, nheads, C // nheads, self.h["wq"].handle, self.h["wk"].handle,
                                        self.h["wv"].handle, self.h["wg"].handle, self.h["bg"].handle,
                                        self.h["wo"].handle, self.h["bo"].handle)
        self.inputs = AttentionInputs(B, S, self.h["q"].handle, self.h["k"].handle, self.h["v"].handle,
                                      self.h["gate"].handle, self.h["avg"].handle)

    def run(self) -> None:
        kutacc_af2_global_attention(self.inputs, self.h["x"], self.h["mask"], self.weights, self.h["out"])


# ---- transition and triangle multiplication (reference include/kutacc.h:321-322, 426-456) --------------------
def _h(t):
    return _vp(t.handle) if t is not None else None


def _ref(s):
    return ctypes.byref(s) if s is not None else None


def kutacc_af2_transition(trans_inputs: TransActInputs, trans_weights: TransWeights, out) -> None:
    lib().kutacc_af2_transition(_ref(trans_inputs), _ref(trans_weights), _h(out))


def kutacc_af2_triangle_multiplication_calc_proj(tm_acts: TmActInputs, mask, tm_weights: TmProjWeights,
                                                 input_prepack: bool = False) -> None:
    lib().kutacc_af2_triangle_multiplication_calc_proj(_ref(tm_acts), _h(mask), _ref(tm_weights), input_prepack)


def kutacc_af2_triangle_multiplication_equation(center_act, left_proj_act, right_proj_act, n_res_gather: int,
                                                is_incoming: bool) -> None:
    lib().kutacc_af2_triangle_multiplication_equation(_h(center_act), _h(left_proj_act), _h(right_proj_act), n_res_gather,
                                                      is_incoming)


def kutacc_af2_triangle_multiplication_gate_and_out_linear(gate, out, tm_acts: TmActInputs, center_act,
                                                           tm_weights: TmLinearWeights, input_prepack: bool = False) -> None:
    lib().kutacc_af2_triangle_multiplication_gate_and_out_linear(_h(gate), _h(out), _ref(tm_acts), _h(center_act),
                                                                 _ref(tm_weights), input_prepack)


def kutacc_af2_triangle_multiplication_last(out, gate, n_res: int, n_res_gather: int, c_o: int) -> None:
    lib().kutacc_af2_triangle_multiplication_last(_h(out), _h(gate), n_res, n_res_gather, c_o)


class Transition:
    """Owner of the handles of one kutacc_af2_transition call.  x [batch, n_res, c_o]; w1 [c_i, c_o], w2 [c_o, c_i]
    stored [out, in]; b1 fp32 [c_i], b2 fp32 [c_o]; mid [batch*n_res, c_i] scratch; out like x."""

    def __init__(self, x, w1, b1, w2, b2, mid, out):
        batch, n_res, c_o = x.shape
        self.keep = (x, w1, b1, w2, b2, mid, out)
        self.h = dict(x=tensor(x), w1=tensor(w1), b1=tensor(b1, K_FP32), w2=tensor(w2), b2=tensor(b2, K_FP32),
                      mid=tensor(mid), out=tensor(out))
        self.inputs = TransActInputs(batch, n_res, self.h["x"].handle, self.h["mid"].handle)
        self.weights = TransWeights(c_o, w1.shape[0], self.h["w1"].handle, self.h["b1"].handle, self.h["w2"].handle,
                                    self.h["b2"].handle)

    def run(self) -> None:
        kutacc_af2_transition(self.inputs, self.weights, self.h["out"])


class TriangleAttentionBlock:
    """One triangle-attention block on device tensors, in place on `pair_act` [n, n, c_z]:
    pair_act += gating_attention(LN(pair_act), pair bias from LN(pair_act) . bias_w^T, mask bias from pair_mask),
    around the starting or the ending node.  Owns the workspace; `run()` is one kutacc_hip_triangle_attention call."""

    def __init__(self, pair_act, pair_mask, ln_gamma, ln_beta, bias_w, wq, wk, wv, wg, bg, wo, bo, nheads, ending_node,
                 eps=1e-5):
        import torch
        n = pair_act.shape[0]
        nbytes = lib().kutacc_hip_triangle_attention_workspace(n, nheads)
        assert nbytes > 0
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=pair_act.device)
        self.keep = (pair_act, pair_mask, ln_gamma, ln_beta, bias_w, wq, wk, wv, wg, bg, wo, bo)
        a = HipTriangleAttentionArgs()
        a.n_res, a.nheads, a.dtype, a.ending_node = n, nheads, K_BF16, 1 if ending_node else 0
        a.pair_act, a.pair_mask = pair_act.data_ptr(), pair_mask.data_ptr()
        a.ln_gamma, a.ln_beta, a.ln_eps = ln_gamma.data_ptr(), ln_beta.data_ptr(), eps
        a.bias_w = bias_w.data_ptr()
        a.query_w, a.key_w, a.value_w, a.gating_w, a.output_w = (t.data_ptr() for t in (wq, wk, wv, wg, wo))
        a.gating_b, a.output_b = bg.data_ptr(), bo.data_ptr()
        a.workspace, a.workspace_bytes = self.workspace.data_ptr(), nbytes
        self.args = a

    def run(self, stream_ptr=None) -> int:
        return lib().kutacc_hip_triangle_attention(ctypes.byref(self.args), stream_ptr)


class TriangleMultiplicationBlock:
    """One triangle-multiplication block on device tensors, in place on `pair_act` [n, n, c_z].  `w` is a dict of
    device tensors: ln_in_gamma/beta [c_z], left/right_proj_w and left/right_gate_w [c_i, c_z] with their fp32 biases
    left/right_proj_b, left/right_gate_b [c_i], ln_center_gamma/beta [c_i], output_w [c_z, c_i], output_b [c_z],
    gating_w [c_z, c_z], gating_b [c_z].  Owns the workspace; `run()` is one kutacc_hip_triangle_multiplication call."""

    def __init__(self, pair_act, pair_mask, w, incoming, eps=1e-5):
        import torch
        n, _, c_z = pair_act.shape
        c_i = w["left_proj_w"].shape[0]
        nbytes = lib().kutacc_hip_triangle_multiplication_workspace(n, c_z, c_i)
        assert nbytes > 0
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=pair_act.device)
        self.keep = (pair_act, pair_mask, w)
        a = HipTriangleMultiplicationArgs()
        a.n_res, a.c_z, a.c_i, a.dtype, a.incoming = n, c_z, c_i, K_BF16, 1 if incoming else 0
        a.pair_act, a.pair_mask, a.ln_eps = pair_act.data_ptr(), pair_mask.data_ptr(), eps
        for name in ("ln_in_gamma", "ln_in_beta", "left_proj_w", "left_proj_b", "left_gate_w", "left_gate_b", "right_proj_w",
                     "right_proj_b", "right_gate_w", "right_gate_b", "ln_center_gamma", "ln_center_beta", "output_w",
                     "output_b", "gating_w", "gating_b"):
            setattr(a, name, w[name].data_ptr())
        a.workspace, a.workspace_bytes = self.workspace.data_ptr(), nbytes
        self.args = a

    def run(self, stream_ptr=None) -> int:
        return lib().kutacc_hip_triangle_multiplication(ctypes.byref(self.args), stream_ptr)


class MsaAttentionBlock:
    """One MSA attention block on device tensors, in place on `msa_act` [n_seq, n_res, c_m]: row-wise with pair bias
    (`pair` = dict with pair_act [n_res, n_res, c_z], pair_ln_gamma, pair_ln_beta [c_z], bias_w [nheads, c_z]) or
    column-wise (`pair` None).  `w`: ln_gamma, ln_beta, wq, wk, wv, wg, bg, wo, bo.  Owns the workspace."""

    def __init__(self, msa_act, msa_mask, w, nheads, pair=None, eps=1e-5):
        import torch
        n_seq, n_res, _ = msa_act.shape
        column = pair is None
        nbytes = lib().kutacc_hip_msa_attention_workspace(n_seq, n_res, nheads, 1 if column else 0)
        assert nbytes > 0
        self.workspace = torch.empty(nbytes, dtype=torch.uint8, device=msa_act.device)
        self.keep = (msa_act, msa_mask, w, pair)
        a = HipMsaAttentionArgs()
        a.n_seq, a.n_res, a.nheads, a.dtype, a.column = n_seq, n_res, nheads, K_BF16, 1 if column else 0
        a.msa_act, a.msa_mask, a.ln_eps = msa_act.data_ptr(), msa_mask.data_ptr(), eps
        a.ln_gamma, a.ln_beta = w["ln_gamma"].data_ptr(), w["ln_beta"].data_ptr()
        if pair is not None:
            a.c_z = pair["pair_act"].shape[-1]
            a.pair_act, a.bias_w = pair["pair_act"].data_ptr(), pair["bias_w"].data_ptr()
            a.pair_ln_gamma, a.pair_ln_beta = pair["pair_ln_gamma"].data_ptr(), pair["pair_ln_beta"].data_ptr()
        a.query_w, a.key_w, a.value_w, a.gating_w, a.output_w = (w[k].data_ptr() for k in ("wq", "wk", "wv", "wg", "wo"))
        a.gating_b, a.output_b = w["bg"].data_ptr(), w["bo"].data_ptr()
        a.workspace, a.workspace_bytes = self.workspace.data_ptr(), nbytes
        self.args = a

    def run(self, stream_ptr=None) -> int:
        return lib().kutacc_hip_msa_attention(ctypes.byref(self.args), stream_ptr)
