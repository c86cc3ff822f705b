"""ctypes front end of the CPU oracle plus an independent numpy fp64 twin.

TEST INFRASTRUCTURE ONLY.  Importers: tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py.  The shipped library (kutacc_amd/) never imports this module.

Functions follow reference src/attention/gating_attention.cpp:33-158 (operator),
src/normalization/layernorm_kernel.h:21-53 (LayerNorm) and src/linear/linear.cpp:21-42 (Linear); see
oracle/kutacc_oracle.c for the line-by-line citations and the pinning status of each function.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkutacc_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i64 = ctypes.c_int64


def build(force: bool = False) -> str:
    """Compile oracle/kutacc_oracle.c with gcc (recipe: oracle/Makefile)."""
    src = os.path.join(_HERE, "kutacc_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libkutacc_oracle.so"], stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_num_threads.restype = ctypes.c_int
    return _lib


def num_threads() -> int:
    return int(lib().oracle_num_threads())


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def ref_exp(x, exp_mode=1):
    """The oracle's model of the reference's fast_exp (src/math/fast_exp.h:21-27) on an array of float32."""
    x = _f32(x).ravel()
    y = np.empty_like(x)
    lib().oracle_ref_exp(x.ctypes.data_as(_f32p), y.ctypes.data_as(_f32p), _i64(x.size), ctypes.c_int(exp_mode))
    return y


def _u16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint16, a.dtype
    return a


def _ptr(a, ty):
    return None if a is None else a.ctypes.data_as(ty)


# ---- bf16 bit helpers (round to nearest even, as reference src/wrapper/svcvt.h:23-30) ----------
def to_bf16_bits(a) -> np.ndarray:
    a = _f32(a)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16(_ptr(a, _f32p), _ptr(out, _u16p), _i64(a.size))
    return out


def from_bf16_bits(a) -> np.ndarray:
    a = _u16(a)
    return (a.astype(np.uint32) << 16).view(np.float32)


def round_bf16(a) -> np.ndarray:
    """fp32 -> bf16 -> fp32."""
    return from_bf16_bits(to_bf16_bits(a))


# ---- R32: the parity oracle ----------------------------------------------------------------------
def gating_attention_f32(x, wq, wk, wv, wg, bg, wo, bo, bias, nb, nheads, return_avg=False):
    """x [B,S,C] fp32; weights [C,C] stored [out,in]; bias [B,S]; nb [H,S,S] or None -> out [B,S,C]."""
    x = _f32(x)
    B, S, C = x.shape
    d = C // nheads
    args = [_f32(a) for a in (wq, wk, wv, wg, bg, wo, bo, bias)]
    nb_c = None if nb is None else _f32(nb)
    out = np.empty((B, S, C), dtype=np.float32)
    avg = np.empty((B, S, C), dtype=np.float32) if return_avg else None
    lib().oracle_gating_attention_f32(
        _ptr(x, _f32p), *[_ptr(a, _f32p) for a in args], _ptr(nb_c, _f32p),
        _i64(B), _i64(S), _i64(nheads), _i64(d), _ptr(out, _f32p), _ptr(avg, _f32p))
    return (out, avg) if return_avg else out


# ---- Rbf16: reference-faithful rounding points, the timed CPU baseline ---------------------------
def gating_attention_bf16(x, wq, wk, wv, wg, bg, wo, bo, bias, nb, nheads, block_size=64, exp_mode=1,
                          return_scratch=False):
    """All tensor arguments are bf16 bit patterns (uint16) except bg/bo (fp32).  Returns out bits."""
    x = _u16(x)
    B, S, C = x.shape
    d = C // nheads
    w = [_u16(a) for a in (wq, wk, wv, wg)]
    wo = _u16(wo)
    bg, bo = _f32(bg), _f32(bo)
    bias = _u16(bias)
    nb_c = None if nb is None else _u16(nb)
    q, k, v, gate, avg, out = (np.empty((B, S, C), dtype=np.uint16) for _ in range(6))
    lib().oracle_gating_attention_bf16(
        _ptr(x, _u16p), *[_ptr(a, _u16p) for a in w], _ptr(bg, _f32p), _ptr(wo, _u16p), _ptr(bo, _f32p),
        _ptr(bias, _u16p), _ptr(nb_c, _u16p), _i64(B), _i64(S), _i64(nheads), _i64(d), _i64(block_size),
        ctypes.c_int(exp_mode), *[_ptr(a, _u16p) for a in (q, k, v, gate, avg, out)])
    if return_scratch:
        return out, dict(q=q, k=k, v=v.reshape(nheads, d, B, S), gate=gate, avg=avg)
    return out


# ---- row operators -------------------------------------------------------------------------------
def layernorm_rows_bf16(x_bits, gamma, beta, eps):
    x_bits = _u16(x_bits)
    size = x_bits.shape[-1]
    rows = x_bits.size // size
    out = np.empty_like(x_bits)
    gamma, beta = _f32(gamma), _f32(beta)
    lib().oracle_layernorm_rows_bf16(_ptr(x_bits, _u16p), _ptr(gamma, _f32p), _ptr(beta, _f32p), _i64(rows),
                                     _i64(size), ctypes.c_float(eps), _ptr(out, _u16p))
    return out


def layernorm_rows_f32(x, gamma, beta, eps):
    x = _f32(x)
    size = x.shape[-1]
    rows = x.size // size
    out = np.empty_like(x)
    gamma, beta = _f32(gamma), _f32(beta)
    lib().oracle_layernorm_rows_f32(_ptr(x, _f32p), _ptr(gamma, _f32p), _ptr(beta, _f32p), _i64(rows), _i64(size),
                                    ctypes.c_float(eps), _ptr(out, _f32p))
    return out


def linear_bf16(act_bits, w_bits, bias=None, beta=0.0, result_bits=None):
    act_bits, w_bits = _u16(act_bits), _u16(w_bits)
    k = act_bits.shape[-1]
    m, n = act_bits.size // k, w_bits.size // k
    res = np.zeros((m, n), dtype=np.uint16) if result_bits is None else _u16(result_bits).reshape(m, n).copy()
    b = None if bias is None else _f32(bias)
    lib().oracle_linear_bf16(_ptr(act_bits, _u16p), _i64(k), _ptr(w_bits, _u16p), _i64(k), _ptr(b, _f32p),
                             _ptr(res, _u16p), _i64(m), _i64(n), _i64(k), ctypes.c_float(beta))
    return res


def linear_f32(act, w, bias=None, beta=0.0, result=None):
    act, w = _f32(act), _f32(w)
    k = act.shape[-1]
    m, n = act.size // k, w.size // k
    res = np.zeros((m, n), dtype=np.float32) if result is None else _f32(result).reshape(m, n).copy()
    b = None if bias is None else _f32(bias)
    lib().oracle_linear_f32(_ptr(act, _f32p), _i64(k), _ptr(w, _f32p), _i64(k), _ptr(b, _f32p), _ptr(res, _f32p),
                            _i64(m), _i64(n), _i64(k), ctypes.c_float(beta))
    return res


# ---- global (extra-MSA column) attention ------------------------------------------------------------
def global_attention_f32(x, mask, wq, wk, wv, wg, bg, wo, bo, nheads, return_q_avg=False):
    """x [B,S,C]; mask [B,S]; wq, wg, wo [C,C] stored [out,in]; wk, wv [d,C]; bg, bo [C] -> out [B,S,C]."""
    x = _f32(x)
    B, S, C = x.shape
    d = C // nheads
    args = [_f32(a) for a in (mask, wq, wk, wv, wg, bg, wo, bo)]
    out = np.empty((B, S, C), dtype=np.float32)
    qa = np.empty((B, C), dtype=np.float32) if return_q_avg else None
    lib().oracle_global_attention_f32(_ptr(x, _f32p), *[_ptr(a, _f32p) for a in args], _i64(B), _i64(S), _i64(nheads),
                                      _i64(d), _ptr(out, _f32p), _ptr(qa, _f32p))
    return (out, qa) if return_q_avg else out


def global_attention_f64_numpy(x, mask, wq, wk, wv, wg, bg, wo, bo, nheads):
    """Textbook float64 formulation of reference src/attention/global_attention.cpp:30-164; the mask bias
    mask*1e9 - 1e9 is formed and added in fp32 (:120-123)."""
    f = lambda a: np.asarray(a, dtype=np.float64)  # noqa: E731
    x, mask = f(x), f(mask)
    B, S, C = x.shape
    H, d = nheads, C // nheads
    q_avg = (mask[:, :, None] * x).sum(axis=1) / (mask.sum(axis=1, keepdims=True) + 1e-10)
    q = (q_avg @ f(wq).T).reshape(B, H, d)
    k = x @ f(wk).T  # [B,S,d]
    v = x @ f(wv).T
    gate = x @ f(wg).T + f(bg)
    scale = float(np.float32(1.0 / np.sqrt(float(d))))
    logits = np.einsum("bhd,bsd->bhs", q, k) * scale
    bias = (np.asarray(mask, dtype=np.float32) * np.float32(1e9) + np.float32(-1e9))
    xl = (logits.astype(np.float32) + bias[:, None, :]).astype(np.float64)
    xl = xl - xl.max(axis=-1, keepdims=True)
    p = np.exp(xl)
    p /= p.sum(axis=-1, keepdims=True)
    wavg = np.einsum("bhs,bsd->bhd", p, v).reshape(B, 1, C)
    gated = wavg / (1.0 + np.exp(-gate))
    return gated @ f(wo).T + f(bo)


# ---- independent numpy fp64 twin (used to pin the C code, and as R64 for golden fixtures) ---------
def gating_attention_f64_numpy(x, wq, wk, wv, wg, bg, wo, bo, bias, nb, nheads, return_avg=False):
    """Textbook formulation in float64; the two bias additions are fp32 additions so that the -1e9
    mask absorbs the logit exactly as in the reference (gating_attention.cpp:113-117)."""
    x = np.asarray(x, dtype=np.float64)
    B, S, C = x.shape
    H, d = nheads, C // nheads
    f = lambda a: np.asarray(a, dtype=np.float64)  # noqa: E731
    q = (x @ f(wq).T).reshape(B, S, H, d)
    k = (x @ f(wk).T).reshape(B, S, H, d)
    v = (x @ f(wv).T).reshape(B, S, H, d)
    g = (x @ f(wg).T + f(bg)).reshape(B, S, H, d)
    logits = np.einsum("bqhd,bkhd->bhqk", q, k) / np.sqrt(float(d))
    xl = logits.astype(np.float32) + np.asarray(bias, dtype=np.float32)[:, None, None, :]
    if nb is not None:
        xl = xl + np.asarray(nb, dtype=np.float32)[None]
    xl = xl.astype(np.float64)
    xl = xl - xl.max(axis=-1, keepdims=True)
    p = np.exp(xl)
    p /= p.sum(axis=-1, keepdims=True)
    avg = np.einsum("bhqk,bkhd->bqhd", p, v) / (1.0 + np.exp(-g))
    avg = avg.reshape(B, S, C)
    out = avg @ f(wo).T + f(bo)
    return (out, avg) if return_avg else out


# ---- transition and triangle multiplication ---------------------------------------------------------
def transition_f32(x, w1, b1, w2, b2, return_mid=False):
    """x [rows, c_o]; w1 [c_i, c_o], w2 [c_o, c_i] stored [out, in]; b1 [c_i], b2 [c_o] -> out [rows, c_o]
    (reference src/attention/transition.cpp:31-38)."""
    x, w1, b1, w2, b2 = (_f32(a) for a in (x, w1, b1, w2, b2))
    c_i, c_o = w1.shape
    rows = x.size // c_o
    out = np.empty((rows, c_o), dtype=np.float32)
    mid = np.empty((rows, c_i), dtype=np.float32) if return_mid else None
    lib().oracle_transition_f32(_ptr(x, _f32p), _ptr(w1, _f32p), _ptr(b1, _f32p), _ptr(w2, _f32p), _ptr(b2, _f32p),
                                _i64(rows), _i64(c_o), _i64(c_i), _ptr(out, _f32p), _ptr(mid, _f32p))
    return (out, mid) if return_mid else out


def tm_calc_proj_f32(x, mask, pw, pb, gw, gb):
    """x [n_res, n_gather, c_o]; mask [n_res, n_gather]; pw, gw [c_i, c_o]; pb, gb [c_i] -> proj [c_i, n_res, n_gather]
    (reference src/attention/triangle_multiplication.cpp:37-66)."""
    x, mask, pw, pb, gw, gb = (_f32(a) for a in (x, mask, pw, pb, gw, gb))
    n_res, n_gather, c_o = x.shape
    c_i = pw.shape[0]
    proj = np.empty((c_i, n_res, n_gather), dtype=np.float32)
    lib().oracle_tm_calc_proj_f32(_ptr(x, _f32p), _ptr(mask, _f32p), _ptr(pw, _f32p), _ptr(pb, _f32p), _ptr(gw, _f32p),
                                  _ptr(gb, _f32p), _i64(n_res * n_gather), _i64(c_o), _i64(c_i), _ptr(proj, _f32p))
    return proj


def tm_equation_f32(left, right, incoming):
    """left, right [c, n, n] -> center [c, n, n] (reference src/attention/triangle_multiplication.cpp:72-101)."""
    left, right = _f32(left), _f32(right)
    c, n, _ = left.shape
    center = np.empty((c, n, n), dtype=np.float32)
    lib().oracle_tm_equation_f32(_ptr(left, _f32p), _ptr(right, _f32p), _i64(c), _i64(n), ctypes.c_int(1 if incoming else 0),
                                 _ptr(center, _f32p))
    return center


def tm_gate_and_out_f32(x, center, gating_w, gating_b, out_w, out_b):
    """gate = x . gating_w^T + gating_b and out = center . out_w^T + out_b over rows (i, j): two plain linears
    (reference src/attention/triangle_multiplication.cpp:115-126).  x [.., c_o], center [.., c_i]."""
    gate = linear_f32(_f32(x).reshape(-1, np.shape(x)[-1]), gating_w, gating_b)
    out = linear_f32(_f32(center).reshape(-1, np.shape(center)[-1]), out_w, out_b)
    return gate, out


def tm_last_f32(out, gate):
    """out * sigmoid(gate) (reference src/attention/triangle_multiplication.cpp:139-146), evaluated in float64."""
    o, g = np.asarray(out, dtype=np.float64), np.asarray(gate, dtype=np.float64)
    return (o / (1.0 + np.exp(-g))).astype(np.float32)
