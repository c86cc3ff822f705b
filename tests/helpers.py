"""Shared plumbing for the parity tests: put a Workload where the call should run, call the C API,
fetch results.  torch only owns memory here."""
from __future__ import annotations

import ctypes

import numpy as np

from kutacc_amd import capi
from kutacc_amd.workloads import Workload, bf16_bits


def torch_dtype(w: Workload):
    import torch
    return torch.bfloat16 if w.dtype == "bf16" else torch.float32


def to_device(w: Workload, device="cuda"):
    """Device tensors in the storage dtype of the workload (fp32 biases stay fp32)."""
    import torch
    dt = torch_dtype(w)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=dt)  # noqa: E731
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device=device, dtype=torch.float32)  # noqa: E731
    B, S, C, H, d = w.B, w.S, w.C, w.H, w.d
    ten = dict(x=t(w.x), wq=t(w.wq), wk=t(w.wk), wv=t(w.wv), wg=t(w.wg), wo=t(w.wo), bg=f(w.bg), bo=f(w.bo),
               bias=t(w.bias), nb=None if w.nb is None else t(w.nb))
    ten["out"] = torch.zeros((B, S, C), device=device, dtype=dt)
    scratch = {n: torch.zeros((B, S, H, d), device=device, dtype=dt) for n in ("q", "k", "gate", "avg")}
    scratch["v"] = torch.zeros((H, d, B, S), device=device, dtype=dt)
    return ten, scratch


def make_op(w: Workload, device="cuda", block_size=64):
    ten, scratch = to_device(w, device)
    op = capi.GatedAttention(ten["x"], ten["wq"], ten["wk"], ten["wv"], ten["wg"], ten["bg"], ten["wo"], ten["bo"],
                             ten["bias"], ten["nb"], w.H, ten["out"], scratch, block_size=block_size)
    return op, ten, scratch


def hip_args(w: Workload, ten, scratch, path=capi.PATH_AUTO) -> capi.HipAttentionArgs:
    """Argument block of the pointer-level entry point for dense tensors."""
    B, S, C, H, d = w.B, w.S, w.C, w.H, w.d
    a = capi.HipAttentionArgs()
    a.batch, a.seq_len, a.nheads, a.head_size = B, S, H, d
    a.dtype = capi.K_BF16 if w.dtype == "bf16" else capi.K_FP32
    a.path = path
    p = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
    a.input, a.input_ld = p(ten["x"]), C
    a.query_w, a.key_w, a.value_w, a.gating_w, a.output_w = (p(ten[k]) for k in ("wq", "wk", "wv", "wg", "wo"))
    a.gating_b, a.output_b = p(ten["bg"]), p(ten["bo"])
    a.bias, a.bias_stride_b = p(ten["bias"]), S
    a.nonbatched_bias = p(ten["nb"])
    a.nb_stride_h, a.nb_stride_q = S * S, S
    a.q, a.k, a.v, a.gate, a.avg = (p(scratch[k]) for k in ("q", "k", "v", "gate", "avg"))
    for n in ("q", "k", "gate", "avg"):
        setattr(a, f"{n}_stride_b", S * C), setattr(a, f"{n}_stride_s", C), setattr(a, f"{n}_stride_h", d)
    a.v_stride_h, a.v_stride_e, a.v_stride_b = d * B * S, B * S, S
    a.out, a.out_ld = p(ten["out"]), C
    return a


def run_hip(w: Workload, ten, scratch, path=capi.PATH_AUTO) -> int:
    import torch
    a = hip_args(w, ten, scratch, path)
    rc = capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None)
    torch.cuda.synchronize()
    return rc


def to_numpy(t) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def host_arrays(w: Workload):
    """numpy arrays in the storage dtype for the host-pointer (staged) path: bf16 as uint16 bits."""
    conv = bf16_bits if w.dtype == "bf16" else (lambda a: np.ascontiguousarray(a, dtype=np.float32))
    B, S, C, H, d = w.B, w.S, w.C, w.H, w.d
    st = np.uint16 if w.dtype == "bf16" else np.float32
    ten = dict(x=conv(w.x), wq=conv(w.wq), wk=conv(w.wk), wv=conv(w.wv), wg=conv(w.wg), wo=conv(w.wo),
               bg=w.bg.astype(np.float32), bo=w.bo.astype(np.float32), bias=conv(w.bias),
               nb=None if w.nb is None else conv(w.nb), out=np.zeros((B, S, C), dtype=st))
    scratch = {n: np.zeros((B, S, H, d), dtype=st) for n in ("q", "k", "gate", "avg")}
    scratch["v"] = np.zeros((H, d, B, S), dtype=st)
    return ten, scratch


def oracle_out(w: Workload, return_avg=False):
    from oracle import oracle
    return oracle.gating_attention_f32(w.x, w.wq, w.wk, w.wv, w.wg, w.bg, w.wo, w.bo, w.bias, w.nb, w.H,
                                       return_avg=return_avg)


def check_close(got, ref, dtype: str, what=""):
    """The parity bar: fp32 path within 1e-4 relative (plus 1e-5 absolute floor); bf16 path within
    2e-2 absolute + 1e-2 relative of the fp32 oracle."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    assert np.all(np.isfinite(got)), f"{what}: non-finite values in result"
    err = np.abs(got - ref)
    tol = (1e-5 + 1e-4 * np.abs(ref)) if dtype == "fp32" else (2e-2 + 1e-2 * np.abs(ref))
    bad = err > tol
    if bad.any():
        i = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} of {err.size} elements outside tolerance; worst at {i}: "
                             f"got {got[i]:.6g} ref {ref[i]:.6g} err {err[i]:.3g} tol {tol[i]:.3g}")
    return float(err.max())


def assert_within(got, ref, tol, what=""):
    """|got - ref| <= tol elementwise, with a short message naming the worst element on failure."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    tol = np.broadcast_to(np.asarray(tol, dtype=np.float64), ref.shape)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    err = np.abs(got - ref)
    bad = ~(err <= tol)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - tol, -np.inf)), err.shape)
        raise AssertionError(f"{what}: {int(bad.sum())} of {err.size} elements outside tolerance; worst at {i}: "
                             f"got {got[i]:.6g} ref {ref[i]:.6g} err {err[i]:.3g} tol {tol[i]:.3g}")
    return float(err.max())


def same_bits(a, b) -> bool:
    """Bitwise equality of two torch tensors, as a plain bool (keeps assertion messages short)."""
    import torch
    return bool(torch.equal(a, b))
