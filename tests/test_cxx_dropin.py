"""A C++ caller compiled against kutacc.h, linked against libkutacc.so and run inside this process.

tests/cxx/dropin_caller.cpp builds its tensor handles with kutacc::TensorWrapper's std::vector<int64_t>&& constructor
and calls the handle-based entry points exactly as a consumer of the Kunpeng library does (reference
test/functest/cal/gating_attention_test.cpp:18-264, include/kutacc.h:484-497).  It exists in up to two builds made by
`kutacc_amd.build.build_dropin_callers()`: libdropin_caller.so (this repository's include/kutacc.h) and, where the
reference tree was present at build time, libdropin_caller_ref.so (the reference's own header).  The CPU tests check the
struct layouts of both builds against each other and run the reference's seven argument-validation cases; the GPU tests
make a real call through each build and compare `out` bit for bit with the ctypes-handle path, and feed the operator
weights that went through kutacc_af2_linear_weight_prepack on the device (reference src/linear/mm.cpp:94-110).
"""
import ctypes
import os

import numpy as np
import pytest

from kutacc_amd import capi
from kutacc_amd.workloads import make_workload

import helpers

HERE = os.path.dirname(os.path.abspath(__file__))
BUILDS = {"own_header": os.path.join(HERE, "cxx", "libdropin_caller.so"),
          "reference_header": os.path.join(HERE, "cxx", "libdropin_caller_ref.so")}

_vp, _i64 = ctypes.c_void_p, ctypes.c_int64


def load(which):
    path = BUILDS[which]
    if not os.path.exists(path):
        if which == "reference_header":
            pytest.skip("no build against the reference header here (made only where /root/reference exists)")
        raise AssertionError(f"{path} is missing: run `python -m kutacc_amd.build`")
    capi.lib()  # the library first, so that the caller binds the copy under test
    L = ctypes.CDLL(path)
    L.dropin_layout.argtypes = [ctypes.POINTER(_i64), ctypes.c_int]
    L.dropin_validation_case.argtypes = [ctypes.c_int]
    L.dropin_component_name.restype = ctypes.c_char_p
    L.dropin_gating_attention.argtypes = [_vp] * 16 + [_i64] * 5
    L.dropin_prepack.argtypes = [_vp, _vp, _i64, _i64, _i64]
    L.dropin_prepack.restype = None
    L.dropin_global_attention.argtypes = [_vp] * 15 + [_i64] * 4
    L.dropin_transition.argtypes = [_vp] * 7 + [_i64] * 4
    return L


def layout(L):
    buf = (_i64 * 64)()
    n = L.dropin_layout(buf, 64)
    return list(buf[:n])


@pytest.mark.parametrize("which", ["own_header", "reference_header"])
def test_struct_layouts_agree_between_headers(which):
    """Every interface struct has the same size and last-member offset whichever header the caller was compiled with
    (the source also carries static_asserts on every member offset, so either build existing is already a check)."""
    got = layout(load(which))
    assert got == layout(load("own_header"))
    assert got[:6] == [48, 40, 80, 72, 56, 48] and got[-3:] == [8, 32, 1]


@pytest.mark.parametrize("which", ["own_header", "reference_header"])
@pytest.mark.parametrize("case", [1, 2, 3, 4, 5, 6, 7])
def test_reference_validation_cases_from_cxx(which, case, capfd):
    """gating_attention_nullptr_1..6 and gating_attention_negative_block_size of the reference's test file: handles that
    are not tensors, one null pointer or a negative block size.  The call must come back, say why on stderr and latch
    the error flag, all before any handle is looked into."""
    L = load(which)
    capi.clear_error()
    assert L.dropin_validation_case(case) == 0
    err = capfd.readouterr().err
    assert capi.error_flag()
    assert "KUTACC_CHECK fail in kutacc_af2_gating_attention" in err
    assert ("nullptr" in err) if case <= 6 else ("<= 0 or overflow" in err)
    capi.clear_error()


@pytest.mark.parametrize("which", ["own_header", "reference_header"])
def test_version_through_the_header_struct(which):
    assert load(which).dropin_component_name() == b"KuTACC"


def _ptr(t):
    return None if t is None else t.data_ptr()


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["own_header", "reference_header"])
@pytest.mark.parametrize("config,batch,seq", [(3, 12, 128), (4, 3, 200), (2, 9, 96)])
def test_cxx_caller_matches_ctypes_handle_path(which, config, batch, seq):
    """TensorWrapper handles made by the C++ constructor, the operator called from C++: `out` and the gated average
    equal, bit for bit, what the same call gives through kutacc_hip_tensor_create handles, and meet the parity bar
    against the oracle."""
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    L = load(which)
    capi.set_stream(None)
    capi.set_blocking(True)
    w = make_workload(config, batch=batch, seq_len=seq)
    print(f"{which}: config {config} B={batch} S={seq}", flush=True)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag()
    ten2, scratch2 = helpers.to_device(w)
    rc = L.dropin_gating_attention(_ptr(ten2["x"]), _ptr(scratch2["q"]), _ptr(scratch2["k"]), _ptr(scratch2["v"]),
                                   _ptr(scratch2["gate"]), _ptr(scratch2["avg"]), _ptr(ten2["bias"]), _ptr(ten2["nb"]),
                                   _ptr(ten2["wq"]), _ptr(ten2["wk"]), _ptr(ten2["wv"]), _ptr(ten2["wg"]), _ptr(ten2["bg"]),
                                   _ptr(ten2["wo"]), _ptr(ten2["bo"]), _ptr(ten2["out"]), w.B, w.S, w.H, w.d, 64)
    torch.cuda.synchronize()
    assert rc == 0 and not capi.error_flag()
    assert capi.last_path() == "fused_mfma"
    assert helpers.same_bits(ten2["out"], ten["out"]), "out differs from the ctypes-handle path"
    assert helpers.same_bits(scratch2["avg"], scratch["avg"]), "gated average differs from the ctypes-handle path"
    helpers.check_close(helpers.to_numpy(ten2["out"]), helpers.oracle_out(w), w.dtype, "out")


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["own_header", "reference_header"])
def test_cxx_caller_global_attention_and_transition(which):
    """The other two operators with struct arguments, called from C++ through TensorWrapper handles
    (kutacc_af2_global_attention, reference include/kutacc.h:292-307; kutacc_af2_transition, :194-214, 321-322): results
    equal the ctypes-handle path bit for bit."""
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    import test_gpu_global_attention as G
    import test_gpu_pair_stack as P
    L = load(which)
    capi.set_stream(None)
    capi.set_blocking(True)
    c = G.make_case(31, 5, 300, 8, 8, "random")
    op, ten, scratch = G.device_op(torch, c)
    op.run()
    assert not capi.error_flag()
    op2, ten2, scratch2 = G.device_op(torch, c)  # a second set of tensors; op2 itself is not run
    rc = L.dropin_global_attention(_ptr(ten2["x"]), _ptr(ten2["mask"]), _ptr(scratch2["q"]), _ptr(scratch2["k"]),
                                   _ptr(scratch2["v"]), _ptr(scratch2["gate"]), _ptr(scratch2["avg"]), _ptr(ten2["wq"]),
                                   _ptr(ten2["wk"]), _ptr(ten2["wv"]), _ptr(ten2["wg"]), _ptr(ten2["bg"]), _ptr(ten2["wo"]),
                                   _ptr(ten2["bo"]), _ptr(ten2["out"]), 5, 300, 8, 8)
    torch.cuda.synchronize()
    assert rc == 0 and not capi.error_flag() and capi.last_path() == "global_mfma"
    assert helpers.same_bits(ten2["out"], ten["out"]), "global attention: out differs from the ctypes-handle path"

    t = P.transition_case(77, 2, 90, 128, 512)
    want, _ = P.run_transition(torch, t)
    x, w1, w2 = (P.dev(torch, t[k]) for k in ("x", "w1", "w2"))
    b1, b2 = P.dev(torch, t["b1"], torch.float32), P.dev(torch, t["b2"], torch.float32)
    mid = torch.zeros((2 * 90, 512), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((2, 90, 128), dtype=torch.bfloat16, device="cuda")
    rc = L.dropin_transition(_ptr(x), _ptr(mid), _ptr(w1), _ptr(b1), _ptr(w2), _ptr(b2), _ptr(out), 2, 90, 128, 512)
    torch.cuda.synchronize()
    assert rc == 0 and not capi.error_flag()
    assert helpers.same_bits(out, want), "transition: out differs from the ctypes-handle path"


@pytest.mark.gpu
def test_prepacked_device_weights_feed_the_operator():
    """Weights that sit in a padded device buffer (leading dimension > k) go through kutacc_af2_linear_weight_prepack on
    the device, called from C++ with the header's default num_threads, and the packed copies are what the operator is
    given: the packed buffer equals the dense matrix bit for bit, its size is what kutacc_af2_gemm_pack_get_size says,
    and `out` equals a call on the original dense weights bit for bit."""
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    L = load("own_header")
    capi.set_stream(None)
    capi.set_blocking(True)
    w = make_workload(3, batch=9, seq_len=160)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag()
    C, pad = w.C, 24
    size = capi.lib().kutacc_af2_gemm_pack_get_size(b"B", b"N", b"N", 1, C, C)
    assert size == C * C
    ten2, scratch2 = helpers.to_device(w)
    for name in ("wq", "wk", "wv", "wg", "wo"):
        padded = torch.full((C, C + pad), 7.0, dtype=torch.bfloat16, device="cuda")
        padded[:, :C] = ten[name]
        packed = torch.zeros(size, dtype=torch.bfloat16, device="cuda")
        L.dropin_prepack(padded.data_ptr(), packed.data_ptr(), C, C, C + pad)
        assert not capi.error_flag()
        assert helpers.same_bits(packed.view(C, C), ten[name]), f"packed {name} differs from the dense matrix"
        ten2[name] = packed.view(C, C)
    op2 = capi.GatedAttention(ten2["x"], ten2["wq"], ten2["wk"], ten2["wv"], ten2["wg"], ten2["bg"], ten2["wo"], ten2["bo"],
                              ten2["bias"], ten2["nb"], w.H, ten2["out"], scratch2, block_size=64)
    op2.run()
    assert not capi.error_flag()
    assert helpers.same_bits(ten2["out"], ten["out"])
    helpers.check_close(helpers.to_numpy(ten2["out"]), helpers.oracle_out(w), w.dtype, "out with prepacked weights")
