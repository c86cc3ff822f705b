"""kutacc_hip_gating_attention_static -- the entry point that allocates nothing and keeps the fragment-major pair bias
in a device array of the library image -- against kutacc_hip_gating_attention on the same inputs, through the C ABI.

Where the batch is large enough for the existing entry point to keep its copy of the pair bias in the caller's q
tensor, both run the same kernels on the same data and `out` and the gated average must agree bit for bit; with a
smaller batch the existing entry point reads the pair bias in place (another softmax formulation) and the two are
compared at the parity bar.  Every result is also held to that bar against the CPU oracle (bf16: 2e-2 absolute +
1e-2 relative of the fp32 oracle).  The calls come in a row on one stream, each smaller than the one before, so that
a call which read what an earlier, larger call left in the shared array would show.
"""
import ctypes

import pytest

from kutacc_amd import capi
from kutacc_amd.workloads import make_workload

import helpers

pytestmark = pytest.mark.gpu


def _run_pair(torch, config, batch, seq, same_route):
    w = make_workload(config, batch=batch, seq_len=seq)
    print(f"static scratch: config {config} B={batch} S={seq}", flush=True)
    ten, scratch = helpers.to_device(w)
    rc = helpers.run_hip(w, ten, scratch, capi.PATH_FUSED)
    assert rc == 0, rc
    assert capi.last_path() == "fused_mfma"

    ten2, scratch2 = helpers.to_device(w)
    a = helpers.hip_args(w, ten2, scratch2, capi.PATH_FUSED)
    a.q = a.k = a.v = a.gate = None  # the entry point must not need them
    rc = capi.lib().kutacc_hip_gating_attention_static(ctypes.byref(a), None)
    torch.cuda.synchronize()
    assert rc == 0, rc
    if same_route:
        assert helpers.same_bits(scratch2["avg"], scratch["avg"]), "gated average differs from the existing entry point"
        assert helpers.same_bits(ten2["out"], ten["out"]), "out differs from the existing entry point"
    else:
        helpers.check_close(helpers.to_numpy(ten2["out"]), helpers.to_numpy(ten["out"]), w.dtype, "out vs existing entry")
    for name in ("q", "k", "v", "gate"):
        assert not bool(scratch2[name].any()), f"{name} was written"
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch2["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, "gated average")
    helpers.check_close(helpers.to_numpy(ten2["out"]), ref_out, w.dtype, "out")


def test_static_scratch_entry_matches_existing_entry_on_shrinking_calls():
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    capi.set_stream(None)
    capi.set_blocking(True)
    # persistent kernel with pair bias (4 and 8 heads), then smaller calls: ragged length, long-sequence kernel, and one
    # without pair bias (no scratch use at all)
    cases = [(3, 12, 384, True), (3, 10, 200, True), (2, 9, 256, True), (5, 20, 520, True), (5, 3, 520, False),
             (3, 4, 33, True), (3, 2, 33, False), (4, 3, 300, True)]
    for config, batch, seq, same_route in cases:
        _run_pair(torch, config, batch, seq, same_route)


def test_static_scratch_entry_rejects_what_it_cannot_run():
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    w = make_workload(1, batch=2, seq_len=16)  # fp32 storage: not a shape of the MFMA kernels
    ten, scratch = helpers.to_device(w)
    a = helpers.hip_args(w, ten, scratch)
    assert capi.lib().kutacc_hip_gating_attention_static(ctypes.byref(a), None) == capi.EUNSUPPORTED
    assert capi.lib().kutacc_hip_gating_attention_static(None, None) == capi.EINVAL
    assert not bool(ten["out"].any())


def test_static_scratch_entry_allocates_nothing_and_records_no_events():
    """After one warm-up call per shape, a run of calls with per-kernel profiling switched on leaves the device's free
    memory where it was (hipMemGetInfo) and adds no entry to the profile (no events are created for this entry)."""
    import torch
    assert torch.cuda.is_available(), "this test needs the GPU"
    capi.set_stream(None)
    lib = capi.lib()
    w = make_workload(3, batch=12, seq_len=384)
    ten, scratch = helpers.to_device(w)
    a = helpers.hip_args(w, ten, scratch, capi.PATH_FUSED)
    a.q = a.k = a.v = a.gate = None
    assert lib.kutacc_hip_gating_attention_static(ctypes.byref(a), None) == 0  # warm-up: symbol address, LDS opt-in
    torch.cuda.synchronize()
    want = ten["out"].clone()

    def profile_entries():
        name = ctypes.create_string_buffer(128)
        ms, launches, flops = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double()
        n = 0
        while lib.kutacc_hip_profile_read(n, name, 128, ctypes.byref(ms), ctypes.byref(launches), ctypes.byref(flops)) == 0:
            n += 1
        return n

    lib.kutacc_hip_profile_enable(1)
    try:
        entries_before = profile_entries()
        free_before, _ = torch.cuda.mem_get_info()
        for _ in range(20):
            assert lib.kutacc_hip_gating_attention_static(ctypes.byref(a), None) == 0
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert free_after == free_before, (free_before, free_after)
        assert profile_entries() == entries_before
    finally:
        lib.kutacc_hip_profile_enable(0)
    assert helpers.same_bits(ten["out"], want)
