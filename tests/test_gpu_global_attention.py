"""GPU parity of kutacc_af2_global_attention (reference src/attention/global_attention.cpp:30-205) against the CPU
oracle, through the C ABI.  bf16 storage; tolerance as for the gated attention: 2e-2 absolute + 1e-2 relative
against the fp32 oracle on the same bf16-rounded inputs."""
import math
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import helpers  # noqa: E402
from kutacc_amd import capi  # noqa: E402
from kutacc_amd.workloads import round_to_bf16  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    capi.lib()
    return torch


def make_case(seed, B, S, H, d, mask_mode="random"):
    rng = np.random.Generator(np.random.PCG64(seed))
    C = H * d
    f = lambda *s: round_to_bf16(rng.standard_normal(s).astype(np.float32))  # noqa: E731
    w = lambda *s: round_to_bf16((rng.standard_normal(s) / math.sqrt(s[-1])).astype(np.float32))  # noqa: E731
    mask = np.ones((B, S), dtype=np.float32)
    if mask_mode == "random":
        mask = (rng.random((B, S)) > 0.25).astype(np.float32)
        mask[:, 0] = 1
        if B > 2:
            mask[B - 1] = 0  # one row with every token masked
    return dict(x=f(B, S, C), mask=mask, wq=w(C, C), wk=w(d, C), wv=w(d, C), wg=w(C, C),
                bg=np.ones(C, dtype=np.float32), wo=w(C, C), bo=rng.standard_normal(C).astype(np.float32), nheads=H)


def oracle_out(c):
    from oracle import oracle
    return oracle.global_attention_f32(c["x"], c["mask"], c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"], c["bo"],
                                       c["nheads"], return_q_avg=True)


def device_op(torch, c, device="cuda"):
    B, S, C = c["x"].shape
    d = C // c["nheads"]
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).to(device)  # noqa: E731
    f32 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)  # noqa: E731
    ten = dict(x=bf(c["x"]), mask=bf(c["mask"].reshape(B, S, 1)), wq=bf(c["wq"]), wk=bf(c["wk"]), wv=bf(c["wv"]),
               wg=bf(c["wg"]), bg=f32(c["bg"]), wo=bf(c["wo"]), bo=f32(c["bo"]),
               out=torch.zeros((B, S, C), dtype=torch.bfloat16, device=device))
    z = lambda *s: torch.zeros(s, dtype=torch.bfloat16, device=device)  # noqa: E731
    scratch = dict(q=z(B, C), k=z(B * S, d), v=z(d, B * S), gate=z(B, S, C), avg=z(B, C))
    op = capi.GlobalAttention(ten["x"], ten["mask"], ten["wq"], ten["wk"], ten["wv"], ten["wg"], ten["bg"], ten["wo"],
                              ten["bo"], c["nheads"], ten["out"], scratch)
    return op, ten, scratch


SHAPES = [
    # B, S, H, d, mask
    (4, 128, 8, 8, "random"), (3, 97, 8, 8, "random"), (2, 1024, 8, 8, "random"), (5, 33, 4, 16, "random"),
    (2, 200, 2, 32, "ones"), (3, 1, 8, 8, "ones"), (6, 7, 16, 4, "random"), (2, 1500, 8, 8, "random"),
    # both workgroup sizes of the kernel: eight waves while a row has a CU to itself (at most 256 rows) or is streamed,
    # four when two rows share a CU
    (300, 512, 8, 8, "random"), (257, 1024, 4, 16, "random"), (256, 640, 8, 8, "random"), (3, 2100, 4, 16, "random"),
    # streamed rows on either side of what the eight-wave layout's LDS holds (7808 positions), and the longest row
    (2, 7808, 8, 8, "random"), (2, 8192, 8, 8, "random"), (1, 12288, 8, 8, "random"),
]


@pytest.mark.parametrize("B,S,H,d,mask_mode", SHAPES)
def test_global_attention_matches_oracle(torch_cuda, B, S, H, d, mask_mode):
    c = make_case(100 + S, B, S, H, d, mask_mode)
    op, ten, scratch = device_op(torch_cuda, c)
    op.run()
    assert not capi.error_flag() and capi.last_path() == "global_mfma"
    rows = list(range(B)) if B <= 8 else sorted({0, 1, B // 2, B - 2, B - 1})  # large batches: the oracle on a few rows
    ref, ref_qavg = oracle_out(dict(c, x=c["x"][rows], mask=c["mask"][rows]))
    helpers.check_close(helpers.to_numpy(ten["out"][rows]), ref, "bf16", "global attention out")
    helpers.assert_within(helpers.to_numpy(scratch["avg"][rows]), ref_qavg, 2.0 ** -8 * np.abs(ref_qavg) + 1e-6, "masked mean q_avg")


def test_global_attention_full_extra_msa_shape(torch_cuda):
    """An extra-MSA sized call (N_res = 256 batch rows of 1024 extra sequences): spot-check rows against the oracle."""
    c = make_case(7, 256, 1024, 8, 8, "random")
    op, ten, _ = device_op(torch_cuda, c)
    op.run()
    assert not capi.error_flag()
    rows = [0, 100, 255]
    sub = dict(c, x=c["x"][rows], mask=c["mask"][rows])
    ref, _ = oracle_out(sub)
    helpers.check_close(helpers.to_numpy(ten["out"][rows]), ref, "bf16", "global attention, extra-MSA shape")


def test_global_attention_host_pointers_match_device_pointers(torch_cuda):
    c = make_case(9, 3, 70, 8, 8)
    op, ten, scratch = device_op(torch_cuda, c)
    op.run()
    from kutacc_amd.workloads import bf16_bits
    B, S, C = c["x"].shape
    hb = lambda a: bf16_bits(np.ascontiguousarray(a))  # noqa: E731
    hten = dict(x=hb(c["x"]), mask=hb(c["mask"].reshape(B, S, 1)), wq=hb(c["wq"]), wk=hb(c["wk"]), wv=hb(c["wv"]),
                wg=hb(c["wg"]), bg=c["bg"].copy(), wo=hb(c["wo"]), bo=c["bo"].copy(), out=np.zeros((B, S, C), np.uint16))
    hz = lambda *s: np.zeros(s, dtype=np.uint16)  # noqa: E731
    hscratch = dict(q=hz(B, C), k=hz(B * S, 8), v=hz(8, B * S), gate=hz(B, S, C), avg=hz(B, C))
    hop = capi.GlobalAttention(hten["x"], hten["mask"], hten["wq"], hten["wk"], hten["wv"], hten["wg"], hten["bg"],
                               hten["wo"], hten["bo"], 8, hten["out"], hscratch)
    hop.run()
    assert not capi.error_flag()
    out_bits = ten["out"].view(torch_cuda.int16).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(hten["out"], out_bits)
    np.testing.assert_array_equal(hscratch["avg"], scratch["avg"].view(torch_cuda.int16).cpu().numpy().view(np.uint16))


def test_global_attention_rejects_other_channel_counts(torch_cuda, capfd):
    c = make_case(3, 2, 16, 4, 8)  # 32 channels
    op, ten, _ = device_op(torch_cuda, c)
    op.run()
    assert capi.error_flag()
    assert "invalid int value" in capfd.readouterr().err


def test_global_attention_rejects_rows_beyond_the_lds(torch_cuda):
    c = make_case(5, 1, 12320, 8, 8)
    op, ten, _ = device_op(torch_cuda, c)
    op.run()
    assert capi.error_flag()
    capi.clear_error()
