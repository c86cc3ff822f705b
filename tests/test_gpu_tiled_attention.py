"""The tiled MFMA route of the gated-attention operator (kutacc_amd/csrc/tiled_attention.hip): the bf16 shapes the fused
head kernels do not take -- rows longer than 1024 positions, head sizes other than 32, channel counts other than 128 and
256 -- against the fp32 oracle, to the bf16 bar (2e-2 absolute + 1e-2 relative); the scratch tensors it leaves against
the oracle's bf16 model of the reference (reference src/attention/gating_attention.cpp:47-66)."""
import numpy as np
import pytest

import helpers
from kutacc_amd import capi
from kutacc_amd.workloads import MASK_BIAS, Workload, layernorm_np, make_workload, round_to_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.set_stream(None)
    capi.set_blocking(True)
    return torch


def draw_workload(seed, B, S, H, d, pair_bias=True, masked=0.1, nb_scale=1.0) -> Workload:
    """A seeded problem of any head size: layer-normalised input rows, weights of variance 1 / fan_in, a key mask on
    about `masked` of the positions (never the first), a pair bias of standard deviation `nb_scale`."""
    rng = np.random.Generator(np.random.PCG64(seed))
    C = H * d
    x = round_to_bf16(layernorm_np(round_to_bf16(rng.standard_normal((B, S, C), dtype=np.float32))))
    weight = lambda: round_to_bf16(rng.standard_normal((C, C), dtype=np.float32) / np.float32(np.sqrt(C)))  # noqa: E731
    wq, wk, wv, wg, wo = (weight() for _ in range(5))
    bg = np.ones(C, dtype=np.float32) + 0.1 * rng.standard_normal(C, dtype=np.float32)
    bo = 0.1 * rng.standard_normal(C, dtype=np.float32)
    keep = rng.random((B, S)) >= masked
    keep[:, 0] = True
    bias = round_to_bf16((MASK_BIAS * (1.0 - keep.astype(np.float32))))
    nb = round_to_bf16(nb_scale * rng.standard_normal((H, S, S), dtype=np.float32)) if pair_bias else None
    return Workload(0, f"drawn B={B} S={S} H={H} d={d}", "bf16", B, S, H, d, x, wq, wk, wv, wg, wo, bg, bo, bias, nb)


def run_and_check(w, path=capi.PATH_AUTO, expect="tiled_mfma"):
    print(f"{w.name} path={path}", flush=True)
    ten, scratch = helpers.to_device(w)
    rc = helpers.run_hip(w, ten, scratch, path)
    assert rc == 0 and capi.last_path() == expect, (rc, capi.last_path())
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, "bf16", "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, "bf16", "out")
    return ten, scratch


@pytest.mark.parametrize("B,S,H,d", [
    (3, 200, 8, 8),    # the extra-MSA shape: 64 channels, head size 8 (one k-step, half of it padding)
    (2, 150, 4, 16),   # the template stack's: head size 16
    (2, 96, 3, 24),    # two k-steps, the second half padding; 72 channels
    (1, 70, 3, 40),    # three k-steps, two blocks of values
    (2, 100, 2, 64),   # four k-steps
    (2, 130, 4, 32),   # a shape the fused kernels take as well, forced onto this route
    (9, 64, 2, 32),    # one whole chunk of keys; nine batch rows: a second group of rows with one member
    (2, 65, 2, 32),    # one key into the second chunk
    (1, 1, 2, 32),     # a single position
    (2, 77, 8, 8),     # a length that is no multiple of 8: the rows of v and of the pair bias are read element by element
    (3, 1000, 5, 16),  # eight query blocks, sixteen chunks, 80 channels
])
def test_shapes_beyond_the_fused_kernels(torch_cuda, B, S, H, d):
    w = draw_workload(100 * d + S, B, S, H, d)
    run_and_check(w, capi.PATH_TILED)
    if d != 32 or H * d not in (128, 256):
        run_and_check(w, capi.PATH_AUTO)   # the automatic choice comes here too ...
        run_and_check(w, capi.PATH_FUSED)  # ... and "MFMA kernels only" includes this route


@pytest.mark.parametrize("B,S,H,d", [(2, 1536, 4, 32), (9, 1100, 4, 32), (1, 2048, 8, 8)])
def test_rows_longer_than_1024_positions(torch_cuda, B, S, H, d):
    """Twelve, nine and sixteen query blocks (a second group of query blocks), 24 / 18 / 32 key chunks; the first two are
    triangle-attention shapes past the fused kernels' longest row."""
    w = draw_workload(7 + S, B, S, H, d)
    run_and_check(w, capi.PATH_AUTO)


@pytest.mark.parametrize("B,S,H,d", [(2048, 2048, 4, 32), (5120, 384, 8, 8)])
def test_benchmarked_shapes_on_sampled_rows(torch_cuda, B, S, H, d):
    """The shapes `bench.py --tiled-route` times (triangle attention at 2048 residues, the extra-MSA row attention), drawn
    on the device: the oracle on a sample of batch rows -- first and last, both sides of the 8-row groups the kernel's
    placement forms, one fully masked -- and finiteness of every other entry."""
    import ctypes
    torch = torch_cuda
    C = H * d
    g = torch.Generator(device="cuda").manual_seed(4000 + S)
    bf = lambda *sh, scale=1.0: (torch.randn(*sh, device="cuda", generator=g) * scale).to(torch.bfloat16)  # noqa: E731
    x = torch.nn.functional.layer_norm(torch.randn(B, S, C, device="cuda", generator=g), (C,)).to(torch.bfloat16)
    ws = [bf(C, C, scale=C ** -0.5) for _ in range(5)]
    bg, bo = torch.ones(C, device="cuda"), torch.randn(C, device="cuda", generator=g) * 0.1
    keep = torch.rand(B, S, device="cuda", generator=g) >= 0.1
    keep[:, 0] = True
    bias = ((~keep).float() * MASK_BIAS).to(torch.bfloat16)
    rows = sorted({0, 1, 7, 8, 9, B // 2 - 1, B // 2, B - 9, B - 8, B - 2, B - 1})
    bias[rows[3], :] = MASK_BIAS  # a fully masked row: a uniform average
    nb = bf(H, S, S)
    out = torch.empty(B, S, C, device="cuda", dtype=torch.bfloat16)
    q, k, gate, avg = (torch.empty(B, S, C, device="cuda", dtype=torch.bfloat16) for _ in range(4))
    v = torch.empty(C, B * S, device="cuda", dtype=torch.bfloat16)
    a = capi.HipAttentionArgs()
    a.batch, a.seq_len, a.nheads, a.head_size, a.dtype, a.path = B, S, H, d, capi.K_BF16, capi.PATH_AUTO
    a.input, a.input_ld = x.data_ptr(), C
    a.query_w, a.key_w, a.value_w, a.gating_w, a.output_w = (w.data_ptr() for w in ws)
    a.gating_b, a.output_b = bg.data_ptr(), bo.data_ptr()
    a.bias, a.bias_stride_b = bias.data_ptr(), S
    a.nonbatched_bias, a.nb_stride_h, a.nb_stride_q = nb.data_ptr(), S * S, S
    a.q, a.k, a.v, a.gate, a.avg = q.data_ptr(), k.data_ptr(), v.data_ptr(), gate.data_ptr(), avg.data_ptr()
    for n in ("q", "k", "gate", "avg"):
        setattr(a, f"{n}_stride_b", S * C), setattr(a, f"{n}_stride_s", C), setattr(a, f"{n}_stride_h", d)
    a.v_stride_h, a.v_stride_e, a.v_stride_b = d * B * S, B * S, S
    a.out, a.out_ld = out.data_ptr(), C
    print(f"B={B} S={S} H={H} d={d}", flush=True)
    assert capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None) == 0
    torch.cuda.synchronize()
    assert capi.last_path() == "tiled_mfma"
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(avg).all())
    from oracle import oracle
    num = lambda t: helpers.to_numpy(t)  # noqa: E731
    ref_out, ref_avg = oracle.gating_attention_f32(num(x[rows]), *(num(w) for w in ws[:4]), num(bg), num(ws[4]), num(bo),
                                                   num(bias[rows]), num(nb), H, return_avg=True)
    helpers.check_close(num(avg[rows]), ref_avg, "bf16", f"gated average, sampled rows of B={B} S={S}")
    helpers.check_close(num(out[rows]), ref_out, "bf16", f"out, sampled rows of B={B} S={S}")


def test_without_pair_bias_and_with_fully_masked_rows(torch_cuda):
    w = draw_workload(5, 4, 300, 8, 8, pair_bias=False)
    w.bias[1, :] = round_to_bf16(np.full(w.S, MASK_BIAS, dtype=np.float32))  # every key of row 1 masked: a uniform average
    run_and_check(w)
    w = draw_workload(6, 3, 1200, 4, 32, pair_bias=True, masked=0.5)
    w.bias[2, :] = round_to_bf16(np.full(w.S, MASK_BIAS, dtype=np.float32))
    run_and_check(w)


def test_large_pair_bias_and_logit_offsets(torch_cuda):
    """A pair bias of standard deviation 10 (what a trained pair representation reaches) and rows whose logits sit
    150 above or below zero: the running maximum absorbs both."""
    w = draw_workload(8, 3, 260, 4, 16, nb_scale=10.0)
    w.nb[:, 5, :] += np.float32(150.0)
    w.nb[:, 9, :] -= np.float32(150.0)
    w.nb = round_to_bf16(w.nb)
    run_and_check(w)


def test_pair_bias_entries_of_minus_infinity(torch_cuda):
    """Pairs excluded by a -inf pair bias get zero weight; a row keeps at least one finite key."""
    w = draw_workload(9, 2, 140, 4, 16)
    rng = np.random.Generator(np.random.PCG64(99))
    drop = rng.random(w.nb.shape) < 0.3
    drop[:, :, 0] = False
    w.nb[drop] = -np.inf
    run_and_check(w)


def test_matches_the_fused_kernels_where_both_run(torch_cuda):
    """Config 3 at 384 positions on both routes: each within the bar of the oracle (checked elsewhere), and within the bar
    of each other on every batch row."""
    import torch
    w = make_workload(3, batch=24)
    ten, scratch = helpers.to_device(w)
    assert helpers.run_hip(w, ten, scratch, capi.PATH_TILED) == 0 and capi.last_path() == "tiled_mfma"
    ten2, scratch2 = helpers.to_device(w)
    assert helpers.run_hip(w, ten2, scratch2, capi.PATH_FUSED) == 0 and capi.last_path() == "fused_mfma"
    a, b = ten["out"].float(), ten2["out"].float()
    assert bool(torch.isfinite(a).all())
    assert float(((a - b).abs() - (2e-2 + 1e-2 * b.abs())).max()) <= 0.0


def test_leaves_q_k_v_gate_as_the_reference_does(torch_cuda):
    """q, k, gate as [B, S, H, d] and v as [H, d, B, S], rounded to bf16 where the reference stores them; the oracle's bf16
    model of the reference holds the same tensors."""
    from oracle import oracle
    w = draw_workload(11, 3, 90, 4, 16)
    ten, scratch = run_and_check(w)
    bits = lambda a: oracle.to_bf16_bits(np.asarray(a, dtype=np.float32))  # noqa: E731
    _, ref = oracle.gating_attention_bf16(bits(w.x), bits(w.wq), bits(w.wk), bits(w.wv), bits(w.wg), w.bg, bits(w.wo), w.bo,
                                          bits(w.bias), bits(w.nb), w.H, return_scratch=True)
    for name in ("q", "k", "gate"):
        got = helpers.to_numpy(scratch[name]).reshape(w.B, w.S, w.C)
        helpers.check_close(got, oracle.from_bf16_bits(ref[name]).reshape(w.B, w.S, w.C), "bf16", name)
    helpers.check_close(helpers.to_numpy(scratch["v"]), oracle.from_bf16_bits(ref["v"]), "bf16", "v")


def test_replays_from_a_hip_graph(torch_cuda):
    """The route's seven launches (five products, the attention, nothing that allocates, clears memory or synchronises)
    captured into a HIP graph on a side stream and replayed three times, with eager work between the replays (the results
    and the scratch tensors overwritten); every replay reproduces the eager result bit for bit."""
    import ctypes
    torch = torch_cuda
    w = draw_workload(21, 5, 200, 8, 8)
    ten, scratch = helpers.to_device(w)
    a = helpers.hip_args(w, ten, scratch, capi.PATH_TILED)
    assert capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None) == 0  # eager: also takes first-call set-up out of the capture
    torch.cuda.synchronize()
    want_out, want_avg = ten["out"].clone(), scratch["avg"].clone()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), torch.cuda.current_stream().cuda_stream) == 0
    for _ in range(3):
        ten["out"].fill_(7.0)
        for t in scratch.values():
            t.fill_(-3.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert helpers.same_bits(ten["out"], want_out) and helpers.same_bits(scratch["avg"], want_avg)


def test_unsupported_layouts_fall_back_to_the_generic_kernels(torch_cuda):
    """A head size that is no multiple of 8 is not this route's: the automatic choice takes the scalar kernels, the forced
    routes refuse."""
    w = draw_workload(12, 2, 50, 4, 12)
    ten, scratch = helpers.to_device(w)
    assert helpers.run_hip(w, ten, scratch, capi.PATH_TILED) == capi.EUNSUPPORTED
    assert helpers.run_hip(w, ten, scratch, capi.PATH_FUSED) == capi.EUNSUPPORTED
    assert helpers.run_hip(w, ten, scratch, capi.PATH_AUTO) == 0 and capi.last_path() == "generic"
    helpers.check_close(helpers.to_numpy(ten["out"]), helpers.oracle_out(w), "bf16", "out")


def test_handle_based_entry_point_takes_the_route(torch_cuda):
    """kutacc_af2_gating_attention with 64 channels and head size 8 (device tensors), and the same call on host pointers
    (staged): same bits."""
    w = draw_workload(13, 4, 120, 8, 8)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag() and capi.last_path() == "tiled_mfma"
    helpers.check_close(helpers.to_numpy(ten["out"]), helpers.oracle_out(w), "bf16", "out")
    hten, hscratch = helpers.host_arrays(w)
    hop = capi.GatedAttention(hten["x"], hten["wq"], hten["wk"], hten["wv"], hten["wg"], hten["bg"], hten["wo"], hten["bo"],
                              hten["bias"], hten["nb"], w.H, hten["out"], hscratch)
    hop.run()
    assert not capi.error_flag() and capi.last_path() == "tiled_mfma"
    np.testing.assert_array_equal(hten["out"], ten["out"].view(torch_cuda.int16).cpu().numpy().view(np.uint16))
