#!/usr/bin/env python3
"""Benchmark of the fused gated-attention operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--no-cpu]

A "step" is one kutacc_af2_gating_attention call on device-resident synthetic inputs of the chosen
configuration (default: config 3, the N_res=384 triangle-attention shape the headline metric is
quoted on).  Prints ONE JSON line: whole-call TFLOP/s from algorithmic flops
(10*B*S*C^2 + 4*B*S^2*C), ms per call, the roofline of the dominant kernel (live hipEvent timing on
the launch stream, read back through kutacc_hip_profile_*) and a CPU baseline (the bf16
restatement of the reference algorithm in oracle/, timed on this host on a bounded batch sample).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

MFMA_BF16_PEAK_TFLOPS = 2516.6  # 256 CU x 2.4 GHz x 4096 flop/clk/CU, dense
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of each kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this same command, each
# counter scaled by what it reads for a 256 MiB copy (profiles/gating_attention_hbm_traffic.txt says how): the file maps
# "config N" -> kernel name -> bytes.  Not re-measured live; a kernel or configuration without an entry reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


SETTLE_SECONDS = 0.3  # untimed calls ahead of the warm-up steps, see main()


def measured_traffic(config, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    v = table.get(f"config {config}", {}).get(kernel)
    return int(v) if v is not None else None


def cpu_baseline(w, budget_s=15.0):
    """Time oracle Rbf16 (reference rounding points, OpenMP on all host cores) on the first rows of the
    batch; rows are independent, so throughput on the sample is throughput on the whole batch."""
    import numpy as np
    from oracle import oracle
    from kutacc_amd.workloads import bf16_bits

    def run(nrows):
        sub = w.batch_slice(np.arange(nrows))
        b = bf16_bits
        args = (b(sub.x), b(sub.wq), b(sub.wk), b(sub.wv), b(sub.wg), sub.bg, b(sub.wo), sub.bo, b(sub.bias),
                None if sub.nb is None else b(sub.nb), sub.H)
        t0 = time.perf_counter()
        oracle.gating_attention_bf16(*args, block_size=64, exp_mode=1)
        return time.perf_counter() - t0, sub.flops()

    probe = min(w.B, max(2, oracle.num_threads() // w.H + 1))
    t_probe, _ = run(probe)
    rows = int(min(w.B, max(probe, probe * budget_s / max(t_probe, 1e-3))))
    t, fl = run(rows)
    return {
        "value": round(fl / t / 1e12, 5), "unit": "TFLOP/s", "cores": oracle.num_threads(), "kind": "port",
        "sample": f"first {rows} of {w.B} batch rows of the same workload, one call, {t:.2f} s "
                  f"(= {t / rows * w.B * 1e3:.0f} ms/call extrapolated to the full batch)",
    }


def producer_rates(config, reps=50):
    """Achieved HBM rates of the HBM-bound kernels around the operator: the two row kernels in front of it, at this
    configuration's pair tensor z [S, S, 128] (LayerNorm over all rows; the fused LN -> [H, c_z] projection ->
    [H, S, S] pair bias, with and without writing the normalised z), and the global (extra-MSA column) attention.
    Algorithmic bytes: rows*c_z*2 read plus what is written (rows*c_z*2 for LN / z_norm, rows*H*2 for the pair bias);
    for the global attention its input read once and its output written once."""
    import numpy as np
    import torch
    from kutacc_amd import capi
    from kutacc_amd.workloads import make_workload

    w = make_workload(config, batch=2, keep_extras=True)
    if "z" not in w.extras:
        return None
    z, wb = w.extras["z"], w.extras["w_bias"]
    S, cz, H = z.shape[0], z.shape[-1], wb.shape[0]
    dz = torch.from_numpy(z).cuda().to(torch.bfloat16)
    dw = torch.from_numpy(wb).cuda().to(torch.bfloat16)
    dg = torch.ones(cz, device="cuda", dtype=torch.float32)
    db = torch.zeros(cz, device="cuda", dtype=torch.float32)
    nb = torch.empty((H, S, S), device="cuda", dtype=torch.bfloat16)
    zn = torch.empty_like(dz)
    L = capi.lib()
    rows = S * S
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn):
        for _ in range(5):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps * 1e-3

    t_ln = timed(lambda: L.kutacc_hip_layernorm_rows(dz.data_ptr(), cz, dg.data_ptr(), db.data_ptr(), zn.data_ptr(), cz,
                                                     rows, cz, 1e-5, capi.K_BF16, stream))
    t_pb = timed(lambda: L.kutacc_hip_pair_bias(dz.data_ptr(), dg.data_ptr(), db.data_ptr(), dw.data_ptr(), nb.data_ptr(),
                                                None, S, S, cz, H, 1e-5, capi.K_BF16, stream))
    t_pbz = timed(lambda: L.kutacc_hip_pair_bias(dz.data_ptr(), dg.data_ptr(), db.data_ptr(), dw.data_ptr(), nb.data_ptr(),
                                                 zn.data_ptr(), S, S, cz, H, 1e-5, capi.K_BF16, stream))
    zb = rows * cz * 2

    # global (extra-MSA column) attention at an extra-MSA sized call: N_res batch rows of 1024 extra sequences, 64 channels
    import math
    gB, gS, gH, gd = (256 if config != 5 else 384), 1024, 8, 8
    g = torch.Generator(device="cuda").manual_seed(5)
    rnd = lambda *sh: torch.randn(*sh, device="cuda", generator=g)  # noqa: E731
    gx = rnd(gB, gS, 64).to(torch.bfloat16)
    gmask = (torch.rand(gB, gS, 1, device="cuda", generator=g) > 0.25).to(torch.bfloat16)
    gw = {n: (rnd(*sh) / math.sqrt(64)).to(torch.bfloat16)
          for n, sh in (("wq", (64, 64)), ("wk", (gd, 64)), ("wv", (gd, 64)), ("wg", (64, 64)), ("wo", (64, 64)))}
    gbg, gbo = torch.ones(64, device="cuda"), torch.zeros(64, device="cuda")
    gout = torch.empty_like(gx)
    gz = lambda *sh: torch.empty(sh, device="cuda", dtype=torch.bfloat16)  # noqa: E731
    gop = capi.GlobalAttention(gx, gmask, gw["wq"], gw["wk"], gw["wv"], gw["wg"], gbg, gw["wo"], gbo, gH, gout,
                               dict(q=gz(gB, 64), k=gz(gB * gS, gd), v=gz(gd, gB * gS), gate=gz(gB, gS, 64), avg=gz(gB, 64)))
    capi.set_stream(stream)
    capi.set_blocking(False)
    t_ga = timed(gop.run)
    capi.set_blocking(True)
    capi.set_stream(None)
    assert not capi.error_flag()
    return {
        "global_attention": {"shape": f"B={gB} S={gS} C=64 H={gH}", "us": round(t_ga * 1e6, 2),
                             "GB/s": round(2 * gB * gS * 64 * 2 / t_ga / 1e9, 1)},
        "shape": f"z [{S},{S},{cz}] bf16, H={H}",
        "layernorm_rows": {"us": round(t_ln * 1e6, 2), "GB/s": round(2 * zb / t_ln / 1e9, 1)},
        "pair_bias": {"us": round(t_pb * 1e6, 2), "GB/s": round((zb + rows * H * 2) / t_pb / 1e9, 1)},
        "pair_bias_with_z_norm": {"us": round(t_pbz * 1e6, 2), "GB/s": round((2 * zb + rows * H * 2) / t_pbz / 1e9, 1)},
        "hbm_peak_GB/s": HBM_PEAK_GBS,
    }


def pair_stack_rates(config, reps=20):
    """Times of the transition and of the four steps of the triangle multiplication (outgoing and incoming equation)
    at this configuration's pair tensor: n = S residues, 128 pair channels, 128 projected channels, hidden layer 512.
    Called through the handle-based entry points, asynchronously on torch's stream, hipEvent-bracketed.  Per step:
    microseconds, algorithmic TFLOP/s (2 flops per multiply-add of the products) and algorithmic GB/s (every operand
    and result of the step once)."""
    import torch
    from kutacc_amd import capi
    from kutacc_amd.workloads import CONFIGS

    n = CONFIGS[config]["S"]
    c_o, c_i, hid = 128, 128, 512
    rows = n * n
    g = torch.Generator(device="cuda").manual_seed(11)
    bf = lambda *sh, scale=1.0: (torch.randn(*sh, device="cuda", generator=g) * scale).to(torch.bfloat16)  # noqa: E731
    f32 = lambda k: torch.randn(k, device="cuda", generator=g) * 0.5  # noqa: E731
    x = bf(n, n, c_o)
    mask = (torch.rand(n, n, device="cuda", generator=g) > 0.1).to(torch.bfloat16)
    stream = torch.cuda.current_stream().cuda_stream
    capi.set_stream(stream)
    capi.set_blocking(False)

    def timed(fn):
        for _ in range(3):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        assert not capi.error_flag()
        return e0.elapsed_time(e1) / reps * 1e-3

    res = {"shape": f"pair activation [{n},{n},{c_o}] bf16, c_i={c_i}, transition hidden {hid}"}

    def report(name, t, flops, nbytes):
        res[name] = {"us": round(t * 1e6, 1), "TFLOP/s": round(flops / t / 1e12, 1), "GB/s": round(nbytes / t / 1e9, 1)}

    # transition
    mid = torch.empty(rows, hid, device="cuda", dtype=torch.bfloat16)
    out = torch.empty(n, n, c_o, device="cuda", dtype=torch.bfloat16)
    tr = capi.Transition(x, bf(hid, c_o, scale=c_o ** -0.5), f32(hid), bf(c_o, hid, scale=hid ** -0.5), f32(c_o), mid, out)
    report("transition", timed(tr.run), 4.0 * rows * c_o * hid, 2.0 * rows * 2 * c_o)  # input and output; the hidden layer stays on chip
    del mid
    # the whole block in place: act += transition(LN(act)), one kernel
    zb = x.clone().reshape(rows, c_o)
    gam, bet = torch.ones(c_o, device="cuda"), torch.zeros(c_o, device="cuda")
    tw1, tb1, tw2, tb2 = bf(hid, c_o, scale=c_o ** -0.5), f32(hid), bf(c_o, hid, scale=hid ** -0.5) * 0.1, f32(c_o) * 0.1

    def run_tb():
        assert capi.lib().kutacc_hip_transition_block(zb.data_ptr(), gam.data_ptr(), bet.data_ptr(), 1e-5, tw1.data_ptr(),
                                                      tb1.data_ptr(), tw2.data_ptr(), tb2.data_ptr(), None, 0, rows, c_o, hid,
                                                      capi.K_BF16, stream) == 0
    report("transition_block (LN + transition + residual)", timed(run_tb), 4.0 * rows * c_o * hid, 2.0 * rows * 2 * c_o)
    # triangle multiplication
    keep = [bf(c_i, c_o, scale=c_o ** -0.5), f32(c_i), bf(c_i, c_o, scale=c_o ** -0.5), f32(c_i)]
    h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
    left = torch.empty(c_i, n, n, device="cuda", dtype=torch.bfloat16)
    right = torch.empty_like(left)
    gate_scratch = torch.empty_like(left)
    hx, hm, hl, hr, hgs = capi.tensor(x), capi.tensor(mask), capi.tensor(left), capi.tensor(right), capi.tensor(gate_scratch)
    pw = capi.TmProjWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle, h[3].handle)
    acts_l = capi.TmActInputs(n, n, hl.handle, hx.handle, hgs.handle)
    acts_r = capi.TmActInputs(n, n, hr.handle, hx.handle, hgs.handle)
    capi.kutacc_af2_triangle_multiplication_calc_proj(acts_r, hm, pw, False)
    t = timed(lambda: capi.kutacc_af2_triangle_multiplication_calc_proj(acts_l, hm, pw, False))
    report("tm_calc_proj (one side)", t, 4.0 * rows * c_o * c_i, 2.0 * rows * (c_o + c_i + 1))
    center = torch.empty_like(left)
    hc = capi.tensor(center)
    for name, incoming in (("tm_equation outgoing", False), ("tm_equation incoming", True)):
        t = timed(lambda: capi.kutacc_af2_triangle_multiplication_equation(hc, hl, hr, n, incoming))
        report(name, t, 2.0 * c_i * n * n * n, 2.0 * 3 * c_i * rows)
    del gate_scratch
    ctr = bf(n, n, c_i)
    gate = torch.empty(n, n, c_o, device="cuda", dtype=torch.bfloat16)
    keep2 = [bf(c_o, c_o, scale=c_o ** -0.5), f32(c_o), bf(c_o, c_i, scale=c_i ** -0.5), f32(c_o)]
    h2 = [capi.tensor(keep2[0]), capi.tensor(keep2[1], capi.K_FP32), capi.tensor(keep2[2]), capi.tensor(keep2[3], capi.K_FP32)]
    lw = capi.TmLinearWeights(c_o, c_i, h2[0].handle, h2[1].handle, h2[2].handle, h2[3].handle)
    hg, ho, hctr = capi.tensor(gate), capi.tensor(out), capi.tensor(ctr)
    acts = capi.TmActInputs(n, n, None, hx.handle, None)
    t = timed(lambda: capi.kutacc_af2_triangle_multiplication_gate_and_out_linear(hg, ho, acts, hctr, lw, False))
    report("tm_gate_and_out_linear", t, 2.0 * rows * c_o * (c_o + c_i), 2.0 * rows * (3 * c_o + c_i))
    t = timed(lambda: capi.kutacc_af2_triangle_multiplication_last(ho, hg, n, n, c_o))
    report("tm_last", t, 0.0, 2.0 * rows * 3 * c_o)
    # whole triangle-attention block (LayerNorm + pair bias, mask bias, attention, residual), both orientations
    heads = c_o // 32
    wts = [bf(c_o, c_o, scale=c_o ** -0.5) for _ in range(5)]
    blk_args = (x.clone(), mask, torch.ones(c_o, device="cuda"), torch.zeros(c_o, device="cuda"),
                bf(heads, c_o, scale=c_o ** -0.5), wts[0], wts[1], wts[2], wts[3], torch.ones(c_o, device="cuda"), wts[4],
                torch.zeros(c_o, device="cuda"), heads)
    attn_flops = 10.0 * rows * c_o * c_o + 4.0 * rows * n * c_o + 2.0 * rows * c_o * heads
    for name, ending in (("triangle_attention_block starting node", False), ("triangle_attention_block ending node", True)):
        blk = capi.TriangleAttentionBlock(*blk_args, ending)

        def run_blk():
            assert blk.run(stream) == 0
        report(name, timed(run_blk), attn_flops, 2.0 * rows * (2 * c_o + 1))
    # whole triangle-multiplication block (two LayerNorms, projections, equation, output step, residual)
    tw = {"ln_in_gamma": torch.ones(c_o, device="cuda"), "ln_in_beta": torch.zeros(c_o, device="cuda"),
          "ln_center_gamma": torch.ones(c_i, device="cuda"), "ln_center_beta": torch.zeros(c_i, device="cuda"),
          "output_w": bf(c_o, c_i, scale=c_i ** -0.5), "output_b": f32(c_o), "gating_w": bf(c_o, c_o, scale=c_o ** -0.5),
          "gating_b": f32(c_o)}
    for side in ("left", "right"):
        tw[side + "_proj_w"], tw[side + "_proj_b"] = bf(c_i, c_o, scale=c_o ** -0.5), f32(c_i)
        tw[side + "_gate_w"], tw[side + "_gate_b"] = bf(c_i, c_o, scale=c_o ** -0.5), f32(c_i)
    tm_flops = 2.0 * rows * c_o * (4 * c_i) + 2.0 * c_i * n * n * n + 2.0 * rows * c_o * (c_o + c_i)
    zt = x.clone()
    for name, incoming in (("triangle_multiplication_block outgoing", False), ("triangle_multiplication_block incoming", True)):
        tmb = capi.TriangleMultiplicationBlock(zt, mask, tw, incoming)

        def run_tmb():
            assert tmb.run(stream) == 0
        report(name, timed(run_tmb), tm_flops, 2.0 * rows * (2 * c_o + 1))
    capi.set_blocking(True)
    capi.set_stream(None)
    res["peaks"] = {"bf16_mfma_TFLOP/s": MFMA_BF16_PEAK_TFLOPS, "hbm_GB/s": HBM_PEAK_GBS}
    return res


def msa_block_rates(reps=20):
    """Times of the two MSA attention blocks at the shapes of configurations 2 and 4: row-wise with pair bias
    (512 sequences x 256 residues, 256 channels, pair bias from a [256, 256, 128] pair tensor) and column-wise
    (1024 sequences x 384 residues).  One kutacc_hip_msa_attention call each, in place, hipEvent-bracketed."""
    import torch
    from kutacc_amd import capi

    g = torch.Generator(device="cuda").manual_seed(13)
    bf = lambda *sh, scale=1.0: (torch.randn(*sh, device="cuda", generator=g) * scale).to(torch.bfloat16)  # noqa: E731
    stream = torch.cuda.current_stream().cuda_stream
    heads, c, cz = 8, 256, 128
    w = {"ln_gamma": torch.ones(c, device="cuda"), "ln_beta": torch.zeros(c, device="cuda"), "bg": torch.ones(c, device="cuda"),
         "bo": torch.zeros(c, device="cuda")}
    for k in ("wq", "wk", "wv", "wg", "wo"):
        w[k] = bf(c, c, scale=c ** -0.5) * (0.1 if k == "wo" else 1.0)
    res = {}
    for name, n_seq, n_res, column in (("msa_row_attention_with_pair_bias 512x256", 512, 256, False),
                                       ("msa_column_attention 1024x384", 1024, 384, True)):
        msa = bf(n_seq, n_res, c)
        mask = (torch.rand(n_seq, n_res, device="cuda", generator=g) > 0.05).to(torch.bfloat16)
        pair = None if column else {"pair_act": bf(n_res, n_res, cz), "pair_ln_gamma": torch.ones(cz, device="cuda"),
                                    "pair_ln_beta": torch.zeros(cz, device="cuda"), "bias_w": bf(heads, cz, scale=cz ** -0.5)}
        blk = capi.MsaAttentionBlock(msa, mask, w, heads, pair)
        for _ in range(3):
            assert blk.run(stream) == 0
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            assert blk.run(stream) == 0
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / reps * 1e-3
        B, S = (n_res, n_seq) if column else (n_seq, n_res)
        flops = 10.0 * B * S * c * c + 4.0 * B * S * S * c
        res[name] = {"us": round(t * 1e6, 1), "TFLOP/s": round(flops / t / 1e12, 1)}
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy: a kernel of known traffic to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run against")
    ap.add_argument("--msa-blocks", action="store_true",
                    help="also time the row-wise (with pair bias) and column-wise MSA attention blocks at the shapes of "
                         "configurations 2 and 4 and report them in an \"msa_blocks\" object")
    ap.add_argument("--pair-stack", action="store_true",
                    help="also time the transition and the triangle-multiplication steps at this configuration's pair "
                         "tensor and report them in a \"pair_stack\" object")
    ap.add_argument("--producers", action="store_true",
                    help="also time the LayerNorm and pair-bias producer kernels at this configuration's pair tensor "
                         "and report their HBM rates in a \"producers\" object")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the operator shards over the batch axis with no "
                 "exchange; multi-GPU runs are not part of it). Use --gpus 1.")

    import torch
    import helpers
    from kutacc_amd import capi
    from kutacc_amd.workloads import make_workload

    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    w = make_workload(a.config)
    op, ten, scratch = helpers.make_op(w, device="cuda:0")
    stream = torch.cuda.current_stream()
    capi.set_stream(stream.cuda_stream)
    capi.set_blocking(False)
    L = capi.lib()

    if a.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # The card idles at its lowest clocks and takes some hundred calls (about 30 ms of work) to settle at the clocks it
    # sustains under this load; the first calls after any pause run up to 25 % slower.  A fixed stretch of untimed calls
    # puts the W warm-up steps and the K timed steps at the sustained state whatever W is.
    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < SETTLE_SECONDS:
        for _ in range(50):
            op.run()
        torch.cuda.synchronize()
    for _ in range(a.warmup):
        op.run()
    assert not capi.error_flag()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        op.run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    assert not capi.error_flag()
    ms = wall / a.steps * 1e3
    tflops = w.flops() / (ms * 1e-3) / 1e12

    # per-kernel durations: same K calls again with hipEvents recorded around each kernel on the stream (a few
    # bracketed calls first, not counted: the first event pairs of a process are slow to create and resolve)
    L.kutacc_hip_profile_enable(1)
    for _ in range(max(3, min(a.warmup, 10))):
        op.run()
    torch.cuda.synchronize()
    L.kutacc_hip_profile_enable(0)
    L.kutacc_hip_profile_enable(1)  # enabling clears the totals
    for _ in range(a.steps):
        op.run()
    torch.cuda.synchronize()
    L.kutacc_hip_profile_enable(0)
    kernels = []
    name = ctypes.create_string_buffer(128)
    tot, cnt, fl = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double()
    i = 0
    while L.kutacc_hip_profile_read(i, name, 128, ctypes.byref(tot), ctypes.byref(cnt), ctypes.byref(fl)) == 0:
        kernels.append(dict(name=name.value.decode(), avg_ms=tot.value / max(cnt.value, 1), launches=cnt.value,
                            flops_per_launch=fl.value))
        i += 1
    # An event pair around a kernel reads the kernel plus the time the command processor takes over the two event
    # packets (an empty pair reads 4-5 us on this part).  The kernels of a call run back to back (the profiler's trace
    # shows no gap), so what the bracketed times of one call add up to beyond the unbracketed time per call is that
    # overhead, spread evenly over the brackets; the roofline uses the kernel's time net of it, which is what
    # rocprofv3 reports (profiles/gating_attention_kernel_stats.txt).
    per_call = sum(k["avg_ms"] * k["launches"] for k in kernels) / max(a.steps, 1)
    brackets_per_call = sum(k["launches"] for k in kernels) / max(a.steps, 1)
    overhead_ms = max(0.0, (per_call - ms) / brackets_per_call) if kernels else 0.0
    dom = max(kernels, key=lambda k: k["avg_ms"] * k["launches"]) if kernels else None
    roofline = None
    if dom:
        net_ms = dom["avg_ms"] - overhead_ms
        ach = dom["flops_per_launch"] / (net_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": dom["name"], "achieved": round(ach, 2), "peak": MFMA_BF16_PEAK_TFLOPS,
                    "unit": "TFLOP/s", "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4),
                    "traffic": measured_traffic(w.config, dom["name"]),
                    "avg_kernel_ms": round(net_ms, 5), "avg_kernel_ms_bracketed": round(dom["avg_ms"], 5),
                    "event_bracket_overhead_ms": round(overhead_ms, 5),
                    "flops_per_launch": dom["flops_per_launch"]}

    capi.set_blocking(True)
    capi.set_stream(None)

    rec = {
        "metric": "gated-attention TFLOP/s + % bf16 MFMA peak; ms/call at N_res=384 tri-attn",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic", "settle_s": SETTLE_SECONDS,
        "config": {"workload": f"config {w.config} {w.name}: B={w.B} S={w.S} C={w.C} H={w.H} d={w.d}",
                   "flops_per_call": w.flops(), "algorithmic_bytes_per_call": w.algorithmic_bytes(),
                   "path": capi.last_path()},
        "frac_mfma_peak": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
        # avg_ms: net of the event-bracket overhead (see above); avg_ms_bracketed: as the event pair read it
        "kernels": [{**{k: (round(v, 5) if isinstance(v, float) else v) for k, v in kk.items()},
                     "avg_ms": round(kk["avg_ms"] - overhead_ms, 5), "avg_ms_bracketed": round(kk["avg_ms"], 5)}
                    for kk in kernels],
        "event_bracket_overhead_ms": round(overhead_ms, 5),
        "roofline": roofline,
        "cpu_baseline": None if a.no_cpu else cpu_baseline(w),
    }
    if a.producers:
        rec["producers"] = producer_rates(a.config)
    if a.pair_stack:
        rec["pair_stack"] = pair_stack_rates(a.config)
    if a.msa_blocks:
        rec["msa_blocks"] = msa_block_rates()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
