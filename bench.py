#!/usr/bin/env python3
"""Benchmark of the fused gated-attention operator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 3] [--windows 5] [--no-cpu] [--no-all-configs]

A "step" is one kutacc_af2_gating_attention call on device-resident synthetic inputs of the chosen
configuration (default: config 3, the N_res=384 triangle-attention shape the headline metric is
quoted on).  Prints ONE JSON line: whole-call TFLOP/s from algorithmic flops
(10*B*S*C^2 + 4*B*S^2*C), ms per call (median of --windows timed windows of exactly K steps; the minimum is
reported too), the shader clock the driver reported during those windows, the roofline of the dominant kernel (live
hipEvent timing on the launch stream, read back through kutacc_hip_profile_*), ms and TFLOP/s of the other four
configurations ("all_configs") and a CPU baseline (the bf16 restatement of the reference algorithm in oracle/, timed
on this host on a bounded batch sample).
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
MFMA_FP32_PEAK_TFLOPS = 157.3   # fp32 matrix (32x32x2 f32 MFMA): 256 flop/clk/CU
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


def cpu_baseline_torch(w, budget_s=6.0):
    """A second CPU figure next to the oracle's: the same operator in PyTorch on the host cores (fp32 tensors, the
    vendor-tuned CPU GEMM behind torch.matmul, scaled_dot_product_attention with the mask and pair bias as an additive
    mask), on the first rows of the batch.  The oracle's GEMM is a plain triple loop; this one shows what a tuned CPU
    GEMM makes of the same work.  It follows the operator's mathematics, not the reference's rounding points."""
    import numpy as np
    import torch
    import torch.nn.functional as F

    H, d, C, S = w.H, w.d, w.C, w.S
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32))  # noqa: E731
    wq, wk, wv, wg, wo, bg, bo = (f(a) for a in (w.wq, w.wk, w.wv, w.wg, w.wo, w.bg, w.bo))
    nb = None if w.nb is None else f(w.nb)

    def run(nrows):
        x, bias = f(w.x[:nrows]), f(w.bias[:nrows])
        t0 = time.perf_counter()
        with torch.no_grad():
            heads = lambda t: t.view(nrows, S, H, d).transpose(1, 2)  # noqa: E731
            q, k, v = heads(x @ wq.T), heads(x @ wk.T), heads(x @ wv.T)
            mask = bias.view(nrows, 1, 1, S)
            if nb is not None:
                mask = mask + nb.view(1, H, S, S)
            o = F.scaled_dot_product_attention(q, k, v, attn_mask=mask.expand(nrows, H, S, S))
            gate = torch.sigmoid(x @ wg.T + bg)
            out = (o.transpose(1, 2).reshape(nrows, S, C) * gate) @ wo.T + bo
        return time.perf_counter() - t0, float(out[0, 0, 0])

    probe = min(w.B, 4)
    run(probe)
    t_probe, _ = run(probe)
    rows = int(min(w.B, max(probe, probe * budget_s / max(t_probe, 1e-3))))
    t, _ = run(rows)
    fl = (10.0 * rows * S * C * C + 4.0 * rows * S * S * C)
    return {"value": round(fl / t / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "torch-cpu",
            "sample": f"first {rows} of {w.B} batch rows, fp32 torch.matmul + scaled_dot_product_attention on the host, one call, "
                      f"{t:.2f} s (= {t / rows * w.B * 1e3:.0f} ms/call extrapolated to the full batch)"}


def host_pointer_call(w, calls=3):
    """One call of the handle-based entry point with every operand in host memory: the library stages operands and
    results through the device per call, so this is the PCIe-inclusive time of the drop-in's compatibility path.
    Reported beside the headline figure, never as `value`."""
    import helpers
    from kutacc_amd import capi

    ten, scratch = helpers.host_arrays(w)
    op = capi.GatedAttention(ten["x"], ten["wq"], ten["wk"], ten["wv"], ten["wg"], ten["bg"], ten["wo"], ten["bo"],
                             ten["bias"], ten["nb"], w.H, ten["out"], scratch, block_size=64)
    op.run()  # first call: the staging buffers are allocated
    times = []
    for _ in range(calls):
        t0 = time.perf_counter()
        op.run()
        times.append((time.perf_counter() - t0) * 1e3)
    assert not capi.error_flag()
    capi.lib().kutacc_hip_release_staging()
    ms = sorted(times)[len(times) // 2]
    return {"ms": round(ms, 3), "calls": calls, "TFLOP/s": round(w.flops() / (ms * 1e-3) / 1e12, 3),
            "note": "host pointers, blocking call: operands copied to the device, results copied back (PCIe-bound); not the headline path"}


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
    and result of the step once), which of the two rooflines bounds the step (the one whose time at peak is the longer:
    the equation at 384 residues has 128 flop per byte against the card's 312 and is HBM-bound; from 1024 on it is not)
    and the fraction of that roofline reached."""
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
        for _ in range(15):  # the first calls after a pause run at the card's idle clocks
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
        # the roofline that bounds the step is the one whose time at peak is the longer; frac = that time / measured
        t_mfma, t_hbm = flops / (MFMA_BF16_PEAK_TFLOPS * 1e12), nbytes / (HBM_PEAK_GBS * 1e9)
        res[name] = {"us": round(t * 1e6, 1), "TFLOP/s": round(flops / t / 1e12, 1), "GB/s": round(nbytes / t / 1e9, 1),
                     "bound": "mfma" if t_mfma > t_hbm else "hbm", "frac": round(max(t_mfma, t_hbm) / t, 3)}

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
        for _ in range(30):  # the first calls after a pause run at the card's idle clocks
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


def tiled_route_rates(reps=3):
    """Times of the operator on the tiled MFMA route (the bf16 shapes beyond the fused head kernels), hipEvent-bracketed
    calls of kutacc_hip_gating_attention on device tensors drawn with torch's generator: triangle attention at 2048
    residues (2048 rows of 2048 positions, 4 heads of 32), the row-wise attention of the extra-MSA stack (5120 sequences
    x 384 residues, 8 heads of 8, pair bias) and, for scale, the headline configuration forced onto this route.  Per
    shape: milliseconds and TFLOP/s on the operator's algorithmic flops (10 B S C^2 + 4 B S^2 C)."""
    import ctypes

    import torch
    from kutacc_amd import capi

    stream = torch.cuda.current_stream().cuda_stream
    res = {}
    for name, B, S, H, d, path in (("triangle_attention 2048 residues (B=2048 S=2048 H=4 d=32)", 2048, 2048, 4, 32, capi.PATH_AUTO),
                                   ("extra_msa_row_attention (B=5120 S=384 H=8 d=8)", 5120, 384, 8, 8, capi.PATH_AUTO),
                                   ("config 3 forced onto the tiled route (B=384 S=384 H=4 d=32)", 384, 384, 4, 32, capi.PATH_TILED)):
        C = H * d
        g = torch.Generator(device="cuda").manual_seed(17)
        bf = lambda *sh, scale=1.0: (torch.randn(*sh, device="cuda", generator=g) * scale).to(torch.bfloat16)  # noqa: E731
        x, ws = bf(B, S, C), [bf(C, C, scale=C ** -0.5) for _ in range(5)]
        bg, bo = torch.ones(C, device="cuda"), torch.zeros(C, device="cuda")
        bias, nb = torch.zeros(B, S, device="cuda", dtype=torch.bfloat16), bf(H, S, S)
        out = torch.empty(B, S, C, device="cuda", dtype=torch.bfloat16)
        q, k, gate, avg = (torch.empty(B, S, C, device="cuda", dtype=torch.bfloat16) for _ in range(4))
        v = torch.empty(C, B * S, device="cuda", dtype=torch.bfloat16)
        a = capi.HipAttentionArgs()
        a.batch, a.seq_len, a.nheads, a.head_size, a.dtype, a.path = B, S, H, d, capi.K_BF16, path
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

        def call():
            assert capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), stream) == 0
        for _ in range(3):
            call()
        assert capi.last_path() == "tiled_mfma", capi.last_path()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            call()
        e1.record()
        torch.cuda.synchronize()
        t = e0.elapsed_time(e1) / reps * 1e-3
        flops = 10.0 * B * S * C * C + 4.0 * B * S * S * C
        res[name] = {"ms": round(t * 1e3, 3), "TFLOP/s": round(flops / t / 1e12, 1),
                     "frac_of_bf16_mfma_peak": round(flops / t / 1e12 / MFMA_BF16_PEAK_TFLOPS, 3)}
        del x, ws, nb, out, q, k, gate, avg, v
        torch.cuda.empty_cache()
    return res


def device_workload(config):
    """Inputs of configuration `config` drawn on the GPU (torch's generator, seed 1000 + config): the same shapes,
    distributions and mask rules as kutacc_amd.workloads.make_workload, without its minute of host-side drawing for the
    large pair tensors.  Used for the timing of the configurations beside the headline one; the parity tests and the
    headline measurement use the seeded numpy workloads.  Returns (op, tensors, scratch, spec)."""
    import numpy as np
    import torch
    from kutacc_amd import capi
    from kutacc_amd.workloads import CONFIGS, C_Z, HEAD_SIZE, MASK_BIAS

    spec = CONFIGS[config]
    B, S, H = spec["B"], spec["S"], spec["H"]
    C = H * HEAD_SIZE
    dt = torch.bfloat16 if spec["dtype"] == "bf16" else torch.float32
    code = capi.K_BF16 if spec["dtype"] == "bf16" else capi.K_FP32
    g = torch.Generator(device="cuda").manual_seed(1000 + config)
    L = capi.lib()

    def normal(*shape, scale=1.0):
        return (torch.randn(*shape, device="cuda", generator=g) * scale).to(dt)

    def layernorm(t):
        rows, size = t.numel() // t.shape[-1], t.shape[-1]
        out = torch.empty_like(t)
        ones, zeros = torch.ones(size, device="cuda"), torch.zeros(size, device="cuda")
        assert L.kutacc_hip_layernorm_rows(t.data_ptr(), size, ones.data_ptr(), zeros.data_ptr(), out.data_ptr(), size, rows,
                                           size, 1e-5, code, None) == 0
        torch.cuda.synchronize()
        return out

    nb = None
    if config in (3, 5):  # the pair tensor is the attention input and the source of the pair bias
        z = normal(S, S, C_Z)
        w_bias = normal(H, C_Z, scale=C_Z ** -0.5)
        x = torch.empty_like(z)
        nb = torch.empty((H, S, S), device="cuda", dtype=dt)
        ones, zeros = torch.ones(C_Z, device="cuda"), torch.zeros(C_Z, device="cuda")
        assert L.kutacc_hip_pair_bias(z.data_ptr(), ones.data_ptr(), zeros.data_ptr(), w_bias.data_ptr(), nb.data_ptr(),
                                      x.data_ptr(), S, S, C_Z, H, 1e-5, code, None) == 0
        torch.cuda.synchronize()
        del z
    else:
        x = layernorm(normal(B, S, C))
        if spec["pair_bias"]:
            zn = layernorm(normal(S, S, C_Z))
            w_bias = normal(H, C_Z, scale=C_Z ** -0.5)
            nb = torch.einsum("ijc,hc->hij", zn.float(), w_bias.float()).to(dt).contiguous()
            del zn
    wq, wk, wv, wg, wo = (normal(C, C, scale=C ** -0.5) for _ in range(5))
    bg, bo = torch.ones(C, device="cuda"), torch.zeros(C, device="cuda")
    rng = np.random.Generator(np.random.PCG64(1000 + config))
    bias = np.zeros((B, S), dtype=np.float32)
    if config in (2, 4):  # residues (2) or sequences (4) padded, the same keys for every batch row
        keep = rng.random(S) >= (0.05 if config == 2 else 0.10)
        keep[0] = True
        bias[:] = (MASK_BIAS * (1.0 - keep.astype(np.float32)))[None, :]
    elif config == 5:  # last 0-15 % of the residues padded, as a pair mask
        pad = int(np.floor(rng.random() * 0.15 * S))
        r = (np.arange(S) < S - pad).astype(np.float32)
        bias[:] = MASK_BIAS * (1.0 - r[:B, None] * r[None, :])
    bias = torch.from_numpy(bias).to(device="cuda", dtype=dt)
    ten = dict(x=x, wq=wq, wk=wk, wv=wv, wg=wg, wo=wo, bg=bg, bo=bo, bias=bias, nb=nb,
               out=torch.zeros((B, S, C), device="cuda", dtype=dt))
    scratch = {n: torch.zeros((B, S, H, HEAD_SIZE), device="cuda", dtype=dt) for n in ("q", "k", "gate", "avg")}
    scratch["v"] = torch.zeros((H, HEAD_SIZE, B, S), device="cuda", dtype=dt)
    op = capi.GatedAttention(x, wq, wk, wv, wg, bg, wo, bo, bias, nb, H, ten["out"], scratch)
    return op, ten, scratch, spec


def settle(op, seconds=SETTLE_SECONDS):
    """Untimed calls until the card sits at the clocks it sustains under this load (see main())."""
    import torch
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            op.run()
        torch.cuda.synchronize()


def timed_window(op, steps):
    """Wall time of exactly `steps` asynchronous calls between two synchronisations, in ms per call."""
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        op.run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def kernel_times(op, steps, warm):
    """Per-kernel durations over `steps` calls: hipEvents recorded by the library around each kernel on the launch stream
    (a few bracketed calls first, not counted: the first event pairs of a process are slow to create and resolve)."""
    import torch
    from kutacc_amd import capi
    L = capi.lib()
    L.kutacc_hip_profile_enable(1)
    for _ in range(warm):
        op.run()
    torch.cuda.synchronize()
    L.kutacc_hip_profile_enable(0)
    L.kutacc_hip_profile_enable(1)  # enabling clears the totals
    for _ in range(steps):
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
    return kernels


def empty_event_pair_ms(stream, n=200):
    """What a pair of events recorded back to back on the launch stream reads with no kernel between them: the part of a
    bracketed kernel time that is the command processor handling the two event packets.  Median of n pairs."""
    import torch
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    with torch.cuda.stream(stream):
        for e0, e1 in pairs:
            e0.record()
            e1.record()
    torch.cuda.synchronize()
    reads = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    return reads[len(reads) // 2]


class ClockSampler:
    """Samples the shader clock the driver reports (sysfs pp_dpm_sclk of the first AMD card: the level marked '*')
    from a host thread while a timed window runs.  Reports None where the file is missing or unreadable."""

    def __init__(self, period_s=0.002):
        import glob
        self.path = next(iter(sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk"))), None)
        self.period = period_s
        self.samples = []
        self._stop = False
        self._thread = None

    def _read(self):
        try:
            with open(self.path) as f:
                for line in f:
                    if "*" in line:
                        return float(line.split(":")[1].lower().replace("mhz", "").replace("*", "").strip())
        except (OSError, ValueError, IndexError, TypeError):
            return None
        return None

    def __enter__(self):
        import threading
        if self.path:
            def loop():
                while not self._stop:
                    v = self._read()
                    if v:
                        self.samples.append(v)
                    time.sleep(self.period)
            self._thread = threading.Thread(target=loop, daemon=True)
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop = True
        if self._thread:
            self._thread.join()

    def mean_mhz(self):
        return round(sum(self.samples) / len(self.samples), 1) if self.samples else None


def config_summary(config, steps, warmup):
    """One of the configurations beside the headline one: settle, warm up, time `steps` calls, per-kernel brackets.
    Returns {ms, TFLOP/s, frac, dominant kernel, path} plus the kernel list."""
    import torch
    from kutacc_amd import capi
    op, ten, scratch, spec = device_workload(config)
    B, S, H = spec["B"], spec["S"], spec["H"]
    C = H * 32
    flops = 10 * B * S * C * C + 4 * B * S * S * C
    settle(op)
    for _ in range(warmup):
        op.run()
    ms = timed_window(op, steps)
    assert not capi.error_flag()
    kernels = kernel_times(op, steps, max(3, min(warmup, 10)))
    dom = max(kernels, key=lambda k: k["avg_ms"] * k["launches"])
    tf = flops / (ms * 1e-3) / 1e12
    rec = {"workload": f"config {config} {spec['name']}: B={B} S={S} C={C} H={H} d=32", "dtype": spec["dtype"], "steps": steps,
           "ms": round(ms, 5), "TFLOP/s": round(tf, 2),
           "frac_mfma_peak": round(tf / (MFMA_BF16_PEAK_TFLOPS if spec["dtype"] == "bf16" else MFMA_FP32_PEAK_TFLOPS), 4),
           "path": capi.last_path(), "dominant_kernel": dom["name"], "dominant_kernel_ms": round(dom["avg_ms"], 5),
           "kernels": [{"name": k["name"], "avg_ms": round(k["avg_ms"], 5), "launches_per_call": k["launches"] // max(steps, 1)}
                       for k in kernels],
           "data": "drawn on the GPU (same shapes, distributions and mask rules as the seeded workload)"}
    del op, ten, scratch
    torch.cuda.empty_cache()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--windows", type=int, default=5, help="timed windows of --steps calls each; the line reports their median and minimum")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-all-configs", action="store_true", help="skip the timing of the other four configurations")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy: a kernel of known traffic to scale the "
                         "FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run against")
    ap.add_argument("--msa-blocks", action="store_true",
                    help="also time the row-wise (with pair bias) and column-wise MSA attention blocks at the shapes of "
                         "configurations 2 and 4 and report them in an \"msa_blocks\" object")
    ap.add_argument("--tiled-route", action="store_true",
                    help="also time the operator on the tiled MFMA route (rows of 2048 positions, head size 8) and report it "
                         "in a \"tiled_route\" object")
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

    if a.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    # The card idles at its lowest clocks and takes some hundred calls (about 30 ms of work) to settle at the clocks it
    # sustains under this load; the first calls after any pause run up to 25 % slower.  A fixed stretch of untimed calls
    # puts the W warm-up steps and the K timed steps at the sustained state whatever W is.
    settle(op)
    for _ in range(a.warmup):
        op.run()
    assert not capi.error_flag()
    # --windows timed windows of exactly K steps each, back to back; ms_per_step is their median
    with ClockSampler() as clock:
        windows = [timed_window(op, a.steps) for _ in range(max(1, a.windows))]
    assert not capi.error_flag()
    ms = sorted(windows)[len(windows) // 2]
    tflops = w.flops() / (ms * 1e-3) / 1e12

    kernels = kernel_times(op, a.steps, max(3, min(a.warmup, 10)))
    # An event pair around a kernel reads the kernel plus the time the command processor takes over the two event
    # packets; an empty pair on the same stream measures that part directly.  avg_ms is what the bracket read;
    # avg_ms_net subtracts the empty pair and is the figure comparable with a profiler's kernel duration.
    overhead_ms = empty_event_pair_ms(stream)
    dom = max(kernels, key=lambda k: k["avg_ms"] * k["launches"]) if kernels else None
    peak = MFMA_BF16_PEAK_TFLOPS if w.dtype == "bf16" else MFMA_FP32_PEAK_TFLOPS  # fp32 storage runs on the fp32 matrix core
    roofline = None
    if dom:
        ach = dom["flops_per_launch"] / (dom["avg_ms"] * 1e-3) / 1e12
        net_ms = max(dom["avg_ms"] - overhead_ms, 1e-6)
        ach_net = dom["flops_per_launch"] / (net_ms * 1e-3) / 1e12
        roofline = {"bound": "mfma", "kernel": dom["name"], "achieved": round(ach, 2), "peak": peak,
                    "unit": "TFLOP/s", "frac": round(ach / peak, 4),
                    "traffic": measured_traffic(w.config, dom["name"]),
                    "traffic_source": "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this command, "
                                      "not re-measured in this run)",
                    "avg_kernel_ms": round(dom["avg_ms"], 5), "avg_kernel_ms_net": round(net_ms, 5),
                    "achieved_net": round(ach_net, 2), "frac_net": round(ach_net / peak, 4),
                    "empty_event_pair_ms": round(overhead_ms, 5),
                    "flops_per_launch": dom["flops_per_launch"]}

    rec = {
        "metric": "gated-attention TFLOP/s + % bf16 MFMA peak; ms/call at N_res=384 tri-attn",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": w.dtype, "data": "synthetic", "settle_s": SETTLE_SECONDS,
        "config": {"workload": f"config {w.config} {w.name}: B={w.B} S={w.S} C={w.C} H={w.H} d={w.d}",
                   "flops_per_call": w.flops(), "algorithmic_bytes_per_call": w.algorithmic_bytes(),
                   "path": capi.last_path()},
        "frac_mfma_peak": round(tflops / peak, 4),
        # ms_per_step and value are the median window; each window is exactly `steps` calls
        "timed_windows": {"count": len(windows), "steps_each": a.steps, "median_ms": round(ms, 5),
                          "min_ms": round(min(windows), 5), "max_ms": round(max(windows), 5),
                          "all_ms": [round(v, 5) for v in windows]},
        "shader_clock_mhz": clock.mean_mhz(), "shader_clock_samples": len(clock.samples),
        "kernels": [{**{k: (round(v, 5) if isinstance(v, float) else v) for k, v in kk.items()},
                     "avg_ms_net": round(max(kk["avg_ms"] - overhead_ms, 0.0), 5)} for kk in kernels],
        "empty_event_pair_ms": round(overhead_ms, 5),
        "roofline": roofline,
    }
    del op, ten, scratch
    torch.cuda.empty_cache()
    if not a.no_all_configs:
        # the other configurations, same settle + warm-up, at least 50 steps each (no CPU leg)
        rec["all_configs"] = {f"config {w.config}": {"ms": round(ms, 5), "TFLOP/s": round(tflops, 2),
                                                      "frac_mfma_peak": round(tflops / peak, 4),
                                                      "path": rec["config"]["path"],
                                                      "dominant_kernel": dom["name"] if dom else None}}
        for c in (1, 2, 4, 5):
            if c != w.config:
                rec["all_configs"][f"config {c}"] = config_summary(c, max(50, min(a.steps, 100)), a.warmup)
    capi.set_blocking(True)
    capi.set_stream(None)
    rec["cpu_baseline"] = None if a.no_cpu else cpu_baseline(w)
    if not a.no_cpu:
        rec["cpu_baseline_torch"] = cpu_baseline_torch(w)
        rec["host_pointer_call"] = host_pointer_call(w)
    if a.producers:
        rec["producers"] = producer_rates(a.config)
    if a.pair_stack:
        rec["pair_stack"] = pair_stack_rates(a.config)
    if a.msa_blocks:
        rec["msa_blocks"] = msa_block_rates()
    if a.tiled_route:
        rec["tiled_route"] = tiled_route_rates()
    print(json.dumps(rec))


if __name__ == "__main__":
    main()
