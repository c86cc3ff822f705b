"""Pins the CPU oracle before anything is compared against it.

The reference ships no numeric test, golden vector or fixture for the gated-attention operator (its
tests only check that invalid arguments do not crash), and it cannot be built on this machine.  The
oracle is therefore pinned by: library routines (torch matmul / scaled_dot_product_attention /
layer_norm / linear), a pure-Python brute force on a tiny case, closed forms and invariants chosen so
that a dropped term, a wrong index or a transposed operand fails at least one of them, and the
committed float64 fixture.
"""
import itertools
import math
import os

import numpy as np
import pytest
import torch

from oracle import oracle

HERE = os.path.dirname(os.path.abspath(__file__))


def make_case(seed, B, S, H, d, nb=True, bias_mode="zeros"):
    rng = np.random.Generator(np.random.PCG64(seed))
    C = H * d
    f = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    case = dict(x=f(B, S, C), wq=f(C, C) / math.sqrt(C), wk=f(C, C) / math.sqrt(C), wv=f(C, C) / math.sqrt(C),
                wg=f(C, C) / math.sqrt(C), bg=f(C), wo=f(C, C) / math.sqrt(C), bo=f(C),
                bias=np.zeros((B, S), dtype=np.float32), nb=f(H, S, S) if nb else None, nheads=H)
    if bias_mode == "random_mask":
        keep = rng.random((B, S)) > 0.3
        keep[:, 0] = True
        case["bias"] = (-1e9 * (1 - keep)).astype(np.float32)
    return case


def run_f32(case, **kw):
    return oracle.gating_attention_f32(case["x"], case["wq"], case["wk"], case["wv"], case["wg"], case["bg"],
                                       case["wo"], case["bo"], case["bias"], case["nb"], case["nheads"], **kw)


def run_f64(case, **kw):
    return oracle.gating_attention_f64_numpy(case["x"], case["wq"], case["wk"], case["wv"], case["wg"], case["bg"],
                                             case["wo"], case["bo"], case["bias"], case["nb"], case["nheads"], **kw)


# ---- library routines --------------------------------------------------------------------------------
@pytest.mark.parametrize("nb,bias_mode", [(True, "zeros"), (False, "zeros"), (True, "random_mask")])
def test_numpy_twin_matches_torch_sdpa(nb, bias_mode):
    c = make_case(1, 3, 17, 2, 8, nb=nb, bias_mode=bias_mode)
    B, S, C = c["x"].shape
    H = c["nheads"]
    d = C // H
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float64))  # noqa: E731
    x = t(c["x"])
    q = (x @ t(c["wq"]).T).reshape(B, S, H, d).transpose(1, 2)
    k = (x @ t(c["wk"]).T).reshape(B, S, H, d).transpose(1, 2)
    v = (x @ t(c["wv"]).T).reshape(B, S, H, d).transpose(1, 2)
    g = torch.sigmoid(x @ t(c["wg"]).T + t(c["bg"]))
    # mask values are moderate here (-1e9 in float64 does not absorb; that case is tested separately)
    mask = t(c["bias"])[:, None, None, :].expand(B, H, S, S).clone()
    if nb:
        mask = mask + t(c["nb"])[None]
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=1.0 / math.sqrt(d))
    o = o.transpose(1, 2).reshape(B, S, C) * g
    ref = (o @ t(c["wo"]).T + t(c["bo"])).numpy()
    got = run_f64(c)
    if bias_mode == "random_mask":
        # with -1e9 the fp32 bias add of the operator rounds the logit away; torch float64 keeps it.
        # masked keys get weight 0 either way and rows always keep key 0, so results agree closely
        np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)
    else:
        np.testing.assert_allclose(got, ref, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(2, 5, 2, 4), (3, 33, 4, 32), (2, 64, 8, 32), (1, 70, 1, 48)])
@pytest.mark.parametrize("nb,bias_mode", [(True, "zeros"), (False, "random_mask"), (True, "random_mask")])
def test_c_oracle_matches_numpy_twin(shape, nb, bias_mode):
    c = make_case(7, *shape, nb=nb, bias_mode=bias_mode)
    out, avg = run_f32(c, return_avg=True)
    ref, ref_avg = run_f64(c, return_avg=True)
    np.testing.assert_allclose(out, ref, rtol=2e-6, atol=2e-6)
    np.testing.assert_allclose(avg, ref_avg, rtol=2e-6, atol=2e-6)


def test_c_oracle_matches_python_bruteforce():
    """Every index written out by hand: catches transposed weights, head/channel mix-ups, wrong
    softmax axis."""
    c = make_case(3, 2, 5, 2, 4)
    c["bias"][0, 3] = -1e9
    B, S, C = c["x"].shape
    H = c["nheads"]
    d = C // H
    x = c["x"].astype(np.float64)
    out = np.zeros((B, S, C))
    for b in range(B):
        avg = np.zeros((S, C))
        for h in range(H):
            def proj(w, s, e, bvec=None):
                o = h * d + e
                acc = sum(x[b, s, i] * float(w[o, i]) for i in range(C))
                return acc + (float(bvec[o]) if bvec is not None else 0.0)
            for qi in range(S):
                logits = []
                for kj in range(S):
                    s_ = sum(proj(c["wq"], qi, e) * proj(c["wk"], kj, e) for e in range(d)) / math.sqrt(d)
                    xl = np.float32(np.float32(s_) + c["bias"][b, kj]) + c["nb"][h, qi, kj]
                    logits.append(float(xl))
                m = max(logits)
                p = [math.exp(v - m) for v in logits]
                z = sum(p)
                for e in range(d):
                    wavg = sum(p[kj] / z * proj(c["wv"], kj, e) for kj in range(S))
                    gate = 1.0 / (1.0 + math.exp(-proj(c["wg"], qi, e, c["bg"])))
                    avg[qi, h * d + e] = wavg * gate
        for s in range(S):
            for o in range(C):
                out[b, s, o] = sum(avg[s, i] * float(c["wo"][o, i]) for i in range(C)) + float(c["bo"][o])
    np.testing.assert_allclose(run_f32(c), out, rtol=2e-6, atol=2e-6)


def test_c_oracle_matches_golden_fixture():
    g = np.load(os.path.join(HERE, "golden", "gating_attention_tiny.npz"))
    B, S, H, d = (int(v) for v in g["dims"])
    for name in ("pair_bias", "no_pair_bias", "masked_key", "masked_row"):
        nb = None if name == "no_pair_bias" else g["in.nb"]
        out, avg = oracle.gating_attention_f32(g["in.x"], g["in.wq"], g["in.wk"], g["in.wv"], g["in.wg"], g["in.bg"],
                                               g["in.wo"], g["in.bo"], g[f"{name}.bias"], nb, H, return_avg=True)
        np.testing.assert_allclose(out, g[f"{name}.out"], rtol=2e-6, atol=2e-6, err_msg=name)
        np.testing.assert_allclose(avg, g[f"{name}.avg"], rtol=2e-6, atol=2e-6, err_msg=name)


# ---- closed forms and invariants --------------------------------------------------------------------
def test_uniform_attention_when_query_weight_is_zero():
    c = make_case(11, 2, 9, 2, 8, nb=False, bias_mode="random_mask")
    c["wq"][:] = 0
    _, avg = run_f32(c, return_avg=True)
    B, S, C = c["x"].shape
    v = c["x"].astype(np.float64) @ c["wv"].astype(np.float64).T
    gate = 1 / (1 + np.exp(-(c["x"].astype(np.float64) @ c["wg"].astype(np.float64).T + c["bg"])))
    for b in range(B):
        keep = c["bias"][b] == 0
        mean_v = v[b][keep].mean(axis=0)
        np.testing.assert_allclose(avg[b], mean_v[None, :] * gate[b], rtol=1e-5, atol=1e-6)


def test_gate_closed_forms():
    c = make_case(12, 2, 7, 2, 8)
    base = dict(c)
    c0 = dict(base, wg=np.zeros_like(c["wg"]), bg=np.zeros_like(c["bg"]))
    c1 = dict(base, wg=np.zeros_like(c["wg"]), bg=np.full_like(c["bg"], 30.0))
    _, a0 = run_f32(c0, return_avg=True)
    _, a1 = run_f32(c1, return_avg=True)
    np.testing.assert_allclose(a0, 0.5 * a1, rtol=1e-6, atol=1e-7)  # sigmoid(0) = 1/2, sigmoid(30) = 1


def test_zero_output_weight_gives_output_bias():
    c = make_case(13, 2, 7, 2, 8)
    c["wo"][:] = 0
    out = run_f32(c)
    np.testing.assert_array_equal(out, np.broadcast_to(c["bo"], out.shape))


def test_constant_values_pass_through_softmax():
    """Rows of P sum to one: if every key has the same value vector, avg equals it (times the gate)."""
    c = make_case(14, 2, 9, 2, 8, bias_mode="random_mask")
    c["x"][:] = c["x"][:, :1, :]  # identical tokens -> identical v for every key (q,k too, harmless)
    _, avg = run_f32(c, return_avg=True)
    x0 = c["x"][:, 0].astype(np.float64)
    v0 = x0 @ c["wv"].astype(np.float64).T
    gate = 1 / (1 + np.exp(-(x0 @ c["wg"].astype(np.float64).T + c["bg"])))
    np.testing.assert_allclose(avg, np.broadcast_to((v0 * gate)[:, None, :], avg.shape), rtol=1e-5, atol=1e-6)


def test_softmax_shift_invariance():
    c = make_case(15, 2, 9, 2, 8)
    out = run_f32(c)
    c2 = dict(c, nb=c["nb"] + np.float32(3.0) * np.ones((1, 9, 1), dtype=np.float32),
              bias=c["bias"] + np.float32(2.0))
    np.testing.assert_allclose(run_f32(c2), out, rtol=1e-5, atol=1e-5)


def test_key_permutation_and_batch_permutation():
    c = make_case(16, 3, 8, 2, 8, bias_mode="random_mask")
    out = run_f32(c)
    # permuting the batch permutes the output
    perm_b = np.array([2, 0, 1])
    cb = dict(c, x=c["x"][perm_b], bias=c["bias"][perm_b])
    np.testing.assert_allclose(run_f32(cb), out[perm_b], rtol=1e-6, atol=1e-6)
    # permuting tokens (queries and keys together, with both biases) permutes the output rows
    perm_s = np.random.Generator(np.random.PCG64(5)).permutation(8)
    cs = dict(c, x=c["x"][:, perm_s], bias=c["bias"][:, perm_s], nb=c["nb"][:, perm_s][:, :, perm_s])
    np.testing.assert_allclose(run_f32(cs), out[:, perm_s], rtol=1e-5, atol=1e-5)


def test_masked_key_has_exactly_zero_weight():
    c = make_case(17, 1, 6, 2, 8)
    c["bias"][0, 2] = -1e9
    _, avg = run_f32(c, return_avg=True)
    # replace the masked token: its k and v change, every other row of avg must not move at all
    c2 = dict(c, x=c["x"].copy())
    c2["x"][0, 2] = 100.0
    _, avg2 = run_f32(c2, return_avg=True)
    rows = [0, 1, 3, 4, 5]
    np.testing.assert_array_equal(avg[0, rows], avg2[0, rows])


def test_fully_masked_row_attends_uniformly():
    """-1e9 absorbs the logit and the pair bias in fp32, so all keys tie (reference
    gating_attention.cpp:113-117 adds in fp32)."""
    c = make_case(18, 2, 6, 2, 8)
    c["bias"][1, :] = -1e9
    _, avg = run_f32(c, return_avg=True)
    x1 = c["x"][1].astype(np.float64)
    v = x1 @ c["wv"].astype(np.float64).T
    gate = 1 / (1 + np.exp(-(x1 @ c["wg"].astype(np.float64).T + c["bg"])))
    np.testing.assert_allclose(avg[1], v.mean(axis=0)[None] * gate, rtol=1e-5, atol=1e-6)


def test_absent_pair_bias_equals_zero_pair_bias():
    c = make_case(19, 2, 7, 2, 8, nb=False)
    out = run_f32(c)
    c2 = dict(c, nb=np.zeros((2, 7, 7), dtype=np.float32))
    np.testing.assert_array_equal(run_f32(c2), out)


# ---- fast_exp emulation (reference src/math/fast_exp.h:21-27) -----------------------------------------
# The FEXPA instruction cannot be run here.  What the arithmetic around it fixes: the result is 2^(n/64) for the integer
# n nearest to x * 64 / ln 2 (ties away from zero), assembled from n's low six bits (table index) and the bits above
# (exponent); a negative n + 8128 saturates to 0 in the unsigned conversion and gives +0.0; x is clamped at ln(FLT_MAX).
def _fexpa_grid():
    rng = np.random.default_rng(7)
    xs = [np.linspace(-100.0, 95.0, 200001), rng.uniform(-20.0, 20.0, 200000), rng.normal(0.0, 1.0, 100000),
          np.array([0.0, -0.0, 1.0, -1.0, 88.0, 88.72283, 88.72284, 88.8, 100.0, 1e30, -87.9, -88.0, -88.1, -1e30])]
    return np.concatenate(xs).astype(np.float32)


def test_fast_exp_emulation_returns_the_nearest_64th_octave():
    x = _fexpa_grid()
    y = oracle.ref_exp(x, 1).astype(np.float64)
    inside = (x > -87.3) & (x < 88.7)  # below -87.34 the exponent field is 0 and the table bits read as a subnormal
    xi, yi = x[inside].astype(np.float64), y[inside]
    steps = 64.0 * np.log2(yi)  # must be integers: the result is a power of 2^(1/64) (mantissa from a 64-entry table)
    n = np.rint(steps)
    assert np.abs(steps - n).max() < 2e-5  # 1 ulp of fp32 in the mantissa is 64 * 1.7e-7 of a step
    # ... and the nearest one to exp(x): the exact position is x * 64 / ln 2; fp32 rounding of the constant 92.33248
    # and of the multiply-add moves it by < 1e-3 of a step at |x| < 88, which only matters next to a tie
    pos = xi * (64.0 / np.log(2.0))
    dist = np.abs(pos - n)
    assert dist.max() <= 0.5 + 2e-3
    # relative error against exp: at most half a step, 2^(1/128) - 1 = 0.543 %
    rel = np.abs(yi / np.exp(xi) - 1.0)
    assert rel.max() <= 2.0 ** (1.0 / 128.0) - 1.0 + 3e-5
    assert rel.max() > 4e-3  # and it is that coarse: a libm exp would pass everything above but this


def test_fast_exp_emulation_ties_round_away_from_zero():
    # x = (k + 0.5) * ln 2 / 64 cannot be hit exactly in fp32, but the integer-valued products can: with x = m / 92.33248
    # rounded to fp32 the fma lands within an ulp of m + 8128, so walk fp32 neighbours until the product is the exact
    # half-integer and check the direction of rounding on the bit level instead
    k = np.arange(-200, 200, dtype=np.float64)
    c = np.float32(92.33248)
    hits = 0
    for kk in k:
        target = kk + 0.5 + 8128.0
        x0 = np.float32((kk + 0.5) / float(c))
        for _ in range(8):  # search the neighbourhood for an x whose single-rounded fma equals the tie exactly
            t = np.float32(np.float64(x0) * np.float64(c) + 8128.0)  # double product is exact enough: one rounding
            if float(t) == target:
                y = float(oracle.ref_exp(np.array([x0], np.float32), 1)[0])
                want = 2.0 ** ((kk + 1.0) / 64.0)  # half away from zero in the biased (positive) domain
                assert abs(y / want - 1.0) < 2e-7, (kk, y, want)
                hits += 1
                break
            x0 = np.nextafter(x0, np.float32(np.inf if float(t) < target else -np.inf), dtype=np.float32)
    assert hits > 50


def test_fast_exp_emulation_special_values():
    e = lambda v: oracle.ref_exp(np.array(v, np.float32), 1)
    assert e([0.0])[0] == 1.0 and e([-0.0])[0] == 1.0
    ln2 = np.float32(np.log(2.0))
    got = e([ln2, -ln2, 2 * ln2])  # n = +-64, 128 exactly (the products are within 1e-5 of the integers)
    np.testing.assert_array_equal(got, np.array([2.0, 0.5, 4.0], np.float32))
    # below -8128 / 92.33248 = -88.03 the biased integer is <= 0, the unsigned conversion saturates and FEXPA(0) is +0.0
    z = e([-88.04, -88.5, -100.0, -1e9, -3e38, -np.inf])
    assert np.all(z == 0.0) and not np.any(np.signbit(z))
    assert e([-88.02])[0] > 0.0
    # the clamp at ln(FLT_MAX): everything at or above it gives the same result (exponent field 255, fraction 0)
    top = e([88.72284, 88.8, 100.0, 1e30, np.inf])
    assert np.all(top == top[0]) and np.isinf(top[0])
    assert np.isfinite(e([88.7])[0])
    # monotone non-decreasing over the whole grid
    x = np.sort(_fexpa_grid())
    y = oracle.ref_exp(x, 1).astype(np.float64)
    assert np.all(np.diff(y[np.isfinite(y)]) >= 0.0) and np.all(np.isinf(y[x >= 88.72284]))
    # exp_mode 0 is libm
    xm = np.linspace(-30, 30, 1001).astype(np.float32)
    np.testing.assert_allclose(oracle.ref_exp(xm, 0), np.exp(xm.astype(np.float64)), rtol=3e-7)


# ---- Rbf16 (reference rounding points) ---------------------------------------------------------------
def to_bits_case(c):
    b = oracle.to_bf16_bits
    return dict(x=b(c["x"]), wq=b(c["wq"]), wk=b(c["wk"]), wv=b(c["wv"]), wg=b(c["wg"]), bg=c["bg"], wo=b(c["wo"]),
                bo=c["bo"], bias=b(c["bias"]), nb=None if c["nb"] is None else b(c["nb"]), nheads=c["nheads"])


def run_bf16(cb, **kw):
    return oracle.gating_attention_bf16(cb["x"], cb["wq"], cb["wk"], cb["wv"], cb["wg"], cb["bg"], cb["wo"], cb["bo"],
                                        cb["bias"], cb["nb"], cb["nheads"], **kw)


@pytest.mark.parametrize("exp_mode", [0, 1])
def test_bf16_restatement_close_to_fp32_oracle(exp_mode):
    c = make_case(21, 3, 48, 4, 32, bias_mode="random_mask")
    cb = to_bits_case(c)
    # the fp32 oracle sees the same bf16-rounded inputs
    cr = {k: (oracle.from_bf16_bits(v) if isinstance(v, np.ndarray) and v.dtype == np.uint16 else v)
          for k, v in cb.items()}
    ref = run_f32(cr)
    got = oracle.from_bf16_bits(run_bf16(cb, exp_mode=exp_mode))
    err = np.abs(got - ref)
    assert np.all(err <= 2e-2 + 1e-2 * np.abs(ref)), float(err.max())


def test_bf16_restatement_independent_of_block_size():
    c = make_case(22, 2, 37, 2, 32)
    cb = to_bits_case(c)
    outs = [run_bf16(cb, block_size=bs) for bs in (1, 5, 16, 37, 64)]
    for o in outs[1:]:
        np.testing.assert_array_equal(o, outs[0])


def test_bf16_restatement_scratch_layouts():
    """q/k/gate/avg come back [B,S,H,d]; v comes back [H,d,B,S] (reference gating_attention.cpp:57-61)."""
    c = make_case(23, 2, 9, 2, 32)
    cb = to_bits_case(c)
    _, s = run_bf16(cb, return_scratch=True)
    x = oracle.from_bf16_bits(cb["x"]).astype(np.float64)
    B, S, C = x.shape
    v_ref = x @ oracle.from_bf16_bits(cb["wv"]).astype(np.float64).T  # [B,S,C]
    v_got = oracle.from_bf16_bits(s["v"]).transpose(2, 3, 0, 1).reshape(B, S, C)
    np.testing.assert_allclose(v_got, v_ref, rtol=1e-2, atol=1e-2)
    q_ref = x @ oracle.from_bf16_bits(cb["wq"]).astype(np.float64).T
    np.testing.assert_allclose(oracle.from_bf16_bits(s["q"]), q_ref, rtol=1e-2, atol=1e-2)


# ---- row operators -----------------------------------------------------------------------------------
def test_bf16_conversion_matches_torch():
    rng = np.random.Generator(np.random.PCG64(31))
    a = np.concatenate([rng.standard_normal(4096).astype(np.float32) * 100,
                        np.array([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf, 1e-40],
                                 dtype=np.float32)])
    bits = oracle.to_bf16_bits(a)
    ref = torch.from_numpy(a).bfloat16().view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(bits, ref)
    np.testing.assert_array_equal(oracle.from_bf16_bits(bits), torch.from_numpy(a).bfloat16().float().numpy())


@pytest.mark.parametrize("size", [128, 256, 37])
def test_layernorm_matches_torch(size):
    rng = np.random.Generator(np.random.PCG64(32))
    x = oracle.round_bf16(rng.standard_normal((50, size)).astype(np.float32) * 3 + 1)
    gamma = rng.standard_normal(size).astype(np.float32)
    beta = rng.standard_normal(size).astype(np.float32)
    got = oracle.from_bf16_bits(oracle.layernorm_rows_bf16(oracle.to_bf16_bits(x), gamma, beta, 1e-5))
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (size,), torch.from_numpy(gamma).double(),
                                         torch.from_numpy(beta).double(), 1e-5).numpy()
    # result is rounded to bf16: half an ulp (2^-9 relative) plus fp32 noise
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-6)
    f32 = oracle.layernorm_rows_f32(x, gamma, beta, 1e-5)
    np.testing.assert_allclose(f32, ref, rtol=1e-5, atol=1e-6)


def test_layernorm_constant_row_gives_beta_and_shift_invariance():
    size = 128
    gamma = np.linspace(0.5, 1.5, size).astype(np.float32)
    beta = np.linspace(-1, 1, size).astype(np.float32)
    const = np.full((1, size), 2.5, dtype=np.float32)
    got = oracle.from_bf16_bits(oracle.layernorm_rows_bf16(oracle.to_bf16_bits(const), gamma, beta, 1e-5))
    np.testing.assert_array_equal(got[0], oracle.round_bf16(beta))
    rng = np.random.Generator(np.random.PCG64(33))
    x = oracle.round_bf16(rng.integers(-8, 8, (4, size)).astype(np.float32) * 0.25)  # exactly representable
    a = oracle.layernorm_rows_bf16(oracle.to_bf16_bits(x), gamma, beta, 1e-5)
    b = oracle.layernorm_rows_bf16(oracle.to_bf16_bits(x + 16.0), gamma, beta, 1e-5)
    diff = np.abs(oracle.from_bf16_bits(a) - oracle.from_bf16_bits(b))
    assert np.all(diff <= 2.0 ** -7 * np.abs(oracle.from_bf16_bits(a)) + 1e-6)


def test_linear_matches_torch():
    rng = np.random.Generator(np.random.PCG64(34))
    act = oracle.round_bf16(rng.standard_normal((37, 128)).astype(np.float32))
    w = oracle.round_bf16(rng.standard_normal((4, 128)).astype(np.float32) / 11)
    bias = rng.standard_normal(4).astype(np.float32)
    ref = torch.nn.functional.linear(torch.from_numpy(act).double(), torch.from_numpy(w).double(),
                                     torch.from_numpy(bias).double()).numpy()
    got = oracle.from_bf16_bits(oracle.linear_bf16(oracle.to_bf16_bits(act), oracle.to_bf16_bits(w), bias))
    assert np.all(np.abs(got - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-6)
    np.testing.assert_allclose(oracle.linear_f32(act, w, bias), ref, rtol=1e-6, atol=1e-6)
    # beta accumulates into the existing result
    prev = oracle.round_bf16(rng.standard_normal((37, 4)).astype(np.float32))
    got2 = oracle.from_bf16_bits(oracle.linear_bf16(oracle.to_bf16_bits(act), oracle.to_bf16_bits(w), None, beta=1.0,
                                                    result_bits=oracle.to_bf16_bits(prev)))
    ref2 = ref - bias + prev
    assert np.all(np.abs(got2 - ref2) <= 2.0 ** -8 * np.abs(ref2) + 1e-6)


# ---- global (extra-MSA column) attention: reference src/attention/global_attention.cpp:30-164 ---------------------
def make_global_case(seed, B, S, H, d, mask_mode="random"):
    rng = np.random.Generator(np.random.PCG64(seed))
    C = H * d
    f = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    mask = np.ones((B, S), dtype=np.float32)
    if mask_mode == "random":
        mask = (rng.random((B, S)) > 0.3).astype(np.float32)
        mask[:, 0] = 1
    return dict(x=f(B, S, C), mask=mask, wq=f(C, C) / math.sqrt(C), wk=f(d, C) / math.sqrt(C), wv=f(d, C) / math.sqrt(C),
                wg=f(C, C) / math.sqrt(C), bg=f(C), wo=f(C, C) / math.sqrt(C), bo=f(C), nheads=H)


def run_global(c, fn=None, **kw):
    fn = fn or oracle.global_attention_f32
    return fn(c["x"], c["mask"], c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"], c["bo"], c["nheads"], **kw)


@pytest.mark.parametrize("mask_mode", ["ones", "random"])
def test_global_numpy_twin_matches_torch_sdpa(mask_mode):
    """Library routine: torch scaled_dot_product_attention with one query per head and a shared key/value head."""
    c = make_global_case(11, 3, 19, 4, 16, mask_mode)
    t = lambda a: torch.from_numpy(np.asarray(a, dtype=np.float64))  # noqa: E731
    x, mask = t(c["x"]), t(c["mask"])
    B, S, C = x.shape
    H, d = c["nheads"], C // c["nheads"]
    q_avg = (mask[:, :, None] * x).sum(1) / (mask.sum(1, keepdim=True) + 1e-10)
    q = torch.nn.functional.linear(q_avg, t(c["wq"])).reshape(B, H, 1, d)
    k = torch.nn.functional.linear(x, t(c["wk"]))[:, None].expand(B, H, S, d)
    v = torch.nn.functional.linear(x, t(c["wv"]))[:, None].expand(B, H, S, d)
    bias = (1e9 * (mask - 1))[:, None, None, :]
    wavg = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=bias, scale=1 / math.sqrt(d))
    gate = torch.sigmoid(torch.nn.functional.linear(x, t(c["wg"]), t(c["bg"])))
    out = torch.nn.functional.linear(gate * wavg.reshape(B, 1, C), t(c["wo"]), t(c["bo"]))
    # the twin forms the mask bias and adds it in fp32, as the reference does: 1e-7-level differences to float64
    np.testing.assert_allclose(run_global(c, oracle.global_attention_f64_numpy), out.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("shape", [(2, 5, 2, 4), (3, 37, 8, 8), (1, 64, 4, 16)])
def test_global_c_oracle_matches_numpy_twin(shape):
    c = make_global_case(12, *shape)
    c["mask"][-1] = 0  # one fully masked row
    np.testing.assert_allclose(run_global(c), run_global(c, oracle.global_attention_f64_numpy), rtol=2e-5, atol=2e-6)


def test_global_c_oracle_matches_python_bruteforce():
    """Every index written out, on a case small enough for pure Python loops."""
    c = make_global_case(13, 2, 4, 2, 3)
    x, mask = c["x"].astype(float), c["mask"].astype(float)
    B, S, C = x.shape
    H, d = 2, 3
    out = np.zeros((B, S, C))
    for b in range(B):
        msum = sum(mask[b, s] for s in range(S))
        q_avg = [sum(mask[b, s] * x[b, s, ch] for s in range(S)) / (msum + 1e-10) for ch in range(C)]
        q = [sum(q_avg[ch] * float(c["wq"][o, ch]) for ch in range(C)) for o in range(C)]
        k = [[sum(x[b, s, ch] * float(c["wk"][e, ch]) for ch in range(C)) for e in range(d)] for s in range(S)]
        v = [[sum(x[b, s, ch] * float(c["wv"][e, ch]) for ch in range(C)) for e in range(d)] for s in range(S)]
        wavg = [0.0] * C
        for h in range(H):
            logit = [sum(q[h * d + e] * k[s][e] for e in range(d)) / math.sqrt(d) + 1e9 * (mask[b, s] - 1) for s in range(S)]
            m = max(logit)
            pe = [math.exp(v_ - m) for v_ in logit]
            z = sum(pe)
            for e in range(d):
                wavg[h * d + e] = sum(pe[s] / z * v[s][e] for s in range(S))
        for s in range(S):
            gated = [wavg[o] / (1 + math.exp(-(sum(x[b, s, ch] * float(c["wg"][o, ch]) for ch in range(C)) + float(c["bg"][o]))))
                     for o in range(C)]
            for o in range(C):
                out[b, s, o] = sum(gated[ch] * float(c["wo"][o, ch]) for ch in range(C)) + float(c["bo"][o])
    np.testing.assert_allclose(run_global(c), out, rtol=2e-5, atol=2e-6)


def test_global_closed_forms():
    c = make_global_case(14, 2, 9, 4, 4, "ones")
    C = 16
    # zero query weight -> uniform attention -> the weighted average is the plain mean of v over the row
    c0 = dict(c, wq=np.zeros_like(c["wq"]), wg=np.zeros_like(c["wg"]), bg=np.zeros(C, np.float32))
    v = c["x"].astype(np.float64) @ c["wv"].astype(np.float64).T          # [B,S,d]
    wavg = np.tile(v.mean(axis=1), (1, 4))                                # every head sees the same mean
    expect = (0.5 * wavg) @ c["wo"].astype(np.float64).T + c["bo"]        # gate = sigmoid(0) = 0.5, same for every token
    got = run_global(c0)
    np.testing.assert_allclose(got, np.broadcast_to(expect[:, None, :], got.shape), rtol=2e-5, atol=2e-6)
    # zero output weight -> the output bias
    np.testing.assert_allclose(run_global(dict(c, wo=np.zeros_like(c["wo"]))), np.broadcast_to(c["bo"], got.shape),
                               rtol=0, atol=1e-7)


def test_global_masked_token_has_no_influence_on_the_others_and_q_avg_ignores_it():
    c = make_global_case(15, 2, 11, 8, 8)
    c["mask"][:, 3] = 0
    base, qa = run_global(c, return_q_avg=True)
    c2 = dict(c, x=c["x"].copy())
    c2["x"][:, 3] = 7.0 * c2["x"][:, 3] + 1.0
    moved, qa2 = run_global(c2, return_q_avg=True)
    others = [s for s in range(11) if s != 3]
    np.testing.assert_array_equal(qa, qa2)
    np.testing.assert_array_equal(base[:, others], moved[:, others])
    assert np.abs(base[:, 3] - moved[:, 3]).max() > 1e-3  # the token's own gate does change its own output


def test_global_fully_masked_row_attends_uniformly():
    c = make_global_case(16, 2, 13, 8, 8, "ones")
    c["mask"][1] = 0
    out, qa = run_global(c, return_q_avg=True)
    assert np.all(qa[1] == 0)
    uni = dict(c, mask=np.ones_like(c["mask"]), wq=np.zeros_like(c["wq"]))
    np.testing.assert_allclose(out[1], run_global(uni)[1], rtol=2e-5, atol=2e-6)


def test_global_token_permutation_permutes_output():
    c = make_global_case(17, 2, 10, 4, 16)
    perm = np.random.Generator(np.random.PCG64(5)).permutation(10)
    c2 = dict(c, x=c["x"][:, perm].copy(), mask=c["mask"][:, perm].copy())
    np.testing.assert_allclose(run_global(c2), run_global(c)[:, perm], rtol=2e-5, atol=2e-6)


# ---- transition and triangle multiplication: reference src/attention/transition.cpp:21-39,
# ---- src/attention/triangle_multiplication.cpp:25-150 -------------------------------------------------------------
def make_pair_case(seed, n_res, n_gather, c_o, c_i):
    rng = np.random.Generator(np.random.PCG64(seed))
    f = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    return dict(x=f(n_res, n_gather, c_o), mask=(rng.random((n_res, n_gather)) > 0.2).astype(np.float32),
                pw=f(c_i, c_o) / math.sqrt(c_o), pb=f(c_i), gw=f(c_i, c_o) / math.sqrt(c_o), gb=f(c_i),
                w1=f(c_i, c_o) / math.sqrt(c_o), b1=f(c_i), w2=f(c_o, c_i) / math.sqrt(c_i), b2=f(c_o),
                left=f(c_i, n_gather, n_gather), right=f(c_i, n_gather, n_gather))


def test_transition_matches_torch_and_bruteforce():
    c = make_pair_case(50, 3, 5, 8, 12)
    out, mid = oracle.transition_f32(c["x"].reshape(-1, 8), c["w1"], c["b1"], c["w2"], c["b2"], return_mid=True)
    t = lambda a: torch.from_numpy(a).double()  # noqa: E731
    h = torch.relu(torch.nn.functional.linear(t(c["x"]).reshape(-1, 8), t(c["w1"]), t(c["b1"])))
    ref = torch.nn.functional.linear(h, t(c["w2"]), t(c["b2"]))
    np.testing.assert_allclose(mid, h.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(out, ref.numpy(), rtol=1e-6, atol=1e-6)
    # pure-Python loops, index by index, on the first two rows
    x = c["x"].reshape(-1, 8).astype(float)
    for r in range(2):
        hid = [max(0.0, sum(x[r][k] * float(c["w1"][j][k]) for k in range(8)) + float(c["b1"][j])) for j in range(12)]
        for o in range(8):
            want = sum(hid[j] * float(c["w2"][o][j]) for j in range(12)) + float(c["b2"][o])
            assert abs(out[r][o] - want) < 1e-5


def test_transition_closed_forms():
    c = make_pair_case(51, 2, 4, 8, 12)
    x = c["x"].reshape(-1, 8)
    # zero first weight: the hidden layer is relu(b1) for every row
    out = oracle.transition_f32(x, np.zeros_like(c["w1"]), c["b1"], c["w2"], c["b2"])
    want = np.maximum(c["b1"].astype(np.float64), 0) @ c["w2"].astype(np.float64).T + c["b2"]
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6, atol=1e-6)
    # a very negative first bias switches every hidden unit off: out == b2
    out = oracle.transition_f32(x, c["w1"], np.full(12, -1e4, np.float32), c["w2"], c["b2"])
    np.testing.assert_allclose(out, np.broadcast_to(c["b2"], out.shape), rtol=0, atol=0)
    # a very positive first bias makes the ReLU the identity: the layer pair collapses to one affine map
    big = np.full(12, 1e3, np.float32)
    out = oracle.transition_f32(x, c["w1"], big, c["w2"], c["b2"])
    w = c["w2"].astype(np.float64) @ c["w1"].astype(np.float64)
    want = x.astype(np.float64) @ w.T + c["w2"].astype(np.float64) @ big + c["b2"]
    np.testing.assert_allclose(out, want, rtol=1e-5, atol=1e-3)


def test_tm_calc_proj_matches_torch_and_closed_forms():
    c = make_pair_case(52, 4, 6, 8, 5)
    got = oracle.tm_calc_proj_f32(c["x"], c["mask"], c["pw"], c["pb"], c["gw"], c["gb"])
    t = lambda a: torch.from_numpy(a).double()  # noqa: E731
    p = torch.nn.functional.linear(t(c["x"]), t(c["pw"]), t(c["pb"]))       # [i, j, c]
    g = torch.sigmoid(torch.nn.functional.linear(t(c["x"]), t(c["gw"]), t(c["gb"])))
    ref = (p * t(c["mask"])[..., None] * g).permute(2, 0, 1)               # channel-first, as the reference stores it
    np.testing.assert_allclose(got, ref.numpy(), rtol=1e-6, atol=1e-6)
    assert got.shape == (5, 4, 6)
    # masked positions are exactly zero, in every channel
    assert np.all(got[:, c["mask"] == 0] == 0)
    # gate weights zero and gate bias 0 -> sigmoid(0) = 1/2; gate bias +40 -> gate 1
    half = oracle.tm_calc_proj_f32(c["x"], c["mask"], c["pw"], c["pb"], np.zeros_like(c["gw"]), np.zeros_like(c["gb"]))
    one = oracle.tm_calc_proj_f32(c["x"], c["mask"], c["pw"], c["pb"], np.zeros_like(c["gw"]), np.full(5, 40, np.float32))
    np.testing.assert_allclose(2 * half, one, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(one, (p * t(c["mask"])[..., None]).permute(2, 0, 1).numpy(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("incoming", [False, True])
def test_tm_equation_matches_einsum_and_bruteforce(incoming):
    c = make_pair_case(53, 7, 7, 4, 3)
    got = oracle.tm_equation_f32(c["left"], c["right"], incoming)
    le, ri = torch.from_numpy(c["left"]).double(), torch.from_numpy(c["right"]).double()
    # AlphaFold's equations with channel-first operands: outgoing 'ikc,jkc->ijc', incoming 'kjc,kic->ijc'
    ref = torch.einsum("ckj,cki->cij", le, ri) if incoming else torch.einsum("cik,cjk->cij", le, ri)
    np.testing.assert_allclose(got, ref.numpy(), rtol=1e-6, atol=1e-6)
    ch, i, j = 2, 3, 5
    if incoming:
        want = sum(float(c["right"][ch, k, i]) * float(c["left"][ch, k, j]) for k in range(7))
    else:
        want = sum(float(c["left"][ch, i, k]) * float(c["right"][ch, j, k]) for k in range(7))
    assert abs(got[ch, i, j] - want) < 1e-5


def test_tm_equation_identities():
    c = make_pair_case(54, 6, 6, 4, 2)
    eye = np.broadcast_to(np.eye(6, dtype=np.float32), (2, 6, 6)).copy()
    # outgoing with right = I returns left; incoming with right = I returns left as well (sum_k I[k,i] left[k,j])
    np.testing.assert_array_equal(oracle.tm_equation_f32(c["left"], eye, False), c["left"])
    np.testing.assert_array_equal(oracle.tm_equation_f32(c["left"], eye, True), c["left"])
    # outgoing with left = I returns right transposed; the two equations are not symmetric in their operands
    np.testing.assert_array_equal(oracle.tm_equation_f32(eye, c["right"], False), c["right"].transpose(0, 2, 1))
    np.testing.assert_array_equal(oracle.tm_equation_f32(eye, c["right"], True), c["right"].transpose(0, 2, 1))
    # incoming(left, right) == outgoing(right^T, left^T)
    a = oracle.tm_equation_f32(c["left"], c["right"], True)
    b = oracle.tm_equation_f32(np.ascontiguousarray(c["right"].transpose(0, 2, 1)),
                               np.ascontiguousarray(c["left"].transpose(0, 2, 1)), False)
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-6)


def test_tm_output_step_matches_torch():
    c = make_pair_case(55, 3, 4, 8, 5)
    rng = np.random.Generator(np.random.PCG64(56))
    center = rng.standard_normal((3, 4, 5)).astype(np.float32)
    gating_w, gating_b = rng.standard_normal((8, 8)).astype(np.float32), rng.standard_normal(8).astype(np.float32)
    out_w, out_b = rng.standard_normal((8, 5)).astype(np.float32), rng.standard_normal(8).astype(np.float32)
    gate, out = oracle.tm_gate_and_out_f32(c["x"], center, gating_w, gating_b, out_w, out_b)
    t = lambda a: torch.from_numpy(a).double()  # noqa: E731
    g_ref = torch.nn.functional.linear(t(c["x"]).reshape(-1, 8), t(gating_w), t(gating_b))
    o_ref = torch.nn.functional.linear(t(center).reshape(-1, 5), t(out_w), t(out_b))
    np.testing.assert_allclose(gate, g_ref.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(out, o_ref.numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(oracle.tm_last_f32(out, gate), (o_ref * torch.sigmoid(g_ref)).numpy(), rtol=1e-6, atol=1e-6)
    np.testing.assert_array_equal(oracle.tm_last_f32(out, np.full_like(gate, 100.0)), out)


def test_pair_stack_oracle_matches_golden_fixture():
    """tests/golden/pair_stack_tiny.npz (float64 einsum expressions, made by tests/golden/make_golden_pair_stack.py)."""
    g = np.load(os.path.join(HERE, "golden", "pair_stack_tiny.npz"))
    i = lambda k: g["in." + k]  # noqa: E731
    out, mid = oracle.transition_f32(i("x").reshape(-1, 8), i("w1"), i("b1"), i("w2"), i("b2"), return_mid=True)
    np.testing.assert_allclose(mid.reshape(6, 6, 12), g["transition.mid"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(out.reshape(6, 6, 8), g["transition.out"], rtol=1e-5, atol=1e-5)
    left = oracle.tm_calc_proj_f32(i("x"), i("mask"), i("left_w"), i("left_b"), i("left_gw"), i("left_gb"))
    right = oracle.tm_calc_proj_f32(i("x"), i("mask"), i("right_w"), i("right_b"), i("right_gw"), i("right_gb"))
    np.testing.assert_allclose(left, g["tm.left"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(right, g["tm.right"], rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.tm_equation_f32(left, right, False), g["tm.outgoing"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.tm_equation_f32(left, right, True), g["tm.incoming"], rtol=1e-5, atol=1e-5)
    gate, proj = oracle.tm_gate_and_out_f32(i("x"), i("center"), i("gating_w"), i("gating_b"), i("out_w"), i("out_b"))
    np.testing.assert_allclose(gate.reshape(6, 6, 8), g["tm.gate"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(proj.reshape(6, 6, 8), g["tm.out"], rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.tm_last_f32(proj, gate).reshape(6, 6, 8), g["tm.last"], rtol=1e-5, atol=1e-5)
