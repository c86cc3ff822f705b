"""Parity of the HIP path against the CPU oracle, through the C ABI, on a real MI355X.

Every test calls libkutacc.so (handle-based kutacc_af2_* entry points, or the pointer-level
kutacc_hip_* layer where a kernel family is forced) on device memory and compares with
oracle/ on the same seeded inputs.  Full-size configurations are run at their real shape on the
GPU; the oracle evaluates a subset of batch rows (rows are independent in this operator), chosen to
include masked rows where the configuration has them.

Tolerances (stated by the task): fp32 storage within 1e-4 relative of the fp32 oracle; bf16 storage
within 2e-2 absolute + 1e-2 relative of the fp32 oracle.
"""
import ctypes
import functools

import numpy as np
import pytest

from kutacc_amd import capi
from kutacc_amd.workloads import CONFIGS, Workload, bf16_bits, make_workload, round_to_bf16

import helpers

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.set_stream(None)
    capi.set_blocking(True)
    return torch


@functools.lru_cache(maxsize=2)
def full_workload(config: int) -> Workload:
    """Full-size inputs are expensive to draw (config 5: 134M normals); tests must not modify them."""
    return make_workload(config)


def oracle_rows(w: Workload, rows):
    sub = w.batch_slice(rows)
    return helpers.oracle_out(sub, return_avg=True)


def pick_rows(w: Workload):
    """Batch rows the oracle evaluates at full shape.  Configurations 1 to 3: every row (the fp32 oracle takes seconds).
    Configurations 4 and 5 (one workgroup per (row, head), dealt to the XCDs by row index modulo 8): the first and the last
    sixteen rows -- both ends of every XCD's range, and for configuration 5 the fully masked rows and the last one that is
    not -- plus sixteen spread over the rest."""
    if w.config in (1, 2, 3):
        return list(range(w.B))
    rows = set(range(16)) | set(range(w.B - 16, w.B)) | set(int(r) for r in np.linspace(16, w.B - 17, 16))
    pad = w.extras.get("pad", 0) if w.config == 5 else 0
    if pad:
        rows |= {w.B - pad - 2, w.B - pad - 1, w.B - pad, w.B - pad + 1}
    return sorted(r for r in rows if 0 <= r < w.B)


# ---- the five configurations, full shape, default kernel selection -------------------------------------
@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_config_full_shape_matches_oracle(torch_cuda, config):
    torch = torch_cuda
    w = full_workload(config)
    print(f"config {config}: B={w.B} S={w.S} H={w.H} dtype={w.dtype}", flush=True)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag()
    if w.dtype == "bf16":
        assert capi.last_path() == "fused_mfma", "bf16 benchmark shapes must run on the MFMA kernels"
    rows = pick_rows(w)
    ref_out, ref_avg = oracle_rows(w, rows)
    out = helpers.to_numpy(ten["out"][rows])
    avg = helpers.to_numpy(scratch["avg"][rows]).reshape(len(rows), w.S, w.C)
    e_avg = helpers.check_close(avg, ref_avg, w.dtype, f"config {config} gated average")
    e_out = helpers.check_close(out, ref_out, w.dtype, f"config {config} out")
    print(f"config {config}: path={capi.last_path()} rows checked {len(rows)} of {w.B} max|err| avg={e_avg:.3g} out={e_out:.3g}",
          flush=True)
    assert bool(torch.isfinite(ten["out"]).all()) and bool(torch.isfinite(scratch["avg"]).all())
    if len(rows) < w.B:
        # Every other row: against the shape-agnostic kernels on the same inputs (an independent kernel family that the
        # reduced-shape tests hold to the oracle row by row).  Both round to bf16 within the parity bar of the fp32
        # oracle, so they agree within that bar of each other.
        ten2, scratch2 = helpers.to_device(w)
        rc = helpers.run_hip(w, ten2, scratch2, capi.PATH_GENERIC)
        assert rc == 0 and capi.last_path() == "generic"
        for name, a, b in (("out", ten["out"], ten2["out"]), ("avg", scratch["avg"].reshape(w.B, w.S, w.C),
                                                             scratch2["avg"].reshape(w.B, w.S, w.C))):
            a, b = a.float(), b.float()
            excess = ((a - b).abs() - (2e-2 + 1e-2 * b.abs())).amax(dim=(1, 2))  # per batch row
            worst = int(excess.argmax())
            assert float(excess.max()) <= 0.0, f"config {config} {name}: batch row {worst} differs from the generic kernels"
            # a per-row checksum: the mean of a row's elements agrees far inside the element-wise bar
            d = (a.double().mean(dim=(1, 2)) - b.double().mean(dim=(1, 2))).abs()
            assert float(d.max()) < 2e-3, f"config {config} {name}: checksum of batch row {int(d.argmax())}"


# ---- both kernel families on reduced shapes, every row checked ---------------------------------------------
SMALL = [
    # config, batch, seq_len
    (1, 3, 64), (2, 4, 256), (3, 5, 384), (4, 3, 1024), (5, 3, 1024),
    (2, 3, 70), (3, 2, 33), (2, 2, 1), (3, 2, 200), (4, 2, 97),
    # ragged lengths with enough batch rows for the fragment-major pair-bias copy to fit the q scratch tensor
    (3, 24, 200), (2, 16, 70), (3, 8, 33), (5, 12, 321),
    # between the persistent kernel's reach and 1024 keys: two and three query blocks per wave of the long-sequence
    # kernel, an odd number of key tiles, with and without the fragment-major pair bias (it needs batch rows enough)
    (5, 3, 512), (5, 20, 450), (5, 2, 650), (4, 2, 768), (4, 3, 400), (3, 16, 736),
    # 256 channels, four query blocks per wave: the weights lie on the V array there; an odd tile count with seven waves,
    # a V array shorter than the weights with five waves, a ragged last block at eight waves
    (4, 2, 800), (4, 3, 640), (4, 2, 1000),
]


@pytest.mark.parametrize("config,batch,seq", SMALL)
@pytest.mark.parametrize("path", [capi.PATH_GENERIC, capi.PATH_FUSED])
def test_reduced_shapes_both_kernel_families(torch_cuda, config, batch, seq, path):
    w = make_workload(config, batch=batch, seq_len=seq)
    if config == 5:
        w.bias[-1, :] = round_to_bf16(np.full(seq, -1e9, dtype=np.float32))  # a fully masked row
    print(f"config {config} B={batch} S={seq} path={path}", flush=True)
    ten, scratch = helpers.to_device(w)
    rc = helpers.run_hip(w, ten, scratch, path)
    assert rc == 0, rc
    if path == capi.PATH_FUSED:
        assert capi.last_path() == ("fused_mfma" if w.dtype == "bf16" else "fp32_mfma")
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, w.dtype, "out")


@pytest.mark.parametrize("config,batch,seq", [c for c in SMALL if c[2] <= 224] + [(2, 5, 224), (3, 4, 129), (4, 3, 160)])
def test_fp32_storage_on_the_fp32_matrix_core(torch_cuda, config, batch, seq):
    """Every reduced shape of up to 224 positions with its tensors stored as fp32 (the values are those of the bf16
    workload, which fp32 holds exactly): the fp32 MFMA path, held to the fp32 bar -- 1e-4 relative (+ 1e-5) of the fp32
    oracle -- with masks, ragged lengths, fully masked rows, with and without pair bias, 128 and 256 channels."""
    w = make_workload(config, batch=batch, seq_len=seq)
    w.dtype = "fp32"
    if config == 5:
        w.bias[-1, :] = -1e9  # a fully masked row
    ten, scratch = helpers.to_device(w)
    rc = helpers.run_hip(w, ten, scratch, capi.PATH_FUSED)
    assert rc == 0 and capi.last_path() == "fp32_mfma", (rc, capi.last_path())
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, "fp32", "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, "fp32", "out")
    for name in ("q", "k", "v", "gate"):
        assert not bool(scratch[name].any()), f"{name} was written"


def test_fp32_storage_beyond_the_matrix_core_path_takes_the_generic_kernels(torch_cuda):
    w = make_workload(1, batch=2, seq_len=225)
    ten, scratch = helpers.to_device(w)
    assert helpers.run_hip(w, ten, scratch, capi.PATH_FUSED) == capi.EUNSUPPORTED
    assert helpers.run_hip(w, ten, scratch, capi.PATH_AUTO) == 0 and capi.last_path() == "generic"
    helpers.check_close(helpers.to_numpy(ten["out"]), helpers.oracle_out(w), "fp32", "out")


@pytest.mark.parametrize("config,batch,seq,plan", [
    # 256 channels: two matrices per group (rows staged through the block's own K/V slots, groups walked backwards), one
    # per group (fragments loaded straight from global memory), and four blocks per wave well below the lengths that pick it
    (4, 2, 512, "2,2"), (4, 2, 500, "3,1"), (4, 2, 512, "4,4"), (4, 3, 300, "2,1"),
    # 128 channels with more blocks per wave than the planner would take
    (5, 3, 384, "2,4"), (5, 2, 330, "4,4"),
])
def test_forced_kernel_plans_match_the_oracle(torch_cuda, config, batch, seq, plan):
    """Routes of the long-sequence kernel that the planner only takes on a device with less LDS, forced through the
    library's tuning hook."""
    w = make_workload(config, batch=batch, seq_len=seq)
    print(f"config {config} B={batch} S={seq} plan={plan}", flush=True)
    ten, scratch = helpers.to_device(w)
    assert capi.set_tuning("plan", plan) == 0
    try:
        rc = helpers.run_hip(w, ten, scratch, capi.PATH_FUSED)
    finally:
        capi.set_tuning("plan", None)
    assert rc == 0, rc
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, w.dtype, "out")


def _sweep_cases():
    """24 seeded shapes over the whole range the MFMA kernels take: any sequence length up to 1024 (ragged tails, odd
    numbers of key tiles, every blocks-per-wave variant of the long-sequence kernel), both channel counts, with and without
    pair bias, batches small and large enough for the fragment-major pair bias, masks with random holes, masked tails
    and fully masked rows."""
    rng = np.random.Generator(np.random.PCG64(20240))
    cases = []
    for i in range(24):
        config = int(rng.choice([2, 3, 4, 5]))
        seq = int(rng.integers(1, 1025)) if i % 3 else int(rng.choice([31, 32, 33, 383, 385, 511, 513, 767, 1023]))
        batch = int(rng.integers(1, 5)) if i % 2 else int(rng.integers(8, 20))
        cases.append((i, config, batch, seq))
    return cases


@pytest.mark.parametrize("index,config,batch,seq", _sweep_cases())
def test_seeded_shape_sweep_matches_oracle(torch_cuda, index, config, batch, seq):
    w = make_workload(config, batch=batch, seq_len=seq)
    rng = np.random.Generator(np.random.PCG64(500 + index))
    kind = index % 4
    if kind == 1:    # random holes
        w.bias[:] = round_to_bf16(np.where(rng.random((batch, seq)) < 0.2, -1e9, 0.0).astype(np.float32))
    elif kind == 2:  # masked tails of random length, one fully masked row
        for b in range(batch):
            w.bias[b, seq - int(rng.integers(0, seq)):] = -1e9
        w.bias[batch - 1, :] = -1e9
    elif kind == 3:  # no mask at all
        w.bias[:] = 0.0
    print(f"sweep {index}: config {config} B={batch} S={seq} mask kind {kind}", flush=True)
    ten, scratch = helpers.to_device(w)
    rc = helpers.run_hip(w, ten, scratch, capi.PATH_FUSED)
    assert rc == 0, rc
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, f"sweep {index} gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, w.dtype, f"sweep {index} out")


# ---- the two-row persistent kernel (128 channels, up to 384 keys), forced wherever it can run --------------------------
@pytest.fixture
def row_pairs_forced():
    assert capi.set_tuning("row_pairs", "1") == 0
    yield
    capi.set_tuning("row_pairs", None)


PAIR_CASES = [
    # config, batch, seq_len, mask kind: None as drawn, "holes", "tails" (+ one fully masked row), "none", "soft" (a finite
    # additive bias on every key: the kernel adds it as two bf16 terms)
    (3, 16, 384, None), (3, 17, 384, "holes"), (3, 9, 200, None), (3, 24, 321, "tails"), (3, 3, 33, "holes"),
    (3, 1, 64, None), (3, 40, 96, "tails"), (5, 18, 352, None), (5, 7, 70, "holes"), (3, 1, 1, None), (3, 26, 383, "none"),
    # 256 channels, eight heads (up to 256 positions)
    (2, 16, 256, None), (2, 70, 200, "holes"), (2, 33, 129, "tails"), (2, 3, 33, None), (2, 64, 256, "none"), (4, 40, 224, "holes"),
    (3, 20, 160, "soft"), (2, 18, 96, "soft"),
]


@pytest.mark.parametrize("config,batch,seq,mask", PAIR_CASES)
@pytest.mark.parametrize("pair_bias", [True, False], ids=["pair bias", "no pair bias"])
def test_two_row_kernel_matches_the_oracle(torch_cuda, row_pairs_forced, config, batch, seq, mask, pair_bias):
    """Batches that leave workgroups with one, an odd and an even number of rows (a workgroup walks rows 8 * groups
    apart), ragged and odd tile counts, every mask kind, with and without pair bias; each row against the oracle."""
    w = make_workload(config, batch=batch, seq_len=seq)
    rng = np.random.Generator(np.random.PCG64(900 + batch + seq))
    if mask == "holes":
        w.bias[:] = round_to_bf16(np.where(rng.random((batch, seq)) < 0.2, -1e9, 0.0).astype(np.float32))
    elif mask == "tails":
        for b in range(batch):
            w.bias[b, seq - int(rng.integers(0, seq)):] = -1e9
        w.bias[batch - 1, :] = -1e9
    elif mask == "none":
        w.bias[:] = 0.0
    elif mask == "soft":
        w.bias[:] = round_to_bf16((rng.standard_normal((batch, seq)) * 3.0).astype(np.float32))
        w.bias[0, : seq // 2] = -np.inf
    if not pair_bias:
        w.nb = None
    ten, scratch = helpers.to_device(w)
    capi.set_tuning("debug", "1")
    try:
        rc = helpers.run_hip(w, ten, scratch, capi.PATH_FUSED)
    finally:
        capi.set_tuning("debug", "0")
    assert rc == 0, rc
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, w.dtype, "out")


def test_two_row_kernel_is_what_the_headline_shape_runs(torch_cuda, capfd):
    """Configuration 3 at a batch that gives every workgroup two rows takes the two-row kernel by itself, and a large
    pair-bias offset (overflow / underflow repeat with shifted rows) leaves its result where the oracle has it."""
    w = make_workload(3, batch=128)
    ten, scratch = helpers.to_device(w)
    capi.set_tuning("debug", "1")
    try:
        assert helpers.run_hip(w, ten, scratch, capi.PATH_FUSED) == 0
    finally:
        capi.set_tuning("debug", "0")
    assert "row_pairs=1" in capfd.readouterr().err
    rows = [0, 1, 63, 64, 127]
    ref_out, _ = oracle_rows(w, rows)
    helpers.check_close(helpers.to_numpy(ten["out"][rows]), ref_out, w.dtype, "two-row kernel, config 3")
    # a constant pair bias of +-150 (exact in bf16; far outside what 2^logit holds unshifted): equals no pair bias at all
    w0 = make_workload(3, batch=128)
    w0.nb = np.zeros_like(w0.nb)
    ref0, _ = oracle_rows(w0, rows)
    for offset in (150.0, -150.0):
        w2 = make_workload(3, batch=128)
        w2.nb = np.full_like(w2.nb, offset)
        ten2, scratch2 = helpers.to_device(w2)
        assert helpers.run_hip(w2, ten2, scratch2, capi.PATH_FUSED) == 0
        helpers.check_close(helpers.to_numpy(ten2["out"][rows]), ref0, w.dtype, f"two-row kernel, constant pair bias {offset:+}")


def test_fp32_storage_meets_fp32_tolerance(torch_cuda):
    w = make_workload(1)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag() and capi.last_path() == "fp32_mfma"  # the fp32 matrix core, not the scalar kernels
    ref = helpers.oracle_out(w)
    got = helpers.to_numpy(ten["out"])
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5)


# ---- properties that hold at any size -----------------------------------------------------------------------
def test_result_independent_of_block_size(torch_cuda):
    """The reference computes full-row softmax whatever the query tiling (gating_attention.cpp:102-121)."""
    w = make_workload(3, batch=6)
    outs = []
    for bs in (1, 64, 384, 1000):
        op, ten, scratch = helpers.make_op(w, block_size=bs)
        op.run()
        assert not capi.error_flag()
        outs.append(ten["out"].clone())
    for o in outs[1:]:
        assert helpers.same_bits(o, outs[0])


def test_batch_permutation_permutes_output(torch_cuda):
    w = make_workload(2, batch=16)
    op, ten, _ = helpers.make_op(w)
    op.run()
    perm = np.random.Generator(np.random.PCG64(9)).permutation(w.B)
    w2 = w.batch_slice(perm)
    op2, ten2, _ = helpers.make_op(w2)
    op2.run()
    assert helpers.same_bits(ten2["out"], ten["out"][torch_cuda.from_numpy(perm).cuda()])


def test_fully_masked_rows_average_values_uniformly_full_size(torch_cuda):
    """Config 5 at full size: every query of a fully masked batch row gets the plain mean of V (times
    its gate), because the -1e9 mask bias absorbs the logits in fp32."""
    w = full_workload(5)
    pad = w.extras["pad"]
    assert pad > 0
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag()
    rows = [w.B - pad, w.B - 1]
    x = w.x[rows].astype(np.float64)
    v = x @ w.wv.astype(np.float64).T
    gate = 1 / (1 + np.exp(-(x @ w.wg.astype(np.float64).T + w.bg)))
    expect = v.mean(axis=1, keepdims=True) * gate
    got = helpers.to_numpy(scratch["avg"][rows]).reshape(2, w.S, w.C)
    helpers.check_close(got, expect, "bf16", "uniform average of fully masked rows")


@pytest.mark.parametrize("offset", [150.0, -150.0])
def test_uniform_pair_bias_offset_changes_nothing(torch_cuda, offset):
    """Softmax is shift invariant: a constant added to the whole pair bias must leave the result alone.
    +-150 is exact in bf16 and far outside what 2^logit can hold unshifted in fp32 (overflow above, a
    whole-row underflow below), so this drives the kernel's repeat with the true row maxima."""
    w = make_workload(3, batch=8, seq_len=128)
    op, ten, _ = helpers.make_op(w)
    op.run()
    w2 = w.batch_slice(np.arange(w.B))
    w2.nb = np.full_like(w.nb, offset)
    w3 = w.batch_slice(np.arange(w.B))
    w3.nb = np.zeros_like(w.nb)
    op2, ten2, _ = helpers.make_op(w2)
    op2.run()
    op3, ten3, _ = helpers.make_op(w3)
    op3.run()
    assert not capi.error_flag()
    a, b2 = helpers.to_numpy(ten3["out"]), helpers.to_numpy(ten2["out"])
    assert np.isfinite(b2).all()
    helpers.assert_within(b2, a, 2.0 ** -7 * np.abs(a) + 3e-3, "constant pair bias vs zero pair bias")
    helpers.check_close(b2, helpers.oracle_out(w3), w.dtype, "constant pair bias vs oracle")


@pytest.mark.parametrize("seq_len,batch", [(128, 8), (384, 16), (520, 24)])
def test_large_pair_bias_keeps_its_precision(torch_cuda, seq_len, batch):
    """A pair bias with entries up to +-30, sigma 10 (what a trained pair representation can reach): the reference adds the
    bf16 values exactly in fp32 (src/attention/gating_attention.cpp:113-117).  The log2-unit route carries nb * log2(e) as
    fp16, 2^-12 of the bias at worst (0.007 nat at |nb| = 30, below the 2^-9 rounding of the bf16 probabilities themselves).
    Carried as bf16 (2^-9 of the bias, 0.06 nat) the same inputs miss the parity bar: 0.13-0.18 off on the gated average,
    rms 9e-3.  Bar here: 3e-2 + 1e-2 |ref| elementwise and rms error below 4e-3 (measured 2.0e-3; 1.7e-3 with the exact adds of
    the natural-log route); persistent kernel (128, 384 keys) and long-sequence kernel (520)."""
    w = make_workload(3, batch=batch, seq_len=seq_len)
    rng = np.random.default_rng(seq_len)
    w.nb = round_to_bf16(np.clip(rng.normal(0.0, 10.0, size=w.nb.shape), -30.0, 30.0).astype(np.float32))
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag() and capi.last_path() == "fused_mfma"
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    got = helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C)
    # elementwise 3e-2 + 1e-2 |ref| (the usual 2e-2 floor is passed by all but one element in 786 432: with logit gaps of
    # +-30 a softmax is nearly one-hot and a single bf16 rounding of q or k can move a weight; the exact-add route shows
    # the same tail)
    helpers.assert_within(got, ref_avg, 3e-2 + 1e-2 * np.abs(ref_avg), "gated average with a large pair bias")
    rms = float(np.sqrt(np.mean((got - ref_avg) ** 2)))
    assert rms < 4e-3, f"rms error of the gated average {rms:.3g}"
    helpers.assert_within(helpers.to_numpy(ten["out"]), ref_out, 3e-2 + 1e-2 * np.abs(ref_out), "out with a large pair bias")


@pytest.mark.parametrize("batch,seq_len", [(8, 160), (2, 160), (8, 520), (2, 520)])
@pytest.mark.parametrize("hole", [-1e9, -np.inf])
def test_pair_bias_entries_that_mask_single_pairs(torch_cuda, hole, batch, seq_len):
    """A pair bias used as a per-(query, key) mask: a tenth of its entries at -1e9 or -inf, never a whole row.  The
    reference's fp32 add (src/attention/gating_attention.cpp:113-117) gives those pairs zero weight.  The fragment-major
    copy carries them as the largest fp16 magnitude; the routes that read the pair bias in place (batch 2: the copy does
    not fit the q tensor) turn -inf into the most negative finite bf16 on its way into the selector product."""
    w = make_workload(3, batch=batch, seq_len=seq_len)
    rng = np.random.default_rng(5)
    holes = rng.random(w.nb.shape) < 0.1
    holes[..., 0] = False  # every query keeps at least one key
    w.nb = np.where(holes, np.float32(hole), w.nb).astype(np.float32)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag() and capi.last_path() == "fused_mfma"
    ref_out, ref_avg = helpers.oracle_out(w, return_avg=True)
    helpers.check_close(helpers.to_numpy(scratch["avg"]).reshape(w.B, w.S, w.C), ref_avg, w.dtype, "gated average")
    helpers.check_close(helpers.to_numpy(ten["out"]), ref_out, w.dtype, "out")


def test_fully_masked_and_leading_masked_rows_short_sequence(torch_cuda):
    """Rows whose every key is masked (uniform average of V) and rows whose first key tile is masked, at a
    sequence length the one-workgroup-per-head kernel handles."""
    w = make_workload(3, batch=8, seq_len=128)
    w.bias[1, :] = -1e9
    w.bias[2, :40] = -1e9
    w.bias[5, 100:] = -1e9
    op, ten, scratch = helpers.make_op(w)
    op.run()
    assert not capi.error_flag()
    helpers.check_close(helpers.to_numpy(ten["out"]), helpers.oracle_out(w), w.dtype, "masked rows")


def test_masked_keys_do_not_leak(torch_cuda):
    """Changing the token behind a masked key must not change any other row.  Not bit for bit: the
    kernel refreshes its running softmax maximum per 32-query block, so a changed neighbour query can
    shift WHEN a row rescales (never what it converges to); the bound is rounding noise of the bf16
    averages (3e-3 absolute on out), against a threefold change of the masked tokens."""
    w = make_workload(2, batch=4)
    masked = np.flatnonzero(w.bias[0] != 0)
    assert masked.size > 0
    op, ten, _ = helpers.make_op(w)
    op.run()
    w2 = w.batch_slice(np.arange(w.B))
    w2.x[:, masked] = round_to_bf16(np.float32(3.0) * w2.x[:, masked] + np.float32(1.0))
    op2, ten2, _ = helpers.make_op(w2)
    op2.run()
    keep = np.flatnonzero(w.bias[0] == 0)
    a, b2 = helpers.to_numpy(ten["out"])[:, keep], helpers.to_numpy(ten2["out"])[:, keep]
    helpers.assert_within(b2, a, 2.0 ** -7 * np.abs(a) + 3e-3, "rows behind unmasked keys")


@pytest.mark.parametrize("batch", [8, 3])
def test_absent_pair_bias_equals_zero_pair_bias(torch_cuda, batch):
    """nb = None and nb = 0 give the same result: bit for bit when both calls take the same kernel route
    (batch 8: the fragment-major copy of the pair bias fits the q scratch tensor), to rounding noise when
    they do not (batch 3: the zero pair bias is read in place, in natural-log units)."""
    w = make_workload(4, batch=batch, seq_len=256)
    op, ten, _ = helpers.make_op(w)
    op.run()
    w2 = w.batch_slice(np.arange(w.B))
    w2.nb = np.zeros((w.H, w.S, w.S), dtype=np.float32)
    op2, ten2, _ = helpers.make_op(w2)
    op2.run()
    assert not capi.error_flag()
    if batch == 8:
        assert helpers.same_bits(ten["out"], ten2["out"])
    else:
        a, b2 = helpers.to_numpy(ten["out"]), helpers.to_numpy(ten2["out"])
        helpers.assert_within(b2, a, 2.0 ** -7 * np.abs(a) + 3e-3, "zero pair bias vs none")


@pytest.mark.parametrize("nb_pad", [16, 3], ids=["pair-bias rows 16B-aligned", "pair-bias rows unaligned"])
@pytest.mark.parametrize("path", [capi.PATH_GENERIC, capi.PATH_FUSED])
def test_strided_tensors_through_the_launch_layer(torch_cuda, path, nb_pad):
    """Padded leading dimensions: input and out rows wider than C, a padded pair bias and mask bias.  Both kernel
    families must read and write only what the strides describe."""
    torch = torch_cuda
    w = make_workload(3, batch=6, seq_len=96)
    B, S, C, H = w.B, w.S, w.C, w.H
    ten, scratch = helpers.to_device(w)
    pad = 16
    x_p = torch.full((B * S, C + pad), 7.0, dtype=torch.bfloat16, device="cuda")
    x_p[:, :C] = ten["x"].reshape(B * S, C)
    out_p = torch.full((B * S, C + pad), -3.0, dtype=torch.bfloat16, device="cuda")
    nb_p = torch.full((H, S + 8, S + nb_pad), 5.0, dtype=torch.bfloat16, device="cuda")
    nb_p[:, :S, :S] = ten["nb"]
    bias_p = torch.full((B, S + pad), -1e9, dtype=torch.bfloat16, device="cuda")
    bias_p[:, :S] = ten["bias"]
    a = helpers.hip_args(w, ten, scratch, path)
    a.input, a.input_ld = x_p.data_ptr(), C + pad
    a.out, a.out_ld = out_p.data_ptr(), C + pad
    a.nonbatched_bias, a.nb_stride_h, a.nb_stride_q = nb_p.data_ptr(), (S + 8) * (S + nb_pad), S + nb_pad
    a.bias, a.bias_stride_b = bias_p.data_ptr(), S + pad
    rc = capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None)
    torch.cuda.synchronize()
    assert rc == 0
    helpers.check_close(helpers.to_numpy(out_p[:, :C]).reshape(B, S, C), helpers.oracle_out(w), w.dtype, "strided out")
    assert bool((out_p[:, C:] == -3.0).all()), "columns beyond C of the padded out rows were written"


@pytest.mark.parametrize("wide", ["input", "out"])
def test_row_pitch_beyond_the_fused_kernels_addressing_takes_the_tiled_route(torch_cuda, wide):
    """The fused MFMA kernels address rows with 32-bit byte offsets and accept row pitches of up to 2^19 elements; a wider
    one must not reach them: the automatic choice, and the choice among MFMA kernels only, go to the tiled route, whose
    products run on the strided GEMM (and are right)."""
    torch = torch_cuda
    w = make_workload(3, batch=1, seq_len=40)
    B, S, C = w.B, w.S, w.C
    ten, scratch = helpers.to_device(w)
    ld = (1 << 19) + 8
    a = helpers.hip_args(w, ten, scratch, capi.PATH_AUTO)
    wide_t = torch.zeros((B * S, ld), dtype=torch.bfloat16, device="cuda")
    if wide == "input":
        wide_t[:, :C] = ten["x"].reshape(B * S, C)
        a.input, a.input_ld = wide_t.data_ptr(), ld
    else:
        a.out, a.out_ld = wide_t.data_ptr(), ld
    rc = capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None)
    torch.cuda.synchronize()
    assert rc == 0 and capi.last_path() == "tiled_mfma"
    got = ten["out"] if wide == "input" else wide_t[:, :C].reshape(B, S, C)
    helpers.check_close(helpers.to_numpy(got), helpers.oracle_out(w), w.dtype, "wide-pitch out")
    a.path = capi.PATH_FUSED
    assert capi.lib().kutacc_hip_gating_attention(ctypes.byref(a), None) == 0 and capi.last_path() == "tiled_mfma"
    torch.cuda.synchronize()
    helpers.check_close(helpers.to_numpy(got), helpers.oracle_out(w), w.dtype, "wide-pitch out, MFMA kernels only")


# ---- boundary behaviour ------------------------------------------------------------------------------------
def test_host_pointers_are_staged_and_match_device_pointers(torch_cuda):
    w = make_workload(3, batch=3, seq_len=96)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    hten, hscratch = helpers.host_arrays(w)
    hop = capi.GatedAttention(hten["x"], hten["wq"], hten["wk"], hten["wv"], hten["wg"], hten["bg"], hten["wo"],
                              hten["bo"], hten["bias"], hten["nb"], w.H, hten["out"], hscratch)
    hop.run()
    assert not capi.error_flag()
    dev_bits = ten["out"].view(torch_cuda.int16).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(hten["out"], dev_bits)
    avg_bits = scratch["avg"].view(torch_cuda.int16).cpu().numpy().view(np.uint16)
    np.testing.assert_array_equal(hscratch["avg"], avg_bits)
    # the device copies are kept between calls: a second call (buffers reused, whatever they held) gives the same bits,
    # and releasing the pool reports what it held
    hten["out"][:] = 0
    hop.run()
    assert not capi.error_flag()
    np.testing.assert_array_equal(hten["out"], dev_bits)
    assert capi.lib().kutacc_hip_release_staging() > 0
    assert capi.lib().kutacc_hip_release_staging() == 0


def test_pointer_checks_can_be_switched_off(torch_cuda):
    """With "pointer_checks" off the entry point classifies `input` only; results on device memory are unchanged."""
    w = make_workload(3, batch=3, seq_len=96)
    op, ten, scratch = helpers.make_op(w)
    op.run()
    want = ten["out"].clone()
    ten["out"].zero_()
    assert capi.set_tuning("pointer_checks", "0") == 0
    try:
        op.run()
    finally:
        capi.set_tuning("pointer_checks", "1")
    assert not capi.error_flag() and helpers.same_bits(ten["out"], want)
    assert capi.set_tuning("no such hook", "1") == capi.EINVAL


def test_reference_scratch_mode_fills_q_k_v_gate(torch_cuda):
    """The reference's kernel leaves its projections in the caller's scratch tensors (reference
    src/attention/gating_attention.cpp:47-66: q and k as projected, v transposed to [H, d, B, S], gate with its bias,
    before the sigmoid).  The fused MFMA kernels never form them in memory; with "scratch" = "reference" the operator runs on the
    tiled MFMA route, which follows the reference's data flow, and the five tensors must match the oracle's bf16 model of
    the reference."""
    from oracle import oracle
    w = make_workload(3, batch=3, seq_len=80)
    op, ten, scratch = helpers.make_op(w)
    assert capi.set_tuning("scratch", "reference") == 0
    try:
        op.run()
        path = capi.last_path()
    finally:
        capi.set_tuning("scratch", "default")
    assert not capi.error_flag() and path == "tiled_mfma"
    bits = lambda a: oracle.to_bf16_bits(np.asarray(a, dtype=np.float32))  # noqa: E731
    _, ref = oracle.gating_attention_bf16(bits(w.x), bits(w.wq), bits(w.wk), bits(w.wv), bits(w.wg), w.bg, bits(w.wo), w.bo,
                                          bits(w.bias), None if w.nb is None else bits(w.nb), w.H, return_scratch=True)
    for name in ("q", "k", "gate", "avg"):
        got = helpers.to_numpy(scratch[name]).reshape(w.B, w.S, w.C)
        helpers.check_close(got, oracle.from_bf16_bits(ref[name]).reshape(w.B, w.S, w.C), w.dtype, name)
    helpers.check_close(helpers.to_numpy(scratch["v"]), oracle.from_bf16_bits(ref["v"]), w.dtype, "v")
    # and the default mode leaves k, v and gate alone
    for t in scratch.values():
        t.zero_()
    op.run()
    assert capi.last_path() == "fused_mfma"
    assert not scratch["k"].any() and not scratch["v"].any() and not scratch["gate"].any()


def test_mixed_host_and_device_pointers_are_rejected(torch_cuda):
    w = make_workload(3, batch=2, seq_len=64)
    ten, scratch = helpers.to_device(w)
    ten["wq"] = ten["wq"].cpu()
    op = capi.GatedAttention(ten["x"], ten["wq"], ten["wk"], ten["wv"], ten["wg"], ten["bg"], ten["wo"], ten["bo"],
                             ten["bias"], ten["nb"], w.H, ten["out"], scratch)
    op.run()
    assert capi.error_flag()
    assert not ten["out"].any()


def test_error_flag_makes_later_gpu_calls_noops(torch_cuda):
    w = make_workload(3, batch=2, seq_len=64)
    op, ten, _ = helpers.make_op(w)
    capi.lib().kutacc_af2_gating_attention(None, None, None, None, None, None, 1)
    assert capi.error_flag()
    op.run()
    assert not ten["out"].any(), "latched error: the call must not touch out"
    capi.clear_error()
    op.run()
    assert ten["out"].any()


def test_non_blocking_mode_on_caller_stream(torch_cuda):
    torch = torch_cuda
    w = make_workload(3, batch=4, seq_len=128)
    op, ten, _ = helpers.make_op(w)
    op.run()
    ref = ten["out"].clone()
    ten["out"].zero_()
    s = torch.cuda.Stream()
    try:
        capi.set_stream(s.cuda_stream)
        capi.set_blocking(False)
        with torch.cuda.stream(s):
            op.run()
        s.synchronize()
    finally:
        capi.set_stream(None)
        capi.set_blocking(True)
    assert helpers.same_bits(ten["out"], ref)


# ---- row operators in front of the path ----------------------------------------------------------------------

def test_layernorm_rows_with_a_pitch_beyond_32_bit_offsets(torch_cuda):
    """The bf16 LayerNorm kernel addresses rows with 32-bit byte offsets where the tensors allow it and keeps a 64-bit form
    for the rest: a row pitch of 2^23 elements (16 MiB between rows) must take that form and give the same rows as the
    dense call."""
    torch = torch_cuda
    rows, size, ld = 40, 128, 1 << 23
    g = torch.Generator(device="cuda").manual_seed(5)
    x = (torch.randn(rows, size, device="cuda", generator=g) * 2 + 0.5).bfloat16()
    gamma, beta = torch.randn(size, device="cuda", generator=g), torch.randn(size, device="cuda", generator=g)
    wide_in = torch.zeros(rows, ld, device="cuda", dtype=torch.bfloat16)
    wide_in[:, :size] = x
    wide_out = torch.full((rows, ld), 3.0, device="cuda", dtype=torch.bfloat16)
    dense_out = torch.zeros_like(x)
    L = capi.lib()
    assert L.kutacc_hip_layernorm_rows(x.data_ptr(), size, gamma.data_ptr(), beta.data_ptr(), dense_out.data_ptr(), size, rows,
                                       size, 1e-5, capi.K_BF16, None) == 0
    assert L.kutacc_hip_layernorm_rows(wide_in.data_ptr(), ld, gamma.data_ptr(), beta.data_ptr(), wide_out.data_ptr(), ld, rows,
                                       size, 1e-5, capi.K_BF16, None) == 0
    torch.cuda.synchronize()
    assert helpers.same_bits(wide_out[:, :size].contiguous(), dense_out)
    assert bool((wide_out[:, size:size + 64] == 3.0).all()), "columns beyond the row were written"


@pytest.mark.parametrize("size", [128, 256, 100])
def test_layernorm_rows_match_oracle(torch_cuda, size):
    from oracle import oracle
    torch = torch_cuda
    rng = np.random.Generator(np.random.PCG64(41))
    x = round_to_bf16(rng.standard_normal((300, size)).astype(np.float32) * 2 + 0.5)
    gamma = rng.standard_normal(size).astype(np.float32)
    beta = rng.standard_normal(size).astype(np.float32)
    dx = torch.from_numpy(x).cuda().bfloat16()
    dg, db = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    dout = torch.zeros_like(dx)
    rc = capi.lib().kutacc_hip_layernorm_rows(dx.data_ptr(), size, dg.data_ptr(), db.data_ptr(), dout.data_ptr(), size,
                                              300, size, 1e-5, capi.K_BF16, None)
    torch.cuda.synchronize()
    assert rc == 0
    ref = oracle.from_bf16_bits(oracle.layernorm_rows_bf16(bf16_bits(x), gamma, beta, 1e-5))
    got = helpers.to_numpy(dout)
    # same formula, different summation order: at most one bf16 ulp apart
    helpers.assert_within(got, ref, 2.0 ** -7 * np.abs(ref) + 1e-6, "layernorm rows")
    assert np.mean(got == ref) > 0.98
    # the single-row entry point of kutacc.h on device pointers
    one = torch.zeros(size, device="cuda", dtype=torch.bfloat16)
    capi.lib().kutacc_af2_layernorm(dx[7].data_ptr(), dg.data_ptr(), db.data_ptr(), size, 1e-5, one.data_ptr())
    assert not capi.error_flag()
    assert helpers.same_bits(one, dout[7])
    # ... and on host pointers (staged)
    hx = bf16_bits(x[7])
    hout = np.zeros(size, dtype=np.uint16)
    capi.lib().kutacc_af2_layernorm(hx.ctypes.data, gamma.ctypes.data, beta.ctypes.data, size, 1e-5, hout.ctypes.data)
    assert not capi.error_flag()
    np.testing.assert_array_equal(hout, dout[7].view(torch.int16).cpu().numpy().view(np.uint16))


def test_linear_matches_oracle(torch_cuda):
    from oracle import oracle
    torch = torch_cuda
    rng = np.random.Generator(np.random.PCG64(42))
    act = round_to_bf16(rng.standard_normal((5, 40, 128)).astype(np.float32))
    wgt = round_to_bf16(rng.standard_normal((4, 128)).astype(np.float32) / 11)
    bias = rng.standard_normal(4).astype(np.float32)
    da, dw = torch.from_numpy(act).cuda().bfloat16(), torch.from_numpy(wgt).cuda().bfloat16()
    dbias = torch.from_numpy(bias).cuda()
    res = torch.zeros((200, 4), device="cuda", dtype=torch.bfloat16)
    ha, hw, hr = capi.tensor(da), capi.tensor(dw), capi.tensor(res)  # keep the descriptors alive over the calls
    capi.lib().kutacc_af2_linear(ha.handle, hw.handle, dbias.data_ptr(), hr.handle, 0)
    assert not capi.error_flag()
    ref = oracle.from_bf16_bits(oracle.linear_bf16(bf16_bits(act), bf16_bits(wgt), bias))
    got = helpers.to_numpy(res)
    helpers.assert_within(got, ref, 2.0 ** -7 * np.abs(ref) + 1e-6, "linear")
    # beta = 1 accumulates onto the previous result, no bias
    capi.lib().kutacc_af2_linear(ha.handle, hw.handle, None, hr.handle, 1)
    ref2 = oracle.from_bf16_bits(oracle.linear_bf16(bf16_bits(act), bf16_bits(wgt), None, beta=1.0,
                                                    result_bits=bf16_bits(got)))
    helpers.assert_within(helpers.to_numpy(res), ref2, 2.0 ** -7 * np.abs(ref2) + 1e-6, "linear beta=1")


def test_pair_bias_producer_at_1024_residues(torch_cuda):
    """z [1024, 1024, 128], four heads: the oracle's LayerNorm + Linear on a sample of rows i (all j), for the producer and
    for the form that reads z transposed."""
    from oracle import oracle
    torch = torch_cuda
    n, cz, H = 1024, 128, 4
    g = torch.Generator(device="cuda").manual_seed(11)
    dz = (torch.randn(n, n, cz, device="cuda", generator=g) * 1.3 + 0.2).to(torch.bfloat16)
    rng = np.random.Generator(np.random.PCG64(12))
    wb = round_to_bf16((rng.standard_normal((H, cz)) / np.sqrt(cz)).astype(np.float32))
    gamma, beta = (rng.random(cz) + 0.5).astype(np.float32), (rng.standard_normal(cz) * 0.1).astype(np.float32)
    dw, dg, db = torch.from_numpy(wb).cuda().bfloat16(), torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    rows = sorted({0, 1, 31, 32, 33, 500, 511, 512, 777, 1000, 1022, 1023})
    for fn_name in ("kutacc_hip_pair_bias", "kutacc_hip_pair_bias_transposed"):
        nb = torch.zeros((H, n, n), device="cuda", dtype=torch.bfloat16)
        zn = torch.zeros_like(dz)
        rc = getattr(capi.lib(), fn_name)(dz.data_ptr(), dg.data_ptr(), db.data_ptr(), dw.data_ptr(), nb.data_ptr(), zn.data_ptr(),
                                          n, n, cz, H, 1e-5, capi.K_BF16, None)
        torch.cuda.synchronize()
        assert rc == 0, (fn_name, rc)
        # row i of the result comes from z[i, :] (plain) or z[:, i] (transposed form)
        src = dz[rows] if fn_name == "kutacc_hip_pair_bias" else dz[:, rows].transpose(0, 1)
        z_rows = helpers.to_numpy(src.contiguous()).reshape(-1, cz)
        zn_bits = oracle.layernorm_rows_bf16(bf16_bits(z_rows), gamma, beta, 1e-5)
        nb_ref = oracle.from_bf16_bits(oracle.linear_bf16(zn_bits, bf16_bits(wb))).reshape(len(rows), n, H).transpose(2, 0, 1)
        zn_ref = oracle.from_bf16_bits(zn_bits).reshape(len(rows), n, cz)
        tol = lambda r: 2.0 ** -7 * np.abs(r) + 1e-2  # noqa: E731  (a one-ulp flip in LN(z) moves nb by ~4e-3)
        helpers.assert_within(helpers.to_numpy(zn[rows]), zn_ref, tol(zn_ref), f"{fn_name}: normalised z")
        helpers.assert_within(helpers.to_numpy(nb[:, rows]), nb_ref, tol(nb_ref), f"{fn_name}: pair bias")
        assert bool(torch.isfinite(nb).all()) and bool(torch.isfinite(zn).all())


@pytest.mark.parametrize("config", [1, 3, 2])
def test_pair_bias_producer_matches_oracle(torch_cuda, config):
    """LN(z) -> [H, c_z] linear -> [H, S, S], one pass; against oracle LayerNorm + Linear + permute."""
    from oracle import oracle
    torch = torch_cuda
    w = make_workload(config, batch=2, keep_extras=True)
    z, wb = w.extras["z"], w.extras["w_bias"]
    S, cz, H = w.S, z.shape[-1], w.H
    gamma = np.ones(cz, dtype=np.float32)
    beta = np.zeros(cz, dtype=np.float32)
    dt = torch.bfloat16 if w.dtype == "bf16" else torch.float32
    code = capi.K_BF16 if w.dtype == "bf16" else capi.K_FP32
    dz = torch.from_numpy(z).cuda().to(dt)
    dw = torch.from_numpy(wb).cuda().to(dt)
    dg, db = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    nb = torch.zeros((H, S, S), device="cuda", dtype=dt)
    zn = torch.zeros_like(dz)
    rc = capi.lib().kutacc_hip_pair_bias(dz.data_ptr(), dg.data_ptr(), db.data_ptr(), dw.data_ptr(), nb.data_ptr(),
                                         zn.data_ptr(), S, S, cz, H, 1e-5, code, None)
    torch.cuda.synchronize()
    assert rc == 0
    if w.dtype == "bf16":
        zn_ref_bits = oracle.layernorm_rows_bf16(bf16_bits(z), gamma, beta, 1e-5)
        nb_ref = oracle.from_bf16_bits(oracle.linear_bf16(zn_ref_bits.reshape(S * S, cz), bf16_bits(wb)))
        zn_ref = oracle.from_bf16_bits(zn_ref_bits)
        tol = lambda r: 2.0 ** -7 * np.abs(r) + 1e-2  # noqa: E731  (a one-ulp flip in LN(z) moves nb by ~4e-3)
    else:
        zn_ref = oracle.layernorm_rows_f32(z, gamma, beta, 1e-5)
        nb_ref = oracle.linear_f32(zn_ref.reshape(S * S, cz), wb)
        tol = lambda r: 1e-4 * np.abs(r) + 1e-5  # noqa: E731
    nb_ref = nb_ref.reshape(S, S, H).transpose(2, 0, 1)
    helpers.assert_within(helpers.to_numpy(zn), zn_ref, tol(zn_ref), "normalised z")
    helpers.assert_within(helpers.to_numpy(nb), nb_ref, tol(nb_ref), "pair bias")
