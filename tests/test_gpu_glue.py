"""The steps between the operators (mask bias, axis swap, residual update, transposed pair-bias producer) and the
triangle-attention block assembled from them, on a real MI355X through the C ABI.

The copies and the residual update are checked bit for bit against torch's own indexing and bf16 addition; the
block is checked against the CPU oracle's LayerNorm, Linear and gated attention composed in numpy (fp32, no
intermediate rounding) at the tolerance of the bf16 path, and, at a full-size pair tensor, through the identity
ending_node(z, mask) == starting_node(z^T, mask^T)^T, which must hold bit for bit.
"""
import ctypes
import math

import numpy as np
import pytest

from kutacc_amd import capi
from kutacc_amd.workloads import round_to_bf16

import helpers

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def torch_cuda():
    import torch
    assert torch.cuda.is_available(), "these tests need the GPU"
    capi.set_stream(None)
    capi.set_blocking(True)
    return torch


def code(torch, t):
    return capi.K_BF16 if t.dtype == torch.bfloat16 else capi.K_FP32


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("transposed", [0, 1])
def test_mask_bias(torch_cuda, dtype, transposed):
    torch = torch_cuda
    dt = getattr(torch, dtype)
    n0, n1 = 37, 52
    g = torch.Generator(device="cuda").manual_seed(3)
    mask_ij = (torch.rand(n0, n1, device="cuda", generator=g) > 0.3).to(dt)
    stored = mask_ij.t().contiguous() if transposed else mask_ij
    bias = torch.full((n0, n1), 7.0, dtype=dt, device="cuda")
    rc = capi.lib().kutacc_hip_mask_bias(stored.data_ptr(), bias.data_ptr(), n0, n1, transposed, code(torch, bias), None)
    torch.cuda.synchronize()
    assert rc == 0
    want = (mask_ij.float() * 1e9 - 1e9).to(dt)
    assert helpers.same_bits(bias, want)
    assert float(bias.max()) == 0.0 and float(bias.min()) < -9e8


@pytest.mark.parametrize("shape,dtype", [((40, 24, 128), "bfloat16"), ((9, 31, 5), "bfloat16"), ((17, 6, 12), "float32"),
                                         ((384, 384, 128), "bfloat16")])
def test_swap_leading_axes_and_residual_add(torch_cuda, shape, dtype):
    torch = torch_cuda
    dt = getattr(torch, dtype)
    n0, n1, c = shape
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(n0, n1, c, device="cuda", generator=g).to(dt)
    out = torch.zeros(n1, n0, c, dtype=dt, device="cuda")
    L = capi.lib()
    assert L.kutacc_hip_swap_leading_axes(x.data_ptr(), out.data_ptr(), n0, n1, c, code(torch, x), None) == 0
    torch.cuda.synchronize()
    assert helpers.same_bits(out, x.transpose(0, 1).contiguous())
    # acc[i, j] += delta[i, j] and acc[i, j] += delta[j, i]
    acc = torch.randn(n0, n1, c, device="cuda", generator=g).to(dt)
    want_plain = (acc.float() + x.float()).to(dt)
    want_swapped = (acc.float() + out.transpose(0, 1).float()).to(dt)
    a1, a2 = acc.clone(), acc.clone()
    assert L.kutacc_hip_residual_add(a1.data_ptr(), x.data_ptr(), n0, n1, c, 0, code(torch, x), None) == 0
    assert L.kutacc_hip_residual_add(a2.data_ptr(), out.data_ptr(), n0, n1, c, 1, code(torch, x), None) == 0
    torch.cuda.synchronize()
    assert helpers.same_bits(a1, want_plain)
    assert helpers.same_bits(a2, want_swapped)
    assert L.kutacc_hip_swap_leading_axes(x.data_ptr(), x.data_ptr(), n0, n1, c, code(torch, x), None) == capi.EINVAL


@pytest.mark.parametrize("n_i,n_j,c_z,heads,dtype", [(48, 48, 128, 4, "bfloat16"), (40, 56, 128, 8, "bfloat16"),
                                                      (9, 14, 64, 3, "bfloat16"), (7, 5, 32, 2, "float32")])
def test_pair_bias_transposed_equals_pair_bias_of_the_swapped_tensor(torch_cuda, n_i, n_j, c_z, heads, dtype):
    torch = torch_cuda
    dt = getattr(torch, dtype)
    g = torch.Generator(device="cuda").manual_seed(9)
    z_t = torch.randn(n_j, n_i, c_z, device="cuda", generator=g).to(dt)  # stored transposed: [j, i, c]
    z = z_t.transpose(0, 1).contiguous()
    w = (torch.randn(heads, c_z, device="cuda", generator=g) / math.sqrt(c_z)).to(dt)
    gamma = torch.rand(c_z, device="cuda", generator=g) + 0.5
    beta = torch.randn(c_z, device="cuda", generator=g) * 0.1
    L = capi.lib()
    res = []
    for fn, src in ((L.kutacc_hip_pair_bias, z), (L.kutacc_hip_pair_bias_transposed, z_t)):
        nb = torch.zeros(heads, n_i, n_j, dtype=dt, device="cuda")
        zn = torch.zeros(n_i, n_j, c_z, dtype=dt, device="cuda")
        assert fn(src.data_ptr(), gamma.data_ptr(), beta.data_ptr(), w.data_ptr(), nb.data_ptr(), zn.data_ptr(), n_i, n_j, c_z,
                  heads, 1e-5, code(torch, z), None) == 0
        torch.cuda.synchronize()
        res.append((nb, zn))
    assert helpers.same_bits(res[0][0], res[1][0]) and helpers.same_bits(res[0][1], res[1][1])


# ---- the block ---------------------------------------------------------------------------------------------------
@pytest.fixture(params=["fused", "separate"])
def layernorm_placement(request):
    """Both placements of the blocks' LayerNorm: inside the attention kernel's row staging (where that kernel can) and as a
    pass of its own.  The setting must hold while the block object is built (it sizes its workspace) and run."""
    assert capi.set_tuning("layernorm", request.param) == 0
    yield request.param
    capi.set_tuning("layernorm", "auto")


def block_case(seed, n, heads):
    rng = np.random.Generator(np.random.PCG64(seed))
    c = heads * 32
    w = lambda o, i: round_to_bf16((rng.standard_normal((o, i)) / math.sqrt(i)).astype(np.float32))  # noqa: E731
    mask = (rng.random((n, n)) > 0.1).astype(np.float32)
    mask[:, -3:] = 0.0  # padded residues: masked as keys for the starting node, whole rows for the ending node
    return dict(z=round_to_bf16(rng.standard_normal((n, n, c)).astype(np.float32)), mask=mask,
                gamma=(rng.random(c) + 0.5).astype(np.float32), beta=(rng.standard_normal(c) * 0.1).astype(np.float32),
                bias_w=w(heads, c), wq=w(c, c), wk=w(c, c), wv=w(c, c), wg=w(c, c), wo=w(c, c),
                bg=np.ones(c, np.float32), bo=(rng.standard_normal(c) * 0.1).astype(np.float32), heads=heads)


def block_oracle(c, ending):
    """AlphaFold's TriangleAttention in numpy on the oracle's operators: orientation swap, LayerNorm, pair bias from
    the normalised tensor, mask bias, gated attention, swap back, residual."""
    from oracle import oracle
    z, mask = c["z"], c["mask"]
    if ending:
        z, mask = z.transpose(1, 0, 2), mask.T
    n, _, ch = z.shape
    zn = oracle.layernorm_rows_f32(np.ascontiguousarray(z).reshape(-1, ch), c["gamma"], c["beta"], 1e-5).reshape(n, n, ch)
    nb = oracle.linear_f32(zn.reshape(-1, ch), c["bias_w"]).reshape(n, n, c["heads"]).transpose(2, 0, 1)
    bias = (mask * np.float32(1e9) - np.float32(1e9)).astype(np.float32)
    out = oracle.gating_attention_f32(zn, c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"], c["bo"], bias,
                                      np.ascontiguousarray(nb), c["heads"])
    if ending:
        out = out.transpose(1, 0, 2)
    return c["z"] + out


def run_block(torch, c, ending, z=None, mask=None):
    dev = lambda a, dt=torch.bfloat16: torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dt)  # noqa: E731
    pair = dev(c["z"]) if z is None else z.clone()
    dmask = dev(c["mask"]) if mask is None else mask
    f32 = torch.float32
    blk = capi.TriangleAttentionBlock(pair, dmask, dev(c["gamma"], f32), dev(c["beta"], f32), dev(c["bias_w"]), dev(c["wq"]),
                                      dev(c["wk"]), dev(c["wv"]), dev(c["wg"]), dev(c["bg"], f32), dev(c["wo"]),
                                      dev(c["bo"], f32), c["heads"], ending)
    rc = blk.run()
    torch.cuda.synchronize()
    assert rc == 0, rc
    return pair


@pytest.mark.parametrize("ending", [False, True], ids=["starting node", "ending node"])
# 64, 96 and 160: whole key tiles, where the producer of the pair bias also writes the copy the attention kernels read
# (96 and 160: an odd tile count, padded with a zero tile)
@pytest.mark.parametrize("n,heads", [(48, 4), (70, 4), (40, 8), (64, 4), (96, 4), (160, 4), (64, 8), (32, 4), (128, 8)])
def test_triangle_attention_block_against_the_oracle(torch_cuda, layernorm_placement, n, heads, ending):
    c = block_case(600 + n, n, heads)
    got = run_block(torch_cuda, c, ending)
    helpers.check_close(helpers.to_numpy(got), block_oracle(c, ending), "bf16", f"block n={n} ending={ending}")


def profiled_kernels(torch, fn):
    """Names of the kernels the library timed while fn ran."""
    import ctypes
    lib = capi.lib()
    lib.kutacc_hip_profile_enable(1)
    try:
        fn()
        torch.cuda.synchronize()
        names, i = [], 0
        name = ctypes.create_string_buffer(128)
        ms, cnt, fl = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double()
        while lib.kutacc_hip_profile_read(i, name, 128, ctypes.byref(ms), ctypes.byref(cnt), ctypes.byref(fl)) == 0:
            names.append(name.value.decode())
            i += 1
        return names
    finally:
        lib.kutacc_hip_profile_enable(0)


@pytest.mark.parametrize("ending", [False, True], ids=["starting node", "ending node"])
@pytest.mark.parametrize("n", [32, 64, 96, 160, 352])
def test_triangle_attention_block_on_the_two_row_kernel(torch_cuda, n, ending):
    """Whole key tiles and the two-row kernel forced wherever it can run: the producer of the pair bias writes the fp32
    tiles that kernel reads (no pre-pass of the operator), one to eleven key tiles, odd counts padded with a zero tile,
    one or several rows per workgroup."""
    c = block_case(900 + n, n, 4)
    assert capi.set_tuning("row_pairs", "1") == 0
    try:
        got = {}
        names = profiled_kernels(torch_cuda, lambda: got.setdefault("z", run_block(torch_cuda, c, ending)))
    finally:
        capi.set_tuning("row_pairs", None)
    assert "persistent_pair_kernel" in names and "pair_bias_tiles_kernel" not in names and "pair_bias_fragments_kernel" not in names, names
    helpers.check_close(helpers.to_numpy(got["z"]), block_oracle(c, ending), "bf16", f"block n={n} ending={ending}, two-row kernel")


@pytest.mark.parametrize("index,n", [(i, int(n)) for i, n in enumerate(np.random.Generator(np.random.PCG64(57)).integers(8, 200, size=8))])
def test_triangle_attention_block_seeded_sweep(torch_cuda, layernorm_placement, index, n):
    """Eight seeded pair sizes between 8 and 199 (ragged key tiles, odd tile counts), four heads, node alternating."""
    ending = bool(index & 1)
    c = block_case(3000 + index, n, 4)
    got = run_block(torch_cuda, c, ending)
    helpers.check_close(helpers.to_numpy(got), block_oracle(c, ending), "bf16", f"block sweep {index}: n={n} ending={ending}")


def test_triangle_attention_block_full_size_orientation_identity(torch_cuda, layernorm_placement):
    """384 residues: the ending-node block equals the starting-node block on the transposed pair tensor and mask,
    transposed back -- the two orientations differ only in which element is read or written where."""
    torch = torch_cuda
    c = block_case(700, 384, 4)
    z = torch.from_numpy(c["z"]).to(device="cuda", dtype=torch.bfloat16)
    mask = torch.from_numpy(c["mask"]).to(device="cuda", dtype=torch.bfloat16)
    end = run_block(torch, c, True, z, mask)
    start_t = run_block(torch, c, False, z.transpose(0, 1).contiguous(), mask.t().contiguous())
    assert helpers.same_bits(end, start_t.transpose(0, 1).contiguous())
    assert not helpers.same_bits(end, z)


def block_oracle_rows(c, ending, rows):
    """block_oracle for the batch rows `rows` of the attention only (rows i of the pair tensor for the starting node,
    columns for the ending node): rows of the attention are independent, so the oracle's LayerNorm and pair bias run on
    the whole tensor and its attention on the sample.  Returns the updated pair_act entries [len(rows), n, c] in the
    orientation of the attention (entry [a, k] is pair_act[rows[a], k] or, ending node, pair_act[k, rows[a]])."""
    from oracle import oracle
    z, mask = c["z"], c["mask"]
    if ending:
        z, mask = z.transpose(1, 0, 2), mask.T
    n, _, ch = z.shape
    zn = oracle.layernorm_rows_f32(np.ascontiguousarray(z).reshape(-1, ch), c["gamma"], c["beta"], 1e-5).reshape(n, n, ch)
    nb = np.ascontiguousarray(oracle.linear_f32(zn.reshape(-1, ch), c["bias_w"]).reshape(n, n, c["heads"]).transpose(2, 0, 1))
    bias = (np.ascontiguousarray(mask[rows]) * np.float32(1e9) - np.float32(1e9)).astype(np.float32)
    out = oracle.gating_attention_f32(np.ascontiguousarray(zn[rows]), c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"],
                                      c["bo"], bias, nb, c["heads"])
    return z[rows] + out


@pytest.mark.parametrize("n", [384, 1024])
def test_triangle_attention_block_full_size_sampled_rows(torch_cuda, n):
    """The pair sizes the block is benchmarked at, both orientations: the oracle on a sample of attention rows (first,
    last, the padded residues, rows on either side of 32-row tile edges), every other entry checked for finiteness."""
    torch = torch_cuda
    c = block_case(7000 + n, n, 4)
    rows = sorted({0, 1, 31, 32, 33, n // 2 - 1, n // 2, n - 34, n - 33, n - 32, n - 4, n - 3, n - 2, n - 1})
    for ending in (False, True):
        res = {}
        names = profiled_kernels(torch, lambda: res.setdefault("z", run_block(torch, c, ending)))
        got = res["z"]
        # 384 residues: the two-row kernel on tiles the producer wrote; 1024: the long-sequence kernel on its fragments
        assert ("persistent_pair_kernel" if n == 384 else "fused_head_kernel") in names, names
        assert "pair_bias_tiles_kernel" not in names and "pair_bias_fragments_kernel" not in names, names
        assert bool(torch.isfinite(got).all())
        want = block_oracle_rows(c, ending, rows)
        sample = got[:, rows].transpose(0, 1) if ending else got[rows]
        helpers.check_close(helpers.to_numpy(sample.contiguous()), want, "bf16", f"block n={n} ending={ending}, sampled rows")


def test_triangle_attention_block_beyond_1024_residues(torch_cuda):
    """1088 residues: past the fused head kernels' longest row, the block runs the same chain as separate passes with the
    operator on the tiled MFMA route.  Both orientations against the oracle on a sample of attention rows."""
    torch = torch_cuda
    n = 1088
    c = block_case(9100, n, 4)
    rows = sorted({0, 1, 31, 32, 127, 128, n // 2, n - 65, n - 64, n - 2, n - 1})
    assert capi.lib().kutacc_hip_triangle_attention_workspace(n, 4) > capi.lib().kutacc_hip_triangle_attention_workspace(1024, 4) * 2
    for ending in (False, True):
        res = {}
        names = profiled_kernels(torch, lambda: res.setdefault("z", run_block(torch, c, ending)))
        got = res["z"]
        assert "attention_tiles_kernel" in names and "residual_add_kernel" in names, names
        assert bool(torch.isfinite(got).all())
        want = block_oracle_rows(c, ending, rows)
        sample = got[:, rows].transpose(0, 1) if ending else got[rows]
        helpers.check_close(helpers.to_numpy(sample.contiguous()), want, "bf16", f"block n={n} ending={ending}, sampled rows")


@pytest.mark.parametrize("n,heads", [(72, 3), (100, 5), (45, 1)])
def test_triangle_attention_block_with_other_channel_counts(torch_cuda, n, heads):
    """96, 160 and 32 channels (heads of 32): no fused head kernel takes them, the block's tiled route does; whole result
    against the oracle's composition, both orientations, lengths that are and are not multiples of 8."""
    for ending in (False, True):
        c = block_case(9200 + n, n, heads)
        got = run_block(torch_cuda, c, ending)
        helpers.check_close(helpers.to_numpy(got), block_oracle(c, ending), "bf16", f"block n={n} heads={heads} ending={ending}")


def test_fused_layernorm_drops_the_normalised_copy_from_the_workspace(torch_cuda):
    """With the LayerNorm inside the attention kernel the blocks keep no normalised activation: the workspace is one
    activation smaller wherever the persistent kernel runs (384 residues), and unchanged where it does not (1024)."""
    L = capi.lib()
    sizes = {}
    for mode in ("fused", "separate"):
        assert capi.set_tuning("layernorm", mode) == 0
        sizes[mode] = (L.kutacc_hip_triangle_attention_workspace(384, 4), L.kutacc_hip_triangle_attention_workspace(1024, 4),
                       L.kutacc_hip_msa_attention_workspace(512, 256, 8, 0))
    capi.set_tuning("layernorm", "auto")
    assert sizes["separate"][0] - sizes["fused"][0] == 384 * 384 * 128 * 2
    assert sizes["separate"][1] == sizes["fused"][1]
    assert sizes["separate"][2] - sizes["fused"][2] == 512 * 256 * 256 * 2


def test_triangle_attention_block_rejects_bad_arguments(torch_cuda):
    torch = torch_cuda
    L = capi.lib()
    assert L.kutacc_hip_triangle_attention(None, None) == capi.EINVAL
    assert L.kutacc_hip_triangle_attention_workspace(0, 4) == -1
    c = block_case(1, 40, 4)
    dev = lambda a, dt=torch.bfloat16: torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dt)  # noqa: E731
    blk = capi.TriangleAttentionBlock(dev(c["z"]), dev(c["mask"]), dev(c["gamma"], torch.float32), dev(c["beta"], torch.float32),
                                      dev(c["bias_w"]), dev(c["wq"]), dev(c["wk"]), dev(c["wv"]), dev(c["wg"]),
                                      dev(c["bg"], torch.float32), dev(c["wo"]), dev(c["bo"], torch.float32), 4, False)
    blk.args.workspace_bytes -= 1
    assert blk.run() == capi.EINVAL
    blk.args.workspace_bytes += 1
    blk.args.nheads = 3  # 96 channels: no MFMA attention kernel
    assert blk.run() in (capi.EUNSUPPORTED, capi.EINVAL)
    torch.cuda.synchronize()


# ---- channel-first LayerNorm and the triangle-multiplication block ------------------------------------------------
@pytest.mark.parametrize("channels,positions,dtype", [(128, 4096, "bfloat16"), (128, 1000, "bfloat16"), (128, 40, "bfloat16"),
                                                      (96, 77, "bfloat16"), (20, 33, "float32")])
def test_layernorm_channel_first(torch_cuda, channels, positions, dtype):
    """Against the oracle's row LayerNorm on the transposed tensor: fast path (128 channels, ragged position counts) and
    the generic kernel."""
    from oracle import oracle
    torch = torch_cuda
    dt = getattr(torch, dtype)
    rng = np.random.Generator(np.random.PCG64(31 + positions))
    x = (rng.standard_normal((channels, positions)) * 2 + rng.standard_normal((1, positions))).astype(np.float32)
    if dtype == "bfloat16":
        x = round_to_bf16(x)
    gamma = (rng.random(channels) + 0.5).astype(np.float32)
    beta = (rng.standard_normal(channels) * 0.2).astype(np.float32)
    dx = torch.from_numpy(x).to(device="cuda", dtype=dt)
    out = torch.full((positions, channels + 8), 9.0, dtype=dt, device="cuda")
    g, b = torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()
    rc = capi.lib().kutacc_hip_layernorm_channel_first(dx.data_ptr(), positions, g.data_ptr(), b.data_ptr(), out.data_ptr(),
                                                       channels + 8, channels, positions, 1e-5, code(torch, dx), None)
    torch.cuda.synchronize()
    assert rc == 0
    ref = oracle.layernorm_rows_f32(np.ascontiguousarray(x.T), gamma, beta, 1e-5)
    helpers.check_close(helpers.to_numpy(out[:, :channels]), ref, "bf16" if dtype == "bfloat16" else "fp32", "channel-first LN")
    assert bool((out[:, channels:] == 9.0).all())


def tm_block_case(seed, n, c_z, c_i):
    rng = np.random.Generator(np.random.PCG64(seed))
    w = lambda o, i: round_to_bf16((rng.standard_normal((o, i)) / math.sqrt(i)).astype(np.float32))  # noqa: E731
    b = lambda k: (rng.standard_normal(k) * 0.3).astype(np.float32)  # noqa: E731
    g = lambda k: (rng.random(k) + 0.5).astype(np.float32)  # noqa: E731
    return dict(z=round_to_bf16(rng.standard_normal((n, n, c_z)).astype(np.float32)),
                mask=(rng.random((n, n)) > 0.15).astype(np.float32),
                ln_in_gamma=g(c_z), ln_in_beta=b(c_z), left_proj_w=w(c_i, c_z), left_proj_b=b(c_i), left_gate_w=w(c_i, c_z),
                left_gate_b=b(c_i), right_proj_w=w(c_i, c_z), right_proj_b=b(c_i), right_gate_w=w(c_i, c_z), right_gate_b=b(c_i),
                ln_center_gamma=g(c_i), ln_center_beta=b(c_i), output_w=w(c_z, c_i), output_b=b(c_z), gating_w=w(c_z, c_z),
                gating_b=b(c_z))


def tm_block_oracle(c, incoming):
    """AlphaFold's TriangleMultiplication in numpy on the oracle's operators (fp32, no intermediate rounding)."""
    from oracle import oracle
    n, _, c_z = c["z"].shape
    c_i = c["left_proj_w"].shape[0]
    act = oracle.layernorm_rows_f32(c["z"].reshape(-1, c_z), c["ln_in_gamma"], c["ln_in_beta"], 1e-5).reshape(n, n, c_z)
    left = oracle.tm_calc_proj_f32(act, c["mask"], c["left_proj_w"], c["left_proj_b"], c["left_gate_w"], c["left_gate_b"])
    right = oracle.tm_calc_proj_f32(act, c["mask"], c["right_proj_w"], c["right_proj_b"], c["right_gate_w"], c["right_gate_b"])
    center = oracle.tm_equation_f32(left, right, incoming)
    center = oracle.layernorm_rows_f32(np.ascontiguousarray(center.transpose(1, 2, 0)).reshape(-1, c_i), c["ln_center_gamma"],
                                       c["ln_center_beta"], 1e-5)
    gate, out = oracle.tm_gate_and_out_f32(act, center, c["gating_w"], c["gating_b"], c["output_w"], c["output_b"])
    return c["z"] + oracle.tm_last_f32(out, gate).reshape(n, n, c_z)


@pytest.mark.parametrize("incoming", [False, True], ids=["outgoing", "incoming"])
# 48: the last kernel takes the centre channel-first, normalises it and projects the gate itself; 46 (positions not in
# whole 16-byte runs): it still projects the gate, behind the stand-alone channel-first LayerNorm; the others: separate passes
@pytest.mark.parametrize("n,c_z,c_i", [(48, 128, 128), (46, 128, 128), (40, 64, 32), (9, 12, 6)])
def test_triangle_multiplication_block_against_the_oracle(torch_cuda, n, c_z, c_i, incoming):
    torch = torch_cuda
    c = tm_block_case(800 + n, n, c_z, c_i)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    pair = dev(c["z"])
    w = {k: dev(v) for k, v in c.items() if k not in ("z", "mask")}
    blk = capi.TriangleMultiplicationBlock(pair, dev(c["mask"]), w, incoming)
    rc = blk.run()
    torch.cuda.synchronize()
    assert rc == 0, rc
    helpers.check_close(helpers.to_numpy(pair), tm_block_oracle(c, incoming), "bf16", f"TM block n={n} incoming={incoming}")


@pytest.mark.parametrize("index,n", [(i, int(n)) for i, n in enumerate(np.random.Generator(np.random.PCG64(31)).integers(8, 90, size=8))])
def test_triangle_multiplication_block_seeded_sweep(torch_cuda, index, n):
    """Eight seeded pair sizes between 8 and 89 at 128 channels (positions in and out of whole 16-byte runs, so both forms of
    the block's last kernel and the stand-alone centre LayerNorm), orientation alternating, against the oracle."""
    torch = torch_cuda
    incoming = bool(index & 1)
    c = tm_block_case(2000 + index, n, 128, 128)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    pair = dev(c["z"])
    w = {k: dev(v) for k, v in c.items() if k not in ("z", "mask")}
    assert capi.TriangleMultiplicationBlock(pair, dev(c["mask"]), w, incoming).run() == 0
    torch.cuda.synchronize()
    helpers.check_close(helpers.to_numpy(pair), tm_block_oracle(c, incoming), "bf16", f"TM block sweep {index}: n={n} incoming={incoming}")


@pytest.mark.parametrize("n", [48, 72, 384])
def test_triangle_multiplication_block_on_each_gated_projection_kernel(torch_cuda, n):
    """The block's two gated projections go out in one launch.  Its default kernel (weights in registers, both sides in
    one pass over the activation) must give the block's result bit for bit as the streaming kernel does, and within the
    rounding of the intermediates as the tiled kernel does."""
    torch = torch_cuda
    case = tm_block_case(900 + n, n, 128, 128)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    w = {k: dev(v) for k, v in case.items() if k not in ("z", "mask")}
    want = {None: "gated_projection_blocks_kernel<2>", "streaming": "gated_projection_kernel<2>", "tiled": "pair_gemm_kernel<gated>"}
    res = {}
    for mode in want:
        assert capi.set_tuning("gated_projection", mode) == 0
        try:
            pair = dev(case["z"])
            capi.lib().kutacc_hip_profile_enable(1)
            assert capi.TriangleMultiplicationBlock(pair, dev(case["mask"]), w, False).run() == 0
            torch.cuda.synchronize()
            names = []
            for i in range(16):
                name = ctypes.create_string_buffer(96)
                ms, cnt, fl = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double()
                if capi.lib().kutacc_hip_profile_read(i, name, 96, ctypes.byref(ms), ctypes.byref(cnt), ctypes.byref(fl)) != 0:
                    break
                names.append(name.value.decode())
        finally:
            capi.lib().kutacc_hip_profile_enable(0)
            capi.set_tuning("gated_projection", None)
        assert want[mode] in names, (mode, names)
        res[mode] = pair
    assert helpers.same_bits(res[None], res["streaming"])
    tiled = helpers.to_numpy(res["tiled"])
    helpers.assert_within(helpers.to_numpy(res[None]), tiled, 4e-2 + 2e-2 * np.abs(tiled), "weights in registers vs tiled kernel")


@pytest.mark.parametrize("incoming", [False, True], ids=["outgoing", "incoming"])
@pytest.mark.parametrize("n", [384, 512, 768])  # 768: the equation on the 256 x 256 tiles
def test_triangle_multiplication_block_full_size(torch_cuda, incoming, n):
    """384 residues, 128 channels, the real shape, 512 and 768 (both gated projections in one pass over the activation).  The oracle follows a sample of output positions (i, j) through the
    whole block: their centre needs the left projections of row i and the right projections of row j (columns for the
    incoming form), which the oracle computes for just those rows."""
    from oracle import oracle
    torch = torch_cuda
    c = 128
    case = tm_block_case(900 + n, n, c, c)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    w = {k: dev(v) for k, v in case.items() if k not in ("z", "mask")}
    pair = dev(case["z"])
    assert capi.TriangleMultiplicationBlock(pair, dev(case["mask"]), w, incoming).run() == 0
    torch.cuda.synchronize()
    got = helpers.to_numpy(pair)
    I, J = [0, 77, 200, n - 1], [5, 100, n - 1]
    act = oracle.layernorm_rows_f32(case["z"].reshape(-1, c), case["ln_in_gamma"], case["ln_in_beta"], 1e-5).reshape(n, n, c)
    proj = lambda side, x, m: oracle.tm_calc_proj_f32(x, m, case[side + "_proj_w"], case[side + "_proj_b"],  # noqa: E731
                                                       case[side + "_gate_w"], case[side + "_gate_b"])
    if not incoming:  # center[c, i, j] = sum_k left[c, i, k] right[c, j, k]
        left, right = proj("left", act[I], case["mask"][I]), proj("right", act[J], case["mask"][J])
        center = np.einsum("cik,cjk->ijc", left.astype(np.float64), right.astype(np.float64))
    else:             # center[c, i, j] = sum_k right[c, k, i] left[c, k, j]
        right = proj("right", np.ascontiguousarray(act[:, I]), np.ascontiguousarray(case["mask"][:, I]))
        left = proj("left", np.ascontiguousarray(act[:, J]), np.ascontiguousarray(case["mask"][:, J]))
        center = np.einsum("cki,ckj->ijc", right.astype(np.float64), left.astype(np.float64))
    center = oracle.layernorm_rows_f32(center.reshape(-1, c).astype(np.float32), case["ln_center_gamma"], case["ln_center_beta"], 1e-5)
    act_ij = act[np.ix_(I, J)].reshape(-1, c)
    gate, out = oracle.tm_gate_and_out_f32(act_ij, center, case["gating_w"], case["gating_b"], case["output_w"], case["output_b"])
    want = case["z"][np.ix_(I, J)].reshape(-1, c) + oracle.tm_last_f32(out, gate)
    helpers.check_close(got[np.ix_(I, J)].reshape(-1, c), want, "bf16", f"TM block {n} incoming={incoming}")
    assert not np.array_equal(got, case["z"])


@pytest.mark.parametrize("m,n,k", [(1000, 128, 128), (333, 256, 128), (520, 128, 256)])
def test_gated_residual_projection(torch_cuda, m, n, k):
    """acc += bf16(a . w^T + bias) * sigmoid(gate) in one kernel, against the same three steps in float64."""
    torch = torch_cuda
    rng = np.random.Generator(np.random.PCG64(40 + m))
    a = round_to_bf16(rng.standard_normal((m, k)).astype(np.float32))
    w = round_to_bf16((rng.standard_normal((n, k)) / math.sqrt(k)).astype(np.float32))
    bias = (rng.standard_normal(n) * 0.3).astype(np.float32)
    gate = round_to_bf16(rng.standard_normal((m, n)).astype(np.float32) * 2)
    acc = round_to_bf16(rng.standard_normal((m, n)).astype(np.float32))
    dev = lambda x, dt=torch.bfloat16: torch.from_numpy(x).to(device="cuda", dtype=dt)  # noqa: E731
    d_acc = dev(acc)
    t = [dev(a), dev(w), dev(bias, torch.float32), dev(gate)]
    rc = capi.lib().kutacc_hip_gated_residual_projection(t[0].data_ptr(), k, t[1].data_ptr(), t[2].data_ptr(), t[3].data_ptr(), n,
                                                         d_acc.data_ptr(), n, m, n, k, capi.K_BF16, None)
    torch.cuda.synchronize()
    assert rc == 0, rc
    o = a.astype(np.float64) @ w.astype(np.float64).T + bias
    want = acc + o / (1.0 + np.exp(-gate.astype(np.float64)))
    helpers.check_close(helpers.to_numpy(d_acc), want, "bf16", "gated residual projection")
    rc = capi.lib().kutacc_hip_gated_residual_projection(t[0].data_ptr(), k, t[1].data_ptr(), t[2].data_ptr(), t[3].data_ptr(), n,
                                                         d_acc.data_ptr(), n, m, 96, k, capi.K_BF16, None)
    assert rc == capi.EUNSUPPORTED


# 65536 + 20000 rows: more than one round of workgroups plus a partial one
@pytest.mark.parametrize("rows,c_o,c_i", [(300, 128, 512), (200, 256, 1024), (64 * 64, 128, 512), (50, 24, 40),
                                          (65536 + 20000, 128, 256)])
def test_transition_block(torch_cuda, rows, c_o, c_i):
    """act += transition(LN(act)) in place: the one-kernel form (pair and MSA channel counts, ragged row counts) and the
    separate-pass form through a workspace, against the oracle's LayerNorm and transition composed in numpy."""
    from oracle import oracle
    torch = torch_cuda
    rng = np.random.Generator(np.random.PCG64(70 + rows))
    x = round_to_bf16((rng.standard_normal((rows, c_o)) * 1.5 + 0.3).astype(np.float32))
    gamma, beta = (rng.random(c_o) + 0.5).astype(np.float32), (rng.standard_normal(c_o) * 0.2).astype(np.float32)
    w1 = round_to_bf16((rng.standard_normal((c_i, c_o)) / math.sqrt(c_o)).astype(np.float32))
    w2 = round_to_bf16((rng.standard_normal((c_o, c_i)) / math.sqrt(c_i)).astype(np.float32))
    b1, b2 = (rng.standard_normal(c_i) * 0.3).astype(np.float32), (rng.standard_normal(c_o) * 0.3).astype(np.float32)
    dev = lambda a, dt=torch.bfloat16: torch.from_numpy(a).to(device="cuda", dtype=dt)  # noqa: E731
    f32 = torch.float32
    act = dev(x)
    t = [dev(gamma, f32), dev(beta, f32), dev(w1), dev(b1, f32), dev(w2), dev(b2, f32)]
    L = capi.lib()
    nbytes = L.kutacc_hip_transition_block_workspace(rows, c_o, c_i)
    assert (nbytes == 0) == (c_o in (128, 256))
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device="cuda")
    rc = L.kutacc_hip_transition_block(act.data_ptr(), t[0].data_ptr(), t[1].data_ptr(), 1e-5, t[2].data_ptr(), t[3].data_ptr(),
                                       t[4].data_ptr(), t[5].data_ptr(), ws.data_ptr() if nbytes else None, nbytes, rows, c_o, c_i,
                                       capi.K_BF16, None)
    torch.cuda.synchronize()
    assert rc == 0, rc
    want = x + oracle.transition_f32(oracle.layernorm_rows_f32(x, gamma, beta, 1e-5), w1, b1, w2, b2)
    helpers.check_close(helpers.to_numpy(act), want, "bf16", f"transition block {rows}x{c_o}->{c_i}")
    if nbytes:  # without its workspace the separate-pass form must refuse
        assert L.kutacc_hip_transition_block(act.data_ptr(), t[0].data_ptr(), t[1].data_ptr(), 1e-5, t[2].data_ptr(),
                                             t[3].data_ptr(), t[4].data_ptr(), t[5].data_ptr(), None, 0, rows, c_o, c_i,
                                             capi.K_BF16, None) == capi.EINVAL


# ---- MSA attention blocks ------------------------------------------------------------------------------------------
def msa_case(seed, n_seq, n_res, heads, c_z):
    rng = np.random.Generator(np.random.PCG64(seed))
    c = heads * 32
    w = lambda o, i: round_to_bf16((rng.standard_normal((o, i)) / math.sqrt(i)).astype(np.float32))  # noqa: E731
    mask = (rng.random((n_seq, n_res)) > 0.1).astype(np.float32)
    mask[:, -2:] = 0.0  # padded residues
    mask[-1, :] = 0.0   # a padded sequence: a fully masked row for the row-wise form
    return dict(m=round_to_bf16(rng.standard_normal((n_seq, n_res, c)).astype(np.float32)), mask=mask,
                z=round_to_bf16(rng.standard_normal((n_res, n_res, c_z)).astype(np.float32)),
                ln_gamma=(rng.random(c) + 0.5).astype(np.float32), ln_beta=(rng.standard_normal(c) * 0.1).astype(np.float32),
                pair_ln_gamma=(rng.random(c_z) + 0.5).astype(np.float32),
                pair_ln_beta=(rng.standard_normal(c_z) * 0.1).astype(np.float32), bias_w=w(heads, c_z),
                wq=w(c, c), wk=w(c, c), wv=w(c, c), wg=w(c, c), wo=w(c, c), bg=np.ones(c, np.float32),
                bo=(rng.standard_normal(c) * 0.1).astype(np.float32), heads=heads)


def msa_oracle(c, column):
    """AlphaFold's MSARowAttentionWithPairBias / MSAColumnAttention in numpy on the oracle's operators."""
    from oracle import oracle
    m, mask = c["m"], c["mask"]
    if column:
        m, mask = m.transpose(1, 0, 2), mask.T
    B, S, ch = m.shape
    mn = oracle.layernorm_rows_f32(np.ascontiguousarray(m).reshape(-1, ch), c["ln_gamma"], c["ln_beta"], 1e-5).reshape(B, S, ch)
    nb = None
    if not column:
        n_res, _, cz = c["z"].shape
        zn = oracle.layernorm_rows_f32(c["z"].reshape(-1, cz), c["pair_ln_gamma"], c["pair_ln_beta"], 1e-5)
        nb = np.ascontiguousarray(oracle.linear_f32(zn, c["bias_w"]).reshape(n_res, n_res, c["heads"]).transpose(2, 0, 1))
    bias = (np.ascontiguousarray(mask) * np.float32(1e9) - np.float32(1e9)).astype(np.float32)
    out = oracle.gating_attention_f32(mn, c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"], c["bo"], bias, nb, c["heads"])
    if column:
        out = out.transpose(1, 0, 2)
    return c["m"] + out


@pytest.mark.parametrize("column", [False, True], ids=["row-wise with pair bias", "column-wise"])
@pytest.mark.parametrize("n_seq,n_res,heads,c_z", [(24, 40, 8, 128), (50, 20, 8, 128), (33, 33, 4, 64), (24, 64, 8, 128),
                                                   (20, 96, 8, 128)])
def test_msa_attention_block_against_the_oracle(torch_cuda, layernorm_placement, n_seq, n_res, heads, c_z, column):
    torch = torch_cuda
    c = msa_case(1000 + n_seq, n_seq, n_res, heads, c_z)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    msa = dev(c["m"])
    w = {k: dev(c[k]) for k in ("ln_gamma", "ln_beta", "wq", "wk", "wv", "wg", "bg", "wo", "bo")}
    pair = None if column else {"pair_act": dev(c["z"]), "pair_ln_gamma": dev(c["pair_ln_gamma"]),
                                "pair_ln_beta": dev(c["pair_ln_beta"]), "bias_w": dev(c["bias_w"])}
    blk = capi.MsaAttentionBlock(msa, dev(c["mask"]), w, heads, pair)
    rc = blk.run()
    torch.cuda.synchronize()
    assert rc == 0, rc
    helpers.check_close(helpers.to_numpy(msa), msa_oracle(c, column), "bf16", f"msa block {n_seq}x{n_res} column={column}")


@pytest.mark.parametrize("n_seq,n_res", [(24, 64), (20, 96), (70, 128), (9, 32)])
def test_msa_row_attention_block_on_the_two_row_kernel(torch_cuda, n_seq, n_res):
    """Row-wise MSA attention (256 channels, eight heads) with whole key tiles and the two-row kernel forced: the
    producer of the pair bias writes that kernel's fp32 tiles, and the operator runs no pre-pass."""
    torch = torch_cuda
    heads, c_z = 8, 128
    c = msa_case(1200 + n_seq, n_seq, n_res, heads, c_z)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    msa = dev(c["m"])
    w = {k: dev(c[k]) for k in ("ln_gamma", "ln_beta", "wq", "wk", "wv", "wg", "bg", "wo", "bo")}
    pair = {"pair_act": dev(c["z"]), "pair_ln_gamma": dev(c["pair_ln_gamma"]), "pair_ln_beta": dev(c["pair_ln_beta"]),
            "bias_w": dev(c["bias_w"])}
    assert capi.set_tuning("row_pairs", "1") == 0
    try:
        blk = capi.MsaAttentionBlock(msa, dev(c["mask"]), w, heads, pair)
        names = profiled_kernels(torch, lambda: blk.run())
    finally:
        capi.set_tuning("row_pairs", None)
    assert "persistent_pair_kernel" in names and "pair_bias_tiles_kernel" not in names and "pair_bias_fragments_kernel" not in names, names
    helpers.check_close(helpers.to_numpy(msa), msa_oracle(c, False), "bf16", f"msa row block {n_seq}x{n_res}, two-row kernel")


def test_layernorm_rows_transposed(torch_cuda):
    torch = torch_cuda
    g = torch.Generator(device="cuda").manual_seed(4)
    for rows_i, rows_j, size, dt in ((20, 36, 256, torch.bfloat16), (7, 9, 24, torch.float32)):
        x_t = torch.randn(rows_j, rows_i, size, device="cuda", generator=g).to(dt)
        gamma = torch.rand(size, device="cuda", generator=g) + 0.5
        beta = torch.randn(size, device="cuda", generator=g) * 0.1
        a, b = torch.zeros(rows_i, rows_j, size, dtype=dt, device="cuda"), torch.zeros(rows_i, rows_j, size, dtype=dt, device="cuda")
        L = capi.lib()
        x = x_t.transpose(0, 1).contiguous()
        assert L.kutacc_hip_layernorm_rows(x.data_ptr(), size, gamma.data_ptr(), beta.data_ptr(), a.data_ptr(), size,
                                           rows_i * rows_j, size, 1e-5, code(torch, x), None) == 0
        assert L.kutacc_hip_layernorm_rows_transposed(x_t.data_ptr(), gamma.data_ptr(), beta.data_ptr(), b.data_ptr(), rows_i,
                                                      rows_j, size, 1e-5, code(torch, x), None) == 0
        torch.cuda.synchronize()
        assert helpers.same_bits(a, b)


def test_pair_stack_blocks_replay_from_a_hip_graph(torch_cuda):
    """The three pair-stack blocks (triangle multiplication, triangle attention, transition) captured into one HIP graph
    on a side stream and replayed three times, with eager work (restoring the pair tensor) between the replays; every
    replay must reproduce the eager result bit for bit.  Nothing in the launch path allocates, frees, memsets or
    synchronises, which is what makes the blocks capturable."""
    torch = torch_cuda
    n, heads = 64, 4
    c = heads * 32
    ca, ct = block_case(1200, n, heads), tm_block_case(1201, n, c, c)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    z0 = dev(ca["z"])
    z = z0.clone()
    mask = dev(ca["mask"])
    tm = capi.TriangleMultiplicationBlock(z, mask, {k: dev(v) for k, v in ct.items() if k not in ("z", "mask")}, False)
    ta = capi.TriangleAttentionBlock(z, mask, dev(ca["gamma"]), dev(ca["beta"]), dev(ca["bias_w"]), dev(ca["wq"]), dev(ca["wk"]),
                                     dev(ca["wv"]), dev(ca["wg"]), dev(ca["bg"]), dev(ca["wo"]), dev(ca["bo"]), heads, True)
    rng = np.random.Generator(np.random.PCG64(5))
    w1 = dev(round_to_bf16((rng.standard_normal((4 * c, c)) / math.sqrt(c)).astype(np.float32)))
    w2 = dev(round_to_bf16((rng.standard_normal((c, 4 * c)) / math.sqrt(4 * c)).astype(np.float32)))
    b1, b2 = dev((rng.standard_normal(4 * c) * 0.1).astype(np.float32)), dev((rng.standard_normal(c) * 0.1).astype(np.float32))
    gam, bet = dev(ca["gamma"]), dev(ca["beta"])
    L = capi.lib()

    def blocks(stream_ptr):
        assert tm.run(stream_ptr) == 0
        assert ta.run(stream_ptr) == 0
        assert L.kutacc_hip_transition_block(z.data_ptr(), gam.data_ptr(), bet.data_ptr(), 1e-5, w1.data_ptr(), b1.data_ptr(),
                                             w2.data_ptr(), b2.data_ptr(), None, 0, n * n, c, 4 * c, capi.K_BF16, stream_ptr) == 0

    blocks(None)  # eager, also takes every first-call set-up (kernel attributes) out of the capture
    torch.cuda.synchronize()
    want = z.clone()
    assert not helpers.same_bits(want, z0)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    z.copy_(z0)
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        blocks(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        z.copy_(z0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert helpers.same_bits(z, want)


@pytest.mark.parametrize("column,n_seq,n_res,heads", [(True, 1088, 24, 8), (False, 20, 1040, 8), (False, 24, 56, 3), (True, 40, 24, 5)])
def test_msa_attention_blocks_on_the_tiled_route(torch_cuda, column, n_seq, n_res, heads):
    """Attention rows of more than 1024 keys (column-wise over 1088 sequences, row-wise over 1040 residues) and channel
    counts other than 128 and 256: the block's separate passes with the operator on the tiled MFMA route, whole result
    against the oracle's composition."""
    torch = torch_cuda
    c = msa_case(9300 + n_seq + n_res, n_seq, n_res, heads, 128)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
        device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
    msa = dev(c["m"])
    w = {k: dev(c[k]) for k in ("ln_gamma", "ln_beta", "wq", "wk", "wv", "wg", "bg", "wo", "bo")}
    pair = None if column else {"pair_act": dev(c["z"]), "pair_ln_gamma": dev(c["pair_ln_gamma"]),
                                "pair_ln_beta": dev(c["pair_ln_beta"]), "bias_w": dev(c["bias_w"])}
    blk = capi.MsaAttentionBlock(msa, dev(c["mask"]), w, heads, pair)
    res = {}
    names = profiled_kernels(torch, lambda: res.setdefault("rc", blk.run()))
    torch.cuda.synchronize()
    assert res["rc"] == 0 and "attention_tiles_kernel" in names, (res, names)
    helpers.check_close(helpers.to_numpy(msa), msa_oracle(c, column), "bf16", f"msa block {n_seq}x{n_res} heads={heads} column={column}")


def test_msa_attention_blocks_full_size_sampled_rows(torch_cuda):
    """The MSA shapes the blocks are benchmarked at -- row-wise with pair bias at 512 sequences x 256 residues, column-wise
    at 1024 sequences x 384 residues -- against the oracle on a sample of attention rows (sequences for the row-wise
    form, residues for the column-wise one), every other entry checked for finiteness."""
    from oracle import oracle
    torch = torch_cuda
    for column, n_seq, n_res in ((False, 512, 256), (True, 1024, 384)):
        c = msa_case(8000 + n_seq, n_seq, n_res, 8, 128)
        dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(  # noqa: E731
            device="cuda", dtype=torch.bfloat16 if a.ndim >= 2 else torch.float32)
        msa = dev(c["m"])
        w = {k: dev(c[k]) for k in ("ln_gamma", "ln_beta", "wq", "wk", "wv", "wg", "bg", "wo", "bo")}
        pair = None if column else {"pair_act": dev(c["z"]), "pair_ln_gamma": dev(c["pair_ln_gamma"]),
                                    "pair_ln_beta": dev(c["pair_ln_beta"]), "bias_w": dev(c["bias_w"])}
        blk = capi.MsaAttentionBlock(msa, dev(c["mask"]), w, 8, pair)
        rc = blk.run()
        torch.cuda.synchronize()
        assert rc == 0, rc
        assert bool(torch.isfinite(msa).all())
        m, mask = (c["m"].transpose(1, 0, 2), c["mask"].T) if column else (c["m"], c["mask"])
        B = m.shape[0]
        rows = sorted({0, 1, 7, 8, 9, B // 2, B - 10, B - 9, B - 8, B - 3, B - 2, B - 1})
        ch = m.shape[-1]
        mn = oracle.layernorm_rows_f32(np.ascontiguousarray(m[rows]).reshape(-1, ch), c["ln_gamma"], c["ln_beta"], 1e-5)
        mn = mn.reshape(len(rows), -1, ch)
        nb = None
        if not column:
            cz = c["z"].shape[-1]
            zn = oracle.layernorm_rows_f32(c["z"].reshape(-1, cz), c["pair_ln_gamma"], c["pair_ln_beta"], 1e-5)
            nb = np.ascontiguousarray(oracle.linear_f32(zn, c["bias_w"]).reshape(n_res, n_res, 8).transpose(2, 0, 1))
        bias = (np.ascontiguousarray(mask[rows]) * np.float32(1e9) - np.float32(1e9)).astype(np.float32)
        out = oracle.gating_attention_f32(mn, c["wq"], c["wk"], c["wv"], c["wg"], c["bg"], c["wo"], c["bo"], bias, nb, 8)
        want = m[rows] + out
        sample = msa[:, rows].transpose(0, 1) if column else msa[rows]
        helpers.check_close(helpers.to_numpy(sample.contiguous()), want, "bf16",
                            f"msa block {n_seq}x{n_res} column={column}, sampled rows")
