"""Parity of the transition and triangle-multiplication operators (and of the strided bf16 GEMM under them)
against the CPU oracle, through the C ABI, on a real MI355X.

Inputs are bf16-representable fp32 draws, so the device and the oracle see the same numbers; the oracle
works in fp32/fp64 without intermediate rounding.  Tolerances: a plain GEMM result is one bf16 rounding away
from the exact value (relative 2^-9), checked at 6e-3 relative + 2e-3 absolute; results that pass through a
second bf16-rounded intermediate (hidden layer of the transition, gated projections) are checked at the bar
of the bf16 path, 2e-2 absolute + 1e-2 relative of the fp32 oracle.
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


def draw(rng, *shape, scale=1.0):
    return round_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


def dev(torch, a, dtype=None):
    return torch.from_numpy(np.ascontiguousarray(a)).to(device="cuda", dtype=dtype or torch.bfloat16)


GEMM_TOL = lambda ref: 2e-3 + 6e-3 * np.abs(ref)  # noqa: E731


def run_gemm(torch, A, B, *, a_mmajor=False, b_mmajor=False, bias=None, bias_axis=0, relu=False, path=capi.PATH_AUTO,
             c_pad=0):
    """A [batches, M, K], B [batches, N, K] as fp32 numpy; operands are stored k-contiguous or transposed (m-major)."""
    nb, M, K = A.shape
    N = B.shape[1]
    dA = dev(torch, A.transpose(0, 2, 1) if a_mmajor else A)
    dB = dev(torch, B.transpose(0, 2, 1) if b_mmajor else B)
    dC = torch.full((nb, M, N + c_pad), -7.0, dtype=torch.bfloat16, device="cuda")
    g = capi.HipGemmArgs()
    g.m, g.n, g.k, g.batches, g.dtype, g.path = M, N, K, nb, capi.K_BF16, path
    g.a, g.a_stride_batch = dA.data_ptr(), M * K
    g.a_stride_m, g.a_stride_k = (1, M) if a_mmajor else (K, 1)
    g.b, g.b_stride_batch = dB.data_ptr(), N * K
    g.b_stride_n, g.b_stride_k = (1, N) if b_mmajor else (K, 1)
    g.c, g.c_stride_m, g.c_stride_batch = dC.data_ptr(), N + c_pad, M * (N + c_pad)
    keep = None
    if bias is not None:
        keep = dev(torch, bias, torch.float32)
        g.bias, g.bias_axis = keep.data_ptr(), bias_axis
    g.relu = 1 if relu else 0
    rc = capi.lib().kutacc_hip_gemm(ctypes.byref(g), None)
    torch.cuda.synchronize()
    assert rc == 0, rc
    out = helpers.to_numpy(dC)
    if c_pad:
        assert np.all(out[:, :, N:] == -7.0), "columns beyond n were written"
    return out[:, :, :N]


def gemm_ref(A, B, bias=None, bias_axis=0, relu=False):
    ref = np.einsum("bmk,bnk->bmn", A.astype(np.float64), B.astype(np.float64))
    if bias_axis == 1:
        ref = ref + bias[None, None, :]
    elif bias_axis == 2:
        ref = ref + bias[None, :, None]
    return np.maximum(ref, 0) if relu else ref


@pytest.mark.parametrize("path", [capi.PATH_FUSED, capi.PATH_GENERIC], ids=["mfma", "scalar"])
@pytest.mark.parametrize("shape", [(1, 128, 128, 64), (1, 300, 136, 72), (3, 72, 264, 200), (2, 40, 8, 8)])
def test_gemm_k_major_operands(torch_cuda, shape, path):
    """Ragged tiles in m and n, a k tail that is not a multiple of the 64-wide step, batches."""
    nb, M, N, K = shape
    rng = np.random.Generator(np.random.PCG64(100 + M))
    A, B = draw(rng, nb, M, K), draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    got = run_gemm(torch_cuda, A, B, path=path, c_pad=8)
    helpers.assert_within(got, gemm_ref(A, B), GEMM_TOL(gemm_ref(A, B)), f"gemm {shape}")


@pytest.mark.parametrize("bias_axis,relu", [(1, False), (1, True), (2, False), (2, True)])
@pytest.mark.parametrize("path", [capi.PATH_FUSED, capi.PATH_GENERIC], ids=["mfma", "scalar"])
def test_gemm_bias_and_relu_epilogues(torch_cuda, path, bias_axis, relu):
    nb, M, N, K = 2, 200, 168, 96
    rng = np.random.Generator(np.random.PCG64(7))
    A, B = draw(rng, nb, M, K), draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    bias = rng.standard_normal(N if bias_axis == 1 else M).astype(np.float32)
    got = run_gemm(torch_cuda, A, B, bias=bias, bias_axis=bias_axis, relu=relu, path=path)
    ref = gemm_ref(A, B, bias, bias_axis, relu)
    helpers.assert_within(got, ref, GEMM_TOL(ref), f"bias axis {bias_axis} relu {relu}")
    if relu:
        assert got.min() >= 0.0


@pytest.mark.parametrize("a_mmajor,b_mmajor", [(True, True), (True, False), (False, True)])
@pytest.mark.parametrize("shape", [(2, 128, 128, 64), (3, 200, 136, 100), (1, 64, 72, 45)])
def test_gemm_m_major_operands(torch_cuda, shape, a_mmajor, b_mmajor):
    """Operands stored transposed (contraction index slowest), as the incoming triangle equation has them."""
    nb, M, N, K = shape
    if not b_mmajor or not a_mmajor:
        K = (K + 7) // 8 * 8  # a k-major operand next to it needs k in whole 16-byte chunks
    rng = np.random.Generator(np.random.PCG64(200 + M + K))
    A, B = draw(rng, nb, M, K), draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    got = run_gemm(torch_cuda, A, B, a_mmajor=a_mmajor, b_mmajor=b_mmajor, path=capi.PATH_FUSED)
    ref = gemm_ref(A, B)
    helpers.assert_within(got, ref, GEMM_TOL(ref), f"m-major {a_mmajor}/{b_mmajor} {shape}")
    same = run_gemm(torch_cuda, A, B, a_mmajor=a_mmajor, b_mmajor=b_mmajor, path=capi.PATH_GENERIC)
    helpers.assert_within(got, same, 1e-3 + 8e-3 * np.abs(same), "mfma vs scalar kernel")


@pytest.fixture
def gemm_tile():
    """Forces the tile size of the matrix products ("256": the large tiles wherever the shape allows, "128": never)."""
    def choose(value):
        assert capi.set_tuning("gemm_tile", value) == 0
    yield choose
    capi.set_tuning("gemm_tile", None)


def first_profiled_kernel(torch, fn):
    capi.lib().kutacc_hip_profile_enable(1)
    try:
        fn()
        torch.cuda.synchronize()
        name = ctypes.create_string_buffer(96)
        ms, cnt, fl = ctypes.c_double(), ctypes.c_int64(), ctypes.c_double()
        assert capi.lib().kutacc_hip_profile_read(0, name, 96, ctypes.byref(ms), ctypes.byref(cnt), ctypes.byref(fl)) == 0
        return name.value.decode()
    finally:
        capi.lib().kutacc_hip_profile_enable(0)


@pytest.mark.parametrize("mmajor", [False, True], ids=["k-major", "m-major"])
@pytest.mark.parametrize("tile", ["256", "192", "direct"])
@pytest.mark.parametrize("units", [(2, 1, 1, 64), (1, 2, 1, 192), (3, 1, 3, 320), (9, 1, 1, 128), (300, 1, 1, 64), (40, 2, 2, 512)])
def test_gemm_large_tiles(torch_cuda, gemm_tile, units, tile, mmajor):
    """The 256 x 256 tiles (128 x 128 per wave; staged through registers, and loaded straight into the LDS) and the
    192 x 192 ones (96 x 96 per wave) against the float64 product and, bit for bit, against the 128 x 128 tiles, which
    add the same products in the same order: one and several k-steps, an odd number of them (the register-staged kernels
    take them in pairs), several tiles per batch, and more tiles than the chip has CUs (a workgroup then walks several,
    its operand pipeline running across the tile boundary).  The direct tiles need three stages of 32 k: the one-step
    cases run with 128 there."""
    nb, mt, nt, K = units
    side = 192 if tile == "192" else 256
    if tile == "direct":
        K = max(K, 128)
    M, N = mt * side, nt * side
    shape = (nb, M, N, K)
    rng = np.random.Generator(np.random.PCG64(300 + M + N + K))
    A, B = draw(rng, nb, M, K), draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    gemm_tile(tile)
    name = first_profiled_kernel(torch_cuda, lambda: run_gemm(torch_cuda, A, B, a_mmajor=mmajor, b_mmajor=mmajor, path=capi.PATH_FUSED))
    assert name.startswith("pair_gemm_direct_kernel" if tile == "direct" else "pair_gemm_big_kernel"), name
    got = run_gemm(torch_cuda, A, B, a_mmajor=mmajor, b_mmajor=mmajor, path=capi.PATH_FUSED, c_pad=8)
    ref = gemm_ref(A, B)
    helpers.assert_within(got, ref, GEMM_TOL(ref), f"large tiles {shape}")
    gemm_tile("128")
    small = run_gemm(torch_cuda, A, B, a_mmajor=mmajor, b_mmajor=mmajor, path=capi.PATH_FUSED, c_pad=8)
    assert np.array_equal(got, small)


@pytest.mark.parametrize("n", [384, 512, 576, 768, 1024])
def test_equation_at_384_residues_and_more_takes_the_large_tiles(torch_cuda, n):
    """128 channels of 512 x 512, 768 x 768 and 1024 x 1024 (whole 256 x 256 tiles, two, four and a half and eight per
    CU: the default rule gives them to the kernel that loads its operands straight into the LDS); of 384 x 384 and
    576 x 576, whose sides are whole 192 x 192 tiles (two and four and a half per CU).  Sampled channels against the
    oracle; the incoming form equals the outgoing one on transposed operands bit for bit."""
    from oracle import oracle
    torch = torch_cuda
    c_i = 128
    g = torch.Generator(device="cuda").manual_seed(77)
    left = (torch.randn(c_i, n, n, device="cuda", generator=g)).to(torch.bfloat16)
    right = (torch.randn(c_i, n, n, device="cuda", generator=g) * n ** -0.5).to(torch.bfloat16)
    for incoming in (False, True):
        name = first_profiled_kernel(torch, lambda: equation(torch, left, right, n, incoming))
        if n % 256 == 0:
            assert name == "pair_gemm_direct_kernel" + ("<m-major>" if incoming else ""), name
        else:
            assert name == "pair_gemm_big_kernel<" + ("m-major, " if incoming else "") + "192>", name
    out_c = equation(torch, left, right, n, False)
    in_c = equation(torch, left, right, n, True)
    chans = [0, 63, 127]
    l_np, r_np = helpers.to_numpy(left[chans]), helpers.to_numpy(right[chans])
    for incoming, got in ((False, out_c), (True, in_c)):
        ref = oracle.tm_equation_f32(l_np, r_np, incoming)
        helpers.assert_within(helpers.to_numpy(got[chans]), ref, 2e-2 + 6e-3 * np.abs(ref), f"equation incoming={incoming}")
    lt, rt = left.transpose(1, 2).contiguous(), right.transpose(1, 2).contiguous()
    swapped = equation(torch, rt, lt, n, False)
    assert helpers.same_bits(swapped, in_c)


@pytest.mark.parametrize("bias_axis,relu", [(1, False), (1, True), (2, False), (2, True), (0, False)])
@pytest.mark.parametrize("path", [capi.PATH_FUSED, capi.PATH_GENERIC], ids=["mfma", "scalar"])
def test_gemm_gated_form_bias_axes(torch_cuda, path, bias_axis, relu):
    """The gated form C = bf16(bf16(relu?(A.B^T + bias)) * mask[n] * sigmoid(bf16(A_gate.B^T + bias_gate))) with the biases
    along either axis: each product takes its own bias, and ReLU applies to the projection only.  Against float64 with the
    same two intermediate roundings."""
    torch = torch_cuda
    nb, M, N, K = 2, 136, 200, 96
    rng = np.random.Generator(np.random.PCG64(31 + bias_axis))
    A, G = draw(rng, nb, M, K), draw(rng, nb, M, K)
    B = draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    mask = (rng.random((nb, N)) > 0.2).astype(np.float32)
    blen = N if bias_axis == 1 else M
    bias, bias_gate = (rng.standard_normal(blen).astype(np.float32) for _ in range(2))
    dA, dG, dB, dmask = dev(torch, A), dev(torch, G), dev(torch, B), dev(torch, mask)
    dC = torch.full((nb, M, N), -7.0, dtype=torch.bfloat16, device="cuda")
    g = capi.HipGemmArgs()
    g.m, g.n, g.k, g.batches, g.dtype, g.path = M, N, K, nb, capi.K_BF16, path
    g.a, g.a_gate, g.a_stride_m, g.a_stride_k, g.a_stride_batch = dA.data_ptr(), dG.data_ptr(), K, 1, M * K
    g.b, g.b_stride_n, g.b_stride_k, g.b_stride_batch = dB.data_ptr(), K, 1, N * K
    g.c, g.c_stride_m, g.c_stride_batch = dC.data_ptr(), N, M * N
    g.mask, g.mask_stride_batch = dmask.data_ptr(), N
    keep = [dev(torch, bias, torch.float32), dev(torch, bias_gate, torch.float32)]
    if bias_axis:
        g.bias, g.bias_gate, g.bias_axis = keep[0].data_ptr(), keep[1].data_ptr(), bias_axis
    g.relu = 1 if relu else 0
    rc = capi.lib().kutacc_hip_gemm(ctypes.byref(g), None)
    torch.cuda.synchronize()
    assert rc == 0, rc
    A, G, B = (round_to_bf16(v) for v in (A, G, B))
    proj = gemm_ref(A, B, bias, bias_axis, relu)
    gate = gemm_ref(G, B, bias_gate, bias_axis, False)
    proj, gate = round_to_bf16(proj.astype(np.float32)).astype(np.float64), round_to_bf16(gate.astype(np.float32)).astype(np.float64)
    ref = proj * mask[:, None, :] / (1.0 + np.exp(-gate))
    got = helpers.to_numpy(dC)
    helpers.assert_within(got, ref, 2e-3 + 1.2e-2 * np.abs(ref), f"gated gemm, bias axis {bias_axis}, relu {relu}")
    assert np.all(got[np.broadcast_to(mask[:, None, :] == 0, got.shape)] == 0), "masked positions must be exactly zero"


def _gemm_sweep():
    rng = np.random.Generator(np.random.PCG64(777))
    cases = []
    for i in range(20):
        nb = int(rng.integers(1, 4))
        M, N, K = (int(8 * rng.integers(1, 60)) for _ in range(3))
        am, bm = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        bias_axis, relu = int(rng.integers(0, 3)), bool(rng.integers(0, 2))
        cases.append((i, nb, M, N, K, am, bm, bias_axis, relu))
    return cases


@pytest.mark.parametrize("index,nb,M,N,K,am,bm,bias_axis,relu", _gemm_sweep())
def test_gemm_seeded_sweep(torch_cuda, index, nb, M, N, K, am, bm, bias_axis, relu):
    """20 seeded combinations of sizes (multiples of 8 up to 472), batches, operand orders and epilogues on the MFMA
    kernel, against float64."""
    rng = np.random.Generator(np.random.PCG64(900 + index))
    A, B = draw(rng, nb, M, K), draw(rng, nb, N, K, scale=1 / math.sqrt(K))
    bias = rng.standard_normal(N if bias_axis == 1 else M).astype(np.float32) if bias_axis else None
    got = run_gemm(torch_cuda, A, B, a_mmajor=am, b_mmajor=bm, bias=bias, bias_axis=bias_axis, relu=relu,
                   path=capi.PATH_FUSED, c_pad=8)
    ref = gemm_ref(A, B, bias, bias_axis, relu)
    helpers.assert_within(got, ref, GEMM_TOL(ref), f"gemm sweep {index}: {nb}x{M}x{N}x{K} am={am} bm={bm}")


def test_gemm_rejects_what_it_cannot_run(torch_cuda):
    torch = torch_cuda
    t = torch.zeros(64 * 64, dtype=torch.bfloat16, device="cuda")
    g = capi.HipGemmArgs()
    g.m, g.n, g.k, g.batches, g.dtype, g.path = 8, 8, 12, 1, capi.K_BF16, capi.PATH_FUSED  # k not a multiple of 8
    g.a, g.a_stride_m, g.a_stride_k = t.data_ptr(), 12, 1
    g.b, g.b_stride_n, g.b_stride_k = t.data_ptr(), 12, 1
    g.c, g.c_stride_m = t.data_ptr(), 8
    assert capi.lib().kutacc_hip_gemm(ctypes.byref(g), None) == capi.EUNSUPPORTED
    g.path = capi.PATH_AUTO
    assert capi.lib().kutacc_hip_gemm(ctypes.byref(g), None) == 0
    g.dtype = capi.K_FP32
    assert capi.lib().kutacc_hip_gemm(ctypes.byref(g), None) == capi.EINVAL
    torch.cuda.synchronize()


# ---- transition ------------------------------------------------------------------------------------------------
def transition_case(seed, batch, n_res, c_o, c_i):
    rng = np.random.Generator(np.random.PCG64(seed))
    return dict(x=draw(rng, batch, n_res, c_o), w1=draw(rng, c_i, c_o, scale=1 / math.sqrt(c_o)),
                b1=rng.standard_normal(c_i).astype(np.float32) * 0.5, w2=draw(rng, c_o, c_i, scale=1 / math.sqrt(c_i)),
                b2=rng.standard_normal(c_o).astype(np.float32) * 0.5)


def run_transition(torch, c, path=None):
    """path None: the handle-based entry point; else kutacc_hip_transition with that path."""
    batch, n_res, c_o = c["x"].shape
    c_i = c["w1"].shape[0]
    mid = torch.full((batch * n_res, c_i), -5.0, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((batch, n_res, c_o), dtype=torch.bfloat16, device="cuda")
    t = [dev(torch, c["x"]), dev(torch, c["w1"]), dev(torch, c["b1"], torch.float32), dev(torch, c["w2"]),
         dev(torch, c["b2"], torch.float32)]
    if path is None:
        op = capi.Transition(*t, mid, out)
        op.run()
        assert not capi.error_flag()
    else:
        rc = capi.lib().kutacc_hip_transition(*[a.data_ptr() for a in t], mid.data_ptr(), out.data_ptr(), batch * n_res,
                                              c_o, c_i, capi.K_BF16, path, None)
        torch.cuda.synchronize()
        assert rc == 0, rc
    return out, mid


@pytest.mark.parametrize("shape", [(2, 37, 128, 512), (3, 50, 256, 1024), (1, 300, 128, 64), (1, 9, 24, 40), (2, 5, 6, 10)])
@pytest.mark.parametrize("path", [None, capi.PATH_GENERIC], ids=["entry point", "two launches"])
def test_transition_small(torch_cuda, shape, path):
    """Pair (128 -> 512) and MSA (256 -> 1024) channel counts at ragged row counts (the one-kernel form through the
    entry point, the two-GEMM form when forced), and channel counts that only the GEMM kernels take."""
    from oracle import oracle
    c = transition_case(300 + shape[2], *shape)
    out, mid = run_transition(torch_cuda, c, path)
    ref, ref_mid = oracle.transition_f32(c["x"].reshape(-1, shape[2]), c["w1"], c["b1"], c["w2"], c["b2"], return_mid=True)
    one_kernel = path is None and shape[2] in (128, 256)
    if one_kernel:
        assert bool((mid == -5.0).all()), "the one-kernel form must leave the intermediate tensor alone"
    else:
        helpers.assert_within(helpers.to_numpy(mid), ref_mid, GEMM_TOL(ref_mid), "hidden layer")
    helpers.check_close(helpers.to_numpy(out).reshape(ref.shape), ref, "bf16", f"transition {shape}")


def _transition_sweep():
    rng = np.random.Generator(np.random.PCG64(4242))
    return [(i, int(rng.integers(1, 4)), int(rng.integers(1, 900)), int(rng.choice([128, 256])), int(64 * rng.integers(1, 17)))
            for i in range(12)]


@pytest.mark.parametrize("index,batch,n_res,c_o,c_i", _transition_sweep())
def test_transition_seeded_sweep(torch_cuda, index, batch, n_res, c_o, c_i):
    """12 seeded row counts (1 to 2700) and hidden widths (64 to 1024) of the one-kernel transition against the oracle."""
    from oracle import oracle
    c = transition_case(1300 + index, batch, n_res, c_o, c_i)
    out, mid = run_transition(torch_cuda, c)
    assert bool((mid == -5.0).all())
    ref = oracle.transition_f32(c["x"].reshape(-1, c_o), c["w1"], c["b1"], c["w2"], c["b2"])
    helpers.check_close(helpers.to_numpy(out).reshape(ref.shape), ref, "bf16", f"transition sweep {index}: {batch}x{n_res}x{c_o}->{c_i}")


def test_transition_forced_paths(torch_cuda):
    c = transition_case(305, 1, 70, 128, 256)
    a, _ = run_transition(torch_cuda, c, capi.PATH_FUSED)
    b, _ = run_transition(torch_cuda, c, capi.PATH_GENERIC)
    # same rounding points (bf16 hidden layer, fp32 accumulation): the two forms differ by summation order only
    helpers.assert_within(helpers.to_numpy(a), helpers.to_numpy(b), 1e-2 + 1e-2 * np.abs(helpers.to_numpy(b)), "fused vs two launches")
    t = torch_cuda.zeros(64, dtype=torch_cuda.bfloat16, device="cuda")
    f = torch_cuda.zeros(64, dtype=torch_cuda.float32, device="cuda")
    L = capi.lib()
    assert L.kutacc_hip_transition(t.data_ptr(), t.data_ptr(), f.data_ptr(), t.data_ptr(), f.data_ptr(), None, t.data_ptr(),
                                   2, 8, 8, capi.K_BF16, capi.PATH_FUSED, None) == capi.EUNSUPPORTED
    assert L.kutacc_hip_transition(t.data_ptr(), t.data_ptr(), f.data_ptr(), t.data_ptr(), f.data_ptr(), None, t.data_ptr(),
                                   2, 8, 8, capi.K_BF16, capi.PATH_AUTO, None) == capi.EINVAL  # needs the intermediate


def test_transition_full_pair_size(torch_cuda):
    """The pair transition of a 384-residue model at its real shape (147456 rows); the oracle checks a sample of
    rows (rows are independent), and a second call on a row permutation must give the permuted result bit for bit."""
    from oracle import oracle
    torch = torch_cuda
    c = transition_case(310, 384, 384, 128, 512)
    out, _ = run_transition(torch, c)
    rows = np.random.Generator(np.random.PCG64(1)).choice(384 * 384, size=1024, replace=False)
    ref = oracle.transition_f32(c["x"].reshape(-1, 128)[rows], c["w1"], c["b1"], c["w2"], c["b2"])
    helpers.check_close(helpers.to_numpy(out).reshape(-1, 128)[rows], ref, "bf16", "transition 384x384")
    c2 = dict(c, x=np.ascontiguousarray(c["x"][::-1]))
    out2, _ = run_transition(torch, c2)
    assert helpers.same_bits(out2, torch.flip(out, dims=[0]))


# ---- triangle multiplication -----------------------------------------------------------------------------------
def tm_case(seed, n, c_o, c_i):
    rng = np.random.Generator(np.random.PCG64(seed))
    w = lambda o, i: draw(rng, o, i, scale=1 / math.sqrt(i))  # noqa: E731
    b = lambda k: (rng.standard_normal(k) * 0.5).astype(np.float32)  # noqa: E731
    return dict(x=draw(rng, n, n, c_o), mask=(rng.random((n, n)) > 0.15).astype(np.float32),
                lpw=w(c_i, c_o), lpb=b(c_i), lgw=w(c_i, c_o), lgb=b(c_i),
                rpw=w(c_i, c_o), rpb=b(c_i), rgw=w(c_i, c_o), rgb=b(c_i),
                gating_w=w(c_o, c_o), gating_b=b(c_o), out_w=w(c_o, c_i), out_b=b(c_o))


def calc_proj(torch, c, side, n, c_o, c_i, dx, dmask):
    proj = torch.zeros((c_i, n, n), dtype=torch.bfloat16, device="cuda")
    gate = torch.zeros_like(proj)
    keep = [dev(torch, c[side + "pw"]), dev(torch, c[side + "pb"], torch.float32), dev(torch, c[side + "gw"]),
            dev(torch, c[side + "gb"], torch.float32)]
    h = [capi.tensor(t) if t.dtype == torch.bfloat16 else capi.tensor(t, capi.K_FP32) for t in keep]
    hp, hx, hg, hm = capi.tensor(proj), capi.tensor(dx), capi.tensor(gate), capi.tensor(dmask)
    acts = capi.TmActInputs(n, n, hp.handle, hx.handle, hg.handle)
    weights = capi.TmProjWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle, h[3].handle)
    capi.kutacc_af2_triangle_multiplication_calc_proj(acts, hm, weights, False)
    assert not capi.error_flag()
    return proj


def equation(torch, left, right, n, incoming):
    center = torch.zeros_like(left)
    hc, hl, hr = capi.tensor(center), capi.tensor(left), capi.tensor(right)
    capi.kutacc_af2_triangle_multiplication_equation(hc, hl, hr, n, incoming)
    assert not capi.error_flag()
    return center


@pytest.mark.parametrize("n,c_o,c_i", [(40, 128, 128), (24, 64, 32), (7, 6, 5)])
@pytest.mark.parametrize("incoming", [False, True], ids=["outgoing", "incoming"])
def test_triangle_multiplication_steps(torch_cuda, n, c_o, c_i, incoming):
    """Each of the four entry points against its oracle function, on the oracle's (unrounded) inputs to that step
    rounded to bf16, so that an error in one step is not hidden by the tolerance of the next."""
    from oracle import oracle
    torch = torch_cuda
    c = tm_case(400 + n, n, c_o, c_i)
    dx, dmask = dev(torch, c["x"]), dev(torch, c["mask"])
    # 1. projections
    left = calc_proj(torch, c, "l", n, c_o, c_i, dx, dmask)
    right = calc_proj(torch, c, "r", n, c_o, c_i, dx, dmask)
    ref_l = oracle.tm_calc_proj_f32(c["x"], c["mask"], c["lpw"], c["lpb"], c["lgw"], c["lgb"])
    ref_r = oracle.tm_calc_proj_f32(c["x"], c["mask"], c["rpw"], c["rpb"], c["rgw"], c["rgb"])
    helpers.check_close(helpers.to_numpy(left), ref_l, "bf16", "left projection")
    helpers.check_close(helpers.to_numpy(right), ref_r, "bf16", "right projection")
    assert bool((left[:, dmask == 0] == 0).all()), "masked positions must be exactly zero"
    # 2. equation, on bf16-rounded oracle projections
    in_l, in_r = round_to_bf16(ref_l), round_to_bf16(ref_r)
    center = equation(torch, dev(torch, in_l), dev(torch, in_r), n, incoming)
    ref_c = oracle.tm_equation_f32(in_l, in_r, incoming)
    helpers.assert_within(helpers.to_numpy(center), ref_c, GEMM_TOL(ref_c), "equation")
    # 3. gate and output projection on a channel-last, normalised centre (the caller's layer norm is not part of the step)
    ctr = round_to_bf16(np.ascontiguousarray(ref_c.transpose(1, 2, 0)) / math.sqrt(n))
    d_ctr = dev(torch, ctr)
    gate = torch.zeros((n, n, c_o), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros_like(gate)
    keep = [dev(torch, c["gating_w"]), dev(torch, c["gating_b"], torch.float32), dev(torch, c["out_w"]),
            dev(torch, c["out_b"], torch.float32)]
    h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
    hx, hg, ho, hc = capi.tensor(dx), capi.tensor(gate), capi.tensor(out), capi.tensor(d_ctr)
    acts = capi.TmActInputs(n, n, None, hx.handle, None)
    weights = capi.TmLinearWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle, h[3].handle)
    capi.kutacc_af2_triangle_multiplication_gate_and_out_linear(hg, ho, acts, hc, weights, False)
    assert not capi.error_flag()
    ref_gate, ref_out = oracle.tm_gate_and_out_f32(c["x"], ctr, c["gating_w"], c["gating_b"], c["out_w"], c["out_b"])
    helpers.assert_within(helpers.to_numpy(gate).reshape(ref_gate.shape), ref_gate, GEMM_TOL(ref_gate), "gate")
    helpers.assert_within(helpers.to_numpy(out).reshape(ref_out.shape), ref_out, GEMM_TOL(ref_out), "output projection")
    # 4. last: out *= sigmoid(gate), on the device's own gate and out
    want = oracle.tm_last_f32(helpers.to_numpy(out), helpers.to_numpy(gate))
    capi.kutacc_af2_triangle_multiplication_last(ho, hg, n, n, c_o)
    assert not capi.error_flag()
    helpers.assert_within(helpers.to_numpy(out), want, 1e-3 + 6e-3 * np.abs(want), "gated output")


def test_triangle_multiplication_full_size_properties(torch_cuda):
    """384 residues, 128 channels at the real shape.  The oracle checks a sample of channels of the equation and a
    sample of positions of the projection; size-independent properties cover the rest: the incoming equation equals
    the outgoing one on transposed operands, and a masked position is exactly zero."""
    from oracle import oracle
    torch = torch_cuda
    n, c_o, c_i = 384, 128, 128
    c = tm_case(500, n, c_o, c_i)
    dx, dmask = dev(torch, c["x"]), dev(torch, c["mask"])
    left = calc_proj(torch, c, "l", n, c_o, c_i, dx, dmask)
    right = calc_proj(torch, c, "r", n, c_o, c_i, dx, dmask)
    rows = np.random.Generator(np.random.PCG64(2)).choice(n, size=6, replace=False)
    ref_rows = oracle.tm_calc_proj_f32(c["x"][rows], c["mask"][rows], c["lpw"], c["lpb"], c["lgw"], c["lgb"])
    helpers.check_close(helpers.to_numpy(left[:, torch.from_numpy(rows).cuda()]), ref_rows, "bf16", "left projection rows")
    assert bool((right[:, dmask == 0] == 0).all())
    out_c = equation(torch, left, right, n, False)
    in_c = equation(torch, left, right, n, True)
    chans = [0, 77, 127]
    l_np, r_np = helpers.to_numpy(left[chans]), helpers.to_numpy(right[chans])
    for incoming, got in ((False, out_c), (True, in_c)):
        ref = oracle.tm_equation_f32(l_np, r_np, incoming)
        helpers.assert_within(helpers.to_numpy(got[chans]), ref, 2e-2 + 6e-3 * np.abs(ref), f"equation incoming={incoming}")
    lt, rt = left.transpose(1, 2).contiguous(), right.transpose(1, 2).contiguous()
    swapped = equation(torch, rt, lt, n, False)  # outgoing(right^T, left^T) == incoming(left, right)
    assert helpers.same_bits(swapped, in_c)


def gated_projection_once(torch, t, c, n_pos, ld_out, mode, ld_w=None):
    """One gated projection [c, n_pos] = f(x [n_pos, c]) through kutacc_hip_gemm under kutacc_hip_set_tuning("gated_projection",
    mode); returns the name of the kernel that ran and the result (allocated with row pitch ld_out, filled with -3)."""
    ld_w = ld_w or c
    assert capi.set_tuning("gated_projection", mode) == 0
    try:
        out = torch.full((c, ld_out), -3.0, dtype=torch.bfloat16, device="cuda")
        g = capi.HipGemmArgs()
        g.m, g.n, g.k, g.batches, g.dtype, g.path = c, n_pos, c, 1, capi.K_BF16, capi.PATH_FUSED
        g.a, g.a_gate, g.a_stride_m, g.a_stride_k = t["pw"].data_ptr(), t["gw"].data_ptr(), ld_w, 1
        g.b, g.b_stride_n, g.b_stride_k = t["x"].data_ptr(), c, 1
        g.c, g.c_stride_m = out.data_ptr(), ld_out
        g.bias, g.bias_gate, g.bias_axis, g.mask = t["pb"].data_ptr(), t["gb"].data_ptr(), 2, t["mask"].data_ptr()
        name = first_profiled_kernel(torch, lambda: capi.lib().kutacc_hip_gemm(ctypes.byref(g), None))
        assert not capi.error_flag()
        return name, out
    finally:
        capi.set_tuning("gated_projection", None)


@pytest.mark.parametrize("n_pos,pad", [(8, 0), (72, 8), (64 * 3 + 8, 0), (384 * 384, 0), (512 * 512 + 40, 24), (64 * 700, 0)])
def test_gated_projection_with_weights_in_registers(torch_cuda, n_pos, pad):
    """The default kernel of the gated projection at 128 channels: a wave keeps the weights of its 32 output channels in
    registers, the workgroup shares the activation through the LDS (loaded straight into it, a ring of stages requested
    ahead).  One step, a ragged last step, fewer steps than the ring is deep, more steps than workgroups, a padded
    output pitch (the padding stays untouched): bit for bit against the streaming kernel, which does the same arithmetic
    in the same order, and a sample of positions against the oracle."""
    from oracle import oracle
    torch = torch_cuda
    c = 128
    rng = np.random.Generator(np.random.PCG64(900 + n_pos))
    x = draw(rng, n_pos, c)
    mask = (rng.random(n_pos) > 0.15).astype(np.float32)
    pw, gw = draw(rng, c, c, scale=1 / math.sqrt(c)), draw(rng, c, c, scale=1 / math.sqrt(c))
    pb, gb = (rng.standard_normal(c) * 0.5).astype(np.float32), (rng.standard_normal(c) * 0.5).astype(np.float32)
    t = dict(x=dev(torch, x), mask=dev(torch, mask), pw=dev(torch, pw), gw=dev(torch, gw), pb=dev(torch, pb, torch.float32),
             gb=dev(torch, gb, torch.float32))
    name, got = gated_projection_once(torch, t, c, n_pos, n_pos + pad, None)
    assert name == "gated_projection_blocks_kernel", name
    name, other = gated_projection_once(torch, t, c, n_pos, n_pos + pad, "streaming")
    assert name == "gated_projection_kernel", name
    assert helpers.same_bits(got, other)
    if pad:
        assert bool((got[:, n_pos:] == -3.0).all())
    sample = np.unique(np.concatenate([np.arange(0, min(96, n_pos)), np.arange(max(0, n_pos - 96), n_pos),
                                       rng.choice(n_pos, size=min(n_pos, 512), replace=False)]))
    ref = oracle.tm_calc_proj_f32(x[sample][None], mask[sample][None], pw, pb, gw, gb)[:, 0]
    helpers.check_close(helpers.to_numpy(got[:, torch.from_numpy(sample).cuda()]), ref, "bf16", "gated projection, weights in registers")
    assert bool((got[:, :n_pos][:, t["mask"] == 0] == 0).all())


def test_gated_projection_streaming_kernel(torch_cuda):
    """The weight-resident streaming kernel of the gated projection (every wave its own positions, the weights in the
    LDS; behind kutacc_hip_set_tuning("gated_projection", "streaming")).  512 x 512 positions plus a ragged tail of 40; the
    oracle checks a sample of positions and the ends of the range, and the tiled kernel on the same operands must agree
    within one bf16 rounding."""
    from oracle import oracle
    torch = torch_cuda
    n_pos, c = 512 * 512 + 40, 128
    rng = np.random.Generator(np.random.PCG64(900))
    x = draw(rng, n_pos, c)
    mask = (rng.random(n_pos) > 0.15).astype(np.float32)
    pw, gw = draw(rng, c, c, scale=1 / math.sqrt(c)), draw(rng, c, c, scale=1 / math.sqrt(c))
    pb, gb = (rng.standard_normal(c) * 0.5).astype(np.float32), (rng.standard_normal(c) * 0.5).astype(np.float32)
    t = dict(x=dev(torch, x), mask=dev(torch, mask), pw=dev(torch, pw), gw=dev(torch, gw), pb=dev(torch, pb, torch.float32),
             gb=dev(torch, gb, torch.float32))
    # weights with a padded leading dimension are outside the dedicated kernels' shapes: the same product on the tiled kernel
    pad_w = lambda w: torch.nn.functional.pad(w, (0, 8)).contiguous()  # noqa: E731
    padded = dict(t, pw=pad_w(t["pw"]), gw=pad_w(t["gw"]))
    outs = [gated_projection_once(torch, t, c, n_pos, n_pos, "streaming"),
            gated_projection_once(torch, padded, c, n_pos, n_pos, "streaming", ld_w=c + 8)]
    assert outs[0][0] == "gated_projection_kernel" and outs[1][0] == "pair_gemm_kernel<gated>", [o[0] for o in outs]
    sample = np.concatenate([np.arange(0, 96), np.arange(n_pos - 96, n_pos),
                             rng.choice(n_pos, size=2048, replace=False)])
    ref = oracle.tm_calc_proj_f32(x[sample][None], mask[sample][None], pw, pb, gw, gb)[:, 0]
    got = helpers.to_numpy(outs[0][1][:, torch.from_numpy(sample).cuda()])
    helpers.check_close(got, ref, "bf16", "streaming gated projection")
    a, b = helpers.to_numpy(outs[0][1]), helpers.to_numpy(outs[1][1])
    helpers.assert_within(a, b, 4e-3 + 1.2e-2 * np.abs(b), "streaming vs tiled kernel")
    assert bool((outs[0][1][:, t["mask"] == 0] == 0).all())


def test_pair_stack_against_the_golden_fixture(torch_cuda):
    """The committed float64 fixture (tests/golden/pair_stack_tiny.npz) through the handle-based entry points.  Its
    inputs are rounded to bf16 on the way to the device, so the comparison runs at the bf16 bar."""
    import os
    torch = torch_cuda
    g = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "pair_stack_tiny.npz"))
    n, c_o, c_i, hid = 6, 8, 4, 12
    d = lambda k, dt=torch.bfloat16: torch.from_numpy(g["in." + k]).to(device="cuda", dtype=dt)  # noqa: E731
    f32 = torch.float32
    # transition
    x = d("x")
    mid = torch.zeros(n * n, hid, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(n, n, c_o, dtype=torch.bfloat16, device="cuda")
    capi.Transition(x, d("w1"), d("b1", f32), d("w2"), d("b2", f32), mid, out).run()
    assert not capi.error_flag()
    helpers.check_close(helpers.to_numpy(out), g["transition.out"], "bf16", "fixture transition")
    # projections and equation
    proj = {}
    for side in ("left", "right"):
        p = torch.zeros(c_i, n, n, dtype=torch.bfloat16, device="cuda")
        keep = [d(side + "_w"), d(side + "_b", f32), d(side + "_gw"), d(side + "_gb", f32), d("mask"), torch.zeros_like(p)]
        h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
        hp, hx, hm, hg = capi.tensor(p), capi.tensor(x), capi.tensor(keep[4]), capi.tensor(keep[5])
        capi.kutacc_af2_triangle_multiplication_calc_proj(capi.TmActInputs(n, n, hp.handle, hx.handle, hg.handle), hm,
                                                          capi.TmProjWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle,
                                                                             h[3].handle), False)
        assert not capi.error_flag()
        helpers.check_close(helpers.to_numpy(p), g["tm." + side], "bf16", f"fixture {side} projection")
        proj[side] = p
    for name, incoming in (("tm.outgoing", False), ("tm.incoming", True)):
        center = equation(torch, proj["left"], proj["right"], n, incoming)
        helpers.check_close(helpers.to_numpy(center), g[name], "bf16", "fixture " + name)
    # output step
    gate = torch.zeros(n, n, c_o, dtype=torch.bfloat16, device="cuda")
    res = torch.zeros_like(gate)
    keep = [d("gating_w"), d("gating_b", f32), d("out_w"), d("out_b", f32), d("center")]
    h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
    hx, hgt, hres, hc = capi.tensor(x), capi.tensor(gate), capi.tensor(res), capi.tensor(keep[4])
    capi.kutacc_af2_triangle_multiplication_gate_and_out_linear(hgt, hres, capi.TmActInputs(n, n, None, hx.handle, None), hc,
                                                                capi.TmLinearWeights(c_o, c_i, h[0].handle, h[1].handle,
                                                                                     h[2].handle, h[3].handle), False)
    capi.kutacc_af2_triangle_multiplication_last(hres, hgt, n, n, c_o)
    assert not capi.error_flag()
    helpers.check_close(helpers.to_numpy(gate), g["tm.gate"], "bf16", "fixture gate")
    helpers.check_close(helpers.to_numpy(res), g["tm.last"], "bf16", "fixture gated output")


# ---- host pointers: staged through the device, bit-identical to the device-pointer call -----------------------
def _bits(t):
    """bf16 torch tensor (device) -> its bit patterns as a numpy uint16 array."""
    import torch
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def _host_bits(a):
    """float32 numpy array that holds bf16-representable values -> bf16 bit patterns (what a host caller passes)."""
    from oracle import oracle
    return oracle.to_bf16_bits(np.ascontiguousarray(a, dtype=np.float32))


def test_transition_host_pointers_match_device_pointers(torch_cuda):
    """The reference's callers hand kutacc_af2_transition host tensors (reference src/attention/transition.cpp:42-67)."""
    torch = torch_cuda
    for shape in [(2, 37, 128, 512), (1, 9, 24, 40)]:  # one-kernel form, two GEMM launches
        c = transition_case(77, *shape)
        out, _ = run_transition(torch, c)
        batch, n_res, c_o, c_i = shape
        h_out = np.zeros((batch, n_res, c_o), np.uint16)
        h_mid = np.zeros((batch * n_res, c_i), np.uint16)
        op = capi.Transition(_host_bits(c["x"]), _host_bits(c["w1"]), c["b1"], _host_bits(c["w2"]), c["b2"], h_mid, h_out)
        op.run()
        assert not capi.error_flag()
        np.testing.assert_array_equal(h_out, _bits(out))
    # mixed memory spaces are rejected
    x = dev(torch, c["x"])
    op = capi.Transition(x, _host_bits(c["w1"]), c["b1"], _host_bits(c["w2"]), c["b2"], h_mid, h_out)
    op.run()
    assert capi.error_flag()
    capi.clear_error()


@pytest.mark.parametrize("incoming", [False, True], ids=["outgoing", "incoming"])
def test_triangle_multiplication_host_pointers_match_device_pointers(torch_cuda, incoming):
    """All four steps on host arrays (reference src/attention/triangle_multiplication.cpp:153-240 takes host tensors)
    against the same steps on device tensors, bit for bit, each step fed the device result of the step before."""
    torch = torch_cuda
    n, c_o, c_i = 40, 128, 128
    c = tm_case(901, n, c_o, c_i)
    dx, dmask = dev(torch, c["x"]), dev(torch, c["mask"])
    hx, hmask = _host_bits(c["x"]), _host_bits(c["mask"])
    sides = {}
    for side in "lr":
        d_proj = calc_proj(torch, c, side, n, c_o, c_i, dx, dmask)
        h_proj = np.zeros((c_i, n, n), np.uint16)
        h_gate = np.zeros_like(h_proj)
        keep = [_host_bits(c[side + "pw"]), c[side + "pb"], _host_bits(c[side + "gw"]), c[side + "gb"]]
        h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
        hp, hxx, hg, hm = capi.tensor(h_proj), capi.tensor(hx), capi.tensor(h_gate), capi.tensor(hmask)
        acts = capi.TmActInputs(n, n, hp.handle, hxx.handle, hg.handle)
        weights = capi.TmProjWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle, h[3].handle)
        capi.kutacc_af2_triangle_multiplication_calc_proj(acts, hm, weights, False)
        assert not capi.error_flag()
        np.testing.assert_array_equal(h_proj, _bits(d_proj))
        sides[side] = (d_proj, h_proj)
    d_center = equation(torch, sides["l"][0], sides["r"][0], n, incoming)
    h_center = np.zeros((c_i, n, n), np.uint16)
    hc, hl, hr = capi.tensor(h_center), capi.tensor(sides["l"][1]), capi.tensor(sides["r"][1])
    capi.kutacc_af2_triangle_multiplication_equation(hc, hl, hr, n, incoming)
    assert not capi.error_flag()
    np.testing.assert_array_equal(h_center, _bits(d_center))
    # gate and output projection on a channel-last centre
    d_ctr = (d_center.permute(1, 2, 0).float() / math.sqrt(n)).to(torch.bfloat16).contiguous()
    h_ctr = _bits(d_ctr)
    d_gate = torch.zeros((n, n, c_o), dtype=torch.bfloat16, device="cuda")
    d_out = torch.zeros_like(d_gate)
    dkeep = [dev(torch, c["gating_w"]), dev(torch, c["gating_b"], torch.float32), dev(torch, c["out_w"]),
             dev(torch, c["out_b"], torch.float32)]
    hkeep = [_host_bits(c["gating_w"]), c["gating_b"], _host_bits(c["out_w"]), c["out_b"]]
    h_gate, h_out = np.zeros((n, n, c_o), np.uint16), np.zeros((n, n, c_o), np.uint16)
    results = []
    for keep, x_, gate_, out_, ctr_ in [(dkeep, dx, d_gate, d_out, d_ctr), (hkeep, hx, h_gate, h_out, h_ctr)]:
        h = [capi.tensor(keep[0]), capi.tensor(keep[1], capi.K_FP32), capi.tensor(keep[2]), capi.tensor(keep[3], capi.K_FP32)]
        hxx, hg, ho, hcc = capi.tensor(x_), capi.tensor(gate_), capi.tensor(out_), capi.tensor(ctr_)
        acts = capi.TmActInputs(n, n, None, hxx.handle, None)
        weights = capi.TmLinearWeights(c_o, c_i, h[0].handle, h[1].handle, h[2].handle, h[3].handle)
        capi.kutacc_af2_triangle_multiplication_gate_and_out_linear(hg, ho, acts, hcc, weights, False)
        assert not capi.error_flag()
        results.append((hg, ho))
    np.testing.assert_array_equal(h_gate, _bits(d_gate))
    np.testing.assert_array_equal(h_out, _bits(d_out))
    for hg, ho in results:
        capi.kutacc_af2_triangle_multiplication_last(ho, hg, n, n, c_o)
        assert not capi.error_flag()
    np.testing.assert_array_equal(h_out, _bits(d_out))
    assert np.any(h_out != 0)
