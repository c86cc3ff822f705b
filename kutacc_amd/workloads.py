"""Seeded synthetic inputs for the five benchmark configurations of the gated-attention operator.

Each configuration is described in operator terms (batch B, seq_len S, nheads H, head_size 32):

  1  MSA row attention, fp32     B=16   S=64   H=8  pair bias from z [64,64,128], mask all ones
  2  MSA row attention, bf16     B=512  S=256  H=8  pair bias from z [256,256,128], 5% residues padded
  3  triangle attention (start)  B=384  S=384  H=4  input = LN(z), pair bias = linear(LN(z)), mask ones
  4  MSA column attention        B=384  S=1024 H=8  no pair bias, 10% of sequences masked
  5  triangle attention (end)    B=1024 S=1024 H=4  input = LN(z^T), last 0-15% residues padded (pair mask)

Values: activations N(0,1), weights N(0, 1/fan_in), gating bias 1, output bias 0, LayerNorm with
gamma=1, beta=0, eps=1e-5 in front of the operator; mask bias = -1e9*(1-mask) as AlphaFold2 builds
it.  RNG: numpy PCG64 seeded with 1000 + config id; draw order: activations (m or z), then z for the
MSA configs, W_q, W_k, W_v, W_g, W_o, pair-bias weight, mask.  All arrays are returned as fp32
values; for bf16 configurations they are already rounded to bf16-representable values.
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np

HEAD_SIZE = 32
C_Z = 128
MASK_BIAS = -1e9

CONFIGS = {
    1: dict(name="msa_row_fp32", B=16, S=64, H=8, dtype="fp32", pair_bias=True),
    2: dict(name="msa_row_bf16", B=512, S=256, H=8, dtype="bf16", pair_bias=True),
    3: dict(name="triangle_start_bf16", B=384, S=384, H=4, dtype="bf16", pair_bias=True),
    4: dict(name="msa_col_bf16", B=384, S=1024, H=8, dtype="bf16", pair_bias=False),
    5: dict(name="triangle_end_bf16", B=1024, S=1024, H=4, dtype="bf16", pair_bias=True),
}


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    """fp32 -> nearest-even bf16 -> fp32, in numpy (no library dependence)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32)
    r = (u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) & np.uint32(0xFFFF0000)
    return r.view(np.float32)


def bf16_bits(a: np.ndarray) -> np.ndarray:
    """bf16 bit patterns (uint16) of an array that is already bf16-representable or to be rounded."""
    return (round_to_bf16(a).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def layernorm_np(x: np.ndarray, eps: float = 1e-5) -> np.ndarray:
    x = x.astype(np.float32)
    mean = x.mean(axis=-1, keepdims=True, dtype=np.float64)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True, dtype=np.float64)
    return ((x - mean) / np.sqrt(var + eps)).astype(np.float32)


@dataclass
class Workload:
    config: int
    name: str
    dtype: str  # "bf16" | "fp32"
    B: int
    S: int
    H: int
    d: int
    x: np.ndarray  # [B, S, C] operator input (already layer-normalised)
    wq: np.ndarray
    wk: np.ndarray
    wv: np.ndarray
    wg: np.ndarray
    wo: np.ndarray
    bg: np.ndarray  # fp32 [C]
    bo: np.ndarray  # fp32 [C]
    bias: np.ndarray  # [B, S] mask bias
    nb: np.ndarray | None  # [H, S, S] pair bias or None
    extras: dict = field(default_factory=dict)  # raw z / pair-bias weight for the producer kernels

    @property
    def C(self) -> int:
        return self.H * self.d

    def flops(self) -> int:
        """Algorithmic flops of one call: five CxC projections plus QK^T and PV."""
        return 10 * self.B * self.S * self.C * self.C + 4 * self.B * self.S * self.S * self.C

    def algorithmic_bytes(self) -> int:
        e = 2 if self.dtype == "bf16" else 4
        n = 2 * self.B * self.S * self.C * e + self.B * self.S * e + 5 * self.C * self.C * e + 2 * self.C * 4
        if self.nb is not None:
            n += self.H * self.S * self.S * e
        return n

    def batch_slice(self, rows) -> "Workload":
        """The same problem restricted to some batch rows (rows are independent in this operator)."""
        rows = np.asarray(rows)
        return Workload(self.config, self.name, self.dtype, len(rows), self.S, self.H, self.d,
                        np.ascontiguousarray(self.x[rows]), self.wq, self.wk, self.wv, self.wg, self.wo, self.bg,
                        self.bo, np.ascontiguousarray(self.bias[rows]), self.nb, self.extras)


def make_workload(config: int, batch: int | None = None, seq_len: int | None = None, keep_extras: bool = False) -> Workload:
    """Build configuration `config`; `batch` / `seq_len` override the extent (for reduced-size tests)."""
    spec = CONFIGS[config]
    B = batch or spec["B"]
    S = seq_len or spec["S"]
    H, d = spec["H"], HEAD_SIZE
    C = H * d
    dtype = spec["dtype"]
    rng = np.random.Generator(np.random.PCG64(1000 + config))
    rnd = round_to_bf16 if dtype == "bf16" else (lambda a: np.ascontiguousarray(a, dtype=np.float32))
    extras = {}

    triangle = config in (3, 5)
    if triangle:
        # the pair tensor is both the attention input (rows i = batch) and the source of the pair bias
        z = rng.standard_normal((S, S, C_Z), dtype=np.float32)
        if config == 5:
            z = np.ascontiguousarray(z.transpose(1, 0, 2))  # ending node: the operator sees z^T
        z = rnd(z)
        zn = rnd(layernorm_np(z))
        x = zn[:B]
    else:
        if config == 4:
            m = rng.standard_normal((S, B, C), dtype=np.float32)  # [N_seq, N_res, c_m]; attention over N_seq
            m = np.ascontiguousarray(m.transpose(1, 0, 2))
        else:
            m = rng.standard_normal((B, S, C), dtype=np.float32)
        x = rnd(layernorm_np(rnd(m)))
        z = zn = None
        if spec["pair_bias"]:
            z = rnd(rng.standard_normal((S, S, C_Z), dtype=np.float32))
            zn = rnd(layernorm_np(z))

    def weight(fan_out, fan_in):
        return rnd(rng.standard_normal((fan_out, fan_in), dtype=np.float32) / np.float32(np.sqrt(fan_in)))

    wq, wk, wv, wg, wo = (weight(C, C) for _ in range(5))
    bg = np.ones(C, dtype=np.float32)
    bo = np.zeros(C, dtype=np.float32)

    nb = None
    if spec["pair_bias"]:
        w_bias = weight(H, C_Z)
        nb = rnd(np.einsum("ijc,hc->hij", zn.astype(np.float32), w_bias, optimize=True))
        if keep_extras:
            extras = dict(z=z, z_norm=zn, w_bias=w_bias)

    bias = np.zeros((B, S), dtype=np.float32)
    if config == 2:
        keep = rng.random(S) >= 0.05  # residue mask shared by every sequence
        keep[0] = True
        bias[:] = (MASK_BIAS * (1.0 - keep.astype(np.float32)))[None, :]
    elif config == 4:
        keep = rng.random(S) >= 0.10  # sequence mask, identical for every residue
        keep[0] = True
        bias[:] = (MASK_BIAS * (1.0 - keep.astype(np.float32)))[None, :]
    elif config == 5:
        pad = int(np.floor(rng.random() * 0.15 * S))
        r = (np.arange(S) < S - pad).astype(np.float32)
        pair = r[:B, None] * r[None, :]  # rows past the padding start are fully masked
        bias[:] = MASK_BIAS * (1.0 - pair)
        extras["pad"] = pad
    bias = rnd(bias)

    return Workload(config, spec["name"], dtype, B, S, H, d, np.ascontiguousarray(x), wq, wk, wv, wg, wo, bg, bo, bias,
                    nb, extras)
