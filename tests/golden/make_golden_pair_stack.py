"""Writes tests/golden/pair_stack_tiny.npz: inputs and float64 results of the transition and of the triangle
multiplication steps on a tiny problem (n = 6 residues, 8 pair channels, 4 projected channels, hidden layer 12),
computed with plain numpy float64 einsum expressions written from the definitions (reference
src/attention/transition.cpp:31-38, src/attention/triangle_multiplication.cpp:37-66, 72-101, 115-126, 139-146) and
independent of oracle/kutacc_oracle.c.  The reference repository holds no numeric fixture for these operators.
Seed 20241.

    python tests/golden/make_golden_pair_stack.py
"""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def main():
    rng = np.random.Generator(np.random.PCG64(20241))
    n, c_o, c_i, hid = 6, 8, 4, 12
    f = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    d = dict(x=f(n, n, c_o), mask=(rng.random((n, n)) > 0.25).astype(np.float32),
             w1=f(hid, c_o) / np.sqrt(c_o), b1=f(hid), w2=f(c_o, hid) / np.sqrt(hid), b2=f(c_o),
             left_w=f(c_i, c_o) / np.sqrt(c_o), left_b=f(c_i), left_gw=f(c_i, c_o) / np.sqrt(c_o), left_gb=f(c_i),
             right_w=f(c_i, c_o) / np.sqrt(c_o), right_b=f(c_i), right_gw=f(c_i, c_o) / np.sqrt(c_o), right_gb=f(c_i),
             center=f(n, n, c_i), gating_w=f(c_o, c_o) / np.sqrt(c_o), gating_b=f(c_o), out_w=f(c_o, c_i) / np.sqrt(c_i),
             out_b=f(c_o))
    D = {k: v.astype(np.float64) for k, v in d.items()}
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))  # noqa: E731
    out = {f"in.{k}": v for k, v in d.items()}
    # transition: rows (i, j), hidden layer relu
    hidden = np.maximum(np.einsum("ijc,hc->ijh", D["x"], D["w1"]) + D["b1"], 0.0)
    out["transition.mid"] = hidden
    out["transition.out"] = np.einsum("ijh,ch->ijc", hidden, D["w2"]) + D["b2"]
    # gated projections, channel-first
    for side in ("left", "right"):
        p = np.einsum("ijc,kc->kij", D["x"], D[side + "_w"]) + D[side + "_b"][:, None, None]
        g = np.einsum("ijc,kc->kij", D["x"], D[side + "_gw"]) + D[side + "_gb"][:, None, None]
        out[f"tm.{side}"] = p * D["mask"][None] * sig(g)
    out["tm.outgoing"] = np.einsum("cik,cjk->cij", out["tm.left"], out["tm.right"])
    out["tm.incoming"] = np.einsum("ckj,cki->cij", out["tm.left"], out["tm.right"])
    gate = np.einsum("ijc,kc->ijk", D["x"], D["gating_w"]) + D["gating_b"]
    proj = np.einsum("ijc,kc->ijk", D["center"], D["out_w"]) + D["out_b"]
    out["tm.gate"], out["tm.out"], out["tm.last"] = gate, proj, proj * sig(gate)
    np.savez(os.path.join(HERE, "pair_stack_tiny.npz"), **out)


if __name__ == "__main__":
    main()
