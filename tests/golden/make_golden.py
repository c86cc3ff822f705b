"""Writes tests/golden/gating_attention_tiny.npz: inputs and float64 results of the gated-attention
operator on tiny problems, computed by the numpy float64 twin in oracle/oracle.py (the reference
repository holds no numeric fixture for this operator, and cannot be executed on this machine).

Cases (B=2, S=5, H=2, d=4): with pair bias; without pair bias; one masked key (bias -1e9 at k=3 of
batch 0); one fully masked row (all keys of batch 1 masked).  Seed 20240.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle  # noqa: E402


def main():
    rng = np.random.Generator(np.random.PCG64(20240))
    B, S, H, d = 2, 5, 2, 4
    C = H * d
    f = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    base = dict(x=f(B, S, C), wq=f(C, C) / np.sqrt(C), wk=f(C, C) / np.sqrt(C), wv=f(C, C) / np.sqrt(C),
                wg=f(C, C) / np.sqrt(C), bg=f(C), wo=f(C, C) / np.sqrt(C), bo=f(C), nb=f(H, S, S))
    out = {}
    for name in ("pair_bias", "no_pair_bias", "masked_key", "masked_row"):
        bias = np.zeros((B, S), dtype=np.float32)
        nb = base["nb"]
        if name == "no_pair_bias":
            nb = None
        if name == "masked_key":
            bias[0, 3] = -1e9
        if name == "masked_row":
            bias[1, :] = -1e9
        res, avg = oracle.gating_attention_f64_numpy(base["x"], base["wq"], base["wk"], base["wv"], base["wg"],
                                                     base["bg"], base["wo"], base["bo"], bias, nb, H, return_avg=True)
        out[f"{name}.bias"] = bias
        out[f"{name}.out"] = res
        out[f"{name}.avg"] = avg
    out.update({f"in.{k}": v for k, v in base.items()})
    out["dims"] = np.array([B, S, H, d])
    np.savez(os.path.join(HERE, "gating_attention_tiny.npz"), **out)


if __name__ == "__main__":
    main()
