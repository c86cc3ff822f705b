"""Developer measurements on the development build of the library (python -m kutacc_amd.build --dev).

    python -m kutacc_amd.devtools timeline [config]   phases of one batch row of the head kernel, per wave, in shader clocks
    python -m kutacc_amd.devtools loop [key_tiles]    the attention tile loop by itself: clocks per key tile at one, two and
                                                      three waves per SIMD, with and without pair bias

Both need a GPU and fail if libkutacc_dev.so has not been built.  The probes write clock64() at fixed points of
persistent_head_kernel / fused_head_kernel (wave leaders of one workgroup in 256); the loop probe runs
attend_block_l2 on operands that never leave the CU.
"""
from __future__ import annotations

import ctypes
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _dev_capi():
    from kutacc_amd import build, capi
    if not os.path.exists(build.DEV_LIB_PATH):
        raise RuntimeError("kutacc_amd/lib/libkutacc_dev.so is missing: run `python -m kutacc_amd.build --dev`")
    capi.LIB_PATH = build.DEV_LIB_PATH
    return capi


def timeline(config: int = 3, calls: int = 300) -> None:
    capi = _dev_capi()
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import torch
    import helpers
    from kutacc_amd.workloads import make_workload

    w = make_workload(config)
    op, ten, scratch = helpers.make_op(w, device="cuda:0")
    for _ in range(calls):
        op.run()
    torch.cuda.synchronize()
    assert not capi.error_flag()
    n = 8 * 16 * 12
    buf = (ctypes.c_ulonglong * n)()
    fn = capi.lib().kutacc_debug_timeline
    fn.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.c_int]
    assert fn(buf, n) == 0
    a = np.array(buf[:], dtype=np.int64).reshape(8, 16, 12)[0]
    print(f"config {w.config} (B={w.B} S={w.S} C={w.C} H={w.H}), path {capi.last_path()}: one workgroup, third batch row of its "
          f"sequence, shader clocks")
    live = [wv for wv in range(16) if a[wv, 0] != 0 and a[wv, 5] != 0]
    if not live:
        print("no probe data: this configuration does not run the persistent head kernel")
        return
    base = min(a[wv, 0] for wv in live)
    print("wave  row start   load+stage  projections  barriers+K/V  attention  epilogue   row end")
    for wv in live:
        t = a[wv]
        print(f"{wv:4d}  {t[0] - base:9d}   {t[1] - t[0]:10d}  {t[2] - t[1]:11d}  {t[3] - t[2]:12d}  {t[4] - t[3]:9d}  "
              f"{t[5] - t[4]:8d}  {t[5] - base:8d}")
    whole = max(a[wv, 11] for wv in live) - min(a[wv, 7] for wv in live)
    rows = (w.B * w.H + 255) // 256
    print(f"whole kernel {whole} clocks for {rows} batch rows per workgroup = {whole / rows:.0f} clocks per row "
          f"(weights staged after {int(a[live[0], 8] - a[live[0], 7])} clocks)")
    nb = (w.S + 31) // 32
    nt = (nb + 1) & ~1
    att = [a[wv, 4] - a[wv, 3] for wv in live]
    print(f"attention of the last wave to finish: {max(att)} clocks for {len(live) // 4 * nt} key tiles per SIMD = "
          f"{max(att) / (len(live) // 4 * nt):.0f} clocks per key tile per SIMD (other waves' projections included)")


def loop(nt: int = 12, reps: int = 200) -> None:
    capi = _dev_capi()
    import torch  # noqa: F401  (one HIP runtime per process: torch's comes first)
    fn = capi.lib().kutacc_debug_attention_loop
    fn.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    print(f"attend_block_l2 alone, {nt} key tiles x {reps} repetitions per wave, one workgroup per CU")
    print("pair bias  waves/SIMD  kernel us  clocks/tile/SIMD  clocks/tile of wave 0  shader clock GHz  MFMA pipe clocks/tile")
    for pair_bias in (1, 0):
        mfma = 224 if pair_bias else 160  # 4 + 2 (selectors) MFMAs of 32 clocks and 2 of 16
        for waves in (4, 8, 12):
            res = (ctypes.c_double * 3)()
            rc = fn(nt, reps, waves, pair_bias, res)
            assert rc == 0, rc
            tiles = reps * nt * (waves // 4)
            print(f"{pair_bias:9d}  {waves // 4:10d}  {res[0]:9.1f}  {res[1] / tiles:16.0f}  {res[2] / (reps * nt):21.0f}  "
                  f"{res[1] / (res[0] * 1e3):16.2f}  {mfma:21d}")


if __name__ == "__main__":
    what = sys.argv[1] if len(sys.argv) > 1 else ""
    arg = int(sys.argv[2]) if len(sys.argv) > 2 else None
    if what == "timeline":
        timeline(arg if arg is not None else 3)
    elif what == "loop":
        loop(arg if arg is not None else 12)
    else:
        sys.exit(__doc__)
