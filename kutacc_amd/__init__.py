"""kutacc_amd: MI355X (gfx950) build of the KuTACC fused gated-attention path.

The product is the shared library kutacc_amd/lib/libkutacc.so (C ABI: include/kutacc.h and
include/kutacc_hip.h).  This package holds its sources (csrc/), the build recipe (build.py), a
ctypes binding used by tests and the benchmark (capi.py) and the seeded benchmark inputs
(workloads.py).  There is no CPU fallback: importing capi without a built library raises.
"""
__all__ = ["build", "capi", "workloads"]
