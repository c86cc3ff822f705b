"""Compile libkutacc.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m kutacc_amd.build          # rebuild kutacc_amd/lib/libkutacc.so
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libkutacc.so")

SOURCES = ["api.cpp", "api_pair_stack.cpp", "api_glue.cpp", "unsupported.cpp", "profiler.cpp", "generic_kernels.hip", "row_kernels.hip", "fused_attention.hip", "fp32_attention.hip", "tiled_attention.hip", "global_attention.hip", "pair_stack.hip", "glue_kernels.hip"]

# -packed-fp32-ops off: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar float code.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument", f"-fmacro-prefix-map={ROOT}/=",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libkutacc.so can only be built with the ROCm toolchain")
    return exe


def build(verbose: bool = False) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    extra = os.environ.get("KUTACC_EXTRA_HIPFLAGS", "").split()  # extra hipcc flags for one-off tuning builds
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(LIB_DIR, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc(), *HIP_FLAGS, *extra, "-x", "hip", "-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c",
               os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        # the host pass does not know the gfx950-only feature flag; that notice is harmless
        lines = [ln for ln in out.splitlines() if "packed-fp32-ops" not in ln]
        if p.returncode != 0:
            failed = True
        if lines and (verbose or p.returncode != 0):
            print(f"--- {src}\n" + "\n".join(lines), flush=True)
    if failed:
        raise RuntimeError("hipcc failed")
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    subprocess.check_call(cmd)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def host_cxx() -> str:
    """ROCm's clang++: the public header uses __bf16, which g++ 11 does not know on x86."""
    for exe in ("/opt/rocm/llvm/bin/clang++", shutil.which("amdclang++"), shutil.which("clang++")):
        if exe and os.path.exists(exe):
            return exe
    raise RuntimeError("no clang++ found for the host-side test caller")


REFERENCE_INCLUDE = "/root/reference/include"


def build_dropin_callers() -> list:
    """tests/cxx/dropin_caller.cpp as a small shared object linked against libkutacc.so, once per public header: this
    repository's (libdropin_caller.so) and, where the reference tree is present, the reference's own include/kutacc.h
    (libdropin_caller_ref.so) -- a caller compiled with the Kunpeng header, run against this library."""
    src = os.path.join(ROOT, "tests", "cxx", "dropin_caller.cpp")
    out_dir = os.path.dirname(src)
    built = []
    variants = [("libdropin_caller.so", os.path.join(ROOT, "include"))]
    if os.path.exists(os.path.join(REFERENCE_INCLUDE, "kutacc.h")):
        variants.append(("libdropin_caller_ref.so", REFERENCE_INCLUDE))
    for name, inc in variants:
        out = os.path.join(out_dir, name)
        cmd = [host_cxx(), "-std=c++17", "-O1", "-fPIC", "-shared", "-Wall", "-D_GLIBCXX_USE_CXX11_ABI=1", "-I", inc, src,
               "-o", out + ".tmp", "-L", LIB_DIR, "-lkutacc", "-Wl,-rpath,$ORIGIN/../../kutacc_amd/lib"]
        subprocess.check_call(cmd)
        os.replace(out + ".tmp", out)
        built.append(out)
    return built


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    print("\n".join(build_dropin_callers()))
