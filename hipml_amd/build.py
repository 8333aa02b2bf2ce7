"""Build libhipml_attn.so (HIP kernels + C ABI) for gfx950 with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhipml_attn.so")

ARCH = "gfx950"
# Packed-FP32 instructions are kept out of the generated code on purpose.
COMMON = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature",
          "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
          "-Wno-unknown-warning-option", "-Wno-option-ignored"]
# (source, extra flags).  exact.hip must not contract a*b+c: its results are bit-compared.
SOURCES = [
    ("exact.hip", ["-ffp-contract=off"]),
    ("decode.hip", []),
    ("prefill.hip", []),
    ("proj.hip", []),
    ("api.cpp", ["-x", "hip"]),
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build_library(verbose: bool = False, extra: list[str] | None = None) -> str:
    """Compile every translation unit and link the shared library; returns its path."""
    cc = hipcc()
    objs = []
    for src, flags in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [cc] + COMMON + flags + (extra or []) + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
        objs.append(obj)
    cmd = [cc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
