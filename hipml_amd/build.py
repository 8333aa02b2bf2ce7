"""Build libhipml_attn.so (HIP kernels + C ABI) for gfx950 with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhipml_attn.so")

ARCH = "gfx950"
# Packed-FP32 instructions are kept out of the generated code on purpose.  The leading scalar arguments of
# a kernel (up to 14 dwords) arrive in registers with the wave instead of through its first memory round
# trip (measured on the decode merge kernel: 0.25-0.3 us per launch).
COMMON = ["--offload-arch=" + ARCH, "-O3", "-fPIC", "-std=c++17", "-Xclang", "-target-feature",
          "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=16",
          "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option", "-Wno-option-ignored"]
# (source, extra flags).  exact.hip must not contract a*b+c: its results are bit-compared.
SOURCES = [
    ("exact.hip", ["-ffp-contract=off"]),
    ("decode.hip", []),
    ("prefill.hip", []),
    ("proj.hip", []),
    ("yardstick.hip", []),
    ("api.cpp", ["-x", "hip"]),
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


# Kernels that keep state in the accumulation registers behind the compiler's back (every use of those
# registers is inside their inline assembly): (source, substring of the mangled kernel name).
HAND_PLACED_ACC = [("prefill.hip", "chunk_f16_t64_kernel")]


def scan_hand_placed_acc(text: list[str], src: str, kernel: str) -> int:
    """The check itself, over the lines of generated assembly: raises if `kernel` is missing, if code outside
    its inline-assembly statements (the compiler's own) names an accumulation register, or if no statement
    does (the scan looks at the wrong text); returns the number of lines inside statements that do."""
    import re
    start = [i for i, l in enumerate(text) if re.match(r"^_Z\w*" + kernel + r"\w*:", l)]
    if not start:
        raise RuntimeError(f"{src}: kernel {kernel} not found in the generated assembly")
    in_asm, n_inside = False, 0
    for l in text[start[0]:]:
        if l.startswith(".Lfunc_end"):
            break
        if "ASMSTART" in l:
            in_asm = True
        elif "ASMEND" in l:
            in_asm = False
        else:
            code = l.split(";")[0]
            acc = re.search(r"\ba\[?\d", code) or "accvgpr" in code
            if acc and in_asm:
                n_inside += 1
            elif acc:
                raise RuntimeError(f"{src}: the compiler uses accumulation registers of its own in {kernel}: "
                                   f"'{code.strip()}'")
    if n_inside == 0:
        raise RuntimeError(f"{src}: no accumulation register found in {kernel}: the check looks at the wrong text")
    return n_inside


def check_hand_placed_acc(cc: str, flags: list[str], src: str, kernel: str) -> None:
    """Fail the build if the compiler itself touches an accumulation register in `kernel` (it parks
    vector registers there under pressure, which would overwrite the kernel's hand-placed state)."""
    cmd = [cc] + COMMON + flags + ["-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", "-"]
    text = subprocess.run(cmd, check=True, capture_output=True, text=True).stdout.split("\n")
    scan_hand_placed_acc(text, src, kernel)


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
        for hsrc, kernel in HAND_PLACED_ACC:
            if hsrc == src:
                check_hand_placed_acc(cc, flags + (extra or []), src, kernel)
    cmd = [cc, "--offload-arch=" + ARCH, "-shared", "-fPIC", "-o", LIB] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
