"""Where a decode launch spends its time: phase stamps from an instrumented build of the decode kernel.

    python -m hipml_amd.decode_phases --build      # here (no GPU needed): libhipml_attn_stamps.so beside the library
    python -m hipml_amd.decode_phases [--seq 32768] [--launches 48]     # on the MI355X box

The instrumented library is the shipped source compiled with -DHIPML_DECODE_STAMPS: wave 0 of every workgroup of
decode_q8_kernel keeps the 100 MHz counter at twelve points in scalar registers and writes them when it is done.
Printed: per point, minimum / mean / maximum over workgroups and launches, in microseconds since the first
workgroup of the same launch started; for the split + merge form and for the one-launch form.
(Reading the counter is a scalar memory operation: a stamp returns only when the scalar loads before it have, so
the third point also waits for the live lengths, which the shipped kernel first needs after the Q conversion, and
an instrumented launch runs about 0.3 us longer than the shipped one.)"""
from __future__ import annotations

import argparse
import ctypes as C
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
STAMPS_LIB = os.path.join(HERE, "libhipml_attn_stamps.so")
POINTS = ["first instruction", "work item found", "first requests issued (Q, K(0)) and live lengths read", "Q operands in registers",
          "K rows of the first tile in LDS", "V rows of the last tile in LDS", "last tile done",
          "partial stored (issue)", "one launch: ticket of the group back", "one launch: group folded and stored",
          "one launch: ticket of the KV head back", "all stores acknowledged (end)"]


def build() -> str:
    from hipml_amd import build as b
    b.build_library()  # the other objects, as shipped
    cc = b.hipcc()
    obj = os.path.join(b.CSRC, "decode_stamps.o")
    subprocess.run([cc] + b.COMMON + ["-DHIPML_DECODE_STAMPS", "-c", os.path.join(b.CSRC, "decode.hip"), "-o", obj],
                   check=True)
    objs = [obj if src == "decode.hip" else os.path.join(b.CSRC, os.path.splitext(src)[0] + ".o")
            for src, _ in b.SOURCES]
    subprocess.run([cc, "--offload-arch=" + b.ARCH, "-shared", "-fPIC", "-o", STAMPS_LIB] + objs, check=True)
    return STAMPS_LIB


def run(seq: int, launches: int) -> None:
    import numpy as np
    import torch
    from hipml_amd import attn
    assert attn._lib is None, "the library is already loaded"
    attn.LIB_PATH = STAMPS_LIB  # the instrumented build instead of the shipped one
    attn.init(0)
    H, KV, HD, layers = 24, 4, 256, 16
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1)
    caches = []
    for _ in range(layers):
        k = torch.empty((KV, seq, 272), dtype=torch.uint8, device="cuda")
        v = torch.empty_like(k)
        for s0 in range(0, seq, 8192):
            n = min(8192, seq - s0)
            attn.kv_encode_bulk(0, torch.randn((n, KV, HD), device="cuda", generator=gen),
                                torch.randn((n, KV, HD), device="cuda", generator=gen), k, v, KV, HD, seq, s0, 0, n)
        caches.append((k, v))
    q = torch.randn((H, HD), device="cuda", generator=gen)
    out = torch.empty((H, HD), device="cuda")
    splits = attn.decode_splits(seq, KV)
    acc = torch.empty((H, splits, HD), device="cuda")
    ml = torch.empty((H, splits, 2), device="cuda")
    step = torch.tensor([seq - 1, seq, 0, 0, seq - 1, seq - 1, seq - 1, seq - 1], dtype=torch.int32, device="cuda")
    wgs = KV * min(splits, 256 // KV)
    host = (C.c_ulonglong * (wgs * 12))()
    read = attn.lib().hipml_dbg_decode_stamps
    read.argtypes, read.restype = [C.c_void_p, C.c_size_t], C.c_int
    for mode, name in ((0, "split + merge launches"), (1, "one launch (hipml_attn_decode_one_launch(1))")):
        attn.decode_one_launch(mode)
        rows = []
        for i in range(launches + 8):
            k, v = caches[i % layers]
            for j in range(4):  # a few launches back to back, as the benchmark issues them; the last one is read
                kk, vv = caches[(i + j) % layers]
                attn.attn_decode_kv(step, 0, q, kk, vv, acc, ml, out, H, KV, HD, seq, 0.0625, splits)
            torch.cuda.synchronize()
            assert read(host, wgs * 12) == 0
            if i >= 8:
                t = np.frombuffer(host, dtype=np.uint64).reshape(wgs, 12).astype(np.float64)
                rows.append(np.where(t > 0, (t - t[:, 0].min()) / 100.0, np.nan))
        t = np.stack(rows)  # [launch][workgroup][point]
        print(f"\n== decode @ {seq}, {wgs} workgroups, {name}: microseconds since the launch's first workgroup started")
        print(f"   {'point':44s} {'min':>8s} {'mean':>8s} {'max':>8s}")
        for p, label in enumerate(POINTS):
            x = t[:, :, p]
            if np.isnan(x).all():
                continue
            print(f"   {label:44s} {np.nanmin(x):8.2f} {np.nanmean(x):8.2f} {np.nanmax(x):8.2f}")
        print(f"   {'end of the last workgroup, mean over launches':44s} {'':8s} {np.nanmean(np.nanmax(t[:, :, 11], axis=1)):8.2f}")
    attn.decode_one_launch(0)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--build", action="store_true")
    ap.add_argument("--seq", type=int, default=32768)
    ap.add_argument("--launches", type=int, default=48)
    a = ap.parse_args()
    if a.build:
        print(build())
        sys.exit(0)
    if not os.path.exists(STAMPS_LIB):
        sys.exit(f"{STAMPS_LIB} is missing: run `python -m hipml_amd.decode_phases --build` first")
    run(a.seq, a.launches)
