"""Writes tests/golden/mini_decode.npz: a small, weights-free regression anchor made with the CPU
oracle of THIS repository (self-generated, not a vector held by the reference): the reference's
mini configuration (6 heads on 1 KV head, head_dim 64, 257 cached rows, scale 0.125;
crates/hipml-core/tests/kv_formats.rs:165-195) through q8_0 and q4_0 quantization and the online
decode definition.  Run from the repository root: python tests/golden/make_mini.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as orc  # noqa: E402

H, KV, HD, SEQ, SCALE = 6, 1, 64, 257, 0.125
r = orc.Rng(0x901D)
q = r.normal_array((H, HD))
k = r.normal_array((KV, SEQ, HD))
v = r.normal_array((KV, SEQ, HD))
out = {"q": q, "k": k, "v": v}
for name, dt in (("q8", 0), ("q4", 1)):
    kb, vb = orc.quantize(dt, k), orc.quantize(dt, v)
    out[f"k_{name}"], out[f"v_{name}"] = kb, vb
    out[f"decode_{name}"] = orc.attn_decode_kv(q, kb, vb, H, KV, HD, SEQ, SCALE, dtype=dt)
np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "mini_decode.npz"), **out)
print("wrote mini_decode.npz", {k_: v_.shape for k_, v_ in out.items()})
