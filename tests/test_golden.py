"""The oracle against the committed fixtures: tests/golden/reference_vectors.json (known answers
the reference's own tests hold, transcribed by hand) and tests/golden/mini_decode.npz (a
self-generated regression anchor, made by tests/golden/make_mini.py)."""
import json
import math
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
Q8, Q4 = 0, 1


def vectors():
    with open(os.path.join(GOLDEN, "reference_vectors.json")) as f:
        return json.load(f)


def test_format_constants_and_f16_vectors(orc):
    v = vectors()
    b = v["block_bytes"]
    assert orc.block_bytes(Q8) == b["q8"] and orc.block_bytes(Q4) == b["q4"]
    assert orc.token_bytes(Q8, 4, 256, 16) == b["token_bytes_q8_4kv_256_16layers"]
    assert orc.token_bytes(Q4, 4, 256, 16) == b["token_bytes_q4_4kv_256_16layers"]
    f = v["f16_round_trip_patterns"]
    for h in f["patterns"]:
        assert orc.f32_to_f16(orc.f16_to_f32(h)) == h
    assert orc.f16_to_f32(orc.f32_to_f16(0.1)) == np.float32(f["f16_of_0p1_as_f32"])
    assert orc.f32_to_f16(np.inf) == f["f16_of_inf"]
    assert orc.f32_to_f16(-0.0) == f["f16_of_minus_zero"]


def test_q8_known_block_bytes(orc):
    k = vectors()["q8_known_block"]
    xs = np.full(32, k["input"]["rest"], dtype=np.float32)
    xs[0], xs[1] = k["input"]["index0"], k["input"]["index1"]
    b = orc.quantize(Q8, xs)
    assert list(b[:2]) == k["scale_bytes"]
    assert np.int8(b[2]) == k["q0"] and np.int8(b[3]) == k["q1"]
    assert np.array_equal(orc.dequantize(Q8, b), xs)


def test_attention_closed_form(orc):
    # one head, head_dim 2, two rows: q = (1, 0), k rows (1, 0) and (0, 0) at scale 1 give weights
    # e/(e+1) and 1/(e+1) on v rows (10, 0) and (0, 100)
    e = math.e
    q = np.float32([1, 0])
    k = np.float32([[1, 0], [0, 0]])
    v = np.float32([[10, 0], [0, 100]])
    out = orc.attn_causal(q, k, v, 1, 1, 2, 2, 1.0)
    assert abs(out[0] - 10 * e / (e + 1)) < 1e-5 and abs(out[1] - 100 / (e + 1)) < 1e-5


def test_mini_anchor_reproduces(orc):
    z = np.load(os.path.join(GOLDEN, "mini_decode.npz"))
    cfg = vectors()["online_vs_two_pass"]
    H, KV, HD, SEQ, SCALE = cfg["heads"], cfg["n_kv"], cfg["head_dim"], cfg["seq"], cfg["scale"]
    for name, dt in (("q8", Q8), ("q4", Q4)):
        kb, vb = orc.quantize(dt, z["k"]), orc.quantize(dt, z["v"])
        assert np.array_equal(kb, z[f"k_{name}"]) and np.array_equal(vb, z[f"v_{name}"])
        got = orc.attn_decode_kv(z["q"], kb, vb, H, KV, HD, SEQ, SCALE, dtype=dt)
        assert np.array_equal(got, z[f"decode_{name}"])
        # and the anchor itself obeys the reference's bound against the unquantized definition
        two_pass = orc.attn_causal(z["q"], z["k"].reshape(SEQ, KV * HD), z["v"].reshape(SEQ, KV * HD), H, KV, HD,
                                   SEQ, SCALE)
        tol = vectors()["q8_vs_f32_cache"]["q8_tolerance" if dt == Q8 else "q4_tolerance"]
        assert np.max(np.abs(got - two_pass)) <= tol * 2.5  # 257 rows of N(0,1), not the 512 of that test
