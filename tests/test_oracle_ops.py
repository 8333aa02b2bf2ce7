"""The oracle's ops against the reference's own unit tests
(crates/hipml-core/tests/{forward_ops,parity_reference,kv_formats}.rs) and
against float64 numpy closed forms."""
import math

import numpy as np
import pytest

Q8, Q4 = 0, 1


def close(a, b, tol):
    return abs(a - b) <= tol * (1.0 + max(abs(a), abs(b)))


def softmax_attention64(q, k, v, scale):
    """q [H,D]; k,v [S,D] for ONE kv head shared by all H; float64."""
    s = (q.astype(np.float64) @ k.astype(np.float64).T) * scale
    s -= s.max(axis=1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=1, keepdims=True)
    return p @ v.astype(np.float64)


# ---- RoPE -------------------------------------------------------------------

def test_rope_multi_full_rotation_is_plain_neox(orc):
    # forward_ops.rs:20-29
    hd = 8
    x = np.array([i * 0.5 - 1.0 for i in range(hd)], dtype=np.float32)
    multi = orc.rope_multi(x, 1, hd, hd, [0] * 4, [3] * 4, 10_000.0)
    neox = orc.rope_neox(x, 1, hd, 3, 10_000.0)
    assert all(close(a, b, 1e-5) for a, b in zip(multi, neox))


def test_rope_multi_rotates_only_first_n_rot(orc):
    # forward_ops.rs:31-46
    hd = 8
    x = np.arange(1, hd + 1, dtype=np.float32)
    y = orc.rope_multi(x, 1, hd, 4, [0] * 4, [5] * 4, 10_000.0)
    assert np.array_equal(y[4:], x[4:])
    assert abs(y[0] - x[0]) > 1e-3 and abs(y[2] - x[2]) > 1e-3
    e0 = x[0] * np.float32(math.cos(5.0)) - x[2] * np.float32(math.sin(5.0))
    assert close(y[0], e0, 1e-5)
    ang = 5.0 * 10_000.0 ** (-2.0 / 4.0)
    e1 = x[1] * np.float32(math.cos(ang)) - x[3] * np.float32(math.sin(ang))
    assert close(y[1], e1, 1e-5)


def test_rope_identity_at_zero_and_norm_preserved(orc):
    # parity_reference.rs:87-107
    heads, dim = 4, 64
    x = orc.Rng(11).normal_array(heads * dim)
    assert np.array_equal(orc.rope_neox(x, heads, dim, 0, 10000.0), x)
    for pos in [1, 37, 4096]:
        y = orc.rope_neox(x, heads, dim, pos, 10000.0).reshape(heads, dim)
        assert np.allclose((x.reshape(heads, dim) ** 2).sum(1), (y ** 2).sum(1), atol=1e-3)


def test_rope_multi_is_textbook_neox_in_float64(orc):
    # qwen35 geometry: head_dim 256, n_rot 64, sections [11,11,10,0], theta 1e7
    heads, hd, n_rot, theta = 3, 256, 64, 1e7
    x = orc.Rng(21).normal_array(heads * hd)
    for pos in [0, 1, 671, 100_000, 131_071]:
        y = orc.rope_multi(x, heads, hd, n_rot, [11, 11, 10, 0], [pos] * 4, theta).reshape(heads, hd)
        xr = x.reshape(heads, hd).astype(np.float64)
        k = np.arange(n_rot // 2)
        ang = pos * theta ** (-2.0 * k / n_rot)
        want = xr.copy()
        want[:, :32] = xr[:, :32] * np.cos(ang) - xr[:, 32:64] * np.sin(ang)
        want[:, 32:64] = xr[:, :32] * np.sin(ang) + xr[:, 32:64] * np.cos(ang)
        assert np.abs(y - want).max() < 2e-6
        assert np.array_equal(y[:, 64:], x.reshape(heads, hd)[:, 64:])


def test_rope_multi_sections_pick_the_position_id(orc):
    # pair k uses section (k % 32): [0,11) temporal, [11,22) height, [22,32) width
    hd, n_rot = 64, 64
    x = orc.Rng(5).normal_array(hd)
    pos = [3, 50, 700, 9000]
    y = orc.rope_multi(x, 1, hd, n_rot, [11, 11, 10, 0], pos, 1e7)
    for k in range(32):
        p = pos[0] if k < 11 else pos[1] if k < 22 else pos[2]
        ang = p * 1e7 ** (-2.0 * k / n_rot)
        want = x[k] * np.float32(math.cos(ang)) - x[k + 32] * np.float32(math.sin(ang))
        assert y[k] == np.float32(want)


# ---- gate -------------------------------------------------------------------

def test_q_gate_closed_form(orc):
    r = orc.Rng(0x5555_6666_7777_8888)
    q, g = r.normal_array(384, 0.5), r.normal_array(384, 2.0)
    y = orc.q_gate(q, g)
    want = q.astype(np.float64) / (1.0 + np.exp(-g.astype(np.float64)))
    assert np.abs(y - want).max() < 1e-6
    assert orc.q_gate(np.float32([2.0]), np.float32([0.0]))[0] == np.float32(1.0)
    assert np.array_equal(orc.sigmoid(np.float32([0.0])), np.float32([0.5]))


# ---- f32 attention ----------------------------------------------------------

def test_attention_hand_computed(orc):
    # parity_reference.rs:222-233
    out = orc.attn_decode_f32([1.0, 0.0], [1.0, 0.0, 0.0, 1.0], [10.0, 0.0, 0.0, 100.0],
                              1, 1, 2, 2, 1.0)
    e = math.e
    assert abs(out[0] - e / (e + 1) * 10) < 1e-5 and abs(out[1] - 100 / (e + 1)) < 1e-5
    # position-major twin, same numbers (one KV head, so the layouts coincide)
    out2 = orc.attn_causal([1.0, 0.0], [1.0, 0.0, 0.0, 1.0], [10.0, 0.0, 0.0, 100.0],
                           1, 1, 2, 2, 1.0)
    assert np.array_equal(out, out2)


def test_attention_uniform_scores_is_mean_of_values(orc):
    # parity_reference.rs:236-254
    heads, kv, dim, seq = 4, 1, 8, 16
    v = orc.Rng(29).normal_array(kv * seq * dim)
    out = orc.attn_decode_f32(np.zeros(heads * dim), np.ones(kv * seq * dim), v, heads, kv, dim,
                              seq, 0.1).reshape(heads, dim)
    assert np.abs(out - v.reshape(seq, dim).mean(0)).max() < 1e-5


def test_attention_routes_query_heads_to_kv_heads(orc):
    # parity_reference.rs:257-276 for the head-major layout ...
    heads, kv, dim, seq = 4, 2, 4, 3
    v = np.concatenate([np.ones(seq * dim), np.full(seq * dim, 7.0)]).astype(np.float32)
    out = orc.attn_decode_f32(np.ones(heads * dim), np.ones(kv * seq * dim), v, heads, kv, dim,
                              seq, 0.1).reshape(heads, dim)
    assert np.allclose(out[:2], 1.0, atol=1e-5) and np.allclose(out[2:], 7.0, atol=1e-5)
    # ... and for the position-major layout of attention.rs
    vpm = np.tile(np.concatenate([np.ones(dim), np.full(dim, 7.0)]), seq).astype(np.float32)
    out = orc.attn_causal(np.ones(heads * dim), np.ones(seq * kv * dim), vpm, heads, kv, dim, seq,
                          0.1).reshape(heads, dim)
    assert np.allclose(out[:2], 1.0, atol=1e-5) and np.allclose(out[2:], 7.0, atol=1e-5)


def test_attention_is_a_convex_combination(orc):
    # parity_reference.rs:279-302
    heads, kv, dim, seq = 2, 1, 6, 32
    r = orc.Rng(31)
    q, k, v = r.normal_array(heads * dim), r.normal_array(seq * dim), r.normal_array(seq * dim)
    out = orc.attn_decode_f32(q, k, v, heads, kv, dim, seq, 0.125).reshape(heads, dim)
    vv = v.reshape(seq, dim)
    assert np.all(out >= vv.min(0) - 1e-5) and np.all(out <= vv.max(0) + 1e-5)


def test_causal_attention_equals_float64_softmax(orc):
    # the shape of the reference's attn_decode_pm_f32 case (attn_parity.rs:112-141)
    heads, kv, dim, seq, scale = 8, 2, 64, 37, 0.125
    r = orc.Rng(0x7777_8888_9999_AAAA)
    q = r.normal_array(heads * dim)
    k = r.normal_array(seq * kv * dim, 0.3)
    v = r.normal_array(seq * kv * dim)
    out = orc.attn_causal(q, k, v, heads, kv, dim, seq, scale).reshape(heads, dim)
    k3, v3, q2 = k.reshape(seq, kv, dim), v.reshape(seq, kv, dim), q.reshape(heads, dim)
    for h in range(heads):
        want = softmax_attention64(q2[h:h + 1], k3[:, h // 4], v3[:, h // 4], scale)[0]
        assert np.abs(out[h] - want).max() < 1e-5
    # a shorter visible prefix ignores the rows past it
    out5 = orc.attn_causal(q, k, v, heads, kv, dim, 5, scale).reshape(heads, dim)
    want = softmax_attention64(q2[:1], k3[:5, 0], v3[:5, 0], scale)[0]
    assert np.abs(out5[0] - want).max() < 1e-5


# ---- quantized decode ---------------------------------------------------------

@pytest.mark.parametrize("dtype", [Q8, Q4])
def test_quantized_attention_equals_attention_over_decoded_values(orc, dtype):
    # kv_formats.rs:165-195
    heads, n_kv, dim, seq = 6, 1, 64, 257
    r = orc.Rng(0xABCD + dtype)
    q = r.normal_array(heads * dim)
    k = r.normal_array(n_kv * seq * dim, 0.3)
    v = r.normal_array(n_kv * seq * dim)
    kb, vb = orc.quantize(dtype, k), orc.quantize(dtype, v)
    quant = orc.attn_decode_kv(q, kb, vb, heads, n_kv, dim, seq, 0.125, dtype)
    dense = orc.attn_decode_f32(q, orc.dequantize(dtype, kb), orc.dequantize(dtype, vb), heads,
                                n_kv, dim, seq, 0.125)
    assert np.abs(quant - dense).max() < 1e-5
    want = softmax_attention64(q.reshape(heads, dim), orc.dequantize(dtype, kb).reshape(seq, dim),
                               orc.dequantize(dtype, vb).reshape(seq, dim), 0.125)
    assert np.abs(quant.reshape(heads, dim) - want).max() < 1e-5


def test_quantized_attention_error_against_f32_cache(orc):
    # kv_formats.rs:198-227
    heads, n_kv, dim, seq = 6, 1, 64, 512
    r = orc.Rng(0xFEED)
    q = r.normal_array(heads * dim)
    k = r.normal_array(n_kv * seq * dim, 0.3)
    v = r.normal_array(n_kv * seq * dim)
    exact = orc.attn_decode_f32(q, k, v, heads, n_kv, dim, seq, 0.125)
    for dtype, bound in [(Q8, 2e-3), (Q4, 3e-2)]:
        got = orc.attn_decode_kv(q, orc.quantize(dtype, k), orc.quantize(dtype, v), heads, n_kv,
                                 dim, seq, 0.125, dtype)
        assert np.abs(exact - got).max() <= bound


def test_decode_kv_gqa_and_stride(orc):
    # 24 q heads on 4 kv heads, cache rows per head (stride) larger than the live length:
    # the result must equal the stride == seq layout the reference uses.
    heads, n_kv, dim, seq, stride = 24, 4, 256, 37, 50
    r = orc.Rng(77)
    q = r.normal_array(heads * dim)
    k = r.normal_array((n_kv, seq, dim))
    v = r.normal_array((n_kv, seq, dim))
    kb = orc.quantize(Q8, k).reshape(n_kv, seq * 272)
    vb = orc.quantize(Q8, v).reshape(n_kv, seq * 272)
    tight = orc.attn_decode_kv(q, kb, vb, heads, n_kv, dim, seq, 0.0625)
    kpad = np.full((n_kv, stride * 272), 0xA5, dtype=np.uint8)
    vpad = np.full((n_kv, stride * 272), 0x5A, dtype=np.uint8)
    kpad[:, :seq * 272], vpad[:, :seq * 272] = kb, vb
    padded = orc.attn_decode_kv(q, kpad, vpad, heads, n_kv, dim, seq, 0.0625, stride=stride)
    assert np.array_equal(tight, padded)
    kd = orc.dequantize(Q8, kb).reshape(n_kv, seq, dim)
    vd = orc.dequantize(Q8, vb).reshape(n_kv, seq, dim)
    for h in [0, 5, 6, 23]:
        want = softmax_attention64(q.reshape(heads, dim)[h:h + 1], kd[h // 6], vd[h // 6], 0.0625)
        assert np.abs(tight.reshape(heads, dim)[h] - want[0]).max() < 1e-5


def test_chunk_expectation_is_row_by_row_causal(orc):
    # the reference's chunk case shape: 37 queries at position 29, cache stride > live length
    # (hipml-cli/src/attn_chunk_parity.rs:117-133)
    heads, n_kv, dim, tok, pos0, pad = 24, 4, 256, 37, 29, 8
    stride = pos0 + tok + pad
    r = orc.Rng(0xC4A0_9876_5432)
    q = r.normal_array((tok, heads, dim))
    k = r.normal_array((stride, n_kv, dim))
    v = r.normal_array((stride, n_kv, dim))
    kb = orc.quantize(Q8, k.transpose(1, 0, 2))
    vb = orc.quantize(Q8, v.transpose(1, 0, 2))
    out = orc.attn_chunk_kv(q, kb, vb, heads, n_kv, dim, pos0, tok, stride, 0.0625, n_threads=4)
    kd = orc.dequantize(Q8, kb).reshape(n_kv, stride, dim)
    vd = orc.dequantize(Q8, vb).reshape(n_kv, stride, dim)
    for t in [0, 17, 36]:
        for h in [0, 11, 23]:
            n = pos0 + t + 1
            want = softmax_attention64(q[t, h:h + 1], kd[h // 6, :n], vd[h // 6, :n], 0.0625)[0]
            assert np.abs(out[t, h] - want).max() < 1e-5
    sub = orc.attn_chunk_kv(q, kb, vb, heads, n_kv, dim, pos0, tok, stride, 0.0625, rows=[36, 0])
    assert np.array_equal(sub[0], out[36]) and np.array_equal(sub[1], out[0])


def test_attn_core_token_is_rope_append_attend_gate(orc):
    # attention.rs:140-161 composed from the separately pinned pieces
    heads, n_kv, dim, n_rot, theta = 24, 4, 256, 64, 1e7
    sections = [11, 11, 10, 0]
    n_ctx = 6
    r = orc.Rng(123)
    kc = np.zeros((n_ctx, n_kv * dim), dtype=np.float32)
    vc = np.zeros((n_ctx, n_kv * dim), dtype=np.float32)
    for pos in range(5):
        q, k, v = r.normal_array(heads * dim), r.normal_array(n_kv * dim), r.normal_array(n_kv * dim)
        g = r.normal_array(heads * dim)
        out, qr, kr = orc.attn_core_token(q, k, v, g, kc, vc, heads, n_kv, dim, n_rot, sections,
                                          pos, theta)
        assert np.array_equal(qr, orc.rope_multi(q, heads, dim, n_rot, sections, [pos] * 4, theta))
        assert np.array_equal(kc[pos], kr) and np.array_equal(vc[pos], v)
        att = orc.attn_causal(qr, kc, vc, heads, n_kv, dim, pos + 1, np.float32(1 / 16))
        assert np.array_equal(out, att * orc.sigmoid(g))


def test_kv_append_writes_one_row(orc):
    # the reference's kv_append_f32 case (attn_parity.rs:80-110)
    n_ctx, width, off = 8, 128, 3
    r = orc.Rng(0x6666_7777_8888_9999)
    kc, vc = r.uniform_array((n_ctx, width)), r.uniform_array((n_ctx, width))
    k, v = r.normal_array(width), r.normal_array(width)
    k0, v0 = kc.copy(), vc.copy()
    orc.kv_append(kc, vc, k, v, off, width)
    k0[off], v0[off] = k, v
    assert np.array_equal(kc, k0) and np.array_equal(vc, v0)


def test_compare_is_abs_or_rel(orc):
    # parity_reference.rs:213-219 and parity.rs:51-53
    ok, _, _ = orc.compare([1.0, 2.0], [1.0, 2.0001], 1e-3, 1e-3)
    assert ok
    ok, max_abs, _ = orc.compare([1.0, 2.0], [1.0, 3.0], 1e-3, 1e-3)
    assert not ok and max_abs > 0.9
    ok, _, _ = orc.compare([1000.0], [1000.5], 1e-3, 1e-3)  # abs fails, rel passes
    assert ok
    ok, _, _ = orc.compare([1e-9], [5e-5], 1e-4, 1e-3)  # rel fails, abs passes
    assert ok


# ---- attention front end: rmsnorm, q|gate split -----------------------------

def test_rmsnorm_unit_rms_and_elementwise_gain(orc):
    # parity_reference.rs:64-85 (n = 513 on purpose, Rng seed 7, normal * 4)
    n = 513
    x = orc.Rng(7).normal_array((n,), 4.0)
    y = orc.rmsnorm(x, np.ones(n, dtype=np.float32), 1e-6)
    rms = math.sqrt(float(np.mean(y.astype(np.float64) ** 2)))
    assert abs(rms - 1.0) < 1e-3
    gain = np.array([(i % 5) + 0.5 for i in range(n)], dtype=np.float32)
    scaled = orc.rmsnorm(x, gain, 1e-6)
    assert np.all(np.abs(scaled - y * gain) < 1e-5)


def test_rmsnorm_closed_forms(orc):
    # constant row c, weight w: y = c / sqrt(c^2 + eps) * w; zero row stays zero
    n, c, eps = 256, np.float32(3.0), np.float32(1e-6)
    w = np.linspace(0.5, 2.0, n).astype(np.float32)
    y = orc.rmsnorm(np.full(n, c, dtype=np.float32), w, float(eps))
    want = (np.float64(c) / np.sqrt(np.float64(c) ** 2 + np.float64(eps))) * w.astype(np.float64)
    assert np.allclose(y, want, rtol=3e-7, atol=0)
    assert np.all(orc.rmsnorm(np.zeros(n, dtype=np.float32), w, 1e-6) == 0.0)
    # float64 definition on random rows, and a sign/eps mistake would show: eps matters at tiny rows
    x = orc.Rng(99).normal_array((n,), 1e-3)
    y = orc.rmsnorm(x, w, 1e-6)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt(np.mean(x64 * x64) + 1e-6) * w
    assert np.allclose(y, want, rtol=2e-6, atol=0)
    assert not np.allclose(y, x64 / np.sqrt(np.mean(x64 * x64)) * w, rtol=1e-3, atol=0)


def test_rmsnorm_tree_order_is_the_same_function(orc):
    # the GPU summation order differs from the index-order sum only in rounding; with squares that
    # sum exactly (small integers) the two are bit-identical, and a power-of-two case has a
    # closed form: x = 1..256 -> sum of squares 5,625,216 exactly
    n = 256
    w = np.ones(n, dtype=np.float32)
    x = np.arange(1, n + 1, dtype=np.float32)
    a = orc.head_rmsnorm(x, w, 1, n, 0.0)
    b = orc.head_rmsnorm(x, w, 1, n, 0.0, tree=True)
    assert np.array_equal(a, b)
    scale = np.float32(1.0) / np.sqrt(np.float32(5625216.0) / np.float32(256.0))
    assert np.array_equal(a, x * scale)
    # random rows: same value to rounding, and per-head independence
    r = orc.Rng(5)
    x = r.normal_array((3 * n,))
    w = r.normal_array((n,))
    a = orc.head_rmsnorm(x, w, 3, n, 1e-6)
    b = orc.head_rmsnorm(x, w, 3, n, 1e-6, tree=True)
    assert np.allclose(a, b, rtol=1e-6, atol=0)
    assert np.array_equal(a[n:2 * n], orc.rmsnorm(x[n:2 * n], w, 1e-6))
    # the tree pairs (t, t + 128) first: a row whose only rounding sits in that pairing tells the
    # orders apart (1 + 2^-24 twice: index order loses both, the tree adds them together first)
    x = np.zeros(n, dtype=np.float32)
    x[0] = 1.0
    x[1] = x[129] = np.float32(2.0 ** -12)      # squares 2^-24 each
    ones = np.ones(n, dtype=np.float32)
    seq = orc.head_rmsnorm(x, ones, 1, n, 0.0)[0]
    tree = orc.head_rmsnorm(x, ones, 1, n, 0.0, tree=True)[0]
    s_seq = np.float32(1.0)                       # (1 + 2^-24) rounds to 1, twice
    s_tree = np.float32(1.0) + np.float32(2.0 ** -23)   # 2^-24 + 2^-24 joined before meeting 1
    assert seq == np.float32(1.0) / np.sqrt(s_seq / np.float32(n))
    assert tree == np.float32(1.0) / np.sqrt(s_tree / np.float32(n))


def test_qg_split_layout(orc):
    # ops.rs:315-330: head h of the joint row is [q_h | gate_h]
    nh, hd = 3, 4
    qg = np.arange(nh * 2 * hd, dtype=np.float32)
    q, g = orc.qg_split(qg, nh, hd)
    assert np.array_equal(q, [0, 1, 2, 3, 8, 9, 10, 11, 16, 17, 18, 19])
    assert np.array_equal(g, [4, 5, 6, 7, 12, 13, 14, 15, 20, 21, 22, 23])


# ---- Q8_0 weight matrices (the output projection after the attention core) ----------------------

def test_q8_0_weight_block_hand_vector(orc):
    # crates/hipml-core/tests/quant_reference.rs:144-156: d = 0.5 (0x3800), q_i = i + 1
    b = np.zeros(34, dtype=np.uint8)
    b[0], b[1] = 0x00, 0x38
    b[2:] = np.arange(1, 33, dtype=np.uint8)
    assert np.array_equal(orc.dequant_q8_0(b), 0.5 * np.arange(1, 33, dtype=np.float32))
    # negative payloads are two's-complement int8
    b[2] = 0x80
    assert orc.dequant_q8_0(b)[0] == -64.0


def test_random_q8_0_bytes_layout(orc):
    # quant.rs:785-796,846-854: the byte stream is next_u64() little-endian, five draws per block
    # (8+8+8+8 and a 2-byte tail), scale bytes overwritten with 0x1400 = 2^-10
    r, r2 = orc.Rng(0x4B51_0005), orc.Rng(0x4B51_0005)
    w = orc.random_q8_0_bytes(r, 3).reshape(3, 34)
    for blk in range(3):
        draws = [r2.next_u64() for _ in range(5)]
        want = b"".join(int(d).to_bytes(8, "little") for d in draws)[:34]
        assert bytes(w[blk][2:]) == want[2:]
        assert w[blk][0] == 0x00 and w[blk][1] == 0x14
    assert orc.f16_to_f32(0x1400) == np.float32(2.0 ** -10)


def test_gemv_and_gemm_q8_0_against_float64(orc):
    # the reference's case shapes: gemv 64x512 (quant_parity.rs:125-133), gemm 64x512 t=4
    # (prefill_parity.rs:209-219); the definition is a plain dot product over dequantized weights
    r = orc.Rng(0x4B51_0005)
    m, k = 64, 512
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array(k)
    blocks = w.reshape(m, k // 32, 34)
    d = blocks[:, :, :2].copy().view(np.float16).astype(np.float64)
    dense = (d * blocks[:, :, 2:].view(np.int8).astype(np.float64)).reshape(m, k)
    y = orc.gemv_q8_0(w, x, m, k)
    assert np.max(np.abs(y - dense @ x.astype(np.float64))) < 1e-4
    # an integer case is exact in f32 whatever the order: d = 1, x = small integers
    wi = w.copy().reshape(-1, 34)
    wi[:, 0], wi[:, 1] = 0x00, 0x3C
    xi = np.round(x * 3).astype(np.float32)
    dense_i = wi[:, 2:].view(np.int8).astype(np.float64).reshape(m, k)
    assert np.array_equal(orc.gemv_q8_0(wi.ravel(), xi, m, k), (dense_i @ xi).astype(np.float32))
    # gemm row t equals the gemv of x[t] (ops.rs:136-176 keeps the same j-ascending sum) ...
    r = orc.Rng(0x9F11_0003)
    w = orc.random_q8_0_bytes(r, m * k // 32)
    xs = r.normal_array((4, k))
    y = orc.gemm_q8_0(w, xs, 4, m, k)
    for t in range(4):
        assert np.array_equal(y[t], orc.gemv_q8_0(w, xs[t], m, k))
    # ... whatever the thread count
    assert np.array_equal(y, orc.gemm_q8_0(w, xs, 4, m, k, n_threads=4))
