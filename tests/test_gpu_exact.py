"""Bit-exact GPU parity: q8_0 KV append and RoPE against the CPU oracle; gate within
the reference's TIGHT tolerance (crates/hipml-core/src/attn_parity.rs:38,68)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import (N_HEADS, N_KV, HD, N_ROT, THETA, SECTIONS, ROW, dev, host,  # noqa: E402
                      step_buffer, report)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)
    attn.rope_table(THETA, N_ROT, 131072)
    yield


def adversarial_rows(rng, rows, width):
    x = rng.normal_array((rows, width))
    x[0, :32] = 0.0                       # all-zero block: d = 0, id = 0
    x[0, 32:64] = 1e-40                   # subnormal amax: 1/d overflows
    x[0, 64:96] = np.float32(3.0e38)      # near f32 max
    x[0, 96] = 63.5                       # exact-scale block of the known vector
    x[0, 97] = -63.5
    x[1 % rows, :32] = np.float32(0.5) * np.arange(-16, 16, dtype=np.float32)  # ties at .5
    x[1 % rows, 32:64] = np.float32(6.1e-5)  # scale near the f16 normal/subnormal edge
    return x


def test_kv_encode_bulk_bytes_equal_oracle():
    # the headline benchmark shape: 672 tokens x 4 kv heads x 256, appended at position 0 of a
    # cache with stride > live length.
    rows, stride, start = 672, 680, 0
    r = orc.Rng(0xDDDD_EEEE_FFFF_0003)
    k = adversarial_rows(r, rows, N_KV * HD)
    v = adversarial_rows(r, rows, N_KV * HD)[::-1].copy()
    kc = torch.full((N_KV, stride, ROW), 0x11, dtype=torch.uint8, device="cuda")
    vc = torch.full((N_KV, stride, ROW), 0x22, dtype=torch.uint8, device="cuda")
    attn.kv_encode_bulk(0, dev(k), dev(v), kc, vc, N_KV, HD, stride, start, 0, rows)
    torch.cuda.synchronize()
    for src, cache, fill in ((k, kc, 0x11), (v, vc, 0x22)):
        want = orc.quantize(0, src.reshape(rows, N_KV, HD).transpose(1, 0, 2))
        got = host(cache)
        assert np.array_equal(got[:, :rows].ravel(), want)
        assert np.all(got[:, rows:] == fill)  # rows past the chunk untouched


def test_kv_encode_bulk_nonzero_start_and_src0():
    rows, stride, start, src0 = 37, 80, 29, 5
    r = orc.Rng(77)
    k = r.normal_array((src0 + rows, N_KV * HD), 1.5)
    v = r.normal_array((src0 + rows, N_KV * HD), 1.5)
    kc = torch.zeros((N_KV, stride, ROW), dtype=torch.uint8, device="cuda")
    vc = torch.zeros((N_KV, stride, ROW), dtype=torch.uint8, device="cuda")
    attn.kv_encode_bulk(0, dev(k), dev(v), kc, vc, N_KV, HD, stride, start, src0, rows)
    torch.cuda.synchronize()
    want = orc.quantize(0, k[src0:].reshape(rows, N_KV, HD).transpose(1, 0, 2))
    assert np.array_equal(host(kc)[:, start:start + rows].ravel(), want)
    want = orc.quantize(0, v[src0:].reshape(rows, N_KV, HD).transpose(1, 0, 2))
    assert np.array_equal(host(vc)[:, start:start + rows].ravel(), want)
    assert not host(kc)[:, :start].any() and not host(kc)[:, start + rows:].any()


@pytest.mark.parametrize("n_kv,hd,seq,pos", [(4, 64, 8, 3), (4, 256, 64, 63), (1, 32, 4, 0)])
def test_kv_encode_single_token_reads_position_from_step(n_kv, hd, seq, pos):
    # the reference's kv_encode_q8 case: 4 heads x 64 at position 3 of 8 (parity.rs:364-379)
    r = orc.Rng(0xDDDD_EEEE_FFFF_0003)
    k = r.normal_array(n_kv * hd, 1.5)
    v = r.normal_array(n_kv * hd, 1.5)
    row = hd // 32 * 34
    kc = torch.zeros((n_kv, seq, row), dtype=torch.uint8, device="cuda")
    vc = torch.zeros((n_kv, seq, row), dtype=torch.uint8, device="cuda")
    attn.kv_encode(step_buffer(pos, pos + 1), 0, dev(k), dev(v), kc, vc, n_kv, hd, seq)
    torch.cuda.synchronize()
    assert np.array_equal(host(kc)[:, pos].ravel(), orc.quantize(0, k))
    assert np.array_equal(host(vc)[:, pos].ravel(), orc.quantize(0, v))
    mask = np.ones(seq, bool)
    mask[pos] = False
    assert not host(kc)[:, mask].any() and not host(vc)[:, mask].any()


def test_kv_encode_rows_per_slot_positions():
    slots, stride = 5, 40
    positions = [0, 39, 7, 7, 21]
    r = orc.Rng(5150)
    k = r.normal_array((slots, N_KV * HD))
    v = r.normal_array((slots, N_KV * HD))
    slot_bytes = N_KV * stride * ROW
    kc = torch.zeros((slots, N_KV, stride, ROW), dtype=torch.uint8, device="cuda")
    vc = torch.zeros((slots, N_KV, stride, ROW), dtype=torch.uint8, device="cuda")
    pos = torch.tensor([[p, p + 1] for p in positions], dtype=torch.int32, device="cuda")
    attn.kv_encode_rows(0, dev(k), dev(v), kc, vc, N_KV, HD, stride, pos, slot_bytes, slots)
    torch.cuda.synchronize()
    for s, p in enumerate(positions):
        assert np.array_equal(host(kc)[s, :, p].ravel(), orc.quantize(0, k[s]))
        assert np.array_equal(host(vc)[s, :, p].ravel(), orc.quantize(0, v[s]))
    assert np.count_nonzero(host(kc).reshape(slots, N_KV, stride, -1).any(-1)) == slots * N_KV


@pytest.mark.parametrize("pos", [0, 37, 671, 100_000, 131_071])
def test_mrope_bits_equal_oracle(pos):
    r = orc.Rng(0x4444_5555_6666_7777)
    x = r.normal_array((N_HEADS, HD))
    ids = [pos, pos, pos, pos]
    y = torch.empty((N_HEADS, HD), dtype=torch.float32, device="cuda")
    attn.mrope(dev(x), y, N_HEADS, HD, N_ROT, SECTIONS,
               torch.tensor(ids, dtype=torch.int32, device="cuda"), THETA)
    torch.cuda.synchronize()
    want = orc.rope_multi(x, N_HEADS, HD, N_ROT, SECTIONS, ids, THETA)
    assert np.array_equal(host(y).view(np.uint32).ravel(), want.view(np.uint32).ravel())


def test_mrope_sections_pick_their_position_id_and_alias_in_place():
    r = orc.Rng(9)
    x = r.normal_array((N_KV, HD))
    ids = [3, 50, 700, 9000]
    xd = dev(x)
    attn.mrope(xd, xd, N_KV, HD, N_ROT, SECTIONS, torch.tensor(ids, dtype=torch.int32, device="cuda"),
               THETA)
    torch.cuda.synchronize()
    want = orc.rope_multi(x, N_KV, HD, N_ROT, SECTIONS, ids, THETA)
    assert np.array_equal(host(xd).view(np.uint32).ravel(), want.view(np.uint32).ravel())


def test_mrope_reference_case_hd64():
    # attn_parity.rs:36-64: 4 heads x 64, n_rot 64, sections 11/11/10/0, pos 37
    r = orc.Rng(0x4444_5555_6666_7777)
    x = r.normal_array((4, 64))
    y = torch.empty((4, 64), dtype=torch.float32, device="cuda")
    attn.mrope(dev(x), y, 4, 64, 64, SECTIONS, torch.tensor([37] * 4, dtype=torch.int32, device="cuda"),
               THETA)
    torch.cuda.synchronize()
    want = orc.rope_multi(x, 4, 64, 64, SECTIONS, [37] * 4, THETA)
    assert np.array_equal(host(y).view(np.uint32).ravel(), want.view(np.uint32).ravel())


def test_mrope_rows_per_row_positions():
    rows = 7
    positions = [0, 1, 512, 16383, 16384, 99_999, 131_071]
    r = orc.Rng(31)
    x = r.normal_array((rows, N_HEADS, HD))
    pos = torch.tensor([[p, p + 1] for p in positions], dtype=torch.int32, device="cuda")
    y = torch.empty((rows, N_HEADS, HD), dtype=torch.float32, device="cuda")
    attn.mrope_rows(dev(x), y, N_HEADS, HD, N_ROT, SECTIONS, pos, rows, THETA)
    torch.cuda.synchronize()
    for i, p in enumerate(positions):
        want = orc.rope_multi(x[i], N_HEADS, HD, N_ROT, SECTIONS, [p] * 4, THETA)
        assert np.array_equal(host(y)[i].view(np.uint32).ravel(), want.view(np.uint32).ravel())


@pytest.mark.parametrize("pos0,tokens", [(0, 672), (29, 37), (100_000, 2048)])
def test_rope_chunk_bits_equal_oracle(pos0, tokens):
    r = orc.Rng(1234 + pos0)
    q = r.normal_array((tokens, N_HEADS, HD))
    k = r.normal_array((tokens, N_KV, HD))
    qd, kd = dev(q), dev(k)
    attn.rope_chunk(qd, kd, N_HEADS, N_KV, HD, N_ROT, THETA, pos0, tokens)
    torch.cuda.synchronize()
    qg, kg = host(qd), host(kd)
    for t in ([0, 1, tokens // 2, tokens - 1] if tokens > 100 else range(tokens)):
        p = [pos0 + t] * 4
        assert np.array_equal(qg[t].view(np.uint32),
                              orc.rope_multi(q[t], N_HEADS, HD, N_ROT, SECTIONS, p, THETA).view(np.uint32))
        assert np.array_equal(kg[t].view(np.uint32),
                              orc.rope_multi(k[t], N_KV, HD, N_ROT, SECTIONS, p, THETA).view(np.uint32))
    # every token, through a checksum of the whole buffers
    want_q = np.stack([orc.rope_multi(q[t], N_HEADS, HD, N_ROT, SECTIONS, [pos0 + t] * 4, THETA)
                       for t in range(tokens)])
    assert np.array_equal(qg.view(np.uint32), want_q.view(np.uint32))


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("pos0,tokens", [(0, 672), (29, 37), (100_000, 300)])
def test_fused_rope_and_append_has_the_bits_of_the_two_launches(pos0, tokens, dtype):
    # rope_chunk + kv_encode_bulk in one launch: q, k and both caches byte for byte, and the cache
    # bytes against the oracle (rope in f64 trig, then the format's quantizer)
    stride = pos0 + tokens + 5
    row = 272 if dtype == 0 else 144
    r = orc.Rng(4321 + pos0 + dtype)
    q = r.normal_array((tokens, N_HEADS, HD))
    k = r.normal_array((tokens, N_KV, HD))
    v = r.normal_array((tokens, N_KV, HD))
    q1, k1, q2, k2, vd = dev(q), dev(k), dev(q), dev(k), dev(v)
    kc1 = torch.full((N_KV, stride, row), 0x5A, dtype=torch.uint8, device="cuda")
    vc1, kc2, vc2 = kc1.clone(), kc1.clone(), kc1.clone()
    attn.rope_chunk(q1, k1, N_HEADS, N_KV, HD, N_ROT, THETA, pos0, tokens)
    attn.kv_encode_bulk(dtype, k1, vd, kc1, vc1, N_KV, HD, stride, pos0, 0, tokens)
    attn.rope_encode_chunk(q2, k2, vd, kc2, vc2, N_HEADS, N_KV, HD, N_ROT, THETA, pos0, tokens, dtype, stride)
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2)
    assert torch.equal(kc1, kc2) and torch.equal(vc1, vc2)
    kr = np.stack([orc.rope_multi(k[t], N_KV, HD, N_ROT, SECTIONS, [pos0 + t] * 4, THETA).reshape(N_KV, HD)
                   for t in range(tokens)])
    want_k = orc.quantize(dtype, np.ascontiguousarray(kr.transpose(1, 0, 2))).reshape(N_KV, tokens, row)
    want_v = orc.quantize(dtype, np.ascontiguousarray(v.transpose(1, 0, 2))).reshape(N_KV, tokens, row)
    assert np.array_equal(host(kc2)[:, pos0:pos0 + tokens], want_k)
    assert np.array_equal(host(vc2)[:, pos0:pos0 + tokens], want_v)
    assert bool((kc2[:, :pos0] == 0x5A).all()) and bool((kc2[:, pos0 + tokens:] == 0x5A).all())


def test_rope_beyond_table_is_an_error_unless_device_angles_are_allowed():
    # bit-exactness is the contract: a position outside the registered table is refused where the host
    # knows it, gives NaN where it lives in device memory, and is computed on the device (within one
    # f32 ulp of the host definition, a tolerance check) only after the explicit opt-in.
    attn.rope_table(THETA, N_ROT, 64)
    try:
        r = orc.Rng(3)
        x = r.normal_array((N_KV, HD))
        far = torch.tensor([70_000] * 4, dtype=torch.int32, device="cuda")
        y = torch.zeros((N_KV, HD), dtype=torch.float32, device="cuda")
        attn.mrope(dev(x), y, N_KV, HD, N_ROT, SECTIONS, far, THETA)
        torch.cuda.synchronize()
        got = host(y)
        assert np.isnan(got[:, :N_ROT]).all()                  # the rotated channels
        assert np.array_equal(got[:, N_ROT:], x[:, N_ROT:])    # the others pass through
        q = torch.zeros((8, N_HEADS, HD), dtype=torch.float32, device="cuda")
        k = torch.zeros((8, N_KV, HD), dtype=torch.float32, device="cuda")
        with pytest.raises(attn.HipmlError) as e:
            attn.rope_chunk(q, k, N_HEADS, N_KV, HD, N_ROT, THETA, 60, 8)  # positions 60..67, table of 64
        assert e.value.code == -4
        attn.rope_chunk(q, k, N_HEADS, N_KV, HD, N_ROT, THETA, 56, 8)      # 56..63: inside
        attn.rope_allow_device_angles(True)
        attn.mrope(dev(x), y, N_KV, HD, N_ROT, SECTIONS, far, THETA)
        attn.rope_chunk(q, k, N_HEADS, N_KV, HD, N_ROT, THETA, 60, 8)
        torch.cuda.synchronize()
        want = orc.rope_multi(x, N_KV, HD, N_ROT, SECTIONS, [70_000] * 4, THETA)
        ok, _, _ = report("mrope device angles (opt-in)", want, host(y), 1e-6, 1e-5)
        assert ok
    finally:
        attn.rope_allow_device_angles(False)
        attn.rope_table(THETA, N_ROT, 131072)


def test_q_gate_over_the_whole_range_of_gates():
    # the kernels take the exponential and the quotient from the hardware's 1-ulp instructions: held to the
    # same 1e-6 / 1e-5 over gates from where the sigmoid underflows to where it is 1, and exact at the ends
    g = np.concatenate([np.linspace(-104.0, 104.0, 8321), [0.0, -0.0, 88.7, -88.7, 1e-30, -1e-30]]).astype(np.float32)
    q = (np.arange(g.size) % 7 - 3).astype(np.float32) * 0.37 + 0.11
    out = dev(q)
    attn.q_gate(out, dev(g), out)
    torch.cuda.synchronize()
    got = host(out)
    ok, _, _ = report("q_gate, gates -104 .. 104", orc.q_gate(q, g), got, 1e-6, 1e-5)
    assert ok
    ends = np.array([-np.inf, np.inf, -1e4, 1e4], np.float32)
    x = np.array([2.5, 2.5, -3.0, -3.0], np.float32)
    o = dev(x)
    attn.q_gate(o, dev(ends), o)
    torch.cuda.synchronize()
    assert np.array_equal(host(o), np.array([0.0, 2.5, -0.0, -3.0], np.float32))


def test_q_gate_within_tight_tolerance():
    # attn_parity.rs:66-78 (n = 384) and the chunk shape 672 x 24 x 256
    r = orc.Rng(0x5555_6666_7777_8888)
    for n in (384, 672 * N_HEADS * HD, 1003):
        q = r.normal_array(n, 0.5)
        g = r.normal_array(n, 2.0)
        qd = dev(q)
        attn.q_gate(qd, dev(g), qd)  # in place, as the reference calls it
        torch.cuda.synchronize()
        ok, _, _ = report(f"q_gate n={n}", orc.q_gate(q, g), host(qd), 1e-6, 1e-5)
        assert ok
