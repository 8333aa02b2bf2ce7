"""Chunk prefill over the f16 copy of a cache (hipml_kv_f16_rows + hipml_attn_chunk_kv_f16).

The copy has no counterpart in the reference; what pins it is its definition: every value is
f16(d * q) of the cache entry (d * q is exact in f32, so that is one rounding), K rows in place and V
transposed in the operand order the header states.  The attention over it is held to the same oracle
and the same gate (2e-3 / 1e-2) as the attention over the cache itself."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, SCALE, dev, host, report  # noqa: E402
from test_gpu_prefill import chunk_inputs, run_chunk, GATE  # noqa: E402

K_TILE_BYTES, VT_TILE_BYTES, K_ROW, VT_ROW = 33_792, 36_864, 528, 144


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def expected_f16(dtype, cache_bytes, n_kv, stride):
    # f16(d * q): dequantize gives d * q exactly in f32
    return orc.dequantize(dtype, cache_bytes.reshape(-1)).reshape(n_kv, stride, HD).astype(np.float16)


def split_copy(copy, n_kv, stride):
    tiles = (stride + 63) // 64
    k16 = copy[: n_kv * tiles * K_TILE_BYTES].reshape(n_kv, tiles, 64, K_ROW)[..., :512].copy().view(np.float16)
    vt = copy[n_kv * tiles * K_TILE_BYTES:].reshape(n_kv, tiles, HD, VT_ROW)[..., :128].copy().view(np.float16)
    return k16, vt, tiles  # [n_kv][tile][64 keys][256], [n_kv][tile][256 d][64 positions]


def key_at_position():
    # position g*8 + j of a 16-key group holds key (j/4)*8 + g*4 + j%4 of the group
    p = np.arange(64)
    grp, g, j = p // 16, (p % 16) // 8, p % 8
    return grp * 16 + (j // 4) * 8 + g * 4 + j % 4


@pytest.mark.parametrize("dtype", [0, 1])
def test_copy_holds_f16_of_every_cache_value_and_completes_partial_tiles(dtype):
    n_kv, stride, live = 2, 200, 150
    r = orc.Rng(0xF16C + dtype)
    kf = r.normal_array((n_kv, stride, HD), 0.7)
    vf = r.normal_array((n_kv, stride, HD), 1.3)
    kb, vb = orc.quantize(dtype, kf), orc.quantize(dtype, vf)
    want_k, want_v = expected_f16(dtype, kb, n_kv, stride), expected_f16(dtype, vb, n_kv, stride)
    kd, vd = dev(kb), dev(vb)
    copy = attn.kv_f16_alloc(stride, n_kv)
    assert copy.numel() == n_kv * 4 * (K_TILE_BYTES + VT_TILE_BYTES)
    copy.fill_(0xEE)
    perm = key_at_position()

    def check(upto):
        torch.cuda.synchronize()
        k16, vt, tiles = split_copy(host(copy), n_kv, stride)
        for t in range((upto + 63) // 64):
            keys = np.minimum(t * 64 + np.arange(64), upto - 1)  # rows past the live ones repeat the last
            assert np.array_equal(k16[:, t].view(np.uint16), want_k[:, keys].view(np.uint16)), (dtype, upto, t)
            got_v = vt[:, t]  # [n_kv][d][position]
            exp_v = want_v[:, keys[perm]].transpose(0, 2, 1)
            assert np.array_equal(got_v.view(np.uint16), exp_v.view(np.uint16)), (dtype, upto, t)

    attn.kv_f16_rows(dtype, kd, vd, copy, n_kv, HD, stride, 0, 100)
    check(100)
    attn.kv_f16_rows(dtype, kd, vd, copy, n_kv, HD, stride, 100, live - 100)  # completes tile 1, adds tile 2
    check(live)
    attn.kv_f16_rows(dtype, kd, vd, copy, n_kv, HD, stride, live, 0)  # nothing to do
    check(live)


def run_chunk_f16(q, kb, vb, pos0, tok, stride, splits, gate=None, want16=False, dtype=0):
    copy = attn.kv_f16_alloc(stride, N_KV)
    copy.fill_(0xFF)  # f16 NaN wherever the conversion does not write
    attn.kv_f16_rows(dtype, dev(kb), dev(vb), copy, N_KV, HD, stride, 0, pos0 + tok)
    out = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    out16 = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float16, device="cuda") if want16 else None
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, N_HEADS, splits)
        acc.fill_(float("nan"))
        ml.fill_(float("nan"))
    attn.chunk_attention_kv_f16(dev(q), copy, None if gate is None else dev(gate), out, out16, N_HEADS, N_KV, HD,
                                pos0, tok, stride, acc, ml, splits)
    torch.cuda.synchronize()
    return host(out16).astype(np.float32) if want16 else host(out)


@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("tok,pos0,pad", [(37, 29, 0), (37, 29, 8), (1, 0, 0), (33, 0, 3), (64, 1000, 24),
                                          (130, 63, 1), (96, 64, 0)])
def test_chunk_over_the_copy_against_the_oracle(tok, pos0, pad, splits):
    q, kb, vb, stride = chunk_inputs(0xC4A0_9876_5432, tok, pos0, pad)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=8)
    got = run_chunk_f16(q, kb, vb, pos0, tok, stride, splits)
    ok, _, _ = report(f"chunk over f16 copy {tok}@{pos0} pad {pad} splits {splits}", want, got, *GATE)
    assert ok
    assert np.isfinite(got).all()


def test_unsplit_chunk_over_the_copy_equals_the_chunk_over_the_cache():
    # same operands, same order of the keys, no slices: the same bits
    tok, pos0 = 100, 300
    q, kb, vb, stride = chunk_inputs(0xF16_0001, tok, pos0, 5)
    a = run_chunk(q, kb, vb, pos0, tok, stride, 1)
    b = run_chunk_f16(q, kb, vb, pos0, tok, stride, 1)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("splits", [1, 3])
def test_prefill_672_at_0_over_the_copy_with_gate_and_f16_rows(splits):
    tok, pos0 = 672, 0
    q, kb, vb, stride = chunk_inputs(0x5EED_0002, tok, pos0, 8)
    gate = orc.Rng(0x6A7E).normal_array((tok, N_HEADS, HD))
    want = orc.q_gate(orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=16), gate)
    got = run_chunk_f16(q, kb, vb, pos0, tok, stride, splits, gate=gate)
    ok, _, _ = report(f"prefill 672@0 over f16 copy, gate, splits {splits}", want, got, *GATE)
    assert ok
    got16 = run_chunk_f16(q, kb, vb, pos0, tok, stride, splits, gate=gate, want16=True)
    assert np.array_equal(got16.astype(np.float16).view(np.uint16), got.astype(np.float16).view(np.uint16))


def test_deep_prefix_sampled_rows_and_q4_cache():
    tok, pos0, pad = 256, 20_000, 16
    stride = pos0 + tok + pad
    r = orc.Rng(0xDEE9_F16)
    q = r.normal_array((tok, N_HEADS, HD))
    kf = r.normal_array((N_KV, stride, HD))
    vf = r.normal_array((N_KV, stride, HD))
    rows = np.array([0, 31, 32, 100, 255], dtype=np.int32)
    for dtype in (0, 1):
        kb = orc.quantize(dtype, kf).reshape(N_KV, stride, -1)
        vb = orc.quantize(dtype, vf).reshape(N_KV, stride, -1)
        splits = attn.chunk_splits(pos0, tok, N_KV)
        assert splits >= 2
        want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, dtype=dtype, rows=rows,
                                 n_threads=16)
        got = run_chunk_f16(q, kb, vb, pos0, tok, stride, splits, dtype=dtype)
        ok, _, _ = report(f"chunk over f16 copy 256@20000, cache dtype {dtype}, splits {splits}", want, got[rows],
                          *GATE)
        assert ok


def test_argument_errors_are_reported():
    copy = attn.kv_f16_alloc(128, N_KV)
    kb = torch.zeros(N_KV * 128 * 272, dtype=torch.uint8, device="cuda")
    with pytest.raises(attn.HipmlError):
        attn.kv_f16_rows(0, kb, kb, copy, N_KV, HD, 128, 100, 29)  # rows past the cache
    with pytest.raises(attn.HipmlError):
        attn.kv_f16_rows(3, kb, kb, copy, N_KV, HD, 128, 0, 10)  # unknown format
    assert attn.kv_f16_bytes(0, 4) == 0


def test_cache_owner_keeps_its_copy_current_through_append_and_restore():
    # DeepKv with a copy: a prefix restored into it and a chunk appended after it give the attention over the
    # copy the same rows as the attention over the cache
    tok, pos0, pad = 48, 200, 8
    q, kb, vb, stride = chunk_inputs(0xF16_0002, tok, pos0, pad)
    kv = attn.DeepKv(N_HEADS, N_KV, HD, stride)
    kv.enable_f16_copy()
    kv.restore(dev(kb[:, :pos0].copy()), dev(vb[:, :pos0].copy()))  # the prefix, as a snapshot would bring it
    kv.k[:, pos0:pos0 + tok] = dev(kb[:, pos0:pos0 + tok].copy())  # the chunk's rows, as an append leaves them
    kv.v[:, pos0:pos0 + tok] = dev(vb[:, pos0:pos0 + tok].copy())
    kv.sync_f16(pos0, tok)
    out = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_kv_f16(dev(q), kv.f16, None, out, None, N_HEADS, N_KV, HD, pos0, tok, stride, None, None, 1)
    torch.cuda.synchronize()
    want = run_chunk(q, kb, vb, pos0, tok, stride, 1)
    assert np.array_equal(host(out).view(np.uint32), want.view(np.uint32))
