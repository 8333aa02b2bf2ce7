"""The f16 shadow of a cache that the library keeps itself (hipml_kv_f16_attach / _detach): behind the
reference's own entry points the chunk attention reads the shadow's tiles, and every way this library writes
cache rows keeps the shadow right -- rows converted behind a bulk append, a restore and the chunk front end,
the whole shadow converted again after an append whose position lives in device memory.  Pinned by bit
equality with hipml_attn_chunk_kv_f16 over a copy made by hand (the same kernel over the same tiles) and by
the chunk gate against the CPU oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, N_ROT, THETA, SCALE, ROW, dev, host, report  # noqa: E402
from test_gpu_prefill import chunk_inputs, GATE  # noqa: E402
from test_gpu_kv_f16 import run_chunk_f16  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


class Attached:
    """A device cache pair with a registered shadow, detached again whatever the test does."""

    def __init__(self, kb, vb, stride, rows, dtype=0, n_kv=N_KV):
        self.k, self.v = dev(kb), dev(vb)
        self.copy = attn.kv_f16_alloc(stride, n_kv)
        self.copy.fill_(0xFF)  # f16 NaN wherever nothing converts
        self.args = (dtype, self.k, self.v, self.copy, n_kv, HD, stride, rows)

    def __enter__(self):
        attn.kv_f16_attach(*self.args)
        return self

    def __exit__(self, *exc):
        attn.kv_f16_detach(self.k)


def attend(q, k, v, pos0, tok, stride, splits, dtype=1, gate=None):
    out = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    acc, ml = attn.chunk_scratch(tok, N_HEADS, max(splits, 2))
    acc.fill_(float("nan"))
    ml.fill_(float("nan"))
    if gate is None:
        attn.chunk_attention_q8_split(dev(q), k, v, out, N_HEADS, N_KV, HD, pos0, tok, dtype, stride, acc, ml, splits)
    else:
        attn.chunk_attention_q8_split_gate(dev(q), k, v, dev(gate), out, N_HEADS, N_KV, HD, pos0, tok, dtype, stride,
                                           acc, ml, splits)
    torch.cuda.synchronize()
    return host(out)


@pytest.mark.parametrize("tok,pos0,pad,splits", [(96, 700, 4, 4), (130, 2000, 30, 8), (64, 64, 0, 2), (700, 6000, 8, 13)])
def test_attention_over_an_attached_cache_reads_the_shadow(tok, pos0, pad, splits):
    q, kb, vb, stride = chunk_inputs(0x5AD0_0001 + tok, tok, pos0, pad)
    rows = np.unique(np.clip(np.array([0, 31, 32, 63, 64, tok - 1]), 0, tok - 1)).astype(np.int32)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, rows=rows, n_threads=16)
    with Attached(kb, vb, stride, pos0 + tok) as c:
        got = attend(q, c.k, c.v, pos0, tok, stride, splits)
    ok, _, _ = report(f"attached cache {tok}@{pos0} splits {splits}", want, got[rows], *GATE)
    assert ok and np.isfinite(got).all()
    # the same kernel over the same tiles as the entry point that takes a copy: the same bits
    use = min(splits, attn.chunk_slices(pos0, tok, N_KV))
    by_hand = run_chunk_f16(q, kb, vb, pos0, tok, stride, use)
    assert np.array_equal(got.view(np.uint32), by_hand.view(np.uint32))


def test_rows_attached_late_are_converted_when_the_attention_needs_them():
    # attached with no rows said to be valid: the first attention converts [0, pos0 + tok)
    tok, pos0 = 80, 900
    q, kb, vb, stride = chunk_inputs(0x5AD0_0002, tok, pos0, 3)
    with Attached(kb, vb, stride, 0) as c:
        got = attend(q, c.k, c.v, pos0, tok, stride, 4)
        again = attend(q, c.k, c.v, pos0, tok, stride, 4)  # now nothing is converted
    by_hand = run_chunk_f16(q, kb, vb, pos0, tok, stride, min(4, attn.chunk_slices(pos0, tok, N_KV)))
    assert np.array_equal(got.view(np.uint32), by_hand.view(np.uint32))
    assert np.array_equal(again.view(np.uint32), by_hand.view(np.uint32))


def test_appends_through_the_library_keep_the_shadow_current():
    # prefix in the cache at attach time; the chunk's rows arrive through kv_encode_bulk, then through the
    # fused RoPE + append, each followed by the attention over the attached cache
    tok, pos0, pad = 72, 500, 4
    stride = pos0 + 2 * tok + pad
    r = orc.Rng(0x5AD0_0003)
    q = r.normal_array((2, tok, N_HEADS, HD))
    kf = r.normal_array((stride, N_KV, HD))
    vf = r.normal_array((stride, N_KV, HD))
    kb = orc.quantize(0, kf.transpose(1, 0, 2)).reshape(N_KV, stride, ROW)
    vb = orc.quantize(0, vf.transpose(1, 0, 2)).reshape(N_KV, stride, ROW)
    start = np.full_like(kb, 0xA5)
    start[:, :pos0] = kb[:, :pos0]
    start_v = np.full_like(vb, 0x5A)
    start_v[:, :pos0] = vb[:, :pos0]
    attn.rope_table(THETA, N_ROT, 4096)
    with Attached(start, start_v, stride, pos0) as c:
        # chunk 1: plain bulk append of rows [pos0, pos0 + tok)
        attn.kv_encode_bulk(0, dev(kf[pos0:pos0 + tok]), dev(vf[pos0:pos0 + tok]), c.k, c.v, N_KV, HD, stride, pos0, 0,
                            tok)
        got1 = attend(q[0], c.k, c.v, pos0, tok, stride, 4)
        # chunk 2: RoPE + append in one launch (the K rows change under the rotation: take them from the cache)
        p1 = pos0 + tok
        qd, kd = dev(q[1]), dev(kf[p1:p1 + tok])
        attn.rope_encode_chunk(qd, kd, dev(vf[p1:p1 + tok]), c.k, c.v, N_HEADS, N_KV, HD, N_ROT, THETA, p1, tok, 0,
                               stride)
        got2 = attend(host(qd), c.k, c.v, p1, tok, stride, 4)
        kb2, vb2, q2 = host(c.k), host(c.v), host(qd)
    assert np.array_equal(kb2[:, :p1], kb[:, :p1])
    use = min(4, attn.chunk_slices(pos0, tok, N_KV))
    assert np.array_equal(got1.view(np.uint32), run_chunk_f16(q[0], kb, vb, pos0, tok, stride, use).view(np.uint32))
    use = min(4, attn.chunk_slices(p1, tok, N_KV))
    assert np.array_equal(got2.view(np.uint32), run_chunk_f16(q2, kb2, vb2, p1, tok, stride, use).view(np.uint32))
    want = orc.attn_chunk_kv(q2, kb2, vb2, N_HEADS, N_KV, HD, p1, tok, stride, SCALE, n_threads=16)
    assert report("attached cache after two appends", want, got2, *GATE)[0]


def test_an_append_at_a_device_side_position_makes_the_next_attention_convert_everything():
    tok, pos0 = 64, 300
    q, kb, vb, stride = chunk_inputs(0x5AD0_0004, tok, pos0, 8)
    r = orc.Rng(0x5AD0_0005)
    k_new, v_new = r.normal_array((N_KV, HD), 2.0), r.normal_array((N_KV, HD), 2.0)
    row = 123  # (a row below the shadow's valid rows: a rejected draft's row being overwritten)
    step = torch.tensor([row, row + 1, 0, 0, row, row, row, row], dtype=torch.int32, device="cuda")
    with Attached(kb, vb, stride, pos0 + tok) as c:
        before = attend(q, c.k, c.v, pos0, tok, stride, 4)
        attn.kv_encode(step, 0, dev(k_new), dev(v_new), c.k, c.v, N_KV, HD, stride)
        after = attend(q, c.k, c.v, pos0, tok, stride, 4)
        kb2, vb2 = host(c.k), host(c.v)
    assert not np.array_equal(kb2[:, row], kb[:, row])
    use = min(4, attn.chunk_slices(pos0, tok, N_KV))
    assert np.array_equal(before.view(np.uint32), run_chunk_f16(q, kb, vb, pos0, tok, stride, use).view(np.uint32))
    assert np.array_equal(after.view(np.uint32), run_chunk_f16(q, kb2, vb2, pos0, tok, stride, use).view(np.uint32))
    assert not np.array_equal(before, after)


def test_a_restored_prefix_reaches_the_shadow_and_detach_ends_it():
    tok, pos0, pad = 48, 200, 8
    q, kb, vb, stride = chunk_inputs(0x5AD0_0006, tok, pos0, pad)
    kv = attn.DeepKv(N_HEADS, N_KV, HD, stride)
    kv.attach_f16()
    try:
        kv.restore(dev(kb[:, :pos0].copy()), dev(vb[:, :pos0].copy()))  # hipml_kv_rows_copy into the attached cache
        r = orc.Rng(0x5AD0_0007)
        kf, vf = r.normal_array((tok, N_KV, HD)), r.normal_array((tok, N_KV, HD))
        attn.kv_encode_bulk(0, dev(kf), dev(vf), kv.k, kv.v, N_KV, HD, stride, pos0, 0, tok)
        got = attend(q, kv.k, kv.v, pos0, tok, stride, 4)
        kb2, vb2 = host(kv.k), host(kv.v)
    finally:
        kv.detach_f16()
    use = min(4, attn.chunk_slices(pos0, tok, N_KV))
    assert np.array_equal(got.view(np.uint32), run_chunk_f16(q, kb2, vb2, pos0, tok, stride, use).view(np.uint32))
    with pytest.raises(attn.HipmlError):
        attn.kv_f16_detach(kv.k)  # no shadow any more
    # without a shadow the same call still answers (its own kernels over the cache)
    plain = attend(q, kv.k, kv.v, pos0, tok, stride, 4)
    want = orc.attn_chunk_kv(q, kb2, vb2, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=16)
    assert report("detached cache", want, plain, *GATE)[0]


def test_q4_cache_with_gate():
    tok, pos0, pad = 70, 1500, 10
    stride = pos0 + tok + pad
    r = orc.Rng(0x5AD0_0008)
    q = r.normal_array((tok, N_HEADS, HD))
    gate = r.normal_array((tok, N_HEADS, HD))
    kb = orc.quantize(1, r.normal_array((N_KV, stride, HD))).reshape(N_KV, stride, -1)
    vb = orc.quantize(1, r.normal_array((N_KV, stride, HD))).reshape(N_KV, stride, -1)
    want = orc.q_gate(orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, dtype=1, n_threads=16),
                      gate)
    with Attached(kb, vb, stride, pos0 + tok, dtype=1) as c:
        got = attend(q, c.k, c.v, pos0, tok, stride, 4, dtype=2, gate=gate)
    assert report("attached q4_0 cache with gate", want, got, *GATE)[0]
