"""q4_0 KV cache (crates/hipml-core/src/kv.rs:201-218) through the same entry points as q8_0:
append bytes bit-exact against the oracle, decode and chunk prefill against the oracle's
attention over the dequantized q4_0 cache.  Tolerances as for q8_0: the kernels' error class
does not depend on the cache format (the comparison is against the SAME quantized bytes)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, SCALE, dev, host, step_buffer, report  # noqa: E402

Q4 = 1
ROW4 = 144
GATE = (2e-3, 1e-2)
KERNEL_CLASS = (1e-3, 5e-3)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def q4_cache(kf, vf, stride=None):
    """kf, vf float32 [n_kv][seq][hd] -> uint8 [n_kv][stride][144]."""
    n_kv, seq, hd = kf.shape
    stride = seq if stride is None else stride
    kb = np.full((n_kv, stride, ROW4), 0xA5, dtype=np.uint8)
    vb = np.full((n_kv, stride, ROW4), 0x5A, dtype=np.uint8)
    kb[:, :seq] = orc.quantize(Q4, kf).reshape(n_kv, seq, ROW4)
    vb[:, :seq] = orc.quantize(Q4, vf).reshape(n_kv, seq, ROW4)
    return kb, vb


def test_q4_encode_bulk_bytes_equal_oracle():
    rows, stride, start, src0 = 300, 333, 17, 3
    r = orc.Rng(0x0404_0001)
    k = r.normal_array((src0 + rows, N_KV * HD), 1.3)
    v = r.normal_array((src0 + rows, N_KV * HD), 0.6)
    # adversarial blocks: all zero, a tie for the largest magnitude with opposite signs (the first
    # wins and fixes the sign of the scale), the extreme at the last lane, values on .5 boundaries
    k[src0, :32] = 0.0
    k[src0, 32:64] = 0.25
    k[src0, 32 + 5] = -3.0
    k[src0, 32 + 20] = 3.0
    k[src0, 64:96] = np.float32(0.125) * np.arange(-16, 16, dtype=np.float32)
    k[src0, 96:128] = 0.01
    k[src0, 127] = 7.75
    v[src0 + 1, :32] = -0.0
    v[src0 + 1, 32:64] = np.float32(1e-30)   # tiny but normal: 1/d is finite
    v[src0 + 1, 64:96] = np.float32(2.5e38)
    kc = torch.full((N_KV, stride, ROW4), 0x11, dtype=torch.uint8, device="cuda")
    vc = torch.full((N_KV, stride, ROW4), 0x22, dtype=torch.uint8, device="cuda")
    attn.kv_encode_bulk(Q4, dev(k), dev(v), kc, vc, N_KV, HD, stride, start, src0, rows)
    torch.cuda.synchronize()
    for src, cache, fill in ((k, kc, 0x11), (v, vc, 0x22)):
        want = orc.quantize(Q4, src[src0:].reshape(rows, N_KV, HD).transpose(1, 0, 2))
        got = host(cache)
        assert np.array_equal(got[:, start:start + rows].ravel(), want)
        assert np.all(got[:, :start] == fill) and np.all(got[:, start + rows:] == fill)


def test_q4_encode_step_append():
    stride, pos = 64, 41
    r = orc.Rng(0x0404_0002)
    k = r.normal_array((N_KV, HD))
    v = r.normal_array((N_KV, HD))
    kc = torch.zeros((N_KV, stride, ROW4), dtype=torch.uint8, device="cuda")
    vc = torch.zeros((N_KV, stride, ROW4), dtype=torch.uint8, device="cuda")
    attn.kv_encode(step_buffer(pos, pos + 1), Q4, dev(k), dev(v), kc, vc, N_KV, HD, stride)
    torch.cuda.synchronize()
    assert np.array_equal(host(kc)[:, pos].ravel(), orc.quantize(Q4, k))
    assert np.array_equal(host(vc)[:, pos].ravel(), orc.quantize(Q4, v))
    assert not host(kc)[:, :pos].any() and not host(kc)[:, pos + 1:].any()


@pytest.mark.parametrize("seq,pad,splits", [(1, 0, 1), (2, 0, 1), (31, 1, 2), (33, 0, 1), (257, 31, 7), (4100, 0, 16),
                                            (8192, 64, None), (24575, 0, None), (24576, 0, None), (32768, 0, None),
                                            (30011, 700, 128)])
def test_q4_decode_matches_oracle(seq, pad, splits):
    # (from 24,576 rows on the launch keeps two workgroups per CU; below it runs one)
    stride = seq + pad
    r = orc.Rng(0x0404_0010 + seq)
    q = r.normal_array((N_HEADS, HD))
    kf = r.normal_array((N_KV, seq, HD))
    vf = r.normal_array((N_KV, seq, HD))
    kb, vb = q4_cache(kf, vf, stride)
    splits = attn.decode_splits(seq, N_KV) if splits is None else splits
    acc = torch.full((N_HEADS, splits, HD), float("nan"), device="cuda")
    ml = torch.full((N_HEADS, splits, 2), float("nan"), device="cuda")
    out = torch.full((N_HEADS, HD), float("nan"), device="cuda")
    attn.attn_decode_kv(step_buffer(seq - 1, seq), Q4, dev(q), dev(kb), dev(vb), acc, ml, out, N_HEADS,
                        N_KV, HD, stride, SCALE, splits)
    torch.cuda.synchronize()
    want = orc.attn_decode_kv(q, kb, vb, N_HEADS, N_KV, HD, seq, SCALE, dtype=Q4, stride=stride)
    ok, ma, _ = report(f"q4 decode seq {seq} splits {splits}", want, host(out).ravel(), *KERNEL_CLASS)
    assert ok
    ok, _, _ = report("  (gate)", want, host(out).ravel(), *GATE)
    assert ok


@pytest.mark.parametrize("pos0,cols,stride,splits", [(700, 3, 1024, 6), (700, 4, 1024, 5), (25000, 4, 25100, 128),
                                                     (5, 2, 64, 3)])
def test_q4_mtp_columns_equal_single_row_decodes(pos0, cols, stride, splits):
    # query rows of one sequence (MTP verify): row r sees keys 0..pos0+r
    seq = pos0 + cols
    r = orc.Rng(0x0404_0020)
    q = r.normal_array((cols, N_HEADS, HD))
    kf = r.normal_array((N_KV, seq, HD))
    vf = r.normal_array((N_KV, seq, HD))
    kb, vb = q4_cache(kf, vf, stride)
    acc = torch.empty((cols, N_HEADS, splits, HD), device="cuda")
    ml = torch.empty((cols, N_HEADS, splits, 2), device="cuda")
    out = torch.empty((cols, N_HEADS, HD), device="cuda")
    pos = torch.tensor([[pos0 + c, pos0 + c + 1] for c in range(cols)], dtype=torch.int32, device="cuda")
    attn.attn_decode_kv_cols(5, pos, dev(q), dev(kb), dev(vb), acc, ml, out, N_HEADS, N_KV, HD, stride,
                             SCALE, splits, cols, N_HEADS * splits * HD, N_HEADS * splits * 2,
                             N_HEADS * HD)
    torch.cuda.synchronize()
    for c in range(cols):
        want = orc.attn_decode_kv(q[c], kb, vb, N_HEADS, N_KV, HD, pos0 + c + 1, SCALE, dtype=Q4,
                                  stride=stride)
        ok, _, _ = report(f"q4 MTP column {c}", want, host(out)[c].ravel(), *KERNEL_CLASS)
        assert ok
        # the reference's column check: a column of a verify group has the bits of its plain decode
        single = torch.empty((N_HEADS, HD), device="cuda")
        attn.attn_decode_kv(step_buffer(pos0 + c, pos0 + c + 1), Q4, dev(q[c]), dev(kb), dev(vb), acc, ml, single,
                            N_HEADS, N_KV, HD, stride, SCALE, splits)
        torch.cuda.synchronize()
        assert np.array_equal(host(single).view(np.uint32), host(out)[c].view(np.uint32))


def test_q4_batched_decode_with_mtp_slots():
    # slots of different depths in one launch (the worker window of the batched decode), two of them verify groups
    # of 3 and 4 rows, the rows of a slot garbage past its live length; every row against the oracle and bit for
    # bit against the plain decode of its row with the same split count
    r = orc.Rng(0x0404_0040)
    depths = [700, 33, 5000, 1, 2049, 12000, 255, 8191]
    cols = [3, 1, 1, 1, 4, 1, 1, 1]
    stride = 12160
    slots = len(depths)
    kc = np.zeros((slots, N_KV, stride, ROW4), dtype=np.uint8)
    vc = np.zeros((slots, N_KV, stride, ROW4), dtype=np.uint8)
    qs, pos = [], []
    for s, (d, c) in enumerate(zip(depths, cols)):
        live = d + c
        kc[s], vc[s] = q4_cache(r.normal_array((N_KV, live, HD)), r.normal_array((N_KV, live, HD)), stride)
        for j in range(c):
            qs.append(r.normal_array((N_HEADS, HD)))
            pos.append((d + j, d + j + 1))
    q = np.stack(qs)
    rows = len(pos)
    splits = attn.batch_splits(stride, N_KV, slots)
    acc = torch.full((rows, N_HEADS, splits, HD), float("nan"), device="cuda")
    ml = torch.full((rows, N_HEADS, splits, 2), float("nan"), device="cuda")
    out = torch.full((rows, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    kd, vd = dev(kc), dev(vc)
    attn.attn_decode_batch_cols(Q4, torch.tensor(pos, dtype=torch.int32, device="cuda"), dev(q), kd, vd, acc, ml, out,
                                N_HEADS, N_KV, HD, stride, SCALE, splits, N_KV * stride * ROW4,
                                N_HEADS * splits * HD, N_HEADS * splits * 2, N_HEADS * HD, cols)
    torch.cuda.synchronize()
    got = host(out)
    assert np.isfinite(got).all()
    row = 0
    for s, c in enumerate(cols):
        for j in range(c):
            want = orc.attn_decode_kv(q[row], kc[s], vc[s], N_HEADS, N_KV, HD, pos[row][1], SCALE, dtype=Q4,
                                      stride=stride)
            ok, ma, _ = orc.compare(want, got[row].ravel(), *KERNEL_CLASS)
            assert ok, f"slot {s} row {j} seq {pos[row][1]}: max_abs {ma}"
            row += 1


@pytest.mark.parametrize("tok,pos0,pad,splits", [(37, 29, 5, 1), (37, 29, 5, 4), (200, 0, 0, 3),
                                                 (96, 3000, 40, 2)])
def test_q4_chunk_prefill_matches_oracle(tok, pos0, pad, splits):
    stride = pos0 + tok + pad
    r = orc.Rng(0x0404_0030 + tok + pos0)
    q = r.normal_array((tok, N_HEADS, HD))
    k = r.normal_array((stride, N_KV, HD))
    v = r.normal_array((stride, N_KV, HD))
    kb = orc.quantize(Q4, k.transpose(1, 0, 2)).reshape(N_KV, stride, ROW4)
    vb = orc.quantize(Q4, v.transpose(1, 0, 2)).reshape(N_KV, stride, ROW4)
    out = torch.full((tok, N_HEADS, HD), float("nan"), device="cuda")
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, N_HEADS, splits)
    attn.chunk_attention_q8_split(dev(q), dev(kb), dev(vb), out, N_HEADS, N_KV, HD, pos0, tok, 2, stride,
                                  acc, ml, splits)
    torch.cuda.synchronize()
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, dtype=Q4,
                             n_threads=8)
    ok, _, _ = report(f"q4 chunk {tok}@{pos0} splits {splits}", want, host(out), *GATE)
    assert ok


def test_unknown_formats_are_refused():
    x = torch.zeros(4096, device="cuda")
    b = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    with pytest.raises(attn.HipmlError):
        attn.attn_decode_kv(step_buffer(0, 1), 9, x, b, b, x, x, x, N_HEADS, N_KV, HD, 1, SCALE, 1)
    with pytest.raises(attn.HipmlError):
        attn.chunk_attention_q8_split(x, b, b, x, N_HEADS, N_KV, HD, 0, 1, 3, 1, None, None, 1)
    with pytest.raises(attn.HipmlError):
        attn.kv_encode_bulk(2, x, x, b, b, N_KV, HD, 4, 0, 0, 1)
