"""Decode at head_dim 64: the reference's parity table runs its decode kernels there too
(crates/hipml-core/src/parity_kv.rs:166-213: 8 query heads, 2 KV heads, scale 0.125, q8_0 and q4_0,
37 keys in one split and 1,000 keys in 7).  The library serves that width with plain fp32 kernels behind the
same entry points; they are held to the reference's own gate for these cases, Tol::DEFAULT 1e-4 / 1e-3
(crates/hipml-core/src/parity.rs:34)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import dev, host, report  # noqa: E402

HD = 64
TOL = (1e-4, 1e-3)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def case(seed, heads, n_kv, seq, dtype, stride=None):
    # the reference's kv_case! recipe (parity_kv.rs:39-60)
    r = orc.Rng(seed)
    q = r.normal_array((heads, HD))
    kf = r.normal_array((n_kv, seq, HD), 0.3)
    vf = r.normal_array((n_kv, seq, HD))
    stride = seq if stride is None else stride
    row = orc.row_bytes(dtype, HD)
    kb = np.full((n_kv, stride, row), 0xA5, np.uint8)
    vb = np.full((n_kv, stride, row), 0x5A, np.uint8)
    kb[:, :seq] = orc.quantize(dtype, kf).reshape(n_kv, seq, row)
    vb[:, :seq] = orc.quantize(dtype, vf).reshape(n_kv, seq, row)
    return q, kb, vb


def scratch(rows, heads, splits):
    acc = torch.full((rows, heads, splits, HD), float("nan"), dtype=torch.float32, device="cuda")
    ml = torch.full((rows, heads, splits, 2), float("nan"), dtype=torch.float32, device="cuda")
    return acc, ml


@pytest.mark.parametrize("name,dtype,seed,seq,splits", [
    ("attn_decode_kv_q8_hd64_s37", 0, 0x9E00_0009, 37, 1),
    ("attn_decode_kv_q8_hd64_s1000", 0, 0x9E00_000A, 1000, 7),
    ("attn_decode_kv_q4_hd64_s37", 1, 0x9E00_000B, 37, 1),
    ("attn_decode_kv_q4_hd64_s1000", 1, 0x9E00_000C, 1000, 7),
])
def test_reference_hd64_cases(name, dtype, seed, seq, splits):
    heads, n_kv, scale = 8, 2, 0.125
    q, kb, vb = case(seed, heads, n_kv, seq, dtype)
    want = orc.attn_decode_kv(q, kb, vb, heads, n_kv, HD, seq, scale, dtype=dtype)
    acc, ml = scratch(1, heads, splits)
    out = torch.full((heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    step = torch.tensor([seq - 1, seq, 0, 0, 0, 0, 0, 0], dtype=torch.int32, device="cuda")
    attn.attn_decode_kv(step, dtype, dev(q), dev(kb), dev(vb), acc, ml, out, heads, n_kv, HD, seq, scale, splits)
    torch.cuda.synchronize()
    ok, _, _ = report(name, want, host(out).ravel(), *TOL)
    assert ok


def test_padded_stride_more_splits_than_keys_and_the_fused_gate():
    heads, n_kv, seq, stride, scale, splits = 8, 2, 45, 64, 0.125, 64
    q, kb, vb = case(0x64AA, heads, n_kv, seq, 0, stride)
    gate = orc.Rng(0x6A7E).normal_array((heads, HD))
    want = orc.attn_decode_kv(q, kb, vb, heads, n_kv, HD, seq, scale, stride=stride)
    acc, ml = scratch(1, heads, splits)
    out = torch.full((heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    step = torch.tensor([seq - 1, seq, 0, 0, 0, 0, 0, 0], dtype=torch.int32, device="cuda")
    attn.attn_decode_kv(step, 0, dev(q), dev(kb), dev(vb), acc, ml, out, heads, n_kv, HD, stride, scale, splits)
    torch.cuda.synchronize()
    ok, _, _ = report("hd64, 45 keys in 64 splits, stride 64", want, host(out).ravel(), *TOL)
    assert ok
    gated = torch.full_like(out, float("nan"))
    attn.attn_decode_kv_gate(step, 0, dev(q), dev(kb), dev(vb), acc, ml, gated, dev(gate), heads, n_kv, HD, stride,
                             scale, splits)
    two = torch.empty_like(out)
    attn.q_gate(out, dev(gate), two)
    torch.cuda.synchronize()
    assert np.array_equal(host(gated).view(np.uint32), host(two).view(np.uint32))


def test_verify_columns_and_batched_slots():
    # three rows of one sequence (causal within the draft), then four slots of different depths with their
    # own caches, one of them with two rows: every row against the oracle at its own length
    heads, n_kv, scale, splits = 8, 2, 0.125, 5
    seq, stride = 300, 320
    _, kb, vb = case(0x64C0, heads, n_kv, seq, 0, stride)
    r = orc.Rng(0x64C1)
    q = r.normal_array((3, heads, HD))
    pos = torch.tensor([[seq - 3, seq - 2], [seq - 2, seq - 1], [seq - 1, seq]], dtype=torch.int32, device="cuda")
    acc, ml = scratch(3, heads, splits)
    out = torch.full((3, heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv_cols(0, pos, dev(q), dev(kb), dev(vb), acc, ml, out, heads, n_kv, HD, stride, scale, splits, 3,
                             heads * splits * HD, heads * splits * 2, heads * HD)
    torch.cuda.synchronize()
    for c in range(3):
        want = orc.attn_decode_kv(q[c], kb, vb, heads, n_kv, HD, seq - 2 + c, scale, stride=stride)
        ok, _, _ = report(f"hd64 verify column {c}", want, host(out)[c].ravel(), *TOL)
        assert ok

    depths, cols = [17, 300, 1, 129], [1, 2, 1, 1]
    slot_bytes = n_kv * stride * orc.row_bytes(0, HD)
    kbs, vbs, qs, seqs = [], [], [], []
    for s, (d, c) in enumerate(zip(depths, cols)):
        _, k1, v1 = case(0x64D0 + s, heads, n_kv, d, 0, stride)
        kbs.append(k1)
        vbs.append(v1)
        for j in range(c):
            qs.append(r.normal_array((heads, HD)))
            seqs.append(d - (c - 1 - j))
    rows = len(qs)
    pos = torch.tensor([[x - 1, x] for x in seqs], dtype=torch.int32, device="cuda")
    acc, ml = scratch(rows, heads, splits)
    out = torch.full((rows, heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_batch_cols(0, pos, dev(np.stack(qs)), dev(np.stack(kbs)), dev(np.stack(vbs)), acc, ml, out, heads,
                                n_kv, HD, stride, scale, splits, slot_bytes, heads * splits * HD, heads * splits * 2,
                                heads * HD, cols)
    torch.cuda.synchronize()
    row = 0
    for s, c in enumerate(cols):
        for j in range(c):
            want = orc.attn_decode_kv(qs[row], kbs[s], vbs[s], heads, n_kv, HD, seqs[row], scale, stride=stride)
            ok, _, _ = report(f"hd64 batch slot {s} row {j} (seq {seqs[row]})", want, host(out)[row].ravel(), *TOL)
            assert ok
            row += 1


def test_other_widths_are_refused():
    q = torch.zeros((8, 128), dtype=torch.float32, device="cuda")
    c = torch.zeros((2, 8, 136), dtype=torch.uint8, device="cuda")
    acc, ml = scratch(1, 8, 1)
    step = torch.tensor([0, 1, 0, 0, 0, 0, 0, 0], dtype=torch.int32, device="cuda")
    with pytest.raises(attn.HipmlError):
        attn.attn_decode_kv(step, 0, q, c, c, acc, ml, q.clone(), 8, 2, 128, 8, 0.1, 1)
