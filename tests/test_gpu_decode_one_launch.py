"""The decode whose workgroups merge their key splits themselves (hipml_attn_decode_one_launch(1)): the
same parity bar as the two-launch form against the CPU oracle, the reference's column check inside the
mode, and what is particular to it: the arrival counters are back at zero after every launch (repeated
launches, graph replays, two streams), groups of eight splits with a ragged last group, splits without a
live key."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import (N_HEADS, N_KV, HD, SCALE, dev, host, quantized_cache, step_buffer,  # noqa: E402
                      decode_scratch, run_decode, report)

GATE = (2e-3, 1e-2)
KERNEL_CLASS = (1e-3, 5e-3)


@pytest.fixture(scope="module", autouse=True)
def _one_launch():
    attn.init(0)
    before = attn.decode_one_launch(1)
    yield
    attn.decode_one_launch(before)


def case(seed, seq, stride=None, heads=N_HEADS, n_kv=N_KV):
    r = orc.Rng(seed)
    q = r.normal_array((heads, HD))
    kf = r.normal_array((n_kv, seq, HD))
    vf = r.normal_array((n_kv, seq, HD))
    kb, vb = quantized_cache(kf, vf, stride)
    return q, kb, vb


def test_the_mode_is_on_and_reads_back():
    assert attn.decode_one_launch(-1) == 1


@pytest.mark.parametrize("seq,stride,splits", [
    (1, 1, 1), (37, 64, 1), (673, 680, 6), (1000, 1000, 7), (1000, 1024, 8), (1000, 1000, 9),
    (4096, 4096, 17), (5000, 8192, 40), (8192, 8192, 64), (9000, 9100, 128), (300, 300, 64),
])
def test_against_the_oracle(seq, stride, splits):
    # one group, full groups, a ragged last group, one workgroup per CU, the merge's limit of 128 splits,
    # and more splits than tiles (splits that see no key)
    q, kb, vb = case(0x01A0_0000 + seq + splits, seq, stride)
    want = orc.attn_decode_kv(q, kb, vb, N_HEADS, N_KV, HD, seq, SCALE, stride=stride)
    got = run_decode(q, kb, vb, N_HEADS, N_KV, seq, stride, SCALE, splits)
    ok, _, _ = report(f"one launch: seq {seq} stride {stride} splits {splits}", want, got, *KERNEL_CLASS)
    assert ok and orc.compare(want, got, *GATE)[0]


def test_benchmark_depth_and_other_head_groupings():
    q, kb, vb = case(0x01A1_0001, 32768)
    want = orc.attn_decode_kv(q, kb, vb, N_HEADS, N_KV, HD, 32768, SCALE)
    got = run_decode(q, kb, vb, N_HEADS, N_KV, 32768, 32768, SCALE, attn.decode_splits(32768, N_KV))
    assert report("one launch: seq 32768", want, got, *KERNEL_CLASS)[0]
    for heads, n_kv in [(8, 1), (6, 2), (5, 5)]:
        q, kb, vb = case(0x01A1_0010 + heads, 2500, 2600, heads, n_kv)
        want = orc.attn_decode_kv(q, kb, vb, heads, n_kv, HD, 2500, SCALE, stride=2600)
        got = run_decode(q, kb, vb, heads, n_kv, 2500, 2600, SCALE, 19)
        assert report(f"one launch: {heads} heads / {n_kv}", want, got, *KERNEL_CLASS)[0]


def test_more_than_128_splits_fall_back_to_the_merge_kernel():
    q, kb, vb = case(0x01A2_0001, 40000, heads=6, n_kv=1)
    want = orc.attn_decode_kv(q, kb, vb, 6, 1, HD, 40000, SCALE)
    got = run_decode(q, kb, vb, 6, 1, 40000, 40000, SCALE, 256)
    assert report("one launch mode, 256 splits", want, got, *KERNEL_CLASS)[0]


def test_seq_zero_gives_zero():
    q, kb, vb = case(0x01A3_0001, 64)
    acc, ml = decode_scratch(N_HEADS, 12)
    out = torch.full((N_HEADS, HD), 7.0, dtype=torch.float32, device="cuda")
    attn.attn_decode_kv(step_buffer(0, 0), 0, dev(q), dev(kb), dev(vb), acc, ml, out, N_HEADS, N_KV, HD, 64,
                        SCALE, 12)
    torch.cuda.synchronize()
    assert not host(out).any()


@pytest.mark.parametrize("cols,pos0,stride,splits", [(2, 700, 720, 5), (3, 700, 720, 11), (4, 700, 720, 5),
                                                     (3, 9000, 9100, 64), (4, 9000, 9100, 128)])
def test_verify_columns_have_the_bits_of_plain_decodes(cols, pos0, stride, splits):
    live = pos0 + cols
    r = orc.Rng(0x01A4_0000 + cols + splits)
    q = r.normal_array((cols, N_HEADS, HD))
    kf = r.normal_array((N_KV, live, HD))
    vf = r.normal_array((N_KV, live, HD))
    kb, vb = quantized_cache(kf, vf, stride)
    acc, ml = decode_scratch(N_HEADS, splits, cols)
    out = torch.full((cols, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    pos = torch.tensor([[pos0 + c, pos0 + c + 1] for c in range(cols)], dtype=torch.int32, device="cuda")
    attn.attn_decode_kv_cols(4, pos, dev(q), dev(kb), dev(vb), acc, ml, out, N_HEADS, N_KV, HD, stride, SCALE,
                             splits, cols, N_HEADS * splits * HD, N_HEADS * splits * 2, N_HEADS * HD)
    torch.cuda.synchronize()
    got = host(out)
    for c in range(cols):
        want = orc.attn_decode_kv(q[c], kb, vb, N_HEADS, N_KV, HD, pos0 + c + 1, SCALE, stride=stride)
        assert orc.compare(want, got[c], *KERNEL_CLASS)[0]
        single = run_decode(q[c], kb, vb, N_HEADS, N_KV, pos0 + c + 1, stride, SCALE, splits)
        assert np.array_equal(single.view(np.uint32), got[c].ravel().view(np.uint32))


def test_gate_in_the_merge_has_the_bits_of_the_gate_kernel():
    seq, stride = 5000, 8192
    q, kb, vb = case(0x01A5_0001, seq, stride)
    gate = orc.Rng(0x01A5_0002).normal_array((N_HEADS, HD))
    splits = attn.decode_splits(seq, N_KV)
    acc, ml = decode_scratch(N_HEADS, splits)
    step = step_buffer(seq - 1, seq)
    two = torch.full((N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv(step, 0, dev(q), dev(kb), dev(vb), acc, ml, two, N_HEADS, N_KV, HD, stride, SCALE, splits)
    attn.q_gate(two, dev(gate), two, N_HEADS * HD)
    one = torch.full((N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv_gate(step, 0, dev(q), dev(kb), dev(vb), acc, ml, one, dev(gate), N_HEADS, N_KV, HD,
                             stride, SCALE, splits)
    torch.cuda.synchronize()
    assert torch.equal(one, two)


def test_counters_are_back_at_zero_after_every_launch():
    # the same call 50 times on one stream, alternating with a call of another shape: same bits every time
    seq = 7000
    q, kb, vb = case(0x01A6_0001, seq)
    q2, kb2, vb2 = case(0x01A6_0002, 1500, 1600)
    qd, kd, vd = dev(q), dev(kb), dev(vb)
    q2d, k2d, v2d = dev(q2), dev(kb2), dev(vb2)
    splits, splits2 = attn.decode_splits(seq, N_KV), 9
    acc, ml = decode_scratch(N_HEADS, splits)
    step, step2 = step_buffer(seq - 1, seq), step_buffer(1499, 1500)
    outs = torch.full((50, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    outs2 = torch.full((50, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    for i in range(50):
        attn.attn_decode_kv(step, 0, qd, kd, vd, acc, ml, outs[i], N_HEADS, N_KV, HD, seq, SCALE, splits)
        attn.attn_decode_kv(step2, 0, q2d, k2d, v2d, acc, ml, outs2[i], N_HEADS, N_KV, HD, 1600, SCALE, splits2)
    torch.cuda.synchronize()
    want = orc.attn_decode_kv(q, kb, vb, N_HEADS, N_KV, HD, seq, SCALE)
    assert orc.compare(want, host(outs[0]).ravel(), *KERNEL_CLASS)[0]
    assert all(torch.equal(outs[0], outs[i]) for i in range(1, 50))
    assert all(torch.equal(outs2[0], outs2[i]) for i in range(1, 50))


def test_two_streams_have_counters_of_their_own():
    seq = 6000
    qa, ka, va = case(0x01A7_0001, seq)
    qb, kb_, vb_ = case(0x01A7_0002, seq)
    splits = attn.decode_splits(seq, N_KV)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    ins = [(dev(qa), dev(ka), dev(va)), (dev(qb), dev(kb_), dev(vb_))]
    scr = [decode_scratch(N_HEADS, splits), decode_scratch(N_HEADS, splits)]
    outs = [torch.full((20, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda") for _ in range(2)]
    step = step_buffer(seq - 1, seq)
    torch.cuda.synchronize()
    for i in range(20):
        for j, st in enumerate((sa, sb)):
            q_, k_, v_ = ins[j]
            attn.attn_decode_kv(step, 0, q_, k_, v_, scr[j][0], scr[j][1], outs[j][i], N_HEADS, N_KV, HD, seq,
                                SCALE, splits, stream=st)
    torch.cuda.synchronize()
    for j, (q_, k_, v_) in enumerate([(qa, ka, va), (qb, kb_, vb_)]):
        want = orc.attn_decode_kv(q_, k_, v_, N_HEADS, N_KV, HD, seq, SCALE)
        assert orc.compare(want, host(outs[j][0]).ravel(), *KERNEL_CLASS)[0]
        assert all(torch.equal(outs[j][0], outs[j][i]) for i in range(1, 20))


def test_a_captured_launch_replays():
    seq = 3000
    q, kb, vb = case(0x01A8_0001, seq, 4096)
    qd, kd, vd = dev(q), dev(kb), dev(vb)
    splits = attn.decode_splits(seq, N_KV)
    acc, ml = decode_scratch(N_HEADS, splits)
    step = step_buffer(seq - 1, seq)
    out = torch.full((N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    eager = torch.full((N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv(step, 0, qd, kd, vd, acc, ml, eager, N_HEADS, N_KV, HD, 4096, SCALE, splits)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        attn.attn_decode_kv(step, 0, qd, kd, vd, acc, ml, out, N_HEADS, N_KV, HD, 4096, SCALE, splits)
    torch.cuda.synchronize()
    for i in range(4):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"
        # eager work between the replays
        attn.attn_decode_kv(step, 0, qd, kd, vd, acc, ml, eager, N_HEADS, N_KV, HD, 4096, SCALE, splits)
        torch.cuda.synchronize()
