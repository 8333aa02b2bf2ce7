"""Chunk prefill with the key slices inside the workgroups (splits = 0 of the chunk entry points): the
kernel for chunks near position 0.  Same oracle and same gate (2e-3 / 1e-2) as the sliced kernel; its
sums are held against a reference exponent that lags the running maximum by up to 2^8, which the gate
covers (f16 keeps its relative precision over that range)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, SCALE, dev, host, report  # noqa: E402
from test_gpu_prefill import chunk_inputs, run_chunk, GATE  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


@pytest.mark.parametrize("tok,pos0,pad", [(1, 0, 0), (33, 0, 3), (37, 29, 0), (37, 29, 8), (96, 64, 0), (130, 63, 1),
                                          (64, 1000, 24), (300, 0, 5), (31, 1, 0), (128, 127, 2)])
def test_reference_chunk_cases(tok, pos0, pad):
    q, kb, vb, stride = chunk_inputs(0xC4A0_9876_5432, tok, pos0, pad)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=8)
    got = run_chunk(q, kb, vb, pos0, tok, stride, 0)
    ok, _, _ = report(f"chunk {tok}@{pos0} pad {pad}, slices inside the workgroups", want, got, *GATE)
    assert ok
    assert np.isfinite(got).all()


def test_prefill_672_at_0_plain_gated_and_as_f16_rows():
    # the headline shape; the policy picks this kernel for it
    tok, pos0 = 672, 0
    assert attn.chunk_splits(pos0, tok, N_KV) == 0
    q, kb, vb, stride = chunk_inputs(0x5EED_0002, tok, pos0, 8)
    gate = orc.Rng(0x6A7E).normal_array((tok, N_HEADS, HD))
    plain = run_chunk(q, kb, vb, pos0, tok, stride, 0)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=16)
    ok, _, _ = report("prefill 672@0, slices inside the workgroups", want, plain, *GATE)
    assert ok
    # the fused gate gives the bits of the attention followed by the gate kernel
    x = dev(plain)
    two = torch.empty_like(x)
    attn.q_gate(x, dev(gate), two)
    fused = torch.full_like(x, float("nan"))
    attn.chunk_attention_q8_split_gate(dev(q), dev(kb), dev(vb), dev(gate), fused, N_HEADS, N_KV, HD, pos0, tok, 1,
                                       stride, None, None, 0)
    torch.cuda.synchronize()
    assert np.array_equal(host(two).view(np.uint32), host(fused).view(np.uint32))
    # and the f16 rows are f16 (nearest even) of those
    out16 = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float16, device="cuda")
    work = torch.empty_like(x)
    attn.chunk_attention_q8_split_gate_f16(dev(q), dev(kb), dev(vb), dev(gate), work, out16, N_HEADS, N_KV, HD, pos0,
                                           tok, 1, stride, None, None, 0)
    torch.cuda.synchronize()
    assert np.array_equal(host(out16).view(np.uint16), host(fused).astype(np.float16).view(np.uint16))


def test_agrees_with_the_sliced_kernel_and_is_repeatable():
    tok, pos0 = 200, 90
    q, kb, vb, stride = chunk_inputs(0x77AA, tok, pos0, 6)
    a = run_chunk(q, kb, vb, pos0, tok, stride, 0)
    b = run_chunk(q, kb, vb, pos0, tok, stride, 0)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))  # fixed order of every sum
    c = run_chunk(q, kb, vb, pos0, tok, stride, 3)
    ok, _, _ = report("in-workgroup slices vs 3 key slices", c, a, 1e-3, 1e-2)
    assert ok


def test_large_scores_move_the_reference_exponent():
    # Q scaled so that scores spread over hundreds of log2 units and the running maximum keeps jumping
    # by more than the lag the kernels allow themselves: the rescaling path.  At this scale the f16 rounding
    # of the Q and K operands moves every kernel 1.5e-2 from the f32 oracle (a score of a few hundred carries
    # an error of a tenth), so the tight check is between the in-workgroup kernel and the single-pass one:
    # the same operands, different moments at which the reference exponent moves (the slices start at
    # different keys), so a mistake in the rescaling of either shows as an error of order one.
    tok, pos0 = 96, 40
    q, kb, vb, stride = chunk_inputs(0xB16_5C0E, tok, pos0, 0)
    q = (q * 12.0).astype(np.float32)
    mono = run_chunk(q, kb, vb, pos0, tok, stride, 1)
    got = run_chunk(q, kb, vb, pos0, tok, stride, 0)
    ok, _, _ = report("large scores, in-workgroup slices vs single pass", mono, got, *GATE)
    assert ok
    assert np.isfinite(got).all()
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=8)
    for name, x in (("in-workgroup slices", got), ("single pass", mono)):
        ok, _, _ = report(f"large scores, {name} vs the oracle (f16 Q and K operands)", want, x, 3e-2, 1e-2)
        assert ok


def test_q4_cache():
    tok, pos0, pad = 150, 20, 3
    stride = pos0 + tok + pad
    r = orc.Rng(0x0404)
    q = r.normal_array((tok, N_HEADS, HD))
    kb = orc.quantize(1, r.normal_array((N_KV, stride, HD))).reshape(N_KV, stride, -1)
    vb = orc.quantize(1, r.normal_array((N_KV, stride, HD))).reshape(N_KV, stride, -1)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, dtype=1, n_threads=8)
    out = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_q8_split(dev(q), dev(kb), dev(vb), out, N_HEADS, N_KV, HD, pos0, tok, 2, stride, None, None, 0)
    torch.cuda.synchronize()
    ok, _, _ = report("q4_0 cache, slices inside the workgroups", want, host(out), *GATE)
    assert ok


@pytest.mark.parametrize("tok,pos0,splits", [(672, 0, 0), (70, 33, 0), (100, 40, 3), (64, 5, 1)])
def test_query_rows_rotated_inside_the_attention_call(tok, pos0, splits):
    # hipml_attn_chunk_rope_q8 on unrotated query rows = hipml_rope_chunk_f32 on them, then the attention:
    # the same bits, with the rows rotated in the kernel (splits 0, q untouched) or in place first
    n_rot, theta = 64, 1e7
    attn.rope_table(theta, n_rot, 2048)
    q, kb, vb, stride = chunk_inputs(0x120E + tok, tok, pos0, 4)
    gate = orc.Rng(0x6A7F + tok).normal_array((tok, N_HEADS, HD))
    kd, vd, gd = dev(kb), dev(vb), dev(gate)
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, N_HEADS, splits)
    # separate calls (k rows are not involved: a dummy stands in)
    q_rot = dev(q)
    k_dummy = torch.zeros((tok, N_KV, HD), dtype=torch.float32, device="cuda")
    attn.rope_chunk(q_rot, k_dummy, N_HEADS, N_KV, HD, n_rot, theta, pos0, tok)
    want = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_q8_split_gate(q_rot, kd, vd, gd, want, N_HEADS, N_KV, HD, pos0, tok, 1, stride, acc, ml,
                                       splits)
    # one call
    q_in = dev(q)
    got = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_rope_q8(q_in, kd, vd, gd, got, None, N_HEADS, N_KV, HD, n_rot, theta, pos0, tok, 1,
                                 stride, acc, ml, splits)
    torch.cuda.synchronize()
    assert np.array_equal(host(got).view(np.uint32), host(want).view(np.uint32))
    if splits == 0:
        assert np.array_equal(host(q_in).view(np.uint32), q.view(np.uint32))  # left as it was
    else:
        assert np.array_equal(host(q_in).view(np.uint32), host(q_rot).view(np.uint32))  # rotated in place
    # f16 rows, no gate
    out16 = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float16, device="cuda")
    work = torch.empty_like(got)
    plain = torch.empty_like(got)
    attn.chunk_attention_q8_split(q_rot, kd, vd, plain, N_HEADS, N_KV, HD, pos0, tok, 1, stride, acc, ml, splits)
    attn.chunk_attention_rope_q8(dev(q), kd, vd, None, work, out16, N_HEADS, N_KV, HD, n_rot, theta, pos0, tok, 1,
                                 stride, acc, ml, splits)
    torch.cuda.synchronize()
    assert np.array_equal(host(out16).view(np.uint16), host(plain).astype(np.float16).view(np.uint16))


def test_fused_append_may_leave_the_query_rows_alone():
    # hipml_rope_encode_chunk_f32 with q = NULL: K rotated, K/V appended, same bits as with q given
    tok, pos0, n_rot, theta = 50, 7, 64, 1e7
    attn.rope_table(theta, n_rot, 2048)
    stride = 64
    r = orc.Rng(0xA99E)
    q = r.normal_array((tok, N_HEADS, HD))
    k = r.normal_array((tok, N_KV, HD))
    v = r.normal_array((tok, N_KV, HD))
    res = []
    for with_q in (True, False):
        kc = torch.zeros((N_KV, stride, 272), dtype=torch.uint8, device="cuda")
        vc = torch.zeros_like(kc)
        kd = dev(k)
        attn.rope_encode_chunk(dev(q) if with_q else None, kd, dev(v), kc, vc, N_HEADS, N_KV, HD, n_rot, theta, pos0,
                               tok, 0, stride)
        torch.cuda.synchronize()
        res.append((host(kc), host(vc), host(kd)))
    for a, b in zip(*res):
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
