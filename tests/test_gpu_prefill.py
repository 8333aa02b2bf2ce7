"""Causal chunk prefill over a q8_0 cache: HIP path vs the oracle's row-by-row
attn_causal_f32 over the dequantized cache.  Tolerance: max-abs 2e-3 / rel 1e-2
(the parity gate of this build; the reference's chunk class is 2e-3 / 2e-2,
crates/hipml-cli/src/attn_chunk_parity.rs:18-20): fp16 operands, fp32 accumulation."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, SCALE, ROW, dev, host, report  # noqa: E402

GATE = (2e-3, 1e-2)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def chunk_inputs(seed, tok, pos0, pad):
    # recipe of run_q8_splits (attn_chunk_parity.rs:117-160): position-major N(0,1) rows,
    # re-packed head-major, quantized on the host.
    stride = pos0 + tok + pad
    r = orc.Rng(seed)
    q = r.normal_array((tok, N_HEADS, HD))
    k = r.normal_array((stride, N_KV, HD))
    v = r.normal_array((stride, N_KV, HD))
    kb = orc.quantize(0, k.transpose(1, 0, 2)).reshape(N_KV, stride, ROW)
    vb = orc.quantize(0, v.transpose(1, 0, 2)).reshape(N_KV, stride, ROW)
    return q, kb, vb, stride


def run_chunk(q, kb, vb, pos0, tok, stride, splits):
    out = torch.full((tok, N_HEADS, HD), float("nan"), dtype=torch.float32, device="cuda")
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, N_HEADS, splits)
        acc.fill_(float("nan"))
        ml.fill_(float("nan"))
    attn.chunk_attention_q8_split(dev(q), dev(kb), dev(vb), out, N_HEADS, N_KV, HD, pos0, tok, 1,
                                  stride, acc, ml, splits)
    torch.cuda.synchronize()
    return host(out)


@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("tok,pos0,pad", [(37, 29, 0), (37, 29, 8), (1, 0, 0), (33, 0, 3), (64, 1000, 24)])
def test_reference_chunk_case(tok, pos0, pad, splits):
    q, kb, vb, stride = chunk_inputs(0xC4A0_9876_5432, tok, pos0, pad)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=8)
    got = run_chunk(q, kb, vb, pos0, tok, stride, splits)
    ok, _, _ = report(f"chunk {tok}@{pos0} pad {pad} splits {splits}", want, got, *GATE)
    assert ok
    assert np.isfinite(got).all()


@pytest.mark.parametrize("splits", [1, 3])
def test_prefill_672_at_0(splits):
    # the headline benchmark shape: 672 tokens at depth 0
    tok, pos0 = 672, 0
    q, kb, vb, stride = chunk_inputs(0x5EED_0002, tok, pos0, 8)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, n_threads=16)
    got = run_chunk(q, kb, vb, pos0, tok, stride, splits)
    ok, _, _ = report(f"prefill 672@0 splits {splits}", want, got, *GATE)
    assert ok


def test_split_and_mono_agree_and_splits_above_diagonal_are_ignored():
    # pos0 = 0 with many splits: late slices sit wholly above the diagonal for early rows
    tok, pos0 = 96, 0
    q, kb, vb, stride = chunk_inputs(77, tok, pos0, 0)
    mono = run_chunk(q, kb, vb, pos0, tok, stride, 1)
    for splits in (2, 8, 16):
        got = run_chunk(q, kb, vb, pos0, tok, stride, splits)
        # f16 probabilities are rounded against a different running maximum per slice
        ok, _, _ = report(f"split {splits} vs mono", mono, got, 1e-3, 1e-2)
        assert ok


def test_deep_chunk_sampled_rows():
    # the long-context benchmark shape at reduced depth for the CPU side: 256 tokens at depth 20,000,
    # every 37th row checked; exercises long-KV tiling and the split merge.
    tok, pos0 = 256, 20_000
    q, kb, vb, stride = chunk_inputs(0x5EED_0004, tok, pos0, 16)
    rows = np.arange(0, tok, 37, dtype=np.int32)
    want = orc.attn_chunk_kv(q, kb, vb, N_HEADS, N_KV, HD, pos0, tok, stride, SCALE, rows=rows,
                             n_threads=16)
    for splits in (1, 8):
        got = run_chunk(q, kb, vb, pos0, tok, stride, splits)
        ok, _, _ = report(f"chunk 256@20000 splits {splits}", want, got[rows], *GATE)
        assert ok


@pytest.mark.parametrize("tok,pos0,splits", [(37, 29, 1), (37, 29, 4), (300, 0, 5), (160, 4000, 3)])
def test_fused_gate_equals_attention_then_gate(tok, pos0, splits):
    # the fused call must give the bits of the two-call sequence it replaces (mono kernel, uniform
    # key slices, per-block slice counts near position 0)
    q, kb, vb, stride = chunk_inputs(0x6A7D + tok, tok, pos0, 11)
    r = orc.Rng(0x6A7E + tok)
    gate = r.normal_array((tok, N_HEADS, HD))
    plain = run_chunk(q, kb, vb, pos0, tok, stride, splits)
    x = dev(plain)
    two = torch.empty_like(x)
    attn.q_gate(x, dev(gate), two)
    fused = torch.empty_like(x)
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, N_HEADS, splits)
    attn.chunk_attention_q8_split_gate(dev(q), dev(kb), dev(vb), dev(gate), fused, N_HEADS, N_KV, HD,
                                       pos0, tok, 1, stride, acc, ml, splits)
    torch.cuda.synchronize()
    assert np.array_equal(host(two), host(fused)), f"fused gate differs ({tok}@{pos0} splits {splits})"
    # and the oracle's gate of the same rows, to the gate kernel's own class (device expf vs libm)
    want = orc.q_gate(plain.ravel(), gate.ravel())
    ok, _, _ = report(f"fused gate {tok}@{pos0} splits {splits}", want, host(fused).ravel(), 1e-6, 1e-5)
    assert ok
    # the same rows delivered as f16 for the output projection: exactly f16 (nearest even) of the above
    work = torch.full_like(x, float("nan"))
    out16 = torch.full(x.shape, float("nan"), dtype=torch.float16, device="cuda")
    attn.chunk_attention_q8_split_gate_f16(dev(q), dev(kb), dev(vb), dev(gate), work, out16, N_HEADS,
                                           N_KV, HD, pos0, tok, 1, stride, acc, ml, splits)
    torch.cuda.synchronize()
    assert np.array_equal(host(out16).view(np.uint16), host(fused).astype(np.float16).view(np.uint16))
