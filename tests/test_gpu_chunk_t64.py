"""The sliced chunk kernel over the f16 copy with 64 tokens per wave (chunk_f16_t64_kernel).

hipml_attn_chunk_kv_f16 runs it whenever the keys are cut into slices, every task block gets all of them and
its cut of the tokens needs no extra round of workgroups (uniform(...) and no_extra_round(...) below restate the
launcher's rules), which is the case deep in a prefix.  Its accumulators live in
registers the compiler does not manage and its softmax is spread over the slots between its MFMAs, so the cases
here go for what that could break: token counts that are no multiple of 64, task counts that are no multiple of
4, every mapping of workgroups to (KV head, slice), the diagonal inside the last slice, slices that end inside
a tile, and scores large enough to move the reference exponent again and again.  Expected values: the CPU
oracle over the same cache bytes, at the chunk gate of the reference (2e-3 / 1e-2)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import HD, SCALE, ROW, dev, host, report  # noqa: E402
from test_gpu_prefill import GATE  # noqa: E402


# two kernels that round the same f16 operands and differ in the order of their sums and in the moments they
# rescale: observed 2.6e-5 .. 8.9e-5 on these cases
SAME_OPERANDS = (1.5e-4, 1e-3)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def uniform(tok, pos0, splits, group):
    # the launcher's rule: task blocks of 8 tasks of 32 tokens; a block whose last token sees fewer key tiles
    # than splits * slice_tiles gets fewer slices, and then the kernel of 32 tokens per wave runs
    ntask = (tok + 31) // 32 * group
    tiles_last = (pos0 + tok + 63) // 64
    slice_tiles = (tiles_last + splits - 1) // splits
    for tb in range((ntask + 7) // 8):
        last_task = min(tb * 8 + 7, ntask - 1)
        last_tok = min((last_task // group + 1) * 32, tok) - 1
        tiles = (pos0 + last_tok + 1 + 63) // 64
        if min(splits, max(1, (tiles + slice_tiles - 1) // slice_tiles)) != splits:
            return False
    return True


def no_extra_round(tok, splits, n_heads, n_kv):
    # the launcher's second rule: the cut into tasks of 64 tokens must not need a round of 256 workgroups more
    # than the cut into tasks of 32
    group, pairs = n_heads // n_kv, n_kv * splits

    def grid(blocks):
        if pairs % 8 != 0 and 8 % pairs == 0:
            return 8 * ((blocks + 8 // pairs - 1) // (8 // pairs))
        return pairs * blocks
    g32 = grid(((tok + 31) // 32 * group + 7) // 8)
    # tasks of 64 tokens x 1 head; up to 32 left-over tokens make tasks of 32 tokens x 2 heads
    rem = tok % 64
    tasks = (tok // 64 + (1 if rem > 32 else 0)) * group + ((group + 1) // 2 if 0 < rem <= 32 else 0)
    g64 = grid((tasks + 3) // 4)
    return (g64 + 255) // 256 <= (g32 + 255) // 256


def inputs(seed, tok, pos0, pad, n_heads, n_kv, q_scale=1.0, k_ramp=0.0):
    stride = pos0 + tok + pad
    r = orc.Rng(seed)
    q = (r.normal_array((tok, n_heads, HD)) * q_scale).astype(np.float32)
    k = r.normal_array((n_kv, stride, HD))
    if k_ramp:
        # keys grow with their position, so the maxima keep growing along the prefix
        k = (k * (1.0 + k_ramp * np.arange(stride, dtype=np.float32) / stride)[None, :, None]).astype(np.float32)
    v = r.normal_array((n_kv, stride, HD))
    kb = orc.quantize(0, k).reshape(n_kv, stride, ROW)
    vb = orc.quantize(0, v).reshape(n_kv, stride, ROW)
    return q, kb, vb, stride


def run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv, gate=None):
    copy = attn.kv_f16_alloc(stride, n_kv)
    copy.fill_(0xFF)  # f16 NaN wherever the conversion does not write
    attn.kv_f16_rows(0, dev(kb), dev(vb), copy, n_kv, HD, stride, 0, pos0 + tok)
    out = torch.full((tok, n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, n_heads, splits)
        acc.fill_(float("nan"))
        ml.fill_(float("nan"))
    attn.chunk_attention_kv_f16(dev(q), copy, None if gate is None else dev(gate), out, None, n_heads, n_kv, HD,
                                pos0, tok, stride, acc, ml, splits)
    torch.cuda.synchronize()
    return host(out)


@pytest.mark.parametrize("tok,pos0,pad,splits,n_heads,n_kv", [
    (100, 5000, 7, 4, 24, 4),    # 36 tokens in the last tile of 64; 12 tasks = 3 workgroups per (KV head, slice)
    (65, 3000, 0, 4, 24, 4),     # one token in the second tile
    (200, 3000, 1, 3, 24, 4),    # 12 (KV head, slice) pairs: neither a multiple nor a divisor of the 8 XCDs
    (70, 2000, 0, 2, 24, 4),     # 8 pairs
    (128, 4096, 0, 2, 6, 1),     # 2 pairs, one KV head: each pair spread over 4 XCDs
    (64, 2500, 5, 5, 8, 2),      # 4 heads per KV head: 4 tasks = exactly one workgroup; 10 pairs
    (96, 2200, 0, 4, 12, 4),     # 3 heads per KV head: 6 tasks, the second workgroup half empty
    (300, 9000, 3, 8, 24, 4),    # 8 slices
    (672, 9000, 0, 4, 24, 4),    # 10 tiles of 64 and 32 tokens more: their tasks pair two heads (63 tasks, 256 workgroups)
    (96, 2600, 2, 4, 12, 4),     # 32 tokens more and 3 heads per KV head: the last pair has one head
    (65, 2100, 0, 3, 10, 2),     # one token more, 5 heads per KV head
    (97, 2300, 1, 4, 24, 4),     # 33 tokens more: a tile of 64 with a ragged second half
])
def test_against_the_oracle(tok, pos0, pad, splits, n_heads, n_kv):
    assert uniform(tok, pos0, splits, n_heads // n_kv) and no_extra_round(tok, splits, n_heads, n_kv)
    q, kb, vb, stride = inputs(0x7640_0000 + tok * 131 + pos0, tok, pos0, pad, n_heads, n_kv)
    want = orc.attn_chunk_kv(q, kb, vb, n_heads, n_kv, HD, pos0, tok, stride, SCALE, n_threads=8)
    got = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv)
    ok, _, _ = report(f"64-token chunk kernel {tok}@{pos0} pad {pad} splits {splits} heads {n_heads}/{n_kv}", want,
                      got, *GATE)
    assert ok
    assert np.isfinite(got).all()
    # An independent kernel over the same tiles: the unsliced pass of the kernel of 32 tokens per wave (compiler-
    # managed accumulators, builtin MFMAs).  It rounds the same operands, so it must agree far inside the gate:
    # a hazard in the hand-placed accumulators shows up as a few 1e-4 here long before it reaches 2e-3 there.
    mono = run(q, kb, vb, pos0, tok, stride, 1, n_heads, n_kv)
    ok, _, _ = report(f"  the same chunk, 64-token kernel vs the single pass of the 32-token kernel", mono, got,
                      *SAME_OPERANDS)
    assert ok


def test_gate_is_applied_by_the_merge():
    tok, pos0, splits, n_heads, n_kv = 130, 4000, 4, 24, 4
    assert uniform(tok, pos0, splits, n_heads // n_kv)
    q, kb, vb, stride = inputs(0x7641_6A7E, tok, pos0, 2, n_heads, n_kv)
    gate = orc.Rng(0x6A7E_7641).normal_array((tok, n_heads, HD))
    plain = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv)
    gated = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv, gate=gate)
    two = torch.empty((tok, n_heads, HD), dtype=torch.float32, device="cuda")
    attn.q_gate(dev(plain), dev(gate), two)
    torch.cuda.synchronize()
    assert np.array_equal(gated.view(np.uint32), host(two).view(np.uint32))


def test_growing_maxima_move_the_reference_exponent():
    # Q scaled and the keys growing along the prefix: the maxima outgrow the reference exponent many times
    # in every slice, so O is rescaled in its registers again and again.  At this scale the f16 rounding of
    # the operands moves any kernel ~1.5e-2 from the f32 oracle; the tight check is against the kernel of 32
    # tokens per wave over the same copy (unsplit: one pass over the keys), which rounds the same operands
    # and rescales at other moments.
    tok, pos0, splits, n_heads, n_kv = 128, 3000, 4, 24, 4
    assert uniform(tok, pos0, splits, n_heads // n_kv)
    q, kb, vb, stride = inputs(0x7642_B16, tok, pos0, 0, n_heads, n_kv, q_scale=8.0, k_ramp=2.0)
    got = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv)
    assert np.isfinite(got).all()
    copy = attn.kv_f16_alloc(stride, n_kv)
    attn.kv_f16_rows(0, dev(kb), dev(vb), copy, n_kv, HD, stride, 0, pos0 + tok)
    mono = torch.full((tok, n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_kv_f16(dev(q), copy, None, mono, None, n_heads, n_kv, HD, pos0, tok, stride, None, None, 1)
    torch.cuda.synchronize()
    ok, _, _ = report("growing maxima, 64-token kernel vs single pass over the same copy", host(mono), got, *GATE)
    assert ok
    want = orc.attn_chunk_kv(q, kb, vb, n_heads, n_kv, HD, pos0, tok, stride, SCALE, n_threads=8)
    ok, _, _ = report("growing maxima, 64-token kernel vs the oracle (f16 Q and K operands)", want, got, 3e-2, 1e-2)
    assert ok


def test_same_bits_on_every_call():
    # the accumulators are state in registers no compiler tracks: a second call, after another launch has
    # used the chip, must give the same bits
    tok, pos0, splits, n_heads, n_kv = 192, 6000, 4, 24, 4
    q, kb, vb, stride = inputs(0x7643_0001, tok, pos0, 0, n_heads, n_kv)
    first = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv)
    other = inputs(0x7643_0002, 64, 1000, 0, n_heads, n_kv)
    run(other[0], other[1], other[2], 1000, 64, other[3], 4, n_heads, n_kv)
    again = run(q, kb, vb, pos0, tok, stride, splits, n_heads, n_kv)
    assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


@pytest.mark.parametrize("dtype", [0, 1])
def test_cache_entry_point_makes_its_tiles_in_the_scratch(dtype):
    # hipml_attn_chunk_splits sizes the scratch of a long chunk deep in a prefix for the slices plus the live
    # rows as f16 tiles; hipml_attn_chunk_q8_split then converts the rows there and runs the 64-token kernel
    # over them: the same bits as hipml_attn_chunk_kv_f16 over a copy made beforehand with the same number of
    # slices, and the oracle's values on sampled rows.  One slice fewer in the scratch and the call runs the
    # kernel that dequantizes for itself: same values within the gate.
    n_heads, n_kv, tok, pos0 = 24, 4, 800, 6500
    stride = pos0 + tok + 12
    splits, slices = attn.chunk_splits(pos0, tok, n_kv), attn.chunk_slices(pos0, tok, n_kv)
    assert slices >= 2 and splits > slices and uniform(tok, pos0, slices, n_heads // n_kv)
    assert no_extra_round(tok, slices, n_heads, n_kv)
    r = orc.Rng(0x7644_0000 + dtype)
    q = r.normal_array((tok, n_heads, HD))
    kb = orc.quantize(dtype, r.normal_array((n_kv, stride, HD))).reshape(n_kv, stride, -1)
    vb = orc.quantize(dtype, r.normal_array((n_kv, stride, HD))).reshape(n_kv, stride, -1)
    gate = r.normal_array((tok, n_heads, HD))

    def over_cache(n):
        # the scratch as the count sizes it, with a guard behind each part: the tiles must end inside it
        qslots, guard = (tok + 31) // 32 * 32, 1 << 20
        flat = torch.full((n * qslots * n_heads * HD + guard,), float("nan"), dtype=torch.float32, device="cuda")
        flat[-guard:] = 12345.0
        ml = torch.full((n * qslots * n_heads * 2 + guard,), float("nan"), dtype=torch.float32, device="cuda")
        ml[-guard:] = 12345.0
        out = torch.full((tok, n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
        attn.chunk_attention_q8_split_gate(dev(q), dev(kb), dev(vb), dev(gate), out, n_heads, n_kv, HD, pos0, tok,
                                           1 + dtype, stride, flat, ml, n)
        torch.cuda.synchronize()
        assert bool((flat[-guard:] == 12345.0).all()) and bool((ml[-guard:] == 12345.0).all())
        return host(out)

    got = over_cache(splits)
    copy = attn.kv_f16_alloc(stride, n_kv)
    attn.kv_f16_rows(dtype, dev(kb), dev(vb), copy, n_kv, HD, stride, 0, pos0 + tok)
    acc, ml = attn.chunk_scratch(tok, n_heads, slices)
    ref = torch.full((tok, n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.chunk_attention_kv_f16(dev(q), copy, dev(gate), ref, None, n_heads, n_kv, HD, pos0, tok, stride, acc, ml,
                                slices)
    torch.cuda.synchronize()
    assert np.array_equal(got.view(np.uint32), host(ref).view(np.uint32))
    rows = np.array([0, 1, 63, 64, 399, 767, 799], dtype=np.int32)
    want = orc.attn_chunk_kv(q, kb, vb, n_heads, n_kv, HD, pos0, tok, stride, SCALE, dtype=dtype, rows=rows,
                             n_threads=8)
    want = want / (1.0 + np.exp(-gate[rows].astype(np.float64)))
    tol = GATE if dtype == 0 else (3e-2, 3e-2)
    ok, _, _ = report(f"chunk {tok}@{pos0} over tiles made in the scratch, cache dtype {dtype}", want, got[rows], *tol)
    assert ok
    less = over_cache(splits - 1)
    ok, _, _ = report("the same chunk with a scratch too small for the tiles", got, less, *GATE)
    assert ok
